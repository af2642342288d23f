"""The SgdOpt::train / validate driver (through the C ABI) on idx files written by the test: against a hand-rolled
loop over the same operator calls (bit-identical parameters), its trace log, checkpoints, resume and validation."""
import os
import struct

import numpy as np
import pytest

from oracle import graph as OG
from rembrandt_amd import configs
from rembrandt_amd.operator import DataSource, SequentialOperatorConfig, SequentialOperatorWorker, SgdOpt
from conftest import assert_close, say

pytestmark = pytest.mark.gpu


def write_idx(path, arr):
    arr = np.ascontiguousarray(arr, np.uint8)
    with open(path, "wb") as f:
        f.write(struct.pack(">I", 0x0800 | arr.ndim))
        for d in arr.shape:
            f.write(struct.pack(">I", d))
        f.write(arr.tobytes())


def make_digits(path_prefix, n, seed):
    """28x28 frames whose class is the position of a bright 6x6 block on a noisy background."""
    rng = np.random.default_rng(seed)
    labels = rng.integers(0, 10, n).astype(np.uint8)
    imgs = rng.integers(0, 60, (n, 28, 28)).astype(np.uint8)
    for i, c in enumerate(labels):
        r, q = divmod(int(c), 4)
        imgs[i, 2 + 8 * r:8 + 8 * r, 1 + 7 * q:7 + 7 * q] = 230
    write_idx(str(path_prefix) + "-images.idx", imgs)
    write_idx(str(path_prefix) + "-labels.idx", labels)
    return imgs, labels


def small_lenet():
    return (SequentialOperatorConfig().data3d((28, 28, 1), normalize=True)
            .conv2d((28, 28, 1), 5, 1, 2, 8, "Rect", ("Normal", 0.05)).pool2d((28, 28, 8), 2, 2, 0, "Max")
            .conv2d((14, 14, 8), 5, 1, 2, 16, "Rect", ("Normal", 0.05)).pool2d((14, 14, 16), 2, 2, 0, "Max")
            .affine(7 * 7 * 16, 64, "Rect", ("Normal", 0.05)).dropout(64, 0.25).affine(64, 10, "Identity", ("Normal", 0.05))
            .softmax_kl_loss(10))


PARAM_OPS = (0, 2, 4, 6)


def manual_loop(w, sgd, imgs, labels, batch, minibatch, first_iter, last_iter):
    """The same operator calls the driver makes, from Python: sequential samples, epochs restart at sample 0."""
    it, pos, losses = first_iter, 0, []
    while it < last_iter:
        loss = 0.0
        for _ in range(minibatch // batch):
            idx = [(pos + i) % len(imgs) for i in range(batch)]
            assert idx[-1] > idx[0], "the test keeps batches inside one epoch"
            pos = (pos + batch) % len(imgs)
            w.load_frames_u8(imgs[idx][:, None])
            w.stage_batch(labels[idx], 1.0 / minibatch)
            w.forward(batch, training=True, t=it)
            w.store_output_categories(batch)
            loss += w.store_loss(batch)
            w.backward(batch)
        sgd.step(w, fused=True)
        it += 1
        losses.append(loss)
    return losses


@pytest.mark.parametrize("momentum", [("Update", 0.9), ("UpdateNesterov", 0.9)], ids=["update", "nesterov"])
def test_train_driver(dev, tmp_path, momentum):
    say("train driver", momentum)
    imgs, labels = make_digits(tmp_path / "train", 256, 1)
    vimgs, vlabels = make_digits(tmp_path / "valid", 100, 2)
    train = DataSource("mnist", tmp_path / "train-images.idx", tmp_path / "train-labels.idx")
    valid = DataSource("mnist", tmp_path / "valid-images.idx", tmp_path / "valid-labels.idx")
    batch, minibatch, ckpt = 32, 64, tmp_path / "ckpt"

    w = SequentialOperatorWorker(small_lenet(), batch, "Backward", shared_seed=(31, 32))
    sgd = SgdOpt(minibatch, 0.05, momentum, 1e-4)
    st = sgd.train(w, train, max_iters=12, valid_data=valid, checkpoint_dir=ckpt, display_iters=4, checkpoint_iters=4,
                   save_iters=4, valid_iters=8)
    assert st["iters"] == 12 and st["epochs"] == 3 and st["valid_runs"] == 1
    assert sorted(os.listdir(ckpt)) == ["checkpoint", "checkpoint.0", "params.latest.blob", "params.t_12.blob", "params.t_4.blob",
                                        "params.t_8.blob", "state.latest.blob.0", "trace_sgd.log"]
    rows = [l.split(",") for l in open(st["log_path"]).read().splitlines()]
    assert rows[0] == ["t", "event", "loss", "error", "elapsed"]
    assert [r[:2] for r in rows[1:]] == [[str(i), "step"] for i in range(1, 9)] + [["8", "valid"]] + [[str(i), "step"] for i in range(9, 13)]
    step_losses = [float(r[2]) for r in rows[1:] if r[1] == "step"]
    assert step_losses[-1] < step_losses[0], "the loss goes down on the toy problem: %r" % step_losses
    assert abs(float(rows[9][2]) - st["valid_loss"]) < 1e-5 and 0.0 <= st["valid_error"] <= 1.0

    # the same run by hand
    w2 = SequentialOperatorWorker(small_lenet(), batch, "Backward", shared_seed=(31, 32))
    w2.init_params()
    sgd2 = SgdOpt(minibatch, 0.05, momentum, 1e-4)
    sgd2.begin(w2)
    losses = manual_loop(w2, sgd2, imgs, labels, batch, minibatch, 0, 12)
    assert all(abs(a - b) <= 1e-6 * max(1.0, abs(a)) + 5e-7 for a, b in zip(losses, step_losses)), (losses, step_losses)
    for i in PARAM_OPS:
        assert np.array_equal(w.read(i, "weights"), w2.read(i, "weights")), "driver == hand-rolled loop, bit for bit"
        assert np.array_equal(w.read(i, "acc_grad_bias"), w2.read(i, "acc_grad_bias"))
    # validation pass == its definition: Inference forward over all samples with weights 1/N
    loss, acc = SgdOpt.validate(w, valid)
    correct, vloss = 0, 0.0
    for b0 in range(0, 100, batch):
        b = min(batch, 100 - b0)
        w2.load_frames_u8(vimgs[b0:b0 + b][:, None])
        w2.stage_batch(vlabels[b0:b0 + b], 1.0 / 100)
        w2.forward(b, training=False, t=0)
        w2.store_output_categories(b)
        correct += int((w2.get_output_categories(b) == vlabels[b0:b0 + b]).sum())
        vloss += w2.store_loss(b)
    assert abs(loss - vloss) <= 1e-5 * max(1.0, abs(vloss)) and abs(acc - correct / 100.0) < 1e-6

    if momentum[0] == "UpdateNesterov":
        # checkpoints hold the plain parameters; the live ones carry the look-ahead W + mu*v (new.rs:623-633)
        chk = SequentialOperatorWorker(small_lenet(), batch, "Backward", shared_seed=(1, 1))
        chk.rollback_state(ckpt)
        for i in PARAM_OPS:
            want = chk.read(i, "weights") + np.float32(momentum[1]) * chk.read(i, "acc_grad_weights")
            np.testing.assert_allclose(w.read(i, "weights"), want, rtol=1e-6, atol=1e-7)
        chk.close()

    # resume: InitOrResume finds checkpoint 12, restores params + momentum, carries on to 14, logs to trace_sgd.log.1
    w3 = SequentialOperatorWorker(small_lenet(), batch, "Backward", shared_seed=(77, 78))
    sgd3 = SgdOpt(minibatch, 0.05, momentum, 1e-4)
    st3 = sgd3.train(w3, train, max_iters=14, checkpoint_dir=ckpt)
    assert st3["iters"] == 14 and st3["log_path"].endswith("trace_sgd.log.1")
    rows3 = [l.split(",")[:2] for l in open(st3["log_path"]).read().splitlines()[1:]]
    assert rows3 == [["13", "step"], ["14", "step"]]
    # by hand: a fresh worker takes the state blob, then two more iterations from sample 0.  Dropout streams restart
    # with the worker, so the hand-rolled worker must be as fresh as the resumed one.
    w4 = SequentialOperatorWorker(small_lenet(), batch, "Backward", shared_seed=(77, 78))
    w4.rollback_state(ckpt)
    sgd4 = SgdOpt(minibatch, 0.05, momentum, 1e-4)
    sgd4.begin(w4)
    sgd4.set_iter_counter(12)   # the optimizer's counter decides the step size and Training{t}
    manual_loop(w4, sgd4, imgs, labels, batch, minibatch, 12, 14)
    for i in PARAM_OPS:
        assert np.array_equal(w3.read(i, "weights"), w4.read(i, "weights")), "resumed run == hand-rolled continuation"
    with pytest.raises(Exception):
        sgd3.train(w3, train, max_iters=20, checkpoint_dir=ckpt, resume_from=16)   # beyond the latest checkpoint
    for x in (w, w2, w3, w4):
        x.close()


@pytest.mark.parametrize("momentum", [("Update", 0.9), ("UpdateNesterov", 0.9)], ids=["update", "nesterov"])
def test_train_driver_against_oracle_loop(dev, tmp_path, momentum):
    """The driver against oracle.graph.sgd_train, an independent restatement of SgdOpt::train / ::validate (pinned on
    the CPU against a torch training loop): same idx files, 10 iterations of two batches each across an epoch boundary,
    Discard checkpoints every 2 iterations, validation (with a partial last batch) every 4.  Checked: the order and
    values of the trace rows, and every parameter and momentum buffer at the end.  The chain pools by averaging so that
    ten steps of rounding differences stay rounding differences."""
    say("train driver vs oracle loop", momentum)
    imgs, labels = make_digits(tmp_path / "train", 192, 3)
    vimgs, vlabels = make_digits(tmp_path / "valid", 52, 4)
    train = DataSource("mnist", tmp_path / "train-images.idx", tmp_path / "train-labels.idx")
    valid = DataSource("mnist", tmp_path / "valid-images.idx", tmp_path / "valid-labels.idx")
    batch, minibatch, iters = 16, 32, 10
    dims = (28, 28, 1)
    layers, ncat = configs._chain(dims, [("conv", 5, 1, 2, 8, "Rect"), ("pool", 2, 2, 0, "Average"),
                                         ("conv", 3, 2, 1, 12, "Rect"), ("fc", 32, "Rect"), ("fc", 10, "Identity")])
    cfg = SequentialOperatorConfig().data3d(dims, normalize=True)
    for l in layers:
        if l[0] == "conv2d":
            cfg.conv2d(l[1], l[2], l[3], l[4], l[5], l[6], ("Normal", 0.08))
        elif l[0] == "pool2d":
            cfg.pool2d(l[1], l[2], l[3], l[4], l[5], l[6])
        else:
            cfg.affine(l[1], l[2], l[3], ("Normal", 0.08))
    cfg.softmax_kl_loss(ncat)
    w = SequentialOperatorWorker(cfg, batch, "Backward", shared_seed=(41, 42))
    # the driver initialises from the worker's shared seed: the same call here gives the oracle its starting point
    w.init_params()
    ref = OG.SequentialOperatorWorker(layers, ncat, batch)
    for i, op in enumerate(ref.hidden):
        if op.p is not None:
            op.p.weights[...] = w.read(i, "weights").reshape(op.p.weights.shape)
    sgd = SgdOpt(minibatch, 0.05, momentum, 1e-3)
    st = sgd.train(w, train, max_iters=iters, valid_data=valid, checkpoint_dir=tmp_path / "ckpt", display_iters=1,
                   checkpoint_iters=2, save_iters=0, valid_iters=4, checkpoint_discard=True)
    rows = [l.split(",") for l in open(st["log_path"]).read().splitlines()][1:]
    f32 = lambda a: a.astype(np.float32)[:, None] / np.float32(255.0)
    want = OG.sgd_train(OG.SgdOpt(0.05, momentum, 1e-3), ref, f32(imgs), labels, minibatch, iters, checkpoint_iters=2,
                        checkpoint_discard=True, valid=(f32(vimgs), vlabels), valid_iters=4)
    assert [(int(r[0]), r[1]) for r in rows] == [(r[0], r[1]) for r in want]
    for got, exp in zip(rows, want):
        assert abs(float(got[2]) - exp[2]) <= 2e-4 * max(1.0, abs(exp[2])), (got, exp)
        assert abs(float(got[3]) - exp[3]) <= 1.0 / minibatch + 1e-4, (got, exp)   # one near-tie may flip
    for i, op in enumerate(ref.hidden):
        if op.p is None:
            continue
        for k in ("weights", "bias", "acc_grad_weights", "acc_grad_bias"):
            assert_close(w.read(i, k), getattr(op.p, k).ravel(), "driver vs oracle loop: %s[%d]" % (k, i), rtol=1e-3, atol=1e-5)
    w.close()
