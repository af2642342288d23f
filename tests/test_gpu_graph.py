"""GPU parity of whole train steps: SequentialOperatorWorker + SgdOpt (through the C ABI) against the
CPU restatement of the reference's operator chain, checkpoint by checkpoint, on the same seeded
inputs.  Order of checks: input -> each out_act -> probabilities -> loss, categories (exact),
accuracy count (exact) -> for each operator in reverse its out_delta (after the in-place ReLU mask),
grad_weights, grad_bias -> after the update: acc_grad_*, weights, bias -> grads == 0 exactly."""
import numpy as np
import pytest

import oracle as O
from oracle import graph as OG
from rembrandt_amd import configs, synth
from rembrandt_amd.operator import SequentialOperatorWorker, SgdOpt
from conftest import assert_close, say

pytestmark = pytest.mark.gpu


def make_pair(net, batch, seed, fuse):
    dims, layers, ncat = net
    cfg = configs.build_config(net)
    w = SequentialOperatorWorker(cfg, batch, "Backward", shared_seed=(seed, seed + 1), fuse_epilogue=fuse)
    w.init_params()
    ref = OG.SequentialOperatorWorker(layers, ncat, batch)
    assert ref.params_len() == cfg.params_len()
    assert w.hidden_count() == len(layers)
    # same initial parameters on both sides
    for i, op in enumerate(ref.hidden):
        assert w.op_kind(i) == op.kind
        if op.p is not None:
            op.p.weights[...] = w.read(i, "weights").reshape(op.p.weights.shape)
            op.p.bias[...] = w.read(i, "bias")
            assert not op.p.bias.any() and op.p.weights.any()
    return w, ref


def check_step(w, ref, sgd, rsgd, x, labels, minibatch, fused_sgd, tag):
    batch = x.shape[0]
    w.load_frames_f32(x)
    w.stage_batch(labels, 1.0 / minibatch)
    ref.stage_batch(labels, 1.0 / minibatch)
    w.forward(batch, training=True, t=sgd.iter_counter())
    ref.forward(x)
    assert_close(w.read(-1, "out_act"), x.ravel(), tag + " input")
    n = len(ref.hidden)
    for i, op in enumerate(ref.hidden):
        assert_close(w.read(i, "out_act"), op.out_act.ravel(), "%s out_act[%d] %s" % (tag, i, op.kind))
    assert_close(w.read(n, "out_act"), ref.out_values.ravel(), tag + " softmax", atol=1e-7)
    w.store_output_categories(batch)
    cats = w.get_output_categories(batch)
    # arg-max is compared on the GPU's own probabilities (bit-exact rule), then against the oracle chain
    assert np.array_equal(cats, np.argmax(w.read(n, "out_act").reshape(batch, -1), axis=1).astype(np.int32))
    ref.store_output_categories()
    loss = w.store_loss(batch)
    assert_close(np.array([loss]), np.array([ref.store_loss()]), tag + " loss")
    w.backward(batch)
    agree = np.array_equal(cats, ref.out_cats)
    if agree:
        assert w.accuracy_count(batch) == ref.accuracy_count()
    assert w.accuracy_count(batch) == int((cats == labels).sum())
    # Max-pool routing is discontinuous in the activations: a last-bit difference between two
    # near-tied taps moves a whole delta.  So the backward chain is compared operator by operator
    # from identical state: the oracle's forward state is first replaced by the GPU's (which has
    # just been checked against it), and each out_delta is re-synchronised after it is compared.
    prev = x
    for i, op in enumerate(ref.hidden):
        op.in_act = np.ascontiguousarray(prev.reshape(op.in_act.shape))
        op.out_act = w.read(i, "out_act").reshape(op.out_act.shape).copy()
        prev = op.out_act
    ref.out_values = w.read(n, "out_act").reshape(batch, -1).copy()
    delta = O.softmax_kl_backward(ref.out_values, ref.labels, ref.weights)
    for i in range(n - 1, -1, -1):
        op = ref.hidden[i]
        d = np.ascontiguousarray(delta.reshape(op.out_act.shape))
        if getattr(op, "act", None) == "Rect":
            O.rect_backprop_inplace(op.out_act, d)   # the GPU buffer is read after its in-place mask
        got = w.read(i, "out_delta")
        assert_close(got, d.ravel(), "%s out_delta[%d] %s" % (tag, i, op.kind))
        op.out_delta = got.reshape(op.out_act.shape).copy()
        delta = op.backward(want_in_delta=i > 0)
        if op.p is not None:
            assert_close(w.read(i, "grad_weights"), op.p.grad_weights.ravel(), "%s grad_weights[%d]" % (tag, i))
            assert_close(w.read(i, "grad_bias"), op.p.grad_bias.ravel(), "%s grad_bias[%d]" % (tag, i))
    sgd.step(w, fused=fused_sgd)
    rsgd.step(ref)
    assert sgd.iter_counter() == rsgd.iter_counter
    for i, op in enumerate(ref.hidden):
        if op.p is None:
            continue
        assert_close(w.read(i, "acc_grad_weights"), op.p.acc_grad_weights.ravel(), "%s acc_grad_weights[%d]" % (tag, i))
        assert_close(w.read(i, "acc_grad_bias"), op.p.acc_grad_bias.ravel(), "%s acc_grad_bias[%d]" % (tag, i))
        assert_close(w.read(i, "weights"), op.p.weights.ravel(), "%s weights[%d]" % (tag, i))
        assert_close(w.read(i, "bias"), op.p.bias.ravel(), "%s bias[%d]" % (tag, i))
        assert not w.read(i, "grad_weights").any() and not w.read(i, "grad_bias").any(), "reset() zeroes the gradients"
    return agree


@pytest.mark.parametrize("fuse,fused_sgd", [(True, True), (False, False)])
def test_lenet_train_steps(dev, fuse, fused_sgd):
    """BASELINE config 1: LeNet, batch 64, U[0,1) inputs, lr 0.01, momentum 0.9, weight decay 5e-4; 3 steps."""
    net, batch = configs.lenet(), 64
    say("lenet fuse", fuse, fused_sgd)
    w, ref = make_pair(net, batch, 0x5EED0001, fuse)
    sgd = SgdOpt(batch, 0.01, ("Update", 0.9), 5e-4)
    rsgd = OG.SgdOpt(0.01, ("Update", 0.9), 5e-4)
    sgd.begin(w)
    rsgd.begin(ref)
    for step in range(3):
        x = synth.uniform(0x5EED0001, 100 + step, (batch, 1, 28, 28))
        labels = synth.integers(0x5EED0001, 200 + step, (batch,), 10)
        check_step(w, ref, sgd, rsgd, x, labels, batch, fused_sgd, "lenet step %d" % step)
    w.close()


def test_cifar_train_steps(dev):
    """BASELINE config 3: CIFAR-10-shaped net, batch 128, N(0,1) inputs, momentum 0.9; 2 steps."""
    net, batch = configs.cifar10(), 128
    w, ref = make_pair(net, batch, 0x5EED0003, True)
    sgd = SgdOpt(batch, 0.01, ("Update", 0.9), 0.0)
    rsgd = OG.SgdOpt(0.01, ("Update", 0.9), 0.0)
    sgd.begin(w)
    rsgd.begin(ref)
    for step in range(2):
        say("cifar step", step)
        x = synth.normal(0x5EED0003, 100 + step, (batch, 3, 32, 32))
        labels = synth.integers(0x5EED0003, 200 + step, (batch,), 10)
        check_step(w, ref, sgd, rsgd, x, labels, batch, True, "cifar step %d" % step)
    w.close()


def test_alexnet_train_step(dev):
    """BASELINE config 4 geometry (AlexNet-shaped: 11x11 stride-4 conv on 227x227, three 3x3/2 max-pools,
    4096-wide affine layers, 1000 classes) at batch 4: one whole step, checkpoint by checkpoint."""
    net, batch = configs.alexnet(), 4
    w, ref = make_pair(net, batch, 0x5EED0004, True)
    sgd = SgdOpt(batch, 0.01, ("Update", 0.9), 0.0)
    rsgd = OG.SgdOpt(0.01, ("Update", 0.9), 0.0)
    sgd.begin(w)
    rsgd.begin(ref)
    say("alexnet step")
    x = synth.normal(0x5EED0004, 100, (batch, 3, 227, 227))
    labels = synth.integers(0x5EED0004, 200, (batch,), 1000)
    check_step(w, ref, sgd, rsgd, x, labels, batch, True, "alexnet step 0")
    w.close()


def test_nin_train_step(dev):
    """BASELINE config 5 geometry (NIN-shaped: 1x1 "cccp" convolutions, ceil-mode max-pools, 6x6 average pool
    into 1000 classes) at batch 2, fp32: one whole step, checkpoint by checkpoint."""
    net, batch = configs.nin(), 2
    w, ref = make_pair(net, batch, 0x5EED0005, True)
    sgd = SgdOpt(batch, 0.01, ("Update", 0.9), 0.0)
    rsgd = OG.SgdOpt(0.01, ("Update", 0.9), 0.0)
    sgd.begin(w)
    rsgd.begin(ref)
    say("nin step")
    x = synth.normal(0x5EED0005, 100, (batch, 3, 224, 224))
    labels = synth.integers(0x5EED0005, 200, (batch,), 1000)
    check_step(w, ref, sgd, rsgd, x, labels, batch, True, "nin step 0")
    w.close()


def test_nin_forward_bf16(dev):
    """BASELINE config 5, forward only with bf16 operands and fp32 accumulation.  Each operator is compared
    from the GPU's own input to it (a last-bit difference upstream may round to a different bf16 value)."""
    net, batch = configs.nin(), 2
    dims, layers, ncat = net
    cfg = configs.build_config(net, init_std=0.05)
    w = SequentialOperatorWorker(cfg, batch, "Forward", shared_seed=(0x5EED0005, 0x5EED0006), bf16_forward=True)
    w.init_params()
    ref = OG.SequentialOperatorWorker(layers, ncat, batch)
    for i, op in enumerate(ref.hidden):
        if op.p is not None:
            op.p.weights[...] = w.read(i, "weights").reshape(op.p.weights.shape)
            op.bf16_forward = True
    say("nin bf16 forward")
    x = synth.normal(0x5EED0005, 101, (batch, 3, 224, 224))
    w.load_frames_f32(x)
    w.forward(batch, training=False, t=0)
    prev = x
    for i, op in enumerate(ref.hidden):
        want = op.forward(np.ascontiguousarray(prev.reshape(op.x_shape if hasattr(op, "x_shape") else prev.shape)))
        got = w.read(i, "out_act")
        assert np.abs(got).max() > 0, "layer %d is not all zero" % i
        assert_close(got, want.ravel(), "nin bf16 out_act[%d] %s" % (i, op.kind))
        prev = got.reshape(want.shape).copy()
    n = len(ref.hidden)
    assert_close(w.read(n, "out_act"), O.softmax_fwd(np.ascontiguousarray(prev.reshape(batch, ncat))).ravel(),
                 "nin bf16 softmax", atol=1e-7)
    w.close()


@pytest.mark.parametrize("flavour", ["Zero", "Update", "UpdateNesterov", "Gradient", "GradientNesterov"])
def test_momentum_flavours(dev, flavour):
    """All five Momentum flavours on a small conv net (3 steps each, unfused BLAS-1 sequence and, where it
    exists, the fused kernel)."""
    net = ((12, 12, 2), *configs._chain((12, 12, 2), [("conv", 3, 1, 1, 6, "Rect"), ("pool", 2, 2, 0, "Max"),
                                                         ("fc", 16, "Rect"), ("fc", 5, "Identity")]))
    batch = 8
    mom = flavour if flavour == "Zero" else (flavour, 0.9)
    for fused_sgd in (False, True):
        say("flavour", flavour, "fused", fused_sgd)
        w, ref = make_pair(net, batch, 77, True)
        sgd, rsgd = SgdOpt(batch, 0.05, mom, 1e-3), OG.SgdOpt(0.05, mom, 1e-3)
        sgd.begin(w)
        rsgd.begin(ref)
        for step in range(3):
            x = synth.normal(77, 10 + step, (batch, 2, 12, 12))
            labels = synth.integers(77, 20 + step, (batch,), 5)
            check_step(w, ref, sgd, rsgd, x, labels, batch, fused_sgd, "%s step %d" % (flavour, step))
        w.close()


def test_gradient_accumulation_over_microbatches(dev):
    """batch_size = minibatch_size / 4: four forward/backward passes accumulate (beta = 1) before one update."""
    net = ((10, 10, 3), *configs._chain((10, 10, 3), [("conv", 3, 1, 1, 8, "Rect"), ("pool", 3, 2, 0, "Average"),
                                                         ("fc", 7, "Identity")]))
    batch, minibatch = 4, 16
    w, ref = make_pair(net, batch, 99, True)
    sgd, rsgd = SgdOpt(minibatch, 0.1, ("Update", 0.5), 0.0), OG.SgdOpt(0.1, ("Update", 0.5), 0.0)
    sgd.begin(w)
    rsgd.begin(ref)
    for micro in range(4):
        x = synth.normal(99, 10 + micro, (batch, 3, 10, 10))
        labels = synth.integers(99, 20 + micro, (batch,), 7)
        w.load_frames_f32(x)
        w.stage_batch(labels, 1.0 / minibatch)
        ref.stage_batch(labels, 1.0 / minibatch)
        w.forward(batch)
        ref.forward(x)
        w.backward(batch)
        ref.backward()
    for i, op in enumerate(ref.hidden):
        if op.p is not None:
            assert_close(w.read(i, "grad_weights"), op.p.grad_weights.ravel(), "accumulated grad_weights[%d]" % i)
            assert_close(w.read(i, "grad_bias"), op.p.grad_bias.ravel(), "accumulated grad_bias[%d]" % i)
    sgd.step(w, fused=True)
    rsgd.step(ref)
    for i, op in enumerate(ref.hidden):
        if op.p is not None:
            assert_close(w.read(i, "weights"), op.p.weights.ravel(), "weights[%d]" % i)
    w.close()


def test_u8_frames_and_save_restore(dev):
    net = ((8, 8, 1), *configs._chain((8, 8, 1), [("conv", 3, 1, 1, 4, "Rect"), ("fc", 3, "Identity")]))
    from rembrandt_amd.operator import SequentialOperatorConfig
    cfg = SequentialOperatorConfig().data3d((8, 8, 1), normalize=True).conv2d((8, 8, 1), 3, 1, 1, 4, "Rect").affine(256, 3, "Identity").softmax_kl_loss(3)
    w = SequentialOperatorWorker(cfg, 5, "Backward")
    w.init_params()
    frames = synth.integers(5, 1, (5, 1, 8, 8), 256).astype(np.uint8)
    w.load_frames_u8(frames)
    w.stage_batch([0, 1, 2, 0, 1], 0.2)
    w.forward(5)
    assert np.array_equal(w.read(-1, "out_act"), (frames.astype(np.float32) * np.float32(1.0 / 255.0)).ravel())
    before = w.read(0, "weights")
    w.save_params()
    w.backward(5)
    w.accumulate_grads(-0.1, 0.0)
    w.update_params(1.0)
    assert not np.array_equal(w.read(0, "weights"), before)
    w.restore_params()
    assert np.array_equal(w.read(0, "weights"), before)
    w.close()


def test_panics(dev):
    from rembrandt_amd.operator import Panic, SequentialOperatorConfig
    cfg = SequentialOperatorConfig().data3d((8, 8, 1)).affine(64, 3, "Identity").softmax_kl_loss(3)
    w = SequentialOperatorWorker(cfg, 4, "Backward")
    with pytest.raises(Panic):
        w.forward(5)          # batch_size <= batch_cap (mod.rs:1076)
    with pytest.raises(Panic):
        w.stage_label(0, 3)   # category < num_categories (new.rs:296-299)
    with pytest.raises(Panic):
        SequentialOperatorWorker(SequentialOperatorConfig().data3d((8, 8, 1)), 4)  # no loss operator
    cfg2 = SequentialOperatorConfig().data3d((8, 8, 1)).affine(64, 3, "Tanh").softmax_kl_loss(3)
    w2 = SequentialOperatorWorker(cfg2, 4, "Backward")
    with pytest.raises(Panic):
        w2.forward(4)         # only Identity / Rect are implemented (mod.rs:1115)
    fwd_only = SequentialOperatorWorker(cfg, 4, "Forward")
    with pytest.raises(Panic):
        fwd_only.backward(4)  # assert!(self.backward.is_some())
    w.close(); w2.close(); fwd_only.close()
