"""GPU parity of whole train steps: SequentialOperatorWorker + SgdOpt (through the C ABI) against the
CPU restatement of the reference's operator chain, checkpoint by checkpoint, on the same seeded
inputs.  Order of checks: input -> each out_act -> probabilities -> loss, categories (exact),
accuracy count (exact) -> for each operator in reverse its out_delta (after the in-place ReLU mask),
grad_weights, grad_bias -> after the update: acc_grad_*, weights, bias -> grads == 0 exactly."""
import os

import numpy as np
import pytest

import oracle as O
from oracle import graph as OG
from rembrandt_amd import configs, synth
from rembrandt_amd.operator import SequentialOperatorConfig, SequentialOperatorWorker, SgdOpt
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
    for i, op in enumerate(ref.hidden):
        if op.kind == "DropoutOperator":   # the uniform samples this forward consumed, regenerated on the host
            seed, stream_id, first = w.dropout_stream(i)
            n = int(np.prod(op.x_shape))
            op.rnd = synth.uniform(seed, stream_id, (first + n,))[first:]
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
    """Benchmark configuration 1: LeNet, batch 64, U[0,1) inputs, lr 0.01, momentum 0.9, weight decay 5e-4; 3 steps."""
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
    """Benchmark configuration 3: CIFAR-10-shaped net, batch 128, N(0,1) inputs, momentum 0.9; 2 steps."""
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
    """Benchmark configuration 4 geometry (AlexNet-shaped: 11x11 stride-4 conv on 227x227, three 3x3/2 max-pools,
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


def test_dropout_lrn_train_steps(dev):
    """A chain with a local response normalisation and two dropout operators (the layer types the example
    `.model` files add around the benchmark operators): 3 steps, each with fresh dropout masks."""
    dims = (14, 14, 3)
    net = (dims, *configs._chain(dims, [("conv", 3, 1, 1, 8, "Rect"), ("lrn", 5, 1e-2, 0.75, 2.0), ("pool", 2, 2, 0, "Max"),
                                        ("dropout", 0.3), ("fc", 32, "Rect"), ("dropout", 0.5), ("fc", 6, "Identity")]))
    batch = 16
    w, ref = make_pair(net, batch, 91, True)
    assert [w.op_kind(i) for i in (1, 3, 5)] == ["LocalResNormOperator", "DropoutOperator", "DropoutOperator"]
    sgd = SgdOpt(batch, 0.05, ("Update", 0.9), 1e-4)
    rsgd = OG.SgdOpt(0.05, ("Update", 0.9), 1e-4)
    sgd.begin(w)
    rsgd.begin(ref)
    masks = []
    for step in range(3):
        say("dropout/lrn step", step)
        x = synth.normal(91, 100 + step, (batch, 3, 14, 14))
        labels = synth.integers(91, 200 + step, (batch,), 6)
        check_step(w, ref, sgd, rsgd, x, labels, batch, True, "dropout/lrn step %d" % step)
        masks.append(ref.hidden[5].mask.copy())
        assert 0.3 < masks[-1].mean() < 0.7
    assert not np.array_equal(masks[0], masks[1]) and not np.array_equal(masks[1], masks[2])
    # Inference: dropout is the identity
    w.forward(batch, training=False, t=0)
    assert np.array_equal(w.read(3, "out_act"), w.read(2, "out_act"))
    w.close()


def test_nin_train_step(dev):
    """Benchmark configuration 5 geometry (NIN-shaped: 1x1 "cccp" convolutions, ceil-mode max-pools, 6x6 average pool
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


def _is_bf16_valued(a):
    return not (np.ascontiguousarray(a, dtype=np.float32).view(np.uint32) & 0xFFFF).any()


def test_nin_forward_bf16(dev):
    """Benchmark configuration 5, forward only with bf16 operands and fp32 accumulation.  Each operator is compared
    from the GPU's own input to it (a last-bit difference upstream may round to a different bf16 value).  A forward-only
    worker keeps the activations between convolutions as packed bf16: such a layer's out_act reads back as the fp32
    result rounded to nearest even, which is compared with the oracle's result rounded the same way (stated looser
    bound: equal except where the last-bit difference of the accumulation moves a value across a rounding boundary,
    then one bf16 step, 2^-7 relative, on at most 0.2 % of the elements; next to zero, the fp32 absolute bound)."""
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
    packed_layers = 0
    for i, op in enumerate(ref.hidden):
        want = op.forward(np.ascontiguousarray(prev.reshape(op.x_shape if hasattr(op, "x_shape") else prev.shape)))
        got = w.read(i, "out_act")
        assert np.abs(got).max() > 0, "layer %d is not all zero" % i
        if _is_bf16_valued(got) and not _is_bf16_valued(want):
            packed_layers += 1
            want_r = O.round_bf16(want).ravel()
            diff = got != want_r
            assert diff.mean() <= 2e-3, "nin bf16 out_act[%d] %s: %.3g of the elements round differently" % (i, op.kind, diff.mean())
            # one bf16 step, or the fp32 tolerance itself where a value lies next to zero (a ReLU's cut)
            slack = 2e-5 * max(1.0, float(np.sqrt(np.mean(want_r.astype(np.float64) ** 2))))
            assert (np.abs(got - want_r) <= 2.0 ** -7 * np.abs(want_r) + slack).all(), "nin bf16 out_act[%d]: more than one bf16 step" % i
        else:
            assert_close(got, want.ravel(), "nin bf16 out_act[%d] %s" % (i, op.kind))
        prev = got.reshape(want.shape).copy()
    assert packed_layers >= 11, packed_layers   # every convolution but the last, which feeds the average pool
    n = len(ref.hidden)
    assert_close(w.read(n, "out_act"), O.softmax_fwd(np.ascontiguousarray(prev.reshape(batch, ncat))).ravel(),
                 "nin bf16 softmax", atol=1e-7)
    w.close()


@pytest.mark.parametrize("name", ["nin", "alexnet", "cifar10"])
def test_bf16_packed_chain_is_bit_identical(dev, name):
    """A forward-only bf16 worker (packed bf16 activations between convolutions, written by the producers' epilogues,
    filters converted once) against a worker that keeps fp32 activations and converts every convolution's input
    (Backward capability): every layer's activations are the other's rounded to bf16, bit for bit, and the final
    probabilities are identical.  Then the converted filters: a second pass repeats the first, and a weight written
    through the worker's buffer is seen by the next pass."""
    net, batch = configs.NETWORKS[name](), 3
    dims, layers, ncat = net
    cfg = configs.build_config(net, init_std=0.05)
    a = SequentialOperatorWorker(cfg, batch, "Forward", shared_seed=(0x5EED0015, 0x5EED0016), bf16_forward=True)
    b = SequentialOperatorWorker(cfg, batch, "Backward", shared_seed=(0x5EED0015, 0x5EED0016), bf16_forward=True)
    a.init_params()
    b.init_params()
    x = synth.normal(0x5EED0015, 101, (batch, dims[2], dims[1], dims[0]))
    n = len(layers)

    def run_and_compare(tag):
        for w in (a, b):
            w.load_frames_f32(x)
            w.forward(batch, training=False, t=0)
        packed = 0
        for i in range(n):
            ga, gb = a.read(i, "out_act"), b.read(i, "out_act")
            assert np.abs(gb).max() > 0
            if not np.array_equal(ga, gb):
                packed += 1
                assert np.array_equal(ga, O.round_bf16(gb)), "%s %s layer %d" % (tag, name, i)
        pa, pb = a.read(n, "out_act"), b.read(n, "out_act")
        assert np.array_equal(pa, pb), "%s %s probabilities" % (tag, name)
        return packed, pa.copy()

    say("bf16 packed chain", name)
    packed, p1 = run_and_compare("first pass")
    assert packed >= {"nin": 11, "alexnet": 3, "cifar10": 0}[name], packed   # (cifar10: stride-1 3-channel first layer, average pools)
    _, p2 = run_and_compare("second pass")
    assert np.array_equal(p1, p2)
    conv_idx = [i for i, l in enumerate(layers) if l[0] == "conv2d"][1]
    wts = a.read(conv_idx, "weights")
    wts[::7] *= np.float32(-1.5)
    a.write(conv_idx, "weights", wts)
    b.write(conv_idx, "weights", wts)
    _, p3 = run_and_compare("after a weight write")
    assert not np.array_equal(p1, p3)
    a.close()
    b.close()


def test_random_networks_train_steps(dev):
    """Seeded sweep over operator chains: 1-3 convolutions (filter 1-5, stride 1-2, any legal padding, Rect or
    Identity) with local response normalisation, max / average pooling and dropout between them, an optional hidden
    affine layer, fused or reference-order epilogues and SGD, every momentum flavour; two checked steps each."""
    import random
    rnd = random.Random(20160419)
    for it in range(14):
        wdt, hgt, c = rnd.choice([8, 11, 14, 16, 20]), rnd.choice([8, 11, 14, 16, 20]), rnd.choice([1, 3, 4, 8])
        dims, spec = (wdt, hgt, c), []
        w_, h_ = wdt, hgt
        for _ in range(rnd.randint(1, 3)):
            k, st = rnd.choice([1, 3, 3, 5]), rnd.choice([1, 1, 2])
            pad = rnd.randint(0, k // 2)
            out = rnd.choice([4, 8, 12, 16, 20, 32])
            if (w_ + 2 * pad - k) // st + 1 < 2 or (h_ + 2 * pad - k) // st + 1 < 2:
                k, st, pad = 1, 1, 0
            spec.append(("conv", k, st, pad, out, rnd.choice(["Rect", "Rect", "Identity"])))
            w_, h_ = (w_ + 2 * pad - k) // st + 1, (h_ + 2 * pad - k) // st + 1
            if rnd.random() < 0.25:
                spec.append(("lrn", rnd.choice([3, 5]), 1e-2, 0.75, 2.0))
            if rnd.random() < 0.6 and w_ >= 3 and h_ >= 3:
                pk, ps = rnd.choice([2, 3]), rnd.choice([1, 2])
                pp = rnd.choice([0, 0, 1]) if pk == 3 else 0
                spec.append(("pool", pk, ps, pp, rnd.choice(["Max", "Max", "Average"])))
                w_, h_ = (w_ + 2 * pp - pk) // ps + 1, (h_ + 2 * pp - pk) // ps + 1
            if rnd.random() < 0.2:
                spec.append(("dropout", 0.3))
        if rnd.random() < 0.6:
            spec.append(("fc", rnd.choice([16, 33, 64]), rnd.choice(["Rect", "Identity"])))
            if rnd.random() < 0.3:
                spec.append(("dropout", 0.5))
        ncat = rnd.choice([3, 5, 10])
        spec.append(("fc", ncat, "Identity"))
        batch = rnd.choice([4, 8, 16, 33])
        fuse, fused_sgd = rnd.random() < 0.7, rnd.random() < 0.6
        flavour = rnd.choice([("Update", 0.9), ("UpdateNesterov", 0.9), ("Gradient", 0.8), "Zero", ("GradientNesterov", 0.9)])
        say("random net", it, dims, spec, "batch", batch, fuse, fused_sgd, flavour)
        net = (dims, *configs._chain(dims, spec))
        w, ref = make_pair(net, batch, 1000 + it, fuse)
        sgd = SgdOpt(batch, 0.05, flavour, 1e-4)
        rsgd = OG.SgdOpt(0.05, flavour, 1e-4)
        sgd.begin(w)
        rsgd.begin(ref)
        for step in range(2):
            x = synth.normal(1000 + it, 100 + step, (batch, dims[2], dims[1], dims[0]))
            labels = synth.integers(1000 + it, 200 + step, (batch,), ncat)
            check_step(w, ref, sgd, rsgd, x, labels, batch, fused_sgd, "random net %d step %d" % (it, step))
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
    """batch_size = minibatch_size / 4: four forward/backward passes accumulate (beta = 1) before one update.  Two
    minibatches: at the start of the second the fused step has left the gradient buffers standing for zeros, so its
    first backward pass overwrites and the other three accumulate."""
    net = ((10, 10, 3), *configs._chain((10, 10, 3), [("conv", 3, 1, 1, 8, "Rect"), ("pool", 3, 2, 0, "Average"),
                                                         ("fc", 7, "Identity")]))
    batch, minibatch = 4, 16
    w, ref = make_pair(net, batch, 99, True)
    sgd, rsgd = SgdOpt(minibatch, 0.1, ("Update", 0.5), 0.0), OG.SgdOpt(0.1, ("Update", 0.5), 0.0)
    sgd.begin(w)
    rsgd.begin(ref)
    for mini in range(2):
        for micro in range(4):
            x = synth.normal(99, 10 + micro + 100 * mini, (batch, 3, 10, 10))
            labels = synth.integers(99, 20 + micro + 100 * mini, (batch,), 7)
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
                assert_close(w.read(i, "weights"), op.p.weights.ravel(), "weights[%d] after minibatch %d" % (i, mini))
    w.close()


@pytest.mark.parametrize("overlap", [False, True])
def test_gradients_standing_for_zeros(dev, overlap):
    """After a fused step the gradient buffers are not zeroed but stand for zeros until the next backward pass
    overwrites them.  Reading them makes the zeros real; a worker whose gradients are read after every step (its
    backward passes then accumulate onto real zeros) must stay bit-identical to one that is left alone, also through
    two steps in a row without a backward pass in between and a step of the unfused sequence."""
    net = configs.lenet()
    dims, layers, ncat = net
    batch = 8
    ws = []
    for _ in range(2):
        w = SequentialOperatorWorker(configs.build_config(net), batch, "Backward", shared_seed=(5, 6), overlap_backward=overlap)
        w.init_params()
        ws.append(w)
    sgds = [SgdOpt(batch, 0.05, ("Update", 0.9), 1e-3) for _ in ws]
    for sgd, w in zip(sgds, ws):
        sgd.begin(w)
    param_layers = [i for i, l in enumerate(layers) if l[0] in ("conv2d", "affine")]
    for step in range(5):
        x = synth.normal(5, 10 + step, (batch, dims[2], dims[1], dims[0]))
        labels = synth.integers(5, 50 + step, (batch,), ncat)
        losses = []
        for k, (sgd, w) in enumerate(zip(sgds, ws)):
            w.load_frames_f32(x)
            w.stage_batch(labels, 1.0 / batch)
            if step == 3:                       # the reference's own call sequence on both
                w.forward(batch, training=True, t=sgd.iter_counter())
                w.backward(batch)
                sgd.step(w, fused=False)
                losses.append(w.store_loss(batch))
            else:
                losses.append(sgd.train_batch(w, batch, fused=True)[0])
            if step == 1:
                sgd.step(w, fused=True)         # a second step on gradients that stand for zeros (momentum only)
            if k == 1:
                for i in param_layers:
                    assert not w.read(i, "grad_weights").any() and not w.read(i, "grad_bias").any(), "gradients after a step"
        assert losses[0] == losses[1], "step %d" % step
        for i in param_layers:
            for name in ("weights", "bias", "acc_grad_weights", "acc_grad_bias"):
                assert np.array_equal(ws[0].read(i, name), ws[1].read(i, name)), (step, i, name)
    for w in ws:
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


@pytest.mark.parametrize("graph", [False, True])
def test_u8_frames_loaded_beside_queued_work(dev, graph):
    """load_frames copies on a stream of its own, after the previous batch's cast has read the staging buffer and
    beside whatever the main stream still holds: batches alternated without any synchronisation between a load and
    the queued steps before it give the results of the same batches run one at a time (with recorded steps, where
    the readers run at replay time, the load waits for the stream instead)."""
    from rembrandt_amd.operator import SequentialOperatorConfig
    dims = (24, 24, 3)
    def make():
        cfg = SequentialOperatorConfig().data3d(dims, normalize=True).conv2d(dims, 3, 1, 1, 16, "Rect") \
            .pool2d((24, 24, 16), 2, 2, 0, "Max").affine(12 * 12 * 16, 5, "Identity").softmax_kl_loss(5)
        w = SequentialOperatorWorker(cfg, 32, "Backward", shared_seed=(9, 10), graph_steps=graph)
        w.init_params()
        return w
    batches = [synth.integers(6, 10 + i, (32, 3, 24, 24), 256).astype(np.uint8) for i in range(3)]
    labels = synth.integers(6, 20, (32,), 5)
    # one at a time, with a full synchronisation (the read-back) after every step
    w = make()
    sgd = SgdOpt(32, 0.05, ("Update", 0.9), 0.0)
    sgd.begin(w)
    w.stage_batch(labels, 1.0 / 32)
    want = []
    for step in range(9):
        w.load_frames_u8(batches[step % 3])
        loss, _ = sgd.train_batch(w, 32)
        want.append((loss, w.read(0, "weights").copy(), w.read(-1, "out_act").copy()))
    w.close()
    # the same steps, each load issued while the step before it is still queued
    w = make()
    sgd = SgdOpt(32, 0.05, ("Update", 0.9), 0.0)
    sgd.begin(w)
    w.stage_batch(labels, 1.0 / 32)
    w.load_frames_u8(batches[0])
    for step in range(9):
        w.forward(32, training=True, t=sgd.iter_counter())
        w.backward(32)
        sgd.step(w, fused=True)
        inputs = None
        if step % 4 == 3:
            inputs = w.read(-1, "out_act").copy()   # now and then look at what the step consumed
        if step + 1 < 9:
            w.load_frames_u8(batches[(step + 1) % 3])   # no synchronisation before this
        loss = w.store_loss(32)
        assert loss == want[step][0], "step %d: loss %r vs %r" % (step, loss, want[step][0])
        if inputs is not None:
            assert np.array_equal(inputs, want[step][2])
    assert np.array_equal(w.read(0, "weights"), want[-1][1])
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


def _tiny_head(cfg, dims, ncat=4):
    return cfg.affine(dims[0] * dims[1] * dims[2], ncat, "Identity", ("Normal", 0.05)).softmax_kl_loss(ncat)


@pytest.mark.parametrize("normalize", [False, True])
def test_data3d_preprocessing(dev, normalize, tmp_path):
    """Data3dOperator: u8 frames -> cast (/255 when normalising) -> SubtractElemwiseMean -> FlipX -> Crop, the order
    the reference's tools use (tools/train-imagenet.rs:63-70), then PCA lighting noise.  The output is compared with
    the numpy restatement for the offsets / coin / coefficients the operator reports having drawn."""
    say("data3d preprocessing", normalize)
    in_dims, crop, batch = (23, 19, 3), (16, 12), 6
    rng = np.random.default_rng(17)
    frames = rng.integers(0, 256, (batch, 3, 19, 23), dtype=np.uint8)
    mean = synth.uniform(18, 1, (3, 19, 23), 0.0, 255.0)
    svecs, svals = synth.normal(18, 2, (3, 3)), synth.uniform(18, 3, (3,))
    # the mean comes from an NdArray file, as in the reference (dims (w, h, c), values W fastest)
    mean_path = tmp_path / "mean.ndarray"
    import struct
    mean_path.write_bytes(b"ND\x00\x01" + struct.pack("<I3Q", 3, 23, 19, 3) + mean.tobytes())
    cfg = (SequentialOperatorConfig().data3d(in_dims, normalize=normalize).subtract_elemwise_mean(mean_path=mean_path)
           .flip_x().crop(*crop).pca_lighting_noise(svecs, svals, 0.1))
    w = SequentialOperatorWorker(_tiny_head(cfg, (crop[0], crop[1], 3)), batch, "Forward", shared_seed=(5, 6))
    assert w.input_out_dims() == (16, 12, 3)
    w.init_params()
    w.load_frames_u8(frames)
    base = frames.astype(np.float32) * (np.float32(1.0 / 255.0) if normalize else np.float32(1.0))
    seen_flip, seen_off = set(), set()
    for t in range(12):
        w.forward(batch, training=True, t=t)
        off_w, off_h, flipped, alphas = w.last_preproc_draws()
        assert 0 <= off_w <= 23 - 16 and 0 <= off_h <= 19 - 12 and alphas.shape == (3 * batch,)
        seen_flip.add(flipped)
        seen_off.add((off_w, off_h))
        want = O.subtract_mean(base, mean, normalize)
        if flipped:
            want = O.flip_x(want)
        want = O.pca3_noise(O.crop_nchw(want, crop[0], crop[1], off_w, off_h), alphas, svals, svecs.ravel())
        got = w.read(-1, "out_act", batch * 3 * 12 * 16)
        assert_close(got, want.ravel(), "data3d training output (draw %d)" % t)
    assert seen_flip == {False, True} and len(seen_off) > 3, "both coin faces and several offsets occur in 12 draws"
    # Inference: centre crop, no flip, no noise
    w.forward(batch, training=False, t=0)
    off_w, off_h, flipped, alphas = w.last_preproc_draws()
    assert (off_w, off_h, flipped, alphas.size) == ((23 - 16) // 2, (19 - 12) // 2, False, 0)
    want = O.crop_nchw(O.subtract_mean(base, mean, normalize), crop[0], crop[1], off_w, off_h)
    assert_close(w.read(-1, "out_act", want.size), want.ravel(), "data3d inference output")
    # fp32 frames take the same path minus the cast, and survive repeated forwards
    w.load_frames_f32(base)
    for _ in range(2):
        w.forward(batch, training=False, t=0)
        assert_close(w.read(-1, "out_act", want.size), want.ravel(), "data3d inference output from fp32 frames")
    w.close()


def test_param_blobs_and_checkpoints(dev, tmp_path):
    """encode/decode_params/state and the checkpoint files: bytes are NdArray records of the documented layout,
    a round trip through another worker reproduces parameters and momentum exactly, rollback picks the iteration."""
    import struct
    net, batch = configs.lenet(), 8
    w, ref = make_pair(net, batch, 123, True)
    sgd = SgdOpt(batch, 0.01, ("Update", 0.9), 5e-4)
    sgd.begin(w)
    x = synth.uniform(123, 1, (batch, 1, 28, 28))
    labels = synth.integers(123, 2, (batch,), 10)
    w.load_frames_f32(x)
    w.stage_batch(labels, 1.0 / batch)
    sgd.train_batch(w, batch)
    blob = w.encode_params()
    # walk the records: conv1 (25, 20), (1, 20), conv2 (500, 50), (1, 50), fc1 (2450, 500), (1, 500), fc2 (500, 10), (1, 10)
    off, bounds = 0, []
    params = {0: "weights", 1: "bias"}
    expect_ops = [i for i in range(w.hidden_count()) if w.op_kind(i) != "Pool2dOperator"]
    k = 0
    while off < len(blob):
        assert blob[off:off + 4] == b"ND\x00\x01"
        (rank,) = struct.unpack_from("<I", blob, off + 4)
        dims = struct.unpack_from("<%dQ" % rank, blob, off + 8)
        n = int(np.prod(dims))
        data = np.frombuffer(blob, np.float32, n, off + 8 + 8 * rank)
        assert np.array_equal(data, w.read(expect_ops[k // 2], params[k % 2])), "record %d holds the device buffer" % k
        bounds.append(dims)
        off += 8 + 8 * rank + 4 * n
        k += 1
    assert bounds == [(25, 20), (1, 20), (500, 50), (1, 50), (2450, 500), (1, 500), (500, 10), (1, 10)]
    state = w.encode_state()
    assert len(state) == 2 * len(blob)

    prefix = tmp_path / "ckpt"
    w.checkpoint_params(1, prefix)
    w.checkpoint_state(prefix)
    sgd.train_batch(w, batch)
    w.checkpoint_params(2, prefix)
    assert sorted(os.listdir(prefix)) == ["checkpoint", "checkpoint.0", "params.latest.blob", "params.t_1.blob",
                                          "params.t_2.blob", "state.latest.blob.0"]
    assert (prefix / "checkpoint").read_text() == "2\n" and (prefix / "checkpoint.0").read_text() == "1\n"
    assert os.readlink(prefix / "params.latest.blob") == "params.t_2.blob"
    assert (prefix / "params.t_1.blob").read_bytes() == blob

    cfg = configs.build_config(net)
    w2 = SequentialOperatorWorker(cfg, batch, "Backward", shared_seed=(9, 9))
    w2.init_params()
    assert w2.can_rollback(tmp_path / "nowhere") is None and w2.can_rollback(prefix) == 2
    w2.rollback_params(prefix)            # latest = t_2
    for i in expect_ops:
        assert np.array_equal(w2.read(i, "weights"), w.read(i, "weights"))
    w2.rollback_params(prefix, t=1)
    assert w2.encode_params() == blob
    w2.rollback_state(prefix)             # params of t=1 plus the momentum buffers
    assert w2.encode_state() == state
    with pytest.raises(Exception):
        w2.rollback_params(prefix, t=3)   # beyond the latest checkpoint
    with pytest.raises(Exception):
        w2.decode_params(blob[:-4])       # truncated
    # a blob of another architecture is refused
    other = SequentialOperatorWorker(configs.build_config(configs.cifar10()), 4, "Forward", shared_seed=(1, 1))
    with pytest.raises(Exception):
        other.decode_params(blob)
    other.close()
    w2.close()
    w.close()
