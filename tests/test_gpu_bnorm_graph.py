"""GPU parity of train steps through the batch-normalised operators (BNormConv2d, StackResConv2d, ProjStackResConv2d of
src/operator/conv.rs) against the CPU restatement, checkpoint by checkpoint: every unit's conv output, batch statistics,
moving statistics, the activation between stacked units, out_act; then, from the GPU's own forward state, every
gradient buffer in the reference's order; then the SGD update of filters, scales and biases."""
import struct

import numpy as np
import pytest

import oracle as O
from oracle import graph as OG
from rembrandt_amd import configs, synth
from rembrandt_amd.operator import SequentialOperatorWorker, SgdOpt
from conftest import assert_close, say

pytestmark = pytest.mark.gpu

UNIT_PARAMS = (("weights", "weights"), ("bn_scale", "scale"), ("bn_bias", "bias"))
UNIT_GRADS = (("grad_weights", "grad_weights"), ("bn_scale_grad", "scale_grad"), ("bn_bias_grad", "bias_grad"))
UNIT_ACCS = (("acc_grad_weights", "acc_grad_weights"), ("acc_bn_scale_grad", "acc_scale_grad"), ("acc_bn_bias_grad", "acc_bias_grad"))


def small_net():
    dims = (16, 16, 3)
    layers, out = configs._chain(dims, [("bnconv", 3, 1, 1, 8, "Rect"), ("pool", 2, 2, 0, "Max"), ("res", "Rect"),
                                        ("projres", 16, 2, "Rect"), ("projres", 24, 1, "Rect"), ("res", "Rect"),
                                        ("pool", 4, 1, 0, "Average"), ("fc", 5, "Identity")])
    return dims, layers, out


def make_pair(net, batch, seed, fuse, mov_avg=("Exponential", 0.1), eps=1e-5, capability="Backward"):
    dims, layers, ncat = net
    cfg = configs.build_config(net, bnorm_mov_avg=mov_avg, bnorm_epsilon=eps)
    w = SequentialOperatorWorker(cfg, batch, capability, shared_seed=(seed, seed + 1), fuse_epilogue=fuse)
    w.init_params()
    ref = OG.SequentialOperatorWorker(layers, ncat, batch, bnorm_mov_avg=mov_avg, bnorm_epsilon=eps)
    assert ref.params_len() == cfg.params_len()
    for i, op in enumerate(ref.hidden):
        assert w.op_kind(i) == op.kind
        if hasattr(op, "units"):
            for k, u in enumerate(op.units):
                u.weights[...] = w.read(i, "u%d.weights" % k).reshape(u.weights.shape)
                assert u.weights.any()
                # Kaiming: N(0, 2 / fan_in)
                fan_in = u.weights[0].size
                if u.weights.size >= 500:   # enough samples for the estimate to be within a quarter
                    assert abs(float(u.weights.std()) / np.sqrt(2.0 / fan_in) - 1.0) < 0.25
                assert np.array_equal(w.read(i, "u%d.bn_scale" % k), np.ones_like(u.scale))
                assert not w.read(i, "u%d.bn_bias" % k).any() and not w.read(i, "u%d.bn_running_mean" % k).any()
                assert np.array_equal(w.read(i, "u%d.bn_running_ivar" % k), np.ones_like(u.scale))
                # a non-trivial affine part, so a swapped scale / bias or a dropped term shows
                u.scale[...] = 1.0 + 0.25 * synth.normal(seed, 300 + 10 * i + k, u.scale.shape)
                u.bias[...] = 0.25 * synth.normal(seed, 400 + 10 * i + k, u.bias.shape)
                w.write(i, "u%d.bn_scale" % k, u.scale)
                w.write(i, "u%d.bn_bias" % k, u.bias)
        elif op.p is not None:
            op.p.weights[...] = w.read(i, "weights").reshape(op.p.weights.shape)
            op.p.bias[...] = w.read(i, "bias")
    return w, ref


def check_forward(w, ref, x, batch, training, t, tag, teacher=False):
    """teacher: every operator of the restatement starts from the GPU's input to that operator, so the comparison
    is per operator (a 20-convolution chain otherwise compounds last-bit differences past the per-tensor bound)."""
    w.load_frames_f32(x)
    w.forward(batch, training=training, t=t)
    n = len(ref.hidden)
    if teacher:
        act = x
        for i, op in enumerate(ref.hidden):
            op.forward(act, training, t) if getattr(op, "wants_phase", False) else op.forward(act)
            act = w.read(i, "out_act").reshape(op.out_act.shape)
        ref.out_values = O.softmax_fwd(np.ascontiguousarray(act.reshape(batch, -1)))
    else:
        ref.forward(x, training=training, t=t)
    for i, op in enumerate(ref.hidden):
        what = "%s [%d] %s" % (tag, i, op.kind)
        for k, u in enumerate(getattr(op, "units", ())):
            assert_close(w.read(i, "u%d.pre_act" % k), u.pre_act.ravel(), "%s unit %d conv output" % (what, k))
            if training:
                assert_close(w.read(i, "u%d.bn_cached_mean" % k), u.cached_mean, "%s unit %d batch mean" % (what, k))
                assert_close(w.read(i, "u%d.bn_cached_ivar" % k), u.cached_ivar, "%s unit %d batch ivar" % (what, k))
            assert_close(w.read(i, "u%d.bn_running_mean" % k), u.running_mean, "%s unit %d running mean" % (what, k))
            assert_close(w.read(i, "u%d.bn_running_ivar" % k), u.running_ivar, "%s unit %d running ivar" % (what, k))
        if hasattr(op, "mid_act"):
            assert_close(w.read(i, "mid_act"), op.mid_act.ravel(), what + " mid_act")
        assert_close(w.read(i, "out_act"), op.out_act.ravel(), what + " out_act")
    assert_close(w.read(n, "out_act"), ref.out_values.ravel(), tag + " softmax", atol=1e-7)


def check_step(w, ref, sgd, rsgd, x, labels, fused_sgd, tag, teacher=False):
    batch = x.shape[0]
    w.stage_batch(labels, 1.0 / batch)
    ref.stage_batch(labels, 1.0 / batch)
    check_forward(w, ref, x, batch, True, sgd.iter_counter(), tag, teacher)
    n = len(ref.hidden)
    loss = w.store_loss(batch)
    assert_close(np.array([loss]), np.array([ref.store_loss()]), tag + " loss")
    w.backward(batch)
    # backward, operator by operator, from the GPU's forward state (max-pool routing and ReLU masks are
    # discontinuous in the activations)
    prev = x
    for i, op in enumerate(ref.hidden):
        for k, u in enumerate(getattr(op, "units", ())):
            u.pre_act = w.read(i, "u%d.pre_act" % k).reshape(u.pre_act.shape).copy()
            u.cached_mean, u.cached_ivar = w.read(i, "u%d.bn_cached_mean" % k), w.read(i, "u%d.bn_cached_ivar" % k)
        if hasattr(op, "mid_act"):
            op.mid_act = w.read(i, "mid_act").reshape(op.mid_act.shape).copy()
        if hasattr(op, "units"):
            first_in = np.ascontiguousarray(prev.reshape(op.units[0].x_shape))
            op.units[0].in_act = first_in
            if len(op.units) > 1:
                op.units[1].in_act = op.mid_act
            if len(op.units) > 2:
                op.units[2].in_act = first_in
        else:
            op.in_act = np.ascontiguousarray(prev.reshape(op.in_act.shape))
        op.out_act = w.read(i, "out_act").reshape(op.out_act.shape).copy()
        prev = op.out_act
    ref.out_values = w.read(n, "out_act").reshape(batch, -1).copy()
    delta = O.softmax_kl_backward(ref.out_values, ref.labels, ref.weights)
    for i in range(n - 1, -1, -1):
        op = ref.hidden[i]
        what = "%s [%d] %s" % (tag, i, op.kind)
        d = np.ascontiguousarray(delta.reshape(op.out_act.shape))
        if getattr(op, "act", None) == "Rect":
            O.rect_backprop_inplace(op.out_act, d)
        got = w.read(i, "out_delta")
        assert_close(got, d.ravel(), what + " out_delta")
        op.out_delta = got.reshape(op.out_act.shape).copy()
        delta = op.backward(want_in_delta=i > 0)
        if hasattr(op, "units"):
            if hasattr(op, "mid_delta"):
                # with fused epilogues the device keeps mid_delta as it was before the ReLU mask (the mask is applied
                # inside the first unit's batch-norm backward); the reference masks it in place
                got_mid = w.read(i, "mid_delta").reshape(op.mid_act.shape).copy()
                if getattr(op, "act", None) == "Rect":
                    O.rect_backprop_inplace(op.mid_act, got_mid)
                assert_close(got_mid.ravel(), op.mid_delta.ravel(), what + " mid_delta")
            for k, u in enumerate(op.units):
                assert_close(w.read(i, "u%d.pre_delta" % k), u.pre_delta.ravel(), "%s unit %d pre_delta" % (what, k))
                for gname, rname in UNIT_GRADS:
                    assert_close(w.read(i, "u%d.%s" % (k, gname)), getattr(u, rname).ravel(), "%s unit %d %s" % (what, k, gname))
        elif op.p is not None:
            assert_close(w.read(i, "grad_weights"), op.p.grad_weights.ravel(), what + " grad_weights")
            assert_close(w.read(i, "grad_bias"), op.p.grad_bias.ravel(), what + " grad_bias")
    sgd.step(w, fused=fused_sgd)
    rsgd.step(ref)
    for i, op in enumerate(ref.hidden):
        what = "%s [%d] %s" % (tag, i, op.kind)
        for k, u in enumerate(getattr(op, "units", ())):
            for gname, rname in UNIT_ACCS + UNIT_PARAMS:
                assert_close(w.read(i, "u%d.%s" % (k, gname)), getattr(u, rname).ravel(), "%s unit %d %s" % (what, k, gname))
            for gname, _ in UNIT_GRADS:
                assert not w.read(i, "u%d.%s" % (k, gname)).any(), "reset() zeroes the gradients"


@pytest.mark.parametrize("fuse,fused_sgd,flavour", [(True, True, "Update"), (False, False, "Update"), (True, False, "GradientNesterov")])
def test_bnorm_residual_train_steps(dev, fuse, fused_sgd, flavour):
    """BNormConv2d -> max-pool -> StackRes -> ProjStackRes (stride 2) -> ProjStackRes (stride 1, wider) -> StackRes ->
    global average pool -> affine: 3 steps with weight decay (which must reach the filters only) and momentum."""
    net, batch = small_net(), 8
    say("bnorm residual steps", fuse, fused_sgd, flavour)
    w, ref = make_pair(net, batch, 0xB4001, fuse)
    assert [w.op_kind(i) for i in (0, 2, 3)] == ["BNormConv2dOperator", "StackResConv2dOperator", "ProjStackResConv2dOperator"]
    sgd = SgdOpt(batch, 0.05, (flavour, 0.9), 1e-3)
    rsgd = OG.SgdOpt(0.05, (flavour, 0.9), 1e-3)
    sgd.begin(w)
    rsgd.begin(ref)
    for step in range(3):
        x = synth.normal(0xB4001, 100 + step, (batch, 3, 16, 16))
        labels = synth.integers(0xB4001, 200 + step, (batch,), 5)
        check_step(w, ref, sgd, rsgd, x, labels, fused_sgd, "bnorm step %d" % step)
    # the moving statistics now differ from their initial values; inference uses them, and leaves them alone
    before = w.read(2, "u1.bn_running_mean").copy()
    assert before.any()
    x = synth.normal(0xB4001, 150, (batch, 3, 16, 16))
    check_forward(w, ref, x, batch, False, 0, "bnorm inference")
    assert np.array_equal(w.read(2, "u1.bn_running_mean"), before)
    w.close()


def test_random_bnorm_residual_networks(dev):
    """Seeded sweep over chains of the batch-normalised operators: a first conv + batch norm (filter 1-5, stride 1-2),
    one to three stacked / projecting residual operators (Rect or Identity, stride 1-2, changing widths) with pooling
    around them; fused or reference-order epilogues and SGD, four momentum flavours; two checked steps each.
    (At least three input channels: a 1x1 filter on one channel makes the conv output a multiple of x, which the
    batch-norm backward projects out, and the filter gradient would be rounding noise around zero.)"""
    import random
    rnd = random.Random(20160420)
    for it in range(12):
        dims = (rnd.choice([8, 12, 16, 20]), rnd.choice([8, 12, 16]), rnd.choice([3, 4, 8]))
        w_, h_ = dims[0], dims[1]
        k, st = rnd.choice([1, 3, 5]), rnd.choice([1, 2])
        spec = [("bnconv", k, st, k // 2, rnd.choice([4, 8, 12, 16]), rnd.choice(["Rect", "Identity"]))]
        w_, h_ = (w_ + 2 * (k // 2) - k) // st + 1, (h_ + 2 * (k // 2) - k) // st + 1
        if rnd.random() < 0.5 and w_ >= 4 and h_ >= 4 and w_ % 2 == 0 and h_ % 2 == 0:
            spec.append(("pool", 2, 2, 0, "Max"))
            w_, h_ = w_ // 2, h_ // 2
        for _ in range(rnd.randint(1, 3)):
            if rnd.random() < 0.45:
                spec.append(("res", rnd.choice(["Rect", "Rect", "Identity"])))
            else:
                st2 = rnd.choice([1, 2]) if min(w_, h_) >= 4 and w_ % 2 == 0 and h_ % 2 == 0 else 1
                spec.append(("projres", rnd.choice([8, 12, 16, 24]), st2, rnd.choice(["Rect", "Rect", "Identity"])))
                w_, h_ = w_ // st2, h_ // st2
        if rnd.random() < 0.5 and w_ >= 2 and h_ >= 2:
            spec.append(("pool", min(w_, h_), 1, 0, "Average"))
        ncat = rnd.choice([3, 5])
        spec.append(("fc", ncat, "Identity"))
        batch = rnd.choice([4, 8, 13])
        fuse, fused_sgd = rnd.random() < 0.7, rnd.random() < 0.6
        flavour = rnd.choice(["Update", "GradientNesterov", "Gradient", "UpdateNesterov"])
        say("random bnorm net", it, dims, spec, batch, fuse, fused_sgd, flavour)
        net = (dims, *configs._chain(dims, spec))
        w, ref = make_pair(net, batch, 2000 + it, fuse)
        sgd = SgdOpt(batch, 0.05, (flavour, 0.9), 1e-3)
        rsgd = OG.SgdOpt(0.05, (flavour, 0.9), 1e-3)
        sgd.begin(w)
        rsgd.begin(ref)
        for step in range(2):
            x = synth.normal(2000 + it, 100 + step, (batch, dims[2], dims[1], dims[0]))
            labels = synth.integers(2000 + it, 200 + step, (batch,), ncat)
            check_step(w, ref, sgd, rsgd, x, labels, fused_sgd, "random bnorm net %d step %d" % (it, step))
        w.close()


def test_bnorm_cumulative_average_and_save_restore(dev):
    """Cumulative moving average (newest batch weighs 1/(1+t)): after forward passes at t = 0, 1, 2 the moving mean is
    the plain average of the three batch means; save_params / restore_params carry the moving statistics."""
    net, batch = small_net(), 8
    w, ref = make_pair(net, batch, 0xB4002, True, mov_avg="Cumulative")
    means = []
    for t in range(3):
        x = synth.normal(0xB4002, 100 + t, (batch, 3, 16, 16))
        check_forward(w, ref, x, batch, True, t, "cumulative t=%d" % t)
        means.append(w.read(0, "u0.bn_cached_mean").astype(np.float64))
    np.testing.assert_allclose(w.read(0, "u0.bn_running_mean"), np.mean(means, axis=0), rtol=1e-5, atol=1e-6)
    w.save_params()
    ref.save_params()
    saved = w.read(0, "u0.bn_running_ivar").copy()
    x = synth.normal(0xB4002, 103, (batch, 3, 16, 16))
    check_forward(w, ref, x, batch, True, 1, "cumulative after save")
    assert not np.array_equal(w.read(0, "u0.bn_running_ivar"), saved)
    w.restore_params()
    ref.restore_params()
    assert np.array_equal(w.read(0, "u0.bn_running_ivar"), saved)
    check_forward(w, ref, x, batch, False, 0, "inference after restore")
    w.close()


def _parse_blob(blob):
    out, off = [], 0
    while off < len(blob):
        assert blob[off:off + 4] == b"ND\x00\x01"
        (nd,) = struct.unpack_from("<I", blob, off + 4)
        dims = struct.unpack_from("<%dQ" % nd, blob, off + 8)
        off += 8 + 8 * nd
        n = int(np.prod(dims))
        out.append((dims, np.frombuffer(blob, "<f4", n, off).copy()))
        off += 4 * n
    return out


def test_bnorm_param_and_state_blobs(dev):
    """encode_params: per unit the filter as (R*S*C, K) then scale, bias, moving mean, moving inverse deviation as
    (1, K) rows; encode_state: momentum of filter / scale / bias, then the cached batch mean and inverse deviation
    (src/operator/conv.rs:361-459, 1340-1480).  decode_* restore a second worker to the same buffers."""
    net, batch = small_net(), 4
    w, ref = make_pair(net, batch, 0xB4003, True)
    sgd = SgdOpt(batch, 0.05, ("Update", 0.9), 0.0)
    sgd.begin(w)
    x = synth.normal(0xB4003, 100, (batch, 3, 16, 16))
    w.load_frames_f32(x)
    w.stage_batch(synth.integers(0xB4003, 200, (batch,), 5), 1.0 / batch)
    w.forward(batch, training=True, t=0)
    w.backward(batch)
    sgd.step(w, fused=True)
    arrays = _parse_blob(w.encode_params())
    state = _parse_blob(w.encode_state())
    # the worker's state blob holds, operator by operator, the parameter arrays and then the optimizer state
    names = ("weights", "bn_scale", "bn_bias", "bn_running_mean", "bn_running_ivar")
    snames = ("acc_grad_weights", "acc_bn_scale_grad", "acc_bn_bias_grad", "bn_cached_mean", "bn_cached_ivar")
    def walk(arrs, pos, i, units, part):
        for k, u in enumerate(units):
            K, Cc, R, _ = u.weights.shape
            for j, nm in enumerate(part):
                dims, vals = arrs[pos]
                assert dims == ((R * R * Cc, K) if j == 0 else (1, K)), (i, k, nm)
                assert np.array_equal(vals, w.read(i, "u%d.%s" % (k, nm))), (i, k, nm)
                pos += 1
        return pos

    pos = spos = 0
    for i, op in enumerate(ref.hidden):
        units = getattr(op, "units", ())
        if units:
            pos = walk(arrays, pos, i, units, names)
            spos = walk(state, spos, i, units, names)
            spos = walk(state, spos, i, units, snames)
        elif op.p is not None:
            pos += 2
            spos += 4
    assert pos == len(arrays) and spos == len(state)
    cfg = configs.build_config(net)
    w2 = SequentialOperatorWorker(cfg, batch, "Backward", shared_seed=(7, 8))
    w2.init_params()
    assert w2.decode_params(w.encode_params()) == len(w.encode_params())
    w2.decode_state(w.encode_state())
    for i, op in enumerate(ref.hidden):
        for k, _ in enumerate(getattr(op, "units", ())):
            for nm in ("weights", "bn_scale", "bn_bias", "bn_running_mean", "bn_running_ivar", "acc_grad_weights",
                       "acc_bn_scale_grad", "acc_bn_bias_grad", "bn_cached_mean", "bn_cached_ivar"):
                assert np.array_equal(w2.read(i, "u%d.%s" % (k, nm)), w.read(i, "u%d.%s" % (k, nm))), nm
    w.close()
    w2.close()


def test_bnorm_training_needs_backward_capability(dev):
    """A Forward-only worker runs inference; the training phase panics as in the reference
    ("batch norm training missing backward operator", src/operator/conv.rs:508-511)."""
    from rembrandt_amd.operator import Panic
    net, batch = small_net(), 4
    cfg = configs.build_config(net)
    w = SequentialOperatorWorker(cfg, batch, "Forward", shared_seed=(3, 4))
    w.init_params()
    w.load_frames_f32(synth.normal(5, 1, (batch, 3, 16, 16)))
    w.forward(batch, training=False, t=0)
    assert np.isfinite(w.read(len(net[1]), "out_act")).all()
    with pytest.raises(Panic, match="batch norm training missing backward operator"):
        w.forward(batch, training=True, t=0)
    w.close()


def test_resnet18_train_step(dev):
    """The reference's ResNet-18 template (src/templates/resnet.rs:367-520) at full geometry, batch 2: one step."""
    net, batch = configs.resnet18(), 2
    say("resnet18 step")
    w, ref = make_pair(net, batch, 0xB4018, True)
    assert w.hidden_count() == 12 and configs.build_config(net).params_len() == ref.params_len()
    sgd = SgdOpt(batch, 0.01, ("Update", 0.9), 1e-4)
    rsgd = OG.SgdOpt(0.01, ("Update", 0.9), 1e-4)
    sgd.begin(w)
    rsgd.begin(ref)
    x = synth.normal(0xB4018, 100, (batch, 3, 224, 224))
    labels = synth.integers(0xB4018, 200, (batch,), 1000)
    check_step(w, ref, sgd, rsgd, x, labels, True, "resnet18 step 0", teacher=True)
    w.close()
