"""GPU parity of the second-generation layer / arch API over the operator chain (src/layer_new.rs:537-617, 1044-1154;
src/arch_new.rs:527-552; src/opt_new.rs:279-325): backward(batch, scale), descend(scale, l2), reset_gradients(momentum),
where the gradient buffers double as the momentum buffers, and the device-side accumulated loss.  Against
oracle.graph's restatement (itself pinned against a torch SGD trajectory by the CPU tests), checkpoint by checkpoint;
activations are teacher-forced before each backward pass because max-pool routing is discontinuous."""
import numpy as np
import pytest

from oracle import graph as OG
from rembrandt_amd import configs, synth
from rembrandt_amd.operator import Panic, SequentialOperatorWorker, SgdOptimization
from conftest import assert_close, say

pytestmark = pytest.mark.gpu

DIMS = (14, 14, 3)
SPEC = [("conv", 3, 1, 1, 8, "Rect"), ("pool", 2, 2, 0, "Max"), ("conv", 3, 2, 1, 12, "Rect"), ("fc", 32, "Rect"),
        ("fc", 7, "Identity")]


def make_pair(batch, seed, fuse, overlap=True):
    net = (DIMS, *configs._chain(DIMS, SPEC))
    dims, layers, ncat = net
    w = SequentialOperatorWorker(configs.build_config(net, init_std=0.2), batch, "Backward", shared_seed=(seed, seed + 1),
                                 fuse_epilogue=fuse, overlap_backward=overlap)
    w.init_params()
    ref = OG.SequentialOperatorWorker(layers, ncat, batch)
    for i, op in enumerate(ref.hidden):
        if op.p is not None:
            op.p.weights[...] = w.read(i, "weights").reshape(op.p.weights.shape)
            op.p.bias[...] = synth.normal(seed, 50 + i, op.p.bias.shape) * 0.1
            w.write(i, "bias", op.p.bias)
    return w, ref, ncat


def compare_forward_then_teacher_force(w, ref, x, batch, tag):
    for i, op in enumerate(ref.hidden):
        assert_close(w.read(i, "out_act"), op.out_act.ravel(), "%s out_act[%d]" % (tag, i))
    n = len(ref.hidden)
    assert_close(w.read(n, "out_act"), ref.out_values.ravel(), tag + " softmax", atol=1e-7)
    prev = x
    for i, op in enumerate(ref.hidden):
        op.in_act = np.ascontiguousarray(prev.reshape(op.in_act.shape))
        op.out_act = w.read(i, "out_act").reshape(op.out_act.shape).copy()
        prev = op.out_act
    ref.out_values = w.read(n, "out_act").reshape(batch, -1).copy()


def compare_params(w, ref, tag, names=("grad_weights", "grad_bias", "weights", "bias")):
    for i, op in enumerate(ref.hidden):
        if op.p is None:
            continue
        for k in names:
            assert_close(w.read(i, k), getattr(op.p, k).ravel(), "%s %s[%d]" % (tag, k, i))


@pytest.mark.parametrize("fuse,fused_descend", [(True, True), (False, False)])
def test_second_generation_minibatches(dev, fuse, fused_descend):
    """SgdOptimization: 3 minibatches of 2 batches each, per-sample weights 1, momentum in the gradient buffers."""
    batch, m = 8, 16
    eta, mu, l2 = 0.2, 0.9, 1e-2
    w, ref, ncat = make_pair(batch, 501, fuse)
    sgd, rsgd = SgdOptimization(m, eta, mu, l2), OG.SgdOptimization(m, eta, mu, l2)
    sgd.begin(w)
    rsgd.begin(ref)
    for t in range(3):
        for k in range(2):
            tag = "gen2 minibatch %d batch %d" % (t, k)
            say(tag, "fuse", fuse, "fused descend", fused_descend)
            x = synth.normal(501, 100 + 2 * t + k, (batch, DIMS[2], DIMS[1], DIMS[0]))
            labels = synth.integers(501, 200 + 2 * t + k, (batch,), ncat)
            w.load_frames_f32(x)
            w.stage_batch(labels, 1.0)
            ref.stage_batch(labels, 1.0)
            # the driver's batch() on the GPU; the same three calls on the oracle with the activations forced in between
            sgd.batch(w, batch)
            ref.forward(x)
            compare_forward_then_teacher_force(w, ref, x, batch, tag)
            ref.backward_scaled(1.0)
            ref.accumulate_loss()
            for i, op in enumerate(ref.hidden):
                assert_close(w.read(i, "out_delta"), op.out_delta.ravel(), "%s out_delta[%d]" % (tag, i))
            compare_params(w, ref, tag, ("grad_weights", "grad_bias"))
        assert_close(np.array([w.store_accumulated_loss()]), ref.acc_loss, "gen2 accumulated loss, minibatch %d" % t)
        sgd.end_minibatch(w, fused=fused_descend)
        rsgd.end_minibatch(ref)
        compare_params(w, ref, "gen2 after minibatch %d" % t)
        assert sgd.iter_counter() == rsgd.t == t + 1
    # the velocity is what reset_gradients left in the gradient buffers: non-zero, unlike after the operator API's reset()
    assert np.abs(w.read(0, "grad_weights")).max() > 0
    w.reset_loss(batch)
    assert w.store_accumulated_loss() == 0.0
    w.close()


def test_second_generation_scaled_backward(dev):
    """backward(batch, scale) with scale != 1 through the worker: convolutions accumulate scale * gradient, affine
    layers accumulate with factor 1 (as the reference's do), deltas are unscaled; on both stream placements."""
    batch = 6
    for overlap in (True, False):
        w, ref, ncat = make_pair(batch, 502, True, overlap)
        x = synth.normal(502, 100, (batch, DIMS[2], DIMS[1], DIMS[0]))
        labels = synth.integers(502, 200, (batch,), ncat)
        w.load_frames_f32(x)
        w.stage_batch(labels, 1.0)
        ref.stage_batch(labels, 1.0)
        w.reset_gradients(0.0)
        for rep, scale in enumerate((0.25, -2.0)):
            say("gen2 scaled backward", scale, "overlap", overlap)
            w.forward(batch, training=True, t=0)
            ref.forward(x)
            compare_forward_then_teacher_force(w, ref, x, batch, "gen2 scale %g" % scale)
            w.backward_scaled(batch, scale)
            ref.backward_scaled(scale)
            for i, op in enumerate(ref.hidden):
                assert_close(w.read(i, "out_delta"), op.out_delta.ravel(), "gen2 scale %g out_delta[%d]" % (scale, i))
            compare_params(w, ref, "gen2 scale %g" % scale, ("grad_weights", "grad_bias"))
        w.descend(0.05, 0.0, fused=True)
        ref.descend(0.05, 0.0)
        compare_params(w, ref, "gen2 descend without l2")
        w.close()


def test_second_generation_refused_for_batch_normalised_operators(dev):
    """The second-generation layer set has no batch-normalised layers; the update is refused, not skipped."""
    dims = (8, 8, 3)
    net = (dims, *configs._chain(dims, [("bnconv", 3, 1, 1, 4, "Rect"), ("fc", 3, "Identity")]))
    w = SequentialOperatorWorker(configs.build_config(net), 4, "Backward", shared_seed=(5, 6))
    w.init_params()
    with pytest.raises(Panic):
        w.descend(0.1, 0.0)
    with pytest.raises(Panic):
        w.reset_gradients(0.9)
    w.close()
