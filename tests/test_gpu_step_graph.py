"""Train steps recorded into a HIP graph and replayed (RHO_EXEC_GRAPH_STEPS) against the same steps launched kernel by
kernel: losses, correct counts and every parameter and momentum buffer bit-identical after every step, over several
replays with fresh inputs, with ordinary (non-recorded) work and synchronisation between the replays."""
import numpy as np
import pytest

from rembrandt_amd import configs, synth
from rembrandt_amd.operator import SequentialOperatorWorker, SgdOpt
from conftest import say

pytestmark = pytest.mark.gpu


def param_buffers(net, read_grads=True):
    names = []
    for i, l in enumerate(net[1]):
        if l[0] in ("conv2d", "affine"):
            names += [(i, b) for b in ("weights", "bias", "acc_grad_weights", "acc_grad_bias") + (("grad_weights",) if read_grads else ())]
        elif l[0] in ("bnorm_conv2d", "stack_res_conv2d", "proj_stack_res_conv2d"):
            units = {"bnorm_conv2d": 1, "stack_res_conv2d": 2, "proj_stack_res_conv2d": 3}[l[0]]
            for u in range(units):
                names += [(i, "u%d.%s" % (u, b)) for b in ("weights", "bn_scale", "bn_bias", "bn_running_mean", "bn_running_ivar",
                                                            "acc_grad_weights", "acc_bn_scale_grad")]
    return names


def run(net, batch, steps, graph, seed, sgd_kwargs, fused=True, toggle_at=None, read_grads=True, fuse_tail=True, extra=(),
        winograd=True):
    dims, layers, ncat = net
    w = SequentialOperatorWorker(configs.build_config(net), batch, "Backward", shared_seed=(seed, seed + 1), graph_steps=graph,
                                 fuse_tail=fuse_tail, winograd=winograd)
    w.init_params()
    sgd = SgdOpt(batch, **sgd_kwargs)
    sgd.begin(w)
    names = param_buffers(net, read_grads)
    out = []
    for step in range(steps):
        if toggle_at is not None and step == toggle_at:
            w.set_overlap_backward(False)
        x = synth.normal(seed, 100 + step, (batch, dims[2], dims[1], dims[0]))
        labels = synth.integers(seed, 200 + step, (batch,), ncat)
        w.load_frames_f32(x)
        w.stage_batch(labels, 1.0 / batch)
        loss, correct = sgd.train_batch(w, batch, fused=fused)
        # work outside the recording between two replays: blocking read-backs of every parameter buffer
        out.append((loss, correct, [w.read(i, b).copy() for (i, b) in names] + [w.read(i, b).copy() for (i, b) in extra]))
    launches = w.graph_launches()
    assert sgd.iter_counter() == steps
    w.close()
    return out, launches


def same(a, b, tag):
    assert len(a) == len(b)
    for step, ((la, ca, pa), (lb, cb, pb)) in enumerate(zip(a, b)):
        assert la == lb and ca == cb, "%s step %d: loss %r vs %r, correct %d vs %d" % (tag, step, la, lb, ca, cb)
        for k, (u, v) in enumerate(zip(pa, pb)):
            assert np.array_equal(u, v), "%s step %d: parameter buffer %d differs" % (tag, step, k)


@pytest.mark.parametrize("name,batch,steps", [("lenet", 64, 8), ("cifar10", 128, 6)])
def test_recorded_steps_equal_launched_steps(dev, name, batch, steps):
    say("step graph", name)
    net = configs.NETWORKS[name]()
    kw = dict(step_size=0.01, momentum=("Update", 0.9), l2_reg_coef=5e-4)
    eager, n0 = run(net, batch, steps, False, 0x6A01, kw)
    graph, n1 = run(net, batch, steps, True, 0x6A01, kw)
    assert n0 == 0
    assert n1 == steps - 2, "iteration 0 and 1 are launched (first sight of their keys), iteration 2 records, the rest replay"
    same(eager, graph, name)
    assert not np.array_equal(graph[-1][2][0], graph[0][2][0]), "the replays did train"


BN_NET_DIMS = (16, 16, 3)


def bn_net():
    return (BN_NET_DIMS, *configs._chain(BN_NET_DIMS, [("bnconv", 3, 1, 1, 8, "Rect"), ("pool", 2, 2, 0, "Max"), ("res", "Rect"),
                                                       ("conv", 3, 1, 1, 8, "Rect"), ("projres", 16, 2, "Rect"),
                                                       ("pool", 4, 1, 0, "Average"), ("fc", 5, "Identity")]))


@pytest.mark.parametrize("name,batch,steps", [("lenet", 64, 7), ("cifar10", 128, 6), ("bn", 16, 7)])
def test_recorded_steps_with_gradients_left_standing_for_zeros(dev, name, batch, steps):
    """The same comparison without ever reading a gradient buffer between steps: the fused step then leaves the gradients
    of the plain convolution and affine operators as they are (they stand for zeros, the next backward pass overwrites
    them), and the recordings are filed under, and replayed in, that state."""
    say("step graph, gradients never read", name)
    net = bn_net() if name == "bn" else configs.NETWORKS[name]()
    kw = dict(step_size=0.01, momentum=("Update", 0.9), l2_reg_coef=5e-4)
    eager, n0 = run(net, batch, steps, False, 0x6A11, kw, read_grads=False)
    graph, n1 = run(net, batch, steps, True, 0x6A11, kw, read_grads=False)
    assert n0 == 0 and n1 > 0
    same(eager, graph, name)
    # and it is the state the gradient-reading run reaches as well
    checked, _ = run(net, batch, steps, False, 0x6A11, kw, read_grads=True)
    for (la, ca, pa), (lb, cb, pb) in zip(eager, checked):
        assert la == lb and ca == cb
    names_g = param_buffers(net, True)
    names_n = param_buffers(net, False)
    for k, nb in enumerate(names_n):
        assert np.array_equal(eager[-1][2][k], checked[-1][2][names_g.index(nb)]), nb


def test_recorded_steps_with_schedule_nesterov_and_placement_switch(dev):
    """A step-size schedule (new scalars at its boundary: launched once, then recorded anew), the unfused Nesterov
    update sequence, and a switch of the backward placement half-way (drops the recordings)."""
    net = configs.lenet()
    kw = dict(momentum=("UpdateNesterov", 0.9), l2_reg_coef=1e-4,
              schedule={"kind": "Anneal1", "steps": [0.02, 0.005], "iters": [0, 5]})
    eager, _ = run(net, 32, 12, False, 0x6A02, kw, fused=False, toggle_at=9)
    graph, n = run(net, 32, 12, True, 0x6A02, kw, fused=False, toggle_at=9)
    same(eager, graph, "lenet nesterov")
    # keys: t=0 | t=1..4 (launch, record, replay x2) | t=5..8 (launch, record, replay x2) | after the switch t=9..11 (launch, record, replay)
    assert n == 3 + 3 + 2


def test_steps_that_cannot_be_recorded_are_launched(dev):
    """Dropout draws a new piece of its random stream per step and a cumulative batch-norm average changes its weight
    per step: such networks run launch by launch even with the flag, with the same results."""
    dims = (12, 12, 3)
    drop = (dims, *configs._chain(dims, [("conv", 3, 1, 1, 8, "Rect"), ("pool", 2, 2, 0, "Max"), ("dropout", 0.4), ("fc", 5, "Identity")]))
    kw = dict(step_size=0.05, momentum=("Update", 0.9), l2_reg_coef=0.0)
    eager, _ = run(drop, 16, 5, False, 0x6A03, kw)
    graph, n = run(drop, 16, 5, True, 0x6A03, kw)
    assert n == 0
    same(eager, graph, "dropout net")


def test_recorded_steps_of_a_batch_normalised_network(dev):
    """Exponential moving average: constant launch arguments from iteration 1 on."""
    dims = (16, 16, 3)
    net = (dims, *configs._chain(dims, [("bnconv", 3, 1, 1, 8, "Rect"), ("pool", 2, 2, 0, "Max"), ("res", "Rect"),
                                        ("projres", 16, 2, "Rect"), ("pool", 4, 1, 0, "Average"), ("fc", 5, "Identity")]))
    kw = dict(step_size=0.05, momentum=("Update", 0.9), l2_reg_coef=1e-3)
    eager, _ = run(net, 8, 7, False, 0x6A04, kw)
    graph, n = run(net, 8, 7, True, 0x6A04, kw)
    assert n == 7 - 2   # t=0 is not safe (first batch weighs 1), t=1 launched, t=2 records, the rest replay
    same(eager, graph, "bnorm net")


def test_recording_is_keyed_by_the_input_loader(dev):
    """The input operator casts u8 frames or copies fp32 frames depending on which loader ran last; a step recorded
    with one must not be replayed for the other.  Alternating loaders with graphs on == the same with graphs off."""
    net = configs.lenet()
    dims, layers, ncat = net
    batch = 16

    def go(graph):
        w = SequentialOperatorWorker(configs.build_config(net), batch, "Backward", shared_seed=(0x6A05, 0x6A06), graph_steps=graph)
        w.init_params()
        sgd = SgdOpt(batch, 0.02, ("Update", 0.9), 0.0)
        sgd.begin(w)
        out = []
        for step in range(10):
            labels = synth.integers(0x6A05, 200 + step, (batch,), ncat)
            if step in (4, 5, 6, 9):   # u8 frames (values 0..255, unnormalised) after fp32 steps were recorded, and back
                w.load_frames_u8(synth.integers(0x6A05, 300 + step, (batch, dims[2], dims[1], dims[0]), 4).astype(np.uint8))
            else:
                w.load_frames_f32(synth.uniform(0x6A05, 100 + step, (batch, dims[2], dims[1], dims[0])))
            w.stage_batch(labels, 1.0 / batch)
            loss, correct = sgd.train_batch(w, batch)
            out.append((loss, correct, [w.read(0, "weights").copy(), w.read(-1, "out_act").copy()]))
        n = w.graph_launches()
        w.close()
        return out, n

    eager, _ = go(False)
    graph, n = go(True)
    same(eager, graph, "alternating loaders")
    assert n > 0, "some steps did replay"


def test_schedule_that_never_repeats_a_step_size_is_launched(dev):
    """Inverse schedule: a new step size every iteration, so no key is ever seen twice; every step is launched and the
    bookkeeping of seen keys stays bounded (100 iterations > its cap)."""
    dims = (8, 8, 1)
    net = (dims, *configs._chain(dims, [("conv", 3, 1, 1, 4, "Rect"), ("fc", 3, "Identity")]))
    kw = dict(momentum=("Update", 0.9), l2_reg_coef=0.0, schedule={"kind": "Inverse", "steps": [0.05, 0.1], "iters": []})
    eager, _ = run(net, 4, 100, False, 0x6A07, kw)
    graph, n = run(net, 4, 100, True, 0x6A07, kw)
    assert n == 0
    same(eager, graph, "inverse schedule")


TAIL_DIMS = (12, 12, 3)


def tail_net(fc1_act, hidden=70):
    return (TAIL_DIMS, *configs._chain(TAIL_DIMS, [("conv", 3, 1, 1, 8, "Rect"), ("pool", 2, 2, 0, "Max"), ("fc", hidden, fc1_act),
                                                   ("fc", 5, "Identity")]))


# lenet and tail_wide have a first classifier layer of more than 2^17 weights: it keeps its tiled products and the two
# launches stand for the second layer and the loss
@pytest.mark.parametrize("name,batch,steps", [("cifar10", 128, 4), ("tail_rect", 7, 3), ("tail_identity", 33, 3),
                                              ("lenet", 64, 4), ("tail_wide", 19, 3)])
def test_classifier_tail_in_two_launches(dev, name, batch, steps):
    """Train steps whose classifier tail (affine, affine, softmax loss) runs as two launches against the same steps
    through the separate operators: same losses, correct counts, parameters, momentum, and the same activations and
    deltas in the buffers the tail's operators expose, to rounding (the two forms add in different orders); and the
    two-launch form did run."""
    import ctypes as C
    from rembrandt_amd import _lib
    from conftest import assert_close
    say("classifier tail", name, batch)
    net = (configs.NETWORKS[name]() if name in configs.NETWORKS else tail_net("Rect", 500) if name == "tail_wide"
           else tail_net("Rect" if name == "tail_rect" else "Identity"))
    from_h = name in ("lenet", "tail_wide")
    layers = net[1]
    fc = [i for i, l in enumerate(layers) if l[0] == "affine"]
    assert len(fc) >= 2 and fc[-1] == len(layers) - 1 and fc[-2] == len(layers) - 2
    extra = [(fc[-2], "out_act"), (fc[-2], "out_delta"), (fc[-1], "out_act"), (fc[-1], "out_delta"), (fc[-2] - 1, "out_delta")]
    kw = dict(step_size=0.01, momentum=("Update", 0.9), l2_reg_coef=5e-4)
    lib = _lib.lib()
    lib.rh_profile_reset(); lib.rh_profile_filter(None); lib.rh_profile_enable(1)
    try:
        fusedrun, _ = run(net, batch, steps, False, 0x7A11, kw, fuse_tail=True, extra=extra)
        n = lib.rh_profile_count()
        tag, work, ms = C.c_char_p(), C.c_double(), C.c_float()
        tags = []
        for i in range(n):
            lib.rh_profile_get(i, C.byref(tag), C.byref(work), C.byref(ms))
            tags.append(tag.value.decode())
    finally:
        lib.rh_profile_enable(0)
    assert tags.count("affine2_softmax_kl_step") == steps and tags.count("affine2_bwd_params") == steps, "the two-launch tail ran"
    assert "softmax_kl_step" not in tags and (from_h or "sgemm_skinny" not in tags)
    plain, _ = run(net, batch, steps, False, 0x7A11, kw, fuse_tail=False, extra=extra)
    for step, ((la, ca, pa), (lb, cb, pb)) in enumerate(zip(fusedrun, plain)):
        assert abs(la - lb) <= 1e-5 * max(1.0, abs(lb)), (step, la, lb)
        assert ca == cb, (step, ca, cb)
        for k, (u, v) in enumerate(zip(pa, pb)):
            assert_close(u, v, "%s step %d buffer %d" % (name, step, k))


def profile_tags(fn):
    """Runs fn() with the library's per-launch records on; returns (fn's result, list of the tags launched)."""
    import ctypes as C
    from rembrandt_amd import _lib
    lib = _lib.lib()
    lib.rh_profile_reset(); lib.rh_profile_filter(None); lib.rh_profile_enable(1)
    try:
        res = fn()
        tag, work, ms = C.c_char_p(), C.c_double(), C.c_float()
        tags = []
        for i in range(lib.rh_profile_count()):
            lib.rh_profile_get(i, C.byref(tag), C.byref(work), C.byref(ms))
            tags.append(tag.value.decode())
    finally:
        lib.rh_profile_enable(0)
        lib.rh_profile_reset()
    return res, tags


WINO_DIMS = (16, 16, 8)
WINO5_DIMS = (24, 24, 8)


def wino_net(kind):
    if kind == "plain":      # conv -> conv (ReLU backward folded into the second layer's data gradient) -> pool -> fc
        spec = [("conv", 3, 1, 1, 128, "Rect"), ("conv", 3, 1, 1, 128, "Rect"), ("conv", 3, 1, 1, 128, "Identity"),
                ("pool", 2, 2, 0, "Max"), ("fc", 10, "Identity")]
    elif kind == "five":     # a 5x5 layer of 64 -> 128 channels on 24 x 24: its forward pass in the same form (four 3x3 blocks), 576 blocks
        spec = [("conv", 3, 1, 1, 64, "Rect"), ("conv", 5, 1, 2, 128, "Rect"), ("pool", 2, 2, 0, "Max"), ("fc", 10, "Identity")]
        return (WINO5_DIMS, *configs._chain(WINO5_DIMS, spec))
    else:                    # batch-normalised residual units: their 3x3 convolutions take the same form
        spec = [("conv", 3, 1, 1, 128, "Rect"), ("res", "Rect"), ("projres", 256, 2, "Rect"), ("pool", 2, 2, 0, "Average"),
                ("fc", 10, "Identity")]
    return (WINO_DIMS, *configs._chain(WINO_DIMS, spec))


@pytest.mark.parametrize("kind", ["plain", "bnorm", "five"])
def test_winograd_steps_match_direct_steps(dev, kind):
    """Train steps whose 3x3 layers of 128 channels run in the Winograd form (all three passes, what the library picks
    by itself at this size; "five": the forward pass of a 5x5 layer) against the same steps with RHO_EXEC_DIRECT_CONV: same losses, counts,
    parameters and momentum to rounding; the Winograd kernels did run in the first and not in the second.
    Two fp32 paths that add in different orders are compared here, through ReLU masks (an activation within rounding
    of zero changes side) and bias gradients (sums of 32768 deltas that largely cancel): relative L2 distance 2e-3 after the first step, 1e-2 after
    the later ones, which start from parameters that already differ (5e-2 behind batch normalisation, whose backward
    pass subtracts means of nearly equal size: the first step, from identical parameters, is the kernels' comparison).
    Parity of the form itself against the fp64-accumulating oracle is test_conv2d_winograd and, at the benchmark's
    size through whole train steps, tests/test_gpu_bench_size.py."""
    net = wino_net(kind)
    batch, steps = 128, 3
    kw = dict(step_size=0.01, momentum=("Update", 0.9), l2_reg_coef=5e-4)
    say("winograd steps", kind)
    (a, _), tags_a = profile_tags(lambda: run(net, batch, steps, False, 0x3141, kw, read_grads=False))
    (b, _), tags_b = profile_tags(lambda: run(net, batch, steps, False, 0x3141, kw, read_grads=False, winograd=False))
    assert "conv_fwd_wino" in tags_a and "wino_transform" in tags_a
    if kind == "five":   # forward only: the backward passes of a 5x5 layer stay direct
        assert "conv_bwd_data_wino" not in tags_a and "conv_bwd_filter_wino" not in tags_a
    else:
        assert "conv_bwd_data_wino" in tags_a and "conv_bwd_filter_wino" in tags_a
    assert not any("wino" in t for t in tags_b)
    for step, ((la, ca, pa), (lb, cb, pb)) in enumerate(zip(a, b)):
        assert abs(la - lb) <= 1e-4 * max(1.0, abs(lb)), (step, la, lb)
        assert abs(ca - cb) <= 1, (step, ca, cb)
        for k, (u, v) in enumerate(zip(pa, pb)):
            u, v = u.astype(np.float64), v.astype(np.float64)
            dist = np.sqrt(((u - v) ** 2).sum()) / max(np.sqrt((v ** 2).sum()), 1e-30)
            bound = 2e-3 if step == 0 else 1e-2 if kind == "plain" else 5e-2
            assert dist <= bound, "%s step %d buffer %d: relative L2 distance %.3g" % (kind, step, k, dist)


@pytest.mark.parametrize("kind", ["plain", "five"])
def test_recorded_steps_of_winograd_networks(dev, kind):
    """Steps whose convolutions run in the Winograd form (transform launches, sliced last-round blocks with their reduction,
    the zero-bordered copy of the 5x5 form), recorded and replayed: the same bits as launched."""
    say("step graph, winograd", kind)
    net = wino_net(kind)
    kw = dict(step_size=0.01, momentum=("Update", 0.9), l2_reg_coef=5e-4)
    eager, n0 = run(net, 128, 5, False, 0x6A11, kw)
    graph, n1 = run(net, 128, 5, True, 0x6A11, kw)
    assert n0 == 0 and n1 == 3
    same(eager, graph, "winograd " + kind)
