"""GPU parity of whole train steps at the sizes the benchmark times: the AlexNet-shaped chain at batch 256 and the
NIN-shaped chain at batch 128, driven exactly as bench.py drives them (rho_sgd_train_batch: fused epilogues, filter /
bias gradients on the second stream, fused SGD steps on the second stream joined lazily by the next forward pass).

The CPU oracle cannot recompute these tensors whole in seconds, so every operator is checked *teacher-forced* from the
GPU's own inputs to it (the buffers of the neighbouring operators, read back after the step) on
  * a random sample of elements, plus elements on the seams of the kernels' tiles, through the oracle's `*_at` functions
    (convolution forward, data and filter gradients),
  * whole sampled planes for the pooling operators, whole tensors for the affine operators (numpy fp64),
  * loss, predicted categories (exact) and accuracy count (exact) from the GPU's own probabilities.
Gradients are zeroed by the fused update, so they are checked through what the update leaves:
v_t = mu*v_{t-1} - eta*g_t on sampled elements, W_t = W_{t-1} + v_t on all of them, bit for bit.
A second worker runs the same steps back to back without any read-back in between (reading a buffer joins the
streams), and must end with bit-identical parameters: the cross-step overlap changes nothing.
The worst absolute / relative error per checked tensor is printed and written to parity_<net>_b<batch>.json in the output folder of the run.
"""
import json
import os

import numpy as np
import pytest

import oracle as O
from rembrandt_amd import configs, synth
from rembrandt_amd.operator import SequentialOperatorWorker, SgdOpt
import conftest
from conftest import assert_close, say

pytestmark = pytest.mark.gpu

ETA, MU = 0.01, 0.9


class ErrorLog:
    def __init__(self):
        self.rows = []

    def check(self, got, ref, what, **kw):
        got64, ref64 = np.asarray(got, np.float64).ravel(), np.asarray(ref, np.float64).ravel()
        err = np.abs(got64 - ref64)
        scale = float(np.sqrt(np.mean(ref64 * ref64))) if ref64.size else 0.0
        big = np.abs(ref64) > 1e-3 * scale if scale > 0 else np.zeros(ref64.shape, bool)
        row = {"tensor": what, "checked": int(ref64.size), "max_abs_err": float(err.max()) if err.size else 0.0,
               "rms_ref": scale, "max_rel_err": float((err[big] / np.abs(ref64[big])).max()) if big.any() else 0.0}
        self.rows.append(row)
        try:
            assert_close(got, ref, what, **kw)
        finally:
            row["max_err_over_scaled_bound"] = conftest.LAST["tight_ratio"]
            say("  parity %-44s n=%-9d max_abs %.3g  max_rel %.3g  (rms %.3g)  x scaled bound %.3g" % (
                what, row["checked"], row["max_abs_err"], row["max_rel_err"], scale, row["max_err_over_scaled_bound"]))

    def exact(self, got, ref, what):
        ok = np.array_equal(got, ref)
        self.rows.append({"tensor": what, "checked": int(np.asarray(ref).size), "exact": bool(ok)})
        say("  parity %-44s n=%-9d exact %s" % (what, np.asarray(ref).size, ok))
        assert ok, what


TOLERANCE_TEXT = ("|got-ref| <= 1e-5*max(1, rms(ref)) + 1e-4*|ref|, relative L2 <= 1e-4, and |got-ref| <= %g * (1e-5*rms(ref) + "
                  "1e-4*|ref|) element by element; integers exact" % conftest.TIGHT_MULTIPLE)


def parity_summary(rec):
    """The per-tensor records of one run by tensor class, as text: what profiles/<net>_b<batch>_train_step_parity.md holds."""
    import collections
    import re
    cls = collections.OrderedDict()
    for t in rec["tensors"]:
        m = re.match(r"\S+ b\d+ step \d+ (.*)", t["tensor"])
        key = re.sub(r"\[\d+\]", "", m.group(1) if m else t["tensor"])
        c = cls.setdefault(key, {"tensors": 0, "checked": 0, "exact": True, "max_abs_err": 0.0, "max_abs_err_over_rms": 0.0,
                                 "max_rel_err": 0.0, "max_err_over_scaled_bound": 0.0})
        c["tensors"] += 1
        c["checked"] += t.get("checked", 0)
        if not t.get("exact", False):
            c["exact"] = False
            c["max_abs_err"] = max(c["max_abs_err"], t["max_abs_err"])
            c["max_abs_err_over_rms"] = max(c["max_abs_err_over_rms"], t["max_abs_err"] / max(t["rms_ref"], 1e-30))
            c["max_rel_err"] = max(c["max_rel_err"], t["max_rel_err"])
            c["max_err_over_scaled_bound"] = max(c["max_err_over_scaled_bound"], t.get("max_err_over_scaled_bound", 0.0))
    out = {"workload": rec["workload"], "batch": rec["batch"], "steps": rec["steps"], "library": rec.get("library"),
           "classes": cls}
    lines = ["# %s-shaped batch-%d train steps as bench.py runs them: worst error per tensor class against the CPU oracle"
             % (rec["workload"], rec["batch"]), "",
             "Command (MI355X box, repository root):", "",
             "    python -m pytest tests/test_gpu_bench_size.py -m gpu -q", "",
             "The test writes `gpurun_out/parity_%s_b%d.json` (one record per checked tensor) and this summary by tensor class "
             "(`gpurun_out/%s_b%d_train_step_parity.md`)." % (rec["workload"], rec["batch"], rec["workload"], rec["batch"]),
             "Tolerance of the test: " + rec["tolerance"] + ".",
             "`max_rel_err` is the largest |got-ref|/|ref| over the checked elements whose |ref| exceeds a thousandth of the",
             "tensor's RMS, `max_abs_err_over_rms` the largest |got-ref| over the tensor's RMS, `x scaled bound` the largest",
             "|got-ref| / (1e-5*rms(ref) + 1e-4*|ref|): the tolerance with its absolute term shrunk to the tensor's own scale.", "",
             "| tensor class | tensors | elements checked | exact | max abs err | max abs err / rms | max rel err | x scaled bound |",
             "|---|---:|---:|---|---:|---:|---:|---:|"]
    for k, c in cls.items():
        f = (lambda v: "" if c["exact"] else "%.3g" % v)
        lines.append("| %s | %d | %d | %s | %s | %s | %s | %s |" % (
            k, c["tensors"], c["checked"], "yes" if c["exact"] else "", f(c["max_abs_err"]), f(c["max_abs_err_over_rms"]),
            f(c["max_rel_err"]), f(c["max_err_over_scaled_bound"])))
    lines += ["", "```json", json.dumps(out, indent=1), "```", ""]
    return "\n".join(lines)


def sample_idx(rng, total, n):
    idx = rng.integers(0, total, min(n, total)).astype(np.int64)
    idx[0], idx[-1] = 0, total - 1
    return idx


def edge_idx(rng, shape, n):
    """Elements of an NCHW tensor on the seams of the kernels' tiles: channel and column (image * plane + pixel)
    positions either side of multiples of 32, where an indexing mistake would touch only a few elements."""
    Nn, K, P, Q = shape
    inner, cols = P * Q, Nn * P * Q
    c = 32 * rng.integers(0, (cols + 31) // 32 + 1, n) + rng.integers(-1, 2, n)
    r = 32 * rng.integers(0, (K + 31) // 32 + 1, n) + rng.integers(-1, 1, n)
    c = np.clip(c, 0, cols - 1).astype(np.int64)
    r = np.clip(r, 0, K - 1).astype(np.int64)
    return (c // inner) * (K * inner) + r * inner + c % inner


def read_params(w, layers):
    out = {}
    for i, l in enumerate(layers):
        if l[0] in ("conv2d", "affine"):
            out[i] = {k: w.read(i, k) for k in ("weights", "bias", "acc_grad_weights", "acc_grad_bias")}
    return out


def read_fwd_params(w, layers):
    return {i: {k: w.read(i, k) for k in ("weights", "bias")} for i, l in enumerate(layers) if l[0] in ("conv2d", "affine")}


def layer_shapes(layers, batch, dims):
    """(x_shape, y_shape) per layer, NCHW."""
    shapes = []
    for l in layers:
        if l[0] == "conv2d":
            (w_, h_, c_), k, st, pad, out = l[1], l[2], l[3], l[4], l[5]
            P, Q = O.out_dim(h_, k, st, pad), O.out_dim(w_, k, st, pad)
            shapes.append(((batch, c_, h_, w_), (batch, out, P, Q)))
        elif l[0] == "pool2d":
            (w_, h_, c_), k, st, pad = l[1], l[2], l[3], l[4]
            rnd = O.ROUND_CEIL if l[6] else O.ROUND_FLOOR
            shapes.append(((batch, c_, h_, w_), (batch, c_, O.out_dim(h_, k, st, pad, rnd), O.out_dim(w_, k, st, pad, rnd))))
        elif l[0] == "affine":
            shapes.append(((batch, l[1]), (batch, l[2])))
        else:
            raise AssertionError("layer type %s is not part of the benchmark chains" % l[0])
    return shapes


def act_of(l):
    return l[6] if l[0] == "conv2d" else l[3] if l[0] == "affine" else "Identity"


def check_forward(w, layers, shapes, x, batch, before, log, rng, tag):
    """Every operator's out_act from the GPU's own input to it; returns the activations and the probabilities."""
    n = len(layers)
    acts = [x] + [w.read(i, "out_act", int(np.prod(shapes[i][1]))).reshape(shapes[i][1]) for i in range(n)]
    probs = w.read(n, "out_act", batch * int(np.prod(shapes[-1][1][1:]))).reshape(batch, -1)
    # ---- forward, each operator from the GPU's own input to it, with the parameters the step started from
    for i, l in enumerate(layers):
        xin, y = np.ascontiguousarray(acts[i].reshape(shapes[i][0])), acts[i + 1]
        name = "%s fwd[%d] %s" % (tag, i, l[0])
        if l[0] == "conv2d":
            K, R = l[5], l[2]
            W_ = before[i]["weights"].reshape(K, shapes[i][0][1], R, R)
            idx = np.concatenate([sample_idx(rng, y.size, 4096), edge_idx(rng, y.shape, 2048)])
            ref = O.conv2d_fwd_at(xin, W_, l[3], l[4], idx).astype(np.float64)
            ref += before[i]["bias"].astype(np.float64)[(idx // (y.shape[2] * y.shape[3])) % K]
            if act_of(l) == "Rect":
                ref = np.maximum(ref, 0.0)
            log.check(y.ravel()[idx], ref.astype(np.float32), name + " (sampled)")
        elif l[0] == "pool2d":
            N_, C_, H_, W__ = shapes[i][0]
            planes = sample_idx(rng, N_ * C_, 64)
            mode = O.POOL_MAX if l[5] == "Max" else O.POOL_AVG
            rnd = O.ROUND_CEIL if l[6] else O.ROUND_FLOOR
            ref = O.pool2d_fwd(xin.reshape(N_ * C_, 1, H_, W__)[planes], l[2], l[3], l[4], mode, rnd)
            got = y.reshape(N_ * C_, 1, y.shape[2], y.shape[3])[planes]
            if l[5] == "Max":
                log.exact(got, ref, name + " (planes)")
            else:
                log.check(got, ref, name + " (planes)")
        else:
            W_ = before[i]["weights"].reshape(l[2], l[1]).astype(np.float64)
            ref = xin.reshape(batch, -1).astype(np.float64) @ W_.T + before[i]["bias"].astype(np.float64)
            if act_of(l) == "Rect":
                ref = np.maximum(ref, 0.0)
            log.check(y, ref.astype(np.float32), name)
    logits = np.ascontiguousarray(acts[n].reshape(batch, -1))
    log.check(probs, O.softmax_fwd(logits), tag + " softmax", atol=1e-7)
    return acts, probs


def check_step(w, layers, shapes, x, labels, batch, before, after, log, rng, tag, loss, correct):
    n = len(layers)
    acts, probs = check_forward(w, layers, shapes, x, batch, before, log, rng, tag)
    weights = np.full((batch,), 1.0 / batch, np.float32)
    ref_loss = float(O.blockreduce_sum(O.softmax_kl_loss1(probs, labels, weights).reshape(1, -1))[0])
    log.check(np.array([loss], np.float32), np.array([ref_loss], np.float32), tag + " loss")
    cats = w.get_output_categories(batch)
    log.exact(cats, np.argmax(probs, axis=1).astype(np.int32), tag + " categories")
    log.exact(np.array([correct]), np.array([int((cats == labels).sum())]), tag + " accuracy count")
    # ---- backward: out_delta of every operator as the chain leaves it (after the in-place ReLU mask)
    deltas = [w.read(i, "out_delta", int(np.prod(shapes[i][1]))).reshape(shapes[i][1]) for i in range(n)]
    ref = O.softmax_kl_backward(probs, labels, weights)
    if act_of(layers[-1]) == "Rect":
        ref = ref * (acts[n].reshape(ref.shape) > 0)
    log.check(deltas[n - 1], ref.reshape(deltas[n - 1].shape), tag + " out_delta[%d] (loss)" % (n - 1))
    for i in range(n - 1, -1, -1):
        l, xin, dy = layers[i], np.ascontiguousarray(acts[i].reshape(shapes[i][0])), deltas[i]
        name = "%s bwd[%d] %s" % (tag, i, l[0])
        mask_prev = i > 0 and act_of(layers[i - 1]) == "Rect"
        if l[0] == "conv2d":
            K, R, C_ = l[5], l[2], shapes[i][0][1]
            W_ = before[i]["weights"].reshape(K, C_, R, R)
            if i > 0:
                idx = np.concatenate([sample_idx(rng, xin.size, 4096), edge_idx(rng, tuple(shapes[i][0]), 2048)])
                ref = O.conv2d_bwd_data_at(W_, dy, shapes[i][0], l[3], l[4], idx)
                if mask_prev:
                    ref = ref * (acts[i].ravel()[idx] > 0)
                log.check(deltas[i - 1].ravel()[idx], ref, name + " in_delta (sampled)")
            idx = sample_idx(rng, W_.size, 768)
            g = O.conv2d_bwd_filter_at(xin, dy, W_.shape, l[3], l[4], idx).astype(np.float64)
            v = MU * before[i]["acc_grad_weights"][idx].astype(np.float64) - ETA * g
            log.check(after[i]["acc_grad_weights"][idx], v.astype(np.float32), name + " acc_grad_weights (sampled)")
            gb = dy.sum(axis=(0, 2, 3), dtype=np.float64)
        elif l[0] == "pool2d":
            if i == 0:
                continue
            N_, C_, H_, W__ = shapes[i][0]
            planes = sample_idx(rng, N_ * C_, 64)
            mode = O.POOL_MAX if l[5] == "Max" else O.POOL_AVG
            rnd = O.ROUND_CEIL if l[6] else O.ROUND_FLOOR
            xs = xin.reshape(N_ * C_, 1, H_, W__)[planes]
            P_, Q_ = shapes[i][1][2], shapes[i][1][3]
            ys = acts[i + 1].reshape(N_ * C_, 1, P_, Q_)[planes]
            ref = O.pool2d_bwd(xs, ys, dy.reshape(N_ * C_, 1, P_, Q_)[planes], l[2], l[3], l[4], mode, rnd)
            if mask_prev:
                ref = ref * (xs > 0)
            log.check(deltas[i - 1].reshape(N_ * C_, 1, H_, W__)[planes], ref, name + " in_delta (planes)")
            continue
        else:
            W_ = before[i]["weights"].reshape(l[2], l[1]).astype(np.float64)
            dy64 = dy.reshape(batch, -1).astype(np.float64)
            if i > 0:
                ref = dy64 @ W_
                if mask_prev:
                    ref = ref * (acts[i].reshape(ref.shape) > 0)
                log.check(deltas[i - 1], ref.astype(np.float32).reshape(deltas[i - 1].shape), name + " in_delta")
            g = dy64.T @ xin.reshape(batch, -1).astype(np.float64)          # [out][in] = the (in, out) column-major array
            v = MU * before[i]["acc_grad_weights"].astype(np.float64) - ETA * g.ravel()
            log.check(after[i]["acc_grad_weights"], v.astype(np.float32), name + " acc_grad_weights")
            gb = dy64.sum(axis=0)
        vb = MU * before[i]["acc_grad_bias"].astype(np.float64) - ETA * gb
        log.check(after[i]["acc_grad_bias"], vb.astype(np.float32), name + " acc_grad_bias")
        # the update itself, on every parameter: W_t = W_{t-1} + v_t in one fp32 rounding
        log.exact(after[i]["weights"], before[i]["weights"] + after[i]["acc_grad_weights"], name + " weights")
        log.exact(after[i]["bias"], before[i]["bias"] + after[i]["acc_grad_bias"], name + " bias")
        assert not w.read(i, "grad_weights").any() and not w.read(i, "grad_bias").any(), name + " gradients are reset"


@pytest.mark.parametrize("netname,batch", [("alexnet", 256), ("nin", 128)])
def test_bench_size_train_steps(dev, netname, batch):
    net = configs.NETWORKS[netname]()
    dims, layers, ncat = net
    seed = 0x5EED0000 + 4
    shapes = layer_shapes(layers, batch, dims)
    x = synth.normal(seed, 100, (batch, dims[2], dims[1], dims[0]))
    labels = synth.integers(seed, 200, (batch,), ncat)
    rng = np.random.default_rng(11)
    log = ErrorLog()
    steps = 2

    def make():
        w = SequentialOperatorWorker(configs.build_config(net), batch, "Backward", shared_seed=(seed, seed + 1))
        w.init_params()
        w.load_frames_f32(x)
        w.stage_batch(labels, 1.0 / batch)
        sgd = SgdOpt(batch, ETA, ("Update", MU), 0.0)
        sgd.begin(w)
        return w, sgd

    # (a) the steps back to back, as the benchmark's timed loop issues them
    say("bench-size", netname, "batch", batch, ": uninterrupted steps")
    w, sgd = make()
    for _ in range(steps):
        sgd.train_batch(w, batch, fused=True)
    final_a = read_params(w, layers)
    w.close()
    # (b) the same steps with every buffer read back and checked after each
    w, sgd = make()
    state = read_params(w, layers)
    for step in range(steps):
        say("bench-size", netname, "checked step", step)
        loss, correct = sgd.train_batch(w, batch, fused=True)
        after = read_params(w, layers)
        check_step(w, layers, shapes, x, labels, batch, state, after, log, rng, "%s b%d step %d" % (netname, batch, step),
                   loss, correct)
        state = after
    w.close()
    for i in state:
        for k in ("weights", "bias", "acc_grad_weights", "acc_grad_bias"):
            log.exact(final_a[i][k], state[i][k], "%s uninterrupted == checked run: %s[%d]" % (netname, k, i))
    try:
        os.makedirs("gpurun_out", exist_ok=True)
        from rembrandt_amd import _lib
        rec = {"workload": netname, "batch": batch, "steps": steps, "tolerance": TOLERANCE_TEXT, "tensors": log.rows,
               "library": _lib.lib().rh_version().decode()}
        with open(os.path.join("gpurun_out", "parity_%s_b%d.json" % (netname, batch)), "w") as f:
            json.dump(rec, f, indent=1)
        with open(os.path.join("gpurun_out", "%s_b%d_train_step_parity.md" % (netname, batch)), "w") as f:
            f.write(parity_summary(rec))
    except OSError:
        pass


def test_partial_batches(dev):
    """Workers built for batch_cap run any batch <= batch_cap with the scratch they allocated at construction: batch
    sizes at which the library cuts the contractions differently (and needs more scratch) than at the capacity.
    Forward-capability worker: AlexNet chain, capacity 256, batch 80 (the tail of a 50 000-image validation set) and
    batch 3.  Backward-capability workers: NIN chain, capacity 256, batch 233; LeNet chain, capacity 128, batch 125."""
    rng = np.random.default_rng(12)
    log = ErrorLog()
    net = configs.alexnet()
    dims, layers, ncat = net
    w = SequentialOperatorWorker(configs.build_config(net), 256, "Forward", shared_seed=(31, 32))
    w.init_params()
    params = read_fwd_params(w, layers)
    for batch in (80, 3):
        say("partial batch: alexnet forward worker, batch", batch)
        x = synth.normal(31, 100 + batch, (batch, dims[2], dims[1], dims[0]))
        w.load_frames_f32(x)
        w.forward(batch, training=False, t=0)
        check_forward(w, layers, layer_shapes(layers, batch, dims), x, batch, params, log, rng, "alexnet cap 256 batch %d" % batch)
    w.close()
    for name, cap, batch in (("nin", 256, 233), ("lenet", 128, 125)):
        net = configs.NETWORKS[name]()
        dims, layers, ncat = net
        say("partial batch:", name, "backward worker, capacity", cap, "batch", batch)
        w = SequentialOperatorWorker(configs.build_config(net), cap, "Backward", shared_seed=(33, 34))
        w.init_params()
        x = synth.normal(33, 100, (batch, dims[2], dims[1], dims[0]))
        labels = synth.integers(33, 200, (batch,), ncat)
        w.load_frames_f32(x)
        w.stage_batch(labels, 1.0 / batch)
        sgd = SgdOpt(batch, ETA, ("Update", MU), 0.0)
        sgd.begin(w)
        before = read_params(w, layers)
        loss, correct = sgd.train_batch(w, batch, fused=True)
        check_step(w, layers, layer_shapes(layers, batch, dims), x, labels, batch, before, read_params(w, layers), log, rng,
                   "%s cap %d batch %d" % (name, cap, batch), loss, correct)
        w.close()
