#!/usr/bin/env python3
"""Benchmark of the hot path: AlexNet-shaped train step (forward + backward + SGD-momentum), batch 256,
fp32, on one MI355X, through the C ABI of librembrandt_hip.so.

Prints ONE JSON line: train images/sec, the roofline position of the dominant kernel (measured live
with HIP events on the stream the kernels run on), a per-kernel breakdown, and the same operator
graph timed on the host cores (CPU oracle, bounded sample) as a reported baseline.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP32_MFMA_TFLOPS = 157.3   # MI355X dense fp32 matrix peak
PEAK_BF16_MFMA_TFLOPS = 2500.0  # MI355X dense bf16 matrix peak
PEAK_HBM_GBS = 8000.0           # MI355X HBM3E

# HBM-side bytes per launch (average over the launches of one step) of the MFMA kernels come from two
# hardware-counter runs of this script under `rocprofv3 --pmc FETCH_SIZE` and `--pmc WRITE_SIZE`, each counter
# scaled by what it reads for the library's plain 256 MiB copy kernel in the same run.  A counter run cannot be
# nested inside this process, so the summary of those runs (a tracked text file) is read here; a kernel it has no
# row for reports `traffic: null`.
TRAFFIC_SUMMARY = {"alexnet": "profiles/alexnet_b256_train_step_hbm_traffic.md"}
PARITY_SUMMARY = "profiles/%s_b%d_train_step_parity.md"
TOLERANCE = "asked: rel 1e-4 / abs 1e-5 (|got-ref| <= 1e-5 + 1e-4*|ref|), indices exact.  Tested: |got-ref| <= " \
            "1e-5*max(1, rms(ref)) + 1e-4*|ref| (the absolute term grows with tensors whose values reach the tens: 1e-5 is " \
            "below the fp32 resolution of their partial sums) and relative L2 <= 1e-4 against the fp64-accumulating CPU " \
            "oracle; for tensors below unit scale (every backward tensor: values 1e-7 and smaller, where an absolute 1e-5 says " \
            "nothing) the element-wise error is held to 2 * (1e-5*rms(ref) + 1e-4*|ref|) as well, reported per tensor class " \
            "as `max_err_over_scaled_bound`; labels, arg-max, masks, counts exact"


def measured_traffic(workload, kernel):
    """Bytes per launch of `kernel` from the counter summary's table: row "| `tag` | .. | fetch KiB | write KiB |",
    scale factors from its "multiply FETCH_SIZE by F" / "multiply WRITE_SIZE by W" line."""
    import re
    rel = TRAFFIC_SUMMARY.get(workload)
    path = os.path.join(ROOT, rel) if rel else None
    if not path or not os.path.exists(path):
        return None, None
    text = open(path).read()
    f = re.search(r"multiply FETCH_SIZE by ([\d.]+)", text)
    w = re.search(r"multiply WRITE_SIZE by ([\d.]+)", text)
    row = re.search(r"^\| `%s` \|[^|]*\|\s*([\d.]+)\s*\|\s*([\d.]+)\s*\|" % re.escape(kernel), text, re.M)
    if not (f and w and row):
        return None, rel
    lib_line = re.search(r"^Library: (.*)$", text, re.M)
    from rembrandt_amd import _lib
    if not lib_line or lib_line.group(1).strip() != _lib.lib().rh_version().decode():
        rel += " (recorded with another build of the library: stale)"
    return 1024.0 * (float(f.group(1)) * float(row.group(1)) + float(w.group(1)) * float(row.group(2))), rel


def recorded_parity(workload, batch):
    """Worst error per tensor class of the benchmark-size parity test (tests/test_gpu_bench_size.py runs this very
    step and checks it against the CPU oracle; this script only reports what that test recorded)."""
    rel = PARITY_SUMMARY % (workload, batch)
    path = os.path.join(ROOT, rel)
    if not os.path.exists(path):
        return {"tolerance": TOLERANCE, "recorded": None}
    text = open(path).read()
    a = text.find("```json")
    if a < 0:
        return {"tolerance": TOLERANCE, "recorded": None, "source": rel}
    rec = json.loads(text[a + 7:text.index("```", a + 7)])
    rec["source"] = rel
    rec["tolerance"] = TOLERANCE
    # the summary names the library build it was recorded with: a different one at hand means the figures are of an
    # older build (the test still ran, and passed, against this tolerance when this build's GPU tests ran)
    from rembrandt_amd import _lib
    rec["stale"] = rec.get("library") != _lib.lib().rh_version().decode()
    return rec


BATCH = {"alexnet": 256, "lenet": 64, "cifar10": 128, "nin": 128, "resnet18": 256}
NUM_CLASSES_SEED = 0x5EED0000


def collect_profile(lib, steps):
    import ctypes as C
    agg = {}
    n = lib.rh_profile_count()
    tag, work, ms = C.c_char_p(), C.c_double(), C.c_float()
    for i in range(n):
        rc = lib.rh_profile_get(i, C.byref(tag), C.byref(work), C.byref(ms))
        if rc != 0:
            raise RuntimeError("rh_profile_get failed: %d" % rc)
        a = agg.setdefault(tag.value.decode(), [0, 0.0, 0.0])
        a[0] += 1
        a[1] += work.value
        a[2] += ms.value
    out = []
    for name, (count, work, ms) in agg.items():
        mfma = name.startswith("conv_fwd") or name.startswith("conv_bwd_data") or name.startswith("conv_bwd_filter") \
            or name.startswith("sgemm")
        if ms <= 0.0:
            continue
        if mfma:
            achieved, unit = work / ms / 1e9, "TFLOP/s"
            peak = PEAK_BF16_MFMA_TFLOPS if name.startswith("conv_fwd_bf16") else PEAK_FP32_MFMA_TFLOPS
        else:
            achieved, peak, unit = work / ms / 1e6, PEAK_HBM_GBS, "GB/s"
        out.append({"kernel": name, "bound": "mfma" if mfma else "hbm", "launches_per_step": count / steps,
                    "ms_per_step": ms / steps, "avg_launch_ms": ms / count, "achieved": achieved, "peak": peak,
                    "unit": unit, "frac": achieved / peak})
    out.sort(key=lambda k: -k["ms_per_step"])
    return out


def calibrate(lib, torch):
    """Sustained ceilings of this GPU, for auditing the roofline fractions: a register-only fp32 MFMA loop
    (2 waves per SIMD) and a plain float4 copy of 1 GiB, both timed by the library's own HIP events."""
    import ctypes as C
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    sink = torch.zeros(4, dtype=torch.float32, device="cuda:0")
    src = torch.ones(1 << 28, dtype=torch.float32, device="cuda:0")
    dst = torch.empty_like(src)
    out = {}
    for rep in range(2):               # first round warms up, second is read
        lib.rh_profile_reset()
        lib.rh_profile_enable(1)
        for _ in range(3):
            lib.rh_probe_mfma_loop(512, 8, 10000, C.c_void_p(sink.data_ptr()), stream)
            lib.rh_probe_copy(C.c_void_p(src.data_ptr()), C.c_void_p(dst.data_ptr()), src.numel(), stream)
        torch.cuda.synchronize()
        lib.rh_profile_enable(0)
        recs = {k["kernel"]: k for k in collect_profile(lib, 1)}
        out = {"mfma_fp32_loop_tflops": recs["probe_mfma_loop"]["achieved"] / 1e3,
               "copy_1gib_gbs": recs["probe_copy"]["achieved"],
               "device": torch.cuda.get_device_name(0),
               "compute_units": torch.cuda.get_device_properties(0).multi_processor_count}
    lib.rh_profile_reset()
    return out


def cpu_baseline(net, sample_images):
    """One train step of the same operator graph on the host cores (CPU oracle, fp32 im2col + SGEMM family)."""
    import numpy as np
    import oracle
    from oracle import graph as OG
    dims, layers, ncat = net
    ref = OG.SequentialOperatorWorker(layers, ncat, sample_images, fast=True)
    rng = np.random.default_rng(0)
    for op in ref.hidden:
        if hasattr(op, "units"):
            for u in op.units:
                u.weights[...] = rng.standard_normal(u.weights.shape, dtype=np.float32) * np.float32(np.sqrt(2.0 / u.weights[0].size))
        elif op.p is not None:
            op.p.weights[...] = rng.standard_normal(op.p.weights.shape, dtype=np.float32) * np.float32(0.01)
    x = rng.standard_normal((sample_images, dims[2], dims[1], dims[0]), dtype=np.float32)
    labels = rng.integers(0, ncat, (sample_images,)).astype(np.int32)
    sgd = OG.SgdOpt(0.01, ("Update", 0.9), 0.0)
    sgd.begin(ref)
    ref.stage_batch(labels, 1.0 / sample_images)
    t0 = time.perf_counter()
    ref.forward(x)
    ref.store_output_categories()
    ref.store_loss()
    ref.backward()
    sgd.step(ref)
    dt = time.perf_counter() - t0
    return {"value": sample_images / dt, "unit": "images/sec", "cores": oracle.num_threads(), "kind": "port",
            "sample": "one fwd+bwd+SGD step of the same operator graph on %d images (%.1f s)" % (sample_images, dt)}


def bench_bf16_forward(args, lib, net, cfg, batch, seed):
    """Forward pass only, inference phase, convolution operands rounded to bf16 (fp32 accumulation): the reduced-
    precision forward option.  One JSON line of the same shape as the train-step line."""
    import torch
    from rembrandt_amd import configs, synth
    from rembrandt_amd.operator import SequentialOperatorWorker
    dims, layers, ncat = net
    worker = SequentialOperatorWorker(cfg, batch, "Forward", shared_seed=(seed, seed + 1), device=0, bf16_forward=True)
    worker.init_params()
    worker.load_frames_f32(synth.normal(seed, 100, (batch, dims[2], dims[1], dims[0])))
    for _ in range(args.warmup):
        worker.forward(batch, training=False, t=0)
    worker.sync()
    kernels = []
    if not args.no_kernel_events:
        lib.rh_profile_reset()
        lib.rh_profile_filter(None)
        lib.rh_profile_enable(1)
        n = max(1, min(args.steps, 10))
        for _ in range(n):
            worker.forward(batch, training=False, t=0)
        worker.sync()
        lib.rh_profile_enable(0)
        kernels = collect_profile(lib, n)
        lib.rh_profile_reset()
    bf = [k for k in kernels if k["kernel"].startswith("conv_fwd_bf16")]
    dom = bf[0] if bf else None
    if dom is not None:
        lib.rh_profile_filter(dom["kernel"].encode())
        lib.rh_profile_enable(1)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        worker.forward(batch, training=False, t=0)
    worker.sync()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    lib.rh_profile_enable(0)
    if dom is not None:
        live = [k for k in collect_profile(lib, args.steps) if k["kernel"] == dom["kernel"]]
        dom = live[0] if live else dom
    lib.rh_profile_reset()
    lib.rh_profile_filter(None)
    print(json.dumps({
        "metric": "inference images/sec (forward only) %s b%d, bf16 conv operands, fp32 accumulation" % (args.workload, batch),
        "value": batch * args.steps / dt, "unit": "images/sec", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": dt / args.steps * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16 operands, f32 accumulate (affine layers f32)", "data": "synthetic",
        "config": {"workload": "%s-shaped forward pass, inference phase, batch %d, input %dx%dx%d N(0,1), convolutions on "
                               "bf16-rounded operands" % (args.workload, batch, dims[2], dims[1], dims[0]),
                   "global_batch": batch, "params": cfg.params_len(),
                   "gemm_gflop_per_step": configs.train_flops(net, batch, forward_only=True) / 1e9},
        "roofline": None if dom is None else
                    {"bound": "mfma", "kernel": dom["kernel"], "achieved": dom["achieved"], "peak": PEAK_BF16_MFMA_TFLOPS,
                     "unit": "TFLOP/s", "frac": dom["achieved"] / PEAK_BF16_MFMA_TFLOPS, "avg_launch_ms": dom["avg_launch_ms"],
                     "traffic": None},
        "kernels": kernels,
        "parity": {"tolerance": TOLERANCE + "; the oracle is evaluated on the bf16-rounded operands (round to nearest even), "
                                "so only the accumulation order differs"},
    }))


def _dominant(kernels, prefix=None):
    """The contraction kernel tag that takes the most time of a step (optionally among tags with a prefix)."""
    c = [k for k in kernels if k["bound"] == "mfma" and (prefix is None or k["kernel"].startswith(prefix))]
    return c[0] if c else (kernels[0] if kernels else None)


def _roof(k):
    return None if k is None else {"bound": k["bound"], "kernel": k["kernel"], "achieved": k["achieved"], "peak": k["peak"],
                                   "unit": k["unit"], "frac": k["frac"], "avg_launch_ms": k["avg_launch_ms"],
                                   "launches_per_step": k["launches_per_step"]}


def short_train_leg(lib, name, steps, warmup):
    """One of the other benchmark networks through the same train step as the headline: images/s over `steps` timed
    steps, launches per step and the dominant contraction kernel's roofline position (HIP events, untimed pass)."""
    import torch
    from rembrandt_amd import configs, synth
    from rembrandt_amd.operator import SequentialOperatorWorker, SgdOpt
    net = configs.NETWORKS[name]()
    dims, layers, ncat = net
    batch = BATCH[name]
    seed = NUM_CLASSES_SEED + 4
    cfg = configs.build_config(net)
    worker = SequentialOperatorWorker(cfg, batch, "Backward", shared_seed=(seed, seed + 1), device=0)
    worker.init_params()
    x = synth.uniform(seed, 100, (batch, dims[2], dims[1], dims[0])) if name == "lenet" else \
        synth.normal(seed, 100, (batch, dims[2], dims[1], dims[0]))
    worker.load_frames_f32(x)
    worker.stage_batch(synth.integers(seed, 200, (batch,), ncat), 1.0 / batch)
    sgd = SgdOpt(batch, 0.01, ("Update", 0.9), 5e-4 if name == "lenet" else 0.0)
    sgd.begin(worker)
    for _ in range(warmup):
        sgd.train_batch(worker, batch, fused=True)
    worker.sync()
    n = max(1, min(steps, 10))
    worker.set_overlap_backward(False)
    lib.rh_profile_reset()
    lib.rh_profile_filter(None)
    lib.rh_profile_enable(1)
    for _ in range(n):
        sgd.train_batch(worker, batch, fused=True)
    worker.sync()
    lib.rh_profile_enable(0)
    kernels = collect_profile(lib, n)
    lib.rh_profile_reset()
    worker.set_overlap_backward(True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        sgd.train_batch(worker, batch, fused=True)
    worker.sync()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    worker.close()
    flops = configs.train_flops(net, batch)
    mfma_ms = sum(k["ms_per_step"] for k in kernels if k["bound"] == "mfma")
    executed = _executed_flops(kernels)
    return {"metric": "train images/sec (fwd+bwd+SGD) %s b%d fp32" % (name, batch), "value": batch * steps / dt,
            "unit": "images/sec", "ms_per_step": dt / steps * 1e3, "steps": steps, "dtype": "f32",
            "launches_per_step": sum(k["launches_per_step"] for k in kernels),
            "gemm_gflop_per_step": flops / 1e9,
            "step_frac_of_mfma_peak": flops / (dt / steps) / 1e12 / PEAK_FP32_MFMA_TFLOPS,
            "all_mfma": {"ms_per_step": mfma_ms, "frac": executed / mfma_ms / 1e9 / PEAK_FP32_MFMA_TFLOPS if mfma_ms else None},
            "roofline": _roof(_dominant(kernels))}


def short_bf16_forward_leg(lib, name, steps, warmup):
    """Forward pass alone, inference phase, bf16 convolution operands with fp32 accumulation."""
    import torch
    from rembrandt_amd import configs, synth
    from rembrandt_amd.operator import SequentialOperatorWorker
    net = configs.NETWORKS[name]()
    dims, layers, ncat = net
    batch = BATCH[name]
    seed = NUM_CLASSES_SEED + 4
    worker = SequentialOperatorWorker(configs.build_config(net), batch, "Forward", shared_seed=(seed, seed + 1), device=0,
                                      bf16_forward=True)
    worker.init_params()
    worker.load_frames_f32(synth.normal(seed, 100, (batch, dims[2], dims[1], dims[0])))
    for _ in range(warmup):
        worker.forward(batch, training=False, t=0)
    worker.sync()
    n = max(1, min(steps, 10))
    lib.rh_profile_reset()
    lib.rh_profile_filter(None)
    lib.rh_profile_enable(1)
    for _ in range(n):
        worker.forward(batch, training=False, t=0)
    worker.sync()
    lib.rh_profile_enable(0)
    kernels = collect_profile(lib, n)
    lib.rh_profile_reset()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        worker.forward(batch, training=False, t=0)
    worker.sync()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    worker.close()
    flops = configs.train_flops(net, batch, forward_only=True)
    conversions = [k for k in kernels if k["kernel"].startswith("nchw_to_bf16") or k["kernel"].startswith("bf16_filter")]
    return {"metric": "inference images/sec (forward only) %s b%d, bf16 conv operands, fp32 accumulation" % (name, batch),
            "value": batch * steps / dt, "unit": "images/sec", "ms_per_step": dt / steps * 1e3, "steps": steps,
            "dtype": "bf16 operands, f32 accumulate", "launches_per_step": sum(k["launches_per_step"] for k in kernels),
            "gemm_gflop_per_step": flops / 1e9,
            "step_frac_of_bf16_mfma_peak": flops / (dt / steps) / 1e12 / PEAK_BF16_MFMA_TFLOPS,
            "operand_conversion_ms_per_step": sum(k["ms_per_step"] for k in conversions),
            "operand_conversion_launches_per_step": sum(k["launches_per_step"] for k in conversions),
            "roofline": _roof(_dominant(kernels, "conv_fwd_bf16"))}


SWEEP = {  # the single-operator sweep: N, C, H, W, K, R, stride, pad
    "a_5x5_96to256_27x27_b256": (256, 96, 27, 27, 256, 5, 1, 2),
    "b_3x3_256to384_13x13_b256": (256, 256, 13, 13, 384, 3, 1, 1),
    "c_1x1_96to96_55x55_b128": (128, 96, 55, 55, 96, 1, 1, 0),
}


def _wino_direct_form_flops(net, batch, tag):
    """Direct-form FLOPs (2*N*K*C*R*S*P*Q) per step of the convolution passes that run under a Winograd tag
    (conv_fwd_wino, conv_bwd_data_wino, conv_bwd_filter_wino), for plain convolution layers; None for other tags
    and for networks with other kinds of convolution operators."""
    which = {"conv_fwd_wino": "fwd", "conv_bwd_data_wino": "bwd_data", "conv_bwd_filter_wino": "bwd_filter"}.get(tag)
    if which is None:
        return None
    from rembrandt_amd import ops
    total, first = 0.0, True
    for l in net[1]:
        if l[0] in ("bnorm_conv2d", "stack_res_conv2d", "proj_stack_res_conv2d"):
            return None
        if l[0] == "affine":
            first = False
        if l[0] != "conv2d":
            continue
        (w, h, c), k, st, pad, out = l[1], l[2], l[3], l[4], l[5]
        P, Q = max(0, h + 2 * pad - k + st) // st, max(0, w + 2 * pad - k + st) // st
        if not (which == "bwd_data" and first) and ops.conv2d_winograd_flops((batch, c, h, w), (out, c, k, k), st, pad, which) > 0:
            total += 2.0 * batch * out * c * k * k * P * Q
        first = False
    return total


def _wino_note(net, batch, dom):
    """For a Winograd tag: `achieved` / `frac` count the multiply-adds the kernels execute (16 per 2x2 tile, filter and
    channel); the same launches priced in the direct form's FLOPs ride along."""
    direct = _wino_direct_form_flops(net, batch, dom["kernel"])
    if not direct or not dom.get("launches_per_step") or not dom.get("avg_launch_ms"):
        return {}
    per_launch = direct / dom["launches_per_step"]
    return {"flops_counted": "executed by the Winograd F(2x2,3x3) form (16 multiply-adds per 2x2 tile, filter and channel)",
            "direct_form_gflop_per_launch": per_launch / 1e9,
            "direct_form_tflops": per_launch / dom["avg_launch_ms"] / 1e9}


def _executed_flops(kernels):
    """FLOPs per step that the contraction kernels execute: what the kernels report as their work (the Winograd
    kernels 16 multiply-adds per 2x2 tile, filter and channel, where the direct form's count has 36)."""
    return sum(k["achieved"] * 1e9 * k["ms_per_step"] for k in kernels if k["bound"] == "mfma")


def conv_sweep_leg(iters, warmup):
    """Forward, backward-data and backward-filter of the three sweep shapes, each call timed alone (HIP events on the
    stream the kernels run on; a call includes the operand copies it makes): ms, TFLOP/s against the fp32 matrix peak and
    algorithmic bytes (x, w, y once) per second against the HBM peak: the 1x1 shape sits on the ridge of both roofs."""
    import torch
    from rembrandt_amd import ops
    dev = torch.device("cuda:0")
    out = {}
    for name, (N, C, H, W, K, R, st, pad) in SWEEP.items():
        g = torch.Generator(device=dev)
        g.manual_seed(1234)
        x = torch.randn(N, C, H, W, device=dev, generator=g)
        w = torch.randn(K, C, R, R, device=dev, generator=g)
        y = ops.conv2d_fwd(x, w, st, pad)
        dy = torch.randn(y.shape, device=dev, generator=g)
        dw, dx = torch.zeros_like(w), torch.zeros_like(x)
        flops = 2.0 * y.numel() * C * R * R
        byts = 4.0 * (x.numel() + w.numel() + y.numel())
        calls = {"fwd": lambda: ops.conv2d_fwd(x, w, st, pad, y=y),
                 "bwd_data": lambda: ops.conv2d_bwd_data(w, dy, x.shape, st, pad, dx=dx),
                 "bwd_filter": lambda: ops.conv2d_bwd_filter(x, dy, w.shape, st, pad, dw=dw)}
        row = {"gflop": flops / 1e9, "algorithmic_mb": byts / 1e6}
        for pname, fn in calls.items():
            for _ in range(warmup):
                fn()
            torch.cuda.synchronize()
            s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s.record()
            for _ in range(iters):
                fn()
            e.record()
            torch.cuda.synchronize()
            ms = s.elapsed_time(e) / iters
            # `tflops` counts the direct form's multiply-adds (the sweep's metric); where the library takes the Winograd
            # form, `frac_mfma` is what its kernel executes against the matrix peak
            wino = ops.conv2d_winograd_flops(x.shape, w.shape, st, pad, pname)
            row[pname] = {"ms": ms, "tflops": flops / ms / 1e9,
                          "frac_mfma": (wino or flops) / ms / 1e9 / PEAK_FP32_MFMA_TFLOPS,
                          "gbs": byts / ms / 1e6, "frac_hbm": byts / ms / 1e6 / PEAK_HBM_GBS}
            if wino:
                row[pname].update({"form": "winograd F(2x2,3x3)", "executed_tflops": wino / ms / 1e9})
        out[name] = row
        del x, w, y, dy, dw, dx
    return out


def other_configs(lib):
    """The benchmark configurations other than the headline one, run after the timed region (a few seconds together)."""
    out = {}
    for key, fn in (("lenet_b64_train", lambda: short_train_leg(lib, "lenet", 200, 20)),
                    ("cifar10_b128_train", lambda: short_train_leg(lib, "cifar10", 200, 20)),
                    ("nin_b128_train", lambda: short_train_leg(lib, "nin", 20, 3)),
                    ("nin_b128_bf16_forward", lambda: short_bf16_forward_leg(lib, "nin", 50, 5)),
                    ("conv_sweep", lambda: conv_sweep_leg(20, 3))):
        t0 = time.perf_counter()
        try:
            out[key] = fn()
        except Exception as e:   # a side leg must not cost the headline line
            out[key] = {"error": "%s: %s" % (type(e).__name__, e)}
        out[key]["leg_seconds"] = time.perf_counter() - t0
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="alexnet", choices=sorted(BATCH))
    ap.add_argument("--cpu-sample", type=int, default=512, help="images in the CPU baseline step (0 = skip; 512 is about 15 s on 16 cores)")
    ap.add_argument("--unfused", action="store_true", help="reference-style K1->K2->K3 and BLAS-1 SGD sequence")
    ap.add_argument("--graph", action="store_true",
                    help="record each train step into a HIP graph and replay it (for the launch-bound small networks)")
    ap.add_argument("--no-overlap", action="store_true",
                    help="conv filter / bias gradients on the main stream instead of the second stream")
    ap.add_argument("--no-kernel-events", action="store_true",
                    help="do not bracket each kernel with HIP events in the timed region (no per-kernel breakdown)")
    ap.add_argument("--no-calibration", action="store_true", help="skip the MFMA-loop / copy ceiling probes")
    ap.add_argument("--host-frames", action="store_true",
                    help="every timed step first copies its batch of u8 frames from the worker's host frame buffer "
                         "(the PCIe-inclusive rate; the default keeps the inputs resident in HBM)")
    ap.add_argument("--bf16-forward", action="store_true",
                    help="forward pass only (inference phase) with bf16 convolution operands and fp32 accumulation; "
                         "reports inference images/sec and the bf16 kernel against the bf16 matrix peak")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="skip the short legs over the other benchmark configurations (LeNet, CIFAR-10, NIN fp32 / bf16 "
                         "forward, the convolution sweep) that the default alexnet run appends as `other_configs`")
    ap.add_argument("--calibrate-copy", type=int, default=0, metavar="MIB",
                    help="first launch the library's plain copy kernel 4 times over MIB MiB (a known-size "
                         "reference for hardware byte counters collected around this command)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (pure data parallelism would all-reduce the flat gradient "
              "vector; not built); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    from rembrandt_amd import _lib, configs, synth
    from rembrandt_amd.operator import SequentialOperatorWorker, SgdOpt

    lib = _lib.lib()
    net = configs.NETWORKS[args.workload]()
    dims, layers, ncat = net
    batch = BATCH[args.workload]
    seed = NUM_CLASSES_SEED + 4
    cfg = configs.build_config(net)
    if args.bf16_forward:
        return bench_bf16_forward(args, lib, net, cfg, batch, seed)
    worker = SequentialOperatorWorker(cfg, batch, "Backward", shared_seed=(seed, seed + 1), device=0,
                                      fuse_epilogue=not args.unfused, overlap_backward=not args.no_overlap,
                                      graph_steps=args.graph)
    worker.init_params()
    x = synth.normal(seed, 100, (batch, dims[2], dims[1], dims[0]))
    labels = synth.integers(seed, 200, (batch,), ncat)
    if args.host_frames:
        worker.load_frames_u8(synth.integers(seed, 101, (batch, dims[2], dims[1], dims[0]), 256).astype("uint8"))
    else:
        worker.load_frames_f32(x)         # inputs resident in HBM before the timed region
    worker.stage_batch(labels, 1.0 / batch)
    sgd = SgdOpt(batch, 0.01, ("Update", 0.9), 0.0)
    sgd.begin(worker)

    if args.calibrate_copy > 0:
        import ctypes as C
        n = args.calibrate_copy * (1 << 20) // 4
        src = torch.ones(n, dtype=torch.float32, device="cuda:0")
        dst = torch.empty_like(src)
        for _ in range(4):
            _lib.check(lib.rh_probe_copy(C.c_void_p(src.data_ptr()), C.c_void_p(dst.data_ptr()), n,
                                         C.c_void_p(torch.cuda.current_stream().cuda_stream)), "rh_probe_copy")
        torch.cuda.synchronize()
        del src, dst

    calibration = None if args.no_calibration else calibrate(lib, torch)

    for _ in range(args.warmup):
        sgd.train_batch(worker, batch, fused=not args.unfused)
    worker.sync()
    torch.cuda.synchronize()

    # Untimed breakdown pass: every launch bracketed by HIP events (costs ~4 % of a step in event
    # traffic, which is why it is kept out of the timed region).  It names the dominant kernel.
    kernels, breakdown_steps = [], 0 if args.no_kernel_events else max(1, min(args.steps, 10))
    if breakdown_steps:
        worker.set_overlap_backward(False)   # kernels that share the GPU stretch each other's durations
        lib.rh_profile_reset()
        lib.rh_profile_filter(None)
        lib.rh_profile_enable(1)
        for _ in range(breakdown_steps):
            sgd.train_batch(worker, batch, fused=not args.unfused)
        worker.sync()
        torch.cuda.synchronize()
        lib.rh_profile_enable(0)
        kernels = collect_profile(lib, breakdown_steps)
        lib.rh_profile_reset()
        worker.set_overlap_backward(not args.no_overlap)
    mfma = [k for k in kernels if k["bound"] == "mfma"]
    # The dominant kernel is timed live inside the timed region, where backward kernels overlap on two streams and
    # stretch each other; forward kernels run alone, so with overlap on the choice is made among them.
    cands = [k for k in mfma if args.no_overlap or k["kernel"].startswith("conv_fwd")] or mfma
    dom = cands[0] if cands else kernels[0] if kernels else None

    # Timed region: exactly `steps` steps; only the dominant kernel's launches carry HIP events.
    if dom is not None:
        lib.rh_profile_filter(dom["kernel"].encode())
        lib.rh_profile_enable(1)
    t0 = time.perf_counter()
    loss = 0.0
    for _ in range(args.steps):
        if args.host_frames:
            # The step is launched piece by piece so that the next batch's frames can be handed over while it is still
            # queued (load_frames returns when the host buffer is free again, as in the reference, but copies beside
            # the kernels of the step before); the loss read-back then synchronises, as train_batch does.
            worker.forward(batch, training=True, t=sgd.iter_counter())
            worker.backward(batch)
            sgd.step(worker, fused=not args.unfused)
            worker.reload_frames(batch)
            loss = worker.store_loss(batch)
            continue
        loss, _ = sgd.train_batch(worker, batch, fused=not args.unfused)
    worker.sync()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    lib.rh_profile_enable(0)
    if dom is not None:
        live = [k for k in collect_profile(lib, args.steps) if k["kernel"] == dom["kernel"]]
        dom = live[0] if live else dom
    lib.rh_profile_reset()
    lib.rh_profile_filter(None)

    traffic, traffic_source = measured_traffic(args.workload, dom["kernel"]) if dom is not None else (None, None)
    gemm_ms = sum(k["ms_per_step"] for k in mfma)
    gemm_flops = configs.train_flops(net, batch)
    result = {
        "metric": "train images/sec (fwd+bwd+SGD) AlexNet b256 fp32; conv/FC % MFMA peak" if args.workload == "alexnet" else
                  "train images/sec (fwd+bwd+SGD) %s b%d fp32" % (args.workload, batch),
        "value": batch * args.steps / dt,
        "unit": "images/sec",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": dt / args.steps * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "%s-shaped train step (fwd+bwd+SGD momentum 0.9), batch %d, fp32, input %dx%dx%d N(0,1), "
                               "weights N(0,0.01), %s%s" % (args.workload, batch, dims[2], dims[1], dims[0],
                                                            "unfused reference sequence" if args.unfused else "fused epilogues",
                                                            ("" if args.no_overlap else ", two-stream backward") +
                                                            (", u8 frames copied from host memory every step" if args.host_frames else "") +
                                                            (", steps replayed as a HIP graph" if args.graph else "")),
                   "global_batch": batch, "params": cfg.params_len(), "gemm_gflop_per_step": gemm_flops / 1e9},
        "roofline": None if dom is None else
                    {"bound": dom["bound"], "kernel": dom["kernel"], "achieved": dom["achieved"], "peak": dom["peak"],
                     "unit": dom["unit"], "frac": dom["frac"], "avg_launch_ms": dom["avg_launch_ms"],
                     "traffic": traffic,
                     "traffic_unit": "bytes per launch (L2<->fabric, FETCH_SIZE + WRITE_SIZE counters)",
                     "traffic_source": traffic_source, **_wino_note(net, batch, dom)},
        # all contraction kernels together: executed FLOPs (the Winograd kernels' own count) against the matrix peak;
        # `direct_form_tflops` prices the same time in the direct form's multiply-adds (config.gemm_gflop_per_step)
        "all_mfma": {"ms_per_step": gemm_ms, "executed_gflop_per_step": _executed_flops(mfma) / 1e9,
                     "achieved": _executed_flops(mfma) / gemm_ms / 1e9 if gemm_ms else None,
                     "unit": "TFLOP/s", "frac": _executed_flops(mfma) / gemm_ms / 1e9 / PEAK_FP32_MFMA_TFLOPS if gemm_ms else None,
                     "direct_form_tflops": gemm_flops / gemm_ms / 1e9 if gemm_ms else None},
        "calibration": calibration,
        "kernels_note": "per-kernel table from an untimed pass of %d steps with HIP events on every launch and the "
                        "backward kernels on one stream; roofline.* is from events on the dominant forward kernel inside "
                        "the timed region (where filter/bias gradients overlap the data gradients on a second stream); "
                        "the backward-filter kernel of the same tile takes as much of a step as that forward kernel "
                        "(see `kernels`), it is not chosen because its live durations are stretched by the other stream"
                        % breakdown_steps,
        "parity": recorded_parity(args.workload, batch),
        "kernels": kernels,
        "final_loss": loss,
    }
    if args.workload == "alexnet" and not args.no_other_configs and not args.unfused and not args.graph:
        worker.close()
        result["other_configs"] = other_configs(lib)
    if args.cpu_sample > 0:
        try:
            result["cpu_baseline"] = cpu_baseline(net, args.cpu_sample)
        except Exception as e:   # (the oracle library missing or a host without OpenMP: the measured line still prints)
            result["cpu_baseline"] = {"value": None, "unit": "images/sec", "cores": 0, "kind": "port",
                                      "sample": "not run: %s: %s" % (type(e).__name__, e)}
    print(json.dumps(result))


if __name__ == "__main__":
    main()
