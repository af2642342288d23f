"""Per-kernel timings through the C ABI: each pass of a layer timed alone, as the conv sweep of the benchmark
configurations asks (fp32 NCHW; x, w, dy ~ N(0,1) unless --relu-data), plus the affine GEMMs and the
bandwidth-bound kernels at AlexNet sizes.

    python -m rembrandt_amd.kernel_bench                 # everything, one JSON line per kernel
    python -m rembrandt_amd.kernel_bench conv --layer sweep_b --passes fwd,bwd_filter --iters 3

Times are HIP-event averages over --iters launches after --warmup launches; `frac` is measured against the
datasheet peaks (fp32 MFMA 157.3 TFLOP/s, bf16 MFMA 2500 TFLOP/s, HBM 8000 GB/s).  A conv "call" includes the
operand copies the scalar-offset loaders make (padded image, transposed filter), i.e. what an operator pays.
"""
import argparse
import json
import sys

PEAK = {"fp32": 157.3, "bf16": 2500.0, "hbm": 8000.0}

CONV_LAYERS = {
    # name: N, C, H, W, K, R, stride, pad
    "sweep_a": (256, 96, 27, 27, 256, 5, 1, 2),     # = AlexNet conv2
    "sweep_b": (256, 256, 13, 13, 384, 3, 1, 1),    # = AlexNet conv3
    "sweep_c": (128, 96, 55, 55, 96, 1, 1, 0),      # 1x1
    "alexnet_conv1": (256, 3, 227, 227, 96, 11, 4, 0),
    "alexnet_conv4": (256, 384, 13, 13, 384, 3, 1, 1),
    "alexnet_conv5": (256, 384, 13, 13, 256, 3, 1, 1),
    # the distinct convolutions of the NIN-shaped network at batch 128 (1x1 "cccp" layers after each spatial one)
    "nin_conv1": (128, 3, 224, 224, 96, 11, 4, 0),
    "nin_cccp1": (128, 96, 54, 54, 96, 1, 1, 0),
    "nin_conv2": (128, 96, 27, 27, 256, 5, 1, 2),
    "nin_cccp3": (128, 256, 27, 27, 256, 1, 1, 0),
    "nin_conv3": (128, 256, 13, 13, 384, 3, 1, 1),
    "nin_cccp5": (128, 384, 13, 13, 384, 1, 1, 0),
    "nin_conv4": (128, 384, 6, 6, 1024, 3, 1, 1),
    "nin_cccp7": (128, 1024, 6, 6, 1024, 1, 1, 0),
    "nin_cccp8": (128, 1024, 6, 6, 1000, 1, 1, 0),
    "stride2_3x3": (64, 64, 56, 56, 128, 3, 2, 1),   # a strided layer in mid-network (its backward-data is needed)
    # the distinct convolutions of the ResNet-18 template at batch 64
    "resnet_conv1": (64, 3, 224, 224, 64, 7, 2, 3),
    "resnet_56_64": (64, 64, 56, 56, 64, 3, 1, 1),
    "resnet_28_128": (64, 128, 28, 28, 128, 3, 1, 1),
    "resnet_14_256": (64, 256, 14, 14, 256, 3, 1, 1),
    "resnet_7_512": (64, 512, 7, 7, 512, 3, 1, 1),
    "resnet_down_256": (64, 128, 28, 28, 256, 3, 2, 1),
    "resnet_down_512": (64, 256, 14, 14, 512, 3, 2, 1),
    "resnet_proj_128": (64, 64, 56, 56, 128, 1, 2, 0),
    "resnet_proj_512": (64, 256, 14, 14, 512, 1, 2, 0),
    # a 1x1 layer that is a plain 4096 x 8192 x 2432 GEMM: what the contraction kernels do without any im2col structure
    "gemm_like_1x1": (8, 2432, 32, 32, 4096, 1, 1, 0),
}
FC_LAYERS = {"alexnet_fc6": (256, 9216, 4096), "alexnet_fc7": (256, 4096, 4096), "alexnet_fc8": (256, 4096, 1000)}


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("what", nargs="*", default=["conv", "fc", "mem"], help="conv | fc | mem")
    ap.add_argument("--layer", default=None, help="a prefix of: %s" % ", ".join(list(CONV_LAYERS) + list(FC_LAYERS)))
    ap.add_argument("--passes", default="fwd,bwd_filter,bwd_data,fwd_bf16")
    ap.add_argument("--iters", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--relu-data", action="store_true", help="x = max(N(0,1), 0): the sparsity real activations have")
    args = ap.parse_args(argv)

    import torch
    if not torch.cuda.is_available():
        print("kernel_bench: no GPU visible", file=sys.stderr)
        return 1
    from . import _lib, ops
    dev = torch.device("cuda:0")
    passes = set(args.passes.split(","))

    def timeit(fn):
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        for _ in range(args.iters):
            fn()
        e.record()
        torch.cuda.synchronize()
        return s.elapsed_time(e) / args.iters

    def report(kernel, layer, ms, work, bound, executed=0.0):
        """executed: the FLOPs the call executes where that is not `work` (the Winograd form of a 3x3 layer: `achieved`
        stays the direct form's multiply-adds per second, `frac` is what the kernel executes against the peak)."""
        unit = "GB/s" if bound == "hbm" else "TFLOP/s"
        achieved = work / ms / (1e6 if bound == "hbm" else 1e9)
        rec = {"kernel": kernel, "layer": layer, "ms": round(ms, 4), "achieved": round(achieved, 1), "unit": unit,
               "peak": PEAK[bound], "frac": round((executed or work) / ms / (1e6 if bound == "hbm" else 1e9) / PEAK[bound], 4)}
        if executed:
            rec.update({"form": "winograd F(2x2,3x3)", "executed": round(executed / ms / 1e9, 1)})
        print(json.dumps(rec), flush=True)

    if "conv" in args.what:
        for name, (N, C, H, W, K, R, st, pad) in CONV_LAYERS.items():
            if args.layer and not name.startswith(args.layer):
                continue
            x = torch.randn(N, C, H, W, device=dev)
            if args.relu_data:
                x = torch.relu(x)
            w = torch.randn(K, C, R, R, device=dev)
            y = ops.conv2d_fwd(x, w, st, pad)
            dy = torch.randn_like(y)
            flops = 2.0 * y.numel() * C * R * R
            if "fwd" in passes:
                report("conv_fwd", name, timeit(lambda: ops.conv2d_fwd(x, w, st, pad, y=y)), flops, "fp32",
                       ops.conv2d_winograd_flops(x.shape, w.shape, st, pad, "fwd"))
            if "bwd_filter" in passes:
                dw = torch.zeros_like(w)
                report("conv_bwd_filter", name, timeit(lambda: ops.conv2d_bwd_filter(x, dy, w.shape, st, pad, dw=dw)), flops, "fp32",
                       ops.conv2d_winograd_flops(x.shape, w.shape, st, pad, "bwd_filter"))
            if "bwd_data" in passes:
                dx = torch.zeros_like(x)
                report("conv_bwd_data", name, timeit(lambda: ops.conv2d_bwd_data(w, dy, x.shape, st, pad, dx=dx)), flops, "fp32",
                       ops.conv2d_winograd_flops(x.shape, w.shape, st, pad, "bwd_data"))
            if "fwd_bf16" in passes:
                report("conv_fwd_bf16", name,
                       timeit(lambda: ops.conv2d_fwd(x, w, st, pad, y=y, algo=_lib.RH_MATH_BF16_MFMA_FP32ACC)), flops, "bf16")
            del x, w, y, dy
    if "fc" in args.what:
        for name, (B, i, o) in FC_LAYERS.items():
            if args.layer and not name.startswith(args.layer):
                continue
            X, Wt, dY = torch.randn(B, i, device=dev), torch.randn(o, i, device=dev), torch.randn(B, o, device=dev)
            Y, dW, dX = torch.empty(B, o, device=dev), torch.zeros(o, i, device=dev), torch.empty(B, i, device=dev)
            flops = 2.0 * B * i * o
            report("sgemm_fwd", name, timeit(lambda: ops.sgemm(1, 0, o, B, i, 1.0, Wt, i, X, i, 0.0, Y, o)), flops, "fp32")
            report("sgemm_bwd_w", name, timeit(lambda: ops.sgemm(0, 1, i, o, B, 1.0, X, i, dY, o, 1.0, dW, i)), flops, "fp32")
            report("sgemm_bwd_x", name, timeit(lambda: ops.sgemm(0, 0, i, B, o, 1.0, Wt, i, dY, o, 0.0, dX, i)), flops, "fp32")
    if "mem" in args.what and not args.layer:
        y = torch.randn(256, 96, 55, 55, device=dev)
        dy, b = torch.randn_like(y), torch.randn(96, device=dev)
        n = y.numel()
        report("relu_fwd", "alexnet_conv1_out", timeit(lambda: ops.rect_inplace(y)), 8.0 * n, "hbm")
        report("relu_bwd", "alexnet_conv1_out", timeit(lambda: ops.rect_backprop_inplace(y, dy)), 12.0 * n, "hbm")
        report("add_bias", "alexnet_conv1_out", timeit(lambda: ops.add_bias_nchw(b, y)), 8.0 * n, "hbm")
        report("bwd_bias", "alexnet_conv1_out", timeit(lambda: ops.conv2d_bwd_bias(dy, two_stage=True)), 4.0 * n, "hbm")
        yp, am = ops.pool2d_fwd(y, 3, 2, 0, _lib.RH_POOL_MAX, want_argmax=True)
        dyp = torch.randn_like(yp)
        m = yp.numel()
        report("pool_max_fwd", "alexnet_pool1", timeit(lambda: ops.pool2d_fwd(y, 3, 2, 0, _lib.RH_POOL_MAX)), 4.0 * (n + m), "hbm")
        report("pool_max_bwd_mask", "alexnet_pool1",
               timeit(lambda: ops.pool2d_bwd(y, yp, dyp, 3, 2, 0, _lib.RH_POOL_MAX, argmax=am)), 4.0 * (n + 2 * m), "hbm")
        report("pool_max_bwd_rescan", "alexnet_pool1",
               timeit(lambda: ops.pool2d_bwd(y, yp, dyp, 3, 2, 0, _lib.RH_POOL_MAX)), 4.0 * (2 * n + 2 * m), "hbm")
        P = 62378344
        W_, g, v = torch.randn(P, device=dev), torch.randn(P, device=dev), torch.zeros(P, device=dev)
        report("sgd_momentum_step", "alexnet_params", timeit(lambda: ops.sgd_momentum_step(W_, g, v, 0.0, -0.01, 0.9, 1.0, True)),
               24.0 * P, "hbm")
        for shp in ((256, 64, 56, 56), (256, 512, 7, 7)):
            xb, dyb = torch.randn(*shp, device=dev), torch.randn(*shp, device=dev)
            Cb, nb = shp[1], xb.numel()
            sc, bi = torch.ones(Cb, device=dev), torch.zeros(Cb, device=dev)
            rm, ri = torch.zeros(Cb, device=dev), torch.ones(Cb, device=dev)
            yb = torch.empty_like(xb)
            _, cm, ci = ops.bnorm_fwd_train(xb, sc, bi, rm, ri, 0.1, 1e-5, y=yb)
            name = "bnorm_%dx%dx%dx%d" % shp
            report("bnorm_fwd_train", name, timeit(lambda: ops.bnorm_fwd_train(xb, sc, bi, rm, ri, 0.1, 1e-5, y=yb, relu=True)),
                   12.0 * nb, "hbm")
            report("bnorm_fwd_infer", name, timeit(lambda: ops.bnorm_fwd_infer(xb, sc, bi, rm, ri, 1e-5, y=yb)), 8.0 * nb, "hbm")
            dxb, ds, db = torch.empty_like(xb), torch.zeros(Cb, device=dev), torch.zeros(Cb, device=dev)
            report("bnorm_bwd", name, timeit(lambda: ops.bnorm_bwd(xb, dyb, sc, cm, ci, 1e-5, dscale=ds, dbias=db, dx=dxb,
                                                                   beta_param=1.0)), 20.0 * nb, "hbm")
            del xb, dyb, yb, dxb
        logits = torch.randn(256, 1000, device=dev)
        report("softmax_fwd", "alexnet_logits", timeit(lambda: ops.softmax_fwd(logits)), 8.0 * logits.numel(), "hbm")
    return 0


if __name__ == "__main__":
    sys.exit(main())
