"""GPU parity at the full sizes of the benchmark configurations, where the CPU oracle cannot recompute
whole tensors in seconds.  Each kernel is checked through the C ABI by
  * the oracle on a random sample of output elements (plus the first and last element),
  * size-independent properties: the adjoint identities <conv(x,w),dy> = <x,bwd_data(w,dy)> = <w,bwd_filter(x,dy)>,
    exact linearity under a power-of-two scale, bit-identical results of repeated launches (the split
    reductions add in a fixed order), sum(dx) = sum(dy) and arg-max-in-window for pooling,
  * the oracle on whole slices where the operator is independent per plane (pooling) or cheap (SGD, affine).
"""
import numpy as np
import pytest
import torch

import oracle as O
from rembrandt_amd import _lib, ops, synth
from conftest import assert_close, say

pytestmark = pytest.mark.gpu


def T(a, dev):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def dot64(a, b):
    return float((a.double() * b.double()).sum().item())


def sample_idx(rng, total, n):
    idx = rng.integers(0, total, n).astype(np.int64)
    idx[0], idx[-1] = 0, total - 1
    return idx


def edge_idx(rng, shape, n):
    """Flat indices of elements of an NCHW tensor that sit on the seams of the kernels' tiles: channel (GEMM row)
    and column (image * plane + pixel) positions one either side of multiples of 32 (the MFMA block; 64-, 96-, 128-
    and 256-wide tiles and wave parts start on these), where an indexing mistake would touch only a few elements."""
    Nn, K, P, Q = shape
    inner, cols = P * Q, Nn * P * Q
    c = 32 * rng.integers(0, (cols + 31) // 32 + 1, n) + rng.integers(-1, 2, n)
    r = 32 * rng.integers(0, (K + 31) // 32 + 1, n) + rng.integers(-1, 1, n)
    c = np.clip(c, 0, cols - 1).astype(np.int64)
    r = np.clip(r, 0, K - 1).astype(np.int64)
    return (c // inner) * (K * inner) + r * inner + c % inner


FULL_CONV = {
    # name: N, C, H, W, K, R, stride, pad
    "sweep_a_alexnet_conv2": (256, 96, 27, 27, 256, 5, 1, 2),
    "sweep_b_alexnet_conv3": (256, 256, 13, 13, 384, 3, 1, 1),
    "sweep_c_1x1": (128, 96, 55, 55, 96, 1, 1, 0),
    "alexnet_conv1": (256, 3, 227, 227, 96, 11, 4, 0),
    "alexnet_conv4": (256, 384, 13, 13, 384, 3, 1, 1),
    "alexnet_conv5": (256, 384, 13, 13, 256, 3, 1, 1),
    # NIN at batch 128: the 3x3 layer into 1024 channels on 6x6, its 1x1 successors (1024 -> 1024 -> 1000), a mid-network 1x1
    "nin_conv4_1024": (128, 384, 6, 6, 1024, 3, 1, 1),
    "nin_cccp7": (128, 1024, 6, 6, 1024, 1, 1, 0),
    "nin_cccp8": (128, 1024, 6, 6, 1000, 1, 1, 0),
    "nin_cccp3": (128, 256, 27, 27, 256, 1, 1, 0),
    # ResNet-18 template at batch 64: 64-row tiles with the halved K step (784 tiles), contraction cut into slices
    # (7x7 and 14x14 extents), a strided 3x3 layer and a strided 1x1 projection
    "resnet_56_64": (64, 64, 56, 56, 64, 3, 1, 1),
    "resnet_14_256": (64, 256, 14, 14, 256, 3, 1, 1),
    "resnet_7_512": (64, 512, 7, 7, 512, 3, 1, 1),
    "resnet_down_512": (64, 256, 14, 14, 512, 3, 2, 1),
    "resnet_proj_128": (64, 64, 56, 56, 128, 1, 2, 0),
    # 784 tiles on 256 CUs: the last 16 tiles are cut into slices (as are the last 164 of alexnet_conv5's 676)
    "resnet_14_256_b256": (256, 256, 14, 14, 256, 3, 1, 1),
    # large 1x1 layers of up to 128 channels: the image through LDS (two row tiles with a pixel count that is a multiple
    # of four; one row tile with ragged image ends; different channel counts on the two sides)
    "lds1x1_64_56x56": (48, 64, 56, 56, 64, 1, 1, 0),
    "lds1x1_32_ragged": (80, 32, 40, 41, 32, 1, 1, 0),
    "lds1x1_64_to_32": (96, 64, 37, 43, 32, 1, 1, 0),
}


@pytest.mark.parametrize("name", sorted(FULL_CONV))
def test_conv2d_full_size(dev, name):
    Nn, C, H, W, K, R, st, pad = FULL_CONV[name]
    say("full-size conv", name)
    rng = np.random.default_rng(5)
    x = synth.normal(21, 1, (Nn, C, H, W))
    w = synth.normal(21, 2, (K, C, R, R))
    xd, wd = T(x, dev), T(w, dev)
    y = ops.conv2d_fwd(xd, wd, st, pad)
    dy = synth.normal(21, 3, tuple(y.shape))
    dyd = T(dy, dev)
    dw = ops.conv2d_bwd_filter(xd, dyd, w.shape, st, pad)
    dx = ops.conv2d_bwd_data(wd, dyd, x.shape, st, pad)

    # sampled oracle
    i_y = sample_idx(rng, y.numel(), 4096)
    assert_close(y.flatten()[T(i_y, dev)].cpu().numpy(), O.conv2d_fwd_at(x, w, st, pad, i_y), name + " fwd (sampled)")
    i_w = sample_idx(rng, dw.numel(), 1024)
    assert_close(dw.flatten()[T(i_w, dev)].cpu().numpy(), O.conv2d_bwd_filter_at(x, dy, w.shape, st, pad, i_w),
                 name + " bwd filter (sampled)")
    i_x = sample_idx(rng, dx.numel(), 4096)
    assert_close(dx.flatten()[T(i_x, dev)].cpu().numpy(), O.conv2d_bwd_data_at(w, dy, x.shape, st, pad, i_x),
                 name + " bwd data (sampled)")
    # and on the seams of the tiles
    e_y = edge_idx(rng, tuple(y.shape), 2048)
    assert_close(y.flatten()[T(e_y, dev)].cpu().numpy(), O.conv2d_fwd_at(x, w, st, pad, e_y), name + " fwd (tile seams)")
    e_x = edge_idx(rng, x.shape, 2048)
    assert_close(dx.flatten()[T(e_x, dev)].cpu().numpy(), O.conv2d_bwd_data_at(w, dy, x.shape, st, pad, e_x),
                 name + " bwd data (tile seams)")

    # adjoint identities over the whole tensors (fp64 sums); scale = size of such a sum for unrelated vectors
    a = dot64(y, dyd)
    scale = float(y.double().norm().item() * dyd.double().norm().item()) / np.sqrt(y.numel())
    assert abs(a - dot64(xd, dx)) <= 1e-4 * scale, (name, "bwd data adjoint", a, dot64(xd, dx), scale)
    assert abs(a - dot64(wd, dw)) <= 1e-4 * scale, (name, "bwd filter adjoint", a, dot64(wd, dw), scale)

    # exact linearity (scaling by 2 is exact in fp32) and run-to-run bit identity
    assert torch.equal(ops.conv2d_fwd(xd, wd * 2.0, st, pad), y * 2.0), name + " fwd linearity"
    assert torch.equal(ops.conv2d_bwd_filter(xd, dyd * 2.0, w.shape, st, pad), dw * 2.0), name + " bwd filter linearity"
    assert torch.equal(ops.conv2d_bwd_data(wd * 2.0, dyd, x.shape, st, pad), dx * 2.0), name + " bwd data linearity"
    assert torch.equal(ops.conv2d_bwd_filter(xd, dyd, w.shape, st, pad), dw), name + " bwd filter repeatable"

    # fused epilogue and the bias gradient at this size
    b = synth.normal(21, 4, (K,))
    yf = ops.conv2d_fwd(xd, wd, st, pad, bias=T(b, dev), relu=True)
    assert torch.equal(yf, torch.relu(y + T(b, dev).view(1, K, 1, 1))), name + " fused bias+relu"
    db = ops.conv2d_bwd_bias(dyd, two_stage=True)
    assert_close(db.cpu().numpy(), dy.sum(axis=(0, 2, 3), dtype=np.float64).astype(np.float32), name + " bias gradient")
    torch.cuda.synchronize()



def test_conv2d_epilogue_on_a_16m_pixel_plane(dev):
    """One image of 4099 x 4099 pixels, eight channels either side: rows of the result are 67 MB apart, so the
    wave-uniform row offsets of the tile epilogue's edge tiles could pass 2^31 and its operand loads (old values for
    beta, the ReLU mask of the data gradient) take their guarded form.  Sampled oracle, whole-tensor identities."""
    Nn, C, H, W, K, R, st, pad = 1, 8, 4099, 4099, 8, 3, 1, 1
    say("conv epilogue, 16 M pixel plane")
    rng = np.random.default_rng(9)
    x = synth.normal(31, 1, (Nn, C, H, W))
    w = synth.normal(31, 2, (K, C, R, R))
    b = synth.normal(31, 3, (K,))
    y0 = synth.normal(31, 4, (Nn, K, H, W))
    xd, wd = T(x, dev), T(w, dev)
    y = ops.conv2d_fwd(xd, wd, st, pad)
    i_y = sample_idx(rng, y.numel(), 4096)
    ref = O.conv2d_fwd_at(x, w, st, pad, i_y)
    assert_close(y.flatten()[T(i_y, dev)].cpu().numpy(), ref, "large plane fwd (sampled)")
    yb = ops.conv2d_fwd(xd, wd, st, pad, bias=T(b, dev), relu=True, alpha=0.5, beta=2.0, y=T(y0, dev))
    kk = (i_y // (H * W)) % K
    want = np.maximum(0.5 * ref.astype(np.float64) + 2.0 * y0.ravel()[i_y] + b[kk], 0.0)
    assert_close(yb.flatten()[T(i_y, dev)].cpu().numpy(), want, "large plane fwd alpha/beta/bias/relu (sampled)")
    del yb
    dy = synth.normal(31, 5, (Nn, K, H, W))
    dyd = T(dy, dev)
    dx0 = synth.normal(31, 6, (Nn, C, H, W))
    dx = ops.conv2d_bwd_data(wd, dyd, x.shape, st, pad)
    i_x = sample_idx(rng, dx.numel(), 4096)
    refx = O.conv2d_bwd_data_at(w, dy, x.shape, st, pad, i_x)
    assert_close(dx.flatten()[T(i_x, dev)].cpu().numpy(), refx, "large plane bwd data (sampled)")
    for alpha, beta in ((1.0, 0.0), (0.5, 2.0)):
        two = ops.conv2d_bwd_data(wd, dyd, x.shape, st, pad, alpha=alpha, beta=beta, dx=T(dx0, dev))
        two = torch.where(xd > 0, two, torch.zeros_like(two))
        one = ops.conv2d_bwd_data(wd, dyd, x.shape, st, pad, alpha=alpha, beta=beta, dx=T(dx0, dev), relu_of=xd)
        assert torch.equal(one, two), "large plane masked data gradient alpha=%g beta=%g" % (alpha, beta)
        del one, two
    a = dot64(y, dyd)
    scale = float(y.double().norm().item() * dyd.double().norm().item()) / np.sqrt(y.numel())
    assert abs(a - dot64(xd, dx)) <= 1e-4 * scale, ("large plane bwd data adjoint", a, dot64(xd, dx), scale)
    torch.cuda.synchronize()


@pytest.mark.parametrize("name", sorted(FULL_CONV))
def test_conv2d_fwd_bf16_full_size(dev, name):
    Nn, C, H, W, K, R, st, pad = FULL_CONV[name]
    say("full-size bf16 conv", name)
    rng = np.random.default_rng(7)
    x = synth.normal(25, 1, (Nn, C, H, W))
    w = synth.normal(25, 2, (K, C, R, R))
    y = ops.conv2d_fwd(T(x, dev), T(w, dev), st, pad, algo=_lib.RH_MATH_BF16_MFMA_FP32ACC)
    i_y = sample_idx(rng, y.numel(), 4096)
    ref = O.conv2d_fwd_at(O.round_bf16(x), O.round_bf16(w), st, pad, i_y)
    assert_close(y.flatten()[T(i_y, dev)].cpu().numpy(), ref, name + " bf16 fwd (sampled)")
    e_y = edge_idx(rng, tuple(y.shape), 2048)
    assert_close(y.flatten()[T(e_y, dev)].cpu().numpy(), O.conv2d_fwd_at(O.round_bf16(x), O.round_bf16(w), st, pad, e_y),
                 name + " bf16 fwd (tile seams)")
    # exact linearity and agreement with the fp32 kernel on operands that are already bf16 values
    xr, wr = T(O.round_bf16(x), dev), T(O.round_bf16(w), dev)
    assert torch.equal(ops.conv2d_fwd(xr, wr * 2.0, st, pad, algo=_lib.RH_MATH_BF16_MFMA_FP32ACC), y * 2.0)
    y32 = ops.conv2d_fwd(xr, wr, st, pad)
    err = float((y32 - y).double().norm().item() / y32.double().norm().item())
    assert err <= 1e-5, (name, "bf16 vs fp32 kernel on bf16-exact operands", err)
    torch.cuda.synchronize()


@pytest.mark.parametrize("shape", [(256, 96, 55, 55), (256, 256, 27, 27), (256, 256, 13, 13)],
                         ids=["alexnet_pool1", "alexnet_pool2", "alexnet_pool5"])
@pytest.mark.parametrize("mode", [_lib.RH_POOL_MAX, _lib.RH_POOL_AVG_INCL_PAD], ids=["max", "avg"])
def test_pool2d_full_size(dev, shape, mode):
    say("full-size pool", shape, mode)
    Nn, C, H, W = shape
    k, st, pad = 3, 2, 0
    rng = np.random.default_rng(6)
    x = synth.normal(22, 1, shape)
    xd = T(x, dev)
    if mode == _lib.RH_POOL_MAX:
        y, am = ops.pool2d_fwd(xd, k, st, pad, mode, want_argmax=True)
    else:
        y, am = ops.pool2d_fwd(xd, k, st, pad, mode), None
    dy = synth.normal(22, 2, tuple(y.shape))
    dyd = T(dy, dev)
    dx = ops.pool2d_bwd(xd, y, dyd, k, st, pad, mode, argmax=am)
    dx_rescan = ops.pool2d_bwd(xd, y, dyd, k, st, pad, mode) if am is not None else dx
    # whole planes against the oracle: pooling is independent per (n, c) plane
    planes = sample_idx(rng, Nn * C, 48)
    xs = x.reshape(Nn * C, 1, H, W)[planes]
    ys, ams = O.pool2d_fwd(xs, k, st, pad, mode, want_argmax=True)
    P, Q = y.shape[2], y.shape[3]
    got_y = y.reshape(Nn * C, 1, P, Q)[T(planes, dev)].cpu().numpy()
    if mode == _lib.RH_POOL_MAX:
        assert np.array_equal(got_y, ys), "max pooling is exact"
        assert np.array_equal(am.reshape(Nn * C, 1, P, Q)[T(planes, dev)].cpu().numpy(), ams)
    else:
        assert_close(got_y, ys, "avg pool fwd")
    dys = dy.reshape(Nn * C, 1, P, Q)[planes]
    dxs = O.pool2d_bwd(xs, ys, dys, k, st, pad, mode)
    assert_close(dx.reshape(Nn * C, 1, H, W)[T(planes, dev)].cpu().numpy(), dxs, "pool bwd")
    # the two forms add an element's (at most four) contributions in different fixed orders
    assert torch.allclose(dx, dx_rescan, rtol=1e-6, atol=2e-6), "mask-driven and window-rescan backward agree"
    assert torch.equal(dx, ops.pool2d_bwd(xd, y, dyd, k, st, pad, mode, argmax=am)), "the backward is deterministic"
    # conservation: every dy lands on exactly one x (max) / is spread with weights summing to 1 (avg, all windows inside)
    tot_dy, tot_dx = float(dyd.double().sum().item()), float(dx.double().sum().item())
    assert abs(tot_dy - tot_dx) <= 1e-5 * float(dyd.double().abs().sum().item())
    torch.cuda.synchronize()


@pytest.mark.parametrize("case", [(1, 0, 4096, 256, 9216), (0, 1, 9216, 4096, 256), (0, 0, 9216, 256, 4096),
                                  (1, 0, 1000, 256, 4096), (1, 0, 4096, 256, 4096), (0, 1, 4096, 4096, 256),
                                  (0, 0, 4096, 256, 4096)],
                         ids=["fc6_fwd", "fc6_bwd_w", "fc6_bwd_x", "fc8_fwd", "fc7_fwd", "fc7_bwd_w", "fc7_bwd_x"])
def test_sgemm_full_size(dev, case):
    """The AlexNet affine GEMMs (column-major, as the operator issues them) against numpy fp64."""
    ta, tb, m, n, k = case
    say("full-size sgemm", case)
    A = synth.normal(23, 1, (m, k) if ta else (k, m))      # column-major lda x cols stored as rows of a C array
    B = synth.normal(23, 2, (k, n) if tb else (n, k))
    C0 = synth.normal(23, 3, (n, m))
    opA = A.astype(np.float64) if ta else A.astype(np.float64).T          # m x k
    opB = B.astype(np.float64).T if tb else B.astype(np.float64)          # n x k (rows = columns of op(B))
    ref = (opB @ opA.T) + C0.astype(np.float64)                           # stored [n][m] = column-major m x n
    Cd = T(C0, dev)
    ops.sgemm(ta, tb, m, n, k, 1.0, T(A, dev), A.shape[1], T(B, dev), B.shape[1], 1.0, Cd, m)
    assert_close(Cd.cpu().numpy(), ref.astype(np.float32), "sgemm %s" % (case,))
    torch.cuda.synchronize()


def test_sgd_and_relu_full_size(dev):
    """Fused SGD step on AlexNet's 62 378 344 parameters, ReLU forward/backward on conv1's 74 M activations."""
    say("full-size sgd")
    n = 62378344
    W, g, v = synth.normal(24, 1, (n,)), synth.normal(24, 2, (n,)), synth.normal(24, 3, (n,))
    Wd, gd, vd = T(W, dev), T(g, dev), T(v, dev)
    ops.sgd_momentum_step(Wd, gd, vd, 5e-4, -0.01, 0.9, 1.0, zero_grad=True)
    O.sgd_momentum_step(W, g, v, 5e-4, -0.01, 0.9, 1.0, True)
    assert_close(Wd.cpu().numpy(), W, "sgd W")
    assert_close(vd.cpu().numpy(), v, "sgd v")
    assert not gd.any().item()
    del Wd, gd, vd
    say("full-size relu")
    y = synth.normal(24, 4, (256, 96 * 55 * 55))
    dy = synth.normal(24, 5, y.shape)
    yd, dyd = T(y, dev), T(dy, dev)
    ops.rect_inplace(yd)
    assert torch.equal(yd, torch.relu(T(y, dev)))
    ops.rect_backprop_inplace(yd, dyd)
    assert torch.equal(dyd, T(dy, dev) * (yd > 0))
    torch.cuda.synchronize()
