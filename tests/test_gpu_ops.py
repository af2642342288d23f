"""GPU parity: every C-ABI kernel against the CPU oracle on the same seeded inputs (small shapes)."""
import ctypes as C_

import numpy as np
import pytest
import torch

import oracle as O
from rembrandt_amd import _lib, ops, synth
from conftest import assert_close, say

pytestmark = pytest.mark.gpu


def T(a, dev):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def N(t):
    return t.detach().cpu().numpy()


CONV_CASES = [
    # N, C, H, W, K, R, stride, pad
    (2, 3, 9, 7, 4, 3, 1, 1),        # tiny, ragged everything
    (3, 5, 13, 13, 20, 5, 1, 2),     # LeNet-like 5x5 pad 2, K=20
    (2, 3, 35, 35, 96, 11, 4, 0),    # AlexNet conv1-like: 11x11 stride 4, K=96
    (4, 16, 14, 14, 50, 5, 1, 2),    # K=50 -> 64-row tile
    (2, 96, 13, 13, 256, 5, 1, 2),   # AlexNet conv2-like channels, 128-row tile, K_gemm 2400
    (3, 40, 9, 9, 130, 3, 1, 1),     # K just above a tile boundary
    (2, 24, 12, 12, 24, 1, 1, 0),    # 1x1
    (2, 6, 15, 15, 10, 3, 2, 1),     # stride 2 with pad
    (1, 4, 10, 10, 8, 3, 3, 0),      # stride 3
    (70, 2, 6, 6, 5, 3, 1, 1),       # many images, pixel tiles straddle images
    # strided backward-data by residue classes: classes without filter taps (1x1), odd extents whose last rows no
    # window covers, 7x7 stride 2 pad 3, stride 4 with padding, a contraction deep enough to be cut into slices,
    # and a stride beyond the class form (zero-dilated copy)
    (2, 8, 12, 12, 16, 1, 2, 0),
    (2, 5, 14, 11, 6, 3, 2, 0),
    (2, 3, 30, 30, 16, 7, 2, 3),
    (2, 4, 21, 21, 6, 5, 4, 2),
    (2, 8, 14, 14, 256, 3, 2, 1),
    (1, 3, 16, 16, 4, 5, 5, 0),
    # 832 / 885 column tiles of 32 x 256 on 768 block slots: the tiles past the last multiple of the CU count are cut
    # into slices of the contraction although the grid takes more than one round (forward and backward-data)
    (52, 32, 66, 66, 32, 3, 1, 0),
    # stride 1 with output rows a multiple of four pixels long on a 128-row tile, padded and unpadded image
    (3, 8, 12, 16, 128, 3, 1, 1),
    (2, 16, 10, 12, 130, 1, 1, 0),
    # 1x1, stride 1, no padding, at most 128 channels on both sides: the register-resident streaming kernel (forward
    # and backward-data) and the pixel loaders for both operands of backward-filter.  Odd channel counts (a last
    # channel pair with one live half), column tiles that straddle images and end ragged, all four row-tile counts.
    (3, 5, 7, 9, 33, 1, 1, 0),
    (2, 96, 9, 11, 96, 1, 1, 0),
    (1, 128, 6, 5, 128, 1, 1, 0),
    (5, 17, 8, 8, 100, 1, 1, 0),
    (2, 64, 13, 13, 20, 1, 1, 0),
    # enough column tiles (313 / 1250) for the per-XCD ranges, with a ragged last range and tiles that straddle images
    (4, 64, 50, 50, 64, 1, 1, 0),
    (5, 32, 89, 90, 96, 1, 1, 0),
    # contractions of 96 and more with full row tiles and channel pairs and an even pixel count per image: the form
    # of the streaming kernel that moves two pixels per lane (forward, masked backward-data) or four (backward-data,
    # pixel count a multiple of four, up to three row tiles); groups of columns that straddle images and end ragged,
    # enough groups for the per-XCD ranges; a short contraction beside them (the one-pixel form)
    (3, 96, 12, 12, 96, 1, 1, 0),
    (2, 128, 10, 10, 64, 1, 1, 0),
    (6, 32, 20, 22, 32, 1, 1, 0),
    (3, 64, 9, 10, 96, 1, 1, 0),
    (4, 96, 64, 66, 96, 1, 1, 0),
    # filter gradients of at most 32 x 64 and 32 x 128 (first layers): the narrow tiles of the gather path
    (4, 1, 12, 12, 20, 5, 1, 2),
    (3, 3, 10, 11, 32, 5, 1, 2),
    (2, 2, 9, 9, 8, 3, 2, 1),
    (2, 4, 8, 8, 30, 5, 1, 0),
]


ALGOS = {"auto": 0, "gather": _lib.RH_ALGO_GATHER, "scalar_offset": _lib.RH_ALGO_SCALAR_OFFSET}


@pytest.mark.parametrize("algo", sorted(ALGOS))
@pytest.mark.parametrize("case", CONV_CASES, ids=[str(c) for c in CONV_CASES])
def test_conv2d_all_passes(dev, case, algo):
    Nn, C, H, W, K, R, st, pad = case
    say("conv case", case, algo)
    algo = ALGOS[algo]
    x = synth.normal(11, 1, (Nn, C, H, W))
    w = synth.normal(11, 2, (K, C, R, R))
    b = synth.normal(11, 3, (K,))
    y_ref = O.conv2d_fwd(x, w, st, pad)
    dy = synth.normal(11, 4, y_ref.shape)
    xd, wd, bd, dyd = T(x, dev), T(w, dev), T(b, dev), T(dy, dev)

    y = ops.conv2d_fwd(xd, wd, st, pad, algo=algo)
    assert_close(N(y), y_ref, "conv fwd")

    # fused bias + relu epilogue == K1 -> K2 -> K3
    yf = ops.conv2d_fwd(xd, wd, st, pad, bias=bd, relu=True, algo=algo)
    ref_f = O.rect_inplace(O.add_bias_nchw(b, y_ref.copy()))
    assert_close(N(yf), ref_f, "conv fwd fused bias+relu")

    # alpha / beta blend
    y0 = synth.normal(11, 5, y_ref.shape)
    yb = ops.conv2d_fwd(xd, wd, st, pad, alpha=0.5, beta=2.0, y=T(y0, dev), algo=algo)
    assert_close(N(yb), O.conv2d_fwd(x, w, st, pad, alpha=0.5, beta=2.0, y=y0.copy()), "conv fwd alpha/beta")

    dw_ref = O.conv2d_bwd_filter(x, dy, w.shape, st, pad)
    dw = ops.conv2d_bwd_filter(xd, dyd, w.shape, st, pad, algo=algo)
    assert_close(N(dw), dw_ref, "conv bwd filter")
    dw0 = synth.normal(11, 6, w.shape)
    dwa = ops.conv2d_bwd_filter(xd, dyd, w.shape, st, pad, alpha=1.0, beta=1.0, dw=T(dw0, dev), algo=algo)
    assert_close(N(dwa), O.conv2d_bwd_filter(x, dy, w.shape, st, pad, 1.0, 1.0, dw0.copy()), "conv bwd filter beta=1")
    # the scaled accumulation of the gen-2 layers: backward(batch, scale) passes `scale` as alpha (src/layer_new.rs:1093-1101)
    dws = ops.conv2d_bwd_filter(xd, dyd, w.shape, st, pad, alpha=0.25, beta=1.0, dw=T(dw0, dev), algo=algo)
    assert_close(N(dws), O.conv2d_bwd_filter(x, dy, w.shape, st, pad, 0.25, 1.0, dw0.copy()), "conv bwd filter alpha=0.25 beta=1")
    dws = ops.conv2d_bwd_filter(xd, dyd, w.shape, st, pad, alpha=-3.0, beta=0.5, dw=T(dw0, dev), algo=algo)
    assert_close(N(dws), O.conv2d_bwd_filter(x, dy, w.shape, st, pad, -3.0, 0.5, dw0.copy()), "conv bwd filter alpha=-3 beta=0.5")

    db = ops.conv2d_bwd_bias(dyd)
    assert_close(N(db), O.conv2d_bwd_bias(dy), "conv bwd bias")
    db0 = synth.normal(11, 7, (K,))
    db2 = ops.conv2d_bwd_bias(dyd, alpha=0.5, beta=1.0, db=T(db0, dev), two_stage=True)
    assert_close(N(db2), O.conv2d_bwd_bias(dy, 0.5, 1.0, db0.copy()), "conv bwd bias (two-stage)")

    # both gradients in one call: the filter gradient bit-identical to the call of its own, the bias gradient within
    # tolerance of the oracle (where the pass over dy carries the plane sums it is added up in another order)
    for alpha, beta in ((1.0, 0.0), (0.25, 1.0)):
        dwc, dbc = ops.conv2d_bwd_filter_bias(xd, dyd, w.shape, st, pad, alpha=alpha, beta=beta, dw=T(dw0, dev), db=T(db0, dev),
                                              algo=algo)
        dws = ops.conv2d_bwd_filter(xd, dyd, w.shape, st, pad, alpha=alpha, beta=beta, dw=T(dw0, dev), algo=algo)
        assert torch.equal(dwc, dws), "filter gradient of the combined call"
        assert_close(N(dbc), O.conv2d_bwd_bias(dy, alpha, beta, db0.copy()), "bias gradient of the combined call")
        dbc2 = ops.conv2d_bwd_filter_bias(xd, dyd, w.shape, st, pad, alpha=alpha, beta=beta, dw=T(dw0, dev), db=T(db0, dev),
                                          algo=algo)[1]
        assert torch.equal(dbc, dbc2), "the combined call is not deterministic"

    dx_ref = O.conv2d_bwd_data(w, dy, x.shape, st, pad)
    dx = ops.conv2d_bwd_data(wd, dyd, x.shape, st, pad, algo=algo)
    assert_close(N(dx), dx_ref, "conv bwd data")
    # with the backward of the ReLU that produced x applied as dx is written: bit-identical to the data gradient
    # followed by the in-place mask (x here stands for that ReLU's output: its sign pattern is all that matters)
    if ops.conv2d_bwd_data_relu_supported(x.shape, w.shape, st, pad):
        dx0 = synth.normal(11, 8, x.shape)
        for alpha, beta in ((1.0, 0.0), (0.5, 2.0)):
            two = ops.conv2d_bwd_data(wd, dyd, x.shape, st, pad, alpha=alpha, beta=beta, dx=T(dx0, dev), algo=algo)
            ops.rect_backprop_inplace(xd, two)
            one = ops.conv2d_bwd_data(wd, dyd, x.shape, st, pad, alpha=alpha, beta=beta, dx=T(dx0, dev), algo=algo, relu_of=xd)
            assert torch.equal(one, two), "masked data gradient alpha=%g beta=%g" % (alpha, beta)
    else:
        assert st > 1
    torch.cuda.synchronize()


# 3x3 stride-1 layers in the Winograd F(2x2, 3x3) form: odd and even extents (tiles that hang over the edge), every
# padding it takes, channel counts that do not fill a group of four, filter counts around the 128-row tile, tile counts
# that are no multiple of the 32-tile block, more blocks than CUs, and the sizes the library takes the form for by itself
WINO_CASES = [
    # N, C, H, W, K, pad
    (2, 8, 6, 6, 8, 1),
    (3, 5, 7, 9, 130, 1),
    (1, 12, 8, 8, 16, 0),
    (2, 16, 5, 6, 20, 2),
    (1, 1, 3, 3, 1, 0),           # one output pixel
    (1, 2, 2, 2, 3, 1),
    (4, 70, 13, 13, 140, 1),
    (2, 64, 13, 13, 96, 1),
    (33, 64, 14, 15, 128, 1),
    (70, 66, 13, 13, 384, 1),     # 3 x 108 blocks
    (70, 64, 13, 13, 384, 1),     # forward: 324 blocks, the 68 past 256 in three slices of the channel loop (6, 6, 4 stages)
    (70, 384, 13, 13, 64, 1),     # the same in the data gradient
    (16, 128, 28, 28, 64, 1),
    (90, 64, 13, 13, 128, 1),     # 4410 tiles: the filter gradient in the form too, its tiles in several slices
]


@pytest.mark.parametrize("case", WINO_CASES, ids=str)
def test_conv2d_winograd(dev, case):
    """RH_ALGO_WINOGRAD against the oracle's direct convolution, forward and backward-data, with every epilogue the
    direct kernels have; the masked data gradient bit-identical to gradient + in-place mask; RH_ALGO_DIRECT and the
    loader bits keep the direct form; other geometries are refused."""
    Nn, C, H, W, K, pad = case
    say("winograd case", case)
    WG = _lib.RH_ALGO_WINOGRAD
    x = synth.normal(15, 1, (Nn, C, H, W))
    w = synth.normal(15, 2, (K, C, 3, 3))
    b = synth.normal(15, 3, (K,))
    y_ref = O.conv2d_fwd(x, w, 1, pad)
    dy = synth.normal(15, 4, y_ref.shape)
    xd, wd, bd, dyd = T(x, dev), T(w, dev), T(b, dev), T(dy, dev)
    y = ops.conv2d_fwd(xd, wd, 1, pad, algo=WG)
    assert_close(N(y), y_ref, "winograd fwd")
    yf = ops.conv2d_fwd(xd, wd, 1, pad, bias=bd, relu=True, algo=WG)
    assert_close(N(yf), O.rect_inplace(O.add_bias_nchw(b, y_ref.copy())), "winograd fwd fused bias+relu")
    # the fused epilogue is the separate passes' arithmetic
    two = ops.conv2d_fwd(xd, wd, 1, pad, algo=WG)
    assert torch.equal(torch.clamp_min(two + bd.view(1, -1, 1, 1), 0.0), yf), "winograd fused epilogue == conv, add_bias, rect"
    y0 = synth.normal(15, 5, y_ref.shape)
    yb = ops.conv2d_fwd(xd, wd, 1, pad, alpha=0.5, beta=2.0, y=T(y0, dev), algo=WG)
    assert_close(N(yb), O.conv2d_fwd(x, w, 1, pad, alpha=0.5, beta=2.0, y=y0.copy()), "winograd fwd alpha/beta")
    dx_ref = O.conv2d_bwd_data(w, dy, x.shape, 1, pad)
    dx = ops.conv2d_bwd_data(wd, dyd, x.shape, 1, pad, algo=WG)
    assert_close(N(dx), dx_ref, "winograd bwd data")
    dx0 = synth.normal(15, 8, x.shape)
    dxb = ops.conv2d_bwd_data(wd, dyd, x.shape, 1, pad, alpha=0.5, beta=2.0, dx=T(dx0, dev), algo=WG)
    assert_close(N(dxb), O.conv2d_bwd_data(w, dy, x.shape, 1, pad, 0.5, 2.0, dx0.copy()), "winograd bwd data alpha/beta")
    for alpha, beta in ((1.0, 0.0), (0.5, 2.0)):
        two = ops.conv2d_bwd_data(wd, dyd, x.shape, 1, pad, alpha=alpha, beta=beta, dx=T(dx0, dev), algo=WG)
        ops.rect_backprop_inplace(xd, two)
        one = ops.conv2d_bwd_data(wd, dyd, x.shape, 1, pad, alpha=alpha, beta=beta, dx=T(dx0, dev), algo=WG, relu_of=xd)
        assert torch.equal(one, two), "winograd masked data gradient alpha=%g beta=%g" % (alpha, beta)
    # the filter gradient in the same form (its sums run over the tiles, cut into slices added in a fixed order)
    dw_ref = O.conv2d_bwd_filter(x, dy, w.shape, 1, pad)
    dw = ops.conv2d_bwd_filter(xd, dyd, w.shape, 1, pad, algo=WG)
    assert_close(N(dw), dw_ref, "winograd bwd filter")
    dw0 = synth.normal(15, 6, w.shape)
    for alpha, beta in ((1.0, 1.0), (0.25, 1.0), (-3.0, 0.5)):
        dwa = ops.conv2d_bwd_filter(xd, dyd, w.shape, 1, pad, alpha=alpha, beta=beta, dw=T(dw0, dev), algo=WG)
        assert_close(N(dwa), O.conv2d_bwd_filter(x, dy, w.shape, 1, pad, alpha, beta, dw0.copy()),
                     "winograd bwd filter alpha=%g beta=%g" % (alpha, beta))
    db0 = synth.normal(15, 7, (K,))
    dwc, dbc = ops.conv2d_bwd_filter_bias(xd, dyd, w.shape, 1, pad, alpha=0.25, beta=1.0, dw=T(dw0, dev), db=T(db0, dev), algo=WG)
    assert torch.equal(dwc, ops.conv2d_bwd_filter(xd, dyd, w.shape, 1, pad, alpha=0.25, beta=1.0, dw=T(dw0, dev), algo=WG))
    assert_close(N(dbc), O.conv2d_bwd_bias(dy, 0.25, 1.0, db0.copy()), "bias gradient of the combined call (winograd)")
    # run to run the same bits
    assert torch.equal(ops.conv2d_fwd(xd, wd, 1, pad, algo=WG), y)
    assert torch.equal(ops.conv2d_bwd_filter(xd, dyd, w.shape, 1, pad, algo=WG), dw)
    # RH_ALGO_SHARED_GPU (other kernels run beside the call): whole blocks only, no sliced tail; the same result up to
    # summation order where a tail was sliced, the same bits where none was
    SH = _lib.RH_ALGO_SHARED_GPU
    ys = ops.conv2d_fwd(xd, wd, 1, pad, algo=WG | SH)
    dxs = ops.conv2d_bwd_data(wd, dyd, x.shape, 1, pad, algo=WG | SH)
    assert_close(N(ys), y_ref, "winograd fwd, shared-GPU hint")
    assert_close(N(dxs), dx_ref, "winograd bwd data, shared-GPU hint")
    blocks_b = -(-C // 128) * -(-(Nn * -(-H // 2) * -(-W // 2)) // 32)
    blocks_f = -(-K // 128) * -(-(Nn * -(-y_ref.shape[2] // 2) * -(-y_ref.shape[3] // 2)) // 32)
    if blocks_f <= 256 or C % 4: assert torch.equal(ys, y)
    if blocks_b <= 256 or K % 4: assert torch.equal(dxs, dx)
    # what the library picks by itself: this form from 64 channels on both sides, 128-row tiles three quarters full and
    # 192 blocks on, else a direct one
    auto = ops.conv2d_fwd(xd, wd, 1, pad)
    direct = ops.conv2d_fwd(xd, wd, 1, pad, algo=_lib.RH_ALGO_DIRECT)
    assert_close(N(direct), y_ref, "RH_ALGO_DIRECT fwd")
    blocks = -(-K // 128) * -(-(Nn * -(-y_ref.shape[2] // 2) * -(-y_ref.shape[3] // 2)) // 32)
    takes = C >= 64 and K >= 64 and 4 * K >= 3 * (-(-K // 128) * 128) and blocks >= 192
    assert torch.equal(auto, y if takes else direct), "library's choice"
    torch.cuda.synchronize()


WINO5_CASES = [
    # N, C, H, W, K, pad
    (2, 3, 9, 9, 8, 2),
    (1, 1, 5, 5, 1, 0),            # one output pixel
    (3, 5, 8, 11, 130, 1),
    (2, 8, 7, 6, 20, 4),
    (2, 16, 12, 13, 64, 3),
    (4, 32, 27, 27, 96, 2),
    (40, 32, 27, 27, 256, 2),      # 504 blocks: whole rounds and sliced tail blocks
    (70, 96, 13, 14, 128, 2),
    (44, 64, 27, 27, 128, 2),      # 539 blocks: the library takes this form by itself
]


@pytest.mark.parametrize("case", WINO5_CASES, ids=str)
def test_conv2d_winograd_5x5_forward(dev, case):
    """RH_ALGO_WINOGRAD on a 5x5 stride-1 layer (forward only): the filter as four 3x3 blocks of its 6x6 zero extension,
    F(2x2, 3x3) on each over the shifted input, added in the transform domain; against the oracle's direct convolution,
    with every epilogue; the backward passes refuse the bit; the library's own choice and RH_ALGO_DIRECT."""
    Nn, C, H, W, K, pad = case
    say("winograd 5x5 case", case)
    WG = _lib.RH_ALGO_WINOGRAD
    x = synth.normal(17, 1, (Nn, C, H, W))
    w = synth.normal(17, 2, (K, C, 5, 5))
    b = synth.normal(17, 3, (K,))
    y_ref = O.conv2d_fwd(x, w, 1, pad)
    xd, wd, bd = T(x, dev), T(w, dev), T(b, dev)
    y = ops.conv2d_fwd(xd, wd, 1, pad, algo=WG)
    assert_close(N(y), y_ref, "winograd 5x5 fwd")
    yf = ops.conv2d_fwd(xd, wd, 1, pad, bias=bd, relu=True, algo=WG)
    assert_close(N(yf), O.rect_inplace(O.add_bias_nchw(b, y_ref.copy())), "winograd 5x5 fwd fused bias+relu")
    assert torch.equal(torch.clamp_min(y + bd.view(1, -1, 1, 1), 0.0), yf), "fused epilogue == conv, add_bias, rect"
    y0 = synth.normal(17, 5, y_ref.shape)
    yb = ops.conv2d_fwd(xd, wd, 1, pad, alpha=0.5, beta=2.0, y=T(y0, dev), algo=WG)
    assert_close(N(yb), O.conv2d_fwd(x, w, 1, pad, alpha=0.5, beta=2.0, y=y0.copy()), "winograd 5x5 fwd alpha/beta")
    assert torch.equal(ops.conv2d_fwd(xd, wd, 1, pad, algo=WG), y), "run to run the same bits"
    assert_close(N(ops.conv2d_fwd(xd, wd, 1, pad, algo=WG | _lib.RH_ALGO_SHARED_GPU)), y_ref, "winograd 5x5 fwd, shared-GPU hint")
    assert ops.conv2d_winograd_flops(x.shape, w.shape, 1, pad, "fwd", algo=WG) == \
        2.0 * 16 * K * 4 * C * Nn * (-(-y_ref.shape[2] // 2)) * (-(-y_ref.shape[3] // 2))
    # forward only
    dy = T(synth.normal(17, 4, y_ref.shape), dev)
    for fn in (lambda: ops.conv2d_bwd_data(wd, dy, x.shape, 1, pad, algo=WG), lambda: ops.conv2d_bwd_filter(xd, dy, w.shape, 1, pad, algo=WG)):
        with pytest.raises(_lib.RembrandtHipError):
            fn()
    # the library's choice: this form for full row tiles and several rounds of blocks, else the direct one
    auto = ops.conv2d_fwd(xd, wd, 1, pad)
    direct = ops.conv2d_fwd(xd, wd, 1, pad, algo=_lib.RH_ALGO_DIRECT)
    assert_close(N(direct), y_ref, "RH_ALGO_DIRECT fwd (5x5)")
    blocks = -(-K // 128) * -(-(Nn * -(-y_ref.shape[2] // 2) * -(-y_ref.shape[3] // 2)) // 32)
    takes = C >= 64 and K >= 64 and 8 * K >= 7 * (-(-K // 128) * 128) and blocks >= 512
    assert torch.equal(auto, y if takes else direct), "library's choice (5x5)"
    torch.cuda.synchronize()


def test_conv2d_winograd_refused_geometries(dev):
    import ctypes as C
    x = torch.zeros((2, 4, 8, 8), device=dev)
    ws = torch.zeros((1 << 22,), dtype=torch.uint8, device=dev)
    for R, st, pad, extra in ((5, 2, 2, 0), (7, 1, 3, 0), (3, 2, 1, 0), (1, 1, 0, 0), (3, 1, 3, 0), (3, 1, 1, _lib.RH_ALGO_GATHER),
                              (3, 1, 1, _lib.RH_ALGO_DIRECT), (3, 1, 1, _lib.RH_MATH_BF16_MFMA_FP32ACC)):
        g = _lib.ConvGeom(2, 4, 8, 8, 4, R, R, st, pad)
        w = torch.zeros((4, 4, R, R), device=dev)
        P = (8 + 2 * pad - R) // st + 1
        y = torch.zeros((2, 4, P, P), device=dev)
        rc = _lib.lib().rh_conv2d_fwd(C.byref(g), 1.0, x.data_ptr(), w.data_ptr(), 0.0, y.data_ptr(), None, ws.data_ptr(), ws.numel(),
                                      _lib.RH_ALGO_WINOGRAD | extra, None)
        assert rc == _lib.RH_E_UNSUPPORTED, (R, st, pad, extra, rc)
        if not (extra & _lib.RH_MATH_BF16_MFMA_FP32ACC):
            rc = _lib.lib().rh_conv2d_bwd_data(C.byref(g), 1.0, w.data_ptr(), y.data_ptr(), 0.0, x.data_ptr(), ws.data_ptr(), ws.numel(),
                                               _lib.RH_ALGO_WINOGRAD | extra, None)
            assert rc == _lib.RH_E_UNSUPPORTED, ("bwd", R, st, pad, extra, rc)
            rc = _lib.lib().rh_conv2d_bwd_filter(C.byref(g), 1.0, x.data_ptr(), y.data_ptr(), 0.0, w.data_ptr(), ws.data_ptr(), ws.numel(),
                                                 _lib.RH_ALGO_WINOGRAD | extra, None)
            assert rc == _lib.RH_E_UNSUPPORTED, ("bwd filter", R, st, pad, extra, rc)


# input channels a multiple of 8 take the packed-operand form (bf16 copies of image and filter in 16-byte groups of
# eight channels): channel groups that do not fill a 64-wide tile, rectangular images, stride with padding, no padding,
# more filters than one row tile, a contraction shorter than one K step
BF16_PACKED_CASES = [
    (3, 72, 11, 9, 40, 3, 2, 1),
    (2, 8, 17, 17, 200, 5, 1, 2),
    (5, 16, 9, 12, 24, 3, 1, 0),
    (2, 8, 6, 6, 3, 1, 1, 0),
    (130, 8, 5, 5, 16, 3, 1, 1),
    # long contractions on grids of 256 and more 256-row tiles take the direct-to-LDS kernel: ragged rows and columns,
    # two row tiles, a strided layer, a 1x1 layer whose contraction is exactly four ring buffers long plus twelve steps;
    # the last two are grids as large on short contractions (the 128x128 kernel)
    (80, 24, 30, 30, 130, 5, 1, 2),
    (40, 64, 31, 29, 500, 3, 1, 1),
    (120, 64, 47, 45, 200, 3, 2, 1),
    (70, 512, 34, 33, 256, 1, 1, 0),
    (70, 8, 34, 33, 384, 1, 1, 0),
    (80, 8, 30, 30, 130, 5, 1, 2),
]


@pytest.mark.parametrize("case", CONV_CASES + BF16_PACKED_CASES, ids=[str(c) for c in CONV_CASES + BF16_PACKED_CASES])
def test_conv2d_fwd_bf16_operands(dev, case):
    """RH_MATH_BF16_MFMA_FP32ACC: operands rounded to bf16 (nearest even), products accumulated in fp32.
    Reference = the fp64-accumulating oracle on operands rounded the same way."""
    Nn, C, H, W, K, R, st, pad = case
    say("bf16 conv case", case)
    x = synth.normal(12, 1, (Nn, C, H, W))
    w = synth.normal(12, 2, (K, C, R, R))
    b = synth.normal(12, 3, (K,))
    y_ref = O.conv2d_fwd(O.round_bf16(x), O.round_bf16(w), st, pad)
    y = ops.conv2d_fwd(T(x, dev), T(w, dev), st, pad, algo=_lib.RH_MATH_BF16_MFMA_FP32ACC)
    assert_close(N(y), y_ref, "bf16 conv fwd")
    yf = ops.conv2d_fwd(T(x, dev), T(w, dev), st, pad, bias=T(b, dev), relu=True, algo=_lib.RH_MATH_BF16_MFMA_FP32ACC)
    assert_close(N(yf), O.rect_inplace(O.add_bias_nchw(b, y_ref.copy())), "bf16 conv fwd fused bias+relu")
    # operands that are already bf16 values give the fp32 path's result up to summation order
    xr, wr = O.round_bf16(x), O.round_bf16(w)
    y32 = ops.conv2d_fwd(T(xr, dev), T(wr, dev), st, pad)
    y16 = ops.conv2d_fwd(T(xr, dev), T(wr, dev), st, pad, algo=_lib.RH_MATH_BF16_MFMA_FP32ACC)
    assert_close(N(y16), N(y32), "bf16 path on bf16-exact operands == fp32 path")
    torch.cuda.synchronize()


BF16_CHAIN_CASES = [
    # N, C, H, W, K, R, stride, pad, halo of the packed result
    (3, 72, 11, 9, 40, 3, 2, 1, 0),
    (2, 8, 17, 17, 200, 5, 1, 2, 2),
    (5, 16, 9, 12, 24, 3, 1, 0, 1),
    (130, 8, 5, 5, 16, 3, 1, 1, 0),
    (80, 24, 30, 30, 136, 5, 1, 2, 1),     # the direct-to-LDS kernel
    (70, 512, 34, 33, 256, 1, 1, 0, 0),
    (4, 3, 35, 35, 16, 7, 2, 0, 0),        # grouped by filter columns: fp32 image in, packed result out
    # 1x1 layers of up to 128 channels with a packed result: the streaming kernel (pixel counts that are not a
    # multiple of the 32-pixel tile, every tile height, rows shorter than a tile, a bordered result)
    (3, 96, 54, 54, 96, 1, 1, 0, 0),
    (5, 32, 7, 5, 128, 1, 1, 0, 2),
    (2, 128, 13, 11, 32, 1, 1, 0, 1),
    (7, 64, 3, 3, 64, 1, 1, 0, 0),
    (3, 256, 9, 10, 256, 1, 1, 0, 1),     # two chunks of 128 output channels, the deep contraction
    (2, 256, 5, 5, 192, 1, 1, 0, 0),      # two chunks of 96
]


@pytest.mark.parametrize("case", BF16_CHAIN_CASES, ids=[str(c) for c in BF16_CHAIN_CASES])
def test_conv2d_fwd_bf16_packed_chain_forms(dev, case):
    """The forms of the bf16 forward that a forward-only chain uses are bit-identical to rh_conv2d_fwd with
    RH_MATH_BF16_MFMA_FP32ACC: a converted filter kept between calls, a packed bf16 input, and a packed bf16 result,
    which holds the fp32 result rounded to nearest even inside a border that stays zero."""
    Nn, C, H, W, K, R, st, pad, halo = case
    say("bf16 chain case", case)
    x = synth.normal(14, 1, (Nn, C, H, W))
    w = synth.normal(14, 2, (K, C, R, R))
    b = synth.normal(14, 3, (K,))
    xd, wd, bd = T(x, dev), T(w, dev), T(b, dev)
    for relu in (False, True):
        legacy = ops.conv2d_fwd(xd, wd, st, pad, bias=bd, relu=relu, algo=_lib.RH_MATH_BF16_MFMA_FP32ACC)
        y = ops.conv2d_fwd_bf16_packed(xd, wd, st, pad, bias=bd, relu=relu)
        assert torch.equal(y, legacy), "fp32 image in, fp32 result"
        yp = ops.conv2d_fwd_bf16_packed(xd, wd, st, pad, bias=bd, relu=relu, out_halo=halo)
        want = O.round_bf16(N(legacy))
        assert np.array_equal(N(ops.bf16_unpack(yp, legacy.shape, halo)), want), "packed result == rounded fp32 result"
        # the border of the packed result is untouched (zero): re-packing the unpacked interior reproduces every byte
        assert torch.equal(ops.bf16_pack(T(want, dev), halo), yp), "border"
        if C % 8 == 0:
            xp = ops.bf16_pack(xd, pad)
            assert np.array_equal(N(ops.bf16_unpack(xp, x.shape, pad)), O.round_bf16(x)), "pack / unpack"
            y2 = ops.conv2d_fwd_bf16_packed(xd, wd, st, pad, bias=bd, relu=relu, x_packed=xp)
            assert torch.equal(y2, legacy), "packed image in, fp32 result"
            yp2 = ops.conv2d_fwd_bf16_packed(xd, wd, st, pad, bias=bd, relu=relu, x_packed=xp, out_halo=halo)
            assert torch.equal(yp2, yp), "packed image in, packed result"
            # (the streaming 1x1 kernel wherever it can run, also where the tiled kernel is the one chosen)
            yp3 = ops.conv2d_fwd_bf16_packed(xd, wd, st, pad, bias=bd, relu=relu, x_packed=xp, out_halo=halo,
                                             algo=_lib.RH_ALGO_SCALAR_OFFSET)
            assert torch.equal(yp3, yp), "packed image in, packed result, streaming kernel where it runs"
    torch.cuda.synchronize()


BF16_POOL_CASES = [
    # N, C, H, W, size, stride, pad, rounding, halo of the result
    (3, 16, 13, 13, 3, 2, 0, 0, 1),
    (2, 96, 54, 54, 3, 2, 0, 1, 2),     # ceil extent: clipped windows at the bottom / right edge
    (4, 8, 9, 7, 2, 2, 0, 0, 0),
    (2, 24, 10, 11, 3, 2, 1, 0, 1),     # padded windows: padding never wins
    (1, 8, 5, 5, 3, 1, 1, 1, 0),
]


@pytest.mark.parametrize("case", BF16_POOL_CASES, ids=[str(c) for c in BF16_POOL_CASES])
def test_pool2d_fwd_bf16_packed(dev, case):
    """Max pooling of packed bf16 activations == the fp32 pooling's result rounded to bf16 (rounding is monotone),
    bit for bit, on inputs with ties, negative values and all-negative windows."""
    Nn, C, H, W, k, st, pad, rnd, halo = case
    say("bf16 pool case", case)
    x = synth.normal(15, 1, (Nn, C, H, W))
    x[:, :, ::3, ::2] = np.float32(-0.75)     # ties
    xd = T(x, dev)
    want = O.round_bf16(N(ops.pool2d_fwd(xd, k, st, pad, _lib.RH_POOL_MAX, rnd)))
    want_oracle = O.round_bf16(O.pool2d_fwd(x, k, st, pad, O.POOL_MAX, rnd))
    assert np.array_equal(want, want_oracle)
    yp, shape = ops.pool2d_fwd_bf16_packed(ops.bf16_pack(xd, 0), x.shape, k, st, pad, rnd, out_halo=halo)
    assert np.array_equal(N(ops.bf16_unpack(yp, shape, halo)), want)
    assert torch.equal(ops.bf16_pack(T(want, dev), halo), yp), "border"
    torch.cuda.synchronize()


SGEMM_CASES = [
    # transA, transB, m, n, k
    (1, 0, 500, 64, 2450),   # affine forward  Y = W^T X
    (0, 1, 300, 500, 64),    # affine bwd-W    dW += X dY^T
    (0, 0, 300, 64, 500),    # affine bwd-X    dX = W dY
    (1, 1, 37, 29, 53),
    (0, 0, 1, 10, 64),
    (0, 1, 1, 130, 70),      # the bias-gradient GEMV shape
    (1, 0, 4096, 32, 1024),  # few tiles, deep contraction -> split path
    # a side of at most sixteen: the plain kernels (a wave per element for long contractions, a thread per element
    # otherwise): a ten-class classifier's forward, data-gradient and weight-gradient products, every transposition
    (1, 0, 10, 64, 500),
    (0, 0, 500, 64, 10),
    (0, 1, 500, 10, 64),
    (0, 1, 64, 10, 128),
    (1, 1, 10, 33, 200),
    (1, 0, 16, 256, 129),
    (0, 0, 3, 5, 1),
]


@pytest.mark.parametrize("case", SGEMM_CASES, ids=[str(c) for c in SGEMM_CASES])
@pytest.mark.parametrize("use_ws", [True, False])
def test_sgemm(dev, case, use_ws):
    tA, tB, m, n, k = case
    say("sgemm case", case, "ws", use_ws)
    a_shape = (m, k) if tA else (k, m)   # memory shape (row-major view of a column-major array)
    b_shape = (k, n) if tB else (n, k)
    lda, ldb, ldc = a_shape[1] + 3, b_shape[1] + 1, m + 2
    A = synth.normal(12, 1, (a_shape[0], lda))
    B = synth.normal(12, 2, (b_shape[0], ldb))
    C0 = synth.normal(12, 3, (n, ldc))
    for alpha, beta in ((1.0, 0.0), (0.5, 1.0)):
        ref = O.sgemm(tA, tB, m, n, k, alpha, A, lda, B, ldb, beta, C0.copy(), ldc)
        Cd = T(C0, dev)
        ops.sgemm(tA, tB, m, n, k, alpha, T(A, dev), lda, T(B, dev), ldb, beta, Cd, ldc, use_workspace=use_ws)
        got = N(Cd)
        assert_close(got[:, :m], ref[:, :m], "sgemm alpha=%g beta=%g" % (alpha, beta))
        assert np.array_equal(got[:, m:], C0[:, m:]), "sgemm wrote outside ldc padding"


@pytest.mark.parametrize("case", [
    # (m = out channels, n = batch, k = in channels): one block, several tiles, a split contraction with the dense
    # 16-byte reduction, one with the many-slice reduction, odd extents with a padded result (scalar reduction)
    (10, 4, 50), (10, 64, 500), (500, 64, 800), (4096, 32, 1024), (96, 16, 9216), (1001, 33, 2450), (1000, 256, 4096),
])
def test_sgemm_bias_act(dev, case):
    """rh_sgemm_bias_act = matrix product, bias row, activation of the affine forward pass in one call: bit-identical
    to the library's own three calls, and within tolerance of the oracle's."""
    m, n, k = case
    W = synth.normal(14, 1, (m, k))
    X = synth.normal(14, 2, (n, k))
    b = synth.normal(14, 3, (m,))
    for ldc, use_ws, relu, beta in ((m, True, True, 0.0), (m + (4 if m % 4 == 0 else 3), True, True, 0.0),
                                    (m, False, False, 0.0), (m, True, True, 0.5)):
        say("sgemm_bias_act", case, "ldc", ldc, "ws", use_ws, "relu", relu, "beta", beta)
        C0 = synth.normal(14, 4, (n, ldc))
        ref = O.sgemm(1, 0, m, n, k, 1.0, W, k, X, k, beta, C0.copy(), ldc)
        ref[:, :m] += b[None, :]
        if relu:
            ref[:, :m] = np.maximum(ref[:, :m], 0)
        Cd = T(C0, dev)
        ops.sgemm(1, 0, m, n, k, 1.0, T(W, dev), k, T(X, dev), k, beta, Cd, ldc, use_workspace=use_ws, bias=T(b, dev), relu=relu)
        got = N(Cd)
        assert_close(got[:, :m], ref[:, :m], "sgemm_bias_act")
        assert np.array_equal(got[:, m:], C0[:, m:]), "wrote into the ldc padding"
        if ldc == m:
            Cs = T(C0, dev)
            ops.sgemm(1, 0, m, n, k, 1.0, T(W, dev), k, T(X, dev), k, beta, Cs, ldc, use_workspace=use_ws)
            ops.add_bias_nchw(T(b, dev), Cs.view(n, m, 1, 1))
            if relu:
                ops.rect_inplace(Cs)
            assert np.array_equal(N(Cs), got), "fused and separate calls differ"


def test_bias_relu(dev):
    for shape in [(3, 7, 5, 9), (2, 96, 27, 27), (64, 500), (5, 3, 16, 20)]:
        say("bias/relu", shape)
        y = synth.normal(13, 1, shape)
        b = synth.normal(13, 2, (shape[1],))
        yd = T(y, dev)
        ops.add_bias_nchw(T(b, dev), yd)
        ref = O.add_bias_nchw(b, y.copy())
        assert_close(N(yd), ref, "add_bias")
        ops.rect_inplace(yd)
        ref = O.rect_inplace(ref)
        assert np.array_equal(N(yd) > 0, ref > 0)
        assert_close(N(yd), ref, "rect")
        dy = synth.normal(13, 3, shape)
        dyd = T(dy, dev)
        ops.rect_backprop_inplace(yd, dyd)
        assert np.array_equal(N(dyd), O.rect_backprop_inplace(ref, dy.copy())), "rect backprop is a pure mask"


POOL_CASES = [
    # N, C, H, size, stride, pad
    (2, 3, 9, 3, 2, 0), (2, 3, 9, 3, 2, 1), (3, 4, 8, 2, 2, 0), (2, 2, 10, 3, 2, 0), (2, 5, 27, 3, 2, 0),
    (1, 2, 6, 6, 1, 0), (2, 3, 7, 3, 1, 1), (2, 2, 13, 3, 3, 1),
    (1, 3, 112, 3, 2, 1),   # planes above a block's LDS share: forward in bands of output rows, backward with
    (1, 2, 130, 3, 2, 0),   # several windows per thread and colour / (130: above 60 KB) by the gather kernel
    (1, 1, 20, 7, 3, 2),    # three colours per axis: gather backward
]


@pytest.mark.parametrize("case", POOL_CASES, ids=[str(c) for c in POOL_CASES])
@pytest.mark.parametrize("mode", [_lib.RH_POOL_MAX, _lib.RH_POOL_AVG_INCL_PAD])
@pytest.mark.parametrize("rounding", [_lib.RH_ROUND_FLOOR, _lib.RH_ROUND_CEIL])
def test_pool2d(dev, case, mode, rounding):
    Nn, C, H, k, st, pad = case
    say("pool case", case, mode, rounding)
    x = synth.normal(14, 1, (Nn, C, H, H + 1))
    # repeated values so that the first-maximum tie rule is exercised
    x = np.round(x * 2) / 2
    y_ref, am_ref = O.pool2d_fwd(x, k, st, pad, mode, rounding, want_argmax=True)
    if y_ref.size == 0:
        pytest.skip("empty output")
    xd = T(x, dev)
    y, am = ops.pool2d_fwd(xd, k, st, pad, mode, rounding, want_argmax=True)
    assert_close(N(y), y_ref, "pool fwd")
    if mode == _lib.RH_POOL_MAX:
        assert np.array_equal(N(am), am_ref), "arg-max mask is bit-exact"
    dy = synth.normal(14, 2, y_ref.shape)
    dx_ref = O.pool2d_bwd(x, y_ref, dy, k, st, pad, mode, rounding)
    dx = ops.pool2d_bwd(xd, y, T(dy, dev), k, st, pad, mode, rounding)
    assert_close(N(dx), dx_ref, "pool bwd (recomputed arg-max)")
    if mode == _lib.RH_POOL_MAX:
        dx2 = ops.pool2d_bwd(xd, y, T(dy, dev), k, st, pad, mode, rounding, argmax=am)
        # same elements, same values up to the order in which an element's (at most four) contributions are added
        assert np.array_equal(N(dx2) == 0, N(dx) == 0), "mask-driven backward routes to the same elements"
        assert_close(N(dx2), dx_ref, "pool bwd (arg-max mask)")
        assert np.allclose(N(dx2), N(dx), rtol=1e-6, atol=2e-6), "mask-driven backward equals recomputed"
        again = ops.pool2d_bwd(xd, y, T(dy, dev), k, st, pad, mode, rounding, argmax=am)
        assert np.array_equal(N(dx2), N(again)), "the mask-driven backward is deterministic"


@pytest.mark.parametrize("case", POOL_CASES + [(2, 3, 55, 3, 2, 0), (3, 2, 31, 5, 4, 2)], ids=str)
@pytest.mark.parametrize("rounding", [_lib.RH_ROUND_FLOOR, _lib.RH_ROUND_CEIL])
def test_pool2d_one_byte_mask(dev, case, rounding):
    """The one-byte mask (the winner's slot r*size + s inside its window, 255 for none) names the same elements as the
    int32 plane index, bit for bit; the pooled values are identical; the backward pass from it, without and with the ReLU
    mask of the operator below folded in, is bit-identical to the one from the int32 mask."""
    Nn, C, H, k, st, pad = case
    shape = (Nn, C, H, H + 1)
    say("pool one-byte mask case", case, rounding)
    if not ops.pool2d_slot_supported(shape, k, st, pad, rounding):
        g = ops.pool_geom(shape, k, st, pad, _lib.RH_POOL_MAX, rounding)
        dummy = torch.zeros(16, device=dev)
        assert _lib.lib().rh_pool2d_fwd_slot(C_.byref(g), dummy.data_ptr(), dummy.data_ptr(), dummy.data_ptr(), None) == _lib.RH_E_UNSUPPORTED
        pytest.skip("no one-byte form for this geometry (three colours per axis or planes beyond the LDS kernels)")
    x = np.round(synth.normal(17, 1, shape) * 2) / 2 - np.float32(0.5)     # ties, and windows that are all negative
    xd = T(x, dev)
    y, am = ops.pool2d_fwd(xd, k, st, pad, _lib.RH_POOL_MAX, rounding, want_argmax=True)
    y2, slot = ops.pool2d_fwd_slot(xd, k, st, pad, rounding)
    assert torch.equal(y, y2)
    am_h, slot_h = N(am), N(slot).astype(np.int64)
    P, Q = am_h.shape[2], am_h.shape[3]
    hs = (np.arange(P) * st - pad)[:, None]
    ws = (np.arange(Q) * st - pad)[None, :]
    plane = (hs + slot_h // k) * shape[3] + ws + slot_h % k
    assert np.array_equal(np.where(slot_h == 255, -1, plane), am_h), "slot names the element the plane index names"
    assert (slot_h[slot_h != 255] < k * k).all()
    dy = T(synth.normal(17, 2, tuple(y.shape)), dev)
    assert torch.equal(ops.pool2d_bwd_slot(shape, dy, slot, k, st, pad, rounding),
                       ops.pool2d_bwd(xd, y, dy, k, st, pad, _lib.RH_POOL_MAX, rounding, argmax=am))
    assert torch.equal(ops.pool2d_bwd_slot(shape, dy, slot, k, st, pad, rounding, relu_y=y),
                       ops.pool2d_bwd_relu(shape, y, dy, k, st, pad, am, rounding))
    torch.cuda.synchronize()


@pytest.mark.parametrize("shape", [(64, 10), (256, 1000), (7, 1), (3, 5000)])
def test_softmax_loss_argmax(dev, shape):
    Nn, C = shape
    say("softmax case", shape)
    x = synth.normal(15, 1, shape, 0.0, 3.0)
    labels = synth.integers(15, 2, (Nn,), C)
    weights = synth.uniform(15, 3, (Nn,), 0.1, 1.0)
    xd, ld, wd = T(x, dev), T(labels, dev), T(weights, dev)
    p_ref = O.softmax_fwd(x)
    p = ops.softmax_fwd(xd)
    assert_close(N(p), p_ref, "softmax", atol=1e-7)
    d = ops.softmax_kl_backward(p, ld, wd)
    assert_close(N(d), O.softmax_kl_backward(N(p), labels, weights), "kl backward", atol=1e-7)
    l1 = ops.softmax_kl_loss1(p, ld, wd)
    l1_ref = O.softmax_kl_loss1(N(p), labels, weights)
    assert_close(N(l1), l1_ref, "kl loss1")
    l1b = ops.softmax_kl_loss1(p, ld, wd, beta=1.0, loss1=l1.clone())
    assert_close(N(l1b), 2 * l1_ref, "kl loss1 accumulate")
    tot = ops.blockreduce_sum(l1.reshape(1, Nn))
    assert_close(N(tot), O.blockreduce_sum(N(l1).reshape(1, Nn)), "loss sum")
    mx, idx = ops.blockreduce_argmax(p)
    mx_ref, idx_ref = O.blockreduce_argmax(N(p))
    assert np.array_equal(N(idx), idx_ref), "arg-max is bit-exact"
    assert np.array_equal(N(mx), mx_ref)


@pytest.mark.parametrize("shape", [(1, 1), (3, 10), (64, 10), (128, 1000), (256, 1000), (700, 37), (5, 3000)])
def test_softmax_kl_step_equals_separate_calls(dev, shape):
    """The one-launch form of the loss operator's train step is bit-identical to the five separate kernels, three
    calls in a row on one counter word (the kernel leaves it at zero)."""
    Nn, C = shape
    counter = None
    for rep in range(3):
        say("softmax_kl_step", shape, "call", rep)
        x = synth.normal(17, rep + 1, shape, 0.0, 3.0)
        if rep == 2 and C > 2:
            x[:, 1] = x[:, 0] = x.max(axis=1) + 1.0      # ties for the maximum: the lowest index wins
        labels = synth.integers(17, 10 + rep, (Nn,), C)
        weights = synth.uniform(17, 20 + rep, (Nn,), 0.1, 1.0)
        xd, ld, wd = T(x, dev), T(labels, dev), T(weights, dev)
        p, mx, idx, l1, tot, dx, counter = ops.softmax_kl_step(xd, ld, wd, counter)
        p_s = ops.softmax_fwd(xd)
        mx_s, idx_s = ops.blockreduce_argmax(p_s)
        l1_s = ops.softmax_kl_loss1(p_s, ld, wd)
        tot_s = ops.blockreduce_sum(l1_s.reshape(1, Nn))
        dx_s = ops.softmax_kl_backward(p_s, ld, wd)
        for name, a, b in (("p", p, p_s), ("max", mx, mx_s), ("argmax", idx, idx_s), ("loss1", l1, l1_s), ("loss", tot, tot_s),
                           ("dx", dx, dx_s)):
            assert np.array_equal(N(a), N(b)), name
        assert int(N(counter)[0]) == 0
        assert_close(N(p), O.softmax_fwd(x), "softmax", atol=1e-7)
        assert np.array_equal(N(idx), O.blockreduce_argmax(N(p))[1])


AFFINE2_CASES = [
    # B, I, H, C, relu
    (64, 800, 160, 10, True),     # a LeNet-like classifier of 2^17 weights
    (128, 1024, 64, 10, True),    # the CIFAR-10 network's
    (1, 7, 5, 3, False),
    (5, 33, 130, 64, True),       # ragged wave groups, the widest class count
    (37, 1022, 1, 2, False),      # odd input count: the element-wise weight-gradient form
    (256, 4096, 32, 17, True),    # the widest input the form takes
]


@pytest.mark.parametrize("case", AFFINE2_CASES)
def test_affine2_softmax_kl_step(dev, case):
    """The classifier tail in two launches against the oracle's separate operators: two affine layers, softmax,
    arg-max, loss, KL delta, the data gradients of both layers, then all four parameter gradients (beta 0 and 1);
    two calls in a row on one counter word."""
    B, I, H, Cc, relu = case
    assert ops.affine2_softmax_kl_step_supported(B, I, H, Cc)
    counter = None
    for rep in range(2):
        say("affine2_softmax_kl_step", case, "call", rep)
        x = synth.normal(41, 10 * rep + 1, (B, I))
        w1 = synth.normal(41, 10 * rep + 2, (H, I), 0.0, 1.0 / np.sqrt(I))
        b1 = synth.normal(41, 10 * rep + 3, (H,), 0.0, 0.5)
        w2 = synth.normal(41, 10 * rep + 4, (Cc, H), 0.0, 1.0 / np.sqrt(H))
        b2 = synth.normal(41, 10 * rep + 5, (Cc,), 0.0, 0.5)
        labels = synth.integers(41, 10 * rep + 6, (B,), Cc)
        weights = synth.uniform(41, 10 * rep + 7, (B,), 0.1, 1.0)
        # the oracle's operators, one after the other (column-major products as AffineOperator issues them)
        h = O.sgemm(1, 0, H, B, I, 1.0, w1, I, x, I, 0.0, np.zeros((B, H), np.float32), H) + b1
        if relu:
            h = np.maximum(h, 0.0).astype(np.float32)
        logits = O.sgemm(1, 0, Cc, B, H, 1.0, w2, H, h, H, 0.0, np.zeros((B, Cc), np.float32), Cc) + b2
        p = O.softmax_fwd(logits)
        dl = O.softmax_kl_backward(p, labels, weights)
        l1 = O.softmax_kl_loss1(p, labels, weights)
        dh = O.sgemm(0, 0, H, B, Cc, 1.0, w2, H, dl, Cc, 0.0, np.zeros((B, H), np.float32), H)
        if relu:
            dh = dh * (h > 0)
        dx = O.sgemm(0, 0, I, B, H, 1.0, w1, I, dh, H, 0.0, np.zeros((B, I), np.float32), I)
        out = ops.affine2_softmax_kl_step(T(x, dev), T(w1, dev), T(b1, dev), T(w2, dev), T(b2, dev), T(labels, dev), T(weights, dev),
                                          relu1=relu, want_dx=(rep == 0), counter=counter)
        counter = out["counter"]
        assert int(N(counter)[0]) == 0
        assert_close(N(out["h"]), h, "affine2 h")
        assert_close(N(out["logits"]), logits, "affine2 logits")
        assert_close(N(out["p"]), p, "affine2 softmax", atol=1e-6)
        assert np.array_equal(N(out["idx"]), O.blockreduce_argmax(N(out["p"]))[1]), "affine2 arg-max of its own probabilities"
        assert np.array_equal(N(out["max"]), N(out["p"]).max(axis=1))
        assert_close(N(out["loss1"]), l1, "affine2 loss1")
        assert_close(N(out["loss"]), np.array([l1.astype(np.float64).sum()], np.float32), "affine2 loss sum")
        assert_close(N(out["dlogits"]), dl, "affine2 dlogits")
        # the hidden delta is masked by the GPU's own h (an h within rounding of 0 may differ in sign from the oracle's)
        dh_gpu_mask = O.sgemm(0, 0, H, B, Cc, 1.0, w2, H, N(out["dlogits"]), Cc, 0.0, np.zeros((B, H), np.float32), H)
        if relu:
            dh_gpu_mask = dh_gpu_mask * (N(out["h"]) > 0)
        assert_close(N(out["dh"]), dh_gpu_mask, "affine2 dh")
        if rep == 0:
            dx_ref = O.sgemm(0, 0, I, B, H, 1.0, w1, I, N(out["dh"]), H, 0.0, np.zeros((B, I), np.float32), I)
            assert_close(N(out["dx"]), dx_ref, "affine2 dx")
            if not relu:
                assert_close(N(out["dx"]), dx, "affine2 dx (oracle chain)")
        # parameter gradients from the GPU's own activations and deltas
        hh, dhh, dll = N(out["h"]), N(out["dh"]), N(out["dlogits"])
        for beta1, beta2 in ((0.0, 0.0), (1.0, 1.0), (0.5, 0.0)):
            dw1_0, db1_0 = synth.normal(41, 10 * rep + 8, (H, I)), synth.normal(41, 10 * rep + 9, (H,))
            dw2_0, db2_0 = synth.normal(41, 10 * rep + 10, (Cc, H)), synth.normal(41, 10 * rep + 11, (Cc,))
            dw1, db1, dw2, db2 = T(dw1_0, dev), T(db1_0, dev), T(dw2_0, dev), T(db2_0, dev)
            ops.affine2_bwd_params(T(x, dev), out["h"], out["dh"], out["dlogits"], dw1, db1, dw2, db2, beta1, beta2)
            r1 = O.sgemm(0, 1, I, H, B, 1.0, x, I, dhh, H, beta1, dw1_0.copy(), I)
            r2 = O.sgemm(0, 1, H, Cc, B, 1.0, hh, H, dll, Cc, beta2, dw2_0.copy(), H)
            assert_close(N(dw1), r1, "affine2 dW1 beta %g" % beta1)
            assert_close(N(dw2), r2, "affine2 dW2 beta %g" % beta2)
            assert_close(N(db1), (dhh.astype(np.float64).sum(axis=0) + beta1 * db1_0).astype(np.float32), "affine2 db1 beta %g" % beta1)
            assert_close(N(db2), (dll.astype(np.float64).sum(axis=0) + beta2 * db2_0).astype(np.float32), "affine2 db2 beta %g" % beta2)


@pytest.mark.parametrize("case", [(64, 500, 10, True), (3, 2048, 64, False), (130, 1, 2, True), (256, 384, 17, True)])
def test_affine_softmax_kl_step_from_h(dev, case):
    """The form that starts from the first layer's output (I = 0, x = NULL): second layer, loss step and the hidden
    delta in one launch, dW2 and db2 in another; h and the first layer's gradients are left untouched."""
    B, H, Cc, relu = case
    assert ops.affine2_softmax_kl_step_supported(B, 0, H, Cc)
    counter = None
    for rep in range(2):
        say("affine_softmax_kl_step_from_h", case, "call", rep)
        h = synth.normal(43, 10 * rep + 1, (B, H))
        if relu:
            h = np.maximum(h, 0.0).astype(np.float32)
        w2 = synth.normal(43, 10 * rep + 4, (Cc, H), 0.0, 1.0 / np.sqrt(H))
        b2 = synth.normal(43, 10 * rep + 5, (Cc,), 0.0, 0.5)
        labels = synth.integers(43, 10 * rep + 6, (B,), Cc)
        weights = synth.uniform(43, 10 * rep + 7, (B,), 0.1, 1.0)
        logits = O.sgemm(1, 0, Cc, B, H, 1.0, w2, H, h, H, 0.0, np.zeros((B, Cc), np.float32), Cc) + b2
        p = O.softmax_fwd(logits)
        dl = O.softmax_kl_backward(p, labels, weights)
        l1 = O.softmax_kl_loss1(p, labels, weights)
        h_dev = T(h, dev)
        out = ops.affine_softmax_kl_step_from_h(h_dev, T(w2, dev), T(b2, dev), T(labels, dev), T(weights, dev), relu1=relu,
                                                counter=counter)
        counter = out["counter"]
        assert int(N(counter)[0]) == 0
        assert np.array_equal(N(h_dev), h), "h is an input here"
        assert_close(N(out["logits"]), logits, "from_h logits")
        assert_close(N(out["p"]), p, "from_h softmax", atol=1e-6)
        assert np.array_equal(N(out["idx"]), O.blockreduce_argmax(N(out["p"]))[1])
        assert np.array_equal(N(out["max"]), N(out["p"]).max(axis=1))
        assert_close(N(out["loss1"]), l1, "from_h loss1")
        assert_close(N(out["loss"]), np.array([l1.astype(np.float64).sum()], np.float32), "from_h loss sum")
        assert_close(N(out["dlogits"]), dl, "from_h dlogits")
        dh = O.sgemm(0, 0, H, B, Cc, 1.0, w2, H, N(out["dlogits"]), Cc, 0.0, np.zeros((B, H), np.float32), H)
        if relu:
            dh = dh * (h > 0)
        assert_close(N(out["dh"]), dh, "from_h dh")
        dll = N(out["dlogits"])
        for beta2 in (0.0, 1.0):
            dw2_0, db2_0 = synth.normal(43, 10 * rep + 10, (Cc, H)), synth.normal(43, 10 * rep + 11, (Cc,))
            dw2, db2 = T(dw2_0, dev), T(db2_0, dev)
            ops.affine_bwd_params_from_h(h_dev, out["dlogits"], dw2, db2, beta2)
            r2 = O.sgemm(0, 1, H, Cc, B, 1.0, h, H, dll, Cc, beta2, dw2_0.copy(), H)
            assert_close(N(dw2), r2, "from_h dW2 beta %g" % beta2)
            assert_close(N(db2), (dll.astype(np.float64).sum(axis=0) + beta2 * db2_0).astype(np.float32), "from_h db2 beta %g" % beta2)
            # with dh and db1: the first layer's bias gradient too, the second layer's unchanged bit for bit
            db1_0 = synth.normal(43, 10 * rep + 12, (H,))
            dw2b, db2b, db1 = T(dw2_0, dev), T(db2_0, dev), T(db1_0, dev)
            ops.affine_bwd_params_from_h(h_dev, out["dlogits"], dw2b, db2b, beta2, dh=out["dh"], db1=db1, beta1=beta2)
            assert torch.equal(dw2b, dw2) and torch.equal(db2b, db2)
            assert_close(N(db1), (N(out["dh"]).astype(np.float64).sum(axis=0) + beta2 * db1_0).astype(np.float32),
                         "from_h db1 beta %g" % beta2)
        # db1 without dh is refused
        assert _lib.lib().rh_affine2_bwd_params(B, 0, H, Cc, None, h_dev.data_ptr(), None, out["dlogits"].data_ptr(), 0.0, None,
                                                db1.data_ptr(), 0.0, dw2.data_ptr(), db2.data_ptr(), None) == _lib.RH_E_INVALID


def test_affine2_softmax_kl_step_limits(dev):
    x8 = torch.zeros((2, 8), device=dev)
    # I = 0 goes with x = NULL and the other way round
    assert _lib.lib().rh_affine2_softmax_kl_step(2, 0, 4, 2, 1, *([x8.data_ptr()] * 19), None) == _lib.RH_E_INVALID
    assert _lib.lib().rh_affine2_softmax_kl_step(2, 8, 4, 2, 1, None, *([x8.data_ptr()] * 18), None) == _lib.RH_E_INVALID
    assert ops.affine2_softmax_kl_step_supported(64, 0, 500, 10)
    assert not ops.affine2_softmax_kl_step_supported(64, 0, 2049, 10)
    assert not ops.affine2_softmax_kl_step_supported(64, 4097, 10, 10)
    assert not ops.affine2_softmax_kl_step_supported(64, 2450, 500, 10)     # more than 2^17 weights in the first layer
    assert not ops.affine2_softmax_kl_step_supported(1024, 4096, 32, 10)    # more than 2^26 multiply-adds over the batch
    assert not ops.affine2_softmax_kl_step_supported(64, 100, 100, 65)
    x = torch.zeros((2, 8), device=dev)
    z = lambda *s: torch.zeros(s, device=dev)
    rc = _lib.lib().rh_affine2_softmax_kl_step(2, 8, 4, 65, 1, *([x.data_ptr()] * 19), None)
    assert rc == _lib.RH_E_UNSUPPORTED


def test_argmax_ties(dev):
    x = np.zeros((4, 700), np.float32)
    x[0, [5, 300, 699]] = 2.0
    x[1, :] = 1.0
    x[2, 699] = 3.0
    x[3, [64, 65]] = 7.0
    mx, idx = ops.blockreduce_argmax(T(x, dev))
    assert N(idx).tolist() == [5, 0, 699, 64]
    assert N(mx).tolist() == [2.0, 1.0, 3.0, 7.0]


@pytest.mark.parametrize("n", [1, 5, 1000, 1 << 20 | 3])
def test_blas1_sgd(dev, n):
    say("blas1/sgd n", n)
    x = synth.normal(16, 1, (n,))
    y = synth.normal(16, 2, (n,))
    yd = T(y, dev)
    ops.saxpy(0.25, T(x, dev), yd)
    assert_close(N(yd), O.saxpy(0.25, x, y.copy()), "saxpy")
    ops.sscal(-1.5, yd)
    assert_close(N(yd), O.sscal(-1.5, O.saxpy(0.25, x, y.copy())), "sscal")
    # unaligned views
    if n > 8:
        yd2 = T(y, dev)
        ops.saxpy(2.0, T(x, dev)[1:], yd2[1:])
        assert_close(N(yd2)[1:], O.saxpy(2.0, x[1:].copy(), y[1:].copy()), "saxpy unaligned")
        assert N(yd2)[0] == y[0]
    W, g, v = synth.normal(16, 3, (n,)), synth.normal(16, 4, (n,)), synth.normal(16, 5, (n,))
    for (l2, scale, mu, apply, zg) in [(5e-4, -0.01, 0.9, 1.0, True), (0.0, 1.0, 0.9, -0.01, False)]:
        Wd, gd, vd = T(W, dev), T(g, dev), T(v, dev)
        ops.sgd_momentum_step(Wd, gd, vd, l2, scale, mu, apply, zg)
        Wr, gr, vr = W.copy(), g.copy(), v.copy()
        O.sgd_momentum_step(Wr, gr, vr, l2, scale, mu, apply, zg)
        assert_close(N(Wd), Wr, "sgd W", atol=1e-7)
        assert_close(N(vd), vr, "sgd v", atol=1e-7)
        assert_close(N(gd), gr, "sgd g", atol=1e-7)
    Wd, gd = T(W, dev), T(g, dev)
    ops.descend(Wd, gd, 0.05, 1e-3)
    Wr, gr = W.copy(), g.copy()
    O.descend(Wr, gr, 0.05, 1e-3)
    assert_close(N(Wd), Wr, "descend W", atol=1e-7)
    assert_close(N(gd), gr, "descend g", atol=1e-7)


def test_sgd_multi_tensor_step(dev):
    """One launch over many parameter blocks == one rh_sgd_momentum_step per block, bit for bit, and the oracle:
    lengths around the 1024-element block and the 4-element vector boundaries, an empty block, unaligned views,
    per-block l2 (zero for some), more blocks than one launch's table holds (48), both zero_grad settings."""
    lens = [1, 3, 4, 5, 96, 1023, 1024, 1025, 4096, 0, 2049, 34848, 1 << 18 | 1] + [7 * i + 1 for i in range(60)]
    say("multi-tensor sgd over", len(lens), "blocks")
    for zg in (True, False):
        host, multi, single = [], [], []
        for k, n in enumerate(lens):
            off = k % 3 if n > 16 else 0        # some blocks start 4 or 8 bytes off a 16-byte boundary
            W, g, v = (synth.normal(17, 10 * k + j, (n + off,)) for j in range(3))
            l2 = 0.0 if k % 4 == 0 else 1e-3 * (1 + k % 5)
            host.append((W[off:].copy(), g[off:].copy(), v[off:].copy(), l2))
            multi.append(tuple(T(a, dev)[off:] for a in (W, g, v)) + (l2,))
            single.append(tuple(T(a, dev)[off:] for a in (W, g, v)) + (l2,))
        ops.sgd_momentum_step_multi(multi, -0.01, 0.9, 1.0, zg)
        for (W, g, v, l2) in single:
            if W.numel():
                ops.sgd_momentum_step(W, g, v, l2, -0.01, 0.9, 1.0, zg)
        for k, ((Wm, gm, vm, _), (Ws, gs, vs, _), (Wh, gh, vh, l2)) in enumerate(zip(multi, single, host)):
            assert torch.equal(Wm, Ws) and torch.equal(gm, gs) and torch.equal(vm, vs), "block %d" % k
            if Wh.size:
                O.sgd_momentum_step(Wh, gh, vh, l2, -0.01, 0.9, 1.0, zg)
                assert_close(N(Wm), Wh, "multi sgd W[%d]" % k, atol=1e-7)
                assert_close(N(vm), vh, "multi sgd v[%d]" % k, atol=1e-7)
                assert_close(N(gm), gh, "multi sgd g[%d]" % k, atol=1e-7)
    assert _lib.lib().rh_sgd_momentum_step_multi(1, None, 1.0, 0.9, 1.0, 1, None) == _lib.RH_E_INVALID
    # keep_grad: those tensors' gradients are read for the update and left untouched (not zeroed, not regularised in
    # place); W and v as in the plain step, the other tensors as without the flag
    lens = (5, 4099, 1 << 16)
    host = [(synth.normal(19, 3 * k + 1, (n,)), synth.normal(19, 3 * k + 2, (n,)), synth.normal(19, 3 * k + 3, (n,))) for k, n in enumerate(lens)]
    for zg in (True, False):
        a = [tuple(T(x, dev) for x in h) + (0.01,) for h in host]
        b = [tuple(T(x, dev) for x in h) + (0.01,) for h in host]
        ops.sgd_momentum_step_multi(a, -0.01, 0.9, 1.0, zg, keep_grad=(0, 2))
        ops.sgd_momentum_step_multi(b, -0.01, 0.9, 1.0, zg)
        for k in range(3):
            assert torch.equal(a[k][0], b[k][0]) and torch.equal(a[k][2], b[k][2]), "keep_grad changed W or v of block %d" % k
            if k in (0, 2):
                assert np.array_equal(N(a[k][1]), host[k][1]), "a kept gradient was written"
            else:
                assert torch.equal(a[k][1], b[k][1])
    torch.cuda.synchronize()


def test_cast_and_fill(dev):
    x = (synth.integers(17, 1, (1000003,), 256)).astype(np.uint8)
    y = ops.cast_u8_f32(T(x, dev), 1.0 / 255.0)
    assert np.array_equal(N(y), O.cast_u8_f32(x, 1.0 / 255.0))
    t = torch.empty(1027, device=dev)
    ops.memset_f32(t[1:], 1.0)
    assert (N(t)[1:] == 1.0).all()


def test_preproc_kernels(dev):
    say("preproc kernels")
    x = synth.normal(13, 1, (5, 3, 37, 41))
    xd = T(x, dev)
    for (cw, ch, ow, oh) in ((41, 37, 0, 0), (32, 32, 9, 5), (1, 1, 40, 36), (17, 3, 0, 34)):
        assert np.array_equal(N(ops.crop_nchw(xd, cw, ch, ow, oh)), O.crop_nchw(x, cw, ch, ow, oh))
    assert np.array_equal(N(ops.flip_x(xd)), O.flip_x(x))
    wide = synth.normal(13, 2, (2, 1, 3, 300))     # wider than the 256 the reference asserts
    assert np.array_equal(N(ops.flip_x(T(wide, dev))), O.flip_x(wide))
    alphas, svals, svecs = synth.normal(13, 3, (15,)), synth.uniform(13, 4, (3,)), synth.normal(13, 5, (9,))
    assert_close(N(ops.pca3_noise(xd, T(alphas, dev), T(svals, dev), T(svecs, dev))), O.pca3_noise(x, alphas, svals, svecs),
                 "pca3 noise")
    # mean subtraction is the bias-add kernel with one "channel" per frame element
    mean = synth.normal(13, 6, (3, 37, 41))
    for normalize in (False, True):
        y = T(x, dev).clone()
        ops.add_bias_nchw(T(mean.ravel(), dev), y.view(5, -1, 1), alpha=(-1.0 / 255.0 if normalize else -1.0), beta=1.0)
        assert_close(N(y), O.subtract_mean(x, mean, normalize), "subtract mean")
    torch.cuda.synchronize()


def test_dropout_and_device_rng(dev):
    say("dropout / device rng")
    n = (1 << 18) + 77
    host = synth.uniform(31, 9, (n + 1000,))
    got = ops.rng_uniform01_device(31, 9, 1000, n, dev)
    assert np.array_equal(N(got), host[1000:]), "device generator == host generator, element by element"
    x, dy = synth.normal(14, 1, (n,)), synth.normal(14, 2, (n,))
    for ratio in (0.5, 0.1, 0.0, 1.0):
        y, mask = ops.dropout(T(x, dev), ratio, 1.0, got)
        y_ref, m_ref = O.dropout(x, ratio, 1.0, host[1000:])
        assert np.array_equal(N(mask), m_ref) and np.array_equal(N(y), y_ref)
        assert np.array_equal(N(ops.dropout_backprop(T(dy, dev), ratio, 1.0, mask)), O.dropout_backprop(dy, 1.0, m_ref))
    torch.cuda.synchronize()


@pytest.mark.parametrize("case", [((2, 7, 5, 6), 5), ((3, 96, 27, 27), 5), ((1, 3, 4, 4), 5), ((2, 10, 3, 3), 4), ((2, 4, 3, 3), 1)])
def test_lrn(dev, case):
    shape, size = case
    say("lrn", case)
    scale, power, min_div = 1e-4, 0.75, 2.0
    x = synth.normal(15, 1, shape) * np.float32(20.0)
    dy = synth.normal(15, 2, shape)
    y, d = ops.lrn_fwd(T(x, dev), size, scale, power, min_div)
    y_ref, d_ref = O.lrn_fwd(x, size, scale, power, min_div)
    assert_close(N(d), d_ref, "lrn denominators")
    assert_close(N(y), y_ref, "lrn fwd")
    dx = ops.lrn_bwd(T(x, dev), y, d, T(dy, dev), size, scale, power, min_div)
    assert_close(N(dx), O.lrn_bwd(x, dy, size, scale, power, min_div), "lrn bwd")
    torch.cuda.synchronize()


@pytest.mark.parametrize("shape", [(4, 3, 5, 6), (6, 5, 1, 1), (3, 2, 7, 7), (1, 4, 3, 3), (8, 64, 56, 56), (16, 512, 7, 7),
                                   (2, 3, 112, 112), (5, 7, 13, 9), (3, 8, 2, 2), (2, 4, 14, 14)])
def test_bnorm(dev, shape):
    """Spatial batch normalisation: training forward (batch statistics, moving averages, blend, fused ReLU),
    inference forward and backward against the fp64 restatement; one channel carries a mean 25x its deviation.
    (Two values per channel are left out: there dx cancels to ~epsilon analytically and has no stable digits.)"""
    say("bnorm", shape)
    C = shape[1]
    x = synth.normal(17, 1, shape) * np.float32(2.0) + np.linspace(-1, 50, C, dtype=np.float32)[None, :, None, None]
    dy = synth.normal(17, 2, shape)
    y0 = synth.normal(17, 3, shape)
    scale, bias = synth.normal(17, 4, (C,)) + np.float32(1.0), synth.normal(17, 5, (C,))
    rm, ri = synth.normal(17, 6, (C,)), np.abs(synth.normal(17, 7, (C,))) + np.float32(0.5)
    eps, ema = 1e-5, 0.1
    y_ref, cm_ref, ci_ref, rm_ref, ri_ref = O.bnorm_fwd_train(x, scale, bias, rm, ri, ema, eps)
    xd, sd, bd = T(x, dev), T(scale, dev), T(bias, dev)
    rmd, rid = T(rm, dev), T(ri, dev)
    y, cm, ci = ops.bnorm_fwd_train(xd, sd, bd, rmd, rid, ema, eps)
    assert_close(N(cm), cm_ref, "batch mean")
    assert_close(N(ci), ci_ref, "batch inverse deviation")
    assert_close(N(rmd), rm_ref, "running mean")
    assert_close(N(rid), ri_ref, "running inverse deviation")
    # normalised values of a channel with |mean| >> deviation lose |mean|/deviation ulps of x itself (fp32 inputs)
    assert_close(N(y), y_ref, "bnorm fwd", atol=2e-5)
    # blend into an existing tensor with the ReLU fused (the residual add of the stacked operators)
    yb = T(y0, dev)
    rm2, ri2 = T(rm, dev), T(ri, dev)
    ops.bnorm_fwd_train(xd, sd, bd, rm2, ri2, ema, eps, alpha=1.0, beta=1.0, y=yb, relu=True)
    want = O.bnorm_fwd_train(x, scale, bias, rm, ri, ema, eps, alpha=1.0, beta=1.0, y=y0)[0]
    got = N(yb)
    unsure = np.abs(want) < 1e-4 * max(1.0, float(np.sqrt((want ** 2).mean())))
    assert np.array_equal((got > 0)[~unsure], (want > 0)[~unsure])
    assert_close(got, np.maximum(want, 0), "bnorm fwd blend + relu", atol=2e-5)
    assert np.array_equal(N(rm2), N(rmd)) and np.array_equal(N(ri2), N(rid)), "statistics do not depend on the blend"
    yi = ops.bnorm_fwd_infer(xd, sd, bd, T(rm, dev), T(ri, dev), eps)
    assert_close(N(yi), O.bnorm_fwd_infer(x, scale, bias, rm, ri), "bnorm inference", atol=2e-5)
    # backward on the statistics the device cached; parameter gradients accumulate with beta_param = 1
    dx_ref, ds_ref, db_ref = O.bnorm_bwd(x, dy, scale, N(cm), N(ci))
    ds0, db0 = synth.normal(17, 8, (C,)), synth.normal(17, 9, (C,))
    dsd, dbd = T(ds0, dev), T(db0, dev)
    dx, _, _ = ops.bnorm_bwd(xd, T(dy, dev), sd, cm, ci, eps, dscale=dsd, dbias=dbd, beta_param=1.0)
    assert_close(N(dx), dx_ref, "bnorm bwd dx", atol=2e-5)
    assert_close(N(dsd), ds_ref.astype(np.float64) + ds0, "bnorm dscale", atol=2e-5)
    assert_close(N(dbd), db_ref.astype(np.float64) + db0, "bnorm dbias", atol=2e-5)
    dx2 = T(y0, dev)
    ops.bnorm_bwd(xd, T(dy, dev), sd, cm, ci, eps, alpha_data=1.0, beta_data=1.0, dx=dx2)
    assert_close(N(dx2), dx_ref.astype(np.float64) + y0, "bnorm bwd dx blended", atol=2e-5)
    # backward through the ReLU the forward pass fused: the mask is the device's own forward output, and must be that
    # exactly (an element the two passes disagree on would be off by a whole dy)
    yr, _, _ = ops.bnorm_fwd_train(xd, sd, bd, T(rm, dev), T(ri, dev), ema, eps, relu=True)
    dym = np.where(N(yr) > 0, dy, np.float32(0.0)).astype(np.float32)
    dxm_ref, dsm_ref, dbm_ref = O.bnorm_bwd(x, dym, scale, N(cm), N(ci))
    dxm, dsm, dbm = ops.bnorm_bwd(xd, T(dy, dev), sd, cm, ci, eps, relu_bias=bd)
    assert_close(N(dxm), dxm_ref, "bnorm bwd through fused relu: dx", atol=2e-5)
    assert_close(N(dsm), dsm_ref, "bnorm bwd through fused relu: dscale", atol=2e-5)
    assert_close(N(dbm), dbm_ref, "bnorm bwd through fused relu: dbias", atol=2e-5)
    same = ops.bnorm_bwd(xd, T(dym, dev), sd, cm, ci, eps)
    assert np.array_equal(N(dxm), N(same[0])) and np.array_equal(N(dsm), N(same[1])), "identical to masking dy beforehand"
    torch.cuda.synchronize()


@pytest.mark.parametrize("case", [(2, 3, 9, 3, 2, 0), (2, 3, 9, 3, 2, 1), (3, 4, 8, 2, 2, 0), (2, 5, 27, 3, 2, 0), (2, 2, 13, 3, 3, 1)])
@pytest.mark.parametrize("rounding", [_lib.RH_ROUND_FLOOR, _lib.RH_ROUND_CEIL])
def test_pool2d_bwd_with_folded_relu_mask(dev, case, rounding):
    """rh_pool2d_bwd_relu == max-pool backward followed by the ReLU backward mask of the pool's input
    (Pool2dOperator::backward then the producer's rect_backprop), on inputs with whole windows of zeros."""
    Nn, C, H, k, st, pad = case
    say("pool bwd + relu case", case, rounding)
    x = O.rect_inplace(synth.normal(16, 1, (Nn, C, H, H)) - np.float32(0.8))     # ~80 % zeros: some windows are all zero
    xd = T(x, dev)
    y, am = ops.pool2d_fwd(xd, k, st, pad, _lib.RH_POOL_MAX, rounding, want_argmax=True)
    assert (N(y) == 0).any() and (N(y) > 0).any()
    dy = synth.normal(16, 2, tuple(y.shape))
    want = O.pool2d_bwd(x, N(y), dy, k, st, pad, O.POOL_MAX, rounding)
    O.rect_backprop_inplace(x, want)
    got = N(ops.pool2d_bwd_relu(x.shape, y, T(dy, dev), k, st, pad, am, rounding))
    assert np.array_equal(got == 0, want == 0), "same elements are masked"
    assert_close(got, want, "pool bwd with folded relu mask")    # elements fed by several windows add in another order
    # and it is bit-identical to the two GPU kernels it replaces
    two = ops.pool2d_bwd(xd, y, T(dy, dev), k, st, pad, _lib.RH_POOL_MAX, rounding, argmax=am)
    ops.rect_backprop_inplace(xd, two)
    assert np.array_equal(got, N(two))
    torch.cuda.synchronize()


@pytest.mark.parametrize("case", [(2, 3, 9, 3, 2, 0), (2, 3, 9, 3, 2, 1), (3, 4, 8, 2, 2, 0), (2, 5, 27, 3, 2, 0), (2, 2, 13, 3, 3, 1)])
@pytest.mark.parametrize("rounding", [_lib.RH_ROUND_FLOOR, _lib.RH_ROUND_CEIL])
def test_avg_pool2d_bwd_with_folded_relu_mask(dev, case, rounding):
    """rh_pool2d_bwd_avg_relu == average-pool backward followed by the ReLU backward mask of the pool's input: against the
    oracle's two passes, and bit-identical to the two GPU kernels it replaces; max pooling is refused."""
    Nn, C, H, k, st, pad = case
    say("avg pool bwd + relu case", case, rounding)
    x = O.rect_inplace(synth.normal(18, 1, (Nn, C, H, H)) - np.float32(0.3))
    xd = T(x, dev)
    y = ops.pool2d_fwd(xd, k, st, pad, _lib.RH_POOL_AVG_INCL_PAD, rounding)
    dy = synth.normal(18, 2, tuple(y.shape))
    want = O.pool2d_bwd(x, N(y), dy, k, st, pad, O.POOL_AVG, rounding)
    O.rect_backprop_inplace(x, want)
    got = ops.pool2d_bwd_avg_relu(xd, T(dy, dev), k, st, pad, rounding)
    assert_close(N(got), want, "avg pool bwd with folded relu mask")
    two = ops.pool2d_bwd(xd, y, T(dy, dev), k, st, pad, _lib.RH_POOL_AVG_INCL_PAD, rounding)
    ops.rect_backprop_inplace(xd, two)
    assert torch.equal(got, two)
    import ctypes as C
    g = ops.pool_geom(x.shape, k, st, pad, _lib.RH_POOL_MAX, rounding)
    assert _lib.lib().rh_pool2d_bwd_avg_relu(C.byref(g), xd.data_ptr(), T(dy, dev).data_ptr(), got.data_ptr(), None) == _lib.RH_E_UNSUPPORTED
    torch.cuda.synchronize()


def test_context_memory_calls(dev):
    """rh_malloc (zero-filled), rh_host_malloc (page-locked, zero-filled), rh_load_sync / rh_store_sync round trip,
    rh_store_begin / rh_store_wait."""
    import ctypes as C
    lib = _lib.lib()
    ctx = C.c_void_p()
    _lib.check(lib.rh_ctx_create(0, C.byref(ctx)), "rh_ctx_create")
    n = 3 * 1000 + 1   # not a multiple of four bytes
    d, h, back = C.c_void_p(), C.c_void_p(), C.c_void_p()
    _lib.check(lib.rh_malloc(ctx, n, C.byref(d)), "rh_malloc")
    _lib.check(lib.rh_host_malloc(ctx, n, C.byref(h)), "rh_host_malloc")
    _lib.check(lib.rh_host_malloc(ctx, n, C.byref(back)), "rh_host_malloc")
    host = (C.c_uint8 * n).from_address(h.value)
    out = (C.c_uint8 * n).from_address(back.value)
    assert not any(host) and not any(out), "page-locked memory starts zeroed"
    _lib.check(lib.rh_store_sync(ctx, back, d, n), "rh_store_sync")
    assert not any(out), "device memory starts zeroed, odd tail included"
    pattern = synth.integers(21, 1, (n,), 256).astype(np.uint8)
    C.memmove(h, pattern.ctypes.data, n)
    _lib.check(lib.rh_load_sync(ctx, d, h, n), "rh_load_sync")
    _lib.check(lib.rh_store_sync(ctx, back, d, n), "rh_store_sync")
    assert np.array_equal(np.frombuffer(out, np.uint8), pattern)
    assert lib.rh_host_malloc(ctx, 16, None) == _lib.RH_E_INVALID and lib.rh_host_free(None, h) == _lib.RH_E_INVALID
    # the store in two halves: the copy is ordered behind what the context's stream holds when it is begun (a fill
    # kernel here), not behind what is enqueued afterwards (a second fill, which the copy must not see)
    nf = 1 << 20
    big, hb = C.c_void_p(), C.c_void_p()
    _lib.check(lib.rh_malloc(ctx, 4 * nf, C.byref(big)), "rh_malloc")
    _lib.check(lib.rh_host_malloc(ctx, 8, C.byref(hb)), "rh_host_malloc")
    stream = C.c_void_p(lib.rh_ctx_stream(ctx))
    assert lib.rh_store_wait(ctx) == 0, "nothing begun: returns at once"
    _lib.check(lib.rh_memset_f32(big, 3.5, nf, stream), "rh_memset_f32")
    _lib.check(lib.rh_store_begin(ctx, hb, C.c_void_p(big.value + 4 * (nf - 2)), 8), "rh_store_begin")
    _lib.check(lib.rh_store_wait(ctx), "rh_store_wait")
    assert list((C.c_float * 2).from_address(hb.value)) == [3.5, 3.5]
    _lib.check(lib.rh_ctx_sync(ctx), "rh_ctx_sync")
    assert lib.rh_store_begin(ctx, None, big, 8) == _lib.RH_E_INVALID and lib.rh_store_begin(None, hb, big, 8) == _lib.RH_E_INVALID
    assert lib.rh_store_begin(ctx, hb, big, 0) == 0 and lib.rh_store_wait(None) == _lib.RH_E_INVALID
    _lib.check(lib.rh_host_free(ctx, hb), "rh_host_free")
    _lib.check(lib.rh_free(ctx, big), "rh_free")
    for p_ in (h, back):
        _lib.check(lib.rh_host_free(ctx, p_), "rh_host_free")
    _lib.check(lib.rh_free(ctx, d), "rh_free")
    _lib.check(lib.rh_ctx_destroy(ctx), "rh_ctx_destroy")


def _check_conv_case_all_passes(dev, case, seed, idx):
    """All three passes, the forced scalar-offset backward-filter and the bf16-operand forward of one geometry."""
    Nn, C, H, W, K, R, st, pad = case
    x = synth.normal(seed, idx * 4 + 1, (Nn, C, H, W))
    w = synth.normal(seed, idx * 4 + 2, (K, C, R, R))
    b = synth.normal(seed, idx * 4 + 3, (K,))
    y_ref = O.conv2d_fwd(x, w, st, pad)
    dy = synth.normal(seed, idx * 4 + 4, y_ref.shape)
    xd, wd, bd, dyd = T(x, dev), T(w, dev), T(b, dev), T(dy, dev)
    tag = " %s" % (case,)
    y = ops.conv2d_fwd(xd, wd, st, pad, bias=bd, relu=True)
    assert_close(N(y), O.rect_inplace(O.add_bias_nchw(b, y_ref.copy())), "fwd" + tag)
    y16 = ops.conv2d_fwd(xd, wd, st, pad, algo=_lib.RH_MATH_BF16_MFMA_FP32ACC)
    assert_close(N(y16), O.conv2d_fwd(O.round_bf16(x), O.round_bf16(w), st, pad), "fwd bf16" + tag)
    dw_ref = O.conv2d_bwd_filter(x, dy, w.shape, st, pad)
    assert_close(N(ops.conv2d_bwd_filter(xd, dyd, w.shape, st, pad)), dw_ref, "bwd_filter" + tag)
    assert_close(N(ops.conv2d_bwd_filter(xd, dyd, w.shape, st, pad, algo=_lib.RH_ALGO_SCALAR_OFFSET)), dw_ref,
                 "bwd_filter scalar-offset" + tag)
    assert_close(N(ops.conv2d_bwd_data(wd, dyd, x.shape, st, pad)), O.conv2d_bwd_data(w, dy, x.shape, st, pad),
                 "bwd_data" + tag)


def test_conv2d_random_geometries(dev):
    """A seeded sweep over convolution geometries (filter 1-7, stride 1-4, any padding below the filter size, channel
    counts on both sides of every tile and group size): all three passes, the forced scalar-offset backward-filter and
    the bf16-operand forward against the oracle.  The hand-picked cases above name the paths; this guards the seams."""
    import random
    rnd = random.Random(20160417)
    done = 0
    while done < 60:
        R = rnd.choice([1, 1, 2, 3, 3, 3, 4, 5, 7])
        st = rnd.choice([1, 1, 1, 2, 2, 3, 4])
        pad = rnd.randint(0, max(0, R - 1))
        C = rnd.choice([1, 2, 3, 4, 7, 8, 12, 16, 24, 33, 40, 64, 72, 96])
        K = rnd.choice([1, 3, 5, 8, 16, 20, 32, 50, 64, 96, 100, 128, 130, 200, 256])
        H, W = rnd.randint(max(R - 2 * pad, 1), 24), rnd.randint(max(R - 2 * pad, 1), 24)
        Nn = rnd.choice([1, 2, 3, 5, 9, 17, 40])
        if Nn * C * H * W * K * R * R > 6e8:
            Nn = 2
        if (H + 2 * pad - R) // st + 1 < 1 or (W + 2 * pad - R) // st + 1 < 1:
            continue
        case = (Nn, C, H, W, K, R, st, pad)
        say("random conv case", done, case)
        _check_conv_case_all_passes(dev, case, 31, done)
        done += 1
    torch.cuda.synchronize()


def test_conv2d_random_midsize_geometries(dev):
    """A seeded sweep over layer-sized geometries (16-256 input and 32-512 output channels, planes of 7-56, batches up
    to 128, capped at 30 GFLOP a pass): grids of tens to over a thousand tiles, so contraction splits, sliced tails in
    one and in several rounds of tiles, the per-layer loader choice of backward-filter and the stride-2 class
    decomposition of backward-data are all met at sizes the hand-picked cases do not name."""
    import random
    rnd = random.Random(20160418)
    done = 0
    while done < 24:
        R = rnd.choice([1, 3, 3, 3, 5])
        st = rnd.choice([1, 1, 1, 2])
        pad = rnd.choice([0, R // 2, R // 2])
        C = rnd.choice([16, 24, 32, 48, 64, 96, 128, 160, 256])
        K = rnd.choice([32, 64, 96, 128, 192, 256, 384, 512])
        H = rnd.randint(7, 56)
        W = rnd.choice([H, H, rnd.randint(7, 56)])
        Nn = rnd.choice([8, 16, 24, 32, 52, 64, 100, 128])
        P, Q = (H + 2 * pad - R) // st + 1, (W + 2 * pad - R) // st + 1
        if P < 1 or Q < 1:
            continue
        while 2.0 * Nn * C * K * R * R * P * Q > 3e10 and Nn > 1:
            Nn //= 2
        case = (Nn, C, H, W, K, R, st, pad)
        say("random mid-size conv case", done, case, "forward tiles", -(-K // 128) * -(-(Nn * P * Q) // 128))
        _check_conv_case_all_passes(dev, case, 51, done)
        done += 1
    torch.cuda.synchronize()


def test_sgemm_and_pool_random_shapes(dev):
    """Seeded sweeps: SGEMM over transposes, odd extents, padded leading dimensions, alpha / beta pairs, with and
    without scratch; pooling over window, stride, padding, both modes and both roundings on rectangular planes."""
    import random
    rnd = random.Random(20160418)
    for it in range(40):
        tA, tB = rnd.randint(0, 1), rnd.randint(0, 1)
        m = rnd.choice([1, 2, 7, 10, 31, 64, 100, 128, 129, 300, 500, 1000, 4096])
        n = rnd.choice([1, 3, 16, 32, 64, 100, 128, 200, 256])
        k = rnd.choice([1, 2, 15, 16, 17, 64, 100, 256, 1000, 2450, 4096])
        if m * n * k > 3e8:
            k = 64
        use_ws = rnd.random() < 0.7
        a_shape = (m, k) if tA else (k, m)
        b_shape = (k, n) if tB else (n, k)
        lda, ldb, ldc = a_shape[1] + rnd.randint(0, 3), b_shape[1] + rnd.randint(0, 2), m + rnd.randint(0, 2)
        alpha, beta = rnd.choice([(1.0, 0.0), (0.5, 1.0), (1.0, 1.0), (-2.0, 0.25)])
        say("random sgemm", it, (tA, tB, m, n, k, lda, ldb, ldc, alpha, beta, use_ws))
        A = synth.normal(41, it * 3 + 1, (a_shape[0], lda))
        B = synth.normal(41, it * 3 + 2, (b_shape[0], ldb))
        C0 = synth.normal(41, it * 3 + 3, (n, ldc))
        ref = O.sgemm(tA, tB, m, n, k, alpha, A, lda, B, ldb, beta, C0.copy(), ldc)
        Cd = T(C0, dev)
        ops.sgemm(tA, tB, m, n, k, alpha, T(A, dev), lda, T(B, dev), ldb, beta, Cd, ldc, use_workspace=use_ws)
        assert_close(N(Cd), ref, "sgemm %d" % it)
    for it in range(40):
        k = rnd.choice([2, 2, 3, 3, 4, 5])
        st = rnd.choice([1, 2, 2, 3])
        pad = rnd.randint(0, k // 2)
        H, W = rnd.randint(k, 40), rnd.randint(k, 40)
        Nn, C = rnd.choice([1, 2, 5]), rnd.choice([1, 3, 8, 17])
        mode = rnd.choice([_lib.RH_POOL_MAX, _lib.RH_POOL_AVG_INCL_PAD])
        rounding = rnd.choice([_lib.RH_ROUND_FLOOR, _lib.RH_ROUND_CEIL])
        say("random pool", it, (Nn, C, H, W, k, st, pad, mode, rounding))
        x = np.round(synth.normal(42, it * 2 + 1, (Nn, C, H, W)) * 2) / 2
        y_ref, am_ref = O.pool2d_fwd(x, k, st, pad, mode, rounding, want_argmax=True)
        if y_ref.size == 0:
            continue
        xd = T(x, dev)
        y, am = ops.pool2d_fwd(xd, k, st, pad, mode, rounding, want_argmax=True)
        assert_close(N(y), y_ref, "pool fwd %d" % it)
        if mode == _lib.RH_POOL_MAX:
            assert np.array_equal(N(am), am_ref), "arg-max mask %d" % it
        dy = synth.normal(42, it * 2 + 2, y_ref.shape)
        dx_ref = O.pool2d_bwd(x, y_ref, dy, k, st, pad, mode, rounding)
        assert_close(N(ops.pool2d_bwd(xd, y, T(dy, dev), k, st, pad, mode, rounding)), dx_ref, "pool bwd %d" % it)
        if mode == _lib.RH_POOL_MAX:
            assert_close(N(ops.pool2d_bwd(xd, y, T(dy, dev), k, st, pad, mode, rounding, argmax=am)), dx_ref,
                         "pool bwd from the mask %d" % it)
    torch.cuda.synchronize()

