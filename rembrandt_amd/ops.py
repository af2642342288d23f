"""Thin wrappers that call the C ABI on torch device tensors.

torch provides device memory and the current HIP stream, nothing else: every function below
passes raw `data_ptr()` values and sizes to librembrandt_hip.so.  Errors raise (the reference
panics on every native error).
"""
import ctypes as C

import torch

from . import _lib
from ._lib import ConvGeom, PoolGeom, check, lib

_ws_cache = {}


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _p(t):
    if t is None:
        return C.c_void_p(0)
    assert t.is_cuda and t.is_contiguous(), "device-resident contiguous tensors only"
    return C.c_void_p(t.data_ptr())


def workspace(nbytes, device):
    """A cached, 256-byte aligned scratch tensor of at least nbytes on `device`."""
    key = str(device)
    ws = _ws_cache.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)
        assert ws.data_ptr() % 256 == 0
        _ws_cache[key] = ws
    return ws


def conv_geom(x_shape, w_shape, stride, pad):
    N, Cc, H, W = x_shape
    K, C2, R, S = w_shape
    assert Cc == C2
    return ConvGeom(N, Cc, H, W, K, R, S, stride, pad)


def conv_out_shape(g):
    out = lib().rh_conv2d_out_dim
    return (g.N, g.K, out(g.H, g.R, g.stride, g.pad), out(g.W, g.S, g.stride, g.pad))


def conv2d_fwd(x, w, stride, pad, bias=None, relu=False, alpha=1.0, beta=0.0, y=None, algo=0):
    g = conv_geom(x.shape, w.shape, stride, pad)
    if y is None:
        y = torch.empty(conv_out_shape(g), dtype=torch.float32, device=x.device)
    need = lib().rh_conv2d_workspace_bytes(C.byref(g), _lib.RH_CONV_FWD)
    ws = workspace(need, x.device)
    flags = (_lib.RH_FUSE_BIAS if bias is not None else 0) | (_lib.RH_FUSE_RELU if relu else 0) | algo
    check(lib().rh_conv2d_fwd(C.byref(g), alpha, _p(x), _p(w), beta, _p(y), _p(bias), _p(ws), ws.numel(), flags,
                              _stream()), "rh_conv2d_fwd")
    return y


def conv2d_bwd_filter(x, dy, w_shape, stride, pad, alpha=1.0, beta=0.0, dw=None, algo=0):
    g = conv_geom(x.shape, w_shape, stride, pad)
    if dw is None:
        dw = torch.zeros(tuple(w_shape), dtype=torch.float32, device=x.device)
    need = lib().rh_conv2d_workspace_bytes(C.byref(g), _lib.RH_CONV_BWD_FILTER)
    ws = workspace(need, x.device)
    check(lib().rh_conv2d_bwd_filter(C.byref(g), alpha, _p(x), _p(dy), beta, _p(dw), _p(ws), ws.numel(), algo,
                                     _stream()), "rh_conv2d_bwd_filter")
    return dw


def conv2d_bwd_filter_bias(x, dy, w_shape, stride, pad, alpha=1.0, beta=0.0, dw=None, db=None, algo=0):
    """Filter and bias gradient in one call (rh_conv2d_bwd_filter_bias)."""
    g = conv_geom(x.shape, w_shape, stride, pad)
    if dw is None:
        dw = torch.zeros(tuple(w_shape), dtype=torch.float32, device=x.device)
    if db is None:
        db = torch.zeros((w_shape[0],), dtype=torch.float32, device=x.device)
    need = lib().rh_conv2d_workspace_bytes(C.byref(g), _lib.RH_CONV_BWD_FILTER)
    ws = workspace(need, x.device)
    check(lib().rh_conv2d_bwd_filter_bias(C.byref(g), alpha, _p(x), _p(dy), beta, _p(dw), _p(db), _p(ws), ws.numel(), algo,
                                          _stream()), "rh_conv2d_bwd_filter_bias")
    return dw, db


def conv2d_bwd_bias(dy, alpha=1.0, beta=0.0, db=None, two_stage=False):
    N, K = dy.shape[0], dy.shape[1]
    plane = dy.numel() // (N * K)
    if db is None:
        db = torch.zeros((K,), dtype=torch.float32, device=dy.device)
    if two_stage:
        ws = workspace(lib().rh_conv2d_bwd_bias_workspace_bytes(N, K, plane), dy.device)
        check(lib().rh_conv2d_bwd_bias_ws(N, K, plane, alpha, _p(dy), beta, _p(db), _p(ws), ws.numel(), _stream()),
              "rh_conv2d_bwd_bias_ws")
    else:
        check(lib().rh_conv2d_bwd_bias(N, K, plane, alpha, _p(dy), beta, _p(db), _stream()), "rh_conv2d_bwd_bias")
    return db


def conv2d_bwd_data(w, dy, x_shape, stride, pad, alpha=1.0, beta=0.0, dx=None, algo=0, relu_of=None):
    """relu_of: this convolution's input (a ReLU's output); its backward mask is applied to dx as it is written
    (rh_conv2d_bwd_data_relu)."""
    g = conv_geom(x_shape, w.shape, stride, pad)
    if dx is None:
        dx = torch.zeros(tuple(x_shape), dtype=torch.float32, device=w.device)
    need = lib().rh_conv2d_workspace_bytes(C.byref(g), _lib.RH_CONV_BWD_DATA)
    ws = workspace(need, w.device)
    if relu_of is not None:
        check(lib().rh_conv2d_bwd_data_relu(C.byref(g), alpha, _p(w), _p(dy), beta, _p(dx), _p(relu_of), _p(ws), ws.numel(),
                                            algo, _stream()), "rh_conv2d_bwd_data_relu")
        return dx
    check(lib().rh_conv2d_bwd_data(C.byref(g), alpha, _p(w), _p(dy), beta, _p(dx), _p(ws), ws.numel(), algo,
                                   _stream()), "rh_conv2d_bwd_data")
    return dx


def conv2d_winograd_flops(x_shape, w_shape, stride, pad, which="fwd", algo=0):
    """FLOPs the pass executes when the library takes the Winograd form for this geometry, 0 for a direct form."""
    N, Cc, H, W = x_shape
    g = _lib.ConvGeom(N, Cc, H, W, w_shape[0], w_shape[2], w_shape[3], stride, pad)
    return float(lib().rh_conv2d_winograd_flops(C.byref(g), {"fwd": 0, "bwd_filter": 1, "bwd_data": 2}[which], algo))


def conv2d_bwd_data_relu_supported(x_shape, w_shape, stride, pad):
    g = conv_geom(x_shape, w_shape, stride, pad)
    return bool(lib().rh_conv2d_bwd_data_relu_supported(C.byref(g)))


def add_bias_nchw(bias, y, alpha=1.0, beta=1.0):
    N, K = y.shape[0], y.shape[1]
    plane = y.numel() // (N * K)
    check(lib().rh_add_bias_nchw(_p(bias), _p(y), plane, K, N, alpha, beta, _stream()), "rh_add_bias_nchw")
    return y


def _check_last(where):
    check(lib().rh_last_error(), where)


def rect_inplace(y):
    lib().rembrandt_kernel_batch_map_rect_inplace(_p(y), y.numel() // y.shape[0], y.shape[0], _stream())
    _check_last("rembrandt_kernel_batch_map_rect_inplace")
    return y


def rect_backprop_inplace(y, dy):
    lib().rembrandt_kernel_batch_map_rect_backprop_inplace(_p(y), y.numel() // y.shape[0], y.shape[0], _p(dy),
                                                           _stream())
    _check_last("rembrandt_kernel_batch_map_rect_backprop_inplace")
    return dy


def sgemm(transA, transB, m, n, k, alpha, A, lda, B, ldb, beta, Cm, ldc, use_workspace=True, bias=None, relu=False):
    """C = alpha op(A) op(B) + beta C; with `bias` (length m) and / or `relu` through rh_sgemm_bias_act."""
    ws, nbytes = None, 0
    if use_workspace:
        nbytes = lib().rh_sgemm_workspace_bytes(m, n, k)
        if nbytes:
            ws = workspace(nbytes, Cm.device)
            nbytes = ws.numel()
    if bias is None and not relu:
        check(lib().rh_sgemm(int(transA), int(transB), m, n, k, alpha, _p(A), lda, _p(B), ldb, beta, _p(Cm), ldc,
                             _p(ws), nbytes, 0, _stream()), "rh_sgemm")
        return Cm
    flags = (_lib.RH_FUSE_BIAS if bias is not None else 0) | (_lib.RH_FUSE_RELU if relu else 0)
    check(lib().rh_sgemm_bias_act(int(transA), int(transB), m, n, k, alpha, _p(A), lda, _p(B), ldb, beta, _p(Cm), ldc,
                                  _p(bias), _p(ws), nbytes, flags, _stream()), "rh_sgemm_bias_act")
    return Cm


def saxpy(alpha, x, y):
    check(lib().rh_saxpy(x.numel(), alpha, _p(x), _p(y), _stream()), "rh_saxpy")
    return y


def sscal(alpha, x):
    check(lib().rh_sscal(x.numel(), alpha, _p(x), _stream()), "rh_sscal")
    return x


def pool_geom(x_shape, size, stride, pad, mode, rounding=_lib.RH_ROUND_FLOOR):
    N, Cc, H, W = x_shape
    return PoolGeom(N, Cc, H, W, size, stride, pad, mode, rounding)


def pool_out_shape(g):
    out = lib().rh_pool2d_out_dim
    return (g.N, g.C, out(g.H, g.size, g.stride, g.pad, g.round), out(g.W, g.size, g.stride, g.pad, g.round))


def pool2d_fwd(x, size, stride, pad, mode, rounding=_lib.RH_ROUND_FLOOR, want_argmax=False):
    g = pool_geom(x.shape, size, stride, pad, mode, rounding)
    y = torch.empty(pool_out_shape(g), dtype=torch.float32, device=x.device)
    am = torch.empty(y.shape, dtype=torch.int32, device=x.device) if want_argmax else None
    check(lib().rh_pool2d_fwd(C.byref(g), _p(x), _p(y), _p(am), _stream()), "rh_pool2d_fwd")
    return (y, am) if want_argmax else y


def pool2d_slot_supported(x_shape, size, stride, pad, rounding=_lib.RH_ROUND_FLOOR):
    g = pool_geom(x_shape, size, stride, pad, _lib.RH_POOL_MAX, rounding)
    return bool(lib().rh_pool2d_slot_supported(C.byref(g)))


def pool2d_fwd_slot(x, size, stride, pad, rounding=_lib.RH_ROUND_FLOOR):
    """Max pooling with the one-byte mask: returns (y, slot) with slot = r*size + s of each window's winner (255: none)."""
    g = pool_geom(x.shape, size, stride, pad, _lib.RH_POOL_MAX, rounding)
    y = torch.empty(pool_out_shape(g), dtype=torch.float32, device=x.device)
    slot = torch.empty(y.shape, dtype=torch.uint8, device=x.device)
    check(lib().rh_pool2d_fwd_slot(C.byref(g), _p(x), _p(y), _p(slot), _stream()), "rh_pool2d_fwd_slot")
    return y, slot


def pool2d_bwd_slot(x_shape, dy, slot, size, stride, pad, rounding=_lib.RH_ROUND_FLOOR, relu_y=None):
    g = pool_geom(x_shape, size, stride, pad, _lib.RH_POOL_MAX, rounding)
    dx = torch.empty(tuple(x_shape), dtype=torch.float32, device=dy.device)
    check(lib().rh_pool2d_bwd_slot(C.byref(g), _p(relu_y), _p(dy), _p(dx), _p(slot), _stream()), "rh_pool2d_bwd_slot")
    return dx


def bf16_pack(x, halo):
    """fp32 NCHW -> packed bf16 activation tensor [n][H + 2 halo][C/8][W + 2 halo][8] (a uint8 tensor; zero border)."""
    Nn, Cc, H, W = x.shape
    nbytes = lib().rh_bf16_act_bytes(Nn, Cc, H, W, halo)
    assert nbytes > 0, "no packed form for this shape"
    xp = torch.zeros(nbytes, dtype=torch.uint8, device=x.device)
    check(lib().rh_bf16_pack_nchw(Nn, Cc, H, W, halo, _p(x), _p(xp), _stream()), "rh_bf16_pack_nchw")
    return xp


def bf16_unpack(xp, shape, halo):
    Nn, Cc, H, W = shape
    x = torch.empty(tuple(shape), dtype=torch.float32, device=xp.device)
    check(lib().rh_bf16_unpack_nchw(Nn, Cc, H, W, halo, _p(xp), _p(x), _stream()), "rh_bf16_unpack_nchw")
    return x


def conv2d_fwd_bf16_packed(x, w, stride, pad, bias=None, relu=False, x_packed=None, out_halo=None, algo=0):
    """The bf16 forward on a converted filter.  Input: `x_packed` (from bf16_pack(x, pad) or a producer) or the fp32 `x`
    (x.shape is used for the geometry either way).  out_halo None: fp32 NCHW result; an int: packed bf16 result with
    that border.  Returns the result tensor."""
    g = conv_geom(x.shape, w.shape, stride, pad)
    fb = lib().rh_conv2d_fwd_bf16_filter_bytes(C.byref(g))
    assert fb > 0, "no packed form for this geometry"
    wprep = torch.empty(fb, dtype=torch.uint8, device=w.device)
    check(lib().rh_conv2d_fwd_bf16_prep_filter(C.byref(g), _p(w), _p(wprep), fb, _stream()), "rh_conv2d_fwd_bf16_prep_filter")
    ws = workspace(lib().rh_conv2d_fwd_bf16_workspace_bytes(C.byref(g)), w.device)
    shape = conv_out_shape(g)
    y = yp = None
    if out_halo is None:
        y = torch.empty(shape, dtype=torch.float32, device=w.device)
    else:
        nbytes = lib().rh_bf16_act_bytes(shape[0], shape[1], shape[2], shape[3], out_halo)
        assert nbytes > 0
        yp = torch.zeros(nbytes, dtype=torch.uint8, device=w.device)
    flags = (_lib.RH_FUSE_BIAS if bias is not None else 0) | (_lib.RH_FUSE_RELU if relu else 0) | algo
    check(lib().rh_conv2d_fwd_bf16_packed(C.byref(g), _p(x_packed), _p(None if x_packed is not None else x), _p(wprep), _p(bias),
                                          _p(y), _p(yp), 0 if out_halo is None else out_halo, _p(ws), ws.numel(), flags,
                                          _stream()), "rh_conv2d_fwd_bf16_packed")
    return y if out_halo is None else yp


def pool2d_fwd_bf16_packed(xp, x_shape, size, stride, pad, rounding=_lib.RH_ROUND_FLOOR, out_halo=0):
    """Max pooling of a packed bf16 activation tensor (border 0) into a packed one with border out_halo."""
    g = pool_geom(x_shape, size, stride, pad, _lib.RH_POOL_MAX, rounding)
    shape = pool_out_shape(g)
    nbytes = lib().rh_bf16_act_bytes(shape[0], shape[1], shape[2], shape[3], out_halo)
    assert nbytes > 0
    yp = torch.zeros(nbytes, dtype=torch.uint8, device=xp.device)
    check(lib().rh_pool2d_fwd_bf16_packed(C.byref(g), _p(xp), _p(yp), out_halo, _stream()), "rh_pool2d_fwd_bf16_packed")
    return yp, shape


def pool2d_bwd(x, y, dy, size, stride, pad, mode, rounding=_lib.RH_ROUND_FLOOR, argmax=None):
    g = pool_geom(x.shape, size, stride, pad, mode, rounding)
    dx = torch.empty(tuple(x.shape), dtype=torch.float32, device=x.device)
    check(lib().rh_pool2d_bwd(C.byref(g), _p(x), _p(y), _p(dy), _p(dx), _p(argmax), _stream()), "rh_pool2d_bwd")
    return dx


def pool2d_bwd_relu(x_shape, y, dy, size, stride, pad, argmax, rounding=_lib.RH_ROUND_FLOOR):
    """Max-pool backward with the producer's ReLU backward mask folded in."""
    g = pool_geom(x_shape, size, stride, pad, _lib.RH_POOL_MAX, rounding)
    dx = torch.empty(tuple(x_shape), dtype=torch.float32, device=dy.device)
    check(lib().rh_pool2d_bwd_relu(C.byref(g), _p(y), _p(dy), _p(dx), _p(argmax), _stream()), "rh_pool2d_bwd_relu")
    return dx


def pool2d_bwd_avg_relu(x, dy, size, stride, pad, rounding=_lib.RH_ROUND_FLOOR):
    """Average-pool backward with the backward of the ReLU that produced the pool's input x folded in."""
    g = pool_geom(x.shape, size, stride, pad, _lib.RH_POOL_AVG_INCL_PAD, rounding)
    dx = torch.empty(tuple(x.shape), dtype=torch.float32, device=dy.device)
    check(lib().rh_pool2d_bwd_avg_relu(C.byref(g), _p(x), _p(dy), _p(dx), _stream()), "rh_pool2d_bwd_avg_relu")
    return dx


def softmax_fwd(x):
    N, Cc = x.shape
    p = torch.empty_like(x)
    check(lib().rh_softmax_fwd(_p(x), _p(p), Cc, N, _stream()), "rh_softmax_fwd")
    return p


def softmax_kl_backward(p, labels, weights):
    N, Cc = p.shape
    dx = torch.empty_like(p)
    lib().rembrandt_kernel_batch_map_softmax_kl_backward(_p(p), Cc, N, _p(labels), _p(weights), _p(dx), _stream())
    _check_last("rembrandt_kernel_batch_map_softmax_kl_backward")
    return dx


def softmax_kl_loss1(p, labels, weights, beta=0.0, loss1=None):
    N, Cc = p.shape
    if loss1 is None:
        loss1 = torch.zeros((N,), dtype=torch.float32, device=p.device)
    lib().rembrandt_kernel_batch_map_softmax_kl_loss1(_p(p), Cc, N, _p(labels), _p(weights), beta, _p(loss1),
                                                      _stream())
    _check_last("rembrandt_kernel_batch_map_softmax_kl_loss1")
    return loss1


def blockreduce_sum(src, beta=0.0, dst=None):
    batch, length = src.shape
    if dst is None:
        dst = torch.zeros((batch,), dtype=torch.float32, device=src.device)
    lib().rembrandt_kernel_batch_blockreduce_sum(_p(src), length, batch, _p(dst), beta, _stream())
    _check_last("rembrandt_kernel_batch_blockreduce_sum")
    return dst


def blockreduce_argmax(src):
    batch, length = src.shape
    mx = torch.empty((batch,), dtype=torch.float32, device=src.device)
    idx = torch.empty((batch,), dtype=torch.int32, device=src.device)
    lib().rembrandt_kernel_batch_blockreduce_argmax(_p(src), length, batch, _p(mx), _p(idx), _stream())
    _check_last("rembrandt_kernel_batch_blockreduce_argmax")
    return mx, idx


def softmax_kl_step(x, labels, weights, counter=None):
    """softmax, row arg-max, per-sample loss, its sum and the KL backward in one launch (rh_softmax_kl_step).
    Returns (p, row max, arg-max, loss1, loss sum, dx, counter)."""
    N, Cc = x.shape
    p, dx = torch.empty_like(x), torch.empty_like(x)
    mx = torch.empty((N,), dtype=torch.float32, device=x.device)
    idx = torch.empty((N,), dtype=torch.int32, device=x.device)
    loss1 = torch.empty((N,), dtype=torch.float32, device=x.device)
    total = torch.empty((1,), dtype=torch.float32, device=x.device)
    if counter is None:
        counter = torch.zeros((1,), dtype=torch.int32, device=x.device)
    check(lib().rh_softmax_kl_step(_p(x), Cc, N, _p(labels), _p(weights), _p(p), _p(mx), _p(idx), _p(loss1), _p(total),
                                   _p(dx), _p(counter), _stream()), "rh_softmax_kl_step")
    return p, mx, idx, loss1, total, dx, counter


def affine2_softmax_kl_step_supported(B, I, H, Cc):
    return bool(lib().rh_affine2_softmax_kl_step_supported(B, I, H, Cc))


def affine2_softmax_kl_step(x, w1, b1, w2, b2, labels, weights, relu1=True, want_dx=True, counter=None):
    """Two affine layers, the loss step and their data gradients in one launch (rh_affine2_softmax_kl_step).
    x: (B, I); w1: (H, I); w2: (C, H).  Returns a dict of every tensor the launch writes."""
    B, I = x.shape
    H, Cc = w1.shape[0], w2.shape[0]
    f = lambda *shape: torch.empty(shape, dtype=torch.float32, device=x.device)
    out = {"h": f(B, H), "logits": f(B, Cc), "p": f(B, Cc), "max": f(B), "idx": torch.empty((B,), dtype=torch.int32, device=x.device),
           "loss1": f(B), "loss": f(1), "dlogits": f(B, Cc), "dh": f(B, H), "dx": f(B, I) if want_dx else None}
    if counter is None:
        counter = torch.zeros((1,), dtype=torch.int32, device=x.device)
    out["counter"] = counter
    check(lib().rh_affine2_softmax_kl_step(B, I, H, Cc, int(relu1), _p(x), _p(w1), _p(b1), _p(w2), _p(b2), _p(labels),
                                           _p(weights), _p(out["h"]), _p(out["logits"]), _p(out["p"]), _p(out["max"]),
                                           _p(out["idx"]), _p(out["loss1"]), _p(out["loss"]), _p(out["dlogits"]), _p(out["dh"]),
                                           _p(out["dx"]) if want_dx else None, _p(counter), _stream()),
          "rh_affine2_softmax_kl_step")
    return out


def affine_softmax_kl_step_from_h(h, w2, b2, labels, weights, relu1=True, counter=None):
    """The same launch started from the first layer's output h (B, H) (I = 0, x = NULL): logits .. dh."""
    B, H = h.shape
    Cc = w2.shape[0]
    f = lambda *shape: torch.empty(shape, dtype=torch.float32, device=h.device)
    out = {"h": h, "logits": f(B, Cc), "p": f(B, Cc), "max": f(B), "idx": torch.empty((B,), dtype=torch.int32, device=h.device),
           "loss1": f(B), "loss": f(1), "dlogits": f(B, Cc), "dh": f(B, H)}
    if counter is None:
        counter = torch.zeros((1,), dtype=torch.int32, device=h.device)
    out["counter"] = counter
    check(lib().rh_affine2_softmax_kl_step(B, 0, H, Cc, int(relu1), None, None, None, _p(w2), _p(b2), _p(labels),
                                           _p(weights), _p(h), _p(out["logits"]), _p(out["p"]), _p(out["max"]),
                                           _p(out["idx"]), _p(out["loss1"]), _p(out["loss"]), _p(out["dlogits"]), _p(out["dh"]),
                                           None, _p(counter), _stream()),
          "rh_affine2_softmax_kl_step")
    return out


def affine_bwd_params_from_h(h, dlogits, dw2, db2, beta2=0.0, dh=None, db1=None, beta1=0.0):
    """dW2 and db2 (rh_affine2_bwd_params with I = 0, x = NULL) and, with dh and db1, db1 = sum_n dh + beta1 * db1."""
    B, H = h.shape
    check(lib().rh_affine2_bwd_params(B, 0, H, dlogits.shape[1], None, _p(h), _p(dh) if dh is not None else None, _p(dlogits),
                                      beta1, None, _p(db1) if db1 is not None else None, beta2, _p(dw2), _p(db2), _stream()),
          "rh_affine2_bwd_params")


def affine2_bwd_params(x, h, dh, dlogits, dw1, db1, dw2, db2, beta1=0.0, beta2=0.0):
    """dW1, db1, dW2, db2 of the two layers in one launch (rh_affine2_bwd_params); out = sum + beta * out."""
    B, I = x.shape
    H, Cc = h.shape[1], dlogits.shape[1]
    check(lib().rh_affine2_bwd_params(B, I, H, Cc, _p(x), _p(h), _p(dh), _p(dlogits), beta1, _p(dw1), _p(db1), beta2, _p(dw2),
                                      _p(db2), _stream()), "rh_affine2_bwd_params")


def sgd_momentum_step(W, g, v, l2, scale, mu, apply, zero_grad=True):
    check(lib().rh_sgd_momentum_step(W.numel(), _p(W), _p(g), _p(v), l2, scale, mu, apply, int(zero_grad),
                                     _stream()), "rh_sgd_momentum_step")


def sgd_momentum_step_multi(tensors, scale, mu, apply, zero_grad=True, keep_grad=()):
    """tensors: sequence of (W, g, v, l2) device tensors; one launch for all of them.  keep_grad: indices of the
    tensors whose gradient the step must leave as it is."""
    arr = (_lib.SgdTensor * len(tensors))()
    for i, (W, g, v, l2) in enumerate(tensors):
        arr[i] = _lib.SgdTensor(W.data_ptr(), g.data_ptr(), v.data_ptr(), W.numel(), l2, 1 if i in keep_grad else 0)
    check(lib().rh_sgd_momentum_step_multi(len(tensors), arr, scale, mu, apply, int(zero_grad), _stream()),
          "rh_sgd_momentum_step_multi")


def descend(W, g, s, l2):
    check(lib().rh_descend(W.numel(), _p(W), _p(g), s, l2, _stream()), "rh_descend")


def cast_u8_f32(x, scale):
    y = torch.empty(x.shape, dtype=torch.float32, device=x.device)
    check(lib().rh_cast_u8_f32(_p(x), _p(y), x.numel(), scale, _stream()), "rh_cast_u8_f32")
    return y


def crop_nchw(x, crop_w, crop_h, off_w, off_h):
    N, Cc, H, W = x.shape
    y = torch.empty((N, Cc, crop_h, crop_w), dtype=torch.float32, device=x.device)
    check(lib().rh_crop_nchw(_p(x), _p(y), N * Cc, W, H, crop_w, crop_h, off_w, off_h, _stream()), "rh_crop_nchw")
    return y


def flip_x(x):
    y = torch.empty_like(x)
    lib().rembrandt_kernel_batch_blockmap256_flip(_p(x), x.shape[-1], x.numel() // x.shape[-1], _p(y), _stream())
    _check_last("rembrandt_kernel_batch_blockmap256_flip")
    return y


def pca3_noise(x, alphas, svals, svecs):
    N, Cc, H, W = x.shape
    assert Cc == 3
    y = torch.empty_like(x)
    lib().rembrandt_kernel_batch_map_preproc_pca3_noise(_p(x), H * W, N, _p(alphas), _p(svals), _p(svecs), _p(y), _stream())
    _check_last("rembrandt_kernel_batch_map_preproc_pca3_noise")
    return y


def dropout(x, ratio, scale, rnd):
    y = torch.empty_like(x)
    mask = torch.empty(x.shape, dtype=torch.int32, device=x.device)
    lib().rembrandt_kernel_map_dropout(_p(x), x.numel(), ratio, scale, _p(rnd), _p(y), _p(mask), _stream())
    _check_last("rembrandt_kernel_map_dropout")
    return y, mask


def dropout_backprop(dy, ratio, scale, mask):
    dx = torch.empty_like(dy)
    lib().rembrandt_kernel_map_dropout_backprop(_p(dy), dy.numel(), ratio, scale, _p(mask), _p(dx), _stream())
    _check_last("rembrandt_kernel_map_dropout_backprop")
    return dx


def rng_uniform01_device(seed, stream_id, first, n, device):
    t = torch.empty((n,), dtype=torch.float32, device=device)
    check(lib().rh_rng_fill_uniform01_device(seed, stream_id, first, _p(t), n, _stream()), "rh_rng_fill_uniform01_device")
    return t


def lrn_geom(x_shape, size, scale, power, min_div):
    N, Cc, H, W = x_shape
    return _lib.LrnGeom(N, Cc, H, W, size, scale, power, min_div)


def lrn_fwd(x, size, scale, power, min_div):
    g = lrn_geom(x.shape, size, scale, power, min_div)
    y, d = torch.empty_like(x), torch.empty_like(x)
    check(lib().rh_lrn_fwd(C.byref(g), _p(x), _p(y), _p(d), _stream()), "rh_lrn_fwd")
    return y, d


def lrn_bwd(x, y, d, dy, size, scale, power, min_div):
    g = lrn_geom(x.shape, size, scale, power, min_div)
    dx = torch.empty_like(x)
    check(lib().rh_lrn_bwd(C.byref(g), _p(x), _p(y), _p(d), _p(dy), _p(dx), _stream()), "rh_lrn_bwd")
    return dx


def _bnorm_ws(x):
    N, Cc, H, W = x.shape
    nbytes = lib().rh_bnorm_workspace_bytes(N, Cc, H * W)
    return torch.empty(nbytes, dtype=torch.uint8, device=x.device), nbytes


def bnorm_fwd_train(x, scale, bias, running_mean, running_ivar, ema_factor, epsilon, alpha=1.0, beta=0.0, y=None, relu=False):
    """Spatial batch-norm, training mode: returns (y, cached_mean, cached_ivar); the running pair is updated in place."""
    N, Cc, H, W = x.shape
    if y is None:
        assert beta == 0.0
        y = torch.empty_like(x)
    cm, ci = torch.empty_like(scale), torch.empty_like(scale)
    ws, nbytes = _bnorm_ws(x)
    check(lib().rh_bnorm_fwd_train(N, Cc, H * W, alpha, _p(x), beta, _p(y), ema_factor, epsilon, _p(scale), _p(bias),
                                   _p(running_mean), _p(running_ivar), _p(cm), _p(ci), _p(ws), nbytes,
                                   _lib.RH_FUSE_RELU if relu else 0, _stream()), "rh_bnorm_fwd_train")
    return y, cm, ci


def bnorm_fwd_infer(x, scale, bias, running_mean, running_ivar, epsilon, alpha=1.0, beta=0.0, y=None, relu=False):
    N, Cc, H, W = x.shape
    if y is None:
        assert beta == 0.0
        y = torch.empty_like(x)
    ws, nbytes = _bnorm_ws(x)
    check(lib().rh_bnorm_fwd_infer(N, Cc, H * W, alpha, _p(x), beta, _p(y), epsilon, _p(scale), _p(bias), _p(running_mean),
                                   _p(running_ivar), _p(ws), nbytes, _lib.RH_FUSE_RELU if relu else 0, _stream()),
          "rh_bnorm_fwd_infer")
    return y


def bnorm_bwd(x, dy, scale, cached_mean, cached_ivar, epsilon, dscale=None, dbias=None, alpha_data=1.0, beta_data=0.0,
              dx=None, alpha_param=1.0, beta_param=0.0, relu_bias=None):
    """Returns (dx, dscale, dbias); with beta_param = 1 the parameter gradients accumulate as in the reference.
    `relu_bias` (the layer's bias): dy is first masked by the ReLU that the forward pass fused (rh_bnorm_bwd_relu)."""
    N, Cc, H, W = x.shape
    if dx is None:
        assert beta_data == 0.0
        dx = torch.empty_like(x)
    if dscale is None:
        assert beta_param == 0.0
        dscale, dbias = torch.empty_like(scale), torch.empty_like(scale)
    ws, nbytes = _bnorm_ws(x)
    if relu_bias is not None:
        check(lib().rh_bnorm_bwd_relu(N, Cc, H * W, alpha_data, beta_data, _p(x), _p(dy), _p(dx), alpha_param, beta_param,
                                      epsilon, _p(scale), _p(relu_bias), _p(dscale), _p(dbias), _p(cached_mean),
                                      _p(cached_ivar), _p(ws), nbytes, _stream()), "rh_bnorm_bwd_relu")
        return dx, dscale, dbias
    check(lib().rh_bnorm_bwd(N, Cc, H * W, alpha_data, beta_data, _p(x), _p(dy), _p(dx), alpha_param, beta_param, epsilon,
                             _p(scale), _p(dscale), _p(dbias), _p(cached_mean), _p(cached_ivar), _p(ws), nbytes, _stream()),
          "rh_bnorm_bwd")
    return dx, dscale, dbias


def memset_f32(t, value):
    check(lib().rh_memset_f32(_p(t), value, t.numel(), _stream()), "rh_memset_f32")
    return t
