"""numpy front end of the CPU oracle (``oracle.c``).

TEST INFRASTRUCTURE ONLY: imported by the tests, by the smoke check and by the benchmark's CPU
baseline leg; the shipped package never imports it.  All arrays are C-contiguous numpy arrays
in the layouts of the reference (NCHW activations, [K][C][R][S] filters, [out][in] affine
weights, [batch][chan] affine activations).

The numpy restatements further down (Data3d preprocessing, dropout, local response normalisation, spatial batch
normalisation) are pinned by the CPU test-suite against torch CPU fp64 routines and their autograd.  Parity unpinned
against the reference itself, whose kernels for these live outside its tree: the dropout comparison (`>` taken,
not `>=`), the LRN arithmetic (the reference's layer is a stub; the published formula its parameters name), and what
the batch-norm buffer `bn_running_ivar` accumulates (taken: the moving average of 1/sqrt(var + epsilon)).
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

POOL_MAX, POOL_AVG = 0, 1
ROUND_FLOOR, ROUND_CEIL = 0, 1


class ConvGeom(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("N", "C", "H", "W", "K", "R", "S", "stride", "pad")]


class PoolGeom(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("N", "C", "H", "W", "size", "stride", "pad", "mode", "round")]


def build(force=False):
    """Compile oracle.c into liboracle.so (gcc, OpenMP)."""
    if force or not os.path.exists(_LIB_PATH) or (
            os.path.getmtime(_LIB_PATH) < os.path.getmtime(os.path.join(_HERE, "oracle.c"))):
        subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"])
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.orc_out_dim_floor.restype = C.c_int32
        _lib.orc_out_dim_ceil.restype = C.c_int32
        _lib.orc_accuracy_count.restype = C.c_int32
        _lib.orc_num_threads.restype = C.c_int
    return _lib


def num_threads():
    return int(lib().orc_num_threads())


def _f(a):
    assert a.dtype == np.float32 and a.flags.c_contiguous
    return a.ctypes.data_as(C.POINTER(C.c_float))


def _i32(a):
    assert a.dtype == np.int32 and a.flags.c_contiguous
    return a.ctypes.data_as(C.POINTER(C.c_int32))


def _i64(a):
    assert a.dtype == np.int64 and a.flags.c_contiguous
    return a.ctypes.data_as(C.POINTER(C.c_int64))


def out_dim(n, size, stride, pad, rounding=ROUND_FLOOR):
    fn = lib().orc_out_dim_ceil if rounding == ROUND_CEIL else lib().orc_out_dim_floor
    return int(fn(C.c_int32(n), C.c_int32(size), C.c_int32(stride), C.c_int32(pad)))


def conv_geom(x_shape, w_shape, stride, pad):
    N, Cc, H, W = x_shape
    K, C2, R, S = w_shape
    assert Cc == C2
    return ConvGeom(N, Cc, H, W, K, R, S, stride, pad)


def conv_out_shape(g):
    return (g.N, g.K, out_dim(g.H, g.R, g.stride, g.pad), out_dim(g.W, g.S, g.stride, g.pad))


# ---- convolution ---------------------------------------------------------------------------
def conv2d_fwd(x, w, stride, pad, alpha=1.0, beta=0.0, y=None):
    g = conv_geom(x.shape, w.shape, stride, pad)
    if y is None:
        y = np.zeros(conv_out_shape(g), np.float32)
    lib().orc_conv2d_fwd(C.byref(g), C.c_float(alpha), _f(x), _f(w), C.c_float(beta), _f(y))
    return y


def conv2d_fwd_at(x, w, stride, pad, idx):
    g = conv_geom(x.shape, w.shape, stride, pad)
    idx = np.ascontiguousarray(idx, np.int64)
    out = np.zeros(idx.shape, np.float32)
    lib().orc_conv2d_fwd_at(C.byref(g), _f(x), _f(w), _i64(idx), C.c_int64(idx.size), _f(out))
    return out


def conv2d_bwd_filter(x, dy, w_shape, stride, pad, alpha=1.0, beta=0.0, dw=None):
    g = conv_geom(x.shape, w_shape, stride, pad)
    if dw is None:
        dw = np.zeros(w_shape, np.float32)
    lib().orc_conv2d_bwd_filter(C.byref(g), C.c_float(alpha), _f(x), _f(dy), C.c_float(beta), _f(dw))
    return dw


def conv2d_bwd_filter_at(x, dy, w_shape, stride, pad, idx):
    g = conv_geom(x.shape, w_shape, stride, pad)
    idx = np.ascontiguousarray(idx, np.int64)
    out = np.zeros(idx.shape, np.float32)
    lib().orc_conv2d_bwd_filter_at(C.byref(g), _f(x), _f(dy), _i64(idx), C.c_int64(idx.size), _f(out))
    return out


def conv2d_bwd_bias(dy, alpha=1.0, beta=0.0, db=None):
    N, K = dy.shape[0], dy.shape[1]
    plane = int(np.prod(dy.shape[2:])) if dy.ndim > 2 else 1
    if db is None:
        db = np.zeros((K,), np.float32)
    lib().orc_conv2d_bwd_bias(C.c_int32(N), C.c_int32(K), C.c_int32(plane), C.c_float(alpha), _f(dy),
                              C.c_float(beta), _f(db))
    return db


def conv2d_bwd_data(w, dy, x_shape, stride, pad, alpha=1.0, beta=0.0, dx=None):
    g = conv_geom(x_shape, w.shape, stride, pad)
    if dx is None:
        dx = np.zeros(x_shape, np.float32)
    lib().orc_conv2d_bwd_data(C.byref(g), C.c_float(alpha), _f(w), _f(dy), C.c_float(beta), _f(dx))
    return dx


def conv2d_bwd_data_at(w, dy, x_shape, stride, pad, idx):
    g = conv_geom(x_shape, w.shape, stride, pad)
    idx = np.ascontiguousarray(idx, np.int64)
    out = np.zeros(idx.shape, np.float32)
    lib().orc_conv2d_bwd_data_at(C.byref(g), _f(w), _f(dy), _i64(idx), C.c_int64(idx.size), _f(out))
    return out


def fast_conv2d_fwd(x, w, stride, pad):
    g = conv_geom(x.shape, w.shape, stride, pad)
    y = np.empty(conv_out_shape(g), np.float32)
    lib().orc_fast_conv2d_fwd(C.byref(g), _f(x), _f(w), _f(y))
    return y


def fast_conv2d_bwd_data(w, dy, x_shape, stride, pad):
    g = conv_geom(x_shape, w.shape, stride, pad)
    dx = np.empty(x_shape, np.float32)
    lib().orc_fast_conv2d_bwd_data(C.byref(g), _f(w), _f(dy), _f(dx))
    return dx


def fast_conv2d_bwd_filter(x, dy, dw, stride, pad):
    """dw += ... in place (beta = 1)."""
    g = conv_geom(x.shape, dw.shape, stride, pad)
    lib().orc_fast_conv2d_bwd_filter(C.byref(g), _f(x), _f(dy), _f(dw))
    return dw


def fast_gemm_rm(A, B, transA=False, transB=False, out=None, accumulate=False):
    """Row-major C[M][N] (+)= op(A)[M][K] op(B)[K][N]; A is [K][M] if transA, B is [N][K] if transB."""
    M, K = (A.shape[1], A.shape[0]) if transA else A.shape
    N = B.shape[0] if transB else B.shape[1]
    if out is None:
        out = np.zeros((M, N), np.float32)
    lib().orc_fast_gemm_rm(C.c_int(int(transA)), C.c_int(int(transB)), C.c_int(M), C.c_int(N), C.c_int(K),
                           _f(A), _f(B), _f(out), C.c_int(int(accumulate)))
    return out


# ---- elementwise ---------------------------------------------------------------------------
def add_bias_nchw(bias, y, alpha=1.0, beta=1.0):
    N, K = y.shape[0], y.shape[1]
    plane = int(np.prod(y.shape[2:])) if y.ndim > 2 else 1
    lib().orc_add_bias_nchw(_f(bias), _f(y), C.c_int32(plane), C.c_int32(K), C.c_int32(N),
                            C.c_float(alpha), C.c_float(beta))
    return y


def rect_inplace(y):
    lib().orc_rect_inplace(_f(y), C.c_int32(y.size // y.shape[0]), C.c_int32(y.shape[0]))
    return y


def rect_backprop_inplace(y, dy):
    lib().orc_rect_backprop_inplace(_f(y), C.c_int32(y.size // y.shape[0]), C.c_int32(y.shape[0]), _f(dy))
    return dy


# ---- BLAS ------------------------------------------------------------------------------------
def sgemm(transA, transB, m, n, k, alpha, A, lda, B, ldb, beta, Cm, ldc):
    lib().orc_sgemm(C.c_int(transA), C.c_int(transB), C.c_int32(m), C.c_int32(n), C.c_int32(k),
                    C.c_float(alpha), _f(A), C.c_int32(lda), _f(B), C.c_int32(ldb), C.c_float(beta),
                    _f(Cm), C.c_int32(ldc))
    return Cm


def saxpy(alpha, x, y):
    lib().orc_saxpy(C.c_int64(x.size), C.c_float(alpha), _f(x), _f(y))
    return y


def sscal(alpha, x):
    lib().orc_sscal(C.c_int64(x.size), C.c_float(alpha), _f(x))
    return x


# ---- pooling -------------------------------------------------------------------------------
def pool_geom(x_shape, size, stride, pad, mode, rounding=ROUND_FLOOR):
    N, Cc, H, W = x_shape
    return PoolGeom(N, Cc, H, W, size, stride, pad, mode, rounding)


def pool_out_shape(g):
    return (g.N, g.C, out_dim(g.H, g.size, g.stride, g.pad, g.round),
            out_dim(g.W, g.size, g.stride, g.pad, g.round))


def pool2d_fwd(x, size, stride, pad, mode, rounding=ROUND_FLOOR, want_argmax=False):
    g = pool_geom(x.shape, size, stride, pad, mode, rounding)
    y = np.zeros(pool_out_shape(g), np.float32)
    am = np.zeros(y.shape, np.int32) if want_argmax else None
    lib().orc_pool2d_fwd(C.byref(g), _f(x), _f(y), _i32(am) if want_argmax else None)
    return (y, am) if want_argmax else y


def pool2d_bwd(x, y, dy, size, stride, pad, mode, rounding=ROUND_FLOOR, argmax=None):
    g = pool_geom(x.shape, size, stride, pad, mode, rounding)
    dx = np.zeros(x.shape, np.float32)
    lib().orc_pool2d_bwd(C.byref(g), _f(x), _f(y), _f(dy), _f(dx), _i32(argmax) if argmax is not None else None)
    return dx


# ---- loss ------------------------------------------------------------------------------------
def softmax_fwd(x):
    N, Cc = x.shape
    p = np.zeros_like(x)
    lib().orc_softmax_fwd(_f(x), _f(p), C.c_int32(Cc), C.c_int32(N))
    return p


def softmax_kl_backward(p, labels, weights):
    N, Cc = p.shape
    dx = np.zeros_like(p)
    lib().orc_softmax_kl_backward(_f(p), C.c_int32(Cc), C.c_int32(N), _i32(labels), _f(weights), _f(dx))
    return dx


def softmax_kl_loss1(p, labels, weights, beta=0.0, loss1=None):
    N, Cc = p.shape
    if loss1 is None:
        loss1 = np.zeros((N,), np.float32)
    lib().orc_softmax_kl_loss1(_f(p), C.c_int32(Cc), C.c_int32(N), _i32(labels), _f(weights), C.c_float(beta),
                               _f(loss1))
    return loss1


def blockreduce_sum(src, beta=0.0, dst=None):
    batch, length = src.shape
    if dst is None:
        dst = np.zeros((batch,), np.float32)
    lib().orc_blockreduce_sum(_f(src), C.c_int32(length), C.c_int32(batch), _f(dst), C.c_float(beta))
    return dst


def blockreduce_argmax(src):
    batch, length = src.shape
    mx = np.zeros((batch,), np.float32)
    idx = np.zeros((batch,), np.int32)
    lib().orc_blockreduce_argmax(_f(src), C.c_int32(length), C.c_int32(batch), _f(mx), _i32(idx))
    return mx, idx


def accuracy_count(labels, cats):
    return int(lib().orc_accuracy_count(_i32(labels), _i32(cats), C.c_int32(labels.size)))


# ---- SGD -------------------------------------------------------------------------------------
def sgd_momentum_step(W, g, v, l2, scale, mu, apply, zero_grad=True):
    lib().orc_sgd_momentum_step(C.c_int64(W.size), _f(W), _f(g), _f(v), C.c_float(l2), C.c_float(scale),
                                C.c_float(mu), C.c_float(apply), C.c_int(int(zero_grad)))


def descend(W, g, s, l2):
    lib().orc_descend(C.c_int64(W.size), _f(W), _f(g), C.c_float(s), C.c_float(l2))


def round_bf16(x):
    """fp32 values rounded to the nearest bf16 (ties to even), returned as fp32."""
    y = np.ascontiguousarray(x, dtype=np.float32).copy()
    lib().orc_round_bf16(_f(y), C.c_int64(y.size))
    return y


def cast_u8_f32(x, scale):
    assert x.dtype == np.uint8 and x.flags.c_contiguous
    y = np.zeros(x.shape, np.float32)
    lib().orc_cast_u8_f32(x.ctypes.data_as(C.POINTER(C.c_uint8)), _f(y), C.c_int64(x.size), C.c_float(scale))
    return y


# ---- Data3d preprocessing, dropout, local response normalisation (numpy restatements) ------------------------

def crop_nchw(x, crop_w, crop_h, off_w, off_h):
    """Strided 4-d copy of Data3dOperator's Crop (src/operator/mod.rs:666-691): one offset for the whole batch."""
    return np.ascontiguousarray(x[:, :, off_h:off_h + crop_h, off_w:off_w + crop_w])


def flip_x(x):
    """FlipX (src/operator/mod.rs:751-777): every row of the batch reversed along the width."""
    return np.ascontiguousarray(x[..., ::-1])


def subtract_mean(x, mean, normalize):
    """SubtractElemwiseMean (src/operator/mod.rs:732-749): x + alpha * mean, alpha = -1/255 if normalize else -1,
    mean broadcast over the batch."""
    alpha = np.float32(-1.0 / 255.0) if normalize else np.float32(-1.0)
    return (x.astype(np.float64) + np.float64(alpha) * mean.astype(np.float64)[None]).astype(np.float32)


def pca3_noise(x, alphas, svals, svecs):
    """AddPixelwisePCALightingNoise in training (src/operator/mod.rs:709-727): channel c of image n is shifted by
    sum_j svecs[j][c] * alphas[n][j] * svals[j] (svecs[j] = the j-th singular vector, as the operator flattens it,
    mod.rs:523-533; which index the kernel treats as the channel is this build's choice)."""
    shift = np.einsum("jc,nj,j->nc", svecs.reshape(3, 3).astype(np.float64), alphas.reshape(-1, 3).astype(np.float64),
                      svals.astype(np.float64))
    return (x.astype(np.float64) + shift[:, :, None, None]).astype(np.float32)


def dropout(x, ratio, scale, rnd):
    """rembrandt_kernel_map_dropout as called at src/operator/mod.rs:2221-2229: keep where rnd > ratio."""
    mask = (rnd > np.float32(ratio)).astype(np.int32)
    return (np.float32(scale) * x * mask).astype(np.float32), mask


def dropout_backprop(dy, scale, mask):
    """rembrandt_kernel_map_dropout_backprop as called at src/operator/mod.rs:2239-2246."""
    return (np.float32(scale) * dy * mask).astype(np.float32)


def lrn_fwd(x, size, scale, power, min_div):
    """Cross-channel local response normalisation with the parameters of examples/imagenet_alexnet.model:31-37
    (cross_size, scale, power, min_div): d = min_div + scale * sum over the clipped channel window of x^2,
    y = x * d^-power.  fp64."""
    N, Cc = x.shape[0], x.shape[1]
    x64 = x.astype(np.float64)
    d = np.empty_like(x64)
    lo, hi = size // 2, (size - 1) // 2
    for c in range(Cc):
        c0, c1 = max(0, c - lo), min(Cc - 1, c + hi)
        d[:, c] = min_div + scale * (x64[:, c0:c1 + 1] ** 2).sum(axis=1)
    return (x64 * d ** (-power)).astype(np.float32), d.astype(np.float32)


def lrn_bwd(x, dy, size, scale, power, min_div):
    """Gradient of lrn_fwd w.r.t. x (fp64): dx[c] = dy[c] d[c]^-p - 2 scale p x[c] sum_{c': c in win(c')} dy[c'] y[c'] / d[c']."""
    Cc = x.shape[1]
    x64, dy64 = x.astype(np.float64), dy.astype(np.float64)
    lo, hi = size // 2, (size - 1) // 2
    d = np.empty_like(x64)
    for c in range(Cc):
        c0, c1 = max(0, c - lo), min(Cc - 1, c + hi)
        d[:, c] = min_div + scale * (x64[:, c0:c1 + 1] ** 2).sum(axis=1)
    y = x64 * d ** (-power)
    t = dy64 * y / d
    dx = dy64 * d ** (-power)
    for c in range(Cc):
        c0, c1 = max(0, c - hi), min(Cc - 1, c + lo)
        dx[:, c] -= 2.0 * scale * power * x64[:, c] * t[:, c0:c1 + 1].sum(axis=1)
    return dx.astype(np.float32)


# ---- spatial batch normalisation (numpy restatement of the cuDNN Spatial mode the reference calls, ------------
# ---- src/operator/conv.rs:493-535, 594-607; fp64 arithmetic on the fp32 inputs) ---------------------------------
def bnorm_mov_avg_at_iter(kind, ema_factor, t):
    """BNormMovingAverage::at_iter (src/operator/conv.rs:58-72)."""
    if kind == "Cumulative":
        return 1.0 / (1.0 + t)
    assert kind == "Exponential"
    return 1.0 if t == 0 else float(ema_factor)


def bnorm_fwd_train(x, scale, bias, running_mean, running_ivar, ema_factor, epsilon, alpha=1.0, beta=0.0, y=None):
    """Returns (y, cached_mean, cached_ivar, new_running_mean, new_running_ivar).  Statistics are per channel over
    (n, h, w), variance biased (divided by m); the moving pair averages mean and inverse standard deviation
    ("parity unpinned" for the second: what cuDNN v4 kept in resultRunningInvVariance is not checkable here)."""
    x64 = x.astype(np.float64)
    mean = x64.mean(axis=(0, 2, 3))
    var = ((x64 - mean[None, :, None, None]) ** 2).mean(axis=(0, 2, 3))
    ivar = 1.0 / np.sqrt(var + epsilon)
    out = scale.astype(np.float64)[None, :, None, None] * (x64 - mean[None, :, None, None]) * ivar[None, :, None, None] \
        + bias.astype(np.float64)[None, :, None, None]
    out = alpha * out
    if beta != 0.0:
        out = out + beta * y.astype(np.float64)
    new_rm = (1.0 - ema_factor) * running_mean.astype(np.float64) + ema_factor * mean
    new_ri = (1.0 - ema_factor) * running_ivar.astype(np.float64) + ema_factor * ivar
    f = np.float32
    return out.astype(f), mean.astype(f), ivar.astype(f), new_rm.astype(f), new_ri.astype(f)


def bnorm_fwd_infer(x, scale, bias, running_mean, running_ivar, alpha=1.0, beta=0.0, y=None):
    b = lambda v: v.astype(np.float64)[None, :, None, None]
    out = alpha * (b(scale) * (x.astype(np.float64) - b(running_mean)) * b(running_ivar) + b(bias))
    if beta != 0.0:
        out = out + beta * y.astype(np.float64)
    return out.astype(np.float32)


def bnorm_bwd(x, dy, scale, cached_mean, cached_ivar):
    """Returns (dx, dscale, dbias) of y = scale*xhat + bias with xhat = (x - mean(x))*ivar(x), the batch statistics
    being functions of x: dx = scale*ivar*(dy - mean(dy) - xhat*mean(dy*xhat))."""
    b = lambda v: v.astype(np.float64)[None, :, None, None]
    x64, dy64 = x.astype(np.float64), dy.astype(np.float64)
    xhat = (x64 - b(cached_mean)) * b(cached_ivar)
    dbias = dy64.sum(axis=(0, 2, 3))
    dscale = (dy64 * xhat).sum(axis=(0, 2, 3))
    m = x.shape[0] * x.shape[2] * x.shape[3]
    dx = b(scale) * b(cached_ivar) * (dy64 - (dbias / m)[None, :, None, None] - xhat * (dscale / m)[None, :, None, None])
    f = np.float32
    return dx.astype(f), dscale.astype(f), dbias.astype(f)
