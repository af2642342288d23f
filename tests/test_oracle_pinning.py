"""CPU: pins the oracle.  The reference holds no golden vectors for this path (its tests assert nothing),
so every oracle function is checked against an independent statement of the same mathematics:
torch CPU fp64 library routines, numpy brute force on tiny inputs, adjoint identities, closed forms.
Each check is chosen so that a plausible mistake (flipped filter, dropped pad, transposed operand,
wrong divisor, wrong tie rule) fails it."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle as O

RNG = np.random.default_rng(1234)


def rnd(*shape):
    return RNG.standard_normal(shape).astype(np.float32)


CONV = [(2, 3, 9, 7, 4, 3, 1, 1), (2, 3, 13, 13, 5, 5, 2, 2), (1, 2, 23, 23, 3, 11, 4, 0), (3, 4, 8, 8, 6, 1, 1, 0),
        (2, 2, 10, 11, 3, 3, 3, 1), (1, 1, 5, 5, 1, 5, 1, 0), (2, 3, 6, 6, 2, 3, 1, 2)]


@pytest.mark.parametrize("case", CONV, ids=[str(c) for c in CONV])
def test_conv_against_torch_fp64(case):
    N, C, H, W, K, R, st, pad = case
    x, w = rnd(N, C, H, W), rnd(K, C, R, R)
    xt = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    wt = torch.tensor(w, dtype=torch.float64, requires_grad=True)
    yt = F.conv2d(xt, wt, stride=st, padding=pad)   # cross-correlation, OIHW weights
    y = O.conv2d_fwd(x, w, st, pad)
    assert y.shape == tuple(yt.shape)
    np.testing.assert_allclose(y, yt.detach().numpy(), rtol=1e-6, atol=1e-6)
    dy = rnd(*y.shape)
    yt.backward(torch.tensor(dy, dtype=torch.float64))
    np.testing.assert_allclose(O.conv2d_bwd_filter(x, dy, w.shape, st, pad), wt.grad.numpy(), rtol=1e-6, atol=1e-5)
    np.testing.assert_allclose(O.conv2d_bwd_data(w, dy, x.shape, st, pad), xt.grad.numpy(), rtol=1e-6, atol=1e-5)
    np.testing.assert_allclose(O.conv2d_bwd_bias(dy), dy.astype(np.float64).sum(axis=(0, 2, 3)), rtol=1e-6, atol=1e-5)
    # alpha / beta
    y0 = rnd(*y.shape)
    np.testing.assert_allclose(O.conv2d_fwd(x, w, st, pad, 0.5, 2.0, y0.copy()), 0.5 * yt.detach().numpy() + 2.0 * y0,
                               rtol=1e-6, atol=1e-5)
    # sampled variants and the fast (im2col + SGEMM) family agree with the full precise family
    idx = RNG.integers(0, y.size, 40)
    assert np.array_equal(O.conv2d_fwd_at(x, w, st, pad, idx), y.ravel()[idx])
    dx = O.conv2d_bwd_data(w, dy, x.shape, st, pad)
    idx = RNG.integers(0, dx.size, 40)
    np.testing.assert_allclose(O.conv2d_bwd_data_at(w, dy, x.shape, st, pad, idx), dx.ravel()[idx], rtol=1e-6, atol=1e-6)
    dw = O.conv2d_bwd_filter(x, dy, w.shape, st, pad)
    idx = RNG.integers(0, dw.size, 40)
    np.testing.assert_allclose(O.conv2d_bwd_filter_at(x, dy, w.shape, st, pad, idx), dw.ravel()[idx], rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(O.fast_conv2d_fwd(x, w, st, pad), y, rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(O.fast_conv2d_bwd_data(w, dy, x.shape, st, pad), dx, rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(O.fast_conv2d_bwd_filter(x, dy, np.zeros_like(w), st, pad), dw, rtol=1e-4, atol=1e-4)


def test_conv_brute_force_and_special_cases():
    # 7-loop definition on a tiny case, written independently
    N, C, H, W, K, R, st, pad = 2, 2, 5, 4, 3, 3, 2, 1
    x, w = rnd(N, C, H, W), rnd(K, C, R, R)
    P, Q = (H + 2 * pad - R) // st + 1, (W + 2 * pad - R) // st + 1
    y = np.zeros((N, K, P, Q))
    for n in range(N):
        for k in range(K):
            for p in range(P):
                for q in range(Q):
                    for c in range(C):
                        for r in range(R):
                            for s in range(R):
                                h, ww = p * st + r - pad, q * st + s - pad
                                if 0 <= h < H and 0 <= ww < W:
                                    y[n, k, p, q] += float(x[n, c, h, ww]) * float(w[k, c, r, s])
    np.testing.assert_allclose(O.conv2d_fwd(x, w, st, pad), y, rtol=1e-6, atol=1e-6)
    # 1x1 stride 1 == per-pixel GEMM; R=H, S=W, pad 0 == affine
    x, w = rnd(3, 5, 4, 4), rnd(7, 5, 1, 1)
    np.testing.assert_allclose(O.conv2d_fwd(x, w, 1, 0), np.einsum("kc,nchw->nkhw", w[:, :, 0, 0].astype(np.float64), x),
                               rtol=1e-6, atol=1e-6)
    x, w = rnd(3, 2, 4, 4), rnd(6, 2, 4, 4)
    np.testing.assert_allclose(O.conv2d_fwd(x, w, 1, 0).reshape(3, 6), x.reshape(3, -1).astype(np.float64) @ w.reshape(6, -1).T,
                               rtol=1e-6, atol=1e-5)


def test_conv_adjoint_identities():
    # <conv(x,w), dy> = <x, bwd_data(w,dy)> = <w, bwd_filter(x,dy)>
    for (N, C, H, W, K, R, st, pad) in CONV:
        x, w = rnd(N, C, H, W), rnd(K, C, R, R)
        y = O.conv2d_fwd(x, w, st, pad).astype(np.float64)
        dy = rnd(*y.shape)
        a = float((y * dy).sum())
        b = float((x.astype(np.float64) * O.conv2d_bwd_data(w, dy, x.shape, st, pad)).sum())
        c = float((w.astype(np.float64) * O.conv2d_bwd_filter(x, dy, w.shape, st, pad)).sum())
        scale = float(np.abs(y * dy).sum()) + 1e-12
        assert abs(a - b) / scale < 1e-6 and abs(a - c) / scale < 1e-6


def test_out_dims():
    # operator-style floor (mod.rs:1393-1398) and gen-1 ceil (layer.rs:1741-1747) extents
    assert [O.out_dim(n, 3, 2, 0) for n in (55, 27, 13)] == [27, 13, 6]
    assert [O.out_dim(n, 3, 2, 0, O.ROUND_CEIL) for n in (54, 27, 13)] == [27, 13, 6]   # NIN 54 -> 27 -> 13 -> 6
    assert [O.out_dim(n, 3, 2, 0) for n in (54, 26, 12)] == [26, 12, 5]
    assert O.out_dim(227, 11, 4, 0) == 55 and O.out_dim(28, 5, 1, 2) == 28 and O.out_dim(32, 3, 2, 1) == 16
    assert O.out_dim(2, 5, 1, 0) == 0 and O.out_dim(2, 5, 1, 0, O.ROUND_CEIL) == 1


POOL = [(9, 3, 2, 0), (9, 3, 2, 1), (8, 2, 2, 0), (10, 3, 2, 0), (7, 3, 1, 1), (13, 3, 3, 1), (6, 6, 1, 0)]


@pytest.mark.parametrize("case", POOL, ids=[str(c) for c in POOL])
@pytest.mark.parametrize("ceil", [False, True])
def test_pool_against_torch_and_brute_force(case, ceil):
    H, k, st, pad = case
    x = np.round(rnd(2, 3, H, H + 1) * 2) / 2     # many exact ties
    rounding = O.ROUND_CEIL if ceil else O.ROUND_FLOOR
    xt = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    # max: torch's max_pool2d pads with -inf and routes ties to the first maximum, as the oracle does
    yt = F.max_pool2d(xt, k, st, pad, ceil_mode=ceil)
    y, am = O.pool2d_fwd(x, k, st, pad, O.POOL_MAX, rounding, want_argmax=True)
    if y.shape == tuple(yt.shape):   # torch drops a ceil-mode window that starts in the padding; the gen-1 extent keeps it
        np.testing.assert_array_equal(y, yt.detach().numpy().astype(np.float32))
        dy = rnd(*y.shape)
        yt.backward(torch.tensor(dy, dtype=torch.float64))
        np.testing.assert_allclose(O.pool2d_bwd(x, y, dy, k, st, pad, O.POOL_MAX, rounding), xt.grad.numpy(), rtol=1e-6, atol=1e-6)
    # brute force for both modes (covers the shapes torch disagrees on, and the k*k divisor of clipped windows)
    P, Q = y.shape[2], y.shape[3]
    ya = O.pool2d_fwd(x, k, st, pad, O.POOL_AVG, rounding)
    dy = rnd(*y.shape)
    dmax, davg = np.zeros(x.shape), np.zeros(x.shape)
    for n in range(2):
        for c in range(3):
            for p in range(P):
                for q in range(Q):
                    taps = [(p * st + r - pad, q * st + s - pad) for r in range(k) for s in range(k)]
                    taps = [(h, w) for (h, w) in taps if 0 <= h < H and 0 <= w < H + 1]
                    vals = [x[n, c, h, w] for (h, w) in taps]
                    if taps:
                        best = int(np.argmax(vals))   # first maximum
                        assert y[n, c, p, q] == vals[best]
                        assert am[n, c, p, q] == taps[best][0] * (H + 1) + taps[best][1]
                        dmax[n, c, taps[best][0], taps[best][1]] += dy[n, c, p, q]
                    else:
                        assert y[n, c, p, q] == 0 and am[n, c, p, q] == -1
                    assert abs(ya[n, c, p, q] - sum(map(float, vals)) / (k * k)) < 1e-6
                    for (h, w) in taps:
                        davg[n, c, h, w] += dy[n, c, p, q] / (k * k)
    np.testing.assert_allclose(O.pool2d_bwd(x, y, dy, k, st, pad, O.POOL_MAX, rounding), dmax, rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(O.pool2d_bwd(x, y, dy, k, st, pad, O.POOL_MAX, rounding, argmax=am), dmax, rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(O.pool2d_bwd(x, ya, dy, k, st, pad, O.POOL_AVG, rounding), davg, rtol=1e-6, atol=1e-6)
    if not ceil:
        yat = F.avg_pool2d(torch.tensor(x, dtype=torch.float64), k, st, pad, count_include_pad=True)
        np.testing.assert_allclose(ya, yat.numpy(), rtol=1e-6, atol=1e-6)


def test_bias_relu_blas():
    y, b = rnd(3, 4, 5, 6), rnd(4)
    np.testing.assert_allclose(O.add_bias_nchw(b, y.copy()), y + b[None, :, None, None], rtol=1e-6)
    np.testing.assert_allclose(O.add_bias_nchw(b, y.copy(), 2.0, 0.5), 0.5 * y + 2.0 * b[None, :, None, None], rtol=1e-6)
    yt = torch.tensor(y, requires_grad=True)
    out = torch.relu(yt)
    np.testing.assert_array_equal(O.rect_inplace(y.copy()), out.detach().numpy())
    dy = rnd(*y.shape)
    out.backward(torch.tensor(dy))
    np.testing.assert_array_equal(O.rect_backprop_inplace(np.maximum(y, 0), dy.copy()), yt.grad.numpy())
    z = np.array([[0.0, -0.0, 1.0]], np.float32)
    assert O.rect_backprop_inplace(z, np.ones_like(z)).tolist() == [[0.0, 0.0, 1.0]]   # sub-gradient 0 at y == 0
    # column-major sgemm in all four transposition cases vs numpy fp64
    m, n, k = 7, 5, 9
    for tA in (0, 1):
        for tB in (0, 1):
            A = rnd(*((m, k) if tA else (k, m)))  # memory shape of column-major (k,m)^T etc.
            B = rnd(*((k, n) if tB else (n, k)))
            C0 = rnd(n, m)
            opA = A.astype(np.float64) if tA else A.T.astype(np.float64)   # (m,k)
            opB = B.astype(np.float64) if tB else B.T.astype(np.float64)   # (k,n)
            want = (0.7 * opA @ opB + 0.3 * C0.T).T
            got = O.sgemm(tA, tB, m, n, k, 0.7, A, A.shape[1], B, B.shape[1], 0.3, C0.copy(), m)
            np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5)
    A, B = rnd(6, 11), rnd(11, 8)
    np.testing.assert_allclose(O.fast_gemm_rm(A, B), A @ B, rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(O.fast_gemm_rm(A.T.copy(), B, transA=True), A @ B, rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(O.fast_gemm_rm(A, B.T.copy(), transB=True), A @ B, rtol=1e-4, atol=1e-4)
    x, yv = rnd(1001), rnd(1001)
    np.testing.assert_allclose(O.saxpy(0.3, x, yv.copy()), yv + np.float32(0.3) * x, rtol=1e-6, atol=1e-7)
    np.testing.assert_array_equal(O.sscal(-2.0, x.copy()), np.float32(-2.0) * x)


def test_softmax_loss_argmax():
    x = rnd(6, 11) * 5
    labels = RNG.integers(0, 11, 6).astype(np.int32)
    wts = RNG.uniform(0.1, 1.0, 6).astype(np.float32)
    p = O.softmax_fwd(x)
    xt = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    logp = torch.log_softmax(xt, dim=1)
    np.testing.assert_allclose(p, logp.exp().detach().numpy(), rtol=1e-6, atol=1e-8)
    np.testing.assert_allclose(p.sum(axis=1), 1.0, rtol=1e-6)
    loss_t = -(torch.tensor(wts, dtype=torch.float64) * logp[torch.arange(6), torch.tensor(labels, dtype=torch.long)]).sum()
    loss_t.backward()
    d = O.softmax_kl_backward(p, labels, wts)
    np.testing.assert_allclose(d, xt.grad.numpy(), rtol=1e-5, atol=1e-7)      # delta = w (p - onehot) IS the CE gradient
    np.testing.assert_allclose(d.sum(axis=1), 0.0, atol=1e-6)
    l1 = O.softmax_kl_loss1(p, labels, wts)
    np.testing.assert_allclose(O.blockreduce_sum(l1.reshape(1, -1))[0], float(loss_t.detach()), rtol=1e-5)
    np.testing.assert_allclose(O.softmax_kl_loss1(p, labels, wts, 1.0, l1.copy()), 2 * l1, rtol=1e-6)
    np.testing.assert_allclose(O.blockreduce_sum(x, 1.0, np.ones(6, np.float32)), 1.0 + x.astype(np.float64).sum(axis=1), rtol=1e-5, atol=1e-5)
    # large logits: max-subtracted softmax stays finite
    big = np.array([[1000.0, 999.0, -1000.0]], np.float32)
    assert np.isfinite(O.softmax_fwd(big)).all()
    mx, idx = O.blockreduce_argmax(p)
    np.testing.assert_array_equal(idx, np.argmax(p, axis=1))
    ties = np.array([[1, 3, 3, 2], [5, 5, 5, 5], [0, 0, 0, 7]], np.float32)
    assert O.blockreduce_argmax(ties)[1].tolist() == [1, 0, 3]               # lowest index wins
    assert O.accuracy_count(np.array([1, 2, 3], np.int32), np.array([1, 0, 3], np.int32)) == 2


@pytest.mark.parametrize("nesterov", [False, True])
def test_sgd_flavours_against_torch_optim(nesterov):
    """Gradient / GradientNesterov are torch.optim.SGD (dampening 0); Update{mu} follows the same
    trajectory at constant step size; one plain step has the closed form W1 = W0 - lr (g + l2 W0)."""
    from oracle import graph as OG
    lr, mu, l2 = 0.05, 0.9, 1e-2
    w0 = rnd(50)
    grads = [rnd(50) for _ in range(4)]

    class One:  # a one-tensor operator with the reference's BLAS-1 methods
        def __init__(self):
            self.p = OG._Params((50,), 1)
            self.p.weights[...] = w0
        def __getattr__(self, name):
            return getattr(self.p, name)

    wt = torch.tensor(w0.astype(np.float64), requires_grad=True)
    opt = torch.optim.SGD([wt], lr=lr, momentum=mu, weight_decay=l2, nesterov=nesterov)
    op = One()
    sgd = OG.SgdOpt(lr, ("GradientNesterov" if nesterov else "Gradient", mu), l2)
    sgd.begin(op)
    upd = One()
    usgd = OG.SgdOpt(lr, ("Update", mu), l2)
    usgd.begin(upd)
    for g in grads:
        wt.grad = torch.tensor(g.astype(np.float64))
        opt.step()
        op.p.grad_weights[...] = g
        sgd.step(op)
        np.testing.assert_allclose(op.p.weights, wt.detach().numpy(), rtol=1e-5, atol=1e-6)
        assert not op.p.grad_weights.any()
        if not nesterov:
            upd.p.grad_weights[...] = g
            usgd.step(upd)
            np.testing.assert_allclose(upd.p.weights, wt.detach().numpy(), rtol=1e-5, atol=1e-6)
    z = One()
    zs = OG.SgdOpt(lr, "Zero", l2)
    zs.begin(z)
    z.p.grad_weights[...] = grads[0]
    zs.step(z)
    np.testing.assert_allclose(z.p.weights, w0 - np.float32(lr) * (grads[0] + np.float32(l2) * w0), rtol=1e-6, atol=1e-7)


def test_update_nesterov_telescopes():
    """UpdateNesterov keeps theta + mu*v in the weights between iterations; un-applying it recovers the
    Update{mu} iterate evaluated at look-ahead gradients (here: constant gradients, so both velocity
    sequences coincide)."""
    from oracle import graph as OG
    lr, mu = 0.1, 0.5
    g = rnd(20)

    class One:
        def __init__(self):
            self.p = OG._Params((20,), 1)
        def __getattr__(self, name):
            return getattr(self.p, name)

    a, b = One(), One()
    sa, sb = OG.SgdOpt(lr, ("UpdateNesterov", mu), 0.0), OG.SgdOpt(lr, ("Update", mu), 0.0)
    sa.begin(a); sb.begin(b)
    for _ in range(4):
        a.p.grad_weights[...] = g
        b.p.grad_weights[...] = g
        sa.step(a); sb.step(b)
        np.testing.assert_allclose(a.p.acc_grad_weights, b.p.acc_grad_weights, rtol=1e-6)
        np.testing.assert_allclose(a.p.weights, b.p.weights + np.float32(mu) * b.p.acc_grad_weights, rtol=1e-5, atol=1e-6)


def test_fused_sgd_step_equals_blas1_sequence():
    W, g, v = rnd(1000), rnd(1000), rnd(1000)
    W2, g2, v2 = W.copy(), g.copy(), v.copy()
    O.sgd_momentum_step(W, g, v, 5e-4, -0.01, 0.9, 1.0, True)
    O.saxpy(5e-4, W2, g2); O.sscal(0.9, v2); O.saxpy(-0.01, g2, v2); O.saxpy(1.0, v2, W2)
    np.testing.assert_allclose(W, W2, rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(v, v2, rtol=1e-6, atol=1e-7)
    assert not g.any()
    W3, g3 = rnd(100), rnd(100)
    W4, g4 = W3.copy(), g3.copy()
    O.descend(W3, g3, 0.1, 1e-3)
    np.testing.assert_allclose(g3, g4 + np.float32(1e-3) * W4, rtol=1e-6)
    np.testing.assert_allclose(W3, W4 - np.float32(0.1) * g3, rtol=1e-6, atol=1e-7)


def test_step_schedules():
    from oracle import graph as OG
    s = {"kind": "Anneal4", "steps": [1.0, 0.5, 0.25, 0.125, 0.0625], "iters": [0, 10, 20, 30, 40]}
    assert [OG.step_size_at(s, t) for t in (0, 9, 10, 19, 20, 29, 30, 39, 40, 1000)] == [1.0, 1.0, 0.5, 0.5, 0.25, 0.25, 0.125, 0.125, 0.0625, 0.0625]
    inv = {"kind": "Inverse", "steps": [0.1, 0.01]}
    assert abs(OG.step_size_at(inv, 100) - 0.1 / (1 + 0.1 * 0.01 * 100)) < 1e-7


def test_cast():
    x = np.arange(256, dtype=np.uint8)
    np.testing.assert_array_equal(O.cast_u8_f32(x, 1.0), x.astype(np.float32))
    np.testing.assert_allclose(O.cast_u8_f32(x, 1 / 255.0), x / 255.0, rtol=1e-6)


def test_graph_gradients_by_finite_differences():
    """The whole oracle chain (conv+ReLU -> avg pool -> affine -> softmax-KL) has the loss gradient it claims:
    central differences on a few weights of every parameter tensor."""
    from oracle import graph as OG
    layers = [("conv2d", (6, 6, 2), 3, 1, 1, 3, "Rect"), ("pool2d", (6, 6, 3), 2, 2, 0, "Average", False),
              ("affine", 27, 4, "Identity")]
    batch = 3
    rng = np.random.default_rng(42)   # own stream: the check must not depend on test order
    net = OG.SequentialOperatorWorker(layers, 4, batch)
    for op in net.hidden:
        if op.p is not None:
            op.p.weights[...] = rng.standard_normal(op.p.weights.shape).astype(np.float32) * 0.5
            op.p.bias[...] = rng.standard_normal(op.p.bias.shape).astype(np.float32) * 0.1
    x = rng.standard_normal((batch, 2, 6, 6)).astype(np.float32)
    net.stage_batch(np.array([0, 3, 1], np.int32), 1.0 / batch)

    def loss():
        net.forward(x)
        p = net.out_values.astype(np.float64)
        return float(-(net.weights * np.log(p[np.arange(batch), net.labels])).sum())

    loss()
    net.backward()
    for op in net.hidden:
        if op.p is None:
            continue
        for arr, grad in ((op.p.weights, op.p.grad_weights), (op.p.bias, op.p.grad_bias)):
            flat, gflat = arr.reshape(-1), grad.reshape(-1)
            for i in rng.integers(0, flat.size, 5):
                old = flat[i]
                eps = 1e-3
                flat[i] = old + eps
                lp = loss()
                flat[i] = old - eps
                lm = loss()
                flat[i] = old
                fd = (lp - lm) / (2 * eps)
                assert abs(fd - gflat[i]) < 2e-3 * max(1.0, abs(fd)), (fd, gflat[i])


def test_round_bf16_matches_torch_round_trip():
    """orc_round_bf16 against torch's float32 -> bfloat16 -> float32 (round to nearest even), on random values,
    exact ties, subnormals, infinities and the largest finite values (which round up to infinity)."""
    rng = np.random.default_rng(9)
    x = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** rng.integers(-30, 30, 20000).astype(np.float32),
        np.array([0.0, -0.0, 1.0, 1.00390625, 1.01171875, 1.005859375, 3.3895314e38, 3.4028235e38, -3.4028235e38,
                  np.inf, -np.inf, 1e-40, -1e-45, 65280.0, 65408.0], np.float32),
        # every tie pattern: bf16 value + exactly half an ulp
        (np.arange(0x3f800000, 0x3f800000 + (1 << 20), 1 << 15, dtype=np.uint32)).view(np.float32),
    ])
    want = torch.from_numpy(x).to(torch.bfloat16).to(torch.float32).numpy()
    got = O.round_bf16(x)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert np.isnan(O.round_bf16(np.array([np.nan], np.float32))[0])


def test_lrn_matches_torch_local_response_norm():
    """lrn_fwd / lrn_bwd against torch's local_response_norm (fp64) and its autograd; torch divides alpha by the
    window size, the `.model` parameter `scale` multiplies the plain sum."""
    rng = np.random.default_rng(10)
    for (shape, size) in (((2, 7, 3, 4), 5), ((1, 3, 2, 2), 5), ((2, 8, 3, 3), 4), ((2, 6, 2, 5), 1)):
        x = rng.standard_normal(shape).astype(np.float32) * 3
        dy = rng.standard_normal(shape).astype(np.float32)
        scale, power, min_div = 1e-2, 0.75, 2.0
        xt = torch.from_numpy(x).double().requires_grad_(True)
        yt = F.local_response_norm(xt, size, alpha=scale * size, beta=power, k=min_div)
        (gx,) = torch.autograd.grad(yt, xt, torch.from_numpy(dy).double())
        y, d = O.lrn_fwd(x, size, scale, power, min_div)
        np.testing.assert_allclose(y, yt.detach().numpy(), rtol=1e-6, atol=1e-7)
        np.testing.assert_allclose(O.lrn_bwd(x, dy, size, scale, power, min_div), gx.numpy(), rtol=1e-5, atol=1e-6)
        assert (d >= min_div).all()


def test_bnorm_matches_torch_batch_norm():
    """bnorm_fwd_train / bnorm_fwd_infer / bnorm_bwd against torch.nn.functional.batch_norm (fp64) and its autograd,
    on a channel with a large mean as well.  torch keeps a running *variance* (unbiased); the reference's buffer is
    named running_ivar, so only the running mean and the cached batch statistics are compared, and the moving
    inverse standard deviation is checked against its own definition (parity unpinned for that buffer)."""
    rng = np.random.default_rng(12)
    for shape in ((4, 3, 5, 6), (2, 5, 1, 1), (3, 2, 7, 7), (1, 4, 3, 3)):
        C = shape[1]
        x = rng.standard_normal(shape).astype(np.float32) * 2 + np.linspace(-1, 50, C, dtype=np.float32)[None, :, None, None]
        dy = rng.standard_normal(shape).astype(np.float32)
        scale, bias = (rng.standard_normal(C).astype(np.float32) + 1, rng.standard_normal(C).astype(np.float32))
        rm, ri = rng.standard_normal(C).astype(np.float32), rng.random(C).astype(np.float32) + 0.5
        eps, ema = 1e-5, 0.1
        xt = torch.from_numpy(x).double().requires_grad_(True)
        st, bt = torch.from_numpy(scale).double().requires_grad_(True), torch.from_numpy(bias).double().requires_grad_(True)
        trm, trv = torch.from_numpy(rm).double().clone(), torch.ones(C, dtype=torch.float64)
        yt = F.batch_norm(xt, trm, trv, st, bt, training=True, momentum=ema, eps=eps)
        gx, gs, gb = torch.autograd.grad(yt, (xt, st, bt), torch.from_numpy(dy).double())
        y, cm, ci, nrm, nri = O.bnorm_fwd_train(x, scale, bias, rm, ri, ema, eps)
        np.testing.assert_allclose(y, yt.detach().numpy(), rtol=1e-6, atol=1e-6)
        np.testing.assert_allclose(nrm, trm.numpy(), rtol=1e-6, atol=1e-6)
        x64 = x.astype(np.float64)
        np.testing.assert_allclose(cm, x64.mean(axis=(0, 2, 3)), rtol=1e-6)
        np.testing.assert_allclose(ci, 1.0 / np.sqrt(x64.var(axis=(0, 2, 3)) + eps), rtol=1e-6)
        np.testing.assert_allclose(nri, 0.9 * ri + 0.1 * ci, rtol=1e-6)
        dx, ds, db = O.bnorm_bwd(x, dy, scale, cm, ci)
        np.testing.assert_allclose(dx, gx.numpy(), rtol=1e-4, atol=1e-5)
        np.testing.assert_allclose(ds, gs.numpy(), rtol=1e-5, atol=1e-5)
        np.testing.assert_allclose(db, gb.numpy(), rtol=1e-5, atol=1e-5)
        # blend and inference: y = alpha*bn(x) + beta*y0; inference with torch's (mean, var) <-> (mean, 1/sqrt(var+eps))
        y0 = rng.standard_normal(shape).astype(np.float32)
        yb = O.bnorm_fwd_train(x, scale, bias, rm, ri, ema, eps, alpha=0.5, beta=2.0, y=y0)[0]
        np.testing.assert_allclose(yb, 0.5 * yt.detach().numpy() + 2.0 * y0, rtol=1e-6, atol=1e-5)
        var = rng.random(C) + 0.3
        yi = F.batch_norm(torch.from_numpy(x).double(), torch.from_numpy(rm).double(), torch.from_numpy(var),
                          torch.from_numpy(scale).double(), torch.from_numpy(bias).double(), training=False, eps=eps)
        got = O.bnorm_fwd_infer(x, scale, bias, rm, (1.0 / np.sqrt(var + eps)).astype(np.float32))
        np.testing.assert_allclose(got, yi.numpy(), rtol=1e-5, atol=1e-5)
    assert O.bnorm_mov_avg_at_iter("Cumulative", 0.1, 0) == 1.0 and O.bnorm_mov_avg_at_iter("Cumulative", 0.1, 3) == 0.25
    assert O.bnorm_mov_avg_at_iter("Exponential", 0.1, 0) == 1.0 and O.bnorm_mov_avg_at_iter("Exponential", 0.1, 7) == 0.1


def _torch_unit(x, u, eps):
    """conv (no bias) + training-mode batch norm of one unit, on torch fp64 leaves."""
    z = F.conv2d(x, u["w"], None, u["stride"], u["pad"])
    return F.batch_norm(z, None, None, u["scale"], u["bias"], training=True, eps=eps)


@pytest.mark.parametrize("kind", ["bnorm_conv2d", "stack_res_conv2d", "proj_stack_res_conv2d_s2", "proj_stack_res_conv2d_s1"])
def test_bnorm_operators_match_torch_autograd(kind):
    """The wiring of the batch-normalised operators (residual add, where the ReLU masks act, which deltas add up)
    against torch autograd of the same composite in fp64: out_act, in_delta and every parameter gradient."""
    from oracle import graph as OG
    rng = np.random.default_rng(13)
    batch, eps = 3, 1e-5
    if kind == "bnorm_conv2d":
        in_dims = (9, 8, 3)
        op = OG.BNormConv2dOperator(batch, in_dims, 3, 2, 1, 5, "Rect", epsilon=eps)
    elif kind == "stack_res_conv2d":
        in_dims = (6, 5, 4)
        op = OG.StackResConv2dOperator(batch, in_dims, "Rect", epsilon=eps)
    elif kind == "proj_stack_res_conv2d_s2":
        in_dims = (8, 6, 3)
        op = OG.ProjStackResConv2dOperator(batch, in_dims, (4, 3, 5), "Rect", epsilon=eps)
    else:
        in_dims = (5, 4, 3)
        op = OG.ProjStackResConv2dOperator(batch, in_dims, (5, 4, 6), "Rect", epsilon=eps)
    tu = []
    for u in op.units:
        u.weights[...] = rng.standard_normal(u.weights.shape) * 0.4
        u.scale[...] = 1 + 0.3 * rng.standard_normal(u.scale.shape)
        u.bias[...] = 0.3 * rng.standard_normal(u.bias.shape)
        tu.append({"w": torch.from_numpy(u.weights).double().requires_grad_(True),
                   "scale": torch.from_numpy(u.scale).double().requires_grad_(True),
                   "bias": torch.from_numpy(u.bias).double().requires_grad_(True), "stride": u.stride, "pad": u.pad})
    x = rng.standard_normal((batch, in_dims[2], in_dims[1], in_dims[0])).astype(np.float32)
    xt = torch.from_numpy(x).double().requires_grad_(True)
    if kind == "bnorm_conv2d":
        yt = torch.relu(_torch_unit(xt, tu[0], eps))
    elif kind == "stack_res_conv2d":
        yt = torch.relu(xt + _torch_unit(torch.relu(_torch_unit(xt, tu[0], eps)), tu[1], eps))
    else:
        yt = torch.relu(_torch_unit(torch.relu(_torch_unit(xt, tu[0], eps)), tu[1], eps) + _torch_unit(xt, tu[2], eps))
    y = op.forward(x, True, 0)
    np.testing.assert_allclose(y, yt.detach().numpy(), rtol=1e-5, atol=1e-5)
    assert tuple(yt.shape[1:]) == (op.out_dims[2], op.out_dims[1], op.out_dims[0])
    dy = rng.standard_normal(y.shape).astype(np.float32)
    leaves = [xt] + [t[k] for t in tu for k in ("w", "scale", "bias")]
    grads = torch.autograd.grad(yt, leaves, torch.from_numpy(dy).double())
    op.out_delta = dy.copy()
    dx = op.backward(True)
    np.testing.assert_allclose(dx, grads[0].numpy(), rtol=1e-4, atol=2e-5)
    for k, u in enumerate(op.units):
        gw, gs, gb = grads[1 + 3 * k: 4 + 3 * k]
        np.testing.assert_allclose(u.grad_weights, gw.numpy(), rtol=1e-4, atol=2e-5)
        np.testing.assert_allclose(u.scale_grad, gs.numpy(), rtol=1e-4, atol=2e-5)
        np.testing.assert_allclose(u.bias_grad, gb.numpy(), rtol=1e-4, atol=2e-5)
    # a second backward accumulates the parameter gradients (beta = 1) until reset()
    g1 = op.units[0].grad_weights.copy()
    op.out_delta = dy.copy()
    op.backward(True)
    np.testing.assert_allclose(op.units[0].grad_weights, 2 * g1, rtol=1e-5, atol=1e-6)
    op.p.reset()
    assert not op.units[0].grad_weights.any() and not op.units[0].scale_grad.any()
    # weight decay reaches the filters only
    op.p.regularize(0.5)
    np.testing.assert_allclose(op.units[0].grad_weights, 0.5 * op.units[0].weights, rtol=1e-6)
    assert not op.units[0].scale_grad.any() and not op.units[0].bias_grad.any()


def test_preproc_and_dropout_restatements():
    rng = np.random.default_rng(11)
    x = rng.standard_normal((3, 3, 9, 8)).astype(np.float32)
    xt = torch.from_numpy(x)
    assert np.array_equal(O.crop_nchw(x, 5, 4, 2, 3), xt[:, :, 3:7, 2:7].numpy())
    assert np.array_equal(O.flip_x(x), torch.flip(xt, dims=[3]).numpy())
    mean = rng.standard_normal((3, 9, 8)).astype(np.float32)
    np.testing.assert_allclose(O.subtract_mean(x, mean, False), x - mean[None], rtol=0, atol=1e-7)
    np.testing.assert_allclose(O.subtract_mean(x, mean, True), x - mean[None] / 255.0, rtol=0, atol=1e-6)
    alphas, svals, svecs = (rng.standard_normal(9).astype(np.float32), rng.random(3).astype(np.float32),
                            rng.standard_normal(9).astype(np.float32))
    want = x.astype(np.float64).copy()
    for n in range(3):
        for c in range(3):
            want[n, c] += sum(float(svecs[j * 3 + c]) * float(alphas[n * 3 + j]) * float(svals[j]) for j in range(3))
    np.testing.assert_allclose(O.pca3_noise(x, alphas, svals, svecs), want, rtol=1e-6, atol=1e-6)
    rnd = rng.random(x.shape).astype(np.float32)
    y, mask = O.dropout(x, 0.5, 1.0, rnd)
    assert mask.sum() == (rnd > 0.5).sum() and np.array_equal(y, np.where(rnd > 0.5, x, 0).astype(np.float32))
    # backward is the adjoint of forward for a fixed mask
    dy = rng.standard_normal(x.shape).astype(np.float32)
    lhs = float((y.astype(np.float64) * dy).sum())
    rhs = float((x.astype(np.float64) * O.dropout_backprop(dy, 1.0, mask)).sum())
    assert abs(lhs - rhs) < 1e-9 * max(1.0, abs(lhs))


def test_second_generation_update_is_torch_sgd_with_the_velocity_in_the_gradient_buffer():
    """The gen-2 rule (backward accumulates unnormalised sums with per-sample weights 1; descend: g += l2*W,
    W -= (eta/m)*g; reset_gradients: g *= mu) keeps buf_t = mu*buf_{t-1} + grad_t + l2*W_{t-1}, i.e. with b = buf/m it
    is torch.optim.SGD(lr=eta, momentum=mu, weight_decay=l2/m, dampening=0) on the mean loss.  Checked on a whole
    conv -> pool -> affine -> affine chain over 4 minibatches of 2 micro-batches each (weights, biases and the
    accumulated device-side loss), against torch autograd in fp64.  A dropped l2 term, a wrong sign, the factor m in
    the wrong place or momentum applied to the wrong buffer all fail it."""
    from oracle import graph as OG
    from rembrandt_amd import configs
    dims = (8, 8, 2)
    layers, ncat = configs._chain(dims, [("conv", 3, 1, 1, 4, "Rect"), ("pool", 2, 2, 0, "Max"), ("fc", 12, "Rect"),
                                         ("fc", 5, "Identity")])
    batch, micro, m = 6, 2, 12
    eta, mu, l2 = 0.3, 0.8, 0.02
    arch = OG.SequentialOperatorWorker(layers, ncat, batch)
    params = []
    for op in arch.hidden:
        if op.p is not None:
            op.p.weights[...] = rnd(*op.p.weights.shape) * 0.3
            op.p.bias[...] = rnd(*op.p.bias.shape) * 0.1
            params += [torch.tensor(op.p.weights.astype(np.float64), requires_grad=True),
                       torch.tensor(op.p.bias.astype(np.float64), requires_grad=True)]
    cw, cb, w1, b1, w2, b2 = params
    topt = torch.optim.SGD(params, lr=eta, momentum=mu, weight_decay=l2 / m)
    sgd = OG.SgdOptimization(m, eta, mu, l2)
    sgd.begin(arch)
    for t in range(4):
        topt.zero_grad()
        total = 0.0
        for k in range(micro):
            x, labels = rnd(batch, 2, 8, 8), np.random.default_rng(100 * t + k).integers(0, ncat, batch).astype(np.int32)
            arch.stage_batch(labels, 1.0)
            sgd.batch(arch, x)
            h = F.max_pool2d(torch.relu(F.conv2d(torch.tensor(x.astype(np.float64)), cw, cb, padding=1)), 2)
            h = torch.relu(h.reshape(batch, -1) @ w1.T + b1) @ w2.T + b2
            loss = F.cross_entropy(h, torch.tensor(labels.astype(np.int64)), reduction="sum")
            (loss / m).backward()
            total += float(loss.detach())
        np.testing.assert_allclose(arch.acc_loss[0], total, rtol=1e-5)
        arch.reset_loss()
        sgd.end_minibatch(arch)
        topt.step()
        got = [a for op in arch.hidden if op.p is not None for a in (op.p.weights, op.p.bias)]
        for a, b in zip(got, params):
            np.testing.assert_allclose(a, b.detach().numpy(), rtol=2e-4, atol=2e-6)
    assert sgd.t == 4
    # the velocity lives in the gradient buffers: after reset_gradients they hold mu * m * (torch's momentum buffer)
    for a, b in zip([a for op in arch.hidden if op.p is not None for a in (op.p.grad_weights, op.p.grad_bias)], params):
        np.testing.assert_allclose(a, mu * m * topt.state[b]["momentum_buffer"].numpy(), rtol=2e-4, atol=2e-5)


def test_second_generation_backward_scale_reaches_convolutions_only():
    """backward(batch, scale): a convolution accumulates scale * (filter, bias) gradients (layer_new.rs:1093-1108), an
    affine layer accumulates with factor 1 whatever the scale (layer_new.rs:583-584), deltas are not scaled."""
    from oracle import graph as OG
    from rembrandt_amd import configs
    dims = (6, 6, 3)
    layers, ncat = configs._chain(dims, [("conv", 3, 1, 0, 4, "Rect"), ("fc", 5, "Identity")])
    batch = 4
    x, labels = rnd(batch, 3, 6, 6), np.array([0, 3, 1, 4], np.int32)
    grads = {}
    for scale in (1.0, 0.25):
        arch = OG.SequentialOperatorWorker(layers, ncat, batch)
        for i, op in enumerate(arch.hidden):
            op.p.weights[...] = np.random.default_rng(i).standard_normal(op.p.weights.shape).astype(np.float32) * 0.3
            op.p.grad_weights[...] = 1.0    # beta = 1: what is there stays
        arch.stage_batch(labels, 1.0)
        arch.forward(x)
        arch.backward_scaled(scale)
        grads[scale] = [(op.p.grad_weights.copy(), op.p.grad_bias.copy(), op.out_delta.copy()) for op in arch.hidden]
    (cw1, cb1, cd1), (aw1, ab1, ad1) = grads[1.0]
    (cw2, cb2, cd2), (aw2, ab2, ad2) = grads[0.25]
    np.testing.assert_allclose(cw2 - 1.0, 0.25 * (cw1 - 1.0), rtol=1e-5, atol=1e-7)
    np.testing.assert_allclose(cb2, 0.25 * cb1, rtol=1e-5, atol=1e-7)
    np.testing.assert_array_equal(aw2, aw1)
    np.testing.assert_array_equal(ab2, ab1)
    np.testing.assert_array_equal(cd2, cd1)
    np.testing.assert_array_equal(ad2, ad1)
    assert np.abs(cw1 - 1.0).max() > 1e-3


@pytest.mark.parametrize("flavour", ["Update", "UpdateNesterov"])
def test_train_loop_restatement_against_a_torch_training_loop(flavour):
    """oracle.graph.sgd_train / sgd_validate (SgdOpt::train, ::validate) against an independent torch loop: minibatches
    of two batches with per-sample weight 1/minibatch (= the mean loss), epochs that restart at sample 0, the trace's
    step rows (loss at the parameters before the update, error rate), validation rows every second checkpoint on the
    *plain* parameters (for UpdateNesterov the stored ones carry the look-ahead mu*v, un-applied around the checkpoint
    block), a last partial validation batch, Discard checkpoints that must leave the trajectory alone, and the final
    parameters.  Update{mu} at constant step is torch SGD(momentum); UpdateNesterov's stored parameters follow torch
    SGD(nesterov=True), its plain parameters are those plus eta*mu*b."""
    from oracle import graph as OG
    from rembrandt_amd import configs
    dims = (6, 6, 1)
    layers, ncat = configs._chain(dims, [("conv", 3, 1, 1, 4, "Rect"), ("pool", 2, 2, 0, "Average"), ("fc", 5, "Identity")])
    batch, minibatch, iters = 4, 8, 7
    eta, mu, l2 = 0.2, 0.7, 1e-2
    rng = np.random.default_rng(3)
    frames = (rng.integers(0, 256, (24, 1, 6, 6)).astype(np.float32) / np.float32(255.0))
    labels = rng.integers(0, ncat, 24).astype(np.int32)
    vframes = (rng.integers(0, 256, (10, 1, 6, 6)).astype(np.float32) / np.float32(255.0))
    vlabels = rng.integers(0, ncat, 10).astype(np.int32)
    arch = OG.SequentialOperatorWorker(layers, ncat, batch)
    params = []
    for op in arch.hidden:
        if op.p is not None:
            op.p.weights[...] = rnd(*op.p.weights.shape) * 0.4
            params += [torch.tensor(op.p.weights.astype(np.float64), requires_grad=True),
                       torch.tensor(op.p.bias.astype(np.float64), requires_grad=True)]
    cw, cb, w1, b1 = params

    def net(x, ps):
        cw_, cb_, w1_, b1_ = ps
        h = F.avg_pool2d(torch.relu(F.conv2d(torch.tensor(x.astype(np.float64)), cw_, cb_, padding=1)), 2)
        return h.reshape(len(x), -1) @ w1_.T + b1_

    rows = OG.sgd_train(OG.SgdOpt(eta, (flavour, mu), l2), arch, frames, labels, minibatch, iters, checkpoint_iters=2,
                        checkpoint_discard=True, valid=(vframes, vlabels), valid_iters=4)
    topt = torch.optim.SGD(params, lr=eta, momentum=mu, weight_decay=l2, nesterov=flavour == "UpdateNesterov")
    want, pos = [], 0
    for it in range(1, iters + 1):
        idx = [(pos + i) % 24 for i in range(minibatch)]
        pos = (pos + minibatch) % 24
        topt.zero_grad()
        logits = net(frames[idx], params)
        loss = F.cross_entropy(logits, torch.tensor(labels[idx].astype(np.int64)))
        loss.backward()
        err = 1.0 - float((logits.argmax(1).numpy() == labels[idx]).mean())
        want.append((it, "step", float(loss.detach()), err))
        topt.step()
        if it % 4 == 0:
            plain = params
            if flavour == "UpdateNesterov":
                plain = [p.detach() + eta * mu * topt.state[p]["momentum_buffer"] for p in params]
            with torch.no_grad():
                vl = net(vframes, plain)
                want.append((it, "valid", float(F.cross_entropy(vl, torch.tensor(vlabels.astype(np.int64)))),
                             1.0 - float((vl.argmax(1).numpy() == vlabels).mean())))
    assert [(r[0], r[1]) for r in rows] == [(r[0], r[1]) for r in want]
    for got, ref in zip(rows, want):
        np.testing.assert_allclose(got[2], ref[2], rtol=2e-5, err_msg=str(ref[:2]))
        assert abs(got[3] - ref[3]) < 1e-9, (got, ref)
    got = [a for op in arch.hidden if op.p is not None for a in (op.p.weights, op.p.bias)]
    for a, b in zip(got, params):
        np.testing.assert_allclose(a, b.detach().numpy(), rtol=2e-4, atol=2e-6)
