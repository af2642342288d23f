"""The entry point that allocates nothing, rh_conv2d_bwd_bias_noalloc: same results as rh_conv2d_bwd_bias_ws (bit for
bit: same kernels, same order of additions) and as the oracle, on two calls in a row of which the second is smaller
(the library's static scratch array keeps the first call's contents), for both forms of the reduction, then again
after other work; and the documented refusal beyond the array's size."""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle as O
from rembrandt_amd import _lib, ops, synth
from conftest import assert_close, say

pytestmark = pytest.mark.gpu


def noalloc_bias(dy, alpha=1.0, beta=0.0, db=None):
    N, K = dy.shape[0], dy.shape[1]
    plane = dy[0, 0].numel()
    if db is None:
        db = torch.zeros(K, dtype=torch.float32, device=dy.device)
    _lib.check(_lib.lib().rh_conv2d_bwd_bias_noalloc(N, K, plane, alpha, C.c_void_p(dy.data_ptr()), beta,
                                                    C.c_void_p(db.data_ptr()),
                                                    C.c_void_p(torch.cuda.current_stream().cuda_stream)),
               "rh_conv2d_bwd_bias_noalloc")
    return db


# (N, K, P, Q): column form (planes under 1024 elements), row form (larger planes), an affine layer (plane 1, no scratch).
# Inputs of more than 2^20 elements with planes of more than one element take the two-stage reduction over the scratch
# array; the second call of the first four pairs does too, over what the first one left there, in the same form and in
# the other one.
PAIRS = [((256, 256, 27, 27), (40, 256, 27, 27)),     # column form after column form
         ((64, 96, 55, 55), (40, 256, 27, 27)),       # column form after row form
         ((256, 384, 13, 13), (64, 64, 56, 56)),      # row form after column form
         ((64, 96, 55, 55), (24, 20, 57, 57)),        # row form after row form
         ((256, 256, 27, 27), (37, 96, 13, 13)),      # a one-stage call (no scratch) after a two-stage one
         ((128, 1000, 1, 1), (3, 7, 1, 1))]


@pytest.mark.parametrize("first,second", PAIRS, ids=[str(p) for p in PAIRS])
def test_noalloc_bias_gradient_matches_workspace_form(dev, first, second):
    lib = _lib.lib()
    assert lib.rh_noalloc_scratch_bytes() == 8 << 20
    other = torch.randn(1 << 20, device=dev)
    if PAIRS.index((first, second)) < 4:   # both calls run the two-stage reduction over the static array
        assert all(lib.rh_conv2d_bwd_bias_workspace_bytes(s[0], s[1], s[2] * s[3]) > 0 for s in (first, second))
    for shape in (first, second):
        say("no-alloc bias gradient", shape)
        N, K, P, Q = shape
        assert lib.rh_conv2d_bwd_bias_workspace_bytes(N, K, P * Q) <= lib.rh_noalloc_scratch_bytes()
        ops.rect_inplace(other)    # unrelated work of the library between the calls
        dy = synth.normal(41, N + K, shape)
        db0 = synth.normal(41, 7, (K,))
        dyd = torch.from_numpy(dy).to(dev)
        for alpha, beta in ((1.0, 0.0), (0.5, 1.0)):
            want = ops.conv2d_bwd_bias(dyd, alpha=alpha, beta=beta, db=torch.from_numpy(db0).to(dev), two_stage=True)
            got = noalloc_bias(dyd, alpha=alpha, beta=beta, db=torch.from_numpy(db0).to(dev))
            assert torch.equal(got, want), "same kernels, same scratch layout: bit-identical"
            assert_close(got.cpu().numpy(), O.conv2d_bwd_bias(dy, alpha, beta, db0.copy()), "no-alloc bias gradient %s" % (shape,))
    torch.cuda.synchronize()


def test_noalloc_refuses_what_does_not_fit(dev):
    lib = _lib.lib()
    N, K, plane = 4, 4096, 1000            # one group of K*plane partial sums: 16.4 MB of scratch
    assert lib.rh_conv2d_bwd_bias_workspace_bytes(N, K, plane) > lib.rh_noalloc_scratch_bytes()
    dy = torch.zeros((N, K, plane), dtype=torch.float32, device=dev)
    db = torch.zeros(K, dtype=torch.float32, device=dev)
    rc = lib.rh_conv2d_bwd_bias_noalloc(N, K, plane, 1.0, C.c_void_p(dy.data_ptr()), 0.0, C.c_void_p(db.data_ptr()), None)
    assert rc == _lib.RH_E_LIMIT
    assert lib.rh_conv2d_bwd_bias_noalloc(0, K, plane, 1.0, C.c_void_p(dy.data_ptr()), 0.0, C.c_void_p(db.data_ptr()), None) \
        == _lib.RH_E_INVALID
    torch.cuda.synchronize()
