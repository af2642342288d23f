import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def assert_close(got, ref, what, rtol=1e-4, atol=1e-5, scale_atol=True):
    """fp32 parity bound |got - ref| <= atol' + rtol*|ref| against the fp64-accumulated oracle.

    atol' = atol * max(1, rms(ref)): an absolute 1e-5 is below the fp32 resolution of the partial
    sums once a tensor's values reach the tens (N(0,1) x N(0,1) contractions of depth ~2400), so
    the absolute term follows the tensor's scale; for unit-scale tensors it is exactly 1e-5.
    """
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape, "%s: shape %s vs %s" % (what, got.shape, ref.shape)
    assert np.isfinite(got).all(), "%s: non-finite values in result" % what
    a = atol
    if scale_atol and ref.size:
        a = atol * max(1.0, float(np.sqrt(np.mean(ref * ref))))
    err = np.abs(got - ref)
    # tensors far below unit scale (gradients ~1e-4) would pass the absolute term vacuously:
    # they must also agree to 1e-4 in relative L2 norm
    ref_norm = float(np.sqrt(np.sum(ref * ref)))
    if ref_norm > 0.0:
        rel_l2 = float(np.sqrt(np.sum(err * err))) / ref_norm
        assert rel_l2 <= 1e-4, "%s: relative L2 error %.3g > 1e-4" % (what, rel_l2)
    bound = a + rtol * np.abs(ref)
    bad = err > bound
    if bad.any():
        i = int(np.argmax(err - bound))
        raise AssertionError("%s: %d of %d elements out of tolerance; worst at flat %d: got %r ref %r (atol %g rtol %g)"
                             % (what, int(bad.sum()), err.size, i, got.ravel()[i], ref.ravel()[i], a, rtol))


@pytest.fixture(scope="session")
def dev():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


def say(*a):
    print(*a, flush=True)
