"""GPU parity of repeat_back (OP_REPEAT_BACK, src/backend/CPUKernels.cpp:2091-2148) against the CPU oracle.

Bar: equality where every partial sum is exact (small integers), otherwise 1e-4 relative to sum |terms|: the
reference adds a destination element's copies one at a time, the kernel adds consecutive runs of that sequence
side by side and then the runs in order.
"""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


@pytest.fixture(scope="module")
def ops():
    from proteinpredictmachinelearning_amd import ops as _ops

    return _ops


def _dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("src_shape,dst_shape", [
    ((37, 19), (19,)),                    # bias gradient: grad [N=19, M=37] -> [19]
    ((2, 4, 3, 5), (1, 4, 1, 5)),         # same rank, two broadcast dimensions
    ((4, 6), (4, 3)),                     # a dimension kept and repeated at once
    ((4, 6), (4, 6)),                     # nothing repeated: a copy
    ((3, 5, 7), (1, 1, 1)),               # everything into one element
    ((7, 5, 3, 2), (3, 2)),               # leading source dimensions summed away
    ((26368, 768), (768,)),               # the MSA QKV projection's bias gradient: runs + fold
    ((10609, 128), (128,)),
    ((300, 1, 64), (1, 64)),
])
def test_exact_on_small_integers(ops, oracle, src_shape, dst_shape):
    rng = np.random.default_rng(sum(src_shape))
    a = rng.integers(-4, 5, size=src_shape).astype(np.float32)
    got = ops.repeat_back(_dev(a), dst_shape).cpu().numpy()
    want = oracle.repeat_back(a, dst_shape)
    assert got.shape == want.shape
    assert (got == want).all()


@pytest.mark.parametrize("src_shape,dst_shape", [((26368, 768), (768,)), ((64, 103, 103, 8), (1, 103, 1, 8)), ((5000, 3), (3,))])
def test_within_the_f32_bar_on_normal_draws(ops, oracle, src_shape, dst_shape):
    rng = np.random.default_rng(7)
    a = rng.standard_normal(src_shape).astype(np.float32)
    got = ops.repeat_back(_dev(a), dst_shape).cpu().numpy().astype(np.float64)
    want = oracle.repeat_back(a, dst_shape).astype(np.float64)
    pad = (1,) * (a.ndim - len(dst_shape)) + tuple(dst_shape)
    axes = tuple(i for i in range(a.ndim) if pad[i] == 1 and a.shape[i] > 1)
    exact = a.astype(np.float64).sum(axis=axes).reshape(dst_shape)
    mass = np.abs(a).astype(np.float64).sum(axis=axes).reshape(dst_shape)
    assert (np.abs(got - want) <= 1e-4 * mass).all()
    # and it is at least as close to the exact sum as the sequential sum is allowed to be
    n_terms = a.size // int(np.prod(dst_shape))
    assert (np.abs(got - exact) <= n_terms * 2.0 ** -24 * mass).all()


def test_bad_arguments(ops):
    from proteinpredictmachinelearning_amd import cabi
    lib = cabi.load()
    buf = torch.zeros(64, device="cuda")
    p = C.c_void_p(buf.data_ptr())
    ok = [8, 8, 1, 1, 8, 1, 1, 1, 1, 8, 1, 1]
    assert lib.repeat_back_hip(p, p, *ok, None) == 0
    assert lib.repeat_back_hip(None, p, *ok, None) == 1
    outside = [8, 8, 1, 1, 8, 1, 1, 1, 1, 9, 1, 1]            # nine copies of a dimension that holds eight
    assert lib.repeat_back_hip(p, p, *outside, None) == 1
    assert b"repeat_back_hip" in lib.ppml_hip_last_error()
    with pytest.raises(ValueError):
        ops.repeat_back(torch.zeros(2, 2, 2, 2, 2, device="cuda"), (2,))


def test_sizes_whose_products_would_wrap_are_refused(ops):
    """r * d computed in 64 bits wraps for sizes near 2^63 and would pass a product test; the launcher compares
    quotients and refuses (nothing is launched, the operands are never read)."""
    import ctypes as C
    lib = ops._lib()
    x = torch.zeros(16, device="cuda")
    p = C.c_void_p(x.data_ptr())
    big = 1 << 62
    # copies x destination size = 2^62 * 4 = 2^64 -> 0 in 64 bits, "inside" a source of 16
    assert lib.repeat_back_hip(p, p, 16, 1, 1, 1, 4, 1, 1, 1, big, 1, 1, 1, None) == 1
    # destination sizes whose product wraps
    assert lib.repeat_back_hip(p, p, big, big, 4, 1, big, big, 4, 1, 1, 1, 1, 1, None) == 1
    # a plain case still runs
    assert lib.repeat_back_hip(p, p, 16, 1, 1, 1, 4, 1, 1, 1, 4, 1, 1, 1, None) == 0
