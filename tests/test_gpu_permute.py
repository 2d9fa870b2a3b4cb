"""GPU parity of the permutation copy (permute_hip) against the CPU oracle: byte movement, so equality."""
import itertools

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


@pytest.fixture(scope="module")
def ops():
    assert torch.cuda.is_available(), "GPU tests need a device"
    from proteinpredictmachinelearning_amd import ops as _ops

    return _ops


def _run(ops, x, axes):
    out = ops.permute(torch.from_numpy(x).cuda(), axes)
    ops.synchronize()
    return out.cpu().numpy()


def test_every_permutation_of_small_tensors(ops, oracle):
    rng = np.random.default_rng(2)
    x4 = rng.standard_normal((3, 5, 70, 66)).astype(np.float32)       # reference dims [66, 70, 5, 3]: ragged 64-tiles
    for axes in itertools.permutations(range(4)):
        assert np.array_equal(_run(ops, x4, axes), oracle.permute(x4, axes)), axes
    x3 = rng.standard_normal((4, 33, 8)).astype(np.float32)          # rows of 8: the 16-byte row copy
    for axes in itertools.permutations(range(3)):
        assert np.array_equal(_run(ops, x3, axes), oracle.permute(x3, axes)), axes
    x2 = rng.standard_normal((129, 65)).astype(np.float32)
    assert np.array_equal(_run(ops, x2, (1, 0)), x2.T)
    x1 = rng.standard_normal(7).astype(np.float32)
    assert np.array_equal(_run(ops, x1, (0,)), x1)


def test_the_attention_bridges_at_the_configured_size(ops):
    """[L, D, h, B] <-> [D, L, h, B] (ComputeGraphHelper.cpp:450-484) at L 256, D 32, h 8, B 103: the
    round trip is the identity and the bridge equals torch's transpose."""
    g = torch.Generator(device="cuda").manual_seed(7)
    x = torch.randn(103, 8, 32, 256, device="cuda", generator=g)     # reference dims [256, 32, 8, 103]
    y = ops.permute(x, (1, 0, 2, 3))
    assert tuple(y.shape) == (103, 8, 256, 32)
    assert torch.equal(y, x.transpose(2, 3).contiguous())
    assert torch.equal(ops.permute(y, (1, 0, 2, 3)), x)
    # more planes than one grid dimension holds
    z = torch.randn(70000, 1, 3, 5, device="cuda", generator=g)
    assert torch.equal(ops.permute(z, (1, 0, 2, 3)), z.transpose(2, 3).contiguous())


def test_refused_arguments(ops):
    from proteinpredictmachinelearning_amd import cabi

    lib = cabi.load()
    x = torch.zeros(24, device="cuda")
    p = x.data_ptr()
    ok = lambda *a: lib.permute_hip(p, p, *a, None)   # noqa: E731
    assert ok(24, 3, 1, 0, 2, 3, 4, 3, 2, 1, 3, 4, 2, 1) == 0
    assert ok(24, 3, 1, 1, 2, 3, 4, 3, 2, 1, 3, 3, 2, 1) == 1       # an axis twice
    assert ok(24, 3, 3, 0, 2, 3, 4, 3, 2, 1, 3, 4, 2, 1) == 1       # axis outside the tensor (CUDAKernels.cpp:1376-1381)
    assert ok(24, 3, 1, 0, 2, 3, 4, 3, 2, 1, 4, 3, 2, 1) == 1       # destination sizes do not follow the axes
    assert ok(25, 3, 1, 0, 2, 3, 4, 3, 2, 1, 3, 4, 2, 1) == 1       # total is not the product
    assert lib.permute_hip(None, p, 24, 3, 1, 0, 2, 3, 4, 3, 2, 1, 3, 4, 2, 1, None) == 1
