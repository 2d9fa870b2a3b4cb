"""The MUL_MAT statistics on the device (include/ppml/MulMatStats.h:39-169; event timing as
src/cuda/CUDAKernels.cu:1693-1732): calls and milliseconds per (path, M, K, N)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


def test_calls_and_milliseconds_per_shape(oracle, capfd):
    from proteinpredictmachinelearning_amd import cabi, ops

    lib = cabi.load()
    g = torch.Generator(device="cuda").manual_seed(1)
    x = torch.randn(408, 256, device="cuda", generator=g)
    w = torch.randn(256, 256, device="cuda", generator=g) * 0.02
    W = ops.Q8Weight.from_f32(w)
    Wp = W.pack()
    big = torch.randn(1 << 21, 32, device="cuda", generator=g)          # 2^21 rows: beyond the reference's 20-bit key
    small = torch.randn(8, 32, device="cuda", generator=g)
    ops.mul_mat(x, w)                                                   # not counted: statistics are off
    before = ops.mulmat_stats_enable(True)
    try:
        lib.ppml_hip_mulmat_stats_reset()
        for _ in range(3):
            ops.mul_mat_q8(Wp, x)                                       # 408 tokens: the low-latency kernel
        ops.mul_mat_q8(Wp, x, path="weight-stationary")
        ops.mul_mat_q8(W, x)
        for _ in range(2):
            ops.mul_mat(x, w)
        ops.mul_mat(big, small)
        rows = {(r["path"], r["M"], r["K"], r["N"]): r for r in ops.mulmat_stats_rows()}
        assert set(rows) == {("hip/q8-low-latency", 256, 256, 408), ("hip/q8-weight-stationary", 256, 256, 408),
                             ("hip/q8-general", 256, 256, 408), ("hip/mul_mat", 408, 256, 256), ("hip/mul_mat", 1 << 21, 32, 8)}
        assert rows[("hip/q8-low-latency", 256, 256, 408)]["calls"] == 3
        assert rows[("hip/q8-weight-stationary", 256, 256, 408)]["calls"] == 1
        assert rows[("hip/q8-general", 256, 256, 408)]["calls"] == 1
        assert rows[("hip/mul_mat", 408, 256, 256)]["calls"] == 2
        for r in rows.values():
            assert 0.0 < r["ms"] < 200.0, r                              # every call was timed, none absurdly
        # three launches of a microsecond-scale kernel cost less than one contraction over 2^21 rows
        assert rows[("hip/q8-low-latency", 256, 256, 408)]["ms"] < rows[("hip/mul_mat", 1 << 21, 32, 8)]["ms"]
        # the shape table sums over the paths and keeps whole dimensions
        buf = (np.zeros(4 * 8, dtype=np.int64))
        import ctypes as C
        n = lib.ppml_hip_mulmat_stats(buf.ctypes.data_as(C.POINTER(C.c_int64)), 8)
        shapes = {tuple(buf[4 * i:4 * i + 3]): buf[4 * i + 3] for i in range(n)}
        assert shapes == {(256, 256, 408): 5, (408, 256, 256): 2, (1 << 21, 32, 8): 1}
        capfd.readouterr()
        lib.ppml_hip_mulmat_stats_dump()
        text = capfd.readouterr().err
        assert "[MULMAT-STAT]" in text and "total calls=8" in text and "hip/q8-weight-stationary" in text and "hip/q8-low-latency" in text
        assert "M=2097152" in text
        lib.ppml_hip_mulmat_stats_reset()
        assert ops.mulmat_stats_rows() == []
    finally:
        ops.mulmat_stats_enable(before)
    ops.mul_mat(x, w)
    assert ops.mulmat_stats_rows() == []
