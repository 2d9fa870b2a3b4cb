"""Pins the CPU oracle before anything is compared against it.

Each check is chosen so that a plausible mistake in the restatement (dropped term, wrong sign or
index, transposed operand, wrong rounding mode) fails: the reference's own test inputs and known
answers where it holds them, the reference's HalfUtils.h compiled as-is where that was built, and
otherwise closed forms, invariants, library special cases and brute force on small inputs.
"""
import ctypes as C

import numpy as np
import pytest


# ----------------------------------------------------------------------------- fp16
def _interesting_floats():
    rng = np.random.default_rng(7)
    bits = [0x00000000, 0x80000000, 0x33000000, 0x33000001, 0x32ffffff, 0x33800000, 0x387fe000,
            0x387fffff, 0x38800000, 0x38801000, 0x38800fff, 0x38801001, 0x477fe000, 0x477fefff,
            0x477ff000, 0x477fffff, 0x47800000, 0x7f7fffff, 0x7f800000, 0xff800000, 0x7fc00000,
            0xffc00001, 0x3f800000, 0x3f801000, 0x3f803000, 0x3f802fff, 0x3a9ff000]
    rnd = rng.integers(0, 2**32, size=200000, dtype=np.uint64).astype(np.uint32)
    # dense coverage of the half range incl. subnormals and ties
    ties = (np.arange(0, 0x7c00, dtype=np.uint32) << 13) + 0x38000000
    return np.concatenate([np.array(bits, dtype=np.uint32), rnd, ties, ties + 0x1000, ties + 0x0fff,
                           ties + 0x1001])


def test_fp32_to_fp16_matches_numpy(oracle):
    u = _interesting_floats()
    f = u.view(np.float32)
    with np.errstate(over="ignore", invalid="ignore"):
        want = f.astype(np.float16).view(np.uint16)
    got = np.array([oracle.fp32_to_fp16(float(x)) if not np.isnan(x) else 0 for x in f], dtype=np.uint16)
    ok = np.isnan(f) | (got == want)
    assert ok.all(), (hex(int(u[~ok][0])), hex(int(got[~ok][0])), hex(int(want[~ok][0])))
    # NaN keeps its sign and becomes the quiet pattern (HalfUtils.h:51)
    assert oracle.lib().orc_fp32_to_fp16(C.c_float(float("nan"))) & 0x7fff == 0x7e00


def test_fp16_to_fp32_all_patterns(oracle):
    h = np.arange(65536, dtype=np.uint16)
    want = h.view(np.float16).astype(np.float32)
    got = np.array([oracle.fp16_to_fp32(int(x)) for x in h], dtype=np.float32)
    nan = np.isnan(want)
    assert (np.isnan(got) == nan).all()
    assert (got.view(np.uint32)[~nan] == want.view(np.uint32)[~nan]).all()


def test_fp16_against_compiled_reference(oracle):
    ref = oracle.ref_half_lib()
    if ref is None:
        pytest.skip("oracle/_ref was not built (reference tree absent at build time)")
    for h in range(65536):
        a, b = oracle.fp16_to_fp32(h), ref.ref_fp16_to_fp32(h)
        assert (a != a and b != b) or np.float32(a).view(np.uint32) == np.float32(b).view(np.uint32), hex(h)
    fn = C.cast(oracle.lib().orc_fp32_to_fp16, C.c_void_p)
    first = C.c_uint32(0)
    # every 251st binary32 pattern (17M values) plus two offset sweeps around the tie patterns
    for start, stride in ((0, 251), (0x1000, 0x2000), (0x0fff, 0x2000), (0x1001, 0x2000)):
        bad = ref.ref_sweep_fp32_to_fp16(fn, start, stride, C.byref(first))
        assert bad == 0, (bad, hex(first.value))


# ----------------------------------------------------------------------------- quantize
def test_quantize_hand_checked_vector(oracle):
    x = (0.01 * (np.arange(32, dtype=np.float64) - 15.5)).astype(np.float32)
    blk = oracle.quantize_q8_0(x)
    assert blk.shape == (1, 34)
    assert int(oracle.block_scales_bits(blk)[0]) == 0x1500
    q = oracle.block_quants(blk)[0]
    assert q[0] == -127 and q[31] == 127
    # symmetric ramp: q is odd-symmetric and monotone
    assert (q == -q[::-1]).all() and (np.diff(q.astype(int)) >= 0).all()


def test_quantize_zero_block_and_rejects_ragged(oracle):
    blk = oracle.quantize_q8_0(np.zeros(64, dtype=np.float32))
    assert (blk == 0).all()                      # d = +0 and q = 0 (QuantBlocks.h:70)
    with pytest.raises(ValueError):
        oracle.quantize_q8_0(np.zeros(33, dtype=np.float32))
    x = np.zeros(31, dtype=np.float32)
    out = np.zeros(34, dtype=np.uint8)
    rc = oracle.lib().orc_quantize_q8_0(x.ctypes.data_as(C.POINTER(C.c_float)), out.ctypes.data_as(C.c_void_p), 31)
    assert rc == 1


def test_quantize_invariants_and_independent_rounding(oracle):
    rng = np.random.default_rng(1)
    x = np.concatenate([
        rng.standard_normal(32 * 2000).astype(np.float32),
        (rng.standard_normal(32 * 500) * 0.02).astype(np.float32),
        (rng.standard_normal(32 * 500) * 1e-6).astype(np.float32),
        (rng.standard_normal(32 * 100) * 1e4).astype(np.float32),
    ]).reshape(-1, 32)
    blk = oracle.quantize_q8_0(x)[:, 0, :]
    q = oracle.block_quants(blk).astype(np.int64)
    dbits = oracle.block_scales_bits(blk)
    amax = np.abs(x).max(axis=1)
    # scale: fp16(RNE) of the binary32 quotient amax/127 -- numpy's own division and half rounding
    d32 = (amax / np.float32(127.0)).astype(np.float32)
    assert (dbits == d32.astype(np.float16).view(np.uint16)).all()
    # the arg-max element maps to +-127, nothing leaves [-127,127]
    arg = np.abs(x).argmax(axis=1)
    rows = np.arange(x.shape[0])
    assert (np.abs(q[rows, arg]) == 127).all()
    assert (np.sign(q[rows, arg]) == np.sign(x[rows, arg])).all()
    assert q.min() >= -127 and q.max() <= 127
    # reconstruction error is at most half a step of the f32 scale
    err = np.abs(x.astype(np.float64) - d32[:, None].astype(np.float64) * q)
    assert (err <= 0.5 * d32[:, None].astype(np.float64) * (1 + 1e-5)).all()
    # independent statement in float64: q = round-half-away(x / d); may differ from the binary32
    # product x*(1/d) only when the exact quotient sits on a rounding boundary
    t = x.astype(np.float64) / d32[:, None].astype(np.float64)
    want = np.sign(t) * np.floor(np.abs(t) + 0.5)
    want = np.clip(want, -127, 127).astype(np.int64)
    diff = want != q
    frac = np.abs(np.abs(t) - np.floor(np.abs(t)) - 0.5)
    assert (frac[diff] < 2e-5).all() and diff.mean() < 1e-4


def test_quantize_ties_round_away_from_zero(oracle):
    # amax = 127 -> d = 1, inv = 1: the quantizer is round() itself
    x = np.zeros(32, dtype=np.float32)
    x[0] = 127.0
    x[1:9] = [0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 0.49999997, -0.49999997]
    q = oracle.block_quants(oracle.quantize_q8_0(x))[0]
    assert list(q[:9]) == [127, 1, -1, 2, -2, 3, -3, 0, 0]


def test_quantize_ignores_nan_in_absmax(oracle):
    # std::fmax drops NaN (QuantBlocks.h:67): the scale comes from the finite elements
    x = np.ones(32, dtype=np.float32)
    x[3] = np.nan
    x[5] = -2.0
    blk = oracle.quantize_q8_0(x)
    assert int(oracle.block_scales_bits(blk)[0]) == int(np.float32(2.0 / 127.0).astype(np.float16).view(np.uint16))
    assert oracle.block_quants(blk)[0][5] == -127


def test_repack_round_trip_and_planes(oracle):
    rng = np.random.default_rng(2)
    blk = oracle.quantize_q8_0(rng.standard_normal((6, 96)).astype(np.float32))
    flat = blk.reshape(-1, 34)
    nb = flat.shape[0]
    packed = oracle.repack_q8_0(flat)
    assert packed.size == nb * 34 == oracle.lib().orc_q8_0_repacked_bytes(nb * 32)
    assert (packed[: nb * 32].reshape(nb, 32) == flat[:, 2:]).all()
    assert (packed[nb * 32:].reshape(nb, 2) == flat[:, :2]).all()
    assert (oracle.unrepack_q8_0(packed) == flat).all()


def test_dequantize_closed_form(oracle):
    rng = np.random.default_rng(3)
    blk = oracle.quantize_q8_0(rng.standard_normal((4, 64)).astype(np.float32))
    d = oracle.block_scales_bits(blk).view(np.float16).astype(np.float32)
    want = (d[..., None] * oracle.block_quants(blk).astype(np.float32)).reshape(4, 64)
    assert (oracle.dequantize_q8_0(blk) == want).all()


# ----------------------------------------------------------------------------- Q8_1 activations
def test_quantize_q8_1_rule(oracle):
    # include/ppml/QuantBlocks.h:81-111: d = vmax / -128 keeps the sign of the largest element,
    # which therefore maps to -128; on equal magnitudes the FIRST element decides the sign;
    # the opposite extreme saturates at +127; s = half(d * sum q) from the binary32 d.
    rng = np.random.default_rng(3)
    x = rng.standard_normal((40, 32)).astype(np.float32)
    x[0] = 0.0                                        # zero block: d = +0, q = 0
    x[1, 5], x[1, 20] = 7.0, -7.0                     # tie: first (+7) wins -> d negative
    x[2, 5], x[2, 20] = -7.0, 7.0                     # tie the other way round -> d positive
    x[1, :5] *= 0.1; x[1, 6:20] *= 0.1; x[1, 21:] *= 0.1
    x[2, :5] *= 0.1; x[2, 6:20] *= 0.1; x[2, 21:] *= 0.1
    blk = oracle.quantize_q8_1(x.reshape(-1)).reshape(40, 36)
    d = np.ascontiguousarray(blk[:, 0:2]).view(np.float16)[:, 0].astype(np.float32)
    s = np.ascontiguousarray(blk[:, 2:4]).view(np.float16)[:, 0]
    q = np.ascontiguousarray(blk[:, 4:]).view(np.int8).astype(np.int32)
    assert (blk[0] == 0).all()
    assert d[1] < 0 and q[1, 5] == -128 and q[1, 20] == 127
    assert d[2] > 0 and q[2, 5] == -128 and q[2, 20] == 127
    for r in range(3, 40):
        i = np.abs(x[r]).argmax()
        assert q[r, i] == -128                         # the extreme element takes the spare code
        d32 = np.float32(x[r, i]) / np.float32(-128.0)
        assert d[r] == np.float32(np.float16(d32))
        # independent float64 statement of the rounding, away from exact ties
        t = x[r].astype(np.float64) / np.float64(d32)
        want = np.clip(np.sign(t) * np.floor(np.abs(t) + 0.5), -128, 127)
        ok = np.abs(np.abs(t) % 1.0 - 0.5) > 1e-4
        assert (q[r][ok] == want[ok]).all()
        assert s[r] == np.float16(d32 * np.float32(q[r].sum()))
        assert np.abs(x[r] - d32 * q[r]).max() <= abs(d32) * (0.5 + 2 ** -10) + (abs(d32) if q[r].max() == 127 else 0)


def test_q8_1_activation_matmul_uses_the_same_settlement(oracle):
    rng = np.random.default_rng(4)
    M, N, K = 7, 5, 96
    w = (rng.standard_normal((M, K)) * 0.02).astype(np.float32)
    x = rng.standard_normal((N, K)).astype(np.float32)
    wq = oracle.quantize_q8_0(w)
    x1 = oracle.quantize_q8_1(x)                                        # [N, nblk, 36]
    as_q8_0 = np.concatenate([x1[..., 0:2], x1[..., 4:]], axis=-1)      # {d, qs}
    want = oracle.mul_mat_q8q8(wq, np.ascontiguousarray(as_q8_0))
    got = oracle.mul_mat_q8_act(wq, x, act=1)
    assert (got.view(np.uint32) == want.view(np.uint32)).all()
    assert (oracle.mul_mat_q8_act(wq, x, act=0) == oracle.mul_mat_q8(wq, x)).all()
    assert (oracle.mul_mat_q8_act(oracle.repack_q8_0(wq), x, act=1, wtype=2) == got).all()
    assert (oracle.mul_mat_q8_act(wq, x, act=1, c_trans=0) == got.T).all()
    full = x.astype(np.float64) @ w.astype(np.float64).T
    assert np.abs(got - full).max() <= 0.02 * np.abs(full).max()


# ----------------------------------------------------------------------------- Q8 dot
def _q8_case(rng, M, N, K):
    w = (rng.standard_normal((M, K)) * 0.02).astype(np.float32)
    x = rng.standard_normal((N, K)).astype(np.float32)
    return w, x


def test_block_sums_brute_force(oracle):
    rng = np.random.default_rng(4)
    w, x = _q8_case(rng, 7, 5, 96)
    wq, xq = oracle.quantize_q8_0(w), oracle.quantize_q8_0(x)
    got = oracle.q8_block_sums(wq, xq)
    want = np.einsum("mbi,nbi->nmb", oracle.block_quants(wq).astype(np.int64), oracle.block_quants(xq).astype(np.int64))
    assert (got == want).all()
    # extreme block: |sum| reaches 32*127*127 without overflow
    hi = np.full((1, 32), 5.0, dtype=np.float32)
    s = oracle.q8_block_sums(oracle.quantize_q8_0(hi), oracle.quantize_q8_0(-hi))
    assert int(s[0, 0, 0]) == -32 * 127 * 127


@pytest.mark.parametrize("c_trans", [0, 1])
def test_q8_matmul_closed_form(oracle, c_trans):
    rng = np.random.default_rng(5)
    M, N, K = 9, 6, 128
    w, x = _q8_case(rng, M, N, K)
    wq, xq = oracle.quantize_q8_0(w), oracle.quantize_q8_0(x)
    sums = oracle.q8_block_sums(wq, xq).astype(np.float64)                 # [N, M, nblk]
    dw = oracle.block_scales_bits(wq).view(np.float16).astype(np.float64)    # [M, nblk]
    da = oracle.block_scales_bits(xq).view(np.float16).astype(np.float64)    # [N, nblk]
    exact = np.einsum("nmb,mb,nb->nm", sums, dw, da)
    for fma in (0, 1):
        got = oracle.mul_mat_q8q8(wq, xq, c_trans=c_trans, fma=fma).astype(np.float64)
        got = got if c_trans else got.T
        assert np.abs(got - exact).max() <= 1e-6 * np.abs(exact).max()
    # special case: equals the f32 GEMM of the dequantised operands up to f32 summation error
    deq = oracle.mul_mat_f32(oracle.dequantize_q8_0(xq), oracle.dequantize_q8_0(wq)).astype(np.float64)
    assert np.abs(deq - exact).max() <= 1e-5 * np.abs(exact).max()
    # and approximates the unquantised product to quantisation accuracy
    full = x.astype(np.float64) @ w.astype(np.float64).T
    assert np.abs(full - exact).max() <= 0.02 * np.abs(full).max()


def test_q8_matmul_end_to_end_and_layouts(oracle):
    rng = np.random.default_rng(6)
    M, N, K = 8, 5, 64
    w, x = _q8_case(rng, M, N, K)
    wq = oracle.quantize_q8_0(w)
    a = oracle.mul_mat_q8(wq, x, wtype=0, c_trans=1)
    b = oracle.mul_mat_q8(oracle.repack_q8_0(wq), x, wtype=2, c_trans=1)
    c = oracle.mul_mat_q8(wq, x, wtype=0, c_trans=0)
    assert (a == b).all() and (a == c.T).all()
    assert (a == oracle.mul_mat_q8q8(wq, oracle.quantize_q8_0(x))).all()
    with pytest.raises(RuntimeError):
        oracle.mul_mat_q8(wq, x, wtype=1)
    # single-block single-output order check: acc = fma(float(sumi), dw*da, 0)
    one = oracle.mul_mat_q8q8(wq[:1, :1], oracle.quantize_q8_0(x)[:1, :1])
    s = int(oracle.q8_block_sums(wq[:1, :1], oracle.quantize_q8_0(x)[:1, :1])[0, 0, 0])
    dw = oracle.block_scales_bits(wq)[0, 0].view(np.float16).astype(np.float32)
    da = oracle.block_scales_bits(oracle.quantize_q8_0(x))[0, 0].view(np.float16).astype(np.float32)
    assert one[0, 0] == np.float32(s) * np.float32(dw * da)


def _round_to_f32(v):
    """Exact rational -> nearest binary32 (ties to even), by integer arithmetic only."""
    from fractions import Fraction

    if v == 0:
        return np.float32(0.0)
    sign = -1 if v < 0 else 1
    v = abs(Fraction(v))
    e = v.numerator.bit_length() - v.denominator.bit_length() - 24
    while v / Fraction(2) ** e >= 2 ** 24:
        e += 1
    while v / Fraction(2) ** e < 2 ** 23:
        e -= 1
    e = max(e, -149)
    q = v / Fraction(2) ** e
    n, rem = divmod(q.numerator, q.denominator)
    twice = 2 * rem
    if twice > q.denominator or (twice == q.denominator and n % 2 == 1):
        n += 1
    return np.float32(sign * float(n) * 2.0 ** e)       # n < 2^24 + 1 and the scaling are exact in double


def test_q8_matmul_settlement_order_bit_exact(oracle):
    # The settlement acc = fma(float(sumi), dw*da, acc), blocks ascending, redone in exact rational
    # arithmetic with one rounding per step.  The case is chosen so that the three plausible
    # mistakes -- multiply and add rounded separately, blocks walked backwards, scales multiplied
    # into the sum one after the other -- each change at least one output bit.
    from fractions import Fraction

    rng = np.random.default_rng(12)
    M, N, K = 6, 5, 256
    w = (rng.standard_normal((M, K)) * np.exp(rng.standard_normal((M, K // 32)).repeat(32, axis=1))).astype(np.float32)
    x = (rng.standard_normal((N, K)) * np.exp(rng.standard_normal((N, K // 32)).repeat(32, axis=1))).astype(np.float32)
    wq, xq = oracle.quantize_q8_0(w), oracle.quantize_q8_0(x)
    sums = oracle.q8_block_sums(wq, xq)
    dw = oracle.block_scales_bits(wq).view(np.float16).astype(np.float32)
    da = oracle.block_scales_bits(xq).view(np.float16).astype(np.float32)

    def settle(order, fused, split_scales=False):
        out = np.zeros((N, M), np.float32)
        for n in range(N):
            for m in range(M):
                acc = np.float32(0.0)
                for b in order:
                    sf = Fraction(int(sums[n, m, b]))
                    if split_scales:
                        t = _round_to_f32(sf * Fraction(float(dw[m, b])))
                        prod = Fraction(float(t)) * Fraction(float(da[n, b]))
                    else:
                        prod = sf * Fraction(float(dw[m, b] * da[n, b]))      # dw*da is exact in binary32
                    if fused:
                        acc = _round_to_f32(prod + Fraction(float(acc)))
                    else:
                        acc = _round_to_f32(Fraction(float(_round_to_f32(prod))) + Fraction(float(acc)))
                out[n, m] = acc
        return out

    blocks = list(range(K // 32))
    want = settle(blocks, fused=True)
    got = oracle.mul_mat_q8q8(wq, xq, c_trans=1, fma=1)
    assert (got.view(np.uint32) == want.view(np.uint32)).all()
    assert (oracle.mul_mat_q8q8(wq, xq, c_trans=1, fma=0).view(np.uint32) == settle(blocks, fused=False).view(np.uint32)).all()
    for wrong in (settle(blocks, fused=False), settle(blocks[::-1], fused=True), settle(blocks, True, split_scales=True)):
        assert (wrong.view(np.uint32) != want.view(np.uint32)).any()


# ----------------------------------------------------------------------------- f32 mul_mat
def test_mul_mat_reference_test_inputs_exact(oracle):
    # tests/test_cuda.cpp:133-167: every product is a multiple of 1/8 and every partial sum is small,
    # so binary32 holds all of them exactly and the answer equals integer arithmetic.
    M, K, N = 17, 9, 23
    A = ((np.arange(M * K) % 11) * 0.5 - 2.0).astype(np.float32).reshape(M, K)
    B = ((np.arange(N * K) % 13) * 0.25 + 0.5).astype(np.float32).reshape(N, K)
    got = oracle.mul_mat_f32(A, B)
    Ai = np.rint(A.astype(np.float64) * 2).astype(np.int64)
    Bi = np.rint(B.astype(np.float64) * 4).astype(np.int64)
    want = (Ai @ Bi.T) / 8.0
    assert got.shape == (M, N) and (got.astype(np.float64) == want).all()
    bias = ((np.arange(N) % 5) * 0.125 - 0.25).astype(np.float32)
    got_b = oracle.mul_mat_f32(A, B, bias)
    assert (got_b.astype(np.float64) == want + bias.astype(np.float64)[None, :]).all()
    for nt in (1, 3):
        assert (oracle.mul_mat_f32(A, B, bias, nthreads=nt) == got_b).all()


def test_mul_mat_bias_enters_first_and_k_ascending(oracle):
    # 1e8 + 1 - 1e8: only "bias first, then k ascending" gives 0; bias last would give 1.
    a = np.array([[1.0, 1.0]], dtype=np.float32)
    b = np.array([[1.0, -1e8]], dtype=np.float32)
    assert oracle.mul_mat_f32(a, b, np.array([1e8], dtype=np.float32))[0, 0] == 0.0
    # ascending k: (1e8 + 1) - 1e8 = 0, descending would give 1
    a = np.array([[1e8, 1.0, -1e8]], dtype=np.float32)
    b = np.ones((1, 3), dtype=np.float32)
    assert oracle.mul_mat_f32(a, b)[0, 0] == 0.0


def test_mul_mat_random_vs_float64(oracle):
    rng = np.random.default_rng(8)
    A = rng.standard_normal((33, 70)).astype(np.float32)
    B = rng.standard_normal((21, 70)).astype(np.float32)
    want = A.astype(np.float64) @ B.astype(np.float64).T
    assert np.abs(oracle.mul_mat_f32(A, B) - want).max() < 1e-4


def test_mul_mat_f16_binary32_sum_and_bias_last(oracle):
    # src/backend/CPUKernels.cpp:392-396, 646-672
    rng = np.random.default_rng(2)
    a = rng.standard_normal((7, 37)).astype(np.float16)
    b = (rng.standard_normal((5, 37)) * 0.02).astype(np.float16)
    bias = rng.standard_normal(5).astype(np.float32)
    got = oracle.mul_mat_f16(a, b, bias)
    want = a.astype(np.float64) @ b.astype(np.float64).T + bias
    assert np.abs(got - want).max() <= 1e-5 * np.abs(want).max()
    # equals the f32 kernel on the widened operands when there is no bias (same products, same order)
    assert (oracle.mul_mat_f16(a, b) == oracle.mul_mat_f32(a.astype(np.float32), b.astype(np.float32))).all()
    # the bias is added LAST here and FIRST on the f32 branch: with bias 2^24 and two products of 1,
    # last gives 2 + 2^24 (a binary32 number), first gives (2^24 + 1) + 1 = 2^24 (each +1 is lost)
    ones = np.ones((1, 2), np.float16)
    big = np.array([2.0 ** 24], np.float32)
    assert oracle.mul_mat_f16(ones, ones, big)[0, 0] == np.float32(2.0 ** 24 + 2)
    assert oracle.mul_mat_f32(ones.astype(np.float32), ones.astype(np.float32), big)[0, 0] == np.float32(2.0 ** 24)


# ----------------------------------------------------------------------------- out_prod
def test_out_prod_reference_small_inputs_exact(oracle):
    # tests/test_cuda.cpp:207-245
    C0, C1, K = 4, 5, 3
    a = ((np.arange(C0 * K) % 7) * 0.5).astype(np.float32).reshape(1, 1, K, C0)
    b = ((np.arange(C1 * K) % 9) * 0.25 - 1.0).astype(np.float32).reshape(1, 1, K, C1)
    got = oracle.out_prod(a, b)
    want = np.einsum("ki,kj->ji", a[0, 0].astype(np.float64), b[0, 0].astype(np.float64))
    assert got.shape == (1, 1, C1, C0) and (got[0, 0].astype(np.float64) == want).all()


def test_out_prod_reference_real_shape_exact(oracle):
    # tests/test_cuda.cpp:262-341: L=51, K=51, 16x64 planes; inputs are multiples of 1/16 and 1/8,
    # so the sums are exact in binary32 whatever the order.
    L, K, P2, P3 = 51, 51, 16, 64
    nA = L * K * P2 * P3
    A = ((np.arange(nA) % 13) * 0.0625 - 0.5).astype(np.float32).reshape(P3, P2, K, L)
    B = ((np.arange(nA) % 7) * 0.125 - 0.25).astype(np.float32).reshape(P3, P2, K, L)
    got = oracle.out_prod(A, B)
    for i3, i2 in ((0, 0), (P3 - 1, P2 - 1), (17, 5)):
        want = np.einsum("ki,kj->ji", A[i3, i2].astype(np.float64), B[i3, i2].astype(np.float64))
        assert (got[i3, i2].astype(np.float64) == want).all()


def test_out_prod_broadcasts_src0_planes(oracle):
    # CPUKernels.cpp:836-858: i02 = i2 / (ne2/ne02), i03 = i3 / (ne3/ne03)
    rng = np.random.default_rng(9)
    s0 = rng.integers(-4, 5, size=(2, 3, 5, 6)).astype(np.float32)      # ne03=2, ne02=3
    s1 = rng.integers(-4, 5, size=(4, 6, 5, 7)).astype(np.float32)      # ne13=4, ne12=6
    got = oracle.out_prod(s0, s1)
    s0b = np.repeat(np.repeat(s0, 2, axis=0), 2, axis=1)
    want = np.einsum("pqki,pqkj->pqji", s0b.astype(np.float64), s1.astype(np.float64))
    assert got.shape == (4, 6, 7, 6) and (got.astype(np.float64) == want).all()


# ----------------------------------------------------------------------------- outer product mean
def test_opm_value_known_answers(oracle):
    # tests/test_outer_product_mean.cpp:10-50
    left = np.array([1, 2, 3, 4, 5, 6, 7, 8], dtype=np.float32).reshape(1, 2, 2, 2)
    right = np.array([1, 0, 0, 1, 1, 1, 0, 0], dtype=np.float32).reshape(1, 2, 2, 2)
    o = oracle.outer_product_mean_value(left, right)
    assert o.shape == (1, 2, 2, 4)
    assert list(o[0, 0, 0]) == [3.0, 2.5, 4.0, 3.0]
    assert o[0, 1, 1, 0] == 0.0 and o[0, 1, 1, 3] == 2.0
    # tests/test_outer_product_mean.cpp:52-70
    left = np.array([[n + i for i in range(2)] for n in range(3)], dtype=np.float32).reshape(1, 3, 2, 1)
    o = oracle.outer_product_mean_value(left, np.ones((1, 3, 2, 1), dtype=np.float32))
    assert np.allclose(o.ravel(), [1.0, 1.0, 2.0, 2.0], rtol=1e-7)


def test_opm_value_vs_einsum(oracle):
    rng = np.random.default_rng(10)
    l = rng.integers(-3, 4, size=(2, 4, 3, 5)).astype(np.float32)
    r = rng.integers(-3, 4, size=(2, 4, 3, 5)).astype(np.float32)
    want = np.einsum("bnid,bnje->bijde", l.astype(np.float64), r.astype(np.float64)).reshape(2, 3, 3, 25) / 4.0
    assert (oracle.outer_product_mean_value(l, r).astype(np.float64) == want).all()


def test_opm_graph_form_vs_einsum(oracle):
    # Layout stated at src/backend/CPUKernels.cpp:975-981: left[d,i,n,b] at ((d*L+i)*N+n)*B+b and
    # dst[(d1*D+d2), i, j, b] at (((d1*D+d2)*L+i)*L+j)*B+b.  D != L != N != B so that any swapped
    # pair of indices changes the result.
    rng = np.random.default_rng(11)
    D, L, N, B = 3, 4, 8, 2
    l = rng.integers(-3, 4, size=(D, L, N, B)).astype(np.float32)
    r = rng.integers(-3, 4, size=(D, L, N, B)).astype(np.float32)
    got = oracle.outer_prod_mean(l, r, D, L, N, B).reshape(D, D, L, L, B)
    want = np.einsum("dinb,ejnb->deijb", l.astype(np.float64), r.astype(np.float64)) / N
    assert (got.astype(np.float64) == want).all()
    # 1/N multiplies the finished sum (CPUKernels.cpp:995,1028): with N=3 sum*inv differs from sum/3
    D, L, N, B = 1, 1, 3, 1
    l = np.array([1.0, 1.0, 1.0], dtype=np.float32)
    got = oracle.outer_prod_mean(l, l, D, L, N, B)
    assert got[0] == np.float32(3.0) * (np.float32(1.0) / np.float32(3.0))


# ----------------------------------------------------------------------------- attention scores
def test_attention_scores_vs_einsum(oracle):
    rng = np.random.default_rng(12)
    NQ, H, D, Lq, Lk = 2, 3, 16, 5, 7
    q = rng.integers(-3, 4, size=(NQ, H, D, Lq)).astype(np.float32)
    k = rng.integers(-3, 4, size=(NQ, H, D, Lk)).astype(np.float32)
    got = oracle.attention_scores(q, k)
    s = np.einsum("bhdi,bhdj->bhij", q.astype(np.float64), k.astype(np.float64)).astype(np.float32)
    want = s * (np.float32(1.0) / np.sqrt(np.float32(D)))          # 1/sqrt(16) = 0.25 exactly
    assert (got == want).all()
    # equals the graph path: out_prod(K,Q) then a scale node (Attention.cpp:264-270)
    kk = np.ascontiguousarray(k.reshape(NQ, H, D, Lk))
    op = oracle.out_prod(kk, q)                                      # [NQ,H,Lq,Lk]
    assert (op * np.float32(0.25) == got).all()


# ----------------------------------------------------------------------------- fused attention forward
def _attention_f64(q, k, v, bias, causal, scale, eps):
    """Textbook softmax attention in float64, written independently of the oracle's loop."""
    B, h, L, d = q.shape
    sc = scale if scale > 0 else 1.0 / np.sqrt(d)
    s = np.einsum("bhid,bhjd->bhij", q.astype(np.float64), k.astype(np.float64)) * sc
    if bias is not None:
        s = s + bias.astype(np.float64)
    if causal:
        s = np.where(np.tril(np.ones((L, L), dtype=bool)), s, -np.inf)
    m = s.max(axis=-1, keepdims=True)
    m = np.where(np.isfinite(m), m, 0.0)
    e = np.exp(s - m)
    l = e.sum(axis=-1, keepdims=True)
    o = np.einsum("bhij,bhjd->bhid", e / (l + eps), v.astype(np.float64))
    with np.errstate(divide="ignore"):
        lse = (m + np.log(l + eps))[..., 0]
    return o, np.where(l[..., 0] > 0, lse, -np.inf)


@pytest.mark.parametrize("B,h,L,d,causal,Bc,use_bias", [
    (2, 3, 37, 8, False, 64, True), (1, 2, 103, 32, False, 64, False), (1, 1, 70, 12, True, 16, True),
    (2, 1, 5, 4, True, 64, False), (1, 2, 130, 64, False, 32, True), (1, 1, 1, 4, False, 64, True),
])
def test_flash_attn_forward_against_the_compiled_reference(oracle, B, h, L, d, causal, Bc, use_bias):
    if oracle.ref_flash_lib() is None:
        pytest.skip("oracle/_ref/libppml_ref_flash.so not built (reference tree absent)")
    rng = np.random.default_rng(L * 131 + d)
    q, k, v = [rng.standard_normal((B, h, L, d)).astype(np.float32) for _ in range(3)]
    bias = (3 * rng.standard_normal((B, h, L, L))).astype(np.float32) if use_bias else None
    o, lse = oracle.flash_attn_forward(q, k, v, bias, causal=causal, Bc=Bc)
    ro, rlse = oracle.ref_flash_attn_forward(q, k, v, bias, causal=causal, Bc=Bc)
    assert (o.view(np.uint32) == ro.view(np.uint32)).all()
    assert (lse.view(np.uint32) == rlse.view(np.uint32)).all()


@pytest.mark.parametrize("causal,use_bias,scale", [(False, True, 0.0), (True, False, 0.0), (False, False, 0.37), (True, True, 2.0)])
def test_flash_attn_forward_against_float64_softmax(oracle, causal, use_bias, scale):
    rng = np.random.default_rng(5)
    B, h, L, d = 2, 2, 77, 16
    q, k, v = [rng.standard_normal((B, h, L, d)).astype(np.float32) for _ in range(3)]
    bias = rng.standard_normal((B, h, L, L)).astype(np.float32) if use_bias else None
    o, lse = oracle.flash_attn_forward(q, k, v, bias, causal=causal, scale=scale, Bc=16)
    wo, wlse = _attention_f64(q, k, v, bias, causal, scale, 1e-9)
    assert np.abs(o - wo).max() <= 2e-6 * max(1.0, np.abs(wo).max())
    assert np.abs(lse - wlse).max() <= 2e-6 * np.abs(wlse).max()


def test_flash_attn_forward_closed_forms(oracle):
    rng = np.random.default_rng(9)
    B, h, L, d = 1, 2, 40, 8
    v = rng.standard_normal((B, h, L, d)).astype(np.float32)
    k = rng.standard_normal((B, h, L, d)).astype(np.float32)
    zero_q = np.zeros((B, h, L, d), dtype=np.float32)
    # equal scores: every output row is the mean of V and LSE = log(L) (a swapped Q/K or a dropped
    # normalisation would not give this); causal: row i is the mean of the first i + 1 rows
    o, lse = oracle.flash_attn_forward(zero_q, k, v, eps=0.0, Bc=16)
    assert np.allclose(o, v.mean(axis=2, keepdims=True), atol=1e-6)
    assert np.allclose(lse, np.log(L), atol=1e-6)
    o, _ = oracle.flash_attn_forward(zero_q, k, v, causal=True, eps=0.0, Bc=16)
    want = np.cumsum(v.astype(np.float64), axis=2) / np.arange(1, L + 1)[None, None, :, None]
    assert np.allclose(o, want, atol=1e-6)
    # a bias that towers over the scores at key (i * 7) % L picks that row of V: bias is indexed [query][key]
    q = rng.standard_normal((B, h, L, d)).astype(np.float32)
    bias = np.zeros((B, h, L, L), dtype=np.float32)
    pick = (np.arange(L) * 7) % L
    bias[:, :, np.arange(L), pick] = 200.0
    o, _ = oracle.flash_attn_forward(q, k, v, bias)
    assert np.allclose(o, v[:, :, pick, :], atol=1e-6)
    # adding a constant per query row to the bias changes LSE by that constant and leaves O alone
    bias = rng.standard_normal((B, h, L, L)).astype(np.float32)
    shift = rng.standard_normal((B, h, L, 1)).astype(np.float32)
    o0, l0 = oracle.flash_attn_forward(q, k, v, bias)
    o1, l1 = oracle.flash_attn_forward(q, k, v, bias + shift)
    assert np.allclose(o0, o1, atol=2e-6) and np.allclose(l1 - l0, shift[..., 0], atol=1e-5)
    # the scale multiplies the dot product only, not the bias
    o2, _ = oracle.flash_attn_forward(2 * q, k, v, bias, scale=0.5)
    o3, _ = oracle.flash_attn_forward(q, k, v, bias, scale=1.0)
    assert np.allclose(o2, o3, atol=2e-6)
    # fully masked row: O = 0 and LSE = -inf; its neighbours are untouched
    bias[0, 1, 3, :] = -np.inf
    o4, l4 = oracle.flash_attn_forward(q, k, v, bias)
    assert (o4[0, 1, 3] == 0).all() and np.isneginf(l4[0, 1, 3]) and np.isfinite(l4[0, 1, 2])
    # bad arguments are refused, not computed
    assert oracle.lib().orc_flash_attn_forward(1, 1, 0, 4, 0, 0.0, 0.0, 64, None, None, None, None, None, None, 1) == 1


# ----------------------------------------------------------------------------- permute
def _np_permute(x, axes):
    """numpy statement of the reference's rule: reference dimension k is numpy axis nd-1-k, and
    dimension p of the result is dimension axes[p] of the source."""
    nd = x.ndim
    return np.ascontiguousarray(np.transpose(x, [nd - 1 - axes[nd - 1 - a] for a in range(nd)]))


def test_permute_hand_case_and_numpy(oracle):
    # dims (reference order) [3, 2]: rows of 3; mat_transpose = axes (1, 0) gives dims [2, 3]
    x = np.arange(6, dtype=np.float32).reshape(2, 3)
    assert oracle.permute(x, (1, 0)).tolist() == [[0, 3], [1, 4], [2, 5]]
    rng = np.random.default_rng(11)
    import itertools
    x4 = rng.standard_normal((3, 4, 5, 6)).astype(np.float32)        # reference dims [6, 5, 4, 3]
    for axes in itertools.permutations(range(4)):
        got = oracle.permute(x4, axes)
        assert got.shape == tuple(x4.shape[::-1][a] for a in axes)[::-1]
        assert np.array_equal(got, _np_permute(x4, axes)), axes
        inverse = [axes.index(k) for k in range(4)]
        assert np.array_equal(oracle.permute(got, inverse), x4), axes
    x3 = rng.standard_normal((4, 5, 6)).astype(np.float32)
    for axes in itertools.permutations(range(3)):
        assert np.array_equal(oracle.permute(x3, axes), _np_permute(x3, axes)), axes
    assert np.array_equal(oracle.permute(x4, (0, 1, 2, 3)), x4)
    # an axis outside the tensor's dimensions is refused (the reference prints and skips the node)
    import ctypes as C
    out = np.zeros(6, dtype=np.float32)
    rc = oracle.lib().orc_permute(x.ctypes.data_as(C.POINTER(C.c_float)), out.ctypes.data_as(C.POINTER(C.c_float)), 2,
                                  (C.c_int32 * 4)(2, 0, 2, 3), (C.c_int64 * 4)(3, 2, 1, 1), (C.c_int64 * 4)(2, 3, 1, 1))
    assert rc == 1 and not out.any()


# ----------------------------------------------------------------------------- triangle multiplication
def test_tri_mul_against_einsum_and_the_finite_guard(oracle):
    rng = np.random.default_rng(21)
    D, I, J, K, Bt, L = 3, 5, 4, 6, 2, 8.0          # 1/8 is exact, small integers keep every sum exact
    # outgoing: left[d,i,k,b], right[d,j,k,b]; incoming: left[d,k,i,b], right[d,k,j,b] (CPUKernels.cpp:895-903)
    lo = rng.integers(-4, 5, size=(D, I, K, Bt)).astype(np.float32)
    ro = rng.integers(-4, 5, size=(D, J, K, Bt)).astype(np.float32)
    want = np.einsum("dikb,djkb->dijb", lo.astype(np.float64), ro.astype(np.float64)) / L
    assert np.array_equal(oracle.tri_mul(lo, ro, D, I, J, K, Bt, L, outgoing=True).reshape(D, I, J, Bt), want)
    li = rng.integers(-4, 5, size=(D, K, I, Bt)).astype(np.float32)
    ri = rng.integers(-4, 5, size=(D, K, J, Bt)).astype(np.float32)
    want = np.einsum("dkib,dkjb->dijb", li.astype(np.float64), ri.astype(np.float64)) / L
    assert np.array_equal(oracle.tri_mul(li, ri, D, I, J, K, Bt, L, outgoing=False).reshape(D, I, J, Bt), want)
    # the two forms differ (a transposed operand would pass one of the checks above, not both)
    assert not np.array_equal(oracle.tri_mul(lo, ro, D, I, J, K, Bt, L, True), oracle.tri_mul(lo.reshape(-1), ro.reshape(-1), D, I, J, K, Bt, L, False))
    # finite guard (CPUKernels.cpp:957-962): NaN -> 0, beyond +-1e4 -> +-1e4, applied after the 1/L
    l1 = np.zeros((1, 4, 2, 1), dtype=np.float32)
    r1 = np.ones((1, 1, 2, 1), dtype=np.float32)
    l1[0, 0, 0, 0] = np.nan
    l1[0, 1, 0, 0] = 3e4          # 3e4 / 2 = 1.5e4 -> 1e4
    l1[0, 2, 0, 0] = -np.inf
    l1[0, 3, 0, 0] = 1.9e4        # 9.5e3 stays
    got = oracle.tri_mul(l1, r1, 1, 4, 1, 2, 1, 2.0, True)
    assert got.tolist() == [0.0, 1e4, -1e4, 9.5e3]


def test_tri_mul_back_against_einsum_and_the_adjoint_identity(oracle):
    rng = np.random.default_rng(22)
    D, I, J, K, Bt, L = 2, 5, 4, 6, 3, 4.0
    for outgoing, ls, rs, gl_eq, gr_eq, f_eq in [
        (True, (D, I, K, Bt), (D, J, K, Bt), "dijb,djkb->dikb", "dijb,dikb->djkb", "dikb,djkb->dijb"),
        (False, (D, K, I, Bt), (D, K, J, Bt), "dijb,dkjb->dkib", "dijb,dkib->dkjb", "dkib,dkjb->dijb"),
    ]:
        left = rng.integers(-3, 4, size=ls).astype(np.float32)
        right = rng.integers(-3, 4, size=rs).astype(np.float32)
        grad = rng.integers(-3, 4, size=(D, I, J, Bt)).astype(np.float32)
        gl, gr = oracle.tri_mul_back(grad, left, right, D, I, J, K, Bt, L, outgoing)
        g64, l64, r64 = grad.astype(np.float64), left.astype(np.float64), right.astype(np.float64)
        assert np.array_equal(gl.reshape(ls), np.einsum(gl_eq, g64, r64) / L), outgoing
        assert np.array_equal(gr.reshape(rs), np.einsum(gr_eq, g64, l64) / L), outgoing
        # adjoint of the forward map (which the einsum above does not know about): <grad, f(l, r)> = <gleft, l> = <gright, r>
        fwd = oracle.tri_mul(left, right, D, I, J, K, Bt, L, outgoing).astype(np.float64)
        assert np.array_equal(fwd.reshape(D, I, J, Bt), np.einsum(f_eq, l64, r64) / L)
        lhs = float((g64.reshape(-1) * fwd).sum())
        assert lhs == float((gl.astype(np.float64) * l64.reshape(-1)).sum()) == float((gr.astype(np.float64) * r64.reshape(-1)).sum())


def test_outer_prod_mean_back_against_einsum_and_the_adjoint_identity(oracle):
    rng = np.random.default_rng(23)
    D, L, N, Bt = 3, 4, 8, 2                           # 1/N exact
    left = rng.integers(-3, 4, size=(D, L, N, Bt)).astype(np.float32)
    right = rng.integers(-3, 4, size=(D, L, N, Bt)).astype(np.float32)
    grad = rng.integers(-3, 4, size=(D, D, L, L, Bt)).astype(np.float32)      # [d1][d2][i][j][b]
    gl, gr = oracle.outer_prod_mean_back(grad, left, right, D, L, N, Bt)
    g64, l64, r64 = grad.astype(np.float64), left.astype(np.float64), right.astype(np.float64)
    assert np.array_equal(gl.reshape(D, L, N, Bt), np.einsum("deijb,ejnb->dinb", g64, r64) / N)
    assert np.array_equal(gr.reshape(D, L, N, Bt), np.einsum("deijb,dinb->ejnb", g64, l64) / N)
    # adjoint of the forward kernel itself: <grad, opm(l, r)> = <gleft, l> = <gright, r>
    fwd = oracle.outer_prod_mean(left.reshape(-1), right.reshape(-1), D, L, N, Bt).astype(np.float64)
    lhs = float((g64.reshape(-1) * fwd).sum())
    assert lhs == float((gl.astype(np.float64) * l64.reshape(-1)).sum()) == float((gr.astype(np.float64) * r64.reshape(-1)).sum())


# ----------------------------------------------------------------------------- fused attention backward
@pytest.mark.parametrize("B,h,L,d,causal,use_bias", [(2, 2, 19, 8, False, True), (1, 3, 40, 16, True, True), (1, 1, 70, 32, False, False)])
def test_flash_attn_backward_against_the_compiled_reference(oracle, B, h, L, d, causal, use_bias):
    if oracle.ref_flash_lib() is None:
        pytest.skip("oracle/_ref/libppml_ref_flash.so not built (reference tree absent)")
    rng = np.random.default_rng(L + d)
    q, k, v, do = [rng.standard_normal((B, h, L, d)).astype(np.float32) for _ in range(4)]
    bias = rng.standard_normal((B, h, L, L)).astype(np.float32) if use_bias else None
    if bias is not None and not causal:
        bias[0, 0, 3, :] = -np.inf                      # a masked row: LSE = -inf, no gradient
    o, lse = oracle.flash_attn_forward(q, k, v, bias, causal=causal)
    got = oracle.flash_attn_backward(q, k, v, bias, o, do, lse, causal=causal)
    want = oracle.ref_flash_attn_backward(q, k, v, bias, o, do, lse, causal=causal)
    for g, w in zip(got, want):
        assert (g.view(np.uint32) == w.view(np.uint32)).all()


def test_flash_attn_backward_against_finite_differences(oracle):
    rng = np.random.default_rng(31)
    B, h, L, d = 1, 2, 9, 4
    q, k, v, do = [rng.standard_normal((B, h, L, d)).astype(np.float32) for _ in range(4)]
    bias = rng.standard_normal((B, h, L, L)).astype(np.float32)
    for causal in (False, True):
        o, lse = oracle.flash_attn_forward(q, k, v, bias, causal=causal, eps=0.0)
        dq, dk, dv, db = oracle.flash_attn_backward(q, k, v, bias, o, do, lse, causal=causal)

        def loss(q_, k_, v_, b_):
            o64, _ = _attention_f64(q_, k_, v_, b_, causal, 0.0, 0.0)
            return float((o64 * do.astype(np.float64)).sum())

        def numeric(which):
            arrs = [q.astype(np.float64), k.astype(np.float64), v.astype(np.float64), bias.astype(np.float64)]
            g = np.zeros_like(arrs[which])
            it = np.nditer(arrs[which], flags=["multi_index"])
            for _ in it:
                idx = it.multi_index
                old = arrs[which][idx]
                arrs[which][idx] = old + 1e-5
                up = loss(*arrs)
                arrs[which][idx] = old - 1e-5
                dn = loss(*arrs)
                arrs[which][idx] = old
                g[idx] = (up - dn) / 2e-5
            return g
        for got, which in ((dq, 0), (dk, 1), (dv, 2), (db, 3)):
            want = numeric(which)
            assert np.abs(got - want).max() <= 2e-4 * max(1.0, np.abs(want).max()), (causal, which)
        # softmax rows: the gradient with respect to the scores sums to zero over the keys
        assert np.abs(db.sum(axis=-1)).max() <= 1e-5
        if causal:
            assert (np.triu(db[0, 0], 1) == 0).all()
    # nothing to compute is refused
    assert oracle.lib().orc_flash_attn_backward(1, 1, 2, 4, 0, 0.0, *([q.ctypes.data_as(__import__("ctypes").POINTER(__import__("ctypes").c_float))] * 7), None, None, None, None) == 1


# ----------------------------------------------------------------------------- repeat_back
def test_repeat_back_bias_gradient_and_broadcast_axes(oracle):
    # the gradient of a mul_mat bias: grad [N, M] (dims[0] = N) -> dbias [N] = sum over the M rows
    # (src/core/ComputeGraph.cpp:742); numpy shapes are outermost first
    rng = np.random.default_rng(31)
    g = rng.integers(-8, 9, size=(23, 17)).astype(np.float32)          # M = 23 rows of N = 17
    assert (oracle.repeat_back(g, (17,)) == g.sum(axis=0)).all()
    # a wrong (right-aligned) pairing of the dimensions would sum 17 // 23 = 0 copies or read one element
    assert not (oracle.repeat_back(g, (17,)) == g[0]).all()
    # same rank, broadcast over dims[1] and dims[3]: [5,1,4,1] from [5,3,4,2]
    x = rng.integers(-5, 6, size=(2, 4, 3, 5)).astype(np.float32)
    assert (oracle.repeat_back(x, (1, 4, 1, 5)) == x.sum(axis=(0, 2), keepdims=True)).all()
    # a dimension that is kept and repeated at once: dst dims[0] = 3 from src dims[0] = 6, copies j0 and j0 + 3
    y = rng.integers(-5, 6, size=(4, 6)).astype(np.float32)
    want = y[:, :3] + y[:, 3:]
    assert (oracle.repeat_back(y, (4, 3)) == want).all()
    # no repetition at all is a copy
    assert (oracle.repeat_back(y, (4, 6)) == y).all()


def test_repeat_back_adds_its_terms_one_at_a_time(oracle):
    # 2^24 + 1 + 1: adding from the left rounds each 1 away (2^24); pairing the ones first gives 2^24 + 2
    col = np.array([[2.0 ** 24], [1.0], [1.0]], dtype=np.float32)       # three rows of one element
    assert oracle.repeat_back(col, (1,))[0] == np.float32(2.0 ** 24)
    col2 = np.array([[1.0], [1.0], [2.0 ** 24]], dtype=np.float32)
    assert oracle.repeat_back(col2, (1,))[0] == np.float32(2.0 ** 24 + 2)
    # with two repeated dimensions the innermost loop is the OUTER dimension (k3 fastest, k0 slowest):
    # src dims [2, 2] -> dst [1, 1]; order of the four terms is (k0,k1) = (0,0), (0,1), (1,0), (1,1)
    m = np.array([[2.0 ** 24, 1.0], [1.0, 1.0]], dtype=np.float32)      # m[i1][i0]
    # (0,0) = 2^24, (0,1) = m[1][0] = 1 -> lost, (1,0) = m[0][1] = 1 -> lost, (1,1) = 1 -> lost
    assert oracle.repeat_back(m, (1, 1))[0, 0] == np.float32(2.0 ** 24)
    m2 = np.array([[1.0, 2.0 ** 24], [1.0, 1.0]], dtype=np.float32)
    # 1 + 1 = 2, + 2^24 = 2^24 + 2, + 1 -> tie, rounds to even: 2^24 + 4?  (2^24 + 3 lies between 2^24+2 and 2^24+4)
    got = oracle.repeat_back(m2, (1, 1))[0, 0]
    assert got == np.float32(np.float32(np.float32(1.0 + 1.0) + np.float32(2.0 ** 24)) + np.float32(1.0))


# ----------------------------------------------------------------------------- element-wise nodes between the contractions
def test_scale_and_relu_are_one_ieee_operation_per_element(oracle):
    rng = np.random.default_rng(40)
    x = rng.standard_normal(1001).astype(np.float32) * np.float32(1e3)
    x[:6] = [0.0, -0.0, np.inf, -np.inf, np.nan, np.float32(1e-42)]
    s = np.float32(1.0 / np.sqrt(np.float32(32.0)))
    got = oracle.scale(x, s)
    want = x * s                                        # numpy's float32 multiply: one rounding
    assert np.array_equal(got.view(np.uint32)[~np.isnan(want)], want.view(np.uint32)[~np.isnan(want)])
    assert np.isnan(got[4])
    assert oracle.scale(np.float32([3.0]), 0.1)[0] == np.float32(3.0) * np.float32(0.1)     # the factor is a binary32
    r = oracle.relu(x)
    assert np.array_equal(r[6:], np.maximum(x[6:], 0))
    # (s > 0) ? s : 0 -- NaN and -0 fail the comparison and give +0; np.maximum would keep both
    assert r[0] == 0 and not np.signbit(r[0]) and r[1] == 0 and not np.signbit(r[1])
    assert r[2] == np.inf and r[3] == 0 and r[4] == 0 and not np.signbit(r[4]) and r[5] == np.float32(1e-42)


def test_bcast_elemwise_is_the_flat_modulo_broadcast(oracle):
    rng = np.random.default_rng(41)
    a = rng.standard_normal((3, 5, 4, 6)).astype(np.float32)
    for shape in [(3, 5, 4, 6), (4, 6), (6,), (1,), (5, 4, 6)]:
        b = (rng.standard_normal(shape) + 3).astype(np.float32)
        tiled = np.resize(b.ravel(), a.size).reshape(a.shape)                    # b[i % bn]
        for op, f in [("add", np.add), ("sub", np.subtract), ("mul", np.multiply), ("div", np.divide)]:
            got = oracle.bcast_elemwise(a, b, op)
            assert got.shape == a.shape
            assert np.array_equal(got.view(np.uint32), f(a, tiled).view(np.uint32)), (shape, op)
        # an operand that covers the innermost dimensions: numpy's own dimension-wise broadcast says the same
        assert np.array_equal(oracle.bcast_elemwise(a, b, "add"), a + b)
    # ... and one that does not (a middle dimension): the flat rule reads other elements than numpy's broadcast
    mid = rng.standard_normal((5, 1, 1)).astype(np.float32)
    assert not np.array_equal(oracle.bcast_elemwise(a, mid, "add"), a + mid)
    # the smaller operand may come first (dst then has the larger one's shape)
    b = rng.standard_normal(6).astype(np.float32)
    assert np.array_equal(oracle.bcast_elemwise(b, a, "sub"), b - a)


def test_softmax_closed_forms(oracle):
    # rows of equal values: expf(0) = 1 exactly, sum = D exactly, so every entry is fl(1 / fl(D + 1e-9))
    for D in (1, 2, 3, 7, 64, 103, 256, 1000):
        got = oracle.softmax(np.full((2, D), 3.25, np.float32))
        want = np.float32(1.0) / (np.float32(D) + np.float32(1e-9))
        assert (got == want).all(), D
    # one dominant entry
    x = np.full((1, 50), -200.0, np.float32)
    x[0, 17] = 5.0
    got = oracle.softmax(x)
    assert got[0, 17] == 1.0 and got.sum() == 1.0
    # against float64 on random rows
    rng = np.random.default_rng(42)
    x = (4 * rng.standard_normal((37, 103))).astype(np.float32)
    e = np.exp(x.astype(np.float64) - x.max(-1, keepdims=True))
    want = e / (e.sum(-1, keepdims=True) + 1e-9)
    np.testing.assert_allclose(oracle.softmax(x), want, rtol=2e-6, atol=1e-12)
    # over the LAST axis only: rows are independent
    y = oracle.softmax(x.reshape(37, 1, 103))
    assert np.array_equal(y.reshape(37, 103), oracle.softmax(x))
    # exact shifts leave the bits alone (the maximum is subtracted first)
    xi = rng.integers(-8, 9, size=(5, 40)).astype(np.float32)
    assert np.array_equal(oracle.softmax(xi), oracle.softmax(xi + 16))
    # the maximum starts from the first element and moves on `>`: a NaN there poisons the row, elsewhere too
    # (through the sum); a row of -inf is NaN (inf - inf); -inf entries beside finite ones are plain zeros
    z = np.zeros((4, 5), np.float32)
    z[0, 0] = np.nan
    z[1, 3] = np.nan
    z[2, :] = -np.inf
    z[3, 1:3] = -np.inf
    s = oracle.softmax(z)
    assert np.isnan(s[0]).all() and np.isnan(s[1]).all() and np.isnan(s[2]).all()
    assert (s[3, 1:3] == 0).all() and np.allclose(s[3, [0, 3, 4]], 1 / 3)


def test_attention_chain_of_nodes_equals_the_fused_reference_on_its_golden_vectors(oracle):
    """out_prod(K,Q) -> scale -> add(bias) -> softmax -> permute, permute(V) -> out_prod, node by node with the oracle's
    restatements (src/modules/Attention.cpp:264-281), against the outputs of the reference's own fused
    flash_attn_forward_cpu held in tests/golden/flash_attn_forward.json (non-causal cases; the fused routine
    accumulates online, so agreement is to rounding)."""
    import json
    import os
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "flash_attn_forward.json")
    with open(path) as f:
        cases = json.load(f)["cases"]
    n = 0
    for c in cases:
        if c["causal"]:
            continue
        shape = (c["B"], c["h"], c["L"], c["d"])
        f32 = lambda bits, shp: np.array(bits, dtype=np.uint32).view(np.float32).reshape(shp)  # noqa: E731
        q, k, v = f32(c["q"], shape), f32(c["k"], shape), f32(c["v"], shape)
        bias = f32(c["bias"], (c["B"], c["h"], c["L"], c["L"])) if c["bias"] is not None else None
        want = f32(c["o"], shape)
        # the graph's tensors are [L, D, h, B] (dims[0] first) = numpy (B, h, D, L)
        kg, qg, vg = (np.ascontiguousarray(t.transpose(0, 1, 3, 2)) for t in (k, q, v))
        scores = oracle.out_prod(kg, qg)                                   # [Lk, Lq, h, B] = numpy (B, h, Lq, Lk)
        scale = c["scale"] if c["scale"] > 0 else 1.0 / np.sqrt(np.float32(c["d"]))
        x = oracle.scale(scores, scale)
        if bias is not None:
            x = oracle.bcast_elemwise(x, bias, "add")
        attn = oracle.softmax(x)
        attn_t = oracle.permute(attn, (1, 0, 2, 3))                        # [Lq, Lk, h, B]
        v_t = oracle.permute(vg, (1, 0, 2, 3))                             # [D, Lk, h, B]
        out = oracle.out_prod(attn_t, v_t)                                 # [Lq, D, h, B] = numpy (B, h, D, Lq)
        got = out.transpose(0, 1, 3, 2)
        rows = np.isfinite(f32(c["lse"], shape[:3]))                       # fully masked rows: O = 0 there, NaN here
        np.testing.assert_allclose(got[rows], want[rows], rtol=2e-5, atol=2e-6)
        n += 1
    assert n >= 2
