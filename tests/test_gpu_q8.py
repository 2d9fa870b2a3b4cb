"""GPU parity of the Q8_0 path against the CPU oracle, through the C ABI.

Bar: quantized bytes, fp16 scales and per-block int32 sums bit-exact; final f32 outputs within 1e-5
relative (measured against the largest magnitude of the row's settled terms, see ``_rel_err``).  The
kernel settles blocks in the oracle's order with the same fma, so the tests also report -- and at
these sizes require -- exact equality of the outputs.
"""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


@pytest.fixture(scope="module")
def ops():
    assert torch.cuda.is_available(), "GPU tests need a device"
    from proteinpredictmachinelearning_amd import ops as _ops

    return _ops


def _dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _rel_err(got, want):
    """max |got - want| / max |want|: the 1e-5 relative bar of the Q8 path."""
    return float(np.abs(got.astype(np.float64) - want.astype(np.float64)).max() / np.abs(want).max())


def _inputs(seed, N, K, M, wscale=0.02):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((N, K)).astype(np.float32)
    w = (rng.standard_normal((M, K)) * wscale).astype(np.float32)
    return x, w


def _q8_1_from_q8_0(blocks):
    """block_q8_1 records {half d; half s=d*sum(q); int8 qs[32]} from block_q8_0 records
    (include/ppml/QuantBlocks.h:38-41, 81-111 for the meaning of s)."""
    flat = blocks.reshape(-1, 34)
    out = np.zeros((flat.shape[0], 36), dtype=np.uint8)
    out[:, 0:2] = flat[:, 0:2]
    d = flat[:, 0:2].copy().view(np.float16)[:, 0].astype(np.float32)
    s = (d * flat[:, 2:].view(np.int8).astype(np.int32).sum(axis=1).astype(np.float32)).astype(np.float16)
    out[:, 2:4] = s.view(np.uint8).reshape(-1, 2)
    out[:, 4:] = flat[:, 2:]
    return out


# ----------------------------------------------------------------------------- quantizer
@pytest.mark.parametrize("rows,K,scale", [(408, 256, 1.0), (7, 32, 1.0), (33, 96, 0.02), (10609, 128, 1.0),
                                          (5, 2048, 1e-6), (3, 64, 1e4)])
def test_quantize_rows_bit_exact(ops, oracle, rows, K, scale):
    rng = np.random.default_rng(rows * 1000 + K)
    x = (rng.standard_normal((rows, K)) * scale).astype(np.float32)
    x[0, :32] = 0.0                                  # an all-zero block
    if K >= 64:
        x[-1, 32:64] = np.linspace(-127, 127, 32)    # d = 1: rounding ties hit exactly
        x[-1, 33] = 0.5
        x[-1, 34] = -2.5
    got = ops.quantize_rows_q8_0(_dev(x)).cpu().numpy()
    want = oracle.quantize_q8_0(x)
    assert got.shape == want.shape
    assert (got == want).all(), f"{(got != want).sum()} differing bytes"


def test_quantize_ties_and_nan_block(ops, oracle):
    x = np.zeros((2, 32), dtype=np.float32)
    x[0, 0] = 127.0
    x[0, 1:9] = [0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 0.49999997, -0.49999997]
    x[1, :] = 1.0
    x[1, 5] = -2.0
    got = ops.quantize_rows_q8_0(_dev(x)).cpu().numpy()
    assert (got == oracle.quantize_q8_0(x)).all()
    assert list(got[0, 0, 2:11].view(np.int8)) == [127, 1, -1, 2, -2, 3, -3, 0, 0]


def _exponent_sweep_blocks(seed):
    """One 32-element block per (largest-magnitude exponent, mantissa draw): every binary32 exponent from the
    subnormals to the top, so that the scale d = amax / 127 and its reciprocal pass through their subnormal,
    normal and overflowing ranges; the other elements are random fractions of the largest one, of either sign."""
    rng = np.random.default_rng(seed)
    exps = np.arange(0, 255, dtype=np.uint32)
    mant = rng.integers(0, 1 << 23, size=(exps.size, 24), dtype=np.uint32)
    mant[:, 0], mant[:, 1] = 0, (1 << 23) - 1
    top = ((exps[:, None] << 23) | mant).view(np.float32).reshape(-1)              # 255 * 24 largest magnitudes
    frac = rng.uniform(-1.0, 1.0, size=(top.size, 32)).astype(np.float32)
    x = (frac.astype(np.float64) * top[:, None].astype(np.float64)).astype(np.float32)
    pos = rng.integers(0, 32, size=top.size)
    x[np.arange(top.size), pos] = top * rng.choice(np.array([-1.0, 1.0], dtype=np.float32), size=top.size)
    x[5] = 0.0                                                                      # an all-zero block among them
    x[6] = -0.0                                                                     # ... of negative zeros
    x[7] = -np.abs(x[7])                                                            # nothing above zero, and
    x[7, 3] = -0.0                                                                  # a negative zero as the largest value
    x[8] = -np.abs(x[8])
    x[8, 0], x[8, 31] = -0.0, 0.0
    return x


def test_quantizers_over_the_whole_exponent_range(ops, oracle):
    # the scale and its reciprocal take a short exact form where both are normal numbers and the IEEE expansion
    # elsewhere: bytes and scales of both rules over every exponent the largest element can have
    x = _exponent_sweep_blocks(77)
    rows = x.shape[0]
    got0 = ops.quantize_rows_q8_0(_dev(x)).cpu().numpy()
    want0 = oracle.quantize_q8_0(x)
    assert (got0 == want0).all(), f"{(got0 != want0).any(axis=(1, 2)).sum()} of {rows} blocks differ (Q8_0 rule)"
    got1 = ops.quantize_rows_q8_1(_dev(x)).cpu().numpy()
    want1 = oracle.quantize_q8_1(x)
    assert (got1 == want1).all(), f"{(got1 != want1).any(axis=(1, 2)).sum()} of {rows} blocks differ (Q8_1 rule)"


@pytest.mark.parametrize("act", ["q8_0", "q8_1"])
@pytest.mark.parametrize("fam", ["general", "weight-stationary", "low-latency-8", "low-latency-16"])
def test_relu_quantizer_over_the_whole_exponent_range(ops, oracle, act, fam):
    # ReLU in front of the quantizer costs nothing in the kernels (signed maximum, clamp at zero): the blocks they
    # make of x must be the blocks of max(x, 0) under both rules, over every exponent, in every kernel family
    blocks = _exponent_sweep_blocks(78)
    K = 128
    x = blocks[: (blocks.shape[0] // 4) * 4].reshape(-1, K)
    _, w = _inputs(5, 1, K, 64)
    W = ops.Q8Weight.from_f32(_dev(w)).pack()
    for relu in (True, False):
        _, xq, _ = ops.mul_mat_q8(W, _dev(x), relu=relu, dump=True, act=act, path=fam)
        xr = np.maximum(x, 0.0) if relu else x
        if act == "q8_0":
            want = oracle.quantize_q8_0(xr)
        else:
            x1 = oracle.quantize_q8_1(xr)
            want = np.ascontiguousarray(np.concatenate([x1[..., 0:2], x1[..., 4:]], axis=-1))
        got = xq.cpu().numpy()
        assert (got == want).all(), f"relu={relu}: {(got != want).any(axis=2).sum()} of {want.shape[0] * want.shape[1]} blocks differ"


def test_dequantize_matches_oracle(ops, oracle):
    x, _ = _inputs(3, 17, 96, 1)
    blk = oracle.quantize_q8_0(x)
    got = ops.dequantize_q8_0(_dev(blk)).cpu().numpy()
    assert (got == oracle.dequantize_q8_0(blk)).all()


def test_quantize_rejects_ragged(ops):
    with pytest.raises(ValueError):
        ops.quantize_rows_q8_0(torch.zeros(4, 33, device="cuda"))
    from proteinpredictmachinelearning_amd import cabi
    lib = cabi.load()
    buf = torch.zeros(64, device="cuda")
    assert lib.quantize_rows_q8_0_hip(C.c_void_p(buf.data_ptr()), C.c_void_p(buf.data_ptr()), 33, None) == 1


# ----------------------------------------------------------------------------- fused linear
SHAPES = [
    # N tokens, K, M out features
    (408, 256, 256),      # the dev-config linear (8 x 51 MSA rows)
    (45, 32, 32),         # one block, ragged token tile
    (100, 96, 100),       # M not a multiple of 32, odd block count
    (64, 1056, 64),       # 33 blocks: K staged through LDS in two chunks
    (70, 128, 800),       # 25 column tiles: more than one column pass per work-group
    (33, 64, 300),        # 10 column tiles (8 waves x 2)
    (1, 512, 128),        # a single token
]


SHAPES += [
    # shapes with a weight-stationary instance when the weight is packed (K/32 in {4,8,16})
    (300, 128, 100),      # four-wave work-groups, four blocks
    (300, 128, 512),      # pair feed-forward up-projection, ragged last token tile
    (200, 512, 128),      # pair feed-forward down-projection
    (1000, 256, 768),     # MSA QKV projection: more token tiles than one pass of work-groups on a small grid
    (77, 256, 700),       # output features not a multiple of 32 (and not of 4 at the edge tile)
    (9000, 128, 100),     # more token tiles than CUs: the persistent loop and its double buffer
]

# one shape per remaining weight-stationary instance (column tiles per wave, K/32, waves per work-group), each
# with a ragged last token tile; WS_INSTANCE_SHAPES below lists every instance with a shape that reaches it
SHAPES += [
    (200, 128, 200),      # (1, 4) eight waves: 7 column tiles
    (150, 128, 700),      # (3, 4): 22 column tiles
    (300, 256, 400),      # (2, 8): 13 column tiles
    (300, 512, 200),      # (1, 16) eight waves: 7 column tiles
    (300, 256, 100),      # (1, 8) four waves: 4 column tiles
    (9000, 256, 400),     # (2, 8) with several token tiles per work-group (staged loads, three LDS buffers in turn)
    (9000, 512, 200),     # (1, 16) likewise: the 64-register staging range
    (17000, 128, 700),    # (3, 4) likewise, with leftover tiles shared between work-groups
    (3001, 512, 128),     # more than 2048 tokens: the library itself picks the low-latency kernel with 16-token units
    (3001, 128, 500),
    (3001, 256, 250),
    (300, 64, 64),        # (1, 2) four waves: K = 64, the 64 -> 64 projections of the full-MSA track
    (300, 64, 256),       # (1, 2) eight waves: its feed-forward 64 -> 256
    (9000, 64, 64),       # likewise with several token tiles per work-group
]

# (column tiles of 32 outputs) -> instance: up to 4 tiles the four-wave kernels, beyond that ceil(tiles / 8) per wave
WS_INSTANCE_SHAPES = {
    # (TPW, NBLK, waves): (N, K, M)
    (1, 2, 4): (300, 64, 64), (1, 2, 8): (300, 64, 256),
    (1, 4, 4): (300, 128, 100), (1, 8, 4): (300, 256, 100), (1, 16, 4): (200, 512, 128),
    (1, 4, 8): (200, 128, 200), (2, 4, 8): (300, 128, 512), (3, 4, 8): (150, 128, 700), (4, 4, 8): (70, 128, 800),
    (1, 8, 8): (408, 256, 256), (2, 8, 8): (300, 256, 400), (3, 8, 8): (1000, 256, 768),
    (1, 16, 8): (300, 512, 200),
}


@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("N,K,M", SHAPES)
def test_fused_linear_bit_exact_internals_and_output(ops, oracle, N, K, M, packed):
    x, w = _inputs(N + K + M, N, K, M)
    wq = oracle.quantize_q8_0(w)
    xq_want = oracle.quantize_q8_0(x)
    W = ops.Q8Weight(_dev(wq.reshape(-1)), M, K, ops.WTYPE_Q8_0)
    if packed:
        W = W.pack()
    out, xq, sums = ops.mul_mat_q8(W, _dev(x), c_trans=1, dump=True)
    out, xq, sums = out.cpu().numpy(), xq.cpu().numpy(), sums.cpu().numpy()
    assert (xq == xq_want).all(), "activation blocks differ from quantize_q8_0_host"
    assert (sums == oracle.q8_block_sums(wq, xq_want)).all(), "per-block int32 sums differ"
    want = oracle.mul_mat_q8(wq, x, wtype=0, c_trans=1, fma=1)
    assert _rel_err(out, want) <= 1e-5
    assert (out == want).all(), f"outputs not bit-identical: rel err {_rel_err(out, want):.3e}"
    # the undumped fast path gives the same bits
    fast = ops.mul_mat_q8(W, _dev(x), c_trans=1).cpu().numpy()
    assert (fast == out).all()
    if not packed:
        # a weight as the reference stores it: where one more launch costs less than the general kernel loses (from 2^27
        # products on; weights of 64 Ki elements with K >= 512 or 768 features at any token count) it is packed into the
        # stream's workspace per call and served by the kernels of the packed layout, where they have an instance
        repacked = N * M * K >= 2 ** 27 or (M * K >= 64 * 1024 and (K >= 512 or M >= 768))
        if repacked and _has_low_latency_instance(K, M) and N <= 4096:
            assert ops.last_q8_path() == "low-latency"
        elif repacked and _has_resident_weight_instance(K, M):
            assert ops.last_q8_path() == "weight-stationary"
        else:
            assert ops.last_q8_path() == "general"
        assert (ops.mul_mat_q8(W, _dev(x), c_trans=1, path="general").cpu().numpy() == out).all()
        assert ops.last_q8_path() == "general"
        return
    # a packed weight: every kernel family that has an instance for the shape, dump form and fast form
    families = ["general"]
    if _has_resident_weight_instance(K, M):
        families += ["weight-stationary", "weight-stationary-whole"]
    if _has_column_parts_instance(K, M):
        families.append("weight-stationary-column-parts")
    if _has_low_latency_instance(K, M):
        families += ["low-latency-8", "low-latency-16"]
        if K == 512:
            families.append("low-latency-32")          # units of 32 tokens: K = 512 only
    for fam in families:
        o2, xq2, sums2 = ops.mul_mat_q8(W, _dev(x), c_trans=1, dump=True, path=fam)
        assert ops.last_q8_path() == _FAMILY_PATH[fam], fam
        assert (o2.cpu().numpy() == want).all() and (xq2.cpu().numpy() == xq_want).all() and (sums2.cpu().numpy() == sums).all(), fam
        assert (ops.mul_mat_q8(W, _dev(x), c_trans=1, path=fam).cpu().numpy() == want).all(), fam
    # the library's own choice: low-latency for few tokens, else weight-stationary, else general
    ops.mul_mat_q8(W, _dev(x), c_trans=1)
    if _has_low_latency_instance(K, M) and N <= 4096:
        assert ops.last_q8_path() == "low-latency"
    elif _has_resident_weight_instance(K, M):
        assert ops.last_q8_path() == "weight-stationary"
    else:
        assert ops.last_q8_path() == "general"


def _takes_tiled(N, K, M):
    """The tiled kernel's own conditions: blocks in pairs, half a narrow tile of features, sixteen work-groups of the
    form it picks (tiles of 128 tokens x 128 features where their rounds over the CUs come cheaper than those of
    tiles twice as wide, which take 1.8 times as long each)."""
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    tiles_t, col_tiles = ((N + 31) // 32 + 3) // 4, (M + 31) // 32
    wide, narrow = tiles_t * ((col_tiles + 7) // 8), tiles_t * ((col_tiles + 3) // 4)
    takes_narrow = -(-narrow // cus) < 1.8 * -(-wide // cus)
    return (K // 32) % 2 == 0 and M >= 64 and (narrow if takes_narrow else wide) >= 16


def _has_resident_weight_instance(K, M):
    tiles, nblk = (M + 31) // 32, K // 32
    tpw = (tiles + 7) // 8
    return K % 32 == 0 and nblk in (2, 4, 8, 16) and (tiles <= 4 or tpw <= {2: 1, 4: 4, 8: 3, 16: 1}[nblk])


_FAMILY_PATH = {"general": "general", "weight-stationary": "weight-stationary", "weight-stationary-whole": "weight-stationary",
                "weight-stationary-column-parts": "weight-stationary", "low-latency-8": "low-latency", "low-latency-16": "low-latency",
                "low-latency-32": "low-latency"}


def _has_column_parts_instance(K, M):
    # several column tiles per wave, K of 128 or 256: that many work-groups can share a token tile, a part of
    # the columns each
    tiles, nblk = (M + 31) // 32, K // 32
    return K % 32 == 0 and nblk in (4, 8) and tiles > 8 and _has_resident_weight_instance(K, M)


def _has_low_latency_instance(K, M):
    # the wave's share of the weight (column tiles wave, wave + 4, ...) must fit 64 registers
    tiles, nblk = (M + 31) // 32, K // 32
    return K % 32 == 0 and nblk in (4, 8, 16) and tiles <= 4 * (16 // nblk)


def test_every_weight_stationary_instance_has_a_shape_in_the_suite():
    # the dispatch rule restated: up to four column tiles -> four-wave work-groups, one tile per wave; beyond
    # that eight waves with ceil(tiles / 8) tiles each.  Every instance the library builds is listed, and each
    # listed shape is one of SHAPES, so the parametrized test above runs it (dump and fast form).
    for (tpw, nblk, waves), (N, K, M) in WS_INSTANCE_SHAPES.items():
        tiles = (M + 31) // 32
        assert K // 32 == nblk
        assert (waves == 4) == (tiles <= 4)
        assert tpw == (1 if waves == 4 else (tiles + 7) // 8)
        assert (N, K, M) in SHAPES, (N, K, M)
    assert len(WS_INSTANCE_SHAPES) == 13


@pytest.mark.parametrize("N,K,M", [(408, 256, 256), (100, 96, 100), (70, 128, 800),
                                   (300, 512, 128), (2100, 256, 768)])      # the last two: packed per call by the library
def test_weight_layouts_and_output_orientations_agree(ops, oracle, N, K, M):
    x, w = _inputs(11 * N + M, N, K, M)
    wq = oracle.quantize_q8_0(w)
    want = oracle.mul_mat_q8(wq, x, wtype=0, c_trans=1, fma=1)
    xd = _dev(x)
    layouts = {
        ops.WTYPE_Q8_0: wq.reshape(-1),
        ops.WTYPE_Q8_1: _q8_1_from_q8_0(wq).reshape(-1),
        ops.WTYPE_Q8_0R: oracle.repack_q8_0(wq),
    }
    repacked = N * M * K >= 2 ** 27 or (M * K >= 64 * 1024 and (K >= 512 or M >= 768))
    for wtype, data in layouts.items():
        W = ops.Q8Weight(_dev(data), M, K, wtype)
        assert (ops.mul_mat_q8(W, xd, c_trans=1).cpu().numpy() == want).all(), wtype
        assert (ops.last_q8_path() != "general") == repacked, wtype
        assert (ops.mul_mat_q8(W, xd, c_trans=0).cpu().numpy() == want.T).all(), wtype
        Wm = W.pack()
        tiles = (((M + 31) // 32) + 1) // 2 * 2          # the packed layout holds an even number of 32-row tiles
        assert Wm.wtype == ops.WTYPE_Q8_0M and Wm.data.numel() == tiles * (K // 32) * 1088
        assert (ops.mul_mat_q8(Wm, xd, c_trans=1).cpu().numpy() == want).all(), wtype
        assert (ops.mul_mat_q8(Wm, xd, c_trans=0).cpu().numpy() == want.T).all(), wtype
    # quantizing the weight on the device gives the same blocks as the host quantizer
    Wd = ops.Q8Weight.from_f32(_dev(w))
    assert (Wd.data.cpu().numpy() == wq.reshape(-1)).all()


@pytest.mark.parametrize("N,K,M", [(300, 256, 1024), (2100, 256, 1024), (500, 128, 1500), (700, 256, 2048), (95, 128, 1100)])
def test_projections_wider_than_a_work_group_holds_go_in_column_parts(ops, oracle, N, K, M):
    """K = 256 beyond 768 output features and K = 128 beyond 1024 (the MSA feed-forward 256 -> 1024 if it is
    quantized) have no instance that keeps the whole weight in one work-group: several work-groups share each token
    tile, 256 columns each, whatever the token count.  Same bits as the oracle, internals included."""
    x, w = _inputs(N + M, N, K, M)
    wq = oracle.quantize_q8_0(w)
    W = ops.Q8Weight(_dev(wq.reshape(-1)), M, K, ops.WTYPE_Q8_0).pack()
    want = oracle.mul_mat_q8(wq, x, wtype=0, c_trans=1, fma=1)
    got = ops.mul_mat_q8(W, _dev(x), c_trans=1)
    assert ops.last_q8_path() == "weight-stationary"
    assert (got.cpu().numpy() == want).all()
    out, xq, sums = ops.mul_mat_q8(W, _dev(x), c_trans=1, dump=True)
    assert ops.last_q8_path() == "weight-stationary"
    xq_want = oracle.quantize_q8_0(x)
    assert (out.cpu().numpy() == want).all() and (xq.cpu().numpy() == xq_want).all()
    assert (sums.cpu().numpy() == oracle.q8_block_sums(wq, xq_want)).all()
    got = ops.mul_mat_q8(W, _dev(x), relu=True).cpu().numpy()
    assert (got == oracle.mul_mat_q8(wq, np.maximum(x, 0.0), wtype=0, c_trans=1, fma=1)).all()
    got = ops.mul_mat_q8(W, _dev(x), act="q8_1").cpu().numpy()
    assert (got == oracle.mul_mat_q8_act(wq, x, act=1, c_trans=1)).all()
    # told not to share the columns out, the call falls to the tiled kernel where there are sixteen tiles of 128 x 256
    # for it, else to the general one: same bits
    got = ops.mul_mat_q8(W, _dev(x), path="weight-stationary-whole")
    assert ops.last_q8_path() == ("tiled" if _takes_tiled(N, K, M) else "general") and (got.cpu().numpy() == want).all()
    # sentinels around C
    buf = torch.full((N * M + 2048,), 7.5, device="cuda")
    ops.mul_mat_q8(W, _dev(x), out=buf[1024:1024 + N * M].view(N, M))
    assert (buf[1024:1024 + N * M].view(N, M).cpu().numpy() == want).all()
    assert (buf[:1024] == 7.5).all() and (buf[1024 + N * M:] == 7.5).all()


# ----------------------------------------------------------------------------- tiled kernel (large weights)
@pytest.mark.parametrize("N,K,M", [(300, 256, 2100),      # ragged tokens and features; narrow tiles (51 work-groups in one round)
                                   (650, 1088, 600),      # 34 blocks; the last column tile of the last work-group is padding
                                   (2048, 64, 130),       # one stage; five column tiles, of a work-group's tiles some repeat the last
                                   (5000, 128, 1000)])    # wide tiles: 160 work-groups of 128 x 256 in one round (320 narrow ones would take two)
def test_tiled_kernel_bit_exact_against_the_oracle(ops, oracle, N, K, M):
    """A packed weight under enough tokens and features for sixteen tiles of 128 x 256: the activations are quantized
    ahead into fragment order and the contraction is cut like a GEMM.  Same block sums, same settlement, blocks
    ascending: the oracle's bits, in both output orientations, with ReLU and with the Q8_1 rule."""
    x, w = _inputs(3 * N + K + M, N, K, M)
    x[N // 2, :32] = 0.0                                # an all-zero block: scale 0, reciprocal replaced by 0
    wq = oracle.quantize_q8_0(w)
    W = ops.Q8Weight(_dev(wq.reshape(-1)), M, K, ops.WTYPE_Q8_0).pack()
    for c_trans in (1, 0):
        want = oracle.mul_mat_q8(wq, x, wtype=0, c_trans=c_trans, fma=1)
        got = ops.mul_mat_q8(W, _dev(x), c_trans=c_trans, path="tiled")
        assert ops.last_q8_path() == "tiled"
        assert (got.cpu().numpy() == want).all(), c_trans
        got = ops.mul_mat_q8(W, _dev(x), c_trans=c_trans, relu=True, path="tiled").cpu().numpy()
        assert (got == oracle.mul_mat_q8(wq, np.maximum(x, 0.0), wtype=0, c_trans=c_trans, fma=1)).all(), c_trans
        got = ops.mul_mat_q8(W, _dev(x), c_trans=c_trans, act="q8_1", path="tiled").cpu().numpy()
        assert ops.last_q8_path() == "tiled"
        assert (got == oracle.mul_mat_q8_act(wq, x, act=1, c_trans=c_trans)).all(), c_trans
    # sentinels around C, ragged last tiles in both directions
    buf = torch.full((N * M + 4096,), 7.5, device="cuda")
    ops.mul_mat_q8(W, _dev(x), out=buf[2048:2048 + N * M].view(N, M), path="tiled")
    assert ops.last_q8_path() == "tiled"
    assert (buf[2048:2048 + N * M].view(N, M).cpu().numpy() == oracle.mul_mat_q8(wq, x, wtype=0, c_trans=1, fma=1)).all()
    assert (buf[:2048] == 7.5).all() and (buf[2048 + N * M:] == 7.5).all()
    # the diagnostic buffers are the general kernel's, and so is the call when that kernel is asked for
    ops.mul_mat_q8(W, _dev(x), dump=True, path="tiled")
    assert ops.last_q8_path() == "general"
    ops.mul_mat_q8(W, _dev(x), path="general")
    assert ops.last_q8_path() == "general"


def test_tiled_kernel_is_the_librarys_choice_for_large_weights(ops):
    """Where the weight-stationary kernels have no instance (K = 2048; 4096 features under K = 512) the library
    takes the tiled kernel from sixteen work-groups on -- in tiles of 128 x 256 or of 128 x 128, whichever has the
    cheaper rounds over the CUs -- and its bits are the general kernel's; an odd number of blocks, few work-groups,
    fewer than 64 features or a weight that is not packed stay with the general kernel."""
    rng = np.random.default_rng(11)
    for N, K, M, want_path in [(408, 2048, 2048, "tiled"), (4096, 512, 4096, "tiled"), (1000, 2080, 512, "general"),
                               (1024, 1024, 256, "tiled"), (512, 1024, 256, "general"), (2048, 1024, 32, "general")]:
        x = _dev(rng.standard_normal((N, K)).astype(np.float32))
        w = _dev((rng.standard_normal((M, K)) * 0.02).astype(np.float32))
        W = ops.Q8Weight.from_f32(w)
        ref = ops.mul_mat_q8(W, x, path="general")
        assert ops.last_q8_path() == "general"
        # the weight as the reference stores it: tiled too where it is larger than anything that stays resident (it is
        # packed into the workspace on the way), else the general kernel
        got = ops.mul_mat_q8(W, x)
        assert ops.last_q8_path() == (want_path if M * K > 256 * 1024 else "general"), (N, K, M)
        assert torch.equal(got.view(torch.int32), ref.view(torch.int32)), (N, K, M)
        Wp = W.pack()
        for c_trans in (1, 0):
            got = ops.mul_mat_q8(Wp, x, c_trans=c_trans)
            assert ops.last_q8_path() == want_path, (N, K, M)
            gen = ops.mul_mat_q8(Wp, x, c_trans=c_trans, path="general")
            assert ops.last_q8_path() == "general"
            assert torch.equal(got.view(torch.int32), gen.view(torch.int32)), (N, K, M, c_trans)
            if c_trans:
                assert torch.equal(got.view(torch.int32), ref.view(torch.int32)), (N, K, M)


def test_tiled_kernel_on_the_references_weight_layouts(ops, oracle):
    """Q8_0, Q8_1 and Q8_0R weights (include/ppml/QuantBlocks.h:33-41, 123-133) beyond 256 Ki elements take the tiled
    kernel through a per-call repack into the workspace: the oracle's bits in both orientations."""
    N, K, M = 300, 512, 1000
    x, w = _inputs(77, N, K, M)
    wq = oracle.quantize_q8_0(w)
    want = oracle.mul_mat_q8(wq, x, wtype=0, c_trans=1, fma=1)
    layouts = {ops.WTYPE_Q8_0: wq.reshape(-1), ops.WTYPE_Q8_1: _q8_1_from_q8_0(wq).reshape(-1), ops.WTYPE_Q8_0R: oracle.repack_q8_0(wq)}
    for wtype, data in layouts.items():
        W = ops.Q8Weight(_dev(data), M, K, wtype)
        got = ops.mul_mat_q8(W, _dev(x), c_trans=1)
        assert ops.last_q8_path() == "tiled", wtype
        assert (got.cpu().numpy() == want).all(), wtype
        got = ops.mul_mat_q8(W, _dev(x), c_trans=0)
        assert ops.last_q8_path() == "tiled" and (got.cpu().numpy() == want.T).all(), wtype
        out, xq, sums = ops.mul_mat_q8(W, _dev(x), c_trans=1, dump=True)       # the diagnostic buffers: the general kernel
        assert ops.last_q8_path() == "general" and (out.cpu().numpy() == want).all(), wtype


def test_workspace_paths_from_several_threads_and_streams(ops):
    """The tiled kernel's quantized activations and the per-call repack of a weight in the reference's layouts live in the
    stream's kept workspace: calls from several host threads, each on a stream of its own, and from two threads that
    share one stream, with sizes that make the buffer grow and shrink in turn, give the bits of the same calls made one
    after the other."""
    import threading
    g = torch.Generator(device="cuda").manual_seed(31)
    cases = []
    for N, K, M, pack in ((600, 1024, 1024, True), (3000, 256, 768, False), (408, 2048, 2048, False), (300, 256, 256, True),
                          (2100, 128, 2050, True)):
        W = ops.Q8Weight.from_f32(torch.randn(M, K, device="cuda", generator=g) * 0.02)
        if pack:
            W = W.pack()
        x = torch.randn(N, K, device="cuda", generator=g)
        ref = ops.mul_mat_q8(W, x).clone()
        cases.append((W, x, ref, ops.last_q8_path()))
    assert [c[3] for c in cases] == ["tiled", "weight-stationary", "tiled", "low-latency", "weight-stationary"]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream() for _ in range(3)]
    errors = []

    def work(stream, seed):
        try:
            rng = np.random.default_rng(seed)
            with torch.cuda.stream(stream):
                for _ in range(20):
                    i = int(rng.integers(len(cases)))
                    W, x, ref, _ = cases[i]
                    out = ops.mul_mat_q8(W, x)
                    stream.synchronize()
                    if not torch.equal(out.view(torch.int32), ref.view(torch.int32)):
                        errors.append((seed, i))
        except Exception as e:                         # noqa: BLE001 -- reported below
            errors.append((seed, repr(e)))

    threads = [threading.Thread(target=work, args=(streams[0], 1)), threading.Thread(target=work, args=(streams[1], 2)),
               threading.Thread(target=work, args=(streams[2], 3)), threading.Thread(target=work, args=(streams[2], 4))]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    torch.cuda.synchronize()
    assert not errors, errors


def test_a_call_on_a_capturing_stream_takes_no_workspace(ops):
    """The tiled kernel's workspace comes from the stream-ordered pool, and a stream under capture gets none (what is
    allocated while a graph is recorded is gone before the graph runs): a call recorded into a graph takes the
    general kernel.  The graph is recorded and dropped, never run."""
    g = torch.Generator(device="cuda").manual_seed(9)
    N, K, M = 600, 1024, 1024
    W = ops.Q8Weight.from_f32(torch.randn(M, K, device="cuda", generator=g) * 0.02).pack()
    x = torch.randn(N, K, device="cuda", generator=g)
    out = torch.empty(N, M, device="cuda")
    ops.mul_mat_q8(W, x, out=out, path="general")        # eager first: nothing is set up for the first time under capture
    ops.mul_mat_q8(W, x, out=out)
    assert ops.last_q8_path() == "tiled"
    want = out.clone()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        ops.mul_mat_q8(W, x, out=out)
        recorded_path = ops.last_q8_path()
    del graph
    assert recorded_path == "general"
    ops.mul_mat_q8(W, x, out=out)                        # and the stream's kept buffer serves eager calls as before
    assert ops.last_q8_path() == "tiled" and torch.equal(out, want)


@pytest.mark.parametrize("key", sorted(WS_INSTANCE_SHAPES))
def test_features_outermost_output_on_the_weight_stationary_kernel(ops, oracle, key):
    """c_trans = 0 (the quantized weight was src[0], src/backend/CUDAKernels.cpp:761-777: C is [M][N]) with a packed
    weight: every weight-stationary instance has a form that stores this orientation; same bits as the oracle."""
    N, K, M = WS_INSTANCE_SHAPES[key]
    x, w = _inputs(5 * N + K + M, N, K, M)
    wq = oracle.quantize_q8_0(w)
    W = ops.Q8Weight(_dev(wq.reshape(-1)), M, K, ops.WTYPE_Q8_0).pack()
    want = oracle.mul_mat_q8(wq, x, wtype=0, c_trans=0, fma=1)
    assert want.shape == (M, N)
    got = ops.mul_mat_q8(W, _dev(x), c_trans=0)
    assert ops.last_q8_path() == "weight-stationary"
    assert (got.cpu().numpy() == want).all()
    # ragged token counts around the 32-token tile, and a single token
    for n in (1, 31, 33, 65):
        got = ops.mul_mat_q8(W, _dev(x[:n]), c_trans=0).cpu().numpy()
        assert got.shape == (M, n) and (got == want[:, :n]).all(), n
    # ReLU in the quantizer and the Q8_1 rule for the activations
    got = ops.mul_mat_q8(W, _dev(x), c_trans=0, relu=True).cpu().numpy()
    assert (got == oracle.mul_mat_q8(wq, np.maximum(x, 0.0), wtype=0, c_trans=0, fma=1)).all()
    got = ops.mul_mat_q8(W, _dev(x), c_trans=0, act="q8_1").cpu().numpy()
    assert (got == oracle.mul_mat_q8_act(wq, x, act=1, c_trans=0)).all()
    # the diagnostic buffers come from the general kernel in this orientation
    out, xq, sums = ops.mul_mat_q8(W, _dev(x), c_trans=0, dump=True)
    assert ops.last_q8_path() == "general" and (out.cpu().numpy() == want).all()
    # the general kernel on request
    assert (ops.mul_mat_q8(W, _dev(x), c_trans=0, path="general").cpu().numpy() == want).all()
    assert ops.last_q8_path() == "general"


@pytest.mark.parametrize("N,K,M", [(26368, 256, 768), (10609, 128, 512), (10609, 512, 128), (8500, 128, 100)])
def test_features_outermost_output_at_the_configured_sizes(ops, N, K, M):
    """Several rounds of tiles per work-group, the leftover tiles shared by column parts, the early quantization of
    the next tile (26368 x 256 -> 768 takes that instance) and rows of C that do not start on a line (10609
    tokens): the transposed result of the token-outermost call, which the oracle pins at these sizes."""
    x, w = _inputs(N + M, N, K, M)
    W = ops.Q8Weight.from_f32(_dev(w)).pack()
    xd = _dev(x)
    want = ops.mul_mat_q8(W, xd, c_trans=1, path="weight-stationary")
    got = ops.mul_mat_q8(W, xd, c_trans=0)
    assert ops.last_q8_path() == "weight-stationary"
    assert got.shape == (M, N) and torch.equal(got, want.T.contiguous())
    # a buffer with sentinels around C: nothing is written outside it
    buf = torch.full((M * N + 2048,), 7.5, device="cuda")
    out = buf[1024:1024 + M * N].view(M, N)
    ops.mul_mat_q8(W, xd, c_trans=0, out=out)
    assert torch.equal(out, got) and (buf[:1024] == 7.5).all() and (buf[1024 + M * N:] == 7.5).all()


def test_relu_fused_into_the_quantizer(ops, oracle):
    # pair-track feed-forward: linear1 -> ReLU -> linear2 (src/modules/Attention.cpp:1097-1104)
    x, w = _inputs(21, 200, 512, 128)
    wq = oracle.quantize_q8_0(w)
    W = ops.Q8Weight(_dev(wq.reshape(-1)), 128, 512, ops.WTYPE_Q8_0).pack()
    want = oracle.mul_mat_q8(wq, np.maximum(x, 0.0), wtype=0, c_trans=1, fma=1)
    for fam in ("auto", "general", "weight-stationary", "low-latency-8", "low-latency-16", "low-latency-32"):
        got = ops.mul_mat_q8(W, _dev(x), relu=True, path=fam).cpu().numpy()
        assert (got == want).all(), fam


def test_status_codes(ops):
    from proteinpredictmachinelearning_amd import cabi
    lib = cabi.load()
    buf = torch.zeros(4096, device="cuda")
    p = C.c_void_p(buf.data_ptr())
    path = C.c_int(7)
    assert lib.mul_mat_q8_hip(p, p, p, 4, 4, 48, 0, 1, C.byref(path), None) == 2 and path.value == 0
    assert lib.mul_mat_q8_hip(p, p, p, 4, 4, 32, 4, 1, C.byref(path), None) == 5
    assert lib.mul_mat_q8_hip(None, p, p, 4, 4, 32, 0, 1, None, None) == 1
    # *path_out: the reference's own rule (src/cuda/MulMatQ8Kernel.cu:493-496): its MMQ kernels (1) from 16 tokens
    # on or for a repacked weight, unless PPML_MMQ=0; the threshold is PPML_MMQ_MIN_N
    import os
    saved = {k: os.environ.pop(k, None) for k in ("PPML_MMQ", "PPML_MMQ_MIN_N")}
    try:
        assert lib.mul_mat_q8_hip(p, p, p, 4, 4, 32, 0, 1, C.byref(path), None) == 0 and path.value == 0
        assert lib.mul_mat_q8_hip(p, p, p, 4, 16, 32, 0, 1, C.byref(path), None) == 0 and path.value == 1
        assert lib.mul_mat_q8_hip(p, p, p, 4, 4, 32, 2, 1, C.byref(path), None) == 0 and path.value == 1
        os.environ["PPML_MMQ_MIN_N"] = "4"
        assert lib.mul_mat_q8_hip(p, p, p, 4, 4, 32, 0, 1, C.byref(path), None) == 0 and path.value == 1
        os.environ["PPML_MMQ"] = "0"
        assert lib.mul_mat_q8_hip(p, p, p, 4, 16, 32, 2, 1, C.byref(path), None) == 0 and path.value == 0
    finally:
        for k, v in saved.items():
            os.environ.pop(k, None)
            if v is not None:
                os.environ[k] = v
    with pytest.raises(ValueError):
        ops.mul_mat_q8(ops.Q8Weight(buf.view(torch.uint8)[:34 * 4], 4, 32, 0), torch.zeros(3, 64, device="cuda"))


# ----------------------------------------------------------------------------- the configured full-size shapes
def test_pair_feed_forward_shapes_full(ops, oracle):
    # X 10609 x 128 -> 512 -> ReLU -> 128, both layers checked against the oracle in full
    x, w1 = _inputs(103, 10609, 128, 512)
    rng = np.random.default_rng(104)
    w2 = (rng.standard_normal((128, 512)) * 0.02).astype(np.float32)
    w1q, w2q = oracle.quantize_q8_0(w1), oracle.quantize_q8_0(w2)
    W1 = ops.Q8Weight(_dev(w1q.reshape(-1)), 512, 128, 0).pack()
    W2 = ops.Q8Weight(_dev(w2q.reshape(-1)), 128, 512, 0).pack()
    y = ops.mul_mat_q8(W1, _dev(x))
    z = ops.mul_mat_q8(W2, y, relu=True).cpu().numpy()
    y = y.cpu().numpy()
    y_want = oracle.mul_mat_q8(w1q, x, fma=1)
    assert _rel_err(y, y_want) <= 1e-5 and (y == y_want).all()
    z_want = oracle.mul_mat_q8(w2q, np.maximum(y_want, 0.0), fma=1)
    assert _rel_err(z, z_want) <= 1e-5 and (z == z_want).all()


def test_down_projection_beyond_the_pair_length_takes_units_of_32_tokens(ops, oracle):
    # K = 512 with more tokens than units of 16 can hold resident (a pair tensor of L = 126: 15876 rows): the
    # low-latency kernel with units of 32 tokens, two work-groups per CU.  Sampled rows against the oracle, bit for bit;
    # rows are independent, so slices of 4000 rows (units of 16) must give the same bits; ReLU in front, ragged end.
    N, K, M = 15876, 512, 128
    x, w = _inputs(126, N, K, M)
    wq = oracle.quantize_q8_0(w)
    W = ops.Q8Weight(_dev(wq.reshape(-1)), M, K, 0).pack()
    xd = _dev(x)
    y = ops.mul_mat_q8(W, xd, relu=True)
    assert ops.last_q8_path() == "low-latency"
    idx = np.r_[0:40, N - 40:N, np.arange(13, N, 499)]
    want = oracle.mul_mat_q8(wq, np.maximum(x[idx], 0.0), fma=1)
    assert (y.cpu().numpy()[idx] == want).all()
    for r0 in range(0, N, 4000):
        part = ops.mul_mat_q8(W, xd[r0:r0 + 4000].contiguous(), relu=True)
        assert torch.equal(part, y[r0:r0 + 4000]), r0
    y1 = ops.mul_mat_q8(W, xd, relu=True, act="q8_1")
    part1 = ops.mul_mat_q8(W, xd[:4000].contiguous(), relu=True, act="q8_1")
    assert torch.equal(part1, y1[:4000])


def test_msa_qkv_shape_full_size_properties(ops, oracle):
    # 26368 x 256 -> 768: rows are independent, so (a) a strided sample of rows must equal the oracle
    # bit for bit, (b) permuting the token rows must permute the output rows, (c) zero rows give zeros.
    N, K, M = 26368, 256, 768
    x, w = _inputs(256103, N, K, M)
    x[12345] = 0.0
    wq = oracle.quantize_q8_0(w)
    W = ops.Q8Weight(_dev(wq.reshape(-1)), M, K, 0).pack()
    xd = _dev(x)
    y = ops.mul_mat_q8(W, xd)
    idx = np.r_[0:64, 12340:12350, N - 40:N, np.arange(97, N, 997)]
    want = oracle.mul_mat_q8(wq, x[idx], fma=1)
    got = y.cpu().numpy()
    assert (got[idx] == want).all()
    assert (got[12345] == 0).all()
    perm = torch.randperm(N, generator=torch.Generator().manual_seed(5)).cuda()
    y_perm = ops.mul_mat_q8(W, xd[perm].contiguous())
    assert torch.equal(y_perm, y[perm])
    # and the result approximates the unquantized product to quantization accuracy
    full = x[idx].astype(np.float64) @ w.astype(np.float64).T
    assert np.abs(got[idx] - full).max() <= 0.03 * np.abs(full).max()
    # From three whole rounds of tiles on, this shape's instance quantizes the next tile at the start of a tile
    # instead of two thirds in (another compiled form).  Rows are independent: a slice of 4096 rows launched alone
    # runs the other form and must give the same bits; so must the diagnostic form of the early kernel, whose dumped
    # blocks and sums are compared with the oracle on the sampled rows; and the same under the Q8_1 activation rule.
    part = ops.mul_mat_q8(W, xd[8192:12288].contiguous())
    assert torch.equal(part, y[8192:12288])
    yd, xq, sums = ops.mul_mat_q8(W, xd, dump=True)
    assert torch.equal(yd, y)
    want_q = oracle.quantize_q8_0(x[idx])
    xq_np = xq.cpu().numpy()
    assert (xq_np.reshape((N,) + want_q.shape[1:])[idx] == want_q).all()
    want_sums = oracle.q8_block_sums(wq, want_q[:80])
    sums_np = sums.cpu().numpy()
    assert (sums_np.reshape((N,) + want_sums.shape[1:])[idx[:80]] == want_sums).all()
    del xq_np, sums_np
    del yd, xq, sums
    y1 = ops.mul_mat_q8(W, xd, act="q8_1")
    part1 = ops.mul_mat_q8(W, xd[8192:12288].contiguous(), act="q8_1")
    assert torch.equal(part1, y1[8192:12288])
    assert not torch.equal(y1, y)


# ----------------------------------------------------------------------------- Q8_1 activation rule
@pytest.mark.parametrize("rows,K,scale", [(408, 256, 1.0), (7, 32, 1.0), (33, 96, 0.02), (2000, 128, 1.0),
                                          (5, 2048, 1e-6), (3, 64, 1e4)])
def test_quantize_rows_q8_1_bit_exact(ops, oracle, rows, K, scale):
    # the activation quantizer of the reference's CUDA path (include/ppml/QuantBlocks.h:81-111):
    # d, s and every quant byte for byte
    rng = np.random.default_rng(rows * 77 + K)
    x = (rng.standard_normal((rows, K)) * scale).astype(np.float32)
    x[0, :32] = 0.0                                   # zero block stores +0
    x[rows - 1, 3], x[rows - 1, 9] = 5.0, -5.0        # equal magnitudes: the first one gives the sign
    x[rows - 1, K - 32 + 30], x[rows - 1, K - 32 + 2] = 6.0, -6.0
    x[rows // 2, 7] = np.nan                          # ignored by the scan
    got = ops.quantize_rows_q8_1(_dev(x)).cpu().numpy()
    want = oracle.quantize_q8_1(x)
    assert got.shape == want.shape == (rows, K // 32, 36)
    nan_blk = (rows // 2, 0)
    mask = np.ones(got.shape[:2], bool)
    mask[nan_blk] = False                             # (int8)NaN is not portable: compare that block apart
    assert (got[mask] == want[mask]).all()
    assert (got[nan_blk][:2] == want[nan_blk][:2]).all()      # its scale comes from the finite elements
    back = ops.dequantize_q8_1(_dev(want)).cpu().numpy()
    d = np.ascontiguousarray(want[..., 0:2]).view(np.float16)[..., 0].astype(np.float32)
    q = np.ascontiguousarray(want[..., 4:]).view(np.int8).astype(np.float32)
    assert (back.reshape(rows, K // 32, 32) == d[..., None] * q).all()


@pytest.mark.parametrize("wname", ["Q8_0", "Q8_0R", "packed"])
@pytest.mark.parametrize("N,K,M,c_trans", [(408, 256, 256, 1), (77, 128, 96, 0), (300, 512, 128, 1), (1000, 256, 768, 1)])
def test_fused_linear_with_q8_1_activations(ops, oracle, wname, N, K, M, c_trans):
    # what mul_mat_q8_cuda computes (src/cuda/MulMatQ8Kernel.cu:483-527): Q8_1 activations, same
    # per-block settlement.  Internals and output bit for bit.
    x, w = _inputs(N + K + M, N, K, M)
    x[N // 2] *= -3.0
    wq = oracle.quantize_q8_0(w)
    if wname == "Q8_0R":
        W = ops.Q8Weight(_dev(oracle.repack_q8_0(wq)), M, K, 2)
    else:
        W = ops.Q8Weight(_dev(wq.reshape(-1)), M, K, 0)
        if wname == "packed":
            W = W.pack()
    y, xq, sums = ops.mul_mat_q8(W, _dev(x), c_trans=c_trans, dump=True, act="q8_1")
    x1 = oracle.quantize_q8_1(x)
    want_xq = np.ascontiguousarray(np.concatenate([x1[..., 0:2], x1[..., 4:]], axis=-1))
    assert (xq.cpu().numpy() == want_xq).all()
    assert (sums.cpu().numpy() == oracle.q8_block_sums(wq, want_xq)).all()
    want = oracle.mul_mat_q8_act(wq, x, act=1, c_trans=c_trans)
    got = y.cpu().numpy()
    assert _rel_err(got, want) <= 1e-5
    assert (got == want).all()
    # without the dump, and the two rules really differ
    y2 = ops.mul_mat_q8(W, _dev(x), c_trans=c_trans, act="q8_1").cpu().numpy()
    assert (y2 == want).all()
    # a packed weight gets the resident-weight kernels under this rule too, in either orientation -- and so does a weight in
    # one of the reference's layouts where the library packs it per call (here: K = 512, and 768 features)
    repacked = N * M * K >= 2 ** 27 or (M * K >= 64 * 1024 and (K >= 512 or M >= 768))
    assert (ops.last_q8_path() != "general") == (wname == "packed" or repacked)
    if wname == "packed" and c_trans == 1:
        for fam in ("weight-stationary", "weight-stationary-column-parts", "low-latency-8", "low-latency-16", "low-latency-32"):
            if fam.startswith("low") and (not _has_low_latency_instance(K, M) or (fam.endswith("32") and K != 512)):
                continue
            if fam.endswith("parts") and not _has_column_parts_instance(K, M):
                continue
            y3 = ops.mul_mat_q8(W, _dev(x), c_trans=1, act="q8_1", path=fam).cpu().numpy()
            assert ops.last_q8_path() == _FAMILY_PATH[fam]
            assert (y3 == want).all(), fam
    assert (ops.mul_mat_q8(W, _dev(x), c_trans=c_trans).cpu().numpy() != want).any()
