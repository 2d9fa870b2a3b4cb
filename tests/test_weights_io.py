"""Load-time side of the int8 path on the CPU: weight selection, layout fingerprint and the checkpoint file of
include/ppml_hip_weights.h against the Python restatement in oracle/gguf_oracle.py, which is itself pinned here
(published FNV-1a vectors, a file written out by hand, the invariants of the format).  No GPU is needed: these
entry points are host code."""
import os
import struct

import numpy as np
import pytest

from oracle import gguf_oracle as orc


@pytest.fixture(scope="module")
def W():
    from proteinpredictmachinelearning_amd import weights

    return weights


# ----------------------------------------------------------------------------- fingerprint
def test_fnv1a_loop_reproduces_the_published_vectors():
    # FNV-1a 64-bit test vectors (Noll): the oracle's byte loop, started from the standard basis
    std = 14695981039346656037
    assert orc.fnv1a_feed(std, b"") == 0xcbf29ce484222325
    assert orc.fnv1a_feed(std, b"a") == 0xaf63dc4c8601ec8c
    assert orc.fnv1a_feed(std, b"foobar") == 0x85944171f73967e8
    # the reference starts from its own constant, one digit short of the standard one (src/model/GGUF.cpp:34)
    assert orc.FNV_OFFSET_BASIS == 1469598103934665603 and orc.FNV_PRIME == 1099511628211
    assert orc.fnv1a_layout_hash([], []) == orc.FNV_OFFSET_BASIS


def test_layout_hash_matches_oracle_and_is_order_sensitive(W):
    rng = np.random.default_rng(3)
    names = ["attention.msa_row.q_proj.weight", "", "bias", "x" * 70]
    shapes = [[256, 768], [32], [1, 2, 3, 4], [2 ** 33, 5]]
    assert W.fnv1a_layout_hash(names, shapes) == orc.fnv1a_layout_hash(names, shapes)
    assert W.fnv1a_layout_hash([], shapes) == orc.fnv1a_layout_hash([], shapes)          # "tensor_<i>" fallback
    assert W.fnv1a_layout_hash(["", "", "", ""], shapes) == W.fnv1a_layout_hash([], shapes)
    # two parameters of equal shape that change places change the fingerprint; so does a dimension
    a = W.fnv1a_layout_hash(["p", "q"], [[4, 4], [4, 4]])
    assert a != W.fnv1a_layout_hash(["q", "p"], [[4, 4], [4, 4]])
    assert a != W.fnv1a_layout_hash(["p", "q"], [[4, 4], [4, 5]])
    assert a != W.fnv1a_layout_hash(["p", "q"], [[4, 4], [16]])
    for _ in range(20):
        n = int(rng.integers(0, 6))
        nm = ["n%d_%d" % (i, rng.integers(100)) if rng.random() < 0.7 else "" for i in range(n)]
        sh = [[int(d) for d in rng.integers(1, 1000, size=rng.integers(1, 5))] for _ in range(n)]
        assert W.fnv1a_layout_hash(nm, sh) == orc.fnv1a_layout_hash(nm, sh)


# ----------------------------------------------------------------------------- weight selection
def test_selection_rule_cases(W):
    # src/model/PPML.cpp:4436-4456
    name = "blocks.3.attention.msa_row.q_proj.weight"
    for env, want in [(None, False), ("", False), ("0", False), ("off", False), ("1", True), ("on", True), ("all", True),
                      ("attention.msa_row.", True), ("attention.pair_row.", False), (" attention.msa_row. ", True),
                      ("foo,\tq_proj\t,bar", True), (",,,", False), ("foo, ,bar", False), ("weight", True),
                      ("OFF", False), ("On", False), ("00", False)]:
        assert W.int8_bigop_selected(name, env) is want, env
        assert orc.int8_bigop_selected(name, env) is want, env
    assert W.int8_bigop_default_list() == orc.int8_bigop_default_list()
    assert W.int8_bigop_default_list().count(",") == 7
    for nm in ["msa2pair_left_proj.weight", "msa2pair_out_proj.bias", "pair2pair_gate_proj.w", "attention.pair_col.o",
               "transition.linear1.weight", "embedding.table"]:
        assert W.int8_bigop_selected(nm, "all") == orc.int8_bigop_selected(nm, "all")
    assert not W.int8_bigop_selected("transition.linear1.weight", "all")
    # "0" as one fragment of a longer list is an ordinary fragment
    assert W.int8_bigop_selected("layer0.w", "0,x") and orc.int8_bigop_selected("layer0.w", "0,x")


def test_shape_rule(W):
    # src/model/PPML.cpp:4481-4488: 2-D, innermost dimension and element count multiples of 32
    for dims, want in [([256, 768], True), ([32, 1], True), ([250, 768], False), ([768], False), ([32, 4, 2], False),
                       ([64, 3], True), ([16, 2], False)]:
        assert W.int8_bigop_shape_ok(dims) is want
        assert orc.int8_bigop_shape_ok(dims) is want


# ----------------------------------------------------------------------------- the file
def _u64(v):
    return struct.pack("<Q", v)


def _u32(v):
    return struct.pack("<I", v)


def test_save_equals_a_file_written_by_hand(W, tmp_path):
    # save_gguf, src/model/GGUF.cpp:247-313, field by field for two small parameters
    a = np.array([1.0, 2.0], dtype=np.float32)
    b = np.array([3.0], dtype=np.float32)
    hash_hex = "%016x" % orc.fnv1a_layout_hash(["a", ""], [[2], [1]])
    exp = b"GGUF" + _u32(3) + _u64(2) + _u64(3)
    exp += _u64(4) + b"step" + _u32(6) + struct.pack("<f", 5.0)
    exp += _u64(11) + b"layout_hash" + _u32(8) + _u64(16) + hash_hex.encode()
    exp += _u64(4) + b"arch" + _u32(8) + _u64(1) + b"x"
    assert len(exp) == 24 + 20 + 47 + 25
    exp += _u64(1) + b"a" + _u32(1) + _u64(2) + _u32(0) + _u64(192)
    exp += _u64(8) + b"tensor_1" + _u32(1) + _u64(1) + _u32(0) + _u64(224)
    assert len(exp) == 189                                     # data start: the next multiple of 32
    exp += b"\0" * 3 + a.tobytes() + b"\0" * 24 + b.tobytes() + b"\0" * 28
    assert len(exp) == 256
    path = str(tmp_path / "tiny.gguf")
    W.save_gguf([a, b], path, float_meta=[("step", 5.0)], str_meta=[("arch", "x")], tensor_names=["a"])
    got = open(path, "rb").read()
    assert got == exp
    assert orc.save_gguf_bytes([([2], 0, a.tobytes()), ([1], 0, b.tobytes())], [("step", 5.0)], [("arch", "x")], ["a"]) == exp


def _random_model(rng, n, with_q8=False):
    params, oparams, names, shapes = [], [], [], []
    for i in range(n):
        nd = int(rng.integers(1, 4))
        shape = [int(d) for d in rng.integers(1, 9, size=nd)]      # numpy order, innermost last
        x = rng.standard_normal(shape).astype(np.float32)
        dims = list(reversed(shape))
        params.append(x)
        oparams.append((dims, 0, x.tobytes()))
        names.append("layer%d.weight" % i if rng.random() < 0.8 else "")
        shapes.append(dims)
    return params, oparams, names, shapes


def test_save_matches_oracle_byte_for_byte_and_keeps_the_format_invariants(W, tmp_path):
    rng = np.random.default_rng(11)
    for trial in range(8):
        params, oparams, names, shapes = _random_model(rng, int(rng.integers(0, 7)))
        extras = [("opt.m.layer%d" % j, rng.standard_normal(int(rng.integers(1, 50))).astype(np.float32)) for j in range(int(rng.integers(0, 3)))]
        fmeta = [("epoch", float(trial)), ("lr", 1.5e-3)][: int(rng.integers(0, 3))]
        smeta = [("ppml.arch", "ppml_v1")][: int(rng.integers(0, 2))]
        path = str(tmp_path / ("m%d.gguf" % trial))
        W.save_gguf(params, path, fmeta, smeta, names, extras)
        got = open(path, "rb").read()
        want = orc.save_gguf_bytes(oparams, fmeta, smeta, names, [(n, x.tobytes()) for n, x in extras])
        assert got == want
        floats, strings, tensors = orc.parse_gguf(got)
        assert len(got) % 32 == 0 or not tensors
        assert len(tensors) == len(params) + len(extras)
        prev_end = 0
        for (name, dims, typ, off), raw in zip(tensors, [p[2] for p in oparams] + [x.tobytes() for _, x in extras]):
            assert off % 32 == 0 and off >= prev_end and typ == 0
            assert got[off:off + len(raw)] == raw              # offsets count from the start of the file
            prev_end = off + len(raw)
        assert strings["layout_hash"] == "%016x" % orc.fnv1a_layout_hash(names, shapes)


def test_load_reads_back_what_was_saved_and_checks_like_the_reference(W, tmp_path):
    rng = np.random.default_rng(5)
    params, oparams, names, shapes = _random_model(rng, 5)
    names = ["p%d" % i for i in range(5)]
    extras = [("opt.m.p0", np.arange(7, dtype=np.float32)), ("opt.v.p0", np.ones(7, dtype=np.float32)),
              ("__g.extra", np.full(3, 2.5, dtype=np.float32)), ("other", np.zeros(2, dtype=np.float32))]
    path = str(tmp_path / "ck.gguf")
    W.save_gguf(params, path, [("epoch", 4.0), ("sample_pos", 123.0)], [("ppml.arch", "ppml_v1")], names, extras)
    loaded, raw = W.load_gguf(path, shapes, names)
    for x, y in zip(params, loaded):
        assert y.dtype == np.float32 and y.shape == x.shape and np.array_equal(x, y)
    assert sorted(raw) == ["__g.extra", "opt.m.p0", "opt.v.p0"]          # src/model/GGUF.cpp:417-430
    assert np.array_equal(raw["opt.m.p0"], np.arange(7, dtype=np.float32))
    with W.GgufFile(path) as f:
        assert len(f) == 9 and f.find("p3") == 3 and f.find("nope") == -1
        assert f.meta_float("epoch") == 4.0 and f.meta_float("sample_pos") == 123.0 and f.meta_float("none") is None
        assert f.meta_string("ppml.arch") == "ppml_v1" and len(f.meta_string("layout_hash")) == 16
        inf = f.info(2)
        assert inf["name"] == "p2" and list(inf["dims"]) == shapes[2] and inf["type"] == 0 and inf["offset"] % 32 == 0
        # the reference's checks and messages (src/model/GGUF.cpp:340-343, 404-415, 438-468)
        f.check_layout(shapes, names)
        f.check_layout(shapes)                                          # the file's own names
        with pytest.raises(RuntimeError, match="Tensor count mismatch: file=9 params=10"):
            f.check_layout(shapes + shapes, names + names)
        bad = [list(s) for s in shapes]
        bad[1][0] += 1
        with pytest.raises(RuntimeError, match=r"Shape mismatch for tensor 1 dim\[0\]"):
            f.check_layout(bad, names)
        bad = [list(s) for s in shapes]
        bad[4] = bad[4] + [1]
        with pytest.raises(RuntimeError, match="Dimension count mismatch for tensor 4"):
            f.check_layout(bad, names)
        swapped = list(names)
        swapped[0], swapped[1] = swapped[1], swapped[0]
        with pytest.raises(RuntimeError, match="Layout mismatch: file=[0-9a-f]{16} current=[0-9a-f]{16}"):
            f.check_layout(shapes, swapped)
    # a prefix of the parameters hashes differently from the whole list: the reference rejects it too
    with pytest.raises(RuntimeError, match="Layout mismatch"):
        W.load_gguf(path, shapes[:3], names[:3])


def test_open_rejects_what_the_reference_rejects(W, tmp_path):
    p = tmp_path / "bad.gguf"
    p.write_bytes(b"GGML" + _u32(3) + _u64(0) + _u64(0))
    with pytest.raises(RuntimeError, match="Not a GGUF file"):
        W.GgufFile(str(p))
    p.write_bytes(b"GGUF" + _u32(2) + _u64(0) + _u64(0))
    with pytest.raises(RuntimeError, match="Wrong version"):
        W.GgufFile(str(p))
    with pytest.raises(RuntimeError, match="cannot open"):
        W.GgufFile(str(tmp_path / "missing.gguf"))
    p.write_bytes(b"GGUF" + _u32(3) + _u64(1) + _u64(0) + _u64(10 ** 9))       # a name longer than the file
    with pytest.raises(RuntimeError):
        W.GgufFile(str(p))


def test_truncated_and_damaged_files_fail_cleanly(W, tmp_path):
    # every prefix of a good file and a few hundred files with bytes overwritten either open and read, or raise:
    # no tensor is ever read from outside the file
    import random

    rng = np.random.default_rng(1)
    params = [rng.standard_normal((3, 5)).astype(np.float32), rng.standard_normal(7).astype(np.float32)]
    good = str(tmp_path / "good.gguf")
    W.save_gguf(params, good, [("epoch", 2.0)], [("arch", "v1")], ["a", "b"], [("opt.m.a", np.ones(4, np.float32))])
    blob = open(good, "rb").read()
    p = tmp_path / "damaged.gguf"

    def exercise():
        try:
            with W.GgufFile(str(p)) as f:
                for i in range(len(f)):
                    try:
                        f.info(i)
                        f.read(i)
                    except (RuntimeError, IndexError):
                        pass
                try:
                    f.check_layout([[5, 3], [7]], ["a", "b"])
                except RuntimeError:
                    pass
            return True
        except RuntimeError:
            return False

    opened = 0
    for n in range(0, len(blob), 3):
        p.write_bytes(blob[:n])
        opened += exercise()
    assert 0 < opened < len(blob) // 3                    # short prefixes are rejected, long ones open
    random.seed(1)
    for _ in range(300):
        b = bytearray(blob)
        for _ in range(random.randint(1, 4)):
            b[random.randrange(len(b))] = random.randrange(256)
        p.write_bytes(bytes(b))
        exercise()


def test_metadata_of_every_type_is_read_or_skipped_like_the_reference(W, tmp_path):
    # src/model/GGUF.cpp:347-390: numbers of all widths become floats, small integers and arrays are skipped
    def kv(key, vtype, payload):
        return _u64(len(key)) + key.encode() + _u32(vtype) + payload
    meta = [kv("u8", 0, b"\x07"), kv("i8", 1, b"\xff"), kv("u16", 2, b"\x01\x02"), kv("i16", 3, b"\x03\x04"),
            kv("u32", 4, _u32(70000)), kv("i32", 5, _u32(12)), kv("f32", 6, struct.pack("<f", 1.25)), kv("flag", 7, b"\x01"),
            kv("s", 8, _u64(3) + b"abc"), kv("arr", 9, _u32(5) + _u64(3) + b"\0" * 12), kv("u64", 10, _u64(2 ** 40)),
            kv("i64", 11, _u64(9)), kv("f64", 12, struct.pack("<d", 2.5))]
    data = np.array([4.0, 5.0, 6.0], dtype=np.float32)
    blob = b"GGUF" + _u32(3) + _u64(1) + _u64(len(meta)) + b"".join(meta)
    info_len = 8 + 1 + 4 + 8 + 4 + 8
    off = (len(blob) + info_len + 31) // 32 * 32
    blob += _u64(1) + b"t" + _u32(1) + _u64(3) + _u32(0) + _u64(off)
    blob += b"\0" * (off - len(blob)) + data.tobytes()
    p = tmp_path / "meta.gguf"
    p.write_bytes(blob)
    floats, strings, tensors = orc.parse_gguf(blob)
    assert floats == {"u32": 70000.0, "i32": 12.0, "f32": 1.25, "u64": float(2 ** 40), "i64": 9.0, "f64": 2.5}
    assert strings == {"s": "abc"} and tensors == [("t", [3], 0, off)]
    with W.GgufFile(str(p)) as f:
        for k, v in floats.items():
            assert f.meta_float(k) == v
        for k in ("u8", "i8", "u16", "i16", "flag", "arr", "s"):
            assert f.meta_float(k) is None
        assert f.meta_string("s") == "abc"
        assert np.array_equal(f.read(0), data)
        f.check_layout([[3]])                                          # no layout_hash in the file: shapes only


def test_q8_0_parameter_is_stored_as_ggml_blocks(W, oracle, tmp_path):
    # beyond the reference, which refuses quantized parameters (src/model/GGUF.cpp:203-213)
    rng = np.random.default_rng(2)
    out_f, K = 6, 64
    w = rng.standard_normal((out_f, K)).astype(np.float32)
    blocks = oracle.quantize_q8_0(w)                                   # [out_f * K / 32] blocks of 34 bytes
    raw = np.ascontiguousarray(blocks).view(np.uint8).reshape(-1)
    assert raw.size == out_f * K // 32 * 34
    bias = rng.standard_normal(out_f).astype(np.float32)
    path = str(tmp_path / "q8.gguf")
    W.save_gguf([W.QuantizedWeight(raw, (K, out_f)), bias], path, tensor_names=["proj.weight", "proj.bias"])
    got = open(path, "rb").read()
    assert got == orc.save_gguf_bytes([([K, out_f], 8, raw.tobytes()), ([out_f], 0, bias.tobytes())], (), (), ["proj.weight", "proj.bias"])
    params, _ = W.load_gguf(path, [[K, out_f], [out_f]], ["proj.weight", "proj.bias"])
    assert isinstance(params[0], W.QuantizedWeight) and params[0].dims == (K, out_f)
    assert np.array_equal(params[0].blocks, raw) and np.array_equal(params[1], bias)
    with W.GgufFile(path) as f:
        assert f.info(0)["type"] == 8 and f.info(0)["nbytes"] == raw.size
    # rows may not split blocks, and the element count must fill whole blocks
    with pytest.raises(RuntimeError, match="cannot be stored"):
        W.save_gguf([W.QuantizedWeight(raw[:34 * 3], (48, 2))], str(tmp_path / "bad.gguf"))


def test_counts_and_dimensions_a_file_cannot_hold_are_refused(W, tmp_path):
    # a header that claims more tensors than the file could describe, and dimensions whose product wraps around
    # 2^64 to a small number: both must end in an ordinary refusal (no allocation by the claimed count, no
    # "small" tensor read from a shape that is not small)
    import struct

    good = str(tmp_path / "good.gguf")
    W.save_gguf([np.arange(15, dtype=np.float32).reshape(3, 5)], good, [], [], ["a"], [])
    blob = bytearray(open(good, "rb").read())
    assert struct.unpack_from("<Q", blob, 8)[0] == 1               # tensor count sits behind magic and version
    p = tmp_path / "bad.gguf"
    huge = bytearray(blob)
    struct.pack_into("<Q", huge, 8, len(blob) // 8)                # fits "count <= file size", not 24 bytes per tensor
    p.write_bytes(huge)
    with pytest.raises(RuntimeError, match="truncated header"):
        W.GgufFile(str(p))
    kv = bytearray(blob)
    struct.pack_into("<Q", kv, 16, len(blob) // 8)
    p.write_bytes(kv)
    with pytest.raises(RuntimeError, match="truncated"):
        W.GgufFile(str(p))
    # dims [5, 3] -> [2^63, 2]: the element count wraps to 0
    at = bytes(blob).index(struct.pack("<QQ", 5, 3))
    wrap = bytearray(blob)
    struct.pack_into("<QQ", wrap, at, 1 << 63, 2)
    p.write_bytes(wrap)
    with pytest.raises(RuntimeError, match="bad tensor info"):
        W.GgufFile(str(p))
