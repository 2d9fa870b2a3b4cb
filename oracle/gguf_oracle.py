"""CPU restatement of the reference's load-time side of the int8 path, in plain Python.

TEST INFRASTRUCTURE ONLY: nothing in the product imports this file; tests use it as the checker of
proteinpredictmachinelearning_amd/csrc/weights_io.hip.

Functions and the reference code they follow (paths relative to the reference tree):
  int8_bigop_default_list, int8_bigop_selected   src/model/PPML.cpp:4431-4456
  int8_bigop_shape_ok                            src/model/PPML.cpp:4481-4488
  fnv1a_layout_hash                              src/model/GGUF.cpp:31-74
  save_gguf_bytes                                src/model/GGUF.cpp:134-191 (layout), 194-316 (writing)
  parse_gguf                                     src/model/GGUF.cpp:318-400

How it is pinned (the reference's GGUF.cpp does not compile here: include/ppml/Tensor.h needs cuda_fp16.h, and
the reference holds no test or fixture of its own for these functions):
  * fnv1a_layout_hash: the byte-feeding and multiplication are checked against the published FNV-1a 64-bit
    test vectors by running the same loop from the standard offset basis; the reference's own basis
    (1469598103934665603, GGUF.cpp:34) is a literal;
  * save_gguf_bytes: a file of two small tensors written out by hand, field by field, in tests/test_weights_io.py,
    plus the invariants the format fixes (32-byte alignment of every tensor, ascending offsets, offsets counted
    from the start of the file, counts in the header);
  * int8_bigop_selected: the cases the reference's comments and code enumerate ("0"/"off", "1"/"on"/"all",
    blanks around fragments, empty fragments, substring match).
The Q8_0 tensor type (ggml type 8) is this build's extension: the reference refuses quantized parameters
(GGUF.cpp:203-213), so that part is pinned by the ggml block layout (34 bytes per 32 elements) and round trips.
"""
import struct

GGUF_MAGIC = 0x46554747
GGUF_VERSION = 3
GGUF_ALIGN = 32
FNV_OFFSET_BASIS = 1469598103934665603          # GGUF.cpp:34 (not the standard basis 14695981039346656037)
FNV_PRIME = 1099511628211
MASK64 = (1 << 64) - 1
TYPE_F32, TYPE_Q8_0 = 0, 8
VT_FLOAT32, VT_STRING = 6, 8


def int8_bigop_default_list():
    return ("attention.msa_row.,attention.msa_col.,attention.pair_row.,attention.pair_col.,"
            "msa2pair_left_proj,msa2pair_right_proj,msa2pair_out_proj,pair2pair_gate_proj")


def int8_bigop_selected(name, env_list):
    if not env_list:
        return False
    lst = env_list
    if lst in ("0", "off"):
        return False
    if lst in ("1", "on", "all"):
        lst = int8_bigop_default_list()
    for tok in lst.split(","):
        tok = tok.strip(" \t")
        if tok and tok in name:
            return True
    return False


def int8_bigop_shape_ok(dims):
    if len(dims) != 2:
        return False
    numel = dims[0] * dims[1]
    return dims[0] % 32 == 0 and numel % 32 == 0


def fnv1a_feed(h, data):
    for b in data:
        h ^= b
        h = (h * FNV_PRIME) & MASK64
    return h


def fnv1a_layout_hash(tensor_names, shapes, basis=FNV_OFFSET_BASIS):
    h = basis
    for i, shape in enumerate(shapes):
        name = tensor_names[i] if i < len(tensor_names) and tensor_names[i] else "tensor_%d" % i
        h = fnv1a_feed(h, name.encode())
        h = fnv1a_feed(h, struct.pack("<I", 0xFF))
        h = fnv1a_feed(h, struct.pack("<I", len(shape)))
        for d in shape:
            h = fnv1a_feed(h, struct.pack("<Q", d))
        h = fnv1a_feed(h, struct.pack("<I", 0xFE))
    return h


def _align_up(n, a):
    return (n + a - 1) // a * a


def _str(s):
    b = s.encode()
    return struct.pack("<Q", len(b)) + b


def save_gguf_bytes(params, float_meta=(), str_meta=(), tensor_names=(), extra_tensors=()):
    """params: list of (dims innermost first, type, raw bytes); extra_tensors: list of (name, raw bytes of a 1-D
    F32 tensor).  Returns the file as bytes."""
    names, infos = [], []
    for i, (dims, typ, data) in enumerate(params):
        names.append(tensor_names[i] if i < len(tensor_names) and tensor_names[i] else "tensor_%d" % i)
        infos.append((list(dims), typ, data))
    for name, data in extra_tensors:
        names.append(name)
        infos.append(([len(data) // 4], TYPE_F32, data))
    layout_hash = fnv1a_layout_hash(list(tensor_names), [p[0] for p in params])
    strings = [("layout_hash", "%016x" % layout_hash)] + list(str_meta)
    head = struct.pack("<IIQQ", GGUF_MAGIC, GGUF_VERSION, len(infos), len(float_meta) + len(strings))
    meta = b""
    for k, v in float_meta:
        meta += _str(k) + struct.pack("<I", VT_FLOAT32) + struct.pack("<f", v)
    for k, v in strings:
        meta += _str(k) + struct.pack("<I", VT_STRING) + _str(v)
    info_bytes = sum(8 + len(n.encode()) + 4 + 8 * len(inf[0]) + 4 + 8 for n, inf in zip(names, infos))
    data_start = _align_up(len(head) + len(meta) + info_bytes, GGUF_ALIGN)
    offsets, cur = [], data_start
    for dims, typ, data in infos:
        offsets.append(cur)
        cur = _align_up(cur + len(data), GGUF_ALIGN)
    tinfo = b""
    for name, (dims, typ, data), off in zip(names, infos, offsets):
        tinfo += _str(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
        tinfo += struct.pack("<I", typ) + struct.pack("<Q", off)
    out = bytearray(head + meta + tinfo)
    out += b"\0" * (data_start - len(out))
    for dims, typ, data in infos:
        out += data
        out += b"\0" * (_align_up(len(out), GGUF_ALIGN) - len(out))
    return bytes(out)


def parse_gguf(blob):
    """Header, metadata and tensor infos as load_gguf reads them: returns (floats, strings, tensors) with
    tensors = [(name, dims, type, offset)]."""
    pos = 0

    def take(fmt):
        nonlocal pos
        v = struct.unpack_from("<" + fmt, blob, pos)[0]
        pos += struct.calcsize("<" + fmt)
        return v

    def take_str():
        nonlocal pos
        n = take("Q")
        s = blob[pos:pos + n].decode()
        pos += n
        return s

    if take("I") != GGUF_MAGIC:
        raise ValueError("Not a GGUF file")
    if take("I") != GGUF_VERSION:
        raise ValueError("Wrong version")
    n_tensors, n_kv = take("Q"), take("Q")
    floats, strings = {}, {}
    for _ in range(n_kv):
        key = take_str()
        vt = take("I")
        if vt in (0, 1, 7):
            pos += 1
        elif vt in (2, 3):
            pos += 2
        elif vt == 6:
            floats[key] = take("f")
        elif vt in (4, 5):
            floats[key] = float(take("I"))
        elif vt in (10, 11):
            floats[key] = float(take("Q"))
        elif vt == 12:
            floats[key] = float(take("d"))
        elif vt == 8:
            strings[key] = take_str()
        elif vt == 9:
            take("I")
            alen = take("Q")
            pos += 4 * alen                              # taken as 4-byte elements (GGUF.cpp:383-389)
        else:
            raise ValueError("unknown metadata type")
    tensors = []
    for _ in range(n_tensors):
        name = take_str()
        nd = take("I")
        dims = [take("Q") for _ in range(nd)]
        typ = take("I")
        off = take("Q")
        tensors.append((name, dims, typ, off))
    return floats, strings, tensors
