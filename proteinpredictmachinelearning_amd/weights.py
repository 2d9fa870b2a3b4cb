"""Load-time side of the int8 path: weight selection, quantization of the selected weights on the device, and
the checkpoint file that carries them.  A thin host mirror of the reference's interface over the C ABI of
``include/ppml_hip_weights.h`` (same names, argument meaning and error behaviour):

* ``int8_bigop_default_list`` / ``int8_bigop_selected``      src/model/PPML.cpp:4431-4456
* ``quantize_big_weight_matrices``                            src/model/PPML.cpp:4461-4551
* ``save_gguf`` / ``load_gguf`` / ``fnv1a_layout_hash``       src/model/GGUF.cpp:194-470, 52-74

The reference refuses to save quantized parameters (GGUF.cpp:203-213); here a Q8_0 parameter is written as
ggml type 8 and read back as the bytes ``mul_mat_q8`` takes.  Errors are raised as ``RuntimeError`` with the
text the reference throws.
"""
from __future__ import annotations

import ctypes as C
import os
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

from . import cabi

TYPE_F32 = 0
TYPE_Q8_0 = 8
QK = 32
Q8_0_BYTES = 34


def int8_bigop_default_list() -> str:
    return cabi.load().ppml_int8_bigop_default_list().decode()


def int8_bigop_selected(name: str, env_list: Optional[str]) -> bool:
    return bool(cabi.load().ppml_int8_bigop_selected(name.encode(), None if env_list is None else env_list.encode()))


def int8_bigop_shape_ok(dims: Sequence[int]) -> bool:
    arr = (C.c_uint64 * max(1, len(dims)))(*dims)
    return bool(cabi.load().ppml_int8_bigop_shape_ok(len(dims), arr))


class QuantizedWeight:
    """A Q8_0 parameter: ``blocks`` is a uint8 array of numel / 32 blocks of 34 bytes (host numpy array or device
    tensor), ``dims`` the logical dimensions, innermost (K) first, as in the reference's tensors."""

    def __init__(self, blocks, dims: Sequence[int]):
        self.blocks = blocks
        self.dims = tuple(int(d) for d in dims)

    @property
    def numel(self) -> int:
        n = 1
        for d in self.dims:
            n *= d
        return n


def quantize_big_weight_matrices(named_params: Sequence[Tuple[str, "object"]], env_list: Optional[str] = None,
                                 training: bool = False):
    """The rule of ``PPMLModel::quantize_big_weight_matrices``: every F32 parameter whose name is selected by
    ``env_list`` (default: the environment variable ``PPML_INT8_BIGOPS``) and whose shape qualifies is replaced by
    its Q8_0 blocks, quantized on the device; nothing happens in training mode.  ``named_params`` holds
    ``(name, tensor)`` with device tensors of shape ``[out, K]`` (dims ``{K, out}`` in the reference's order).
    Returns ``(new list, report)`` with ``report = {"done", "skipped_shape", "bytes_before", "bytes_after"}``."""
    from . import ops

    if env_list is None:
        env_list = os.environ.get("PPML_INT8_BIGOPS")
    report = {"done": 0, "skipped_shape": 0, "bytes_before": 0, "bytes_after": 0}
    out = list(named_params)
    if not env_list or env_list in ("0", "off") or training:
        return out, report
    for i, (name, t) in enumerate(out):
        if isinstance(t, QuantizedWeight):
            continue                                   # already quantized: the rule is idempotent
        if not int8_bigop_selected(name, env_list):
            continue
        dims = tuple(reversed(t.shape))                # innermost first
        if not int8_bigop_shape_ok(dims):
            report["skipped_shape"] += 1
            continue
        blocks = ops.quantize_rows_q8_0(t.contiguous())
        out[i] = (name, QuantizedWeight(blocks, dims))
        report["done"] += 1
        report["bytes_before"] += t.numel() * 4
        report["bytes_after"] += t.numel() // QK * Q8_0_BYTES
    return out, report


def fnv1a_layout_hash(tensor_names: Sequence[str], shapes: Sequence[Sequence[int]]) -> int:
    n = len(shapes)
    names = (C.c_char_p * max(1, n))(*[(tensor_names[i] if i < len(tensor_names) else "").encode() for i in range(n)])
    ndims = (C.c_uint32 * max(1, n))(*[len(s) for s in shapes])
    flat = [int(d) for s in shapes for d in s]
    dims = (C.c_uint64 * max(1, len(flat)))(*flat)
    return int(cabi.load().ppml_gguf_layout_hash(n, names, ndims, dims))


def _host_bytes(t) -> np.ndarray:
    if isinstance(t, np.ndarray):
        return np.ascontiguousarray(t)
    return np.ascontiguousarray(t.detach().cpu().numpy())


def save_gguf(params: Sequence, path: str, float_meta: Sequence[Tuple[str, float]] = (),
              str_meta: Sequence[Tuple[str, str]] = (), tensor_names: Sequence[str] = (),
              extra_tensors: Sequence[Tuple[str, "object"]] = ()) -> None:
    """``save_gguf`` of the reference.  ``params``: float32 arrays / tensors (numpy shape ``[.., K]``, written with
    the innermost dimension first as the reference's tensors have it) or ``QuantizedWeight``; ``extra_tensors``:
    ``(name, 1-D float32)`` optimizer state, outside the layout fingerprint."""
    lib = cabi.load()
    n_params, n_extra = len(params), len(extra_tensors)
    descs = (cabi.GgufTensor * max(1, n_params + n_extra))()
    keep = []
    for i, prm in enumerate(params):
        name = tensor_names[i] if i < len(tensor_names) else ""
        if isinstance(prm, QuantizedWeight):
            data, dims, typ = _host_bytes(prm.blocks).view(np.uint8).reshape(-1), prm.dims, TYPE_Q8_0
        else:
            data = _host_bytes(prm).astype(np.float32, copy=False)
            dims, typ = tuple(reversed(data.shape)) if data.ndim else (1,), TYPE_F32
        keep.append(data)
        descs[i].name = name.encode()
        descs[i].ndim = len(dims)
        for d in range(4):
            descs[i].dims[d] = dims[d] if d < len(dims) else 1
        descs[i].type = typ
        descs[i].data = data.ctypes.data
    for j, (name, arr) in enumerate(extra_tensors):
        data = _host_bytes(arr).astype(np.float32, copy=False).reshape(-1)
        keep.append(data)
        d = descs[n_params + j]
        d.name, d.ndim, d.type, d.data = name.encode(), 1, TYPE_F32, data.ctypes.data
        d.dims[0], d.dims[1], d.dims[2], d.dims[3] = data.size, 1, 1, 1
    fk = (C.c_char_p * max(1, len(float_meta)))(*[k.encode() for k, _ in float_meta])
    fv = (C.c_float * max(1, len(float_meta)))(*[float(v) for _, v in float_meta])
    sk = (C.c_char_p * max(1, len(str_meta)))(*[k.encode() for k, _ in str_meta])
    sv = (C.c_char_p * max(1, len(str_meta)))(*[v.encode() for _, v in str_meta])
    rc = lib.ppml_gguf_save(path.encode(), descs, n_params, n_extra, fk, fv, len(float_meta), sk, sv, len(str_meta))
    if rc:
        raise RuntimeError(cabi.last_error())


class GgufFile:
    """An open checkpoint: tensor infos and metadata parsed as ``load_gguf`` parses them."""

    def __init__(self, path: str):
        self._lib = cabi.load()
        self._h = self._lib.ppml_gguf_open(path.encode())
        if not self._h:
            raise RuntimeError(cabi.last_error())
        self._size = os.path.getsize(path)

    def close(self) -> None:
        if self._h:
            self._lib.ppml_gguf_close(self._h)
            self._h = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __len__(self) -> int:
        return int(self._lib.ppml_gguf_tensor_count(self._h))

    def info(self, i: int) -> Dict:
        name, ndim, typ = C.c_char_p(), C.c_uint32(), C.c_uint32()
        dims, off, nb = (C.c_uint64 * 4)(), C.c_uint64(), C.c_uint64()
        if self._lib.ppml_gguf_tensor_info(self._h, i, C.byref(name), C.byref(ndim), dims, C.byref(typ), C.byref(off), C.byref(nb)):
            raise IndexError(cabi.last_error())
        return {"name": name.value.decode(errors="replace"), "dims": tuple(dims[d] for d in range(ndim.value)), "type": typ.value,
                "offset": off.value, "nbytes": nb.value}

    def find(self, name: str) -> int:
        return int(self._lib.ppml_gguf_find_tensor(self._h, name.encode()))

    def read(self, i: int):
        """Tensor i: a float32 array of numpy shape ``reversed(dims)`` or a ``QuantizedWeight`` with host blocks."""
        inf = self.info(i)
        if inf["nbytes"] == 0 or inf["offset"] > self._size or inf["nbytes"] > self._size - inf["offset"]:
            raise RuntimeError(f"tensor {inf['name']!r} has an unknown type or lies outside the file")
        buf = np.empty(inf["nbytes"], dtype=np.uint8)
        if self._lib.ppml_gguf_read_tensor(self._h, i, buf.ctypes.data, buf.size):
            raise RuntimeError(cabi.last_error())
        if inf["type"] == TYPE_Q8_0:
            return QuantizedWeight(buf, inf["dims"])
        try:
            return buf.view(np.float32).reshape(tuple(reversed(inf["dims"])))
        except ValueError as e:                      # dimensions whose product does not fit the stored size
            raise RuntimeError(f"tensor {inf['name']!r}: {e}") from None

    def meta_float(self, key: str) -> Optional[float]:
        v = C.c_float()
        return None if self._lib.ppml_gguf_meta_float(self._h, key.encode(), C.byref(v)) else float(v.value)

    def meta_string(self, key: str) -> Optional[str]:
        s = self._lib.ppml_gguf_meta_string(self._h, key.encode())
        return None if s is None else s.decode()

    def check_layout(self, shapes: Sequence[Sequence[int]], tensor_names: Optional[Sequence[str]] = None) -> None:
        n = len(shapes)
        names = None
        if tensor_names:
            names = (C.c_char_p * max(1, n))(*[(tensor_names[i] if i < len(tensor_names) else "").encode() for i in range(n)])
        ndims = (C.c_uint32 * max(1, n))(*[len(s) for s in shapes])
        flat = [int(d) for s in shapes for d in s]
        dims = (C.c_uint64 * max(1, len(flat)))(*flat)
        if self._lib.ppml_gguf_check_layout(self._h, n, names, ndims, dims):
            raise RuntimeError(cabi.last_error())


def load_gguf(path: str, shapes: Sequence[Sequence[int]], tensor_names: Sequence[str] = ()):
    """``load_gguf`` of the reference for a model whose parameters have ``shapes`` (innermost dimension first):
    checks count, shapes and the layout fingerprint, and returns ``(params, raw_tensors)``: the parameters in file
    order (float32 arrays or ``QuantizedWeight``) and the extra 1-D tensors named ``opt.*`` / ``__g.*``
    (src/model/GGUF.cpp:417-430).  Metadata are read through ``GgufFile.meta_float`` / ``meta_string``."""
    with GgufFile(path) as f:
        f.check_layout(shapes, tensor_names or None)
        params = [f.read(i) for i in range(len(shapes))]
        raw: Dict[str, np.ndarray] = {}
        for i in range(len(shapes), len(f)):
            inf = f.info(i)
            if not (inf["name"].startswith("opt.") or inf["name"].startswith("__g.")) or len(inf["dims"]) != 1:
                continue
            raw[inf["name"]] = f.read(i).reshape(-1)
        return params, raw
