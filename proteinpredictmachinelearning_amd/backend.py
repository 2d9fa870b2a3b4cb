"""Graph-level driver: tensor nodes and the backend's ``graph_compute`` through the C ABI of
``include/ppml_hip_backend.h``.

The shape is the one the reference's tests use (tests/test_cuda.cpp:39-51 and 108-110): make device
leaves, make one node per op, hand the node list to ``graph_compute``, synchronize, copy back.
Numeric values of ops, types and statuses are the reference's (include/ppml/Tensor.h:35-64,
136-278; include/ppml/Backend.h:168-173).
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import cabi

# tensor_type
F32, F16, Q8_0, Q8_1, Q8_0R, Q8_0M = 0, 1, 8, 9, 19, 64
# tensor_op
OP_ADD, OP_SUB, OP_MUL, OP_DIV = 2, 6, 7, 8
OP_REPEAT_BACK = 21
OP_UNARY = 88
UNARY_OP_RELU = 4                      # include/ppml/ComputeGraph.h:20-25, kept in op_params[0]
FLAG_INPUT, FLAG_OUTPUT = 1, 2         # include/ppml/Tensor.h:19-22
OP_NONE, OP_MUL_MAT, OP_OUT_PROD, OP_SCALE, OP_RESHAPE, OP_VIEW, OP_PERMUTE, OP_TRANSPOSE, OP_SOFT_MAX = 0, 30, 32, 33, 37, 38, 39, 40, 47
OP_FLASH_ATTN_EXT, OP_FLASH_ATTN_BACK, OP_TRI_MUL, OP_TRI_MUL_BACK, OP_OUTER_PROD_MEAN, OP_OUTER_PROD_MEAN_BACK = \
    75, 76, 100, 101, 102, 103
# Status
SUCCESS, ALLOC_FAILED, NOT_SUPPORTED, ABORTED = 0, 1, 2, 3


class Tensor:
    """One tensor node.  ``dims[0]`` is the innermost dimension, as in the reference."""

    def __init__(self, dims, type=F32, op=OP_NONE, src=()):
        self._lib = cabi.load()
        self.dims = tuple(int(d) for d in dims)
        arr = (C.c_int64 * max(1, len(self.dims)))(*self.dims)
        self.handle = self._lib.ppml_hip_tensor_create(op, type, len(self.dims), arr)
        if not self.handle:
            raise ValueError(f"bad tensor description {dims}")
        self.src = list(src)
        for i, s in enumerate(self.src):
            if s is not None:
                self._lib.ppml_hip_tensor_set_src(self.handle, i, s.handle)

    def __del__(self):
        if getattr(self, "handle", None):
            self._lib.ppml_hip_tensor_destroy(self.handle)
            self.handle = None

    @property
    def nbytes(self) -> int:
        return self._lib.ppml_hip_tensor_nbytes(self.handle)

    @property
    def type(self) -> int:
        return self._lib.ppml_hip_tensor_type(self.handle)

    def bind(self, device_ptr: int) -> "Tensor":
        self._lib.ppml_hip_tensor_set_data(self.handle, C.c_void_p(device_ptr))
        return self

    def set_param(self, index: int, value) -> "Tensor":
        """op_params[index]: a Python float is stored by its binary32 bit pattern, an int as it is."""
        if isinstance(value, float):
            self._lib.ppml_hip_tensor_set_param(self.handle, index, value)
        else:
            self._lib.ppml_hip_tensor_set_param_i32(self.handle, index, int(value))
        return self

    def set_flag(self, flag: int) -> "Tensor":
        """The node's flag bits; a tensor marked FLAG_OUTPUT is never folded into a neighbour."""
        self._lib.ppml_hip_tensor_set_flag(self.handle, int(flag))
        return self

    def view_of(self, base: "Tensor", byte_offset: int = 0) -> "Tensor":
        self._base = base
        self._lib.ppml_hip_tensor_set_view(self.handle, base.handle, byte_offset)
        return self


class Backend:
    def __init__(self, device: int = 0):
        self._lib = cabi.load()
        self.handle = self._lib.ppml_hip_backend_create(device)
        if not self.handle:
            raise RuntimeError("no usable gfx950 device: " + cabi.last_error())

    def __del__(self):
        if getattr(self, "handle", None):
            self._lib.ppml_hip_backend_destroy(self.handle)
            self.handle = None

    @property
    def name(self) -> str:
        return self._lib.ppml_hip_backend_name(self.handle).decode()

    @property
    def priority(self) -> int:
        return self._lib.ppml_hip_backend_priority(self.handle)

    @property
    def last_error(self) -> str:
        return self._lib.ppml_hip_backend_last_error(self.handle).decode()

    def set_skip_alloc(self, on: bool) -> None:
        self._lib.ppml_hip_backend_set_skip_alloc(self.handle, int(on))

    def set_q8_1_activations(self, on: bool) -> None:
        self._lib.ppml_hip_backend_set_q8_1_activations(self.handle, int(on))

    def set_fuse_attention_bridges(self, on: bool) -> None:
        self._lib.ppml_hip_backend_set_fuse_attention_bridges(self.handle, int(on))

    def set_fuse_relu_into_q8(self, on: bool) -> None:
        self._lib.ppml_hip_backend_set_fuse_relu_into_q8(self.handle, int(on))

    def set_fuse_scale_into_out_prod(self, on: bool) -> None:
        self._lib.ppml_hip_backend_set_fuse_scale_into_out_prod(self.handle, int(on))

    def set_fuse_add_into_soft_max(self, on: bool) -> None:
        """On by default: an OP_ADD read only by an OP_SOFT_MAX (the attention bias) is added inside the softmax kernel."""
        self._lib.ppml_hip_backend_set_fuse_add_into_soft_max(self.handle, int(on))

    def set_fuse_permutes_into_out_prod(self, on: bool) -> None:
        """On by default: an OP_OUT_PROD of two {1,0,2,3} permutations nobody else reads contracts the unpermuted tensors."""
        self._lib.ppml_hip_backend_set_fuse_permutes_into_out_prod(self.handle, int(on))

    def set_fuse_permutes_into_mul_mat(self, on: bool) -> None:
        """On by default: an F32 OP_MUL_MAT of two matrix transpositions nobody else reads (a LinearLayer's weight
        gradient) contracts the untransposed matrices over their rows."""
        self._lib.ppml_hip_backend_set_fuse_permutes_into_mul_mat(self.handle, int(on))

    def set_fuse_attention_chain(self, on: bool) -> None:
        self._lib.ppml_hip_backend_set_fuse_attention_chain(self.handle, int(on))

    @property
    def nodes_fused_away(self) -> int:
        """Nodes the last graph_compute folded into a neighbour and did not execute."""
        return self._lib.ppml_hip_backend_nodes_fused_away(self.handle)

    def set_f32_arithmetic(self, mode) -> None:
        """"split", "fp32", or None for the calling thread's own choice (ppml_hip_backend_set_f32_arithmetic)."""
        self._lib.ppml_hip_backend_set_f32_arithmetic(self.handle, {"split": 0, "fp32": 1, None: -1}[mode])

    @property
    def host_shadows_made(self) -> int:
        """Host-resident sources the last graph_compute copied to the device for its duration."""
        return self._lib.ppml_hip_backend_host_shadows_made(self.handle)

    def upload(self, t: Tensor, host: np.ndarray) -> Tensor:
        host = np.ascontiguousarray(host)
        rc = self._lib.ppml_hip_tensor_upload(self.handle, t.handle, host.ctypes.data_as(C.c_void_p), host.nbytes)
        if rc:
            raise RuntimeError(f"upload failed with status {rc} (tensor needs {t.nbytes} bytes, got {host.nbytes})")
        return t

    def download(self, t: Tensor, dtype=np.float32) -> np.ndarray:
        out = np.empty(t.nbytes // np.dtype(dtype).itemsize, dtype=dtype)
        rc = self._lib.ppml_hip_tensor_download(self.handle, t.handle, out.ctypes.data_as(C.c_void_p), out.nbytes)
        if rc:
            raise RuntimeError(f"download failed with status {rc}")
        return out

    def supports_op(self, node: Tensor) -> bool:
        return bool(self._lib.ppml_hip_backend_supports_op(self.handle, node.handle))

    def graph_compute(self, nodes) -> int:
        arr = (C.c_void_p * len(nodes))(*[n.handle for n in nodes])
        return self._lib.ppml_hip_backend_graph_compute(self.handle, arr, len(nodes))

    def pack_weight(self, w: Tensor) -> int:
        return self._lib.ppml_hip_backend_pack_weight(self.handle, w.handle)

    def synchronize(self) -> None:
        self._lib.ppml_hip_backend_synchronize(self.handle)


def supports_op(node: Tensor) -> bool:
    """The scheduling rule alone; needs no device."""
    return bool(cabi.load().ppml_hip_backend_supports_op(None, node.handle))
