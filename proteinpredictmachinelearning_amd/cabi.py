"""ctypes binding of the gfx950 backend library (``lib/libppml_hip.so``).

The signatures below are the ones ``include/ppml_hip.h`` declares.  There is no fallback: if the
library is missing, or it was built for another GPU, loading fails loudly.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libppml_hip.so")

_i, _i64, _f, _vp = C.c_int, C.c_int64, C.c_float, C.c_void_p

# name -> (restype, argtypes); every symbol include/ppml_hip.h declares
SIGNATURES = {
    "ppml_hip_abi_version": (_i, []),
    "ppml_hip_init": (_i, [_i]),
    "ppml_hip_synchronize": (_i, []),
    "ppml_hip_last_error": (C.c_char_p, []),
    "ppml_hip_set_f32_arithmetic": (_i, [_i]),
    "mul_mat_hip": (_i, [_vp, _vp, _vp, _i, _i, _i, _vp, _vp]),
    "mul_mat_f16_hip": (_i, [_vp, _vp, _vp, _i, _i, _i, _vp, _vp]),
    "quantize_rows_q8_0_hip": (_i, [_vp, _vp, _i64, _vp]),
    "dequantize_q8_0_hip": (_i, [_vp, _vp, _i64, _vp]),
    "quantize_rows_q8_1_hip": (_i, [_vp, _vp, _i64, _vp]),
    "dequantize_q8_1_hip": (_i, [_vp, _vp, _i64, _vp]),
    "q8_weight_packed_bytes_hip": (C.c_size_t, [_i, _i]),
    "q8_weight_pack_hip": (_i, [_vp, _i, _i, _i, _vp, _vp]),
    "mul_mat_q8_hip": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, C.POINTER(_i), _vp]),
    "mul_mat_q8_ex_hip": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp, _vp, _vp]),
    "out_prod_hip": (_i, [_vp, _vp, _vp] + [_i64] * 12 + [_vp]),
    "out_prod_scaled_hip": (_i, [_vp, _vp, _vp] + [_i64] * 12 + [_f, _vp]),
    "out_prod_tt_hip": (_i, [_vp, _vp, _vp] + [_i64] * 12 + [_vp]),
    "outer_prod_mean_hip": (_i, [_vp, _vp, _vp] + [_i64] * 4 + [_f, _vp]),
    "outer_prod_mean_back_hip": (_i, [_vp] * 5 + [_i64] * 4 + [_f, _vp]),
    "outer_product_mean_value_hip": (_i, [_vp, _vp, _vp] + [_i64] * 4 + [_vp]),
    "mul_mat_tn_hip": (_i, [_vp, _vp, _vp, _i, _i, _i, _f, _vp]),
    "mul_mat_tn_noalloc_hip": (_i, [_vp, _vp, _vp, _i, _i, _i, _f, _vp]),
    "tri_mul_hip": (_i, [_vp, _vp, _vp] + [_i64] * 5 + [_f, _i, _vp]),
    "tri_mul_back_hip": (_i, [_vp] * 5 + [_i64] * 5 + [_f, _i, _vp]),
    "flash_attn_forward_hip": (_i, [_i] * 5 + [_f, _f, _i] + [_vp] * 7),
    "flash_attn_backward_hip": (_i, [_i] * 5 + [_f] + [_vp] * 12),
    "flash_attn_forward_ex_hip": (_i, [_i] * 5 + [_f, _f, _i] + [_vp] * 6 + [_i, _vp]),
    "permute_hip": (_i, [_vp, _vp, _i64, _i] + [_i] * 4 + [_i64] * 8 + [_vp]),
    "repeat_back_hip": (_i, [_vp, _vp] + [_i64] * 12 + [_vp]),
    "scale_hip": (_i, [_vp, _vp, _f, _i64, _vp]),
    "unary_hip": (_i, [_vp, _vp, _i64, _i, _vp]),
    "bcast_elemwise_hip": (_i, [_vp, _vp, _vp, _i64, _i64, _i64, _i, _vp]),
    "softmax_hip": (_i, [_vp, _vp, _i, _i, _vp]),
    "softmax_add_hip": (_i, [_vp, _vp, _vp, _i, _i, _i, _vp]),
    "ppml_hip_mulmat_stats": (_i, [C.POINTER(_i64), _i]),
    "ppml_hip_mulmat_stats_enable": (_i, [_i]),
    "ppml_hip_mulmat_stats_rows": (_i, [_vp, _i]),
    "ppml_hip_mulmat_stats_dump": (None, []),
    "ppml_hip_mulmat_stats_reset": (None, []),
    "ppml_hip_q8_last_path": (_i, []),
}


class MulMatStat(C.Structure):
    """``ppml_hip_mulmat_stat`` of include/ppml_hip.h."""
    _fields_ = [("path", C.c_char * 32), ("M", C.c_int64), ("K", C.c_int64), ("N", C.c_int64),
                ("calls", C.c_int64), ("ms", C.c_double)]


# every symbol include/ppml_hip_backend.h declares (the executor driver above the launchers)
BACKEND_SIGNATURES = {
    "ppml_hip_backend_create": (_vp, [_i]),
    "ppml_hip_backend_destroy": (None, [_vp]),
    "ppml_hip_backend_name": (C.c_char_p, [_vp]),
    "ppml_hip_backend_last_error": (C.c_char_p, [_vp]),
    "ppml_hip_backend_priority": (_i, [_vp]),
    "ppml_hip_backend_synchronize": (None, [_vp]),
    "ppml_hip_tensor_create": (_vp, [_i, _i, _i, C.POINTER(_i64)]),
    "ppml_hip_tensor_destroy": (None, [_vp]),
    "ppml_hip_tensor_set_src": (None, [_vp, _i, _vp]),
    "ppml_hip_tensor_set_data": (None, [_vp, _vp]),
    "ppml_hip_tensor_set_view": (None, [_vp, _vp, C.c_size_t]),
    "ppml_hip_tensor_set_param": (None, [_vp, _i, _f]),
    "ppml_hip_tensor_set_param_i32": (None, [_vp, _i, _i]),
    "ppml_hip_tensor_set_flag": (None, [_vp, _i]),
    "ppml_hip_tensor_nbytes": (C.c_size_t, [_vp]),
    "ppml_hip_tensor_type": (_i, [_vp]),
    "ppml_hip_tensor_upload": (_i, [_vp, _vp, _vp, C.c_size_t]),
    "ppml_hip_tensor_download": (_i, [_vp, _vp, _vp, C.c_size_t]),
    "ppml_hip_backend_supports_op": (_i, [_vp, _vp]),
    "ppml_hip_backend_set_skip_alloc": (None, [_vp, _i]),
    "ppml_hip_backend_set_q8_1_activations": (None, [_vp, _i]),
    "ppml_hip_backend_set_fuse_attention_bridges": (None, [_vp, _i]),
    "ppml_hip_backend_set_fuse_relu_into_q8": (None, [_vp, _i]),
    "ppml_hip_backend_set_fuse_scale_into_out_prod": (None, [_vp, _i]),
    "ppml_hip_backend_set_fuse_add_into_soft_max": (None, [_vp, _i]),
    "ppml_hip_backend_set_fuse_permutes_into_out_prod": (None, [_vp, _i]),
    "ppml_hip_backend_set_fuse_permutes_into_mul_mat": (None, [_vp, _i]),
    "ppml_hip_backend_set_fuse_attention_chain": (None, [_vp, _i]),
    "ppml_hip_backend_nodes_fused_away": (_i, [_vp]),
    "ppml_hip_backend_set_f32_arithmetic": (None, [_vp, _i]),
    "ppml_hip_backend_host_shadows_made": (_i, [_vp]),
    "ppml_hip_backend_graph_compute": (_i, [_vp, C.POINTER(_vp), _i]),
    "ppml_hip_backend_pack_weight": (_i, [_vp, _vp]),
}

_lib = None


class BackendError(RuntimeError):
    """A launcher returned a non-zero status."""

    def __init__(self, name: str, rc: int, text: str):
        super().__init__(f"{name} failed with status {rc}: {text}")
        self.rc = rc


class GgufTensor(C.Structure):
    """``ppml_gguf_tensor`` of include/ppml_hip_weights.h."""
    _fields_ = [("name", C.c_char_p), ("ndim", C.c_uint32), ("dims", C.c_uint64 * 4), ("type", C.c_uint32),
                ("data", C.c_void_p)]


_u32, _u64, _sz, _cp = C.c_uint32, C.c_uint64, C.c_size_t, C.c_char_p
_strs = C.POINTER(C.c_char_p)

# every symbol include/ppml_hip_weights.h declares (weight selection and the checkpoint file; host code only)
WEIGHTS_SIGNATURES = {
    "ppml_int8_bigop_default_list": (_cp, []),
    "ppml_int8_bigop_selected": (_i, [_cp, _cp]),
    "ppml_int8_bigop_shape_ok": (_i, [_u32, C.POINTER(_u64)]),
    "ppml_gguf_layout_hash": (_u64, [_sz, _strs, C.POINTER(_u32), C.POINTER(_u64)]),
    "ppml_gguf_save": (_i, [_cp, C.POINTER(GgufTensor), _sz, _sz, _strs, C.POINTER(_f), _sz, _strs, _strs, _sz]),
    "ppml_gguf_open": (_vp, [_cp]),
    "ppml_gguf_close": (None, [_vp]),
    "ppml_gguf_tensor_count": (_sz, [_vp]),
    "ppml_gguf_tensor_info": (_i, [_vp, _sz, C.POINTER(_cp), C.POINTER(_u32), C.POINTER(_u64), C.POINTER(_u32),
                                   C.POINTER(_u64), C.POINTER(_u64)]),
    "ppml_gguf_find_tensor": (_i64, [_vp, _cp]),
    "ppml_gguf_read_tensor": (_i, [_vp, _sz, _vp, _sz]),
    "ppml_gguf_meta_float": (_i, [_vp, _cp, C.POINTER(_f)]),
    "ppml_gguf_meta_string": (_cp, [_vp, _cp]),
    "ppml_gguf_check_layout": (_i, [_vp, _sz, _strs, C.POINTER(_u32), C.POINTER(_u64)]),
}


def load() -> C.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `make -C proteinpredictmachinelearning_amd/csrc` "
            "(or __graft_entry__.build()); this backend has no CPU fallback")
    # A process holds one HIP runtime: the first one loaded.  PyTorch ships its own and does not find the GPU through
    # another, so where PyTorch is installed it is imported first and this library binds to the runtime it brought.
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in list(SIGNATURES.items()) + list(BACKEND_SIGNATURES.items()) + list(WEIGHTS_SIGNATURES.items()):
        fn = getattr(lib, name)          # AttributeError if the library lacks a declared symbol
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def last_error() -> str:
    return load().ppml_hip_last_error().decode(errors="replace")


def check(name: str, rc: int) -> None:
    if rc != 0:
        raise BackendError(name, rc, last_error())
