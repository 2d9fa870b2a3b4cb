"""ctypes binding of the CPU oracle (``oracle/libppml_oracle.so``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py`` -- as the checker, never as the thing measured or shipped.
The GPU package never imports this module.

Array conventions follow the reference: Q8_0 blocks are 34-byte records ``{fp16 d; int8 qs[32]}``
held here as ``uint8`` arrays of shape ``[..., nblocks, 34]``.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libppml_oracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "libppml_ref_half.so")
_REF_FLASH_PATH = os.path.join(_HERE, "_ref", "libppml_ref_flash.so")

QK = 32
BLOCK_BYTES = 34


def build(force: bool = False) -> None:
    """Compile the oracle (and the reference's HalfUtils.h wrapper when the reference is mounted)."""
    args = ["make", "-C", _HERE]
    if force:
        args.append("-B")
    subprocess.run(args, check=True, stdout=subprocess.DEVNULL)


def _load() -> C.CDLL:
    if not os.path.exists(_LIB_PATH):
        build()
    lib = C.CDLL(_LIB_PATH)
    f32p, i32p, vp = C.POINTER(C.c_float), C.POINTER(C.c_int32), C.c_void_p
    i64 = C.c_int64
    lib.orc_fp32_to_fp16.restype = C.c_uint16
    lib.orc_fp32_to_fp16.argtypes = [C.c_float]
    lib.orc_fp16_to_fp32.restype = C.c_float
    lib.orc_fp16_to_fp32.argtypes = [C.c_uint16]
    lib.orc_quantize_q8_0.restype = C.c_int
    lib.orc_quantize_q8_0.argtypes = [f32p, vp, i64]
    lib.orc_q8_0_repacked_bytes.restype = C.c_size_t
    lib.orc_q8_0_repacked_bytes.argtypes = [i64]
    lib.orc_repack_q8_0.restype = None
    lib.orc_repack_q8_0.argtypes = [vp, i64, vp]
    lib.orc_unrepack_q8_0.restype = None
    lib.orc_unrepack_q8_0.argtypes = [vp, i64, vp]
    lib.orc_dequantize_q8_0.restype = None
    lib.orc_dequantize_q8_0.argtypes = [vp, f32p, i64]
    lib.orc_q8_block_sums.restype = C.c_int
    lib.orc_q8_block_sums.argtypes = [vp, vp, i32p, C.c_int, C.c_int, C.c_int]
    lib.orc_mul_mat_q8q8.restype = C.c_int
    lib.orc_mul_mat_q8q8.argtypes = [vp, vp, f32p] + [C.c_int] * 6
    lib.orc_mul_mat_q8.restype = C.c_int
    lib.orc_mul_mat_q8.argtypes = [vp, f32p, f32p] + [C.c_int] * 7
    lib.orc_quantize_q8_1.restype = C.c_int
    lib.orc_quantize_q8_1.argtypes = [f32p, vp, i64]
    lib.orc_mul_mat_q8_act.restype = C.c_int
    lib.orc_mul_mat_q8_act.argtypes = [vp, f32p, f32p] + [C.c_int] * 8
    lib.orc_mul_mat_f32.restype = None
    lib.orc_mul_mat_f32.argtypes = [f32p, f32p, f32p, C.c_int, C.c_int, C.c_int, f32p, C.c_int]
    lib.orc_mul_mat_f16.restype = None
    lib.orc_mul_mat_f16.argtypes = [C.POINTER(C.c_uint16), C.POINTER(C.c_uint16), f32p, C.c_int, C.c_int, C.c_int, f32p, C.c_int]
    lib.orc_out_prod.restype = None
    lib.orc_out_prod.argtypes = [f32p, f32p, f32p] + [i64] * 12 + [C.c_int]
    lib.orc_outer_prod_mean.restype = None
    lib.orc_outer_prod_mean.argtypes = [f32p, f32p, f32p] + [i64] * 4 + [C.c_int]
    lib.orc_outer_product_mean_value.restype = None
    lib.orc_outer_product_mean_value.argtypes = [f32p, f32p, f32p] + [i64] * 4 + [C.c_int]
    lib.orc_attention_scores.restype = None
    lib.orc_attention_scores.argtypes = [f32p, f32p, f32p] + [i64] * 5 + [C.c_int]
    lib.orc_flash_attn_forward.restype = C.c_int
    lib.orc_flash_attn_forward.argtypes = ([C.c_int] * 5 + [C.c_float, C.c_float, C.c_int] + [f32p] * 6 + [C.c_int])
    lib.orc_tri_mul.restype = None
    lib.orc_tri_mul.argtypes = [f32p, f32p, f32p] + [i64] * 5 + [C.c_float, C.c_int, C.c_int]
    lib.orc_outer_prod_mean_back.restype = None
    lib.orc_outer_prod_mean_back.argtypes = [f32p] * 5 + [i64] * 4 + [C.c_int]
    lib.orc_tri_mul_back.restype = None
    lib.orc_tri_mul_back.argtypes = [f32p] * 5 + [i64] * 5 + [C.c_float, C.c_int, C.c_int]
    lib.orc_permute.restype = C.c_int
    lib.orc_permute.argtypes = [f32p, f32p, C.c_int, C.POINTER(C.c_int32), C.POINTER(i64), C.POINTER(i64)]
    lib.orc_flash_attn_backward.restype = C.c_int
    lib.orc_flash_attn_backward.argtypes = [C.c_int] * 5 + [C.c_float] + [f32p] * 11
    lib.orc_repeat_back.restype = None
    lib.orc_repeat_back.argtypes = [f32p, f32p, C.c_int, C.POINTER(i64), C.c_int, C.POINTER(i64)]
    lib.orc_scale.restype = None
    lib.orc_scale.argtypes = [f32p, f32p, i64, C.c_float, C.c_int]
    lib.orc_relu.restype = None
    lib.orc_relu.argtypes = [f32p, f32p, i64, C.c_int]
    lib.orc_bcast_elemwise.restype = C.c_int
    lib.orc_bcast_elemwise.argtypes = [f32p, f32p, f32p, i64, i64, i64, C.c_int, C.c_int]
    lib.orc_softmax.restype = None
    lib.orc_softmax.argtypes = [f32p, f32p, i64, i64, C.c_int]
    lib.orc_max_threads.restype = C.c_int
    return lib


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        _lib = _load()
    return _lib


def ref_half_lib():
    """The reference's own HalfUtils.h compiled as-is, or None when it was never built."""
    if not os.path.exists(_REF_PATH):
        return None
    ref = C.CDLL(_REF_PATH)
    ref.ref_fp32_to_fp16.restype = C.c_uint16
    ref.ref_fp32_to_fp16.argtypes = [C.c_float]
    ref.ref_fp16_to_fp32.restype = C.c_float
    ref.ref_fp16_to_fp32.argtypes = [C.c_uint16]
    ref.ref_sweep_fp32_to_fp16.restype = C.c_int64
    ref.ref_sweep_fp32_to_fp16.argtypes = [C.c_void_p, C.c_uint32, C.c_uint32, C.POINTER(C.c_uint32)]
    return ref


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def _fp(a: np.ndarray):
    return a.ctypes.data_as(C.POINTER(C.c_float))


def _vp(a: np.ndarray):
    return a.ctypes.data_as(C.c_void_p)


def max_threads() -> int:
    return int(lib().orc_max_threads())


def fp32_to_fp16(x: float) -> int:
    return int(lib().orc_fp32_to_fp16(C.c_float(x)))


def fp16_to_fp32(h: int) -> float:
    return float(lib().orc_fp16_to_fp32(C.c_uint16(h)))


def quantize_q8_0(x) -> np.ndarray:
    """f32 [..., K] -> uint8 [..., K/32, 34] (QuantBlocks.h:62-79)."""
    x = _f32(x)
    n = x.size
    if n % QK:
        raise ValueError("element count is not a multiple of 32")
    out = np.empty((n // QK, BLOCK_BYTES), dtype=np.uint8)
    rc = lib().orc_quantize_q8_0(_fp(x), _vp(out), n)
    assert rc == 0
    return out.reshape(x.shape[:-1] + (x.shape[-1] // QK, BLOCK_BYTES))


def block_scales_bits(blocks: np.ndarray) -> np.ndarray:
    return np.ascontiguousarray(blocks[..., :2]).view(np.uint16)[..., 0]


def block_quants(blocks: np.ndarray) -> np.ndarray:
    return np.ascontiguousarray(blocks[..., 2:]).view(np.int8)


def repack_q8_0(blocks: np.ndarray) -> np.ndarray:
    blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
    nb = blocks.size // BLOCK_BYTES
    out = np.empty(nb * BLOCK_BYTES, dtype=np.uint8)
    lib().orc_repack_q8_0(_vp(blocks), nb, _vp(out))
    return out


def unrepack_q8_0(packed: np.ndarray) -> np.ndarray:
    packed = np.ascontiguousarray(packed, dtype=np.uint8)
    nb = packed.size // BLOCK_BYTES
    out = np.empty((nb, BLOCK_BYTES), dtype=np.uint8)
    lib().orc_unrepack_q8_0(_vp(packed), nb, _vp(out))
    return out


def dequantize_q8_0(blocks: np.ndarray) -> np.ndarray:
    blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
    nb = blocks.size // BLOCK_BYTES
    out = np.empty(nb * QK, dtype=np.float32)
    lib().orc_dequantize_q8_0(_vp(blocks), _fp(out), nb * QK)
    return out.reshape(blocks.shape[:-2] + (blocks.shape[-2] * QK,))


def q8_block_sums(wq: np.ndarray, xq: np.ndarray) -> np.ndarray:
    """wq [M, nblk, 34], xq [N, nblk, 34] -> int32 [N, M, nblk]."""
    wq = np.ascontiguousarray(wq, dtype=np.uint8)
    xq = np.ascontiguousarray(xq, dtype=np.uint8)
    M, nblk = wq.shape[0], wq.shape[1]
    N = xq.shape[0]
    out = np.empty((N, M, nblk), dtype=np.int32)
    rc = lib().orc_q8_block_sums(_vp(wq), _vp(xq), out.ctypes.data_as(C.POINTER(C.c_int32)),
                                 M, N, nblk * QK)
    assert rc == 0, rc
    return out


def mul_mat_q8q8(wq, xq, c_trans=1, fma=1, nthreads=0) -> np.ndarray:
    wq = np.ascontiguousarray(wq, dtype=np.uint8)
    xq = np.ascontiguousarray(xq, dtype=np.uint8)
    M, nblk = wq.shape[0], wq.shape[1]
    N = xq.shape[0]
    out = np.empty((N, M) if c_trans else (M, N), dtype=np.float32)
    rc = lib().orc_mul_mat_q8q8(_vp(wq), _vp(xq), _fp(out), M, N, nblk * QK, c_trans, fma, nthreads)
    assert rc == 0, rc
    return out


def mul_mat_q8(w, x, wtype=0, c_trans=1, fma=1, nthreads=0) -> np.ndarray:
    """w: Q8_0 weight bytes (wtype 0: [M, K/32, 34]; wtype 2: flat Q8_0R), x f32 [N, K]."""
    x = _f32(x)
    N, K = x.shape
    w = np.ascontiguousarray(w, dtype=np.uint8)
    M = w.size // (K // QK * BLOCK_BYTES)
    out = np.empty((N, M) if c_trans else (M, N), dtype=np.float32)
    rc = lib().orc_mul_mat_q8(_vp(w), _fp(x), _fp(out), M, N, K, wtype, c_trans, fma, nthreads)
    if rc:
        raise RuntimeError(f"orc_mul_mat_q8 rc={rc}")
    return out


def quantize_q8_1(x) -> np.ndarray:
    """f32 [..., K] -> uint8 [..., K/32, 36] block_q8_1 records (QuantBlocks.h:81-111)."""
    x = _f32(x)
    n = x.size
    if n % QK:
        raise ValueError("element count is not a multiple of 32")
    out = np.empty((n // QK, 36), dtype=np.uint8)
    rc = lib().orc_quantize_q8_1(_fp(x), _vp(out), n)
    assert rc == 0
    return out.reshape(x.shape[:-1] + (x.shape[-1] // QK, 36))


def mul_mat_q8_act(w, x, act=1, wtype=0, c_trans=1, fma=1, nthreads=0) -> np.ndarray:
    """mul_mat_q8 with the activation rule selectable (0 = Q8_0, 1 = Q8_1)."""
    x = _f32(x)
    N, K = x.shape
    w = np.ascontiguousarray(w, dtype=np.uint8)
    M = w.size // (K // QK * BLOCK_BYTES)
    out = np.empty((N, M) if c_trans else (M, N), dtype=np.float32)
    rc = lib().orc_mul_mat_q8_act(_vp(w), _fp(x), _fp(out), M, N, K, wtype, c_trans, fma, act, nthreads)
    if rc:
        raise RuntimeError(f"orc_mul_mat_q8_act rc={rc}")
    return out


def mul_mat_f32(a, b, bias=None, nthreads=0) -> np.ndarray:
    """a [M,K], b [N,K] -> [M,N] (CPUKernels.cpp:763-771)."""
    a, b = _f32(a), _f32(b)
    M, K = a.shape
    N = b.shape[0]
    out = np.empty((M, N), dtype=np.float32)
    bp = None
    if bias is not None:
        bias = _f32(bias)
        bp = _fp(bias)
    lib().orc_mul_mat_f32(_fp(a), _fp(b), _fp(out), M, K, N, bp, nthreads)
    return out


def mul_mat_f16(a16, b16, bias=None, nthreads=0) -> np.ndarray:
    """a16 [M,K], b16 [N,K] float16 -> f32 [M,N] (CPUKernels.cpp:646-672: binary32 sum, bias last)."""
    a16 = np.ascontiguousarray(a16, dtype=np.float16)
    b16 = np.ascontiguousarray(b16, dtype=np.float16)
    M, K = a16.shape
    N = b16.shape[0]
    assert b16.shape[1] == K
    out = np.empty((M, N), dtype=np.float32)
    bp = None if bias is None else _fp(_f32(bias))
    u16p = C.POINTER(C.c_uint16)
    lib().orc_mul_mat_f16(a16.view(np.uint16).ctypes.data_as(u16p), b16.view(np.uint16).ctypes.data_as(u16p),
                          _fp(out), M, K, N, bp, nthreads)
    return out


def out_prod(s0, s1, nthreads=0) -> np.ndarray:
    """Arrays are numpy-shaped outermost first: s0 [ne03,ne02,ne01,ne00], s1 [ne13,ne12,ne11,ne10]
    -> dst [ne3,ne2,ne1(=ne10),ne0(=ne00)] (CPUKernels.cpp:787-887)."""
    s0, s1 = _f32(s0), _f32(s1)
    ne03, ne02, ne01, ne00 = s0.shape
    ne13, ne12, ne11, ne10 = s1.shape
    ne0, ne1, ne2, ne3 = ne00, ne10, max(ne02, ne12), max(ne03, ne13)
    out = np.empty((ne3, ne2, ne1, ne0), dtype=np.float32)
    lib().orc_out_prod(_fp(s0), _fp(s1), _fp(out), ne00, ne01, ne02, ne03, ne10, ne11, ne12, ne13,
                       ne0, ne1, ne2, ne3, nthreads)
    return out


def outer_prod_mean(left, right, D, L, N, B, nthreads=0) -> np.ndarray:
    """Graph form; flat buffers indexed exactly as CPUKernels.cpp:1006-1028."""
    left, right = _f32(left).ravel(), _f32(right).ravel()
    out = np.empty(D * D * L * L * B, dtype=np.float32)
    lib().orc_outer_prod_mean(_fp(left), _fp(right), _fp(out), D, L, N, B, nthreads)
    return out


def outer_product_mean_value(left, right, nthreads=0) -> np.ndarray:
    """Value form: left/right (B,N,L,D) -> (B,L,L,D*D) (MathUtils.cpp:387-437)."""
    left, right = _f32(left), _f32(right)
    B, N, L, D = left.shape
    out = np.empty((B, L, L, D * D), dtype=np.float32)
    lib().orc_outer_product_mean_value(_fp(left), _fp(right), _fp(out), B, N, L, D, nthreads)
    return out


def attention_scores(q, k, nthreads=0) -> np.ndarray:
    """Q (NQ,H,D,Lq), K (NQ,H,D,Lk) -> (NQ,H,Lq,Lk) incl. 1/sqrt(D) (Attention.cpp:58-79)."""
    q, k = _f32(q), _f32(k)
    NQ, H, D, Lq = q.shape
    Lk = k.shape[3]
    out = np.empty((NQ, H, Lq, Lk), dtype=np.float32)
    lib().orc_attention_scores(_fp(q), _fp(k), _fp(out), NQ, H, D, Lq, Lk, nthreads)
    return out


def _opt_fp(a):
    return _fp(a) if a is not None else C.POINTER(C.c_float)()


def flash_attn_forward(q, k, v, bias=None, causal=False, scale=0.0, eps=1e-9, Bc=64, nthreads=0):
    """Q, K, V (B,h,L,d), bias (B,h,L,L) or None -> O (B,h,L,d), LSE (B,h,L)  (FlashAttn.cpp:55-135)."""
    q, k, v = _f32(q), _f32(k), _f32(v)
    B, h, L, d = q.shape
    bias = _f32(bias) if bias is not None else None
    o = np.empty_like(q)
    lse = np.empty((B, h, L), dtype=np.float32)
    rc = lib().orc_flash_attn_forward(B, h, L, d, int(causal), scale, eps, Bc, _fp(q), _fp(k), _fp(v), _opt_fp(bias),
                                      _fp(o), _fp(lse), nthreads or max_threads())
    if rc:
        raise ValueError(f"orc_flash_attn_forward rc={rc}")
    return o, lse


def ref_flash_lib():
    """The reference's own src/ops/FlashAttn.cpp compiled as-is, or None when it was never built."""
    if not os.path.exists(_REF_FLASH_PATH):
        return None
    ref = C.CDLL(_REF_FLASH_PATH)
    f32p = C.POINTER(C.c_float)
    ref.ref_flash_attn_forward.restype = C.c_int
    ref.ref_flash_attn_forward.argtypes = [C.c_int] * 5 + [C.c_float, C.c_float, C.c_int] + [f32p] * 6
    ref.ref_flash_attn_forward_plain.restype = C.c_int
    ref.ref_flash_attn_forward_plain.argtypes = [C.c_int] * 5 + [C.c_float] + [f32p] * 6
    ref.ref_flash_attn_backward.restype = C.c_int
    ref.ref_flash_attn_backward.argtypes = [C.c_int] * 5 + [C.c_float] + [f32p] * 11
    return ref


def ref_flash_attn_forward(q, k, v, bias=None, causal=False, scale=0.0, eps=1e-9, Bc=64, plain=False):
    """Same arguments through the compiled reference; `plain` = its three-pass routine (no eps)."""
    ref = ref_flash_lib()
    if ref is None:
        return None
    q, k, v = _f32(q), _f32(k), _f32(v)
    B, h, L, d = q.shape
    bias = _f32(bias) if bias is not None else None
    o = np.empty_like(q)
    lse = np.empty((B, h, L), dtype=np.float32)
    if plain:
        rc = ref.ref_flash_attn_forward_plain(B, h, L, d, int(causal), scale, _fp(q), _fp(k), _fp(v), _opt_fp(bias), _fp(o), _fp(lse))
    else:
        rc = ref.ref_flash_attn_forward(B, h, L, d, int(causal), scale, eps, Bc, _fp(q), _fp(k), _fp(v), _opt_fp(bias), _fp(o), _fp(lse))
    if rc:
        raise ValueError(f"reference refused the arguments (rc={rc})")
    return o, lse


def permute(x, axes) -> np.ndarray:
    """kernel_permute (CPUKernels.cpp:1669-1717).  `x` is a numpy array whose LAST axis is the reference's
    dims[0]; `axes` is in the reference's numbering (dimension p of the result is dimension axes[p] of x)."""
    x = _f32(x)
    nd = x.ndim
    sd = list(x.shape[::-1]) + [1] * (4 - nd)
    ax = [int(a) for a in axes] + list(range(nd, 4))
    dd = [sd[ax[p]] if 0 <= ax[p] < 4 else 1 for p in range(nd)] + [1] * (4 - nd)
    out = np.empty(tuple(dd[:nd][::-1]), dtype=np.float32)
    rc = lib().orc_permute(_fp(x), _fp(out), nd, (C.c_int32 * 4)(*ax), (C.c_int64 * 4)(*sd), (C.c_int64 * 4)(*dd))
    if rc:
        raise ValueError(f"orc_permute rc={rc}")
    return out


def tri_mul(left, right, D, I, J, K, B, L, outgoing=True, nthreads=0) -> np.ndarray:
    """kernel_tri_mul (CPUKernels.cpp:907-968) on flat operands; returns the flat [D*I*J*B] result."""
    left, right = _f32(left).reshape(-1), _f32(right).reshape(-1)
    assert left.size == D * I * K * B and right.size == D * J * K * B
    out = np.empty(D * I * J * B, dtype=np.float32)
    lib().orc_tri_mul(_fp(left), _fp(right), _fp(out), D, I, J, K, B, L, int(outgoing), nthreads or max_threads())
    return out


def tri_mul_back(grad, left, right, D, I, J, K, B, L, outgoing=True, nthreads=0):
    """kernel_tri_mul_back (CPUKernels.cpp:1238-1367): returns (gleft, gright), flat, shaped like left and right."""
    grad, left, right = _f32(grad).reshape(-1), _f32(left).reshape(-1), _f32(right).reshape(-1)
    assert grad.size == D * I * J * B and left.size == D * I * K * B and right.size == D * J * K * B
    gl = np.empty(D * I * K * B, dtype=np.float32)
    gr = np.empty(D * J * K * B, dtype=np.float32)
    lib().orc_tri_mul_back(_fp(grad), _fp(left), _fp(right), _fp(gl), _fp(gr), D, I, J, K, B, L, int(outgoing),
                           nthreads or max_threads())
    return gl, gr


def outer_prod_mean_back(grad, left, right, D, L, N, B, nthreads=0):
    """kernel_outer_prod_mean_back (CPUKernels.cpp:1034-1105): returns (gleft, gright), flat [D*L*N*B] each."""
    grad, left, right = _f32(grad).reshape(-1), _f32(left).reshape(-1), _f32(right).reshape(-1)
    assert grad.size == D * D * L * L * B and left.size == D * L * N * B and right.size == D * L * N * B
    gl = np.empty(D * L * N * B, dtype=np.float32)
    gr = np.empty(D * L * N * B, dtype=np.float32)
    lib().orc_outer_prod_mean_back(_fp(grad), _fp(left), _fp(right), _fp(gl), _fp(gr), D, L, N, B, nthreads or max_threads())
    return gl, gr


def _flash_backward(fn, q, k, v, bias, o, do, lse, causal, scale, want_dbias):
    q, k, v, o, do, lse = _f32(q), _f32(k), _f32(v), _f32(o), _f32(do), _f32(lse)
    B, h, L, d = q.shape
    bias = _f32(bias) if bias is not None else None
    dq, dk, dv = np.empty_like(q), np.empty_like(q), np.empty_like(q)
    db = np.empty((B, h, L, L), dtype=np.float32) if want_dbias else None
    rc = fn(B, h, L, d, int(causal), scale, _fp(q), _fp(k), _fp(v), _opt_fp(bias), _fp(o), _fp(do), _fp(lse),
            _fp(dq), _fp(dk), _fp(dv), _opt_fp(db))
    if rc:
        raise ValueError(f"flash attention backward refused the arguments (rc={rc})")
    return dq, dk, dv, db


def flash_attn_backward(q, k, v, bias, o, do, lse, causal=False, scale=0.0, want_dbias=True):
    """FlashAttn.cpp:140-210: (dQ, dK, dV, dbias) from dO and the forward's O and LSE."""
    return _flash_backward(lib().orc_flash_attn_backward, q, k, v, bias, o, do, lse, causal, scale, want_dbias)


def ref_flash_attn_backward(q, k, v, bias, o, do, lse, causal=False, scale=0.0, want_dbias=True):
    """The same through the compiled reference, or None when it was never built."""
    ref = ref_flash_lib()
    if ref is None:
        return None
    return _flash_backward(ref.ref_flash_attn_backward, q, k, v, bias, o, do, lse, causal, scale, want_dbias)


def repeat_back(src, dst_shape) -> np.ndarray:
    """kernel_repeat_back (CPUKernels.cpp:2091-2148).  `src` is a numpy array whose LAST axis is the reference's
    dims[0]; `dst_shape` is the result's shape in the same (numpy) order."""
    src = _f32(src)
    dst_shape = tuple(int(d) for d in dst_shape)
    sd = list(src.shape[::-1]) + [1] * (4 - src.ndim)
    dd = list(dst_shape[::-1]) + [1] * (4 - len(dst_shape))
    out = np.empty(dst_shape, dtype=np.float32)
    lib().orc_repeat_back(_fp(src), _fp(out), src.ndim, (C.c_int64 * 4)(*sd), len(dst_shape), (C.c_int64 * 4)(*dd))
    return out


def scale(x, s, nthreads=0) -> np.ndarray:
    """kernel_scale (CPUKernels.cpp:1737-1754): x * s element by element."""
    x = _f32(x)
    out = np.empty_like(x)
    lib().orc_scale(_fp(x), _fp(out), x.size, float(np.float32(s)), nthreads)
    return out


def relu(x, nthreads=0) -> np.ndarray:
    """compute_forward_relu (CPUKernels.cpp:2649-2657): (x > 0) ? x : 0."""
    x = _f32(x)
    out = np.empty_like(x)
    lib().orc_relu(_fp(x), _fp(out), x.size, nthreads)
    return out


ELEMWISE_OPS = {"add": 0, "sub": 1, "mul": 2, "div": 3}


def bcast_elemwise(a, b, op="add", nthreads=0) -> np.ndarray:
    """kernel_elemwise (CPUKernels.cpp:446-596).  The result has the shape of the larger operand (the reference's
    dst is a copy of src[0]'s shape); the other one repeats along the flat order, i % numel."""
    a, b = _f32(a), _f32(b)
    big = a if a.size >= b.size else b
    out = np.empty_like(big)
    rc = lib().orc_bcast_elemwise(_fp(a), _fp(b), _fp(out), big.size, a.size, b.size, ELEMWISE_OPS[op], nthreads)
    if rc:
        raise ValueError("orc_bcast_elemwise: bad arguments")
    return out


def softmax(x, nthreads=0) -> np.ndarray:
    """kernel_softmax (CPUKernels.cpp:1446-1467) over the LAST numpy axis (the reference's dims[0])."""
    x = _f32(x)
    out = np.empty_like(x)
    D = x.shape[-1]
    lib().orc_softmax(_fp(x), _fp(out), x.size // D, D, nthreads)
    return out
