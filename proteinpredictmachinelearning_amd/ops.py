"""Host-side operators of the gfx950 mul_mat backend on top of the C ABI.

Function names, argument order, shape contracts and error behaviour follow the reference's graph-op
builders (src/core/ComputeGraphHelper.cpp:262-345, 1748-1764) and its dispatch wrapper
(src/backend/CUDAKernels.cpp:717-847).  torch is used for device memory and streams only; all
arithmetic happens in the HIP library.  Shapes are written numpy style (outermost first), i.e. the
reverse of the reference's ``dims[0]``-innermost notation.
"""
from __future__ import annotations

import ctypes as C
import math

import torch

from . import cabi

QK = 32
BLOCK_BYTES = 34
WTYPE_Q8_0, WTYPE_Q8_1, WTYPE_Q8_0R, WTYPE_Q8_0M = 0, 1, 2, 3

_initialised = set()


def _lib():
    lib = cabi.load()
    if not torch.cuda.is_available():
        raise RuntimeError("the gfx950 backend needs a GPU; there is no CPU path")
    dev = torch.cuda.current_device()
    if dev not in _initialised:
        cabi.check("ppml_hip_init", lib.ppml_hip_init(dev))
        _initialised.add(dev)
    return lib


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _dev_f32(t: torch.Tensor, name: str) -> torch.Tensor:
    if not t.is_cuda or t.dtype != torch.float32:
        raise TypeError(f"{name} must be a float32 device tensor")
    return t.contiguous()


def _ptr(t) -> C.c_void_p:
    return C.c_void_p(0 if t is None else t.data_ptr())


Q8_PATH_NAMES = {0: "general", 1: "weight-stationary", 2: "low-latency", 3: "tiled"}


def last_q8_path() -> str:
    """Kernel family that served this thread's last mul_mat_q8 call (``ppml_hip_q8_last_path``)."""
    return Q8_PATH_NAMES[_lib().ppml_hip_q8_last_path()]


def mulmat_stats_enable(on: bool) -> bool:
    """Switches the MUL_MAT statistics (include/ppml/MulMatStats.h) on or off; returns the previous state."""
    return bool(cabi.load().ppml_hip_mulmat_stats_enable(1 if on else 0))


def mulmat_stats_rows():
    """The statistics table as a list of dicts {path, M, K, N, calls, ms}, ordered by (path, M, K, N)."""
    lib = cabi.load()
    n = lib.ppml_hip_mulmat_stats_rows(None, 0)
    rows = (cabi.MulMatStat * max(n, 1))()
    n = min(lib.ppml_hip_mulmat_stats_rows(C.cast(rows, C.c_void_p), n), n)
    return [{"path": rows[i].path.decode(), "M": rows[i].M, "K": rows[i].K, "N": rows[i].N, "calls": rows[i].calls,
             "ms": rows[i].ms} for i in range(n)]


def synchronize() -> None:
    cabi.check("ppml_hip_synchronize", _lib().ppml_hip_synchronize())


# ----------------------------------------------------------------------------- f32
def set_f32_arithmetic(mode: str) -> str:
    """Matrix pipe of the f32 contractions: "split" (default: bf16 pipe, exact three-way split) or "fp32"
    (fp32 MFMA).  Returns the previous setting."""
    before = _lib().ppml_hip_set_f32_arithmetic({"split": 0, "fp32": 1}[mode])
    return "fp32" if before == 1 else "split"


def mul_mat(a: torch.Tensor, b: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
    """a [M,K], b [N,K] -> [M,N] = a @ b.T (+ bias[N]); src/core/ComputeGraphHelper.cpp:262-314."""
    a, b = _dev_f32(a, "a"), _dev_f32(b, "b")
    if a.dim() != 2 or b.dim() != 2 or a.shape[1] != b.shape[1]:
        raise ValueError(f"mul_mat: inner dimensions differ, a {tuple(a.shape)} b {tuple(b.shape)}")
    M, K = a.shape
    N = b.shape[0]
    if bias is not None:
        bias = _dev_f32(bias, "bias")
        if bias.numel() != N:          # the reference drops a bias of the wrong length with a message
            raise ValueError(f"mul_mat: bias has {bias.numel()} elements, expected {N}")
    out = torch.empty((M, N), dtype=torch.float32, device=a.device)
    lib = _lib()
    cabi.check("mul_mat_hip", lib.mul_mat_hip(_ptr(a), _ptr(b), _ptr(out), M, K, N, _ptr(bias), _stream()))
    return out


def mul_mat_f16(a: torch.Tensor, b: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
    """F16 x F16 -> F32 mul_mat: a [M,K], b [N,K] float16 on the device, binary32 products and sum,
    bias (f32 [N]) added to the finished sum (src/backend/CPUKernels.cpp:646-672)."""
    for t, name in ((a, "a"), (b, "b")):
        if not t.is_cuda or t.dtype != torch.float16:
            raise TypeError(f"mul_mat_f16: {name} must be a float16 tensor on the device")
    a, b = a.contiguous(), b.contiguous()
    if a.dim() != 2 or b.dim() != 2 or a.shape[1] != b.shape[1]:
        raise ValueError(f"mul_mat_f16: a {tuple(a.shape)} and b {tuple(b.shape)} do not share K")
    M, K = a.shape
    N = b.shape[0]
    if bias is not None:
        bias = _dev_f32(bias, "bias")
        if bias.numel() != N:
            raise ValueError("mul_mat_f16: bias length is not N")
    out = torch.empty((M, N), dtype=torch.float32, device=a.device)
    cabi.check("mul_mat_f16_hip", _lib().mul_mat_f16_hip(_ptr(a), _ptr(b), _ptr(out), M, K, N, _ptr(bias), _stream()))
    return out


def mul_mat_tn(a: torch.Tensor, b: torch.Tensor, alpha: float = 1.0) -> torch.Tensor:
    """a [K,M], b [K,N] -> alpha * a.T @ b (the dense form of outer-product-mean)."""
    a, b = _dev_f32(a, "a"), _dev_f32(b, "b")
    if a.dim() != 2 or b.dim() != 2 or a.shape[0] != b.shape[0]:
        raise ValueError("mul_mat_tn: contraction lengths differ")
    K, M = a.shape
    N = b.shape[1]
    out = torch.empty((M, N), dtype=torch.float32, device=a.device)
    cabi.check("mul_mat_tn_hip", _lib().mul_mat_tn_hip(_ptr(a), _ptr(b), _ptr(out), M, K, N, alpha, _stream()))
    return out


def out_prod(a: torch.Tensor, b: torch.Tensor, scale: float | None = None, out: torch.Tensor | None = None) -> torch.Tensor:
    """a [ne03,ne02,K,ne00], b [ne13,ne12,K,ne10] -> [ne13,ne12,ne10,ne00];
    src/core/ComputeGraphHelper.cpp:318-345, broadcast of src/backend/CPUKernels.cpp:836-858.
    ``scale`` fuses the OP_SCALE node that follows in the attention path.  ``out``: a contiguous float32
    device tensor of the result's size to write into (any 4-byte alignment) instead of a new one."""
    a, b = _dev_f32(a, "a"), _dev_f32(b, "b")
    while a.dim() < 4:
        a = a.unsqueeze(0)
    while b.dim() < 4:
        b = b.unsqueeze(0)
    ne03, ne02, ne01, ne00 = a.shape
    ne13, ne12, ne11, ne10 = b.shape
    if ne01 != ne11:
        raise ValueError(f"out_prod: contraction dims differ ({ne01} vs {ne11})")
    ne0, ne1, ne2, ne3 = ne00, ne10, max(ne02, ne12), max(ne03, ne13)
    if out is None:
        out = torch.empty((ne3, ne2, ne1, ne0), dtype=torch.float32, device=a.device)
    elif out.dtype != torch.float32 or out.device != a.device or not out.is_contiguous() or out.numel() != ne0 * ne1 * ne2 * ne3:
        raise ValueError("out_prod: `out` must be a contiguous float32 tensor of the result's size on the operands' device")
    else:
        out = out.view(ne3, ne2, ne1, ne0)
    dims = [ne00, ne01, ne02, ne03, ne10, ne11, ne12, ne13, ne0, ne1, ne2, ne3]
    lib = _lib()
    if scale is None:
        rc = lib.out_prod_hip(_ptr(a), _ptr(b), _ptr(out), *dims, _stream())
    else:
        rc = lib.out_prod_scaled_hip(_ptr(a), _ptr(b), _ptr(out), *dims, scale, _stream())
    cabi.check("out_prod_hip", rc)
    return out


def attention_logits(k: torch.Tensor, q: torch.Tensor, head_dim: int | None = None, out: torch.Tensor | None = None) -> torch.Tensor:
    """out_prod(K, Q) * 1/sqrt(head_dim), steps 1-2 of src/modules/Attention.cpp:264-270."""
    d = k.shape[-2] if head_dim is None else head_dim
    return out_prod(k, q, scale=1.0 / math.sqrt(float(d)), out=out)


def outer_product_mean(left: torch.Tensor, right: torch.Tensor, D: int, L: int, N: int, B: int) -> torch.Tensor:
    """Graph form (src/core/ComputeGraphHelper.cpp:1748-1764): flat buffers indexed as
    src/backend/CPUKernels.cpp:1006-1028; returns the flat [D*D*L*L*B] result."""
    left, right = _dev_f32(left, "left").reshape(-1), _dev_f32(right, "right").reshape(-1)
    if left.numel() != D * L * N * B or right.numel() != D * L * N * B:
        raise ValueError("outer_product_mean: operand size does not match D*L*N*B")
    out = torch.empty(D * D * L * L * B, dtype=torch.float32, device=left.device)
    cabi.check("outer_prod_mean_hip",
               _lib().outer_prod_mean_hip(_ptr(left), _ptr(right), _ptr(out), D, L, N, B, 1.0 / float(N), _stream()))
    return out


def outer_prod_mean_back(grad: torch.Tensor, left: torch.Tensor, right: torch.Tensor, D: int, L: int, N: int, B: int,
                         want_left: bool = True, want_right: bool = True):
    """Gradients of outer_prod_mean's operands (src/backend/CPUKernels.cpp:1034-1105); flat tensors."""
    grad, left, right = _dev_f32(grad, "grad"), _dev_f32(left, "left"), _dev_f32(right, "right")
    if grad.numel() != D * D * L * L * B or left.numel() != D * L * N * B or right.numel() != D * L * N * B:
        raise ValueError("outer_prod_mean_back: operand size does not match D, L, N, B")
    if not (want_left or want_right):
        raise ValueError("outer_prod_mean_back: at least one gradient must be wanted")
    gl = torch.empty(D * L * N * B, dtype=torch.float32, device=grad.device) if want_left else None
    gr = torch.empty(D * L * N * B, dtype=torch.float32, device=grad.device) if want_right else None
    cabi.check("outer_prod_mean_back_hip",
               _lib().outer_prod_mean_back_hip(_ptr(grad), _ptr(left), _ptr(right), _ptr(gl) if gl is not None else None,
                                               _ptr(gr) if gr is not None else None, D, L, N, B, 1.0 / float(N), _stream()))
    return gl, gr


def outer_product_mean_value(left: torch.Tensor, right: torch.Tensor) -> torch.Tensor:
    """Value form (src/ops/MathUtils.cpp:387-437): (B,N,L,D) x (B,N,L,D) -> (B,L,L,D*D)."""
    left, right = _dev_f32(left, "left"), _dev_f32(right, "right")
    if left.dim() != 4 or right.dim() != 4:
        raise ValueError("outer_product_mean expects 4D tensors")
    if left.shape[0] != right.shape[0] or left.shape[2] != right.shape[2] or left.shape[3] != right.shape[3] \
            or left.shape[1] != right.shape[1]:
        raise ValueError("outer_product_mean dimension mismatch: batch/residue/feature dims differ")
    B, N, L, D = left.shape
    out = torch.empty((B, L, L, D * D), dtype=torch.float32, device=left.device)
    cabi.check("outer_product_mean_value_hip",
               _lib().outer_product_mean_value_hip(_ptr(left), _ptr(right), _ptr(out), B, N, L, D, _stream()))
    return out


def tri_mul(left: torch.Tensor, right: torch.Tensor, D: int, I: int, J: int, K: int, B: int, L: float,
            outgoing: bool = True) -> torch.Tensor:
    """Triangle multiplication, graph form (src/backend/CPUKernels.cpp:907-968): flat operands indexed as the
    kernel does (d outermost, b innermost); returns the flat [D*I*J*B] result incl. the 1/L and the finite guard."""
    left, right = _dev_f32(left, "left"), _dev_f32(right, "right")
    if L == 0:
        raise ValueError("tri_mul: L must not be zero")
    if left.numel() != D * I * K * B or right.numel() != D * J * K * B:
        raise ValueError("tri_mul: operand size does not match D, I, J, K, B")
    out = torch.empty(D * I * J * B, dtype=torch.float32, device=left.device)
    cabi.check("tri_mul_hip", _lib().tri_mul_hip(_ptr(left), _ptr(right), _ptr(out), D, I, J, K, B, 1.0 / float(L),
                                                 int(outgoing), _stream()))
    return out


def tri_mul_back(grad: torch.Tensor, left: torch.Tensor, right: torch.Tensor, D: int, I: int, J: int, K: int, B: int,
                 L: float, outgoing: bool = True, want_left: bool = True, want_right: bool = True):
    """Gradients of tri_mul's operands (src/backend/CPUKernels.cpp:1238-1367); flat tensors, same indexing."""
    grad, left, right = _dev_f32(grad, "grad"), _dev_f32(left, "left"), _dev_f32(right, "right")
    if L == 0 or not (want_left or want_right):
        raise ValueError("tri_mul_back: L must not be zero and at least one gradient must be wanted")
    if grad.numel() != D * I * J * B or left.numel() != D * I * K * B or right.numel() != D * J * K * B:
        raise ValueError("tri_mul_back: operand size does not match D, I, J, K, B")
    gl = torch.empty(D * I * K * B, dtype=torch.float32, device=grad.device) if want_left else None
    gr = torch.empty(D * J * K * B, dtype=torch.float32, device=grad.device) if want_right else None
    cabi.check("tri_mul_back_hip",
               _lib().tri_mul_back_hip(_ptr(grad), _ptr(left), _ptr(right), _ptr(gl) if gl is not None else None,
                                       _ptr(gr) if gr is not None else None, D, I, J, K, B, 1.0 / float(L), int(outgoing), _stream()))
    return gl, gr


def flash_attn_forward(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, bias: torch.Tensor | None = None,
                       causal: bool = False, scale: float = 0.0, eps: float = 1e-9, Bc: int = 64,
                       want_lse: bool = True, in_ld: bool = False, out_ld: bool = False):
    """Fused attention forward (include/ppml/FlashAttn.h:8-65): Q, K, V (B,h,L,d), bias (B,h,L,L) or None
    -> O (B,h,L,d) and LSE (B,h,L) (None when not wanted).  in_ld: Q, K, V are (B,h,d,L) instead (the graph
    tensors before their layout bridge); out_ld: O is returned as (B,h,d,L)."""
    q, k, v = _dev_f32(q, "q"), _dev_f32(k, "k"), _dev_f32(v, "v")
    if q.dim() != 4 or q.shape != k.shape or q.shape != v.shape:
        raise ValueError("flash_attn_forward: Q, K and V must be 4-D tensors of one shape (B,h,L,d)")
    B, h, L, d = q.shape
    if in_ld:
        L, d = d, L
    if bias is not None:
        bias = _dev_f32(bias, "bias")
        if tuple(bias.shape) != (B, h, L, L):
            raise ValueError("flash_attn_forward: bias must be (B,h,L,L)")
    o = torch.empty((B, h, d, L) if out_ld else (B, h, L, d), dtype=torch.float32, device=q.device)
    lse = torch.empty((B, h, L), dtype=torch.float32, device=q.device) if want_lse else None
    cabi.check("flash_attn_forward_ex_hip",
               _lib().flash_attn_forward_ex_hip(B, h, L, d, int(causal), scale, eps, Bc, _ptr(q), _ptr(k), _ptr(v),
                                                _ptr(bias) if bias is not None else None, _ptr(o),
                                                _ptr(lse) if lse is not None else None,
                                                int(in_ld) | (int(out_ld) << 1), _stream()))
    return o, lse


def flash_attn_backward(q, k, v, bias, o, do, lse, causal: bool = False, scale: float = 0.0,
                        want=("dq", "dk", "dv", "dbias")):
    """Fused attention backward (include/ppml/FlashAttn.h:67-101): returns (dQ, dK, dV, dbias), None for the
    gradients not named in `want`."""
    q, k, v, o, do, lse = (_dev_f32(t, n) for t, n in ((q, "q"), (k, "k"), (v, "v"), (o, "o"), (do, "do"), (lse, "lse")))
    B, h, L, d = q.shape
    if bias is not None:
        bias = _dev_f32(bias, "bias")
    dq = torch.empty_like(q) if "dq" in want else None
    dk = torch.empty_like(q) if "dk" in want else None
    dv = torch.empty_like(q) if "dv" in want else None
    db = torch.empty((B, h, L, L), dtype=torch.float32, device=q.device) if "dbias" in want else None
    opt = lambda t: _ptr(t) if t is not None else None      # noqa: E731
    cabi.check("flash_attn_backward_hip",
               _lib().flash_attn_backward_hip(B, h, L, d, int(causal), scale, _ptr(q), _ptr(k), _ptr(v), opt(bias), _ptr(o),
                                              _ptr(do), _ptr(lse), opt(dq), opt(dk), opt(dv), opt(db), _stream()))
    return dq, dk, dv, db


def permute(x: torch.Tensor, axes) -> torch.Tensor:
    """The reference's permute as a copy (src/backend/CPUKernels.cpp:1669-1717).  `x` is a dense tensor whose
    LAST torch dimension is the reference's dims[0]; `axes` is in the reference's numbering: dimension p of
    the result (dims[p]) is dimension axes[p] of the source."""
    x = _dev_f32(x, "x")
    nd = x.dim()
    axes = [int(a) for a in axes]
    if nd < 1 or nd > 4 or sorted(axes) != list(range(nd)):
        raise ValueError("permute: axes must be a permutation of the tensor's dimensions (at most 4)")
    sd = list(x.shape[::-1]) + [1] * (4 - nd)                      # reference order: innermost first
    dd = [sd[axes[p]] for p in range(nd)] + [1] * (4 - nd)
    ax = axes + list(range(nd, 4))
    out = torch.empty(tuple(dd[:nd][::-1]), dtype=torch.float32, device=x.device)
    cabi.check("permute_hip", _lib().permute_hip(_ptr(x), _ptr(out), x.numel(), nd, *ax, *sd, *dd, _stream()))
    return out


def repeat_back(a: torch.Tensor, b_shape) -> torch.Tensor:
    """The builder's ``repeat_back(a, b)`` (src/core/ComputeGraphHelper.cpp:114-133) with the kernel's index rule
    (src/backend/CPUKernels.cpp:2091-2148): `a` summed over the copies that a broadcast of a tensor of shape
    `b_shape` made.  Shapes are torch order (LAST dimension = the reference's dims[0]); dimension d of the
    result meets dimension d of `a` counted from dims[0], missing dimensions count as 1."""
    a = _dev_f32(a, "a")
    b_shape = tuple(int(d) for d in b_shape)
    if a.dim() < 1 or a.dim() > 4 or len(b_shape) < 1 or len(b_shape) > 4:
        raise ValueError("repeat_back: tensors have 1 to 4 dimensions")
    sd = list(a.shape[::-1]) + [1] * (4 - a.dim())
    dd = list(b_shape[::-1]) + [1] * (4 - len(b_shape))
    off = 0 if a.dim() >= len(b_shape) else a.dim() - len(b_shape)
    rd = []
    for d in range(4):
        sdim = sd[d + off] if 0 <= d + off < 4 else 1
        rd.append(sdim // dd[d] if dd[d] > 0 else 1)
    out = torch.empty(b_shape, dtype=torch.float32, device=a.device)
    cabi.check("repeat_back_hip", _lib().repeat_back_hip(_ptr(a), _ptr(out), *sd, *dd, *rd, _stream()))
    return out


# ----------------------------------------------------------------------------- Q8_0
def scale(x: torch.Tensor, s: float) -> torch.Tensor:
    """The reference's scale() node (src/core/ComputeGraphHelper.cpp:235-243; kernel src/backend/CPUKernels.cpp:1737-1754)."""
    x = _dev_f32(x, "x")
    out = torch.empty_like(x)
    cabi.check("scale_hip", _lib().scale_hip(_ptr(x), _ptr(out), float(s), x.numel(), _stream()))
    return out


UNARY_OP_RELU = 4


def relu(x: torch.Tensor) -> torch.Tensor:
    """The reference's relu() node (src/core/ComputeGraphHelper.cpp:513-520; kernel src/backend/CPUKernels.cpp:2649-2657)."""
    x = _dev_f32(x, "x")
    out = torch.empty_like(x)
    cabi.check("unary_hip", _lib().unary_hip(_ptr(x), _ptr(out), x.numel(), UNARY_OP_RELU, _stream()))
    return out


ELEMWISE_OPS = {"add": 0, "sub": 1, "mul": 2, "div": 3}


def bcast_elemwise(a: torch.Tensor, b: torch.Tensor, op: str = "add") -> torch.Tensor:
    """add / sub / mul / div with the reference's broadcast (src/backend/CPUKernels.cpp:446-596): the result has
    the shape of `a` (the reference's dst is a copy of src[0]'s shape, ComputeGraphHelper.cpp:61-124) and an operand
    with fewer elements repeats along the flat order, so it must cover the innermost dimensions."""
    a, b = _dev_f32(a, "a"), _dev_f32(b, "b")
    if op not in ELEMWISE_OPS:
        raise ValueError(f"bcast_elemwise: op must be one of {sorted(ELEMWISE_OPS)}")
    n = a.numel()
    if b.numel() == 0 or b.numel() > n or n % b.numel() != 0:
        raise ValueError(f"bcast_elemwise: {b.numel()} elements do not repeat into {n}")
    out = torch.empty_like(a)
    cabi.check("bcast_elemwise_hip", _lib().bcast_elemwise_hip(_ptr(a), _ptr(b), _ptr(out), n, n, b.numel(), ELEMWISE_OPS[op], _stream()))
    return out


def softmax(x: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
    """The reference's softmax() node over dims[0], the LAST torch dimension (src/core/ComputeGraphHelper.cpp:420-425;
    kernel src/backend/CPUKernels.cpp:1446-1467, incl. its 1 / (sum + 1e-9)).  With ``bias`` (whole rows of x's row
    length, a count that divides x's): softmax(x + bias) with the add node in front folded in, the same bits as
    softmax(bcast_elemwise(x, bias, "add"))."""
    x = _dev_f32(x, "x")
    if x.dim() < 1 or x.shape[-1] == 0:
        raise ValueError("softmax: needs a non-empty innermost dimension")
    out = torch.empty_like(x)
    N = x.shape[-1]
    M = x.numel() // N
    if bias is None:
        cabi.check("softmax_hip", _lib().softmax_hip(_ptr(x), _ptr(out), M, N, _stream()))
        return out
    bias = _dev_f32(bias, "bias")
    if bias.numel() == 0 or bias.numel() % N or M % (bias.numel() // N):
        raise ValueError("softmax: the bias must be whole rows of x's row length, a number of them that divides x's")
    cabi.check("softmax_add_hip", _lib().softmax_add_hip(_ptr(x), _ptr(bias), _ptr(out), M, N, bias.numel() // N, _stream()))
    return out


def out_prod_tt(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """out_prod of the {1,0,2,3} permutations of a and b without the copies: a [ne03,ne02,ne01,K], b [ne13,ne12,ne11,K]
    -> [ne13,ne12,ne11,ne01], contraction over the LAST torch dimension of both (src/modules/Attention.cpp:277-281:
    out_prod(permute(attn), permute(V))).  The bits of out_prod on the permuted copies."""
    a, b = _dev_f32(a, "a"), _dev_f32(b, "b")
    while a.dim() < 4:
        a = a.unsqueeze(0)
    while b.dim() < 4:
        b = b.unsqueeze(0)
    ne03, ne02, ne01, ne00 = a.shape
    ne13, ne12, ne11, ne10 = b.shape
    if ne00 != ne10:
        raise ValueError(f"out_prod_tt: contraction dims differ ({ne00} vs {ne10})")
    ne0, ne1, ne2, ne3 = ne01, ne11, max(ne02, ne12), max(ne03, ne13)
    out = torch.empty((ne3, ne2, ne1, ne0), dtype=torch.float32, device=a.device)
    dims = [ne00, ne01, ne02, ne03, ne10, ne11, ne12, ne13, ne0, ne1, ne2, ne3]
    cabi.check("out_prod_tt_hip", _lib().out_prod_tt_hip(_ptr(a), _ptr(b), _ptr(out), *dims, _stream()))
    return out


def quantize_rows_q8_0(x: torch.Tensor) -> torch.Tensor:
    """f32 [..., K] -> uint8 [..., K/32, 34] block_q8_0 records (include/ppml/QuantBlocks.h:62-79)."""
    x = _dev_f32(x, "x")
    ne = x.numel()
    if x.shape[-1] % QK:
        raise ValueError("quantize_rows_q8_0: innermost dimension is not a multiple of 32")
    out = torch.empty(x.shape[:-1] + (x.shape[-1] // QK, BLOCK_BYTES), dtype=torch.uint8, device=x.device)
    cabi.check("quantize_rows_q8_0_hip", _lib().quantize_rows_q8_0_hip(_ptr(x), _ptr(out), ne, _stream()))
    return out


def quantize_rows_q8_1(x: torch.Tensor) -> torch.Tensor:
    """f32 [..., K] -> uint8 [..., K/32, 36] block_q8_1 records, the reference's activation quantizer
    (include/ppml/QuantBlocks.h:81-111): d = vmax / -128, quants in [-128, 127], s = d * sum(q)."""
    x = _dev_f32(x, "x")
    ne = x.numel()
    if x.shape[-1] % QK:
        raise ValueError("quantize_rows_q8_1: innermost dimension is not a multiple of 32")
    out = torch.empty(x.shape[:-1] + (x.shape[-1] // QK, 36), dtype=torch.uint8, device=x.device)
    cabi.check("quantize_rows_q8_1_hip", _lib().quantize_rows_q8_1_hip(_ptr(x), _ptr(out), ne, _stream()))
    return out


def dequantize_q8_1(blocks: torch.Tensor) -> torch.Tensor:
    if not blocks.is_cuda or blocks.dtype != torch.uint8 or blocks.shape[-1] != 36:
        raise TypeError("dequantize_q8_1 expects uint8 [..., nblocks, 36] on the device")
    blocks = blocks.contiguous()
    nb = blocks.numel() // 36
    out = torch.empty(blocks.shape[:-2] + (blocks.shape[-2] * QK,), dtype=torch.float32, device=blocks.device)
    cabi.check("dequantize_q8_1_hip", _lib().dequantize_q8_1_hip(_ptr(blocks), _ptr(out), nb * QK, _stream()))
    return out


def dequantize_q8_0(blocks: torch.Tensor) -> torch.Tensor:
    if not blocks.is_cuda or blocks.dtype != torch.uint8 or blocks.shape[-1] != BLOCK_BYTES:
        raise TypeError("dequantize_q8_0 expects uint8 [..., nblocks, 34] on the device")
    blocks = blocks.contiguous()
    nb = blocks.numel() // BLOCK_BYTES
    out = torch.empty(blocks.shape[:-2] + (blocks.shape[-2] * QK,), dtype=torch.float32, device=blocks.device)
    cabi.check("dequantize_q8_0_hip", _lib().dequantize_q8_0_hip(_ptr(blocks), _ptr(out), nb * QK, _stream()))
    return out


class Q8Weight:
    """A quantized M x K weight resident on the device (rows = out features).

    ``data`` holds the bytes in layout ``wtype``; ``pack()`` returns the MFMA-fragment copy made
    once per weight, the step the reference does with its Q8_0R repack
    (src/model/PPML.cpp:4504-4528)."""

    def __init__(self, data: torch.Tensor, M: int, K: int, wtype: int):
        if K % QK:
            raise ValueError("quantized weights need K % 32 == 0 (blocks never cross a row)")
        self.data, self.M, self.K, self.wtype = data.contiguous(), M, K, wtype

    @classmethod
    def from_f32(cls, w: torch.Tensor) -> "Q8Weight":
        w = _dev_f32(w, "w")
        M, K = w.shape
        return cls(quantize_rows_q8_0(w).reshape(-1), M, K, WTYPE_Q8_0)

    def pack(self) -> "Q8Weight":
        if self.wtype == WTYPE_Q8_0M:
            return self
        lib = _lib()
        nbytes = lib.q8_weight_packed_bytes_hip(self.M, self.K)
        out = torch.empty(nbytes, dtype=torch.uint8, device=self.data.device)
        cabi.check("q8_weight_pack_hip",
                   lib.q8_weight_pack_hip(_ptr(self.data), self.wtype, self.M, self.K, _ptr(out), _stream()))
        return Q8Weight(out, self.M, self.K, WTYPE_Q8_0M)


_Q8_PATH_FLAGS = {"auto": 0, "weight-stationary": 4, "general": 4 | 8 | 256, "tiled": 4 | 8, "low-latency": 0, "low-latency-8": 16, "low-latency-16": 32, "low-latency-32": 48,
                  "weight-stationary-column-parts": 4 | 64, "weight-stationary-whole": 4 | 128}


def mul_mat_q8(w: Q8Weight, x: torch.Tensor, c_trans: int = 1, relu: bool = False,
               dump: bool = False, act: str = "q8_0", path: str = "auto", out: torch.Tensor = None):
    """Q8_0 linear: x f32 [N,K] (rows = tokens) times quantized w [M,K] -> [N,M] (c_trans=1, the
    LinearLayer orientation) or [M,N] (c_trans=0); src/backend/CUDAKernels.cpp:740-789.
    With ``dump`` also returns the kernel's own Q8_0 blocks of x and its per-block int32 sums.
    ``act`` selects the rule the activations are quantized with: "q8_0" (the CPU contract) or
    "q8_1" (what the reference's CUDA launcher does, src/cuda/MulMatQ8Kernel.cu:483-527).
    ``path`` restricts the kernel choice for a packed weight ("weight-stationary": not the low-latency kernel;
    "general": the general kernel only; "tiled": neither the low-latency nor the weight-stationary kernel, i.e. the tiled
    one wherever the problem is large enough for it; "low-latency-8" / "-16" / "-32": that unit size wherever an instance exists (32: K = 512 only);
    "weight-stationary-column-parts" / "-whole": that kernel with the columns shared out between work-groups
    wherever an instance exists / never); every choice gives the same bits.
    ``out``: a contiguous f32 device tensor of the result's shape to write into instead of a new one."""
    if act not in ("q8_0", "q8_1"):
        raise ValueError("mul_mat_q8: act must be 'q8_0' or 'q8_1'")
    x = _dev_f32(x, "x")
    if x.dim() != 2 or x.shape[1] != w.K:
        raise ValueError(f"mul_mat_q8: activations {tuple(x.shape)} do not match weight K={w.K}")
    N, K = x.shape
    M = w.M
    shape = (N, M) if c_trans else (M, N)
    if out is None:
        out = torch.empty(shape, dtype=torch.float32, device=x.device)
    elif (tuple(out.shape) != shape or out.dtype != torch.float32 or not out.is_contiguous() or out.device != x.device):
        raise ValueError(f"mul_mat_q8: out must be a contiguous f32 tensor of shape {shape} on {x.device}")
    lib = _lib()
    if not dump and not relu and act == "q8_0" and path == "auto":
        path = C.c_int(0)
        cabi.check("mul_mat_q8_hip", lib.mul_mat_q8_hip(_ptr(w.data), _ptr(x), _ptr(out), M, N, K, w.wtype,
                                                         c_trans, C.byref(path), _stream()))
        return out
    xq = sums = None
    if dump:
        xq = torch.empty((N, K // QK, BLOCK_BYTES), dtype=torch.uint8, device=x.device)
        sums = torch.empty((N, M, K // QK), dtype=torch.int32, device=x.device)
    cabi.check("mul_mat_q8_ex_hip", lib.mul_mat_q8_ex_hip(_ptr(w.data), _ptr(x), _ptr(out), M, N, K, w.wtype,
                                                           c_trans, (1 if relu else 0) | (2 if act == "q8_1" else 0) | _Q8_PATH_FLAGS[path],
                                                           _ptr(xq), _ptr(sums), _stream()))
    return (out, xq, sums) if dump else out
