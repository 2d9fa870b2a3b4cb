"""Scheduling rules and tensor bookkeeping of the executor; no GPU needed.

The table restates what the reference's CUDA backend answers for the three ops of this path
(src/backend/CUDABackend.cpp:121-163 OP_MUL_MAT, OP_OUT_PROD; 410-416 OP_OUTER_PROD_MEAN).
"""
import pytest

from proteinpredictmachinelearning_amd import backend as B


def _mm(t0, t1, out=B.F32, bias=None, k0=64, k1=64):
    s0 = B.Tensor((k0, 5), t0)
    s1 = B.Tensor((k1, 7), t1)
    src = [s0, s1] + ([B.Tensor((7,), bias)] if bias is not None else [])
    return B.Tensor((7, 5), out, B.OP_MUL_MAT, src)


@pytest.mark.parametrize("t0,t1,out,bias,want", [
    (B.F32, B.F32, B.F32, None, True),
    (B.F32, B.F32, B.F32, B.F32, True),          # bias epilogue: f32 path only
    (B.F32, B.F32, B.F16, None, False),
    (B.Q8_0, B.F32, B.F32, None, True),          # weight in src0 (ggml convention)
    (B.F32, B.Q8_0, B.F32, None, True),          # weight in src1 (LinearLayer convention)
    (B.F32, B.Q8_1, B.F32, None, True),
    (B.F32, B.Q8_0R, B.F32, None, True),
    (B.F32, B.Q8_0M, B.F32, None, True),
    (B.Q8_0, B.Q8_0, B.F32, None, False),        # exactly one side may be quantized
    (B.Q8_0, B.F32, B.F32, B.F32, False),        # no bias on the quantized path
    (B.F32, B.Q8_0, B.F32, B.F32, False),
    (B.Q8_0, B.F16, B.F32, None, False),         # activations must be f32
    (B.F32, B.Q8_0, B.F16, None, False),
    (B.F16, B.F16, B.F32, None, True),           # halves in, f32 out
    (B.F16, B.F16, B.F32, B.F32, False),         # no bias epilogue on the F16 path
    (B.F16, B.F16, B.F16, None, False),
    (B.F32, B.F16, B.F32, None, False),
])
def test_supports_op_mul_mat(t0, t1, out, bias, want):
    assert B.supports_op(_mm(t0, t1, out, bias)) is want


def test_supports_op_rejects_quantized_rows_that_split_a_block():
    assert B.supports_op(_mm(B.F32, B.Q8_0, k0=48, k1=48)) is False      # 48 % 32 != 0
    assert B.supports_op(_mm(B.F32, B.Q8_0, k0=96, k1=96)) is True


def test_supports_op_other_ops():
    a = B.Tensor((4, 3, 2, 2))
    b = B.Tensor((5, 3, 2, 2))
    assert B.supports_op(B.Tensor((4, 5, 2, 2), B.F32, B.OP_OUT_PROD, [a, b]))
    assert not B.supports_op(B.Tensor((4, 5, 2, 2), B.F32, B.OP_OUT_PROD, [a]))
    assert not B.supports_op(B.Tensor((4, 5, 2, 2), B.F16, B.OP_OUT_PROD, [a, b]))
    l = B.Tensor((3, 4, 8, 2))
    assert B.supports_op(B.Tensor((9, 4, 4, 2), B.F32, B.OP_OUTER_PROD_MEAN, [l, l]))
    l3 = B.Tensor((3, 4, 8))
    assert not B.supports_op(B.Tensor((9, 4, 4, 1), B.F32, B.OP_OUTER_PROD_MEAN, [l3, l3]))
    # no-op nodes are accepted (and skipped by the executor); everything else belongs to other backends
    assert B.supports_op(B.Tensor((4,), B.F32, B.OP_VIEW, [a]))
    assert B.supports_op(B.Tensor((4,), B.F32, B.OP_RESHAPE, [a]))
    assert not B.supports_op(B.Tensor((4, 3, 2, 2), B.F32, 24, [a]))          # OP_NORM: not on this path


def test_supports_op_elementwise_nodes_between_the_contractions():
    # src/backend/CUDABackend.cpp:340-344 OP_SCALE, 470-493 OP_UNARY (sub-type in op_params[0]),
    # 94-98 OP_ADD..OP_DIV, 236-237 OP_SOFT_MAX -- all f32 here
    a = B.Tensor((4, 3, 2, 2))
    h = B.Tensor((4, 3, 2, 2), B.F16)
    assert B.supports_op(B.Tensor((4, 3, 2, 2), B.F32, B.OP_SCALE, [a]))
    assert not B.supports_op(B.Tensor((4, 3, 2, 2), B.F32, B.OP_SCALE, []))
    assert not B.supports_op(B.Tensor((4, 3, 2, 2), B.F32, B.OP_SCALE, [h]))
    assert B.supports_op(B.Tensor((4, 3, 2, 2), B.F32, B.OP_SOFT_MAX, [a]))
    assert not B.supports_op(B.Tensor((4, 3, 2, 2), B.F16, B.OP_SOFT_MAX, [a]))
    relu = B.Tensor((4, 3, 2, 2), B.F32, B.OP_UNARY, [a]).set_param(0, B.UNARY_OP_RELU)
    assert B.supports_op(relu)
    for other in (0, 5, 7, 10, 13):              # ABS, GELU, SILU, SIGMOID, EXP: the CUDA backend's, not this path's
        assert not B.supports_op(B.Tensor((4, 3, 2, 2), B.F32, B.OP_UNARY, [a]).set_param(0, other))
    bias = B.Tensor((4, 3))
    for op in (B.OP_ADD, B.OP_SUB, B.OP_MUL, B.OP_DIV):
        assert B.supports_op(B.Tensor((4, 3, 2, 2), B.F32, op, [a, bias]))
        assert not B.supports_op(B.Tensor((4, 3, 2, 2), B.F32, op, [a]))
        assert not B.supports_op(B.Tensor((4, 3, 2, 2), B.F32, op, [a, h]))


def test_supports_op_fused_attention():
    # src/backend/CUDABackend.cpp:457-463: Q, K, V present, f32, head dimension (dims[0]) a multiple of 4 up to 64
    def node(d, type=B.F32, n_src=3):
        qkv = [B.Tensor((d, 10, 2, 1), type) for _ in range(n_src)]
        return B.Tensor((d, 10, 2, 1), B.F32, B.OP_FLASH_ATTN_EXT, qkv), qkv
    for d, want in [(4, True), (32, True), (64, True), (68, False), (6, False), (128, False)]:
        n, keep = node(d)
        assert B.supports_op(n) == want, d
    n, keep = node(32, B.F16)
    assert not B.supports_op(n)
    n, keep = node(32, B.F32, n_src=2)
    assert not B.supports_op(n)


def test_tensor_nbytes_follows_the_block_records():
    # include/ppml/Tensor.h:327-352: quantized bytes = blocks * record size; invalid shapes have none
    assert B.Tensor((256, 768), B.F32).nbytes == 256 * 768 * 4
    assert B.Tensor((256, 768), B.F16).nbytes == 256 * 768 * 2
    assert B.Tensor((256, 768), B.Q8_0).nbytes == 768 * 8 * 34
    assert B.Tensor((256, 768), B.Q8_0R).nbytes == 768 * 8 * 34
    assert B.Tensor((256, 768), B.Q8_1).nbytes == 768 * 8 * 36
    assert B.Tensor((250, 768), B.Q8_0).nbytes == 0
    assert B.Tensor((256, 768), B.Q8_0M).nbytes == 24 * 8 * (1024 + 64)
    with pytest.raises(ValueError):
        B.Tensor((1, 2, 3, 4, 5))


def test_graph_compute_without_backend_is_refused():
    from proteinpredictmachinelearning_amd import cabi

    assert cabi.load().ppml_hip_backend_graph_compute(None, None, 0) == B.NOT_SUPPORTED


def test_supports_op_permute():
    # src/backend/CUDABackend.cpp:113-119: f32 in, f32 out
    a = B.Tensor((4, 3, 2, 2))
    assert B.supports_op(B.Tensor((3, 4, 2, 2), B.F32, B.OP_PERMUTE, [a]))
    assert B.supports_op(B.Tensor((3, 4, 2, 2), B.F32, B.OP_TRANSPOSE, [a]))
    assert not B.supports_op(B.Tensor((3, 4, 2, 2), B.F32, B.OP_PERMUTE, []))
    assert not B.supports_op(B.Tensor((3, 4, 2, 2), B.F16, B.OP_PERMUTE, [a]))


def test_supports_op_tri_mul():
    # src/backend/CUDABackend.cpp:395-402: both operands and the result 4-D f32
    l, r = B.Tensor((8, 5, 6, 1)), B.Tensor((8, 4, 6, 1))
    assert B.supports_op(B.Tensor((8, 5, 4, 1), B.F32, B.OP_TRI_MUL, [l, r]))
    assert not B.supports_op(B.Tensor((8, 5, 4, 1), B.F32, B.OP_TRI_MUL, [l]))
    assert not B.supports_op(B.Tensor((8, 5, 4), B.F32, B.OP_TRI_MUL, [l, r]))
    assert not B.supports_op(B.Tensor((8, 5, 4, 1), B.F32, B.OP_TRI_MUL, [B.Tensor((8, 5, 6, 1), B.F16), r]))


def test_supports_op_tri_mul_back():
    # src/backend/CUDABackend.cpp:404-409
    g, l, r = B.Tensor((8, 5, 4, 1)), B.Tensor((8, 5, 6, 1)), B.Tensor((8, 4, 6, 1))
    gl, gr = B.Tensor((8, 5, 6, 1)), B.Tensor((8, 4, 6, 1))
    assert B.supports_op(B.Tensor((1,), B.F32, B.OP_TRI_MUL_BACK, [g, l, r, gl, gr]))
    assert B.supports_op(B.Tensor((1,), B.F32, B.OP_TRI_MUL_BACK, [g, l, r, None, gr]))
    assert not B.supports_op(B.Tensor((1,), B.F32, B.OP_TRI_MUL_BACK, [g, l, r]))
    assert not B.supports_op(B.Tensor((1,), B.F32, B.OP_TRI_MUL_BACK, [g, l, None, gl, gr]))


def test_supports_op_fused_attention_backward():
    # src/backend/CUDABackend.cpp:465-471 (the reference's CUDA kernel stops at d = 32; this one at 64)
    for d, want in [(4, True), (32, True), (64, True), (68, False), (6, False)]:
        q = B.Tensor((d, 10, 2, 1))
        assert B.supports_op(B.Tensor((10, 10, 2, 1), B.F32, B.OP_FLASH_ATTN_BACK, [q])) == want, d
    assert not B.supports_op(B.Tensor((10, 10, 2, 1), B.F32, B.OP_FLASH_ATTN_BACK, []))
    assert not B.supports_op(B.Tensor((10, 10, 2, 1), B.F32, B.OP_FLASH_ATTN_BACK, [B.Tensor((32, 10, 2, 1), B.F16)]))
