"""The executor on the GPU: nodes built like the reference's tests build them
(tests/test_cuda.cpp:39-51, 108-110), run through graph_compute, compared with the CPU oracle."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from proteinpredictmachinelearning_amd import backend as B  # noqa: E402


@pytest.fixture(scope="module")
def be():
    return B.Backend(0)


def _leaf(be, arr, type=B.F32, dims=None):
    arr = np.ascontiguousarray(arr)
    t = B.Tensor(dims if dims is not None else arr.shape[::-1], type)
    return be.upload(t, arr)


def test_identity(be):
    assert be.name == "HIP-gfx950" and be.priority == 1


def test_mul_mat_node_reference_inputs(be, oracle):
    # tests/test_cuda.cpp:133-167; dims are innermost-first: A [K, M], B [K, N], C [N, M]
    M, K, N = 17, 9, 23
    A = ((np.arange(M * K) % 11) * 0.5 - 2.0).astype(np.float32).reshape(M, K)
    Bm = ((np.arange(N * K) % 13) * 0.25 + 0.5).astype(np.float32).reshape(N, K)
    bias = ((np.arange(N) % 5) * 0.125 - 0.25).astype(np.float32)
    a, b, c = _leaf(be, A), _leaf(be, Bm), _leaf(be, bias)
    node = B.Tensor((N, M), B.F32, B.OP_MUL_MAT, [a, b])
    nodeb = B.Tensor((N, M), B.F32, B.OP_MUL_MAT, [a, b, c])
    assert be.supports_op(node) and be.supports_op(nodeb)
    assert be.graph_compute([node, nodeb]) == B.SUCCESS, be.last_error
    assert (be.download(node).reshape(M, N) == oracle.mul_mat_f32(A, Bm)).all()
    assert (be.download(nodeb).reshape(M, N) == oracle.mul_mat_f32(A, Bm, bias)).all()


@pytest.mark.parametrize("wname", ["Q8_0", "Q8_1", "Q8_0R", "packed"])
@pytest.mark.parametrize("wside", [0, 1])
def test_quantized_mul_mat_node(be, oracle, wname, wside):
    rows, K, F = 77, 128, 96        # tokens, in features, out features
    rng = np.random.default_rng(5)
    x = rng.standard_normal((rows, K)).astype(np.float32)
    w = (rng.standard_normal((F, K)) * 0.02).astype(np.float32)
    wq = oracle.quantize_q8_0(w)                                    # [F][K/32] 34-byte records
    if wname == "Q8_1":                                             # d, s, qs: s is not read
        rec = np.frombuffer(wq.tobytes(), dtype=np.uint8).reshape(-1, 34)
        raw = np.concatenate([rec[:, :2], np.zeros((rec.shape[0], 2), np.uint8), rec[:, 2:]], axis=1)
        wt = _leaf(be, raw.reshape(-1), B.Q8_1, (K, F))
    elif wname == "Q8_0R":
        wt = _leaf(be, np.frombuffer(oracle.repack_q8_0(wq).tobytes(), np.uint8), B.Q8_0R, (K, F))
    else:
        wt = _leaf(be, np.frombuffer(wq.tobytes(), np.uint8), B.Q8_0, (K, F))
    if wname == "packed":
        assert be.pack_weight(wt) == B.SUCCESS, be.last_error
        assert wt.type == B.Q8_0M
        assert be.pack_weight(wt) == B.SUCCESS                      # idempotent
    xt = _leaf(be, x)
    want = oracle.mul_mat_q8(wq, x, wtype=0, c_trans=1, fma=1)      # [rows][F]
    if wside == 1:      # mul_mat(x, W): node [F, rows], rows of the result are tokens
        node = B.Tensor((F, rows), B.F32, B.OP_MUL_MAT, [xt, wt])
        got = be_run(be, node).reshape(rows, F)
    else:               # mul_mat(W, x): node [rows, F], rows of the result are out features
        node = B.Tensor((rows, F), B.F32, B.OP_MUL_MAT, [wt, xt])
        got = be_run(be, node).reshape(F, rows).T
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-6 * np.abs(want).max())


def test_f16_mul_mat_node(be, oracle):
    M, K, N = 19, 24, 11
    rng = np.random.default_rng(10)
    a = rng.integers(-6, 7, size=(M, K)).astype(np.float16)
    b = rng.integers(-6, 7, size=(N, K)).astype(np.float16)
    at = _leaf(be, a.view(np.uint8).reshape(-1), B.F16, (K, M))
    bt = _leaf(be, b.view(np.uint8).reshape(-1), B.F16, (K, N))
    node = B.Tensor((N, M), B.F32, B.OP_MUL_MAT, [at, bt])
    got = be_run(be, node).reshape(M, N)
    assert (got == oracle.mul_mat_f16(a, b)).all()
    withbias = B.Tensor((N, M), B.F32, B.OP_MUL_MAT, [at, bt, _leaf(be, np.zeros(N, np.float32))])
    assert not be.supports_op(withbias)
    assert be.graph_compute([withbias]) == B.NOT_SUPPORTED


def test_quantized_mul_mat_node_with_cuda_activation_rule(be, oracle):
    rows, K, F = 50, 64, 40
    rng = np.random.default_rng(6)
    x = rng.standard_normal((rows, K)).astype(np.float32)
    wq = oracle.quantize_q8_0((rng.standard_normal((F, K)) * 0.02).astype(np.float32))
    wt = _leaf(be, np.frombuffer(wq.tobytes(), np.uint8), B.Q8_0, (K, F))
    xt = _leaf(be, x)
    be.set_q8_1_activations(True)
    try:
        got = be_run(be, B.Tensor((F, rows), B.F32, B.OP_MUL_MAT, [xt, wt])).reshape(rows, F)
    finally:
        be.set_q8_1_activations(False)
    assert (got == oracle.mul_mat_q8_act(wq, x, act=1)).all()
    got0 = be_run(be, B.Tensor((F, rows), B.F32, B.OP_MUL_MAT, [xt, wt])).reshape(rows, F)
    assert (got0 == oracle.mul_mat_q8(wq, x)).all()


def be_run(be, node):
    assert be.supports_op(node)
    assert be.graph_compute([node]) == B.SUCCESS, be.last_error
    return be.download(node)


def test_quantized_mul_mat_with_bias_is_refused(be, oracle):
    x = np.ones((4, 32), np.float32)
    wq = oracle.quantize_q8_0(np.ones((8, 32), np.float32))
    wt = _leaf(be, np.frombuffer(wq.tobytes(), np.uint8), B.Q8_0, (32, 8))
    node = B.Tensor((8, 4), B.F32, B.OP_MUL_MAT, [_leaf(be, x), wt, _leaf(be, np.zeros(8, np.float32))])
    assert not be.supports_op(node)
    assert be.graph_compute([node]) == B.NOT_SUPPORTED
    assert "not supported" in be.last_error


def test_out_prod_and_outer_prod_mean_nodes(be, oracle):
    rng = np.random.default_rng(3)
    s0 = rng.integers(-3, 4, size=(2, 3, 10, 7)).astype(np.float32)
    s1 = rng.integers(-3, 4, size=(2, 6, 10, 5)).astype(np.float32)
    a, b = _leaf(be, s0), _leaf(be, s1)
    op = B.Tensor((7, 5, 6, 2), B.F32, B.OP_OUT_PROD, [a, b])
    D, L, N, Bt = 3, 4, 8, 2
    l = rng.integers(-3, 4, size=D * L * N * Bt).astype(np.float32)
    r = rng.integers(-3, 4, size=D * L * N * Bt).astype(np.float32)
    lt, rt = _leaf(be, l, dims=(D, L, N, Bt)), _leaf(be, r, dims=(D, L, N, Bt))
    opm = B.Tensor((D * D, L, L, Bt), B.F32, B.OP_OUTER_PROD_MEAN, [lt, rt])
    assert be.graph_compute([op, opm]) == B.SUCCESS, be.last_error
    assert (be.download(op).reshape(2, 6, 5, 7) == oracle.out_prod(s0, s1)).all()
    assert (be.download(opm) == oracle.outer_prod_mean(l, r, D, L, N, Bt)).all()


def test_fused_attention_node(be, oracle):
    # the node ComputeGraphHelper.cpp:450-484 builds: src 0..2 = Q, K, V as [d, L, h, B], src 3 = bias,
    # src 4 = LSE output; op_params 0 scale, 1 causal, 2 softmax eps, 3 Br, 4 Bc
    rng = np.random.default_rng(8)
    Bt, h, L, d = 2, 3, 77, 32
    q, k, v = [rng.standard_normal((Bt, h, L, d)).astype(np.float32) for _ in range(3)]
    bias = rng.standard_normal((Bt, h, L, L)).astype(np.float32)
    scale = 1.0 / np.sqrt(8.0)                  # the caller's head_dim, not d (Attention.cpp:254-262)
    for with_bias, causal, with_lse in [(True, False, True), (False, True, False)]:
        qt, kt, vt = _leaf(be, q), _leaf(be, k), _leaf(be, v)
        bt = _leaf(be, bias) if with_bias else None
        lse = B.Tensor((L, h, Bt)) if with_lse else None        # unbound: the executor allocates it
        node = B.Tensor((d, L, h, Bt), B.F32, B.OP_FLASH_ATTN_EXT, [qt, kt, vt, bt, lse])
        node.set_param(0, float(scale)).set_param(1, int(causal)).set_param(2, 1e-9).set_param(3, 64).set_param(4, 64)
        assert be.supports_op(node)
        assert be.graph_compute([node]) == B.SUCCESS, be.last_error
        be.synchronize()
        want_o, want_lse = oracle.flash_attn_forward(q, k, v, bias if with_bias else None, causal=causal, scale=scale)
        got = be.download(node).reshape(Bt, h, L, d)
        assert np.abs(got - want_o).max() <= 1e-4 * np.abs(want_o).max()
        if with_lse:
            assert np.abs(be.download(lse).reshape(Bt, h, L) - want_lse).max() <= 1e-5 * (1 + np.abs(want_lse).max())
    # a head dimension the kernel does not take is refused before anything runs
    bad = B.Tensor((68, 8, 1, 1), B.F32, B.OP_FLASH_ATTN_EXT, [_leaf(be, np.zeros((1, 1, 8, 68), np.float32)) for _ in range(3)])
    assert be.graph_compute([bad]) == B.NOT_SUPPORTED


def test_fused_attention_subgraph_as_the_reference_builds_it(be, oracle):
    # ComputeGraphHelper.cpp:450-484: Q, K, V arrive as [L, D, h, B]; three permutes make [D, L, h, B], the fused
    # node runs, a last permute gives [L, D, h, B] back -- six nodes, all on this backend
    rng = np.random.default_rng(9)
    Bt, h, L, d = 2, 2, 40, 16
    q, k, v = [rng.standard_normal((Bt, h, L, d)).astype(np.float32) for _ in range(3)]     # flash layout values
    bias = rng.standard_normal((Bt, h, L, L)).astype(np.float32)
    leaves = [_leaf(be, np.ascontiguousarray(x.transpose(0, 1, 3, 2))) for x in (q, k, v)]    # dims [L, D, h, B]
    perms = []
    for t in leaves:
        n = B.Tensor((d, L, h, Bt), B.F32, B.OP_PERMUTE, [t])
        for i, a in enumerate((1, 0, 2, 3)):
            n.set_param(i, a)
        perms.append(n)
    flash = B.Tensor((d, L, h, Bt), B.F32, B.OP_FLASH_ATTN_EXT, perms + [_leaf(be, bias), B.Tensor((L, h, Bt))])
    flash.set_param(0, float(1.0 / np.sqrt(d))).set_param(1, 0).set_param(2, 1e-9).set_param(3, 64).set_param(4, 64)
    out = B.Tensor((L, d, h, Bt), B.F32, B.OP_TRANSPOSE, [flash])
    for i, a in enumerate((1, 0, 2, 3)):
        out.set_param(i, a)
    assert be.graph_compute(perms + [flash, out]) == B.SUCCESS, be.last_error
    be.synchronize()
    want, _ = oracle.flash_attn_forward(q, k, v, bias)
    got = be.download(out).reshape(Bt, h, d, L).transpose(0, 1, 3, 2)
    assert np.abs(got - want).max() <= 1e-4 * np.abs(want).max()
    assert np.array_equal(be.download(perms[0]).reshape(Bt, h, L, d), q)
    # an axis map outside the tensor's dimensions is refused (src/backend/CUDAKernels.cpp:1376-1381)
    bad = B.Tensor((d, L, h, Bt), B.F32, B.OP_PERMUTE, [leaves[0]])
    bad.set_param(0, 7)
    assert be.graph_compute([bad]) == B.NOT_SUPPORTED


def test_tri_mul_node(be, oracle):
    # ComputeGraphHelper.cpp:390-413: node [D, I, J, B]; op_params[0] = L (float), low byte of op_params[4] = outgoing
    rng = np.random.default_rng(12)
    D, I, J, K, Bt = 4, 9, 7, 11, 1
    for outgoing in (True, False):
        ldims = (D, I, K, Bt) if outgoing else (D, K, I, Bt)
        rdims = (D, J, K, Bt) if outgoing else (D, K, J, Bt)
        left = rng.standard_normal(D * I * K * Bt).astype(np.float32)
        right = rng.standard_normal(D * J * K * Bt).astype(np.float32)
        node = B.Tensor((D, I, J, Bt), B.F32, B.OP_TRI_MUL, [_leaf(be, left, dims=ldims), _leaf(be, right, dims=rdims)])
        node.set_param(0, float(K)).set_param(4, int(outgoing))
        assert be.graph_compute([node]) == B.SUCCESS, be.last_error
        want = oracle.tri_mul(left, right, D, I, J, K, Bt, float(K), outgoing)
        assert np.abs(be.download(node) - want).max() <= 1e-4 * np.abs(want).max()
    node.set_param(0, 0.0)                              # L == 0 (src/backend/CUDAKernels.cpp:1165)
    assert be.graph_compute([node]) == B.NOT_SUPPORTED


def test_fused_attention_subgraph_without_its_bridges(oracle):
    """The same six-node subgraph with set_fuse_attention_bridges(1): the four permutations are not executed
    (their tensors stay unbound), the result equals the unfused run; a bridge with a second reader is kept."""
    be2 = B.Backend(0)
    rng = np.random.default_rng(10)
    Bt, h, L, d = 2, 2, 70, 32
    q, k, v = [rng.standard_normal((Bt, h, L, d)).astype(np.float32) for _ in range(3)]
    bias = rng.standard_normal((Bt, h, L, L)).astype(np.float32)
    want, want_lse = oracle.flash_attn_forward(q, k, v, bias)

    def build(extra_reader):
        leaves = [_leaf(be2, np.ascontiguousarray(x.transpose(0, 1, 3, 2))) for x in (q, k, v)]
        perms = []
        for t in leaves:
            n = B.Tensor((d, L, h, Bt), B.F32, B.OP_PERMUTE, [t])
            for i, a in enumerate((1, 0, 2, 3)):
                n.set_param(i, a)
            perms.append(n)
        lse = B.Tensor((L, h, Bt))
        flash = B.Tensor((d, L, h, Bt), B.F32, B.OP_FLASH_ATTN_EXT, perms + [_leaf(be2, bias), lse])
        flash.set_param(0, float(1.0 / np.sqrt(d))).set_param(1, 0).set_param(2, 1e-9).set_param(3, 64).set_param(4, 64)
        out = B.Tensor((L, d, h, Bt), B.F32, B.OP_PERMUTE, [flash])
        for i, a in enumerate((1, 0, 2, 3)):
            out.set_param(i, a)
        nodes = perms + [flash, out]
        if extra_reader:                                # a second reader of the permuted Q: its bridge must run
            again = B.Tensor((L, d, h, Bt), B.F32, B.OP_PERMUTE, [perms[0]])
            for i, a in enumerate((1, 0, 2, 3)):
                again.set_param(i, a)
            nodes.append(again)
        return leaves, perms, flash, lse, out, nodes

    be2.set_fuse_attention_bridges(True)
    leaves, perms, flash, lse, out, nodes = build(False)
    assert be2.graph_compute(nodes) == B.SUCCESS, be2.last_error
    be2.synchronize()
    got = be2.download(out).reshape(Bt, h, d, L).transpose(0, 1, 3, 2)
    assert np.abs(got - want).max() <= 1e-4 * np.abs(want).max()
    assert np.abs(be2.download(lse).reshape(Bt, h, L) - want_lse).max() <= 1e-5 * (1 + np.abs(want_lse).max())
    with pytest.raises(RuntimeError):
        be2.download(perms[0])                          # never allocated: the bridge was not executed
    with pytest.raises(RuntimeError):
        be2.download(flash)

    leaves, perms, flash, lse, out, nodes = build(True)
    assert be2.graph_compute(nodes) == B.SUCCESS, be2.last_error
    be2.synchronize()
    assert np.array_equal(be2.download(perms[0]).reshape(Bt, h, L, d), q)      # inputs not fused this time
    got = be2.download(out).reshape(Bt, h, d, L).transpose(0, 1, 3, 2)            # the trailing bridge still is
    assert np.abs(got - want).max() <= 1e-4 * np.abs(want).max()
    assert np.array_equal(be2.download(nodes[-1]).reshape(Bt, h, d, L), q.transpose(0, 1, 3, 2))

    be2.set_fuse_attention_bridges(False)
    leaves, perms, flash, lse, out, nodes = build(False)
    assert be2.graph_compute(nodes) == B.SUCCESS, be2.last_error
    be2.synchronize()
    assert np.array_equal(be2.download(perms[1]).reshape(Bt, h, L, d), k)
    assert np.abs(be2.download(flash).reshape(Bt, h, L, d) - want).max() <= 1e-4 * np.abs(want).max()


def test_tri_mul_back_node(be, oracle):
    # src/backend/CUDAKernels.cpp:1172-1201: outputs live in src[3] / src[4]; unbound ones are allocated here
    rng = np.random.default_rng(13)
    D, I, J, K, Bt = 3, 9, 7, 11, 1
    for outgoing in (True, False):
        ldims = (D, I, K, Bt) if outgoing else (D, K, I, Bt)
        rdims = (D, J, K, Bt) if outgoing else (D, K, J, Bt)
        left = rng.standard_normal(D * I * K * Bt).astype(np.float32)
        right = rng.standard_normal(D * J * K * Bt).astype(np.float32)
        grad = rng.standard_normal(D * I * J * Bt).astype(np.float32)
        gl, gr = B.Tensor(ldims), B.Tensor(rdims)
        node = B.Tensor((1,), B.F32, B.OP_TRI_MUL_BACK, [_leaf(be, grad, dims=(D, I, J, Bt)), _leaf(be, left, dims=ldims),
                                                         _leaf(be, right, dims=rdims), gl, gr])
        node.set_param(0, float(K)).set_param(4, int(outgoing))
        assert be.graph_compute([node]) == B.SUCCESS, be.last_error
        want_l, want_r = oracle.tri_mul_back(grad, left, right, D, I, J, K, Bt, float(K), outgoing)
        assert np.abs(be.download(gl) - want_l).max() <= 1e-4 * np.abs(want_l).max()
        assert np.abs(be.download(gr) - want_r).max() <= 1e-4 * np.abs(want_r).max()


def test_fused_attention_backward_node(be, oracle):
    # src/backend/CUDAKernels.cpp:905-924: src 0..2 Q K V, 3 bias, 4 O, 5 dO, 6 LSE, 7..9 dQ dK dV; dbias in the
    # node itself when op_params[5] != 0
    rng = np.random.default_rng(16)
    Bt, h, L, d = 1, 2, 50, 16
    q, k, v, do = [rng.standard_normal((Bt, h, L, d)).astype(np.float32) for _ in range(4)]
    bias = rng.standard_normal((Bt, h, L, L)).astype(np.float32)
    o, lse = oracle.flash_attn_forward(q, k, v, bias)
    want = oracle.flash_attn_backward(q, k, v, bias, o, do, lse)
    for want_dbias in (1, 0):
        dq, dk, dv = B.Tensor((d, L, h, Bt)), B.Tensor((d, L, h, Bt)), B.Tensor((d, L, h, Bt))
        node = B.Tensor((L, L, h, Bt), B.F32, B.OP_FLASH_ATTN_BACK,
                        [_leaf(be, q), _leaf(be, k), _leaf(be, v), _leaf(be, bias), _leaf(be, o), _leaf(be, do), _leaf(be, lse), dq, dk, dv])
        node.set_param(0, float(1.0 / np.sqrt(d))).set_param(1, 0).set_param(5, want_dbias)
        assert be.supports_op(node)
        assert be.graph_compute([node]) == B.SUCCESS, be.last_error
        for t, w in ((dq, want[0]), (dk, want[1]), (dv, want[2])):
            assert np.abs(be.download(t).reshape(w.shape) - w).max() <= 1e-4 * np.abs(w).max()
        if want_dbias:
            assert np.abs(be.download(node).reshape(want[3].shape) - want[3]).max() <= 1e-4 * np.abs(want[3]).max()
        else:
            with pytest.raises(RuntimeError):
                be.download(node)                       # not asked for: not even allocated


def test_outer_prod_mean_back_node(be, oracle):
    # src/backend/CUDAKernels.cpp:1223-1245
    rng = np.random.default_rng(15)
    D, L, N, Bt = 3, 6, 8, 2
    left = rng.standard_normal(D * L * N * Bt).astype(np.float32)
    right = rng.standard_normal(D * L * N * Bt).astype(np.float32)
    grad = rng.standard_normal(D * D * L * L * Bt).astype(np.float32)
    gl, gr = B.Tensor((D, L, N, Bt)), B.Tensor((D, L, N, Bt))
    node = B.Tensor((1,), B.F32, B.OP_OUTER_PROD_MEAN_BACK,
                    [_leaf(be, grad, dims=(D * D, L, L, Bt)), _leaf(be, left, dims=(D, L, N, Bt)), _leaf(be, right, dims=(D, L, N, Bt)), gl, gr])
    assert be.supports_op(node)
    assert be.graph_compute([node]) == B.SUCCESS, be.last_error
    want_l, want_r = oracle.outer_prod_mean_back(grad, left, right, D, L, N, Bt)
    assert np.abs(be.download(gl) - want_l).max() <= 1e-4 * np.abs(want_l).max()
    assert np.abs(be.download(gr) - want_r).max() <= 1e-4 * np.abs(want_r).max()


def test_backward_gemms_of_mul_mat_as_the_reference_builds_them(be, oracle):
    """ComputeGraph.cpp:708-741: for y = mul_mat(A, W) (A dims [K,M], W dims [K,N], y dims [N,M]) the gradients are
    dA = mul_mat(grad, mat_transpose(W)) and dW = mul_mat(mat_transpose(grad), mat_transpose(A)), where
    mat_transpose is a permutation copy: five nodes, all on this backend.  Checked against grad @ W and grad^T @ A."""
    rng = np.random.default_rng(14)
    M, K, N = 37, 24, 19
    A = rng.integers(-3, 4, size=(M, K)).astype(np.float32)       # dims [K, M]
    W = rng.integers(-3, 4, size=(N, K)).astype(np.float32)       # dims [K, N]
    G = rng.integers(-3, 4, size=(M, N)).astype(np.float32)       # dims [N, M]
    a, w, g = _leaf(be, A), _leaf(be, W), _leaf(be, G)

    def mat_t(t, dims):
        n = B.Tensor(dims, B.F32, B.OP_PERMUTE, [t])
        n.set_param(0, 1).set_param(1, 0)
        return n
    wt, gt, at = mat_t(w, (N, K)), mat_t(g, (M, N)), mat_t(a, (M, K))
    dA = B.Tensor((K, M), B.F32, B.OP_MUL_MAT, [g, wt])          # mul_mat(a, b): dims [b.dims[1], a.dims[1]]
    dW = B.Tensor((K, N), B.F32, B.OP_MUL_MAT, [gt, at])
    assert be.graph_compute([wt, dA, gt, at, dW]) == B.SUCCESS, be.last_error
    assert np.array_equal(be.download(dA).reshape(M, K), G @ W)
    assert np.array_equal(be.download(dW).reshape(N, K), G.T @ A)


def test_view_sources_are_resolved_and_noop_nodes_skipped(be, oracle):
    # a reshape node built with only src[0] set, and an offset view with view_src set, both feed a
    # mul_mat (src/backend/CUDABackend.cpp:800-819)
    M, K, N = 6, 8, 5
    rng = np.random.default_rng(8)
    big = rng.integers(-4, 5, size=(2 * M, K)).astype(np.float32)       # two stacked A matrices
    Bm = rng.integers(-4, 5, size=(N, K)).astype(np.float32)
    base = _leaf(be, big)
    second = B.Tensor((K, M), B.F32, B.OP_VIEW).view_of(base, M * K * 4)
    flat = _leaf(be, Bm.reshape(-1))
    resh = B.Tensor((K, N), B.F32, B.OP_RESHAPE, [flat])
    node = B.Tensor((N, M), B.F32, B.OP_MUL_MAT, [second, resh])
    assert be.graph_compute([second, resh, node]) == B.SUCCESS, be.last_error
    assert (be.download(node).reshape(M, N) == oracle.mul_mat_f32(big[M:], Bm)).all()


def test_failure_statuses(be):
    a = _leaf(be, np.ones((3, 4), np.float32))
    b = _leaf(be, np.ones((5, 4), np.float32))
    # an op without a kernel here: NOT_SUPPORTED, nothing launched
    assert be.graph_compute([B.Tensor((4, 3), B.F32, 24, [a])]) == B.NOT_SUPPORTED          # OP_NORM
    # a unary sub-type this path does not carry (op_params[0] = 7, SILU)
    assert be.graph_compute([B.Tensor((4, 3), B.F32, B.OP_UNARY, [a]).set_param(0, 7)]) == B.NOT_SUPPORTED
    # a source nobody bound
    ghost = B.Tensor((4, 5))
    assert be.graph_compute([B.Tensor((5, 3), B.F32, B.OP_MUL_MAT, [a, ghost])]) == B.NOT_SUPPORTED
    assert "src1" in be.last_error
    # a host pointer under a scheduler (skip_alloc): the copies across backends are the scheduler's nodes, so
    # the executor refuses it (src/backend/CUDABackend.cpp:824-830, 894-973)
    host = np.ones((5, 4), np.float32)
    fake = B.Tensor((4, 5)).bind(host.ctypes.data)
    import torch
    out = torch.zeros(15, device="cuda")
    be.set_skip_alloc(True)
    try:
        assert be.graph_compute([B.Tensor((5, 3), B.F32, B.OP_MUL_MAT, [a, fake]).bind(out.data_ptr())]) == B.NOT_SUPPORTED
        assert "src1" in be.last_error
        assert be.graph_compute([B.Tensor((5, 3), B.F32, B.OP_MUL_MAT, [a, b]).bind(out.data_ptr())]) == B.SUCCESS
    finally:
        be.set_skip_alloc(False)
    assert (out.cpu().numpy() == 4.0).all()
    # a host pointer as the OUTPUT is never covered
    res = np.zeros((3, 5), np.float32)
    assert be.graph_compute([B.Tensor((5, 3), B.F32, B.OP_MUL_MAT, [a, b]).bind(res.ctypes.data)]) == B.NOT_SUPPORTED
    # shapes that do not match the node
    assert be.graph_compute([B.Tensor((6, 3), B.F32, B.OP_MUL_MAT, [a, b])]) == B.NOT_SUPPORTED
    # with a scheduler in charge of allocation the executor allocates nothing
    be.set_skip_alloc(True)
    try:
        assert be.graph_compute([B.Tensor((5, 3), B.F32, B.OP_MUL_MAT, [a, b])]) == B.NOT_SUPPORTED
    finally:
        be.set_skip_alloc(False)
    # and the backend still works afterwards
    node = B.Tensor((5, 3), B.F32, B.OP_MUL_MAT, [a, b])
    assert be.graph_compute([node]) == B.SUCCESS
    assert (be.download(node) == 4.0).all()


def test_host_resident_leaves_get_device_shadows(be, oracle):
    # single-backend mode: sources bound to host memory (leaves nobody uploaded) are copied to the device for
    # the length of graph_compute and the tensors' own fields are put back afterwards
    # (src/backend/CUDABackend.cpp:521-577, 824-830)
    M, K, N = 29, 40, 21
    rng = np.random.default_rng(21)
    A = rng.integers(-4, 5, size=(M, K)).astype(np.float32)
    Wm = rng.integers(-4, 5, size=(N, K)).astype(np.float32)
    bias = rng.integers(-4, 5, size=N).astype(np.float32)
    a = B.Tensor((K, M)).bind(A.ctypes.data)                      # host
    w = _leaf(be, Wm)                                             # device
    c = B.Tensor((N,)).bind(bias.ctypes.data)                     # host
    node = B.Tensor((N, M), B.F32, B.OP_MUL_MAT, [a, w, c])
    # a second node reads the same host leaf, and a view of it: one shadow per tensor, views follow their root
    half = B.Tensor((K, M // 2), B.F32, B.OP_VIEW).view_of(a, 0)
    node2 = B.Tensor((N, M // 2), B.F32, B.OP_MUL_MAT, [half, w])
    assert be.graph_compute([node, half, node2]) == B.SUCCESS, be.last_error
    assert be.host_shadows_made == 2                              # a and bias; the view borrowed a's copy
    assert (be.download(node).reshape(M, N) == oracle.mul_mat_f32(A, Wm, bias)).all()
    assert (be.download(node2).reshape(M // 2, N) == oracle.mul_mat_f32(A[:M // 2], Wm)).all()
    # the host tensors are host tensors again (and the view unbound again): a second run uploads the (changed)
    # contents anew, whichever of the two comes first
    A[:] = A[::-1].copy()
    node4 = B.Tensor((N, M // 2), B.F32, B.OP_MUL_MAT, [half, w])
    assert be.graph_compute([half, node4]) == B.SUCCESS, be.last_error
    assert (be.download(node4).reshape(M // 2, N) == oracle.mul_mat_f32(A[:M // 2], Wm)).all()
    node3 = B.Tensor((N, M), B.F32, B.OP_MUL_MAT, [a, w])
    assert be.graph_compute([node3]) == B.SUCCESS, be.last_error
    assert be.host_shadows_made == 1
    assert (be.download(node3).reshape(M, N) == oracle.mul_mat_f32(A, Wm)).all()
    # a quantized host weight is sized by its blocks
    wq = oracle.quantize_q8_0((rng.standard_normal((N, 64)) * 0.02).astype(np.float32))
    raw = np.frombuffer(wq.tobytes(), np.uint8).copy()
    x = rng.standard_normal((M, 64)).astype(np.float32)
    wt = B.Tensor((64, N), B.Q8_0).bind(raw.ctypes.data)
    qn = B.Tensor((N, M), B.F32, B.OP_MUL_MAT, [_leaf(be, x), wt])
    assert be.graph_compute([qn]) == B.SUCCESS, be.last_error
    assert (be.download(qn).reshape(M, N) == oracle.mul_mat_q8(wq, x, wtype=0, c_trans=1, fma=1)).all()


@pytest.mark.parametrize("src_dims,dst_dims", [((19, 37), (19,)), ((5, 3, 4, 2), (5, 1, 4, 1)), ((6, 4), (3, 4)),
                                               ((768, 2000), (768,)), ((8, 51, 6), (8, 1, 6))])
def test_repeat_back_node(be, oracle, src_dims, dst_dims):
    # OP_REPEAT_BACK, the bias gradient of a mul_mat (src/core/ComputeGraph.cpp:742): dims innermost first
    rng = np.random.default_rng(len(src_dims) * 100 + src_dims[0])
    g = rng.integers(-6, 7, size=src_dims[::-1]).astype(np.float32)
    node = B.Tensor(dst_dims, B.F32, B.OP_REPEAT_BACK, [_leaf(be, g)])
    assert be.supports_op(node)
    got = be_run(be, node).reshape(dst_dims[::-1])
    assert (got == oracle.repeat_back(g, dst_dims[::-1])).all()      # small integers: exact in any order


def test_backward_of_a_biased_linear_stays_on_the_device(be, oracle):
    """ComputeGraph.cpp:708-742 for y = mul_mat(A, W, bias): dA, dW as above and dbias = repeat_back(grad, bias);
    six nodes, none of which leaves this backend."""
    rng = np.random.default_rng(16)
    M, K, N = 45, 32, 27
    A = rng.integers(-3, 4, size=(M, K)).astype(np.float32)
    W = rng.integers(-3, 4, size=(N, K)).astype(np.float32)
    G = rng.integers(-3, 4, size=(M, N)).astype(np.float32)
    a, w, g = _leaf(be, A), _leaf(be, W), _leaf(be, G)

    def mat_t(t, dims):
        n = B.Tensor(dims, B.F32, B.OP_PERMUTE, [t])
        n.set_param(0, 1).set_param(1, 0)
        return n
    wt, gt, at = mat_t(w, (N, K)), mat_t(g, (M, N)), mat_t(a, (M, K))
    dA = B.Tensor((K, M), B.F32, B.OP_MUL_MAT, [g, wt])
    dW = B.Tensor((K, N), B.F32, B.OP_MUL_MAT, [gt, at])
    db = B.Tensor((N,), B.F32, B.OP_REPEAT_BACK, [g])
    nodes = [wt, dA, gt, at, dW, db]
    assert all(be.supports_op(n) for n in nodes)
    assert be.graph_compute(nodes) == B.SUCCESS, be.last_error
    assert np.array_equal(be.download(dA).reshape(M, K), G @ W)
    assert np.array_equal(be.download(dW).reshape(N, K), G.T @ A)
    assert np.array_equal(be.download(db), G.sum(axis=0))
    assert np.array_equal(be.download(db), oracle.repeat_back(G, (N,)))


@pytest.mark.parametrize("T,K,N", [(2601, 128, 256), (10609, 128, 512), (300, 40, 24)])
def test_weight_gradient_reads_the_untransposed_matrices(be, T, K, N):
    """dW = mul_mat(mat_transpose(grad), mat_transpose(x)) (src/core/ComputeGraph.cpp:733-738): the two transpositions
    are not executed when nobody else reads them, the contraction runs over the rows of grad and x as they lie, and the
    result has the bits of the three nodes run one by one.  A transposition somebody else reads stays a node."""
    rng = np.random.default_rng(T)
    X = rng.standard_normal((T, K)).astype(np.float32)
    G = rng.standard_normal((T, N)).astype(np.float32)

    def build(extra_reader):
        x, g = _leaf(be, X), _leaf(be, G)
        gt = B.Tensor((T, N), B.F32, B.OP_PERMUTE, [g]); gt.set_param(0, 1).set_param(1, 0)
        xt = B.Tensor((T, K), B.F32, B.OP_PERMUTE, [x]); xt.set_param(0, 1).set_param(1, 0)
        dW = B.Tensor((K, N), B.F32, B.OP_MUL_MAT, [gt, xt])
        nodes = [gt, xt, dW]
        if extra_reader:
            other = B.Tensor((T, K), B.F32, B.OP_SCALE, [xt]).set_param(0, 2.0)
            nodes.append(other)
        return nodes, dW, xt

    results = {}
    for fused in (True, False):
        be.set_fuse_permutes_into_mul_mat(fused)
        try:
            nodes, dW, xt = build(False)
            assert be.graph_compute(nodes) == B.SUCCESS, be.last_error
            assert be.nodes_fused_away == (2 if fused else 0)
            results[fused] = be.download(dW).reshape(N, K)
        finally:
            be.set_fuse_permutes_into_mul_mat(True)
    assert np.array_equal(results[True].view(np.int32), results[False].view(np.int32))
    want = G.astype(np.float64).T @ X.astype(np.float64)
    bound = (np.abs(G.astype(np.float64)).T @ np.abs(X.astype(np.float64))) * (T + 2) * 2.0 ** -24
    assert np.all(np.abs(results[True] - want) <= bound)
    nodes, dW, xt = build(True)
    assert be.graph_compute(nodes) == B.SUCCESS, be.last_error
    assert be.nodes_fused_away == 0
    assert np.array_equal(be.download(dW).reshape(N, K).view(np.int32), results[False].view(np.int32))
    assert np.array_equal(be.download(xt).reshape(K, T), X.T)


def test_f32_arithmetic_is_a_field_of_the_backend(be, oracle):
    # two backends with different pipes do not disturb each other or the calling thread's own setting
    import torch
    from proteinpredictmachinelearning_amd import ops
    M, K, N = 70, 40, 50
    rng = np.random.default_rng(3)
    A = rng.standard_normal((M, K)).astype(np.float32)
    Wm = rng.standard_normal((N, K)).astype(np.float32)
    # what each pipe gives through the launcher: the sums differ in their last bits, which tells the pipes apart
    per_pipe = {}
    for pipe in ("split", "fp32"):
        before = ops.set_f32_arithmetic(pipe)
        try:
            per_pipe[pipe] = ops.mul_mat(torch.from_numpy(A).cuda(), torch.from_numpy(Wm).cuda()).cpu().numpy()
        finally:
            ops.set_f32_arithmetic(before)
    assert not np.array_equal(per_pipe["split"], per_pipe["fp32"])
    other = B.Backend(0)
    other.set_f32_arithmetic("fp32")
    be.set_f32_arithmetic("split")
    assert ops.set_f32_arithmetic("split") in ("split", "fp32")
    try:
        for _ in range(2):
            n1 = B.Tensor((N, M), B.F32, B.OP_MUL_MAT, [_leaf(be, A), _leaf(be, Wm)])
            n2 = B.Tensor((N, M), B.F32, B.OP_MUL_MAT, [_leaf(other, A), _leaf(other, Wm)])
            assert be.graph_compute([n1]) == B.SUCCESS and other.graph_compute([n2]) == B.SUCCESS
            assert np.array_equal(be.download(n1).reshape(M, N), per_pipe["split"])
            assert np.array_equal(other.download(n2).reshape(M, N), per_pipe["fp32"])
        assert ops.set_f32_arithmetic("split") == "split"        # the thread's setting came back after each call
    finally:
        other.set_f32_arithmetic(None)
        be.set_f32_arithmetic(None)


# ----------------------------------------------------------------------------- element-wise nodes and their folding
def _q8_leaf(be, oracle, w, layout):
    """A quantized weight leaf [K, F] in one of the layouts the reference's loader produces (PPML.cpp:4504-4528)."""
    F, K = w.shape
    wq = oracle.quantize_q8_0(w)
    if layout == "Q8_0R":
        t = _leaf(be, np.frombuffer(oracle.repack_q8_0(wq).tobytes(), np.uint8), B.Q8_0R, (K, F))
    else:
        t = _leaf(be, np.frombuffer(wq.tobytes(), np.uint8), B.Q8_0, (K, F))
        if layout == "packed":
            assert be.pack_weight(t) == B.SUCCESS, be.last_error
    return t, wq


def _feed_forward_graph(be, x_leaf, w1, w2, L, D, H):
    """FeedForward::forward_graph without its layer norm (src/modules/Attention.cpp:1097-1104; dropout is the identity
    in evaluation, src/ops/Dropout.cpp:87-91), each linear as LinearLayer::forward_graph builds it
    (src/model/Embedding.cpp:120-153): view to [D_in, tokens] -> mul_mat -> view back."""
    tok = L * L
    x_flat = B.Tensor((D, tok), B.F32, B.OP_VIEW).view_of(x_leaf)
    h_flat = B.Tensor((H, tok), B.F32, B.OP_MUL_MAT, [x_flat, w1])
    h = B.Tensor((H, L, L, 1), B.F32, B.OP_VIEW).view_of(h_flat)
    r = B.Tensor((H, L, L, 1), B.F32, B.OP_UNARY, [h]).set_param(0, B.UNARY_OP_RELU)
    r_flat = B.Tensor((H, tok), B.F32, B.OP_VIEW).view_of(r)
    y_flat = B.Tensor((D, tok), B.F32, B.OP_MUL_MAT, [r_flat, w2])
    y = B.Tensor((D, L, L, 1), B.F32, B.OP_VIEW).view_of(y_flat)
    return [x_flat, h_flat, h, r, r_flat, y_flat, y], r, y_flat


@pytest.mark.parametrize("layout", ["Q8_0R", "packed"])
@pytest.mark.parametrize("L", [19, 103])
def test_pair_feed_forward_graph_fused_and_node_by_node(be, oracle, layout, L):
    """linear1 128 -> 512, relu, linear2 512 -> 128 on the pair track (L = 103: the configured 10609 tokens): the ReLU
    node folded into the second matmul's quantizer, and executed as a node of its own -- the same bits both ways, and
    the oracle's."""
    D, H = 128, 512
    rng = np.random.default_rng(L)
    x = rng.standard_normal((L * L, D)).astype(np.float32)
    w1 = (rng.standard_normal((H, D)) * 0.02).astype(np.float32)
    w2 = (rng.standard_normal((D, H)) * 0.02).astype(np.float32)
    w1t, w1q = _q8_leaf(be, oracle, w1, layout)
    w2t, w2q = _q8_leaf(be, oracle, w2, layout)
    hidden = oracle.mul_mat_q8(w1q, x, wtype=0, c_trans=1, fma=1)
    want = oracle.mul_mat_q8(w2q, oracle.relu(hidden), wtype=0, c_trans=1, fma=1)
    xl = _leaf(be, x, dims=(D, L, L, 1))
    results = []
    for fuse in (True, False):
        be.set_fuse_relu_into_q8(fuse)
        try:
            graph, relu, y_flat = _feed_forward_graph(be, xl, w1t, w2t, L, D, H)
            assert be.graph_compute(graph) == B.SUCCESS, be.last_error
            assert be.nodes_fused_away == (1 if fuse else 0)
            got = be.download(y_flat).reshape(L * L, D)
            if not fuse:                                        # the node ran: its own tensor holds relu(hidden)
                assert np.array_equal(be.download(relu).reshape(L * L, H), oracle.relu(hidden))
        finally:
            be.set_fuse_relu_into_q8(True)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), fuse
        results.append(got)
    assert np.array_equal(results[0], results[1])


def test_relu_is_not_folded_when_somebody_else_needs_it(be, oracle):
    D, H, L = 64, 96, 9
    rng = np.random.default_rng(77)
    x = rng.standard_normal((L * L, D)).astype(np.float32)
    w1 = (rng.standard_normal((H, D)) * 0.05).astype(np.float32)
    w2 = (rng.standard_normal((D, H)) * 0.05).astype(np.float32)
    w1t, w1q = _q8_leaf(be, oracle, w1, "Q8_0")
    w2t, w2q = _q8_leaf(be, oracle, w2, "Q8_0")
    hidden = oracle.mul_mat_q8(w1q, x)
    want = oracle.mul_mat_q8(w2q, oracle.relu(hidden))
    xl = _leaf(be, x, dims=(D, L, L, 1))
    # marked as an output of the graph (include/ppml/Tensor.h:21): it has to be written
    graph, relu, y_flat = _feed_forward_graph(be, xl, w1t, w2t, L, D, H)
    relu.set_flag(B.FLAG_OUTPUT)
    assert be.graph_compute(graph) == B.SUCCESS, be.last_error
    assert be.nodes_fused_away == 0
    assert np.array_equal(be.download(relu).reshape(L * L, H), oracle.relu(hidden))
    assert np.array_equal(be.download(y_flat).reshape(L * L, D), want)
    # a second reader of the ReLU (here a scale node)
    graph, relu, y_flat = _feed_forward_graph(be, xl, w1t, w2t, L, D, H)
    other = B.Tensor((H, L, L, 1), B.F32, B.OP_SCALE, [relu]).set_param(0, 2.0)
    assert be.graph_compute(graph + [other]) == B.SUCCESS, be.last_error
    assert be.nodes_fused_away == 0
    assert np.array_equal(be.download(other).reshape(L * L, H), oracle.relu(hidden) * np.float32(2))
    assert np.array_equal(be.download(y_flat).reshape(L * L, D), want)
    # a ReLU in front of an f32 matmul stays a node (there is no quantizer to fold it into)
    wf = _leaf(be, w2)
    h = _leaf(be, hidden)
    r = B.Tensor((H, L * L), B.F32, B.OP_UNARY, [h]).set_param(0, B.UNARY_OP_RELU)
    y = B.Tensor((D, L * L), B.F32, B.OP_MUL_MAT, [r, wf])
    assert be.graph_compute([r, y]) == B.SUCCESS, be.last_error
    assert be.nodes_fused_away == 0
    ref = oracle.mul_mat_f32(oracle.relu(hidden), w2)
    np.testing.assert_allclose(be.download(y).reshape(L * L, D), ref, rtol=0, atol=1e-4 * np.abs(ref).max())


def _logits_graph(k_leaf, q_leaf, L, H, planes, scale):
    scores = B.Tensor((L, L, H, planes), B.F32, B.OP_OUT_PROD, [k_leaf, q_leaf])
    scaled = B.Tensor((L, L, H, planes), B.F32, B.OP_SCALE, [scores]).set_param(0, float(scale))
    return scores, scaled


def test_attention_logits_graph_fused_and_node_by_node(be, oracle):
    """out_prod(K, Q) -> scale(1/sqrt(D)) as src/modules/Attention.cpp:264-270 builds it, at the pair-track shape
    (103 x 4 heads planes of 103 x 103 over D = 32): one scaled contraction, and two nodes -- the same bits."""
    L, D, H, Bt = 103, 32, 4, 103
    rng = np.random.default_rng(12)
    scale = float(np.float32(1.0) / np.sqrt(np.float32(D)))
    for exact in (True, False):
        if exact:       # small integers: every product and sum is exact, so one rounding (the scale) is all there is
            k = rng.integers(-4, 5, size=(Bt, H, D, L)).astype(np.float32)
            q = rng.integers(-4, 5, size=(Bt, H, D, L)).astype(np.float32)
        else:
            k = rng.standard_normal((Bt, H, D, L)).astype(np.float32)
            q = rng.standard_normal((Bt, H, D, L)).astype(np.float32)
        want = oracle.scale(oracle.out_prod(k, q), scale)
        kl, ql = _leaf(be, k), _leaf(be, q)
        outs = []
        for fuse in (True, False):
            be.set_fuse_scale_into_out_prod(fuse)
            try:
                scores, scaled = _logits_graph(kl, ql, L, H, Bt, scale)
                assert be.graph_compute([scores, scaled]) == B.SUCCESS, be.last_error
                assert be.nodes_fused_away == (1 if fuse else 0)
                outs.append(be.download(scaled).reshape(want.shape))
            finally:
                be.set_fuse_scale_into_out_prod(True)
        assert np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32))
        if exact:
            assert np.array_equal(outs[0].view(np.uint32), want.view(np.uint32))
        else:           # f32 GEMM bar: 1e-4 of the magnitude sum (k ascending on the CPU, matrix pipe here)
            bound = 1e-4 * scale * float(np.abs(k).max() * np.abs(q).max() * D)
            assert np.abs(outs[0] - want).max() <= bound
    # scores that something else reads, or that are an output, stay a node of their own
    scores, scaled = _logits_graph(kl, ql, L, H, Bt, scale)
    scores.set_flag(B.FLAG_OUTPUT)
    assert be.graph_compute([scores, scaled]) == B.SUCCESS and be.nodes_fused_away == 0
    assert np.array_equal(be.download(scaled).view(np.uint32), outs[0].reshape(-1).view(np.uint32))


def _attention_chain_graph(be, kl, ql, vl, bias_leaf, L, D, H, Bt, scale):
    """SelfAttention::forward_graph, default path (src/modules/Attention.cpp:264-281)."""
    scores = B.Tensor((L, L, H, Bt), B.F32, B.OP_OUT_PROD, [kl, ql])
    scaled = B.Tensor((L, L, H, Bt), B.F32, B.OP_SCALE, [scores]).set_param(0, float(scale))
    nodes = [scores, scaled]
    x = scaled
    if bias_leaf is not None:
        x = B.Tensor((L, L, H, Bt), B.F32, B.OP_ADD, [scaled, bias_leaf])
        nodes.append(x)
    attn = B.Tensor((L, L, H, Bt), B.F32, B.OP_SOFT_MAX, [x])
    attn_t = B.Tensor((L, L, H, Bt), B.F32, B.OP_PERMUTE, [attn])
    v_t = B.Tensor((D, L, H, Bt), B.F32, B.OP_PERMUTE, [vl])
    for p in (attn_t, v_t):
        for i, a in enumerate((1, 0, 2, 3)):
            p.set_param(i, a)
    out = B.Tensor((L, D, H, Bt), B.F32, B.OP_OUT_PROD, [attn_t, v_t])
    return nodes + [attn, attn_t, v_t, out], out


@pytest.mark.parametrize("with_bias", [True, False])
def test_default_attention_chain_stays_on_the_device(be, oracle, with_bias):
    """The chain the reference builds when PPML_FLASH_ATTN is off, node by node on this backend, against the oracle's
    restatement of the same nodes; then the same graph with the chain recognised and run as one fused launch."""
    L, D, H, Bt = 51, 32, 4, 6
    rng = np.random.default_rng(31 + with_bias)
    k, q, v = (rng.standard_normal((Bt, H, D, L)).astype(np.float32) for _ in range(3))       # graph layout [L, D, H, B]
    bias = rng.standard_normal((Bt, H, L, L)).astype(np.float32) if with_bias else None
    scale = float(np.float32(1.0) / np.sqrt(np.float32(D)))
    x = oracle.scale(oracle.out_prod(k, q), scale)
    if with_bias:
        x = oracle.bcast_elemwise(x, bias, "add")
    want = oracle.out_prod(oracle.permute(oracle.softmax(x), (1, 0, 2, 3)), oracle.permute(v, (1, 0, 2, 3)))
    kl, ql, vl = _leaf(be, k), _leaf(be, q), _leaf(be, v)
    bl = _leaf(be, bias) if with_bias else None
    graph, out = _attention_chain_graph(be, kl, ql, vl, bl, L, D, H, Bt, scale)
    assert all(be.supports_op(n) for n in graph)
    assert be.graph_compute(graph) == B.SUCCESS, be.last_error
    # the scale goes into the logits, the bias add into the softmax, the two permutations into the second contraction:
    # three launches (out_prod_scaled, softmax_add, out_prod_tt) for the seven (six) nodes
    assert be.nodes_fused_away == (4 if with_bias else 3)
    got = be.download(out).reshape(want.shape)
    np.testing.assert_allclose(got, want, rtol=0, atol=1e-4 * np.abs(want).max())
    # every node on its own: the same bits
    for setter in (be.set_fuse_scale_into_out_prod, be.set_fuse_add_into_soft_max, be.set_fuse_permutes_into_out_prod):
        setter(False)
    try:
        graph, out = _attention_chain_graph(be, kl, ql, vl, bl, L, D, H, Bt, scale)
        assert be.graph_compute(graph) == B.SUCCESS, be.last_error
        assert be.nodes_fused_away == 0
        plain = be.download(out).reshape(want.shape)
        probs = be.download(graph[-4]).reshape(Bt, H, L, L)              # the softmax node's own tensor
        np.testing.assert_allclose(probs, oracle.softmax(x), rtol=1e-5, atol=1e-37)
    finally:
        for setter in (be.set_fuse_scale_into_out_prod, be.set_fuse_add_into_soft_max, be.set_fuse_permutes_into_out_prod):
            setter(True)
    assert np.array_equal(plain.view(np.uint32), got.view(np.uint32))
    # one pass at a time
    for setter in (be.set_fuse_add_into_soft_max, be.set_fuse_permutes_into_out_prod):
        setter(False)
        try:
            graph, out = _attention_chain_graph(be, kl, ql, vl, bl, L, D, H, Bt, scale)
            assert be.graph_compute(graph) == B.SUCCESS, be.last_error
            assert np.array_equal(be.download(out).reshape(want.shape).view(np.uint32), got.view(np.uint32))
        finally:
            setter(True)
    # opt in: the whole chain as one launch
    be.set_fuse_attention_chain(True)
    try:
        graph, out = _attention_chain_graph(be, kl, ql, vl, bl, L, D, H, Bt, scale)
        assert be.graph_compute(graph) == B.SUCCESS, be.last_error
        assert be.nodes_fused_away == (6 if with_bias else 5)
        fused = be.download(out).reshape(want.shape)
    finally:
        be.set_fuse_attention_chain(False)
    np.testing.assert_allclose(fused, want, rtol=0, atol=1e-4 * np.abs(want).max())
    # and against the reference's fused routine itself (layouts [B][h][L][d])
    o, _ = oracle.flash_attn_forward(q.transpose(0, 1, 3, 2).copy(), k.transpose(0, 1, 3, 2).copy(), v.transpose(0, 1, 3, 2).copy(),
                                     bias, scale=scale)
    np.testing.assert_allclose(fused.transpose(0, 1, 3, 2), o, rtol=0, atol=2e-5 * np.abs(o).max())


def test_attention_chain_is_left_alone_when_an_intermediate_is_read_elsewhere(be, oracle):
    L, D, H, Bt = 20, 16, 2, 3
    rng = np.random.default_rng(5)
    k, q, v = (rng.standard_normal((Bt, H, D, L)).astype(np.float32) for _ in range(3))
    kl, ql, vl = _leaf(be, k), _leaf(be, q), _leaf(be, v)
    be.set_fuse_attention_chain(True)
    try:
        graph, out = _attention_chain_graph(be, kl, ql, vl, None, L, D, H, Bt, 0.25)
        attn = graph[2]
        attn.set_flag(B.FLAG_OUTPUT)                                  # the probabilities are wanted (e.g. for a backward pass)
        assert be.graph_compute(graph) == B.SUCCESS, be.last_error
        assert be.nodes_fused_away == 3                               # the scale into the logits, the permutations into the second contraction
        probs = oracle.softmax(oracle.scale(oracle.out_prod(k, q), 0.25))
        np.testing.assert_allclose(be.download(attn).reshape(probs.shape), probs, rtol=1e-4, atol=1e-7)
    finally:
        be.set_fuse_attention_chain(False)


def test_bias_add_and_permutations_stay_nodes_when_somebody_else_needs_them(be, oracle):
    L, D, H, Bt = 20, 16, 2, 3
    rng = np.random.default_rng(6)
    k, q, v = (rng.standard_normal((Bt, H, D, L)).astype(np.float32) for _ in range(3))
    bias = rng.standard_normal((Bt, H, L, L)).astype(np.float32)
    kl, ql, vl, bl = _leaf(be, k), _leaf(be, q), _leaf(be, v), _leaf(be, bias)
    x = oracle.bcast_elemwise(oracle.scale(oracle.out_prod(k, q), 0.25), bias, "add")
    want = oracle.out_prod(oracle.permute(oracle.softmax(x), (1, 0, 2, 3)), oracle.permute(v, (1, 0, 2, 3)))
    # the sum and the permuted probabilities flagged as outputs of the graph: both are written, nothing is folded
    # but the scale
    graph, out = _attention_chain_graph(be, kl, ql, vl, bl, L, D, H, Bt, 0.25)
    added, attn_t = graph[2], graph[4]                              # the OP_ADD node and permute(softmax)
    added.set_flag(B.FLAG_OUTPUT)
    attn_t.set_flag(B.FLAG_OUTPUT)
    assert be.graph_compute(graph) == B.SUCCESS, be.last_error
    assert be.nodes_fused_away == 1
    np.testing.assert_allclose(be.download(added).reshape(x.shape), x, rtol=0, atol=1e-4 * np.abs(x).max())      # (the logits are an f32 contraction)
    np.testing.assert_allclose(be.download(attn_t).reshape(Bt, H, L, L), oracle.softmax(x).transpose(0, 1, 3, 2), rtol=1e-5, atol=1e-37)
    np.testing.assert_allclose(be.download(out).reshape(want.shape), want, rtol=0, atol=1e-4 * np.abs(want).max())
    # a bias that is one plane for all (whole rows, a count that divides the softmax's): folded, same bits as the nodes
    small = rng.standard_normal((L, L)).astype(np.float32)
    sl = _leaf(be, small)
    outs = []
    for fold in (True, False):
        be.set_fuse_add_into_soft_max(fold)
        try:
            graph, out = _attention_chain_graph(be, kl, ql, vl, sl, L, D, H, Bt, 0.25)
            assert be.graph_compute(graph) == B.SUCCESS, be.last_error
            assert be.nodes_fused_away == (4 if fold else 3)
            outs.append(be.download(out))
        finally:
            be.set_fuse_add_into_soft_max(True)
    assert np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32))
    # an add whose FIRST operand is the short one is left alone (the folded form adds whole rows to a full-size input)
    scores = B.Tensor((L, L, H, Bt), B.F32, B.OP_OUT_PROD, [kl, ql])
    swapped = B.Tensor((L, L, H, Bt), B.F32, B.OP_ADD, [sl, scores])
    attn = B.Tensor((L, L, H, Bt), B.F32, B.OP_SOFT_MAX, [swapped])
    assert be.graph_compute([scores, swapped, attn]) == B.SUCCESS, be.last_error
    assert be.nodes_fused_away == 0
    ref = oracle.softmax(oracle.bcast_elemwise(small, oracle.out_prod(k, q), "add"))
    np.testing.assert_allclose(be.download(attn).reshape(ref.shape), ref, rtol=2e-5, atol=1e-30)
