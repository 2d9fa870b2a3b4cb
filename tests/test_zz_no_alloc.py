"""The entry point that allocates nothing, mul_mat_tn_noalloc_hip, against mul_mat_tn_hip through the C ABI.

Both run the same kernels on the same operands (the workspace is a static device array instead of a pool
allocation), so the bar here is equality of every output bit, which is inside the f32 bar of 1e-4 relative.
Collected last on purpose: it must pass in a fresh process and after every other test.
"""
import ctypes as C

import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


def _call(fn, a, b, out, M, K, N, alpha):
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    return fn(C.c_void_p(a.data_ptr()), C.c_void_p(b.data_ptr()), C.c_void_p(out.data_ptr()), M, K, N, alpha, stream)


def test_no_alloc_entry_point_matches_the_allocating_one_on_calls_in_a_row():
    from proteinpredictmachinelearning_amd import cabi, ops

    lib = ops._lib()                                    # loads the library and runs ppml_hip_init on the device
    g = torch.Generator(device="cuda").manual_seed(77)
    # (M, K, N): a large one whose planes take 36 of the 64 MiB; a smaller one that still splits ahead; one that
    # is cut into K slices (planes + partial sums, 61.5 MiB); one small enough to need no workspace at all
    shapes = [(12288, 256, 12288), (4100, 77, 3900), (1024, 2048, 1030), (300, 64, 200)]
    cases = []
    for M, K, N in shapes:
        a = torch.randn(K, M, device="cuda", generator=g) * 0.1
        b = torch.randn(K, N, device="cuda", generator=g) * 0.1
        cases.append((M, K, N, a, b, torch.empty(M, N, device="cuda"), torch.full((M, N), float("nan"), device="cuda")))
    # reference results first (this grows the allocating entry point's pool, which is not ours to watch)
    for M, K, N, a, b, want, _ in cases:
        assert _call(lib.mul_mat_tn_hip, a, b, want, M, K, N, 1.0 / K) == 0, cabi.last_error()
    torch.cuda.synchronize()
    free_before, _total = torch.cuda.mem_get_info()
    # two passes over the cases, back to back on one stream: every call after the first finds the previous
    # call's planes and partial sums in the workspace, larger ones after smaller ones and the other way round
    for _ in range(2):
        for M, K, N, a, b, _, got in cases:
            assert _call(lib.mul_mat_tn_noalloc_hip, a, b, got, M, K, N, 1.0 / K) == 0, cabi.last_error()
        for M, K, N, a, b, _, got in reversed(cases):
            assert _call(lib.mul_mat_tn_noalloc_hip, a, b, got, M, K, N, 1.0 / K) == 0, cabi.last_error()
    torch.cuda.synchronize()
    free_after, _total = torch.cuda.mem_get_info()
    # (free memory may grow meanwhile -- the runtime hands back what earlier tests of this process let go of --, but a
    # call that allocates would shrink it)
    assert free_after >= free_before, "device memory was taken during calls that must not allocate"
    for M, K, N, a, b, want, got in cases:
        assert torch.equal(got, want), (M, K, N)
        # and the result is the contraction: a sample against float64
        ref = (a[:, :64].double().t() @ b[:, :48].double()) / K
        assert ((got[:64, :48].double() - ref).abs() <= 1e-4 * (a[:, :64].double().abs().t() @ b[:, :48].double().abs()) / K).all()


def test_no_alloc_entry_point_refuses_what_does_not_fit():
    from proteinpredictmachinelearning_amd import cabi, ops

    lib = ops._lib()
    one = torch.zeros(16, device="cuda")
    # 4096^3 wants 192 MiB of planes (and 1 KiB of guard flags): refused before anything is launched (the operands
    # are never read)
    assert _call(lib.mul_mat_tn_noalloc_hip, one, one, one, 4096, 4096, 4096, 1.0) == 1
    msg = cabi.last_error()
    assert str(201326592 + 1024) in msg and "67108864" in msg, msg
    assert _call(lib.mul_mat_tn_noalloc_hip, one, one, one, 0, 4, 4, 1.0) == 1
    null = C.c_void_p(0)
    assert lib.mul_mat_tn_noalloc_hip(null, null, null, 4, 4, 4, 1.0, None) == 1


def test_no_alloc_entry_point_inside_a_captured_graph():
    """What the entry point is for: two calls recorded into a HIP graph, replayed several times with eager work and
    synchronisations of the program's own in between, every replay checked against the allocating entry point."""
    from proteinpredictmachinelearning_amd import cabi, ops

    lib = ops._lib()
    g = torch.Generator(device="cuda").manual_seed(5)
    shapes = [(4100, 77, 3900), (1024, 2048, 1030)]          # planes split ahead; K slices with partial sums
    ops_in = [(M, K, N, torch.randn(K, M, device="cuda", generator=g), torch.randn(K, N, device="cuda", generator=g),
               torch.full((M, N), float("nan"), device="cuda")) for M, K, N in shapes]
    # one eager call first: nothing is looked up or created for the first time while the stream is being captured
    for M, K, N, a, b, out in ops_in:
        assert _call(lib.mul_mat_tn_noalloc_hip, a, b, out, M, K, N, 0.5) == 0, cabi.last_error()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for M, K, N, a, b, out in ops_in:
            assert _call(lib.mul_mat_tn_noalloc_hip, a, b, out, M, K, N, 0.5) == 0, cabi.last_error()
    for replay in range(4):
        for M, K, N, a, b, out in ops_in:                   # new operands for every replay, written the eager way
            a.normal_(generator=g)
            b.normal_(generator=g)
            out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for M, K, N, a, b, out in ops_in:
            want = torch.empty_like(out)
            assert _call(lib.mul_mat_tn_hip, a, b, want, M, K, N, 0.5) == 0, cabi.last_error()
            torch.cuda.synchronize()
            assert torch.equal(out, want), (replay, M, K, N)
