"""Load-time side of the int8 path on the GPU: the selected weights are quantized on the device by the rule of
quantize_big_weight_matrices (src/model/PPML.cpp:4461-4551), travel through the checkpoint file as Q8_0 blocks,
and drive mul_mat_q8 with the same result as before the trip.  Bytes are compared exactly."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


def test_selected_weights_are_quantized_saved_loaded_and_used(oracle, tmp_path):
    from proteinpredictmachinelearning_amd import ops, weights as W

    assert torch.cuda.is_available(), "GPU tests need a device"
    g = torch.Generator(device="cuda").manual_seed(7)
    named = [
        ("blocks.0.attention.msa_row.qkv.weight", torch.randn(768, 256, device="cuda", generator=g) * 0.02),
        ("blocks.0.attention.msa_row.qkv.bias", torch.randn(768, device="cuda", generator=g)),
        ("blocks.0.transition.linear1.weight", torch.randn(512, 128, device="cuda", generator=g)),
        ("blocks.0.msa2pair_left_proj.weight", torch.randn(32, 250, device="cuda", generator=g)),     # K % 32 != 0
        ("blocks.0.msa2pair_out_proj.weight", torch.randn(128, 1024, device="cuda", generator=g) * 0.05),
    ]
    # training mode and an unset switch leave everything alone (PPML.cpp:4462-4471)
    same, rep = W.quantize_big_weight_matrices(named, "all", training=True)
    assert rep["done"] == 0 and all(a[1] is b[1] for a, b in zip(named, same))
    same, rep = W.quantize_big_weight_matrices(named, "off")
    assert rep["done"] == 0
    quant, rep = W.quantize_big_weight_matrices(named, "all")
    # the selected bias (1-D) and the projection with K = 250 fail the shape rule (PPML.cpp:4481-4488)
    assert rep == {"done": 2, "skipped_shape": 2, "bytes_before": (768 * 256 + 128 * 1024) * 4,
                   "bytes_after": (768 * 256 + 128 * 1024) // 32 * 34}
    kinds = [isinstance(t, W.QuantizedWeight) for _, t in quant]
    assert kinds == [True, False, False, False, True]          # the transition is not on the list
    again, rep2 = W.quantize_big_weight_matrices(quant, "all")
    assert rep2["done"] == 0 and rep2["skipped_shape"] == 2     # idempotent
    # the device quantizer's bytes are the host rule's (quantize_q8_0_host, include/ppml/QuantBlocks.h:62-79)
    for i in (0, 4):
        want = np.ascontiguousarray(oracle.quantize_q8_0(named[i][1].cpu().numpy())).view(np.uint8).reshape(-1)
        assert np.array_equal(quant[i][1].blocks.cpu().numpy().reshape(-1), want)
        assert quant[i][1].dims == tuple(reversed(named[i][1].shape))

    path = str(tmp_path / "int8.gguf")
    names = [n for n, _ in quant]
    W.save_gguf([t for _, t in quant], path, [("epoch", 1.0)], [("ppml.arch", "ppml_v1")], names)
    shapes = [t.dims if isinstance(t, W.QuantizedWeight) else tuple(reversed(t.shape)) for _, t in quant]
    loaded, raw = W.load_gguf(path, shapes, names)
    assert raw == {}
    x = torch.randn(408, 256, device="cuda", generator=g)
    x2 = torch.randn(200, 1024, device="cuda", generator=g)
    for i, xin in ((0, x), (4, x2)):
        lw = loaded[i]
        assert isinstance(lw, W.QuantizedWeight)
        assert np.array_equal(lw.blocks, quant[i][1].blocks.cpu().numpy().reshape(-1))
        K, M = lw.dims
        from_file = ops.Q8Weight(torch.from_numpy(lw.blocks).cuda(), M, K, ops.WTYPE_Q8_0)
        in_memory = ops.Q8Weight(quant[i][1].blocks.reshape(-1), M, K, ops.WTYPE_Q8_0)
        y_file = ops.mul_mat_q8(from_file.pack(), xin)
        y_mem = ops.mul_mat_q8(in_memory, xin)
        assert torch.equal(y_file, y_mem)
        want = oracle.mul_mat_q8(oracle.quantize_q8_0(named[i][1].cpu().numpy()), xin.cpu().numpy(), wtype=0, c_trans=1, fma=1)
        assert np.array_equal(y_file.cpu().numpy(), want)
    for i in (1, 2, 3):
        assert np.array_equal(loaded[i], named[i][1].cpu().numpy())
