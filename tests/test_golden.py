"""The CPU oracle against the known answers the reference's own tests hold (tests/golden)."""
import json
import os

import numpy as np

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_known_answers.json")


def _load():
    with open(GOLDEN) as f:
        return json.load(f)


def _pattern(expr, n):
    i = np.arange(n)
    return eval(expr, {"__builtins__": {}}, {"i": i}).astype(np.float32)      # arithmetic on `i` only


def test_outer_product_mean_value_known_answers(oracle):
    for case in _load()["outer_product_mean_value"]:
        shape = case["shape_BNLD"]
        left = np.array(case["left"], np.float32).reshape(shape)
        right = np.array(case["right"], np.float32).reshape(shape)
        out = oracle.outer_product_mean_value(left, right)
        assert list(out.shape) == case["out_shape"]
        flat = out.reshape(-1)
        for idx, want in case["expected_at"].items():
            assert flat[int(idx)] == np.float32(want), (case["source"], idx)


def test_mul_mat_reference_inputs_are_integer_exact(oracle):
    g = _load()["mul_mat_f32"]
    M, K, N = g["M"], g["K"], g["N"]
    A = _pattern(g["A_pattern"], M * K).reshape(M, K)
    B = _pattern(g["B_pattern"], N * K).reshape(N, K)
    got = oracle.mul_mat_f32(A, B)
    want = ((A * 8).astype(np.int64) @ (B * 8).astype(np.int64).T) / 64.0     # multiples of 1/8: integers
    assert (got.astype(np.float64) == want).all()


def test_out_prod_reference_inputs_are_integer_exact(oracle):
    small, real = _load()["out_prod"]
    a = _pattern(small["a_pattern"], small["C0"] * small["K"]).reshape(1, 1, small["K"], small["C0"])
    b = _pattern(small["b_pattern"], small["C1"] * small["K"]).reshape(1, 1, small["K"], small["C1"])
    want = np.einsum("pqki,pqkj->pqji", (a * 4).astype(np.int64), (b * 4).astype(np.int64)) / 16.0
    assert (oracle.out_prod(a, b).astype(np.float64) == want).all()
    n = real["L"] * real["K"] * real["planes2"] * real["planes3"]
    shape = (real["planes3"], real["planes2"], real["K"], real["L"])
    a = _pattern(real["a_pattern"], n).reshape(shape)
    b = _pattern(real["b_pattern"], n).reshape(shape)
    want = np.einsum("pqki,pqkj->pqji", (a * 16).astype(np.int64), (b * 8).astype(np.int64)) / 128.0
    assert (oracle.out_prod(a, b).astype(np.float64) == want).all()


def test_quantizer_hand_vector(oracle):
    g = _load()["quantize_q8_0_hand_vector"]
    x = _pattern("0.01 * (i - 15.5)", 32)
    blk = oracle.quantize_q8_0(x)
    assert int(oracle.block_scales_bits(blk).reshape(-1)[0]) == int(g["d_bits"], 16)
    q = oracle.block_quants(blk).reshape(-1)
    assert q[0] == g["q0"] and q[31] == g["q31"]
