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


# ----------------------------------------------------------------------------- fused attention forward
FLASH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "flash_attn_forward.json")


def flash_cases():
    """Inputs and outputs of the reference's own flash_attn_forward_cpu (written by make_flash_attn_vectors.py)."""
    with open(FLASH) as f:
        data = json.load(f)
    for c in data["cases"]:
        shape = (c["B"], c["h"], c["L"], c["d"])
        f32 = lambda bits, shp: np.array(bits, dtype=np.uint32).view(np.float32).reshape(shp)  # noqa: E731
        yield {"cfg": c, "q": f32(c["q"], shape), "k": f32(c["k"], shape), "v": f32(c["v"], shape),
               "bias": f32(c["bias"], (c["B"], c["h"], c["L"], c["L"])) if c["bias"] is not None else None,
               "o": f32(c["o"], shape), "lse": f32(c["lse"], shape[:3])}


def test_flash_attn_forward_matches_the_reference_vectors_bit_for_bit(oracle):
    n = 0
    for c in flash_cases():
        cfg = c["cfg"]
        o, lse = oracle.flash_attn_forward(c["q"], c["k"], c["v"], c["bias"], causal=cfg["causal"], scale=cfg["scale"],
                                           eps=cfg["eps"], Bc=cfg["Bc"])
        assert (o.view(np.uint32) == c["o"].view(np.uint32)).all(), cfg["L"]
        assert (lse.view(np.uint32) == c["lse"].view(np.uint32)).all(), cfg["L"]
        n += 1
    assert n == 4
    # the vectors do contain the special row: fully masked -> O = 0, LSE = -inf
    first = next(flash_cases())
    assert np.isneginf(first["lse"][0, 0, 1]) and (first["o"][0, 0, 1] == 0).all()


def test_flash_attn_backward_matches_the_reference_vectors_bit_for_bit(oracle):
    with open(FLASH) as f:
        cases = json.load(f)["backward_cases"]
    assert len(cases) == 2
    for c in cases:
        shape = (c["B"], c["h"], c["L"], c["d"])
        f32 = lambda bits, shp: np.array(bits, dtype=np.uint32).view(np.float32).reshape(shp)  # noqa: E731
        sq = (c["B"], c["h"], c["L"], c["L"])
        bias = f32(c["bias"], sq) if c["bias"] is not None else None
        got = oracle.flash_attn_backward(f32(c["q"], shape), f32(c["k"], shape), f32(c["v"], shape), bias, f32(c["o"], shape),
                                         f32(c["do"], shape), f32(c["lse"], shape[:3]), causal=c["causal"])
        for g, key, shp in zip(got, ("dq", "dk", "dv", "dbias"), (shape, shape, shape, sq)):
            assert (g.view(np.uint32) == f32(c[key], shp).view(np.uint32)).all(), key
