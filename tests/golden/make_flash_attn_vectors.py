#!/usr/bin/env python3
"""Writes tests/golden/flash_attn_forward.json from the reference's own fused attention forward.

The reference routine (src/ops/FlashAttn.cpp) is compiled as-is into oracle/_ref/libppml_ref_flash.so by
`make -C oracle` wherever the reference tree is mounted; this script calls that library on small seeded
inputs and stores inputs and outputs, so that the oracle stays pinned where the reference is absent.
Floats are stored as binary32 bit patterns (exact).  Run from the repository root:

    python3 tests/golden/make_flash_attn_vectors.py
"""
import json
import os
import sys

import numpy as np

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", ".."))
import oracle  # noqa: E402

CASES = [
    # B, h, L, d, causal, Bc, bias, scale, eps, seed
    (1, 2, 7, 4, False, 64, True, 0.0, 1e-9, 11),
    (2, 1, 19, 8, True, 4, True, 0.25, 1e-9, 12),
    (1, 1, 33, 12, False, 16, False, 0.0, 0.0, 13),
    (1, 3, 5, 4, True, 64, False, 0.0, 1e-9, 14),
]


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).reshape(-1).tolist()


def main():
    if oracle.ref_flash_lib() is None:
        sys.exit("oracle/_ref/libppml_ref_flash.so is missing: run `make -C oracle` with the reference mounted")
    out = []
    for B, h, L, d, causal, Bc, use_bias, scale, eps, seed in CASES:
        rng = np.random.default_rng(seed)
        q, k, v = [rng.standard_normal((B, h, L, d)).astype(np.float32) for _ in range(3)]
        bias = (2.0 * rng.standard_normal((B, h, L, L))).astype(np.float32) if use_bias else None
        if bias is not None and not causal:
            bias[0, 0, 1, :] = -np.inf          # one fully masked row: O = 0, LSE = -inf
        o, lse = oracle.ref_flash_attn_forward(q, k, v, bias, causal=causal, scale=scale, eps=eps, Bc=Bc)
        out.append({"B": B, "h": h, "L": L, "d": d, "causal": causal, "Bc": Bc, "scale": scale, "eps": eps,
                    "q": bits(q), "k": bits(k), "v": bits(v), "bias": bits(bias) if bias is not None else None,
                    "o": bits(o), "lse": bits(lse)})
    back = []
    for B, h, L, d, causal, use_bias, seed in [(1, 2, 9, 4, False, True, 21), (1, 1, 17, 8, True, True, 22)]:
        rng = np.random.default_rng(seed)
        q, k, v, do = [rng.standard_normal((B, h, L, d)).astype(np.float32) for _ in range(4)]
        bias = rng.standard_normal((B, h, L, L)).astype(np.float32) if use_bias else None
        if bias is not None and not causal:
            bias[0, 1, 2, :] = -np.inf
        o, lse = oracle.ref_flash_attn_forward(q, k, v, bias, causal=causal)
        dq, dk, dv, db = oracle.ref_flash_attn_backward(q, k, v, bias, o, do, lse, causal=causal)
        back.append({"B": B, "h": h, "L": L, "d": d, "causal": causal, "q": bits(q), "k": bits(k), "v": bits(v),
                     "bias": bits(bias) if bias is not None else None, "o": bits(o), "lse": bits(lse), "do": bits(do),
                     "dq": bits(dq), "dk": bits(dk), "dv": bits(dv), "dbias": bits(db)})
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "flash_attn_forward.json")
    with open(path, "w") as f:
        json.dump({"source": "flash_attn_forward_cpu, src/ops/FlashAttn.cpp:55-135, compiled from the reference tree",
                   "encoding": "binary32 bit patterns, C order", "cases": out,
                   "backward_source": "flash_attn_backward_cpu, src/ops/FlashAttn.cpp:140-210, same build",
                   "backward_cases": back}, f)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
