"""Writes tests/golden/sdpa_fp64.npz: inputs and outputs (computed in fp64) of torch's CPU
scaled_dot_product_attention (a library routine, not the reference) on small
shapes, so that the oracle's attention can be checked without torch at hand.

Run from the repository root:  python tests/golden/make_sdpa_fixtures.py
"""
import os

import numpy as np
import torch

# tokens, heads, kv_heads, head_dim, causal
CASES = [(1, 1, 1, 128, False), (7, 2, 2, 128, False), (33, 4, 2, 32, False), (31, 2, 1, 16, False),
         (20, 3, 3, 128, True), (16, 1, 1, 512, False), (40, 2, 2, 128, False)]


def main():
    out = {}
    for i, (tokens, heads, kv, dim, causal) in enumerate(CASES):
        rng = np.random.default_rng(1000 + i)
        q = rng.standard_normal((tokens, heads, dim), dtype=np.float32)
        k = rng.standard_normal((tokens, kv, dim), dtype=np.float32)
        v = rng.standard_normal((tokens, kv, dim), dtype=np.float32)
        rep = heads // kv
        tq = torch.from_numpy(q).double().permute(1, 0, 2)[None]
        tk = torch.from_numpy(k).double().permute(1, 0, 2).repeat_interleave(rep, 0)[None]
        tv = torch.from_numpy(v).double().permute(1, 0, 2).repeat_interleave(rep, 0)[None]
        o = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, is_causal=causal)
        out[f"shape{i}"] = np.array([tokens, heads, kv, dim, int(causal)], np.int64)
        out[f"q{i}"], out[f"k{i}"], out[f"v{i}"] = q, k, v
        out[f"o{i}"] = o[0].permute(1, 0, 2).numpy().astype(np.float32)  # fp64 result, stored rounded once
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "sdpa_fp64.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
