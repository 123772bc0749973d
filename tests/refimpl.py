"""Oracle-side reference for a workload: the reference's CPU sequence
(norm -> rope -> scalar attention) on the same seeded draws, for all rows or
for a sample of query tokens. Test infrastructure only."""
from __future__ import annotations

import numpy as np

from oracle import zoracle as zo
from zdraw_amd import workloads as wl

# Stated tolerance of the bf16 path against the fp32 reference.
MAX_ABS = 2e-2
MEAN_ABS = 2e-3


def prepared_qk(w: wl.Workload, b: int, q=None, k=None):
    """Q and K of segment b after the model's norm + rope, via the oracle."""
    q = w.q[b] if q is None else q
    k = w.k[b] if k is None else k
    ones = np.ones(wl.HEAD_DIM, np.float32)
    if w.kind == "plain":
        return q, k
    if w.kind == "klein":
        cos, sin = zo.klein_build_rope_ref(w.grid[0], w.grid[1], w.ref_grid[0], w.ref_grid[1],
                                           theta=w.theta, txt_len=w.txt_len)
        qn = zo.klein_apply_rope(zo.klein_rms_norm_heads(q, ones), cos, sin)
        kn = zo.klein_apply_rope(zo.klein_rms_norm_heads(k, ones), cos, sin)
        return qn, kn
    cfg = zo.RopeConfig(wl.ZIMAGE_DIMS, wl.ZIMAGE_LENS, wl.ZIMAGE_THETA)
    vals = zo.zrope_fill(cfg)
    # positions rebuilt with the oracle's own helpers (zstep_shape.zig:58-66)
    gh, gw = w.grid
    cap_total = zo.zseq_padded_len(w.extra["cap_tokens"])
    img_total = zo.zseq_padded_len(gh * gw)
    pos = np.zeros((img_total + cap_total, 3), np.uintp)
    pos[:gh * gw] = zo.zseq_grid((1, gh, gw), (cap_total + 1, 0, 0))
    pos[img_total:] = zo.zseq_grid((cap_total, 1, 1), (1, 0, 0))
    qn = zo.zimage_rotate(zo.zimage_norm_heads(q, ones, wl.ZIMAGE_EPS), vals, cfg, pos)
    kn = zo.zimage_rotate(zo.zimage_norm_heads(k, ones, wl.ZIMAGE_EPS), vals, cfg, pos)
    return qn, kn


def reference_rows(w: wl.Workload, tokens=None, threads=8):
    """fp32 reference output [B][len(tokens)][H][128] for the listed query
    tokens (all tokens when None)."""
    toks = list(range(w.tokens)) if tokens is None else [int(t) for t in tokens]
    cfg = zo.Config(w.tokens, w.heads, w.heads, wl.HEAD_DIM)
    outs = []
    for b in range(w.batch):
        qn, kn = prepared_qk(w, b)
        pad = w.key_pad[b] if w.key_pad is not None else None
        outs.append(zo.attention_token_list(qn, kn, w.v[b], cfg, toks, key_pad=pad, threads=threads))
    return np.stack(outs)


def sample_tokens(w: wl.Workload, n: int, seed=1):
    """Query tokens that cover the first/last rows, the text/image boundary
    and workgroup-block edges, plus random ones."""
    rng = np.random.default_rng(seed)
    fixed = {0, 1, 31, 32, 63, 64, 127, 128, 255, 256, w.tokens - 1, w.tokens - 2, w.tokens // 2}
    if w.txt_len:
        fixed |= {w.txt_len - 1, w.txt_len, w.txt_len + 1}
    if w.text_lens:
        for n_txt in w.text_lens:
            fixed |= {n_txt - 1, n_txt}
    fixed = sorted(t for t in fixed if 0 <= t < w.tokens)
    rest = rng.choice(w.tokens, size=max(0, n - len(fixed)), replace=False).tolist()
    return sorted(set(fixed) | set(rest))


def check_close(got, want, what=""):
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    mx, mean = float(err.max()), float(err.mean())
    assert np.isfinite(got).all(), f"{what}: non-finite output"
    assert mx <= MAX_ABS and mean <= MEAN_ABS, f"{what}: max abs {mx:.3e} (<= {MAX_ABS}), mean abs {mean:.3e} (<= {MEAN_ABS})"
    return mx, mean
