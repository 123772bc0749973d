"""Pins the oracle's scalar attention (oracle/attention_ref.c).

Sources of truth used here, none of which retype the oracle's formula:
  * the reference's own known-answer tests (runtime/attention.zig:115-156,
    metal/mattn_test.zig:15-31), restated with the same inputs and tolerances;
  * an fp64 brute force written with numpy matrix ops (different algorithm
    shape: whole-matrix softmax, not the per-row three-pass loop);
  * torch's CPU scaled_dot_product_attention in fp64 (a library routine);
  * invariants a dropped term / wrong index / transposed operand would break.
"""
import numpy as np
import pytest

from oracle import zoracle as zo


def cfg(tokens, heads, kv_heads, head_dim, causal=False, valid=0):
    return zo.Config(tokens, heads, kv_heads, head_dim, causal, valid)


def brute_force(q, k, v, c: zo.Config, key_pad=None):
    """fp64 whole-matrix attention, independent of the oracle's loop form."""
    q = np.asarray(q, np.float64).reshape(c.tokens, c.heads, c.head_dim)
    k = np.asarray(k, np.float64).reshape(c.tokens, c.kv_heads, c.head_dim)
    v = np.asarray(v, np.float64).reshape(c.tokens, c.kv_heads, c.head_dim)
    out = np.zeros_like(q)
    allowed = np.ones((c.tokens, c.tokens), bool)
    if c.causal:
        allowed &= np.tril(np.ones((c.tokens, c.tokens), bool))
    if c.valid:
        allowed[:, c.valid:] = False
    if key_pad is not None:
        allowed[:, np.asarray(key_pad, bool)] = False
    for h in range(c.heads):
        g = h * c.kv_heads // c.heads
        s = q[:, h, :] @ k[:, g, :].T / np.sqrt(np.float64(c.head_dim))
        s = np.where(allowed, s, -np.inf)
        s = s - s.max(axis=1, keepdims=True)
        p = np.exp(s)
        p /= p.sum(axis=1, keepdims=True)
        out[:, h, :] = p @ v[:, g, :]
    return out


# --- reference known-answer tests -----------------------------------------
def test_single_token_returns_value():
    # runtime/attention.zig:115-123
    out = zo.attention_run([1.0, 0.0], [1.0, 0.0], [3.0, 4.0], cfg(1, 1, 1, 2, causal=True))
    assert abs(out.ravel()[0] - 3.0) < 1e-4 and abs(out.ravel()[1] - 4.0) < 1e-4


def test_causal_ignores_future_tokens():
    # runtime/attention.zig:125-133
    out = zo.attention_run([1.0, 1.0], [1.0, 1.0], [2.0, 6.0], cfg(2, 1, 1, 1, causal=True))
    assert abs(out.ravel()[0] - 2.0) < 1e-4 and abs(out.ravel()[1] - 4.0) < 1e-4


def test_padding_limit_masks_trailing_keys():
    # runtime/attention.zig:135-156
    q, k, v = [1, 1, 1], [0, 0, 100], [1, 2, 99]
    base = cfg(3, 1, 1, 1, causal=True)
    open_out = zo.attention_run(q, k, v, base).ravel()
    masked = zo.attention_run(q, k, v, cfg(3, 1, 1, 1, causal=True, valid=2)).ravel()
    assert open_out[0] == masked[0] and open_out[1] == masked[1]
    assert abs(open_out[2] - 99.0) < 1e-3
    assert abs(masked[2] - 1.5) < 1e-5


def test_two_token_identity_case():
    # metal/mattn_test.zig:15-31 (inputs); expected values from the closed form
    # softmax([a, 0]) with a = 1/sqrt(2): row0 = w*(2,4) + (1-w)*(6,8).
    q = [1.0, 0.0, 0.0, 1.0]
    out = zo.attention_run(q, q, [2.0, 4.0, 6.0, 8.0], cfg(2, 1, 1, 2)).reshape(2, 2)
    w = 1.0 / (1.0 + np.exp(-1.0 / np.sqrt(2.0)))
    want = np.array([[2 * w + 6 * (1 - w), 4 * w + 8 * (1 - w)],
                     [6 * w + 2 * (1 - w), 8 * w + 4 * (1 - w)]])
    assert np.allclose(out, want, atol=1e-4)


# --- shape errors (runtime/attention.zig:45-60) ------------------------------
@pytest.mark.parametrize("bad", [
    dict(tokens=0), dict(heads=0), dict(kv_heads=0), dict(head_dim=0), dict(heads=3, kv_heads=2),
])
def test_invalid_shape_config(bad):
    base = dict(tokens=2, heads=2, kv_heads=2, head_dim=4)
    base.update(bad)
    c = cfg(**base)
    n = max(1, c.tokens * c.heads * c.head_dim)
    z = np.zeros(n, np.float32)
    with pytest.raises(zo.OracleError) as e:
        zo.attention_run(z, z, z, c)
    assert e.value.code == zo.INVALID_SHAPE


def test_invalid_slice_lengths():
    c = cfg(2, 2, 2, 4)
    n = 16
    z = np.zeros(n, np.float32)
    with pytest.raises(zo.OracleError):
        zo.attention_run(z[:-1], z, z, c)
    with pytest.raises(zo.OracleError):
        zo.attention_run(z, z[:-1], z, c)
    with pytest.raises(zo.OracleError):
        zo.attention_run(z, z, z, c, scratch_len=1)
    with pytest.raises(zo.OracleError):
        zo.attention_run(z, z, z, c, out_len=n + 1)


# --- brute force and library cross-checks -----------------------------------
# Shapes follow metal/mattn_test.zig:35-54 (flash_cases and block_cases).
SHAPES = [
    (1, 2, 2, 8, False), (31, 2, 1, 16, False), (32, 1, 1, 128, False),
    (97, 3, 3, 64, True), (257, 2, 2, 128, False), (16, 1, 1, 256, False),
    (16, 1, 1, 128, False), (48, 2, 2, 128, False), (53, 3, 3, 128, False),
    (288, 4, 4, 128, False), (289, 2, 2, 128, False), (40, 4, 2, 32, True),
]


@pytest.mark.parametrize("tokens,heads,kv,dim,causal", SHAPES)
def test_matches_fp64_brute_force(tokens, heads, kv, dim, causal):
    rng = np.random.default_rng(tokens * 31 + heads)
    q = rng.standard_normal((tokens, heads, dim), dtype=np.float32)
    k = rng.standard_normal((tokens, kv, dim), dtype=np.float32)
    v = rng.standard_normal((tokens, kv, dim), dtype=np.float32)
    c = cfg(tokens, heads, kv, dim, causal)
    got = zo.attention_run(q, k, v, c)
    want = brute_force(q, k, v, c)
    assert np.abs(got - want).max() < 2e-5


@pytest.mark.parametrize("tokens,heads,kv,dim,causal", SHAPES[:8])
def test_matches_torch_sdpa_fp64(tokens, heads, kv, dim, causal):
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(7 + tokens)
    q = rng.standard_normal((tokens, heads, dim), dtype=np.float32)
    k = rng.standard_normal((tokens, kv, dim), dtype=np.float32)
    v = rng.standard_normal((tokens, kv, dim), dtype=np.float32)
    got = zo.attention_run(q, k, v, cfg(tokens, heads, kv, dim, causal))
    rep = heads // kv
    tq = torch.from_numpy(q).double().permute(1, 0, 2)[None]
    tk = torch.from_numpy(k).double().permute(1, 0, 2).repeat_interleave(rep, 0)[None]
    tv = torch.from_numpy(v).double().permute(1, 0, 2).repeat_interleave(rep, 0)[None]
    want = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, is_causal=causal)
    want = want[0].permute(1, 0, 2).numpy()
    assert np.abs(got - want).max() < 2e-5


def test_matches_committed_sdpa_fixtures():
    # tests/golden/sdpa_fp64.npz (written by tests/golden/make_sdpa_fixtures.py): the same
    # library cross-check as above on fixed inputs, without torch at hand
    import os
    z = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "sdpa_fp64.npz"))
    n = sum(1 for name in z.files if name.startswith("shape"))
    assert n >= 7
    for i in range(n):
        tokens, heads, kv, dim, causal = (int(x) for x in z[f"shape{i}"])
        got = zo.attention_run(z[f"q{i}"], z[f"k{i}"], z[f"v{i}"], cfg(tokens, heads, kv, dim, bool(causal)))
        assert np.abs(got - z[f"o{i}"]).max() < 2e-5, (i, tokens, heads, kv, dim, causal)


def test_valid_limit_matches_brute_force():
    rng = np.random.default_rng(3)
    c = cfg(50, 2, 2, 16, valid=37)
    q, k, v = (rng.standard_normal((50, 2, 16), dtype=np.float32) for _ in range(3))
    assert np.abs(zo.attention_run(q, k, v, c) - brute_force(q, k, v, c)).max() < 2e-5


# --- invariants ----------------------------------------------------------------
def test_uniform_logits_give_mean_of_v():
    rng = np.random.default_rng(0)
    tokens, dim = 33, 16
    q = np.zeros((tokens, 1, dim), np.float32)
    k = rng.standard_normal((tokens, 1, dim), dtype=np.float32)
    v = rng.standard_normal((tokens, 1, dim), dtype=np.float32)
    out = zo.attention_run(q, k, v, cfg(tokens, 1, 1, dim))
    assert np.allclose(out[:, 0, :], v[:, 0, :].mean(axis=0), atol=1e-5)


def test_dominant_key_selects_its_value():
    tokens, dim = 9, 4
    q = np.zeros((tokens, 1, dim), np.float32)
    q[:, 0, 0] = 1.0
    k = np.zeros((tokens, 1, dim), np.float32)
    k[5, 0, 0] = 1000.0
    v = np.arange(tokens * dim, dtype=np.float32).reshape(tokens, 1, dim)
    out = zo.attention_run(q, k, v, cfg(tokens, 1, 1, dim))
    assert np.allclose(out[:, 0, :], v[5, 0, :], atol=1e-4)


def test_key_permutation_invariance():
    rng = np.random.default_rng(1)
    tokens, heads, dim = 40, 2, 32
    q, k, v = (rng.standard_normal((tokens, heads, dim), dtype=np.float32) for _ in range(3))
    perm = rng.permutation(tokens)
    c = cfg(tokens, heads, heads, dim)
    a = zo.attention_run(q, k, v, c)
    b = zo.attention_run(q, k[perm], v[perm], c)
    assert np.abs(a - b).max() < 1e-5  # only fp32 summation order differs


def test_q_and_k_are_not_interchangeable():
    # a transposed-operand mistake (scores = k.q^T read by rows) fails this
    rng = np.random.default_rng(2)
    tokens, dim = 12, 8
    q, k, v = (rng.standard_normal((tokens, 1, dim), dtype=np.float32) for _ in range(3))
    c = cfg(tokens, 1, 1, dim)
    assert np.abs(zo.attention_run(q, k, v, c) - zo.attention_run(k, q, v, c)).max() > 1e-2
    assert np.abs(zo.attention_run(q, k, v, c) - brute_force(q, k, v, c)).max() < 2e-5


def test_scale_is_inverse_sqrt_head_dim():
    # two keys, logits differ by exactly ln(3)*sqrt(D) before scaling -> p = (3/4, 1/4)
    dim = 16
    q = np.zeros((2, 1, dim), np.float32)
    q[:, 0, 0] = 1.0
    k = np.zeros((2, 1, dim), np.float32)
    k[0, 0, 0] = np.log(3.0) * np.sqrt(dim)
    v = np.array([[[1.0] + [0.0] * (dim - 1)], [[0.0] * dim]], np.float32)
    out = zo.attention_run(q, k, v, cfg(2, 1, 1, dim))
    assert abs(out[0, 0, 0] - 0.75) < 1e-5


def test_rows_are_independent_and_bit_equal():
    rng = np.random.default_rng(5)
    tokens, heads, dim = 64, 3, 16
    q, k, v = (rng.standard_normal((tokens, heads, dim), dtype=np.float32) for _ in range(3))
    c = cfg(tokens, heads, heads, dim)
    full = zo.attention_run(q, k, v, c)
    part = zo.attention_rows(q, k, v, c, 10, 20)
    assert np.array_equal(part[10:20], full[10:20])
    assert not part[:10].any() and not part[20:].any()
    listed = zo.attention_token_list(q, k, v, c, [3, 63, 17], threads=3)
    assert np.array_equal(listed, full[[3, 63, 17]])


# --- the key-padding mask extension ----------------------------------------------
def test_mask_equals_deleting_keys_bitwise():
    rng = np.random.default_rng(11)
    tokens, heads, dim = 70, 2, 32
    q, k, v = (rng.standard_normal((tokens, heads, dim), dtype=np.float32) for _ in range(3))
    pad = np.zeros(tokens, np.uint8)
    pad[13:41] = 1  # interior range, like ragged text padding
    c = cfg(tokens, heads, heads, dim)
    masked = zo.attention_rows(q, k, v, c, 0, tokens, key_pad=pad)
    keep = np.flatnonzero(pad == 0)
    # delete the keys, keep all queries: run per query row against the reduced set
    n = keep.size
    c2 = cfg(n, heads, heads, dim)
    for row in (0, 12, 13, 40, 41, 69):
        q2 = np.zeros((n, heads, dim), np.float32)
        q2[0] = q[row]
        ref = zo.attention_rows(q2, k[keep], v[keep], c2, 0, 1)[0]
        assert np.array_equal(masked[row], ref)
    assert np.abs(masked - brute_force(q, k, v, c, key_pad=pad)).max() < 2e-5


def test_suffix_mask_equals_valid():
    rng = np.random.default_rng(12)
    tokens, heads, dim = 45, 2, 16
    q, k, v = (rng.standard_normal((tokens, heads, dim), dtype=np.float32) for _ in range(3))
    pad = np.zeros(tokens, np.uint8)
    pad[30:] = 1
    a = zo.attention_rows(q, k, v, cfg(tokens, heads, heads, dim), 0, tokens, key_pad=pad)
    b = zo.attention_run(q, k, v, cfg(tokens, heads, heads, dim, valid=30))
    assert np.array_equal(a, b)


def test_batches_are_independent_segments():
    # the batched layout is a loop over segments (klein/zflux2_resident.zig:1803-1833)
    rng = np.random.default_rng(13)
    tokens, heads, dim, nb = 20, 2, 16, 3
    q, k, v = (rng.standard_normal((nb, tokens, heads, dim), dtype=np.float32) for _ in range(3))
    c = cfg(tokens, heads, heads, dim)
    outs = [zo.attention_run(q[b], k[b], v[b], c) for b in range(nb)]
    q2 = q.copy()
    q2[1] += 1.0
    outs2 = [zo.attention_run(q2[b], k[b], v[b], c) for b in range(nb)]
    assert np.array_equal(outs[0], outs2[0]) and np.array_equal(outs[2], outs2[2])
    assert not np.array_equal(outs[1], outs2[1])
