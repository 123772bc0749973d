"""The attention segment of one Z-Image layer (q/k/v projections, QK-norm + rope,
attention, output projection: metal_api.m:7103-7108, 7134-7212) through the C ABI,
on a padded sequence built the way the reference builds it, against the oracle
chain (runtime/ops.zig linear, zimage/zattn.zig:45-82 norm -> rope -> attention).

Tolerance: the attention path's bar in units of the output's scale (max |err| <=
2e-2 s, mean |err| <= 2e-3 s, s = rms of the expected output): q, k, v and the
mixed heads each pass a 16-bit rounding whose last bit may flip between the two
summation orders.
"""
import ctypes as C

import numpy as np
import pytest

from oracle import zoracle as zo
from zdraw_amd import hip, host
from zdraw_amd import workloads as wl

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = host.Context.init()
    yield c
    c.deinit()


def to16(x, wdt):
    if wdt == hip.W_BF16:
        bits = host.f32_to_bf16_bits(x)
        return bits, host.bf16_bits_to_f32(bits)
    h = x.astype(np.float16)
    return h.view(np.uint16), h.astype(np.float32)


def padded_sequence(rng, hidden, grid, cap_real):
    """Image tokens first, then caption, both padded to a multiple of 32
    (zimage/zunify.zig:16-37, zseq.zig:38-71); pad slots carry the learned pad rows
    (x_pad / cap_pad) and the positions padWithIds gives them."""
    img_real = grid[0] * grid[1]
    cap_total = zo.zseq_padded_len(cap_real)
    img_feat = rng.standard_normal((img_real, hidden), dtype=np.float32)
    cap_feat = rng.standard_normal((cap_real, hidden), dtype=np.float32)
    x_pad, cap_pad = (rng.standard_normal(hidden, dtype=np.float32) for _ in range(2))
    img, img_pos, img_mask, _ = zo.zseq_pad_with_ids(img_feat, hidden, (1, grid[0], grid[1]), (cap_total + 1, 0, 0))
    cap, cap_pos, cap_mask, _ = zo.zseq_pad_with_ids(cap_feat, hidden, (cap_total, 1, 1), (1, 0, 0))
    img[img_mask] = x_pad
    cap[cap_mask] = cap_pad
    assert img_mask.sum() == img.shape[0] - img_real and img.shape[0] % 32 == 0
    assert cap_mask.sum() == cap_total - cap_real and (cap_pos[-1] == (cap_total, 0, 0)).all()
    assert (img_pos[img_real:] == 0).all()  # image pad slots sit at the origin
    x, pos, _ = zo.zunify_basic(img, img_pos, cap, cap_pos, hidden)
    return x, pos


@pytest.mark.parametrize("act,wdt,ndt", [(hip.F32, hip.W_F16, hip.W_F32), (hip.F32, hip.W_F16, hip.W_F16),
                                         (hip.F32, hip.W_BF16, hip.W_BF16), (hip.BF16, hip.W_BF16, hip.W_BF16),
                                         (hip.BF16, hip.W_BF16, hip.W_F32)])
def test_chain_attention_segment_matches_oracle_chain(ctx, act, wdt, ndt):
    L = hip.lib()
    rng = np.random.default_rng(31)
    heads = 2
    hidden = inner = heads * 128
    x, pos = padded_sequence(rng, hidden, (5, 7), 20)
    tokens = x.shape[0]
    assert tokens == 64 + 32
    ws = [rng.standard_normal((inner, hidden), dtype=np.float32) * np.float32(hidden ** -0.5) for _ in range(3)]
    w_proj = rng.standard_normal((hidden, inner), dtype=np.float32) * np.float32(inner ** -0.5)
    nq, nk = (1.0 + 0.1 * rng.standard_normal(128).astype(np.float32) for _ in range(2))
    cfg = zo.RopeConfig(wl.ZIMAGE_DIMS, wl.ZIMAGE_LENS, wl.ZIMAGE_THETA)
    vals = zo.zrope_fill(cfg)
    bases = zo.zrope_axis_bases(cfg)

    # norm weights sit at a byte offset inside a larger buffer, as QkNormParams allows
    def norm_bytes(v):
        if ndt == hip.W_F32:
            return v.astype(np.float32).tobytes(), v.astype(np.float32)
        bits, back = to16(v, ndt)
        return bits.tobytes(), back
    qn_bytes, nq_r = norm_bytes(nq)
    kn_bytes, nk_r = norm_bytes(nk)
    norm_buf = ctx.buffer(np.frombuffer(b"\0" * 64 + qn_bytes + b"\0" * 32 + kn_bytes, dtype=np.uint8))
    q_off, k_off = 64, 64 + len(qn_bytes) + 32

    wbits = [to16(w, wdt) for w in ws + [w_proj]]
    # one weight buffer, four byte offsets (GemmParams.weight_offset)
    wbuf = ctx.buffer(np.concatenate([b.ravel() for b, _ in wbits]))
    woff = [0, inner * hidden * 2, 2 * inner * hidden * 2, 3 * inner * hidden * 2]
    if act == hip.F32:
        xin, xr = x, to16(x, wdt)[1]
        esz = 4
    else:
        bits, xr = to16(x, hip.W_BF16)
        xin, esz = bits, 2
    nb = ctx.buffer(xin)
    qb, kb, vb, mixb = (ctx.buffer(nbytes=tokens * inner * esz) for _ in range(4))
    ob = ctx.buffer(nbytes=tokens * hidden * esz)
    posb = ctx.buffer(np.ascontiguousarray(pos, dtype=np.uint64))
    ropeb = ctx.buffer(vals)

    p = hip.ChainAttnParams()
    for name, off, (m, k, n) in (("q", woff[0], (tokens, hidden, inner)), ("k", woff[1], (tokens, hidden, inner)),
                                 ("v", woff[2], (tokens, hidden, inner)), ("proj", woff[3], (tokens, inner, hidden))):
        setattr(p, name, hip.GemmParams(m, k, n, wdt, hip.GEMM_HALF, off))
    p.qk = hip.QkNormParams(tokens, heads, heads, 128, ndt, ndt, *wl.ZIMAGE_DIMS, wl.ZIMAGE_EPS, q_off, k_off, *bases)
    p.attn = hip.AttnParams(tokens, heads, heads, 128, 0, 0)
    p.act_dtype = act
    p.score_bound = host.score_bound(nq_r, nk_r, None, None)
    bufs = hip.ChainAttnBuffers(nb.handle, qb.handle, kb.handle, vb.handle, mixb.handle, ob.handle)
    wts = hip.ChainAttnWeights(wbuf.handle, wbuf.handle, wbuf.handle, norm_buf.handle, norm_buf.handle,
                               posb.handle, ropeb.handle, wbuf.handle)
    batch = L.zdraw_hip_batch_begin(ctx.queue)
    d0 = L.zdraw_hip_dispatch_count()
    assert L.zdraw_hip_run_chain_attn_enc(batch, C.byref(bufs), C.byref(wts), C.byref(p)) == 0, hip.last_error()
    assert L.zdraw_hip_batch_end(batch) == 0
    assert L.zdraw_hip_dispatch_count() - d0 == 4  # q/k/v projections in one launch, pre-pass, attention, projection
    if act == hip.F32:
        got = ob.read(np.float32, (tokens, hidden))
    else:
        got = host.bf16_bits_to_f32(ob.read(np.uint16, (tokens, hidden)))

    # oracle chain with the same hand-over roundings
    hand = (lambda a: a) if act == hip.F32 else (lambda a: to16(a, hip.W_BF16)[1])
    q, k, v = (hand(zo.linear_batch(xr, wr)).reshape(tokens, heads, 128) for _, wr in wbits[:3])
    qn = zo.zimage_rotate(zo.zimage_norm_heads(q, nq_r, wl.ZIMAGE_EPS), vals, cfg, pos)
    kn = zo.zimage_rotate(zo.zimage_norm_heads(k, nk_r, wl.ZIMAGE_EPS), vals, cfg, pos)
    mix = zo.attention_run(qn, kn, v, zo.Config(tokens, heads, heads, 128)).reshape(tokens, inner)
    want = zo.linear_batch(to16(hand(mix), wdt)[1], wbits[3][1])
    s = float(np.sqrt(np.mean(want.astype(np.float64) ** 2)))
    err = np.abs(got - want)
    assert err.max() <= 2e-2 * max(s, 1.0) and err.mean() <= 2e-3 * max(s, 1.0), (err.max(), err.mean(), s)
    # the pad rows are ordinary rows: they are attended to and produce output
    assert np.abs(got[35:64]).max() > 0 and np.abs(got[64 + 20:]).max() > 0
    for b in (nb, qb, kb, vb, mixb, ob, posb, ropeb, wbuf, norm_buf):
        b.release()


def test_chain_attention_segment_refuses_what_it_cannot_run(ctx):
    # 1 = unavailable with nothing enqueued (the caller keeps its own path), negative = invalid
    L = hip.lib()
    tokens, heads = 32, 1
    hidden = 128
    z = ctx.buffer(nbytes=tokens * hidden * 4)
    w = ctx.buffer(nbytes=4 * hidden * hidden * 2)
    nw = ctx.buffer(np.ones(128, np.float32))
    cfg = zo.RopeConfig(wl.ZIMAGE_DIMS, wl.ZIMAGE_LENS, wl.ZIMAGE_THETA)
    vals = zo.zrope_fill(cfg)
    bases = zo.zrope_axis_bases(cfg)
    posb = ctx.buffer(np.zeros((tokens, 3), np.uint64))
    ropeb = ctx.buffer(vals)

    def make(wdt=hip.W_F16, mode=hip.GEMM_HALF, act=hip.F32, ndt=hip.W_F32, m=tokens):
        p = hip.ChainAttnParams()
        for name in ("q", "k", "v", "proj"):
            setattr(p, name, hip.GemmParams(m, hidden, hidden, wdt, mode, 0))
        p.qk = hip.QkNormParams(tokens, heads, heads, 128, ndt, ndt, *wl.ZIMAGE_DIMS, wl.ZIMAGE_EPS, 0, 0, *bases)
        p.attn = hip.AttnParams(tokens, heads, heads, 128, 0, 0)
        p.act_dtype = act
        return p

    bufs = hip.ChainAttnBuffers(*([z.handle] * 6))
    wts = hip.ChainAttnWeights(w.handle, w.handle, w.handle, nw.handle, nw.handle, posb.handle, ropeb.handle, w.handle)
    batch = L.zdraw_hip_batch_begin(ctx.queue)
    d0 = L.zdraw_hip_dispatch_count()
    run = lambda p: L.zdraw_hip_run_chain_attn_enc(batch, C.byref(bufs), C.byref(wts), C.byref(p))
    assert run(make(mode=hip.GEMM_EXACT)) == hip.UNAVAILABLE
    assert run(make(wdt=hip.W_F32)) == hip.UNAVAILABLE
    assert run(make(act=hip.BF16)) == hip.UNAVAILABLE          # bf16 activations with f16 weights
    assert run(make(act=hip.F16)) == hip.UNAVAILABLE
    assert run(make(ndt=7)) == hip.UNAVAILABLE
    assert run(make(m=tokens + 1)) == hip.INVALID
    assert L.zdraw_hip_dispatch_count() == d0
    assert L.zdraw_hip_batch_end(batch) == 0
    for b in (z, w, nw, posb, ropeb):
        b.release()


def test_full_size_segment_rerun_builds_and_exact_scaling(ctx):
    # The zimage_1024 shape (4608 tokens, 30 heads, hidden 3840, bf16): the q/k/v group is 810
    # tiles and the output projection 270, so both run their last round split along k. No CPU
    # oracle finishes this size; what the domain fixes instead: a rerun gives the same bits;
    # the eight-wave GEMM build, which never splits, gives the same values up to the order of
    # the fp32 sums; doubling the projection weights (exact in bf16) doubles every output bit
    # for bit; and f32 activation buffers holding the same bf16 values agree to rounding.
    L = hip.lib()
    w = wl.by_name("zimage_1024", seed=3)
    tokens, heads = w.tokens, w.heads
    hidden = inner = heads * 128
    for m_, k_, n_, g_, want in ((tokens, hidden, inner, 3, (42, 6)), (tokens, inner, hidden, 1, (14, 8))):
        t, s = C.c_uint32(), C.c_uint32()
        L.zdraw_hip_gemm_tail_plan(m_, k_, n_, g_, 256, C.byref(t), C.byref(s))
        assert (t.value, s.value) == want
    rng = np.random.default_rng(3)
    x = host.bf16_bits_to_f32(host.f32_to_bf16_bits(rng.standard_normal((tokens, hidden), dtype=np.float32)))
    wall = rng.standard_normal((4, inner, hidden), dtype=np.float32) * np.float32(hidden ** -0.5)
    wall2 = wall.copy()
    wall2[3] *= 2.0
    ones = ctx.buffer(np.ones(128, np.float32))
    posb = ctx.buffer(np.ascontiguousarray(w.pos, dtype=np.uint64))
    ropeb = ctx.buffer(w.rope_pairs)

    def run(act, weights, build=1):
        esz = 4 if act == hip.F32 else 2
        nb = ctx.buffer(x if act == hip.F32 else host.f32_to_bf16_bits(x))
        wb = ctx.buffer(host.f32_to_bf16_bits(weights))
        qb, kb, vb, mixb, ob = (ctx.buffer(nbytes=tokens * inner * esz) for _ in range(5))
        p = hip.ChainAttnParams()
        for i, name in enumerate(("q", "k", "v", "proj")):
            setattr(p, name, hip.GemmParams(tokens, hidden, inner, hip.W_BF16, hip.GEMM_HALF, i * inner * hidden * 2))
        p.qk = hip.QkNormParams(tokens, heads, heads, 128, hip.W_F32, hip.W_F32, *wl.ZIMAGE_DIMS, wl.ZIMAGE_EPS, 0, 0,
                                *w.rope_bases)
        p.attn = hip.AttnParams(tokens, heads, heads, 128, 0, 0)
        p.act_dtype = act
        p.score_bound = host.score_bound(np.ones(128, np.float32), np.ones(128, np.float32), None, None)
        bufs = hip.ChainAttnBuffers(nb.handle, qb.handle, kb.handle, vb.handle, mixb.handle, ob.handle)
        wts = hip.ChainAttnWeights(wb.handle, wb.handle, wb.handle, ones.handle, ones.handle, posb.handle, ropeb.handle,
                                   wb.handle)
        L.zdraw_hip_set_gemm_build(build)
        try:
            batch = L.zdraw_hip_batch_begin(ctx.queue)
            rc = L.zdraw_hip_run_chain_attn_enc(batch, C.byref(bufs), C.byref(wts), C.byref(p))
            assert L.zdraw_hip_batch_end(batch) == 0
        finally:
            L.zdraw_hip_set_gemm_build(1)
        assert rc == 0, hip.last_error()
        out = ob.read(np.float32, (tokens, hidden)) if act == hip.F32 else host.bf16_bits_to_f32(ob.read(np.uint16, (tokens, hidden)))
        for b in (nb, wb, qb, kb, vb, mixb, ob):
            b.release()
        return out

    base = run(hip.BF16, wall)
    assert np.isfinite(base).all() and np.abs(base).max() > 0
    assert np.array_equal(base.view(np.uint32), run(hip.BF16, wall).view(np.uint32))
    assert np.array_equal((2.0 * base).view(np.uint32), run(hip.BF16, wall2).view(np.uint32))
    scale = float(np.sqrt(np.mean(base.astype(np.float64) ** 2)))
    whole = run(hip.BF16, wall, build=0)
    err = np.abs(base - whole)
    assert err.max() <= 2e-2 * scale and err.mean() <= 2e-3 * scale, (err.max(), err.mean(), scale)
    # f32 buffers keep q, k, v and the attention output unrounded between the steps: four bf16
    # hand-over roundings apart, so half a percent of the output's scale on average
    f32 = run(hip.F32, wall)
    err = np.abs(base - f32)
    assert err.max() <= 1e-1 * scale and err.mean() <= 1e-2 * scale, (err.max(), err.mean(), scale)
    for b in (ones, posb, ropeb):
        b.release()
