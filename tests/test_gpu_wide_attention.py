"""One wide head (heads = 1, head_dim = 512: the VAE mid-block) through the host
mirror and the C ABI, against the CPU oracle (runtime/attention.zig).

Tolerance: the bf16 attention bar, max |err| <= 2e-2 and mean |err| <= 2e-3 on
outputs of unit scale (Q, K, V rounded to bf16, fp32 accumulation); the
reference's own test of its wide kernel (metal/mattn_test.zig:138-230) uses
N(0, 0.25) inputs, the smallest multiple of 64 past 6144 tokens, sampled rows
including both row blocks of the first, a middle and the last workgroup, and
byte-equal reruns: restated here.
"""
import ctypes as C

import numpy as np
import pytest

from oracle import zoracle as zo
from tests import refimpl
from zdraw_amd import hip, host

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = host.Context.init()
    yield c
    c.deinit()


def draw(rng, tokens, scale=1.0):
    return tuple((rng.standard_normal((tokens, 1, 512), dtype=np.float32) * np.float32(scale)) for _ in range(3))


@pytest.mark.parametrize("tokens", [64, 128, 448, 1024])
def test_wide_head_matches_oracle_on_every_row(ctx, tokens):
    rng = np.random.default_rng(40 + tokens)
    q, k, v = draw(rng, tokens)
    cfg = host.Config(tokens, 1, 1, 512)
    got = ctx.run(q, k, v, cfg).reshape(tokens, 1, 512)
    want = zo.attention_run(q, k, v, zo.Config(tokens, 1, 1, 512))
    refimpl.check_close(got, want, f"wide head, {tokens} tokens")
    # pooled and caller-owned-handle forms run the same kernel: same bytes
    again = ctx.run_pooled(q, k, v, cfg).reshape(tokens, 1, 512)
    assert np.array_equal(got, again)


def test_wide_head_reference_case_sampled_rows_and_rerun(ctx):
    # metal/mattn_test.zig:138-230
    tokens = 6208
    rng = np.random.default_rng(0x51DE)
    q, k, v = draw(rng, tokens, 0.5)
    cfg = host.Config(tokens, 1, 1, 512)
    got = ctx.run(q, k, v, cfg).reshape(tokens, 1, 512)
    again = ctx.run(q, k, v, cfg).reshape(tokens, 1, 512)
    assert got.tobytes() == again.tobytes()
    assert np.isfinite(got).all()
    ocfg = zo.Config(tokens, 1, 1, 512)
    rows = [0, 7, 8, 15, 16, 31, 32, 63, 64, 3103, 6191, 6207]
    want = zo.attention_token_list(q, k, v, ocfg, rows)
    err = np.abs(got[rows] - want.reshape(len(rows), 1, 512))
    # the reference's bar for its half-precision MMA kernel on these inputs is 2e-3 absolute
    assert err.max() <= 2e-3, err.max()
    # every row is written: with 6208 keys of N(0, 0.25) values no output row can be exactly zero
    assert (np.abs(got).max(axis=(1, 2)) > 0).all()


def test_wide_head_at_the_1024_px_length_sampled_rows_and_rerun(ctx):
    # 16384 tokens, the VAE mid-block of a 1024 px render and the length the kernel's throughput
    # is quoted on: one workgroup per CU, no key ranges. Sampled rows in the manner of
    # metal/mattn_test.zig:138-224 (both halves of the first, a middle and the last query tile,
    # rows of every wave), N(0, 1) operands at the bf16 bar, byte-equal rerun.
    tokens = 16384
    rng = np.random.default_rng(0x16384)
    q, k, v = draw(rng, tokens)
    cfg = host.Config(tokens, 1, 1, 512)
    got = ctx.run(q, k, v, cfg).reshape(tokens, 1, 512)
    again = ctx.run(q, k, v, cfg).reshape(tokens, 1, 512)
    assert got.tobytes() == again.tobytes()
    assert np.isfinite(got).all()
    rows = [0, 31, 32, 63, 64, 95, 96, 127, 128, 8191, 8192, 8255, 12345, 16256, 16319, 16352, 16383]
    want = zo.attention_token_list(q, k, v, zo.Config(tokens, 1, 1, 512), rows)
    refimpl.check_close(got[rows], want.reshape(len(rows), 1, 512), "wide head, 16384 tokens")
    assert (np.abs(got).max(axis=(1, 2)) > 0).all()


def test_wide_head_sharp_softmax_and_large_scores(ctx):
    # rows whose scores span a wide range (no QK-norm in front of this attention): a key along
    # the query's direction scores about 34 against a field of N(0, 1) scores; the running
    # maximum must follow it wherever in the sequence it sits (first block, last block, middle),
    # and the blocks far below it must contribute next to nothing. (The planted keys are kept
    # moderate: a bf16 operand's rounding error grows with the score, for every other row too.)
    tokens = 256
    rng = np.random.default_rng(77)
    q, k, v = draw(rng, tokens)
    for i, j in ((3, 0), (40, 255), (200, 100)):
        k[j, 0] = 1.5 * q[i, 0] / np.linalg.norm(q[i, 0]) * np.sqrt(512.0)
    got = ctx.run(q, k, v, host.Config(tokens, 1, 1, 512)).reshape(tokens, 1, 512)
    want = zo.attention_run(q, k, v, zo.Config(tokens, 1, 1, 512))
    refimpl.check_close(got, want, "sharp softmax")
    for i, j in ((3, 0), (40, 255), (200, 100)):
        assert np.abs(want[i, 0] - v[j, 0]).max() < 1e-3  # the planted key really takes the whole row


def test_wide_head_reference_point_moves_several_times(ctx):
    # 1152 tokens (nine query tiles, 36 key blocks): rows whose best key so far is overtaken
    # three times, 8 to 11 in the score each time, so the accumulated O is rescaled in place
    # with earlier contributions still in it (each planted key keeps e^-8 .. e^-11 of the
    # weight of the next); rows in every wave of a tile and in both halves of the output dims
    # are checked against the oracle like all others.
    tokens = 1152
    rng = np.random.default_rng(78)
    q, k, v = draw(rng, tokens)
    rows = (5, 37, 70, 127, 600, 1151)
    for n, i in enumerate(rows):
        unit = q[i, 0] / np.linalg.norm(q[i, 0]) * np.sqrt(512.0)
        for level, j in ((0.45, 40 + n), (0.8, 500 + n), (1.3, 1100 + n)):  # scores about 10, 18, 29
            k[j, 0] = level * unit
    got = ctx.run(q, k, v, host.Config(tokens, 1, 1, 512)).reshape(tokens, 1, 512)
    want = zo.attention_run(q, k, v, zo.Config(tokens, 1, 1, 512))
    refimpl.check_close(got, want, "several moves of the reference point")
    for n, i in enumerate(rows):
        assert np.abs(want[i, 0] - v[1100 + n, 0]).max() < 1e-2  # the last planted key takes the row


def test_wide_head_scores_that_outgrow_the_fixed_reference_take_the_safe_kernel(ctx):
    # The fast kernel exponentiates every score of a row against the largest score of the first
    # block of its key range and flags a query tile whose row sums show a score more than 2^90
    # above that; flagged tiles are formed again by the running-maximum kernel that follows every
    # launch. Ordinary data flags nothing; a key 75 nats (108 in log2) above a field of N(0, 1)
    # scores, late in a range, flags its tile and only that one, and the rows still match.
    L = hip.lib()
    tokens = 1024
    rng = np.random.default_rng(79)
    q, k, v = draw(rng, tokens)
    cfg = host.Config(tokens, 1, 1, 512)
    got = ctx.run(q, k, v, cfg).reshape(tokens, 1, 512)
    assert L.zdraw_hip_wide_redo_tiles() == 0
    refimpl.check_close(got, zo.attention_run(q, k, v, zo.Config(tokens, 1, 1, 512)), "ordinary data")
    # rows 300 and 301 (tile 2) lean on keys 900 and 901, row 900 (tile 7) on key 1000: keys in the fifth and
    # the last block of the fourth key range (1024 tokens run as four ranges of eight blocks)
    for i, j in ((300, 900), (301, 901), (900, 1000)):
        k[j, 0] = 3.3 * q[i, 0] / np.linalg.norm(q[i, 0]) * np.sqrt(512.0)
    got = ctx.run(q, k, v, cfg).reshape(tokens, 1, 512)
    flagged = L.zdraw_hip_wide_redo_tiles()
    assert flagged == 2, flagged
    assert np.isfinite(got).all()
    want = zo.attention_run(q, k, v, zo.Config(tokens, 1, 1, 512))
    # (a bf16 operand's rounding error grows with the score: the planted rows are sharp one-hot
    # rows and are compared as such; every other row at the usual bar)
    others = np.ones(tokens, bool)
    others[[300, 301, 900]] = False
    refimpl.check_close(got[others], want[others], "rows beside the planted ones")
    for i, j in ((300, 900), (301, 901), (900, 1000)):
        assert np.abs(got[i, 0] - v[j, 0]).max() < 2e-2
    again = ctx.run(q, k, v, cfg).reshape(tokens, 1, 512)
    assert got.tobytes() == again.tobytes()


def test_wide_head_refusals_leave_nothing_enqueued(ctx):
    L = hip.lib()
    d0 = L.zdraw_hip_dispatch_count()
    z = np.zeros((96, 1, 512), np.float32)
    with pytest.raises(host.UnsupportedShape):  # tokens % 64 != 0 (mattn.zig:265)
        ctx.run(z, z, z, host.Config(96, 1, 1, 512))
    z2 = np.zeros((64, 2, 512), np.float32)
    with pytest.raises(host.UnsupportedShape):  # heads != 1 (mattn.zig:263)
        ctx.run(z2, z2, z2, host.Config(64, 2, 2, 512))
    z3 = np.zeros((64, 1, 256), np.float32)
    with pytest.raises(host.UnsupportedShape):
        ctx.run(z3, z3, z3, host.Config(64, 1, 1, 256))
    z4 = np.zeros((64, 1, 512), np.float32)
    with pytest.raises(host.UnsupportedShape):  # causal shapes are refused on the host
        ctx.run(z4, z4, z4, host.Config(64, 1, 1, 512, True))
    assert L.zdraw_hip_dispatch_count() == d0
    # C ABI: the wide pipeline runs kernel = wide only, and the block pipeline refuses width 512
    err = C.create_string_buffer(128)
    wide = L.zdraw_hip_compile(ctx.device, None, b"attention_wide_mfma", err, 128)
    assert wide, err.value
    assert L.zdraw_hip_pipeline_threads(wide) == 512
    b = ctx.buffer(z4)
    o = ctx.buffer(nbytes=z4.nbytes)
    p = hip.AttnParams(64, 1, 1, 512, 0, 0)
    assert L.zdraw_hip_run_attention(ctx.queue, wide, b.handle, b.handle, b.handle, o.handle, C.byref(p), hip.K_BLOCK, 512) == 1
    assert L.zdraw_hip_run_attention(ctx.queue, ctx.block_pipeline, b.handle, b.handle, b.handle, o.handle, C.byref(p), hip.K_BLOCK, 512) == 1
    p_short = hip.AttnParams(128, 1, 1, 512, 0, 0)  # buffers hold 64 rows
    assert L.zdraw_hip_run_attention(ctx.queue, wide, b.handle, b.handle, b.handle, o.handle, C.byref(p_short), hip.K_WIDE, 512) == 2
    assert L.zdraw_hip_dispatch_count() == d0
    assert L.zdraw_hip_run_attention(ctx.queue, wide, b.handle, b.handle, b.handle, o.handle, C.byref(p), hip.K_WIDE, 512) == 0
    assert L.zdraw_hip_dispatch_count() == d0 + 2  # rounding pass + attention
    # all-zero scores: every output row is the mean of V = 0
    assert not o.read(np.float32, z4.shape).any()
    L.zdraw_hip_release_pipeline(wide)
    b.release()
    o.release()


def test_wide_head_batch_offsets(ctx):
    # zdraw_metal_run_attention_enc_off: segments at byte offsets inside one buffer
    L = hip.lib()
    rng = np.random.default_rng(5)
    tokens, nseg = 128, 2
    q, k, v = (rng.standard_normal((nseg, tokens, 1, 512), dtype=np.float32) for _ in range(3))
    qb, kb, vb = ctx.buffer(q), ctx.buffer(k), ctx.buffer(v)
    ob = ctx.buffer(nbytes=q.nbytes)
    err = C.create_string_buffer(128)
    wide = L.zdraw_hip_compile(ctx.device, None, b"attention_wide_mfma", err, 128)
    p = hip.AttnParams(tokens, 1, 1, 512, 0, 0)
    seg = tokens * 512 * 4
    batch = L.zdraw_hip_batch_begin(ctx.queue)
    for i in range(nseg):
        assert L.zdraw_hip_run_attention_enc_off(batch, wide, qb.handle, kb.handle, vb.handle, ob.handle, C.byref(p),
                                                 hip.K_WIDE, 512, i * seg, i * seg) == 0, hip.last_error()
    assert L.zdraw_hip_batch_end(batch) == 0
    got = ob.read(np.float32, q.shape)
    for i in range(nseg):
        refimpl.check_close(got[i], zo.attention_run(q[i], k[i], v[i], zo.Config(tokens, 1, 1, 512)), f"segment {i}")
    L.zdraw_hip_release_pipeline(wide)
    for b in (qb, kb, vb, ob):
        b.release()
