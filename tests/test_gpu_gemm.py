"""Parity of the projection GEMM (C = A x W^T) with the CPU oracle, through the
C ABI. The reference's half mode rounds both operands to the weight's 16-bit
type and accumulates in fp32 (metal/mgemm.zig, gemm_mode.zig); so does the
kernel. Two bars, both stated where they are used:
  * against the oracle fed the SAME rounded operands only the summation order
    differs: |err| <= 2e-5 * sqrt(k) * (rms of A) * (rms of W) ... in practice 1e-6 relative;
  * against the fp32 oracle on the un-rounded operands: max |err| <= 2e-2 * s,
    mean |err| <= 2e-3 * s with s = sqrt(k) * rms(A) * rms(W) (the attention
    path's tolerance in units of the output's scale).
"""
import ctypes as C

import numpy as np
import pytest

from oracle import zoracle as zo
from zdraw_amd import hip, host

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = host.Context.init()
    yield c
    c.deinit()


@pytest.fixture(scope="module")
def pipe(ctx):
    L = hip.lib()
    err = C.create_string_buffer(128)
    p = L.zdraw_hip_compile(ctx.device, None, b"gemm_half", err, 128)
    assert p, err.value
    yield p
    L.zdraw_hip_release_pipeline(p)


def to16(x, wdt):
    """fp32 -> the 16-bit type's bits and the value they decode to."""
    if wdt == hip.W_BF16:
        bits = host.f32_to_bf16_bits(x)
        return bits, host.bf16_bits_to_f32(bits)
    h = x.astype(np.float16)
    return h.view(np.uint16), h.astype(np.float32)


def from16(bits, wdt):
    return host.bf16_bits_to_f32(bits) if wdt == hip.W_BF16 else bits.view(np.float16).astype(np.float32)


def act_dtype(wdt):
    return hip.BF16 if wdt == hip.W_BF16 else hip.F16


def run_ext(ctx, a_host, w_bits, m, k, n, wdt, a_dtype, c_dtype, lda=0, ldc=0, a_off=0, c_off=0, c_init=None):
    L = hip.lib()
    ab, wb = ctx.buffer(a_host), ctx.buffer(w_bits)
    esz = 4 if c_dtype == hip.F32 else 2
    rows = m
    pitch = ldc or n
    cb = ctx.buffer(c_init) if c_init is not None else ctx.buffer(nbytes=c_off + rows * pitch * esz)
    params = hip.GemmParams(m, k, n, wdt, hip.GEMM_HALF, 0)
    ext = hip.GemmExt(a_off, c_off, lda, 0, ldc, a_dtype, c_dtype)
    batch = L.zdraw_hip_batch_begin(ctx.queue)
    rc = L.zdraw_hip_run_gemm_ext_enc(batch, ab.handle, wb.handle, cb.handle, C.byref(params), C.byref(ext))
    assert L.zdraw_hip_batch_end(batch) == 0
    assert rc == 0, hip.last_error()
    raw = cb.read(np.uint8, (cb.nbytes,))
    for b in (ab, wb, cb):
        b.release()
    return raw


def check(got, want_same_rounding, want_fp32, k, a, w, what):
    s = np.sqrt(k) * np.sqrt(np.mean(a.astype(np.float64) ** 2)) * np.sqrt(np.mean(w.astype(np.float64) ** 2))
    e1 = np.abs(got - want_same_rounding)
    assert e1.max() <= 2e-5 * s + 1e-6, f"{what}: vs oracle on rounded operands max {e1.max():.3e} (scale {s:.3e})"
    e2 = np.abs(got - want_fp32)
    assert e2.max() <= 2e-2 * s and e2.mean() <= 2e-3 * s, f"{what}: vs fp32 oracle max {e2.max():.3e} mean {e2.mean():.3e}"


def test_reference_bf16_ffn_shaped_case(ctx, pipe):
    # mlinear_test.zig:82-121 through the blocking entry (metal_c.zig:160-167): f32 A, bf16 W, f32 C, tolerance 0.005
    L = hip.lib()
    m, k, n = 32, 8, 32
    x = ((np.arange(m * k) % 7).astype(np.float32) * np.float32(0.1) - np.float32(0.3)).reshape(m, k)
    raw = (np.arange(n * k) % 11).astype(np.float32) * np.float32(0.05) - np.float32(0.25)
    hi = (raw.view(np.uint32) >> 16).astype(np.uint16).reshape(n, k)
    wv = host.bf16_bits_to_f32(hi)
    ab, wb, cb = ctx.buffer(x), ctx.buffer(hi), ctx.buffer(nbytes=m * n * 4)
    params = hip.GemmParams(m, k, n, hip.W_BF16, hip.GEMM_HALF, 0)
    assert L.zdraw_hip_run_gemm(ctx.queue, pipe, ab.handle, wb.handle, cb.handle, C.byref(params)) == 0, hip.last_error()
    got = cb.read(np.float32, (m, n))
    want = zo.linear_batch(x, wv)
    assert np.abs(got - want).max() <= 0.005
    for b in (ab, wb, cb):
        b.release()


def test_small_known_answer_shapes_take_the_fallback_contract(ctx, pipe):
    # mlinear_test.zig:33-46 is 2 x 2: below this backend's k % 8 granule -> 1 = unavailable,
    # nothing enqueued, the caller keeps its own path (runtime/linear_fast.zig:14-29)
    L = hip.lib()
    ab, wb, cb = ctx.buffer(np.zeros(16, np.float32)), ctx.buffer(np.zeros(16, np.uint16)), ctx.buffer(nbytes=64)
    d0, f0 = L.zdraw_hip_dispatch_count(), L.zdraw_hip_attn_fallback_count()
    for params in (hip.GemmParams(1, 2, 2, hip.W_F16, hip.GEMM_HALF, 0),      # k % 8 != 0
                   hip.GemmParams(8, 8, 8, hip.W_F32, hip.GEMM_HALF, 0),      # f32 weights
                   hip.GemmParams(8, 8, 8, hip.W_BF16, hip.GEMM_EXACT, 0),    # exact mode
                   hip.GemmParams(8, 8, 8, 4, 4, 0)):                         # packed W6
        assert L.zdraw_hip_run_gemm(ctx.queue, pipe, ab.handle, wb.handle, cb.handle, C.byref(params)) == 1
    assert L.zdraw_hip_dispatch_count() == d0 and L.zdraw_hip_attn_fallback_count() == f0 + 4
    # malformed: buffer too small, zero dimension
    assert L.zdraw_hip_run_gemm(ctx.queue, pipe, ab.handle, wb.handle, cb.handle,
                                C.byref(hip.GemmParams(64, 64, 64, hip.W_BF16, hip.GEMM_HALF, 0))) == 2
    assert L.zdraw_hip_run_gemm(ctx.queue, pipe, ab.handle, wb.handle, cb.handle,
                                C.byref(hip.GemmParams(0, 8, 8, hip.W_BF16, hip.GEMM_HALF, 0))) == 2
    for b in (ab, wb, cb):
        b.release()


SHAPES = [(32, 64, 32), (256, 64, 256), (300, 72, 260), (513, 200, 257), (64, 1024, 96), (600, 320, 520)]


@pytest.mark.parametrize("wdt", [hip.W_BF16, hip.W_F16])
@pytest.mark.parametrize("a16", [False, True])
@pytest.mark.parametrize("c16", [False, True])
@pytest.mark.parametrize("shape", SHAPES)
def test_random_matrices_against_the_oracle(ctx, shape, wdt, a16, c16):
    m, k, n = shape
    rng = np.random.default_rng(m * 7 + k * 3 + n)
    a = rng.standard_normal((m, k), dtype=np.float32)
    w = rng.standard_normal((n, k), dtype=np.float32) * np.float32(0.5)
    w_bits, w_val = to16(w, wdt)
    a_bits, a_val = to16(a, wdt)
    adt = act_dtype(wdt)
    raw = run_ext(ctx, a_bits if a16 else a, w_bits, m, k, n, wdt, adt if a16 else hip.F32, adt if c16 else hip.F32)
    got = from16(raw.view(np.uint16).reshape(m, n), wdt) if c16 else raw.view(np.float32).reshape(m, n)
    same = zo.linear_batch(a_val, w_val)          # the kernel rounds f32 activations exactly like to16()
    full = zo.linear_batch(a, w)
    if c16:  # the output rounding adds half an ulp of the 16-bit type
        same = from16(to16(same, wdt)[0], wdt)
        s = np.sqrt(k) * a.std() * w.std()
        assert np.abs(got - same).max() <= (2.0 ** -7 if wdt == hip.W_BF16 else 2.0 ** -10) * np.abs(same).max() + 2e-5 * s
        e2 = np.abs(got - full)
        assert e2.max() <= 3e-2 * s and e2.mean() <= 4e-3 * s
    else:
        check(got, same, full, k, a, w, f"{shape} wdt={wdt} a16={a16}")


def test_offsets_and_leading_dimensions(ctx):
    # a stream's rows written straight into a shared, wider C at a row/column offset
    # (klein/zflux2_resident.zig:1467-1513), A read from a wider matrix
    m, k, n = 70, 96, 40
    lda, ldc = 128, 200
    rng = np.random.default_rng(3)
    big_a = rng.standard_normal((m + 5, lda), dtype=np.float32)
    w = rng.standard_normal((n, k), dtype=np.float32)
    w_bits, w_val = to16(w, hip.W_BF16)
    a_row0, a_col0, c_row0, c_col0 = 3, 16, 9, 24
    c_rows = c_row0 + m + 2
    c_init = np.full((c_rows, ldc), 7.0, np.float32)
    raw = run_ext(ctx, big_a, w_bits, m, k, n, hip.W_BF16, hip.F32, hip.F32, lda=lda, ldc=ldc,
                  a_off=(a_row0 * lda + a_col0) * 4, c_off=(c_row0 * ldc + c_col0) * 4, c_init=c_init)
    got = raw.view(np.float32).reshape(c_rows, ldc)
    a = np.ascontiguousarray(big_a[a_row0:a_row0 + m, a_col0:a_col0 + k])
    want = zo.linear_batch(host.bf16_bits_to_f32(host.f32_to_bf16_bits(a)), w_val)
    block = got[c_row0:c_row0 + m, c_col0:c_col0 + n]
    check(block, want, zo.linear_batch(a, w), k, a, w, "offset block")
    mask = np.ones_like(got, bool)
    mask[c_row0:c_row0 + m, c_col0:c_col0 + n] = False
    assert (got[mask] == 7.0).all(), "wrote outside the addressed block"


def test_reference_offset_entries_and_bit_stability(ctx, pipe):
    # zdraw_metal_run_gemm_off_enc / _f16a_enc: f32 (or 16-bit) A at a byte offset, f32 C at a byte offset
    L = hip.lib()
    m, k, n = 96, 128, 64
    rng = np.random.default_rng(9)
    a = rng.standard_normal((2 * m, k), dtype=np.float32)
    w = rng.standard_normal((n, k), dtype=np.float32)
    w_bits, w_val = to16(w, hip.W_F16)
    a_bits, a_val = to16(a, hip.W_F16)
    ab, a16b, wb = ctx.buffer(a), ctx.buffer(a_bits), ctx.buffer(w_bits)
    cb = ctx.buffer(nbytes=2 * m * n * 4)
    params = hip.GemmParams(m, k, n, hip.W_F16, hip.GEMM_HALF, 0)
    outs = []
    for rep in range(3):
        batch = L.zdraw_hip_batch_begin(ctx.queue)
        assert L.zdraw_hip_run_gemm_off_enc(batch, pipe, ab.handle, wb.handle, cb.handle, C.byref(params),
                                            m * k * 4, m * n * 4) == 0, hip.last_error()
        assert L.zdraw_hip_run_gemm_f16a_enc(batch, a16b.handle, wb.handle, cb.handle, C.byref(params), 0, 0) == 0
        assert L.zdraw_hip_batch_end(batch) == 0
        outs.append(cb.read(np.float32, (2, m, n)))
    assert all(np.array_equal(outs[0].view(np.uint32), o.view(np.uint32)) for o in outs[1:])
    want = zo.linear_batch(a_val, w_val).reshape(2, m, n)
    s = np.sqrt(k) * a.std() * w.std()
    assert np.abs(outs[0][1] - want[1]).max() <= 2e-5 * s   # off_enc: second half of A -> second half of C
    assert np.abs(outs[0][0] - want[0]).max() <= 2e-5 * s   # f16a_enc: first half, A already half
    for b in (ab, a16b, wb, cb):
        b.release()


def test_single_block_chain_projection_attention_projection(ctx):
    # The attention segment of a Klein single block (klein/zflux2_resident.zig:1986-2058):
    # q, k, v = x W^T with W three row ranges of ONE fused weight (weight_offset selects them),
    # written as bf16 token-major rows; QK-norm + rope + attention writes O into the first
    # `hidden` columns of the concat operand (pitch hidden + inner); the out projection reads
    # that operand whole. Checked against the oracle chain with the same bf16 hand-over points.
    from tests import refimpl
    from zdraw_amd import workloads as wl

    L = hip.lib()
    w = wl.by_name("klein_1024", seed=21, small=True)
    tokens, heads = w.tokens, w.heads
    hidden, inner = heads * 128, 2 * heads * 128
    pitch = hidden + inner
    rng = np.random.default_rng(4)
    x = rng.standard_normal((tokens, hidden), dtype=np.float32)
    w_qkv = rng.standard_normal((3 * hidden, hidden), dtype=np.float32) * np.float32(hidden ** -0.5)
    w_out = rng.standard_normal((hidden, pitch), dtype=np.float32) * np.float32(pitch ** -0.5)
    mlp = rng.standard_normal((tokens, inner), dtype=np.float32)
    nq, nk = (1.0 + 0.1 * rng.standard_normal(128).astype(np.float32) for _ in range(2))
    rb = lambda a: host.bf16_bits_to_f32(host.f32_to_bf16_bits(a))

    xb, wqkvb, woutb = ctx.buffer(host.f32_to_bf16_bits(x)), ctx.buffer(host.f32_to_bf16_bits(w_qkv)), ctx.buffer(host.f32_to_bf16_bits(w_out))
    qkv = [ctx.buffer(nbytes=tokens * hidden * 2) for _ in range(3)]
    cat0 = np.zeros((tokens, pitch), np.uint16)
    cat0[:, hidden:] = host.f32_to_bf16_bits(mlp)
    cat = ctx.buffer(cat0)
    out = ctx.buffer(nbytes=tokens * hidden * 4)
    nqb, nkb = ctx.buffer(nq), ctx.buffer(nk)
    cos, sin = ctx.buffer(w.rope_cos), ctx.buffer(w.rope_sin)

    batch = L.zdraw_hip_batch_begin(ctx.queue)
    ext = hip.GemmExt(0, 0, 0, 0, 0, hip.BF16, hip.BF16)
    for i in range(3):
        params = hip.GemmParams(tokens, hidden, hidden, hip.W_BF16, hip.GEMM_HALF, i * hidden * hidden * 2)
        assert L.zdraw_hip_run_gemm_ext_enc(batch, xb.handle, wqkvb.handle, qkv[i].handle, C.byref(params), C.byref(ext)) == 0, hip.last_error()
    assert L.zdraw_hip_batch_end(batch) == 0
    ctx.joint_klein(qkv[0], qkv[1], qkv[2], cat, tokens=tokens, heads=heads, norm_q=nqb, norm_k=nkb,
                    rope_cos=cos, rope_sin=sin, out_row_stride=pitch, k_site=hip.K_PREPASS,
                    score_bound=host.score_bound(nq, nk, None, None))
    batch = L.zdraw_hip_batch_begin(ctx.queue)
    params = hip.GemmParams(tokens, pitch, hidden, hip.W_BF16, hip.GEMM_HALF, 0)
    assert L.zdraw_hip_run_gemm_f16a_enc(batch, cat.handle, woutb.handle, out.handle, C.byref(params), 0, 0) == 0, hip.last_error()
    assert L.zdraw_hip_batch_end(batch) == 0
    got = out.read(np.float32, (tokens, hidden))

    # oracle chain
    xr, wr = rb(x), rb(w_qkv)
    q, k, v = (rb(zo.linear_batch(xr, wr[i * hidden:(i + 1) * hidden])).reshape(tokens, heads, 128) for i in range(3))
    c2, s2 = zo.klein_build_rope_ref(w.grid[0], w.grid[1], theta=w.theta, txt_len=w.txt_len)
    qn = zo.klein_apply_rope(zo.klein_rms_norm_heads(q, nq), c2, s2)
    kn = zo.klein_apply_rope(zo.klein_rms_norm_heads(k, nk), c2, s2)
    o = zo.attention_run(qn, kn, v, zo.Config(tokens, heads, heads, 128)).reshape(tokens, hidden)
    catr = np.concatenate([rb(o), rb(mlp)], axis=1)
    want = zo.linear_batch(catr, rb(w_out))
    # q, k, v and O each pass through a bf16 hand-over whose rounding can flip on a last-bit
    # difference, so the bar is the attention path's: 2e-2 max / 2e-3 mean in units of the output scale
    s = float(np.sqrt(np.mean(want.astype(np.float64) ** 2)))
    err = np.abs(got - want)
    assert err.max() <= 2e-2 * max(s, 1.0) and err.mean() <= 2e-3 * max(s, 1.0), (err.max(), err.mean(), s)
    for b in [xb, wqkvb, woutb, cat, out, nqb, nkb, cos, sin] + qkv:
        b.release()


@pytest.mark.parametrize("count", [2, 3])
@pytest.mark.parametrize("same_shape", [True, False])
def test_pair_and_triple_of_one_activation(ctx, pipe, count, same_shape):
    # metal_c.zig:175-198: gate/up (pair) and q/k/v (triple) products of one f32 A, blocking.
    # Equal shapes run as ONE launch, unequal ones as one launch each; results are those of
    # `count` separate zdraw_hip_run_gemm calls, bit for bit.
    L = hip.lib()
    rng = np.random.default_rng(17 + count)
    m, k = 300, 136
    ns = [264] * count if same_shape else [264, 128, 40][:count]
    a = rng.standard_normal((m, k), dtype=np.float32)
    ws = [rng.standard_normal((n, k), dtype=np.float32) * np.float32(k ** -0.5) for n in ns]
    # all weights in one buffer behind a 32-byte header: weight_offset selects them
    bits = [to16(w, hip.W_F16)[0] for w in ws]
    blob = np.concatenate([np.zeros(16, np.uint16)] + [b.ravel() for b in bits])
    offs = [32 + 2 * sum(n * k for n in ns[:i]) for i in range(count)]
    ab, wb = ctx.buffer(a), ctx.buffer(blob)
    cbs = [ctx.buffer(nbytes=m * n * 4) for n in ns]
    ps = [hip.GemmParams(m, k, n, hip.W_F16, hip.GEMM_HALF, off) for n, off in zip(ns, offs)]
    d0 = L.zdraw_hip_dispatch_count()
    if count == 2:
        rc = L.zdraw_hip_run_gemm_pair(ctx.queue, pipe, ab.handle, wb.handle, cbs[0].handle, C.byref(ps[0]),
                                       wb.handle, cbs[1].handle, C.byref(ps[1]))
    else:
        rc = L.zdraw_hip_run_gemm_triple(ctx.queue, pipe, ab.handle, wb.handle, cbs[0].handle, C.byref(ps[0]),
                                         wb.handle, cbs[1].handle, C.byref(ps[1]), wb.handle, cbs[2].handle, C.byref(ps[2]))
    assert rc == 0, hip.last_error()
    assert L.zdraw_hip_dispatch_count() - d0 == (1 if same_shape else count)
    ar = to16(a, hip.W_F16)[1]
    for i, n in enumerate(ns):
        got = cbs[i].read(np.float32, (m, n))
        wr = from16(bits[i], hip.W_F16)
        check(got, zo.linear_batch(ar, wr), zo.linear_batch(a, ws[i]), k, a, ws[i], f"product {i} of {count}")
        single = ctx.buffer(nbytes=m * n * 4)
        assert L.zdraw_hip_run_gemm(ctx.queue, pipe, ab.handle, wb.handle, single.handle, C.byref(ps[i])) == 0
        assert np.array_equal(single.read(np.float32, (m, n)), got)
        single.release()
    # a product this backend does not run refuses the whole call before anything is enqueued
    bad = hip.GemmParams(m, k, ns[-1], hip.W_F32, hip.GEMM_HALF, 0)
    d0 = L.zdraw_hip_dispatch_count()
    if count == 2 and not same_shape:
        assert L.zdraw_hip_run_gemm_pair(ctx.queue, pipe, ab.handle, wb.handle, cbs[0].handle, C.byref(ps[0]),
                                         wb.handle, cbs[1].handle, C.byref(bad)) == 1
        assert L.zdraw_hip_dispatch_count() == d0
    for b in [ab, wb] + cbs:
        b.release()


@pytest.mark.parametrize("a32", [False, True])
@pytest.mark.parametrize("c_dtype", [hip.F32, hip.BF16])
@pytest.mark.parametrize("build", [1, 0])
def test_many_tile_problem_runs_the_256_tile_builds(ctx, build, c_dtype, a32):
    # 13 x 13 = 169 tiles of 256 x 256 (ragged last row and column of tiles): enough tiles for
    # the 256-tile builds (four waves by default, eight behind the knob), which the small
    # shapes above never reach; with 16-bit C the interior tiles leave through LDS as whole
    # rows and the edge tiles element by element. Against the oracle on identically rounded
    # operands. a32: f32 activations, which are rounded once into scratch ahead of the product
    # and then take the same builds.
    L = hip.lib()
    rng = np.random.default_rng(23)
    m, k, n = 3300, 128, 3290
    ldc = 3296  # rows of C start 16-byte aligned
    a = rng.standard_normal((m, k), dtype=np.float32)
    w = rng.standard_normal((n, k), dtype=np.float32) * np.float32(k ** -0.5)
    a_bits, ar = to16(a, hip.W_BF16)
    w_bits, wr = to16(w, hip.W_BF16)
    L.zdraw_hip_set_gemm_build(build)
    try:
        raw = run_ext(ctx, a if a32 else a_bits, w_bits, m, k, n, hip.W_BF16, hip.F32 if a32 else hip.BF16, c_dtype, ldc=ldc,
                      c_init=np.zeros(m * ldc * (4 if c_dtype == hip.F32 else 2), np.uint8))
    finally:
        L.zdraw_hip_set_gemm_build(1)
    want = zo.linear_batch(ar, wr)
    if c_dtype == hip.F32:
        got = raw.view(np.float32).reshape(m, ldc)[:, :n]
        check(got, want, zo.linear_batch(a, w), k, a, w, f"169 tiles, build {build}")
        tol = 1e-4
    else:
        full = raw.view(np.uint16).reshape(m, ldc)
        got = from16(full[:, :n], hip.W_BF16)
        assert not full[:, n:].any()  # the pad columns of the pitch stay untouched
        s = np.sqrt(k) * np.sqrt(np.mean(ar.astype(np.float64) ** 2)) * np.sqrt(np.mean(wr.astype(np.float64) ** 2))
        err = np.abs(got - want)
        assert err.max() <= 2 ** -8 * np.abs(want).max() + 2e-5 * s  # one bf16 rounding of the fp32 result
        tol = 2 ** -8 * np.abs(want).max() + 1e-4
    # rows and columns of the ragged edge tiles
    assert np.abs(got[-1] - want[-1]).max() < tol and np.abs(got[:, -1] - want[:, -1]).max() < tol


@pytest.mark.parametrize("wdt", [hip.W_BF16, hip.W_F16])
@pytest.mark.parametrize("k", [64, 192, 320])
def test_four_wave_build_with_one_three_and_five_slabs(ctx, k, wdt):
    # the four-wave loop takes two slabs per trip and requests slabs two ahead: one slab (no
    # trip, the odd tail only), three and five (trips plus the tail), 169 tiles each; bf16 and
    # f16 operands (the two MFMA instructions of that build)
    rng = np.random.default_rng(31 + k)
    m, n = 3300, 3290
    a = rng.standard_normal((m, k), dtype=np.float32)
    w = rng.standard_normal((n, k), dtype=np.float32) * np.float32(k ** -0.5)
    a_bits, ar = to16(a, wdt)
    w_bits, wr = to16(w, wdt)
    raw = run_ext(ctx, a_bits, w_bits, m, k, n, wdt, act_dtype(wdt), hip.F32)
    got = raw.view(np.float32).reshape(m, n)
    check(got, zo.linear_batch(ar, wr), zo.linear_batch(a, w), k, a, w, f"k = {k}")
    again = run_ext(ctx, a_bits, w_bits, m, k, n, wdt, act_dtype(wdt), hip.F32)
    assert np.array_equal(raw, again)


@pytest.mark.parametrize("build", [1, 0])
def test_256_tile_builds_16_bit_output_with_unaligned_rows(ctx, build):
    # the same 169 tiles with a pitch of 3291 elements: no row of C starts on 16 bytes, so every
    # 16-bit store is made element by element (four waves: after the turn through LDS; eight
    # waves: from the registers); the pad column of the pitch and the guard behind the last row
    # stay untouched
    L = hip.lib()
    rng = np.random.default_rng(29)
    m, k, n, ldc = 3300, 128, 3290, 3291
    a = rng.standard_normal((m, k), dtype=np.float32)
    w = rng.standard_normal((n, k), dtype=np.float32) * np.float32(k ** -0.5)
    a_bits, ar = to16(a, hip.W_BF16)
    w_bits, wr = to16(w, hip.W_BF16)
    guard = 64
    init = np.full(m * ldc + guard, 0x7e7e, np.uint16)
    L.zdraw_hip_set_gemm_build(build)
    try:
        raw = run_ext(ctx, a_bits, w_bits, m, k, n, hip.W_BF16, hip.BF16, hip.BF16, ldc=ldc, c_init=init.view(np.uint8))
    finally:
        L.zdraw_hip_set_gemm_build(1)
    flat = raw.view(np.uint16)
    assert (flat[m * ldc:] == 0x7e7e).all()
    full = flat[:m * ldc].reshape(m, ldc)
    assert (full[:, n:] == 0x7e7e).all()
    got = from16(full[:, :n], hip.W_BF16)
    want = zo.linear_batch(ar, wr)
    s = np.sqrt(k) * np.sqrt(np.mean(ar.astype(np.float64) ** 2)) * np.sqrt(np.mean(wr.astype(np.float64) ** 2))
    assert np.abs(got - want).max() <= 2 ** -8 * np.abs(want).max() + 2e-5 * s  # one bf16 rounding of the fp32 result


@pytest.mark.parametrize("wdt", [hip.W_BF16, hip.W_F16])
@pytest.mark.parametrize("ldc", [256, 251])
def test_small_tile_build_16_bit_output_edges_and_pitch(ctx, wdt, ldc):
    # Few tiles, 16-bit activations, k a multiple of 64: the 128-tile build. With rows of C on
    # 16 bytes (ldc 256) its 16-bit output leaves through LDS as whole rows: the last rows
    # (m = 200 of 256) must not be stored, the last column chunk (n = 250: two of eight
    # columns) goes element by element, and the pad columns of the pitch stay untouched. With
    # ldc 251 the rows are not aligned and the direct stores run instead. Same results.
    rng = np.random.default_rng(5 + ldc)
    m, k, n = 200, 128, 250
    a = rng.standard_normal((m, k), dtype=np.float32)
    w = rng.standard_normal((n, k), dtype=np.float32) * np.float32(k ** -0.5)
    a_bits, ar = to16(a, wdt)
    w_bits, wr = to16(w, wdt)
    adt = act_dtype(wdt)
    guard = 64  # elements behind the last row: must stay as they were
    init = np.full(m * ldc + guard, 0x7e7e, np.uint16)
    raw = run_ext(ctx, a_bits, w_bits, m, k, n, wdt, adt, adt, ldc=ldc, c_init=init.view(np.uint8))
    flat = raw.view(np.uint16)
    assert (flat[m * ldc:] == 0x7e7e).all()
    full = flat[:m * ldc].reshape(m, ldc)
    assert (full[:, n:] == 0x7e7e).all()
    got = from16(full[:, :n], wdt)
    want = from16(to16(zo.linear_batch(ar, wr), wdt)[0], wdt)
    ulp = 2.0 ** -7 if wdt == hip.W_BF16 else 2.0 ** -10
    assert np.abs(got - want).max() <= ulp * np.abs(want).max() + 1e-5


def _split_tail_case(rng, m, k, n):
    a = rng.standard_normal((m, k), dtype=np.float32)
    w = rng.standard_normal((n, k), dtype=np.float32) * np.float32(k ** -0.5)
    a_bits, ar = to16(a, hip.W_BF16)
    w_bits, wr = to16(w, hip.W_BF16)
    return a_bits, ar, w_bits, wr


@pytest.mark.parametrize("c_dtype", [hip.BF16, hip.F32])
def test_k_split_last_round_matches_whole_tiles_and_oracle(ctx, c_dtype):
    # 17 x 16 = 272 tiles of 256 x 256 on 256 CUs: the 16 tiles of the second round run as 4
    # ranges of k each (19 slabs: 5, 5, 5, 4) and are put together by the merge kernel; ragged
    # last row and column of tiles, pitch wider than the row. Checked against the oracle on
    # identically rounded operands (rows of the split tiles and rows elsewhere), against an
    # fp32 product of the whole matrix, against the eight-wave build (which never splits), and
    # for bit-equal reruns.
    L = hip.lib()
    m, k, n, ldc = 4322, 1216, 4090, 4096
    t, s = C.c_uint32(), C.c_uint32()
    L.zdraw_hip_gemm_tail_plan(m, k, n, 1, 256, C.byref(t), C.byref(s))
    assert (t.value, s.value) == (16, 4)
    a_bits, ar, w_bits, wr = _split_tail_case(np.random.default_rng(41), m, k, n)
    esz = 4 if c_dtype == hip.F32 else 2
    init = np.full(m * ldc * esz, 0x5a, np.uint8)

    def run(build):
        L.zdraw_hip_set_gemm_build(build)
        try:
            raw = run_ext(ctx, a_bits, w_bits, m, k, n, hip.W_BF16, hip.BF16, c_dtype, ldc=ldc, c_init=init)
        finally:
            L.zdraw_hip_set_gemm_build(1)
        if c_dtype == hip.F32:
            full = raw.view(np.float32).reshape(m, ldc)
            assert (raw.reshape(m, ldc * 4)[:, n * 4:] == 0x5a).all()
            return full[:, :n].copy()
        full = raw.view(np.uint16).reshape(m, ldc)
        assert (full[:, n:] == 0x5a5a).all()  # the pad columns of the pitch stay untouched
        return from16(full[:, :n], hip.W_BF16)

    got = run(1)
    assert np.array_equal(got, run(1))
    whole = run(0)
    scale = np.sqrt(k) * np.sqrt(np.mean(ar.astype(np.float64) ** 2)) * np.sqrt(np.mean(wr.astype(np.float64) ** 2))
    ulp = 2.0 ** -8 * max(np.abs(whole).max(), 1.0) if c_dtype == hip.BF16 else 0.0
    assert np.abs(got - whole).max() <= 2 * ulp + 2e-5 * scale  # same products, another summation order
    ref32 = ar @ wr.T
    assert np.abs(got - ref32).max() <= ulp + 1e-4 * scale
    rows = np.unique(np.concatenate([np.arange(m - 300, m), np.random.default_rng(3).choice(m - 300, 200, replace=False)]))
    want = zo.linear_batch(ar[rows], wr)
    assert np.abs(got[rows] - want).max() <= ulp + 2e-5 * scale


def test_k_split_last_round_of_a_group(ctx):
    # two products of one bf16 A through the grouped entry: 2 x (17 x 8) = 272 tiles, the 16
    # split tiles all belong to the second product; against the oracle and the one-by-one runs
    L = hip.lib()
    m, k, n = 4322, 1216, 2040
    t, s = C.c_uint32(), C.c_uint32()
    L.zdraw_hip_gemm_tail_plan(m, k, n, 2, 256, C.byref(t), C.byref(s))
    assert (t.value, s.value) == (16, 4)
    rng = np.random.default_rng(43)
    a_bits, ar, w0_bits, w0r = _split_tail_case(rng, m, k, n)
    w1 = rng.standard_normal((n, k), dtype=np.float32) * np.float32(k ** -0.5)
    w1_bits, w1r = to16(w1, hip.W_BF16)
    ab = ctx.buffer(a_bits)
    wb = ctx.buffer(np.concatenate([w0_bits.ravel(), w1_bits.ravel()]))
    cbs = [ctx.buffer(np.zeros(m * n, np.uint16)) for _ in range(2)]
    ps = [hip.GemmParams(m, k, n, hip.W_BF16, hip.GEMM_HALF, off) for off in (0, n * k * 2)]
    ext = hip.GemmExt(0, 0, 0, 0, 0, hip.BF16, hip.BF16)
    ws = (C.c_void_p * 2)(wb.handle, wb.handle)
    cs = (C.c_void_p * 2)(cbs[0].handle, cbs[1].handle)
    pp = (C.POINTER(hip.GemmParams) * 2)(C.pointer(ps[0]), C.pointer(ps[1]))
    d0 = L.zdraw_hip_dispatch_count()
    batch = L.zdraw_hip_batch_begin(ctx.queue)
    rc = L.zdraw_hip_run_gemm_group_ext_enc(batch, ab.handle, ws, cs, pp, 2, C.byref(ext))
    assert L.zdraw_hip_batch_end(batch) == 0
    assert rc == 0, hip.last_error()
    assert L.zdraw_hip_dispatch_count() - d0 == 1
    scale = np.sqrt(k) * np.sqrt(np.mean(ar.astype(np.float64) ** 2)) * np.sqrt(np.mean(w0r.astype(np.float64) ** 2))
    rows = np.unique(np.concatenate([np.arange(m - 300, m), np.arange(0, m - 300, 37)]))
    for i, wr in enumerate((w0r, w1r)):
        got = from16(cbs[i].read(np.uint16, (m, n)), hip.W_BF16)
        ulp = 2.0 ** -8 * max(np.abs(got).max(), 1.0)
        assert np.abs(got - ar @ wr.T).max() <= ulp + 1e-4 * scale
        assert np.abs(got[rows] - zo.linear_batch(ar[rows], wr)).max() <= ulp + 2e-5 * scale
        one = run_ext(ctx, a_bits, np.concatenate([w0_bits.ravel(), w1_bits.ravel()]), m, k, n, hip.W_BF16, hip.BF16, hip.BF16)
        if i == 0:
            assert np.abs(from16(one.view(np.uint16).reshape(m, n), hip.W_BF16) - got).max() <= 2 * ulp + 2e-5 * scale
    # a count outside 1..3 and a product this backend does not run leave nothing enqueued
    d0 = L.zdraw_hip_dispatch_count()
    batch = L.zdraw_hip_batch_begin(ctx.queue)
    assert L.zdraw_hip_run_gemm_group_ext_enc(batch, ab.handle, ws, cs, pp, 4, C.byref(ext)) < 0
    bad = hip.GemmParams(m, k, n, hip.W_F32, hip.GEMM_HALF, 0)
    pp_bad = (C.POINTER(hip.GemmParams) * 2)(C.pointer(ps[0]), C.pointer(bad))
    assert L.zdraw_hip_run_gemm_group_ext_enc(batch, ab.handle, ws, cs, pp_bad, 2, C.byref(ext)) == 1
    assert L.zdraw_hip_batch_end(batch) == 0
    assert L.zdraw_hip_dispatch_count() == d0
    for b in [ab, wb] + cbs:
        b.release()
