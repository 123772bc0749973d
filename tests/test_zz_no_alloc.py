"""The fused entry that allocates nothing (zdraw_hip_run_attention_fused_noalloc_enc): its
scratch is an array inside the library's device code. Through the C ABI, bit for bit against
zdraw_hip_run_attention_fused_enc on the same operands, on calls in a row that shrink (the
array keeps the previous call's contents), and the size limit."""
import ctypes as C
import sys

import numpy as np
import pytest

from zdraw_amd import hip, host, workloads as wl

pytestmark = pytest.mark.gpu


def say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def ctx():
    c = host.Context.init()
    yield c
    c.deinit()


def _both(ctx, res):
    """One pass through the allocating entry, one through the no-allocation entry: outputs."""
    L = hip.lib()
    outs = []
    for fn in (L.zdraw_hip_run_attention_fused_enc, L.zdraw_hip_run_attention_fused_noalloc_enc):
        res.o.write(np.full(res.o.nbytes, 0x7B, np.uint8))  # a stale output cannot pass for a result
        b = L.zdraw_hip_batch_begin(ctx.queue)
        assert b
        rc = fn(b, res.q.handle, res.k.handle, res.v.handle, res.o.handle, C.byref(res.params), C.byref(res.ext),
                C.byref(res.ops))
        assert L.zdraw_hip_batch_end(b) == 0
        assert rc == 0, hip.last_error()
        outs.append(res.read_output())
    return outs


def _klein(seed, heads, grid, txt_len, batch=1):
    return wl.klein(seed=seed, batch=batch, heads=heads, grid=grid, txt_len=txt_len, name=f"klein {heads}x{grid}")


def test_noalloc_entry_matches_the_allocating_entry_on_shrinking_calls(ctx):
    # first a call whose tiles are split along the keys (parts and their merge go through the
    # array too), then smaller ones, f32 operands (V's bf16 copy), Z-Image, a key mask
    cases = [
        ("klein 1600 tokens x 4 heads, bf16", _klein(1, 4, (32, 34), 512), hip.BF16, True),
        ("klein 700 tokens x 2 heads, bf16", _klein(2, 2, (20, 30), 100), hip.BF16, True),
        ("klein 700 tokens x 2 heads, f32 rows, running maximum", _klein(3, 2, (20, 30), 100), hip.F32, False),
        ("zimage small", wl.by_name("zimage_1024", seed=4, small=True), hip.BF16, True),
        ("ragged edit small, 2 segments", wl.by_name("klein_edit_ragged", seed=5, small=True), hip.BF16, True),
    ]
    for name, w, dtype, bounded in cases:
        say(f"no-alloc: {name}")
        res = wl.Resident(ctx, w, dtype=dtype, k_site=hip.K_PREPASS, bounded=bounded)
        want, got = _both(ctx, res)
        again = _both(ctx, res)[1]
        res.release()
        assert np.isfinite(want).all() and (np.abs(want).max(axis=-1) > 0).all()
        assert np.array_equal(want.view(np.uint32), got.view(np.uint32)), name
        assert np.array_equal(got.view(np.uint32), again.view(np.uint32)), name


def test_noalloc_entry_takes_no_device_memory_on_a_new_queue_with_weights_it_sees_first(ctx):
    import torch

    L = hip.lib()
    # kernels loaded and the device's array looked up: one pass on the shared queue
    warm = wl.Resident(ctx, _klein(6, 2, (20, 30), 100), dtype=hip.BF16, k_site=hip.K_PREPASS, bounded=True)
    _both(ctx, warm)
    warm.release()
    # a second context: its queue has run nothing, its weight buffers are new to the library
    # (their maxima, which the bounded softmax needs, are read during the call below)
    c2 = host.Context.init()
    try:
        res = wl.Resident(c2, _klein(7, 2, (24, 26), 76), dtype=hip.BF16, k_site=hip.K_PREPASS, bounded=True)
        res.o.write(np.full(res.o.nbytes, 0x7B, np.uint8))
        torch.cuda.synchronize()
        free0 = torch.cuda.mem_get_info()[0]
        b = L.zdraw_hip_batch_begin(c2.queue)
        assert b
        say("no-alloc: new queue, new weights")
        rc = L.zdraw_hip_run_attention_fused_noalloc_enc(b, res.q.handle, res.k.handle, res.v.handle, res.o.handle,
                                                         C.byref(res.params), C.byref(res.ext), C.byref(res.ops))
        assert L.zdraw_hip_batch_end(b) == 0
        assert rc == 0, hip.last_error()
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free0, "the call changed the device's free memory"
        got = res.read_output()
        want = _both(c2, res)[0]  # the allocating entry, afterwards
        res.release()
        assert np.isfinite(want).all() and (np.abs(want).max(axis=-1) > 0).all()
        assert np.array_equal(want.view(np.uint32), got.view(np.uint32))
    finally:
        c2.deinit()


def test_noalloc_entry_refuses_what_does_not_fit_its_array(ctx):
    L = hip.lib()
    # bf16 Q' and K' of B x H x S rows: 512 bytes per row; 138240 rows do not fit 64 MiB
    heads, tokens = 30, 4608
    assert heads * tokens * 512 > hip.NOALLOC_SCRATCH_BYTES
    n = tokens * heads * 128
    buf = ctx.buffer(nbytes=n * 2)
    ones = ctx.buffer(np.ones(128, np.float32))
    table = ctx.buffer(nbytes=tokens * 128 * 4)
    p = hip.AttnParams(tokens, heads, heads, 128, 0, 0)
    x = hip.AttnExt()
    for s in (x.q_stride, x.k_stride, x.v_stride, x.out_stride):
        s[0], s[1], s[2] = 0, heads * 128, 128
    x.batch, x.in_dtype, x.out_dtype, x.qk_mode, x.k_site, x.eps = 1, hip.BF16, hip.BF16, hip.QK_KLEIN, hip.K_PREPASS, 1e-6
    ops = hip.QkOperands()
    ops.q_weight = ops.k_weight = ones.handle
    ops.rope_cos = ops.rope_sin = table.handle
    b = L.zdraw_hip_batch_begin(ctx.queue)
    d0, f0 = L.zdraw_hip_dispatch_count(), L.zdraw_hip_attn_fallback_count()
    rc = L.zdraw_hip_run_attention_fused_noalloc_enc(b, buf.handle, buf.handle, buf.handle, buf.handle, C.byref(p),
                                                     C.byref(x), C.byref(ops))
    assert rc == hip.UNAVAILABLE and "scratch" in hip.last_error()
    assert L.zdraw_hip_dispatch_count() == d0 and L.zdraw_hip_attn_fallback_count() == f0 + 1
    # what needs no scratch at all (norm and rope in the tile load) still runs at that size
    x.k_site = hip.K_IN_TILE_LOAD
    x.qk_mode = hip.QK_NONE
    p2 = hip.AttnParams(256, heads, heads, 128, 0, 0)
    rc = L.zdraw_hip_run_attention_fused_noalloc_enc(b, buf.handle, buf.handle, buf.handle, buf.handle, C.byref(p2),
                                                     C.byref(x), None)
    assert rc == 0, hip.last_error()
    assert L.zdraw_hip_batch_end(b) == 0
    for h in (buf, ones, table):
        h.release()
