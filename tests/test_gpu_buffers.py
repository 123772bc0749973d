"""GPU tests of the buffer boundary (metal_c.zig:12-33): how weights reach the library.

The reference binds every weight through mbuffer.Cache.bindView: a no-copy buffer over the
host bytes of the mmapped checkpoint plus a file offset (metal/mbuffer.zig:70-139,
metal/mqk.zig:37-38, 97-98). These tests bind weights exactly that way and check the result
against the oracle; then the interop form over device memory, which must refuse anything
that is not device memory, and whose contents the library must never cache.
"""
import ctypes as C
import sys

import numpy as np
import pytest

from oracle import zoracle as zo
from tests import refimpl
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


def _qk_pipeline(ctx):
    err = C.create_string_buffer(128)
    pipe = hip.lib().zdraw_hip_compile(ctx.device, b"", b"qk_norm_rope", err, 128)
    assert pipe, err.value
    return pipe


_CODES = {
    "f32": (hip.W_F32, lambda a: a.astype(np.float32), lambda a: a),
    "bf16": (hip.W_BF16, host.f32_to_bf16_bits, host.bf16_bits_to_f32),
    "f16": (hip.W_F16, lambda a: a.astype(np.float16), lambda a: a.astype(np.float32)),
}


# q type, k type, q byte offset, k byte offset: file offsets that are only element-aligned, two
# types in one call, and the aligned single-type case that needs no staging beside them
@pytest.mark.parametrize("qt,kt,q_off,k_off", [("f16", "f16", 1002, 3006), ("f16", "bf16", 258, 5006),
                                               ("f32", "f16", 4100, 7002), ("bf16", "bf16", 64, 576)])
def test_no_copy_binds_host_weight_bytes_at_file_offsets(ctx, qt, kt, q_off, k_off):
    # mbuffer.Cache.sourceBuffer + mqk.run: one no-copy buffer over the whole "checkpoint", the
    # norm weights addressed by their file offsets, each with its own element type
    L = hip.lib()
    rng = np.random.default_rng(q_off + k_off)
    tokens, heads, kv_heads = 45, 3, 3
    cfg = zo.RopeConfig(wl.ZIMAGE_DIMS, wl.ZIMAGE_LENS, wl.ZIMAGE_THETA)
    vals = zo.zrope_fill(cfg)
    bases = zo.zrope_axis_bases(cfg)
    pos = np.stack([rng.integers(0, 1536, tokens), rng.integers(0, 512, tokens), rng.integers(0, 512, tokens)], 1).astype(np.uint64)
    q = rng.standard_normal((tokens, heads, 128), dtype=np.float32)
    k = rng.standard_normal((tokens, kv_heads, 128), dtype=np.float32)
    wq = (1.0 + 0.3 * rng.standard_normal(128)).astype(np.float32)
    wk = (1.0 + 0.3 * rng.standard_normal(128)).astype(np.float32)
    (qc, qenc, qdec), (kc, kenc, kdec) = _CODES[qt], _CODES[kt]
    # the host "file": other tensors' bytes all around the two weight vectors
    blob = rng.integers(0, 256, 8192, dtype=np.uint8)
    eq, ek = qenc(wq), kenc(wk)
    blob[q_off:q_off + eq.nbytes] = eq.view(np.uint8)
    blob[k_off:k_off + ek.nbytes] = ek.view(np.uint8)
    # an address that is not page-aligned either (the Metal call refuses those; this one takes any)
    backing = np.zeros(blob.size + 24, np.uint8)
    view = backing[24:]
    view[:] = blob
    weights = L.zdraw_hip_create_buffer_no_copy(ctx.device, view.ctypes.data_as(C.c_void_p), view.size)
    assert weights, hip.last_error()
    assert L.zdraw_hip_buffer_length(weights) == view.size
    backing[:] = 0xA5  # the caller keeps owning its bytes; the library read them when the buffer was made
    posb, ropeb = ctx.buffer(pos), ctx.buffer(vals)
    qb, kb = ctx.buffer(q), ctx.buffer(k)
    pipe = _qk_pipeline(ctx)
    qp = hip.QkNormParams(tokens, heads, kv_heads, 128, qc, kc, *wl.ZIMAGE_DIMS, wl.ZIMAGE_EPS, q_off, k_off, *bases)
    rc = L.zdraw_hip_run_qk_norm_rope(ctx.queue, pipe, qb.handle, kb.handle, weights, weights, posb.handle, ropeb.handle,
                                      C.byref(qp), 256)
    assert rc == 0, hip.last_error()
    gq, gk = qb.read(np.float32, q.shape), kb.read(np.float32, k.shape)
    want_q = zo.zimage_rotate(zo.zimage_norm_heads(q, qdec(eq), wl.ZIMAGE_EPS), vals, cfg, pos.astype(np.uintp))
    want_k = zo.zimage_rotate(zo.zimage_norm_heads(k, kdec(ek), wl.ZIMAGE_EPS), vals, cfg, pos.astype(np.uintp))
    assert np.abs(gq - want_q).max() < 5e-6 * np.abs(want_q).max() + 2e-6
    assert np.abs(gk - want_k).max() < 5e-6 * np.abs(want_k).max() + 2e-6
    # an offset that splits an element is malformed: refused before anything runs
    d0 = L.zdraw_hip_dispatch_count()
    odd = hip.QkNormParams(tokens, heads, kv_heads, 128, qc, kc, *wl.ZIMAGE_DIMS, wl.ZIMAGE_EPS, q_off + 1, k_off, *bases)
    assert L.zdraw_hip_run_qk_norm_rope(ctx.queue, pipe, qb.handle, kb.handle, weights, weights, posb.handle,
                                        ropeb.handle, C.byref(odd), 256) == hip.INVALID
    assert L.zdraw_hip_dispatch_count() == d0
    L.zdraw_hip_release_pipeline(pipe)
    L.zdraw_hip_release_weight_buffer(weights)  # metal_c.zig:32
    for b in (posb, ropeb, qb, kb):
        b.release()


def test_wrap_device_memory_refuses_what_is_not_device_memory(ctx):
    L = hip.lib()
    d0 = L.zdraw_hip_dispatch_count()
    host_bytes = np.ones(4096, np.uint8)
    assert not L.zdraw_hip_wrap_device_memory(ctx.device, host_bytes.ctypes.data_as(C.c_void_p), host_bytes.size)
    assert b"wrap_device_memory" in L.zdraw_hip_last_error()
    assert not L.zdraw_hip_wrap_device_memory(ctx.device, None, 16)
    assert not L.zdraw_hip_wrap_device_memory(ctx.device, C.c_void_p(0x1000), 16)  # no allocation there
    own = ctx.buffer(nbytes=4096)
    ptr = L.zdraw_hip_buffer_device_ptr(own.handle)
    assert ptr
    whole = L.zdraw_hip_wrap_device_memory(ctx.device, ptr, 4096)
    inner = L.zdraw_hip_wrap_device_memory(ctx.device, ptr + 1024, 3072)
    assert whole and inner
    assert not L.zdraw_hip_wrap_device_memory(ctx.device, ptr, 4097)          # longer than the allocation
    assert not L.zdraw_hip_wrap_device_memory(ctx.device, ptr + 1024, 3073)   # runs past its end
    assert L.zdraw_hip_dispatch_count() == d0                                  # nothing was launched
    # the wrap is a view: bytes written through it are the owner's bytes, and releasing it frees nothing
    pattern = np.arange(3072, dtype=np.uint32).astype(np.uint8)
    L.zdraw_hip_write_buffer(inner, pattern.ctypes.data_as(C.c_void_p), pattern.size)
    L.zdraw_hip_release_buffer(inner)
    L.zdraw_hip_release_buffer(whole)
    assert np.array_equal(own.read(np.uint8, 4096)[1024:], pattern)
    own.release()


def _klein_case(seed):
    w = wl.by_name("klein_1024", seed=seed, small=True)
    w.k[0, 50] = w.q[0, 50]  # a key parallel to its own token's query: |w|^2 * sqrt(128) nats
    return w


def _klein_want(w, weight):
    rb = lambda a: host.bf16_bits_to_f32(host.f32_to_bf16_bits(a))
    wv = np.full(128, weight, np.float32)
    qn = zo.klein_apply_rope(zo.klein_rms_norm_heads(rb(w.q[0]), wv), w.rope_cos, w.rope_sin)
    kn = zo.klein_apply_rope(zo.klein_rms_norm_heads(rb(w.k[0]), wv), w.rope_cos, w.rope_sin)
    c = np.float32(1.4426950408889634 / np.sqrt(128.0))
    # operands as the MFMAs see them (the scores of the weight-3 case spread over a hundred nats)
    return zo.attention_run(rb(qn * c) / c, rb(kn), rb(w.v[0]), zo.Config(w.tokens, w.heads, w.heads, 128))


class _NoCopyView:
    def __init__(self, handle):
        self.handle = handle


def test_weights_that_change_behind_a_wrapper_never_take_the_bounded_form(ctx):
    # Norm weights in memory another runtime owns (a torch tensor), wrapped for the call. The
    # caller claims |q'.k'|/sqrt(128) <= 12, true while the weights are 0.5; then the other
    # runtime overwrites them with 3.0 (101 nats for the planted key) without telling anyone.
    # The library must not have kept a maximum for memory it does not own: the second call runs
    # the running-maximum form and stays finite and right.
    import torch
    L = hip.lib()
    w = _klein_case(31)
    tq = torch.full((128,), 0.5, dtype=torch.float32, device="cuda:0")
    tk = torch.full((128,), 0.5, dtype=torch.float32, device="cuda:0")
    torch.cuda.synchronize()
    hq = L.zdraw_hip_wrap_device_memory(ctx.device, tq.data_ptr(), 512)
    hk = L.zdraw_hip_wrap_device_memory(ctx.device, tk.data_ptr(), 512)
    assert hq and hk, hip.last_error()
    bufs = [ctx.buffer(host.f32_to_bf16_bits(a)) for a in (w.q, w.k, w.v)]
    cos, sin = ctx.buffer(w.rope_cos), ctx.buffer(w.rope_sin)

    def run(bound):
        o = ctx.buffer(nbytes=w.q.size * 2)
        ctx.joint_klein(bufs[0], bufs[1], bufs[2], o, tokens=w.tokens, heads=w.heads, norm_q=_NoCopyView(hq),
                        norm_k=_NoCopyView(hk), rope_cos=cos, rope_sin=sin, k_site=hip.K_PREPASS, score_bound=bound)
        out = host.bf16_bits_to_f32(o.read(np.uint16, w.q.shape))[0]
        o.release()
        return out

    refimpl.check_close(run(12.0), _klein_want(w, 0.5), "wrapped weights 0.5")
    tq.fill_(3.0)
    tk.fill_(3.0)
    torch.cuda.synchronize()
    big = run(12.0)
    assert np.isfinite(big).all()
    assert np.array_equal(big.view(np.uint32), run(0.0).view(np.uint32))  # the running-maximum build ran
    refimpl.check_close(big, _klein_want(w, 3.0), "wrapped weights 3.0")
    L.zdraw_hip_release_buffer(hq)
    L.zdraw_hip_release_buffer(hk)
    for b in bufs + [cos, sin]:
        b.release()


def test_an_owned_weight_buffer_whose_address_was_handed_out_is_not_cached_either(ctx):
    # the same through zdraw_hip_buffer_device_ptr: the library allocated the weights, took the
    # bounded form on them once (their maximum is then on record), handed their address out, and
    # someone wrote 3.0 there through another handle
    import torch
    L = hip.lib()
    w = _klein_case(32)
    half = np.full(128, 0.5, np.float32)
    wq, wk = ctx.buffer(half), ctx.buffer(half)
    bufs = [ctx.buffer(host.f32_to_bf16_bits(a)) for a in (w.q, w.k, w.v)]
    cos, sin = ctx.buffer(w.rope_cos), ctx.buffer(w.rope_sin)

    def run(bound):
        o = ctx.buffer(nbytes=w.q.size * 2)
        ctx.joint_klein(bufs[0], bufs[1], bufs[2], o, tokens=w.tokens, heads=w.heads, norm_q=wq, norm_k=wk,
                        rope_cos=cos, rope_sin=sin, k_site=hip.K_PREPASS, score_bound=bound)
        out = host.bf16_bits_to_f32(o.read(np.uint16, w.q.shape))[0]
        o.release()
        return out

    refimpl.check_close(run(12.0), _klein_want(w, 0.5), "owned weights 0.5")
    three = torch.full((128,), 3.0, dtype=torch.float32, device="cuda:0")
    for b in (wq, wk):
        # a device-to-device copy by the other runtime, behind the library's back
        _copy_to_device_ptr(three, L.zdraw_hip_buffer_device_ptr(b.handle))
    torch.cuda.synchronize()
    big = run(12.0)
    assert np.isfinite(big).all()
    assert np.array_equal(big.view(np.uint32), run(0.0).view(np.uint32))
    refimpl.check_close(big, _klein_want(w, 3.0), "owned weights overwritten with 3.0")
    for b in bufs + [cos, sin, wq, wk]:
        b.release()


def _copy_to_device_ptr(src, ptr):
    """Copies a device tensor's bytes to a raw device address with the HIP runtime itself
    (hipMemcpy, device to device): a write this library knows nothing about."""
    import torch
    hip.lib()
    rt = C.CDLL(None)  # the HIP runtime that libzdraw_hip.so brought into the process
    rt.hipMemcpy.restype = C.c_int
    rt.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
    torch.cuda.synchronize()
    assert rt.hipMemcpy(ptr, src.data_ptr(), src.numel() * src.element_size(), 3) == 0  # hipMemcpyDeviceToDevice


def test_read_buffer_any_is_ordered_after_the_queue(ctx):
    # metal_c.zig:24-29: the readback that waits for the queue's work; here inside an open batch,
    # before batch_end, it already sees the launch's output
    L = hip.lib()
    w = wl.by_name("klein_512_x4", seed=33, small=True)
    res = wl.Resident(ctx, w, dtype=hip.BF16, k_site=hip.K_PREPASS)
    want = res.run()
    res.o.write(np.zeros(res.o.nbytes, np.uint8))
    b = L.zdraw_hip_batch_begin(ctx.queue)
    assert res.launch(b) == 0, hip.last_error()
    raw = np.empty(res.o.nbytes // 2, np.uint16)
    assert L.zdraw_hip_read_buffer_any(ctx.queue, res.o.handle, raw.ctypes.data_as(C.c_void_p), raw.nbytes) == 0
    assert L.zdraw_hip_batch_end(b) == 0
    assert np.array_equal(host.bf16_bits_to_f32(raw.reshape(want.shape)).view(np.uint32), want.view(np.uint32))
    assert L.zdraw_hip_read_buffer_any(ctx.queue, res.o.handle, raw.ctypes.data_as(C.c_void_p), res.o.nbytes + 1) == hip.ERR_HANDLE
    assert L.zdraw_hip_read_buffer_any(None, res.o.handle, raw.ctypes.data_as(C.c_void_p), 16) == hip.ERR_HANDLE
    res.release()
