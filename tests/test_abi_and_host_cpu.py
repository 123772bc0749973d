"""CPU-only checks of the boundary: the C-ABI library loads and exports every
declared symbol, struct sizes match the header, and the host layer's error
behaviour without a device follows the reference's contract. No GPU compute."""
import ctypes as C
import os
import re

import numpy as np
import pytest

from oracle import zoracle as zo
from zdraw_amd import hip, host, workloads as wl

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_symbols():
    """Every function include/*.h declares (the boundary and the measurement aids)."""
    names = set()
    inc = os.path.join(ROOT, "include")
    headers = sorted(f for f in os.listdir(inc) if f.endswith(".h"))
    assert "zdraw_hip.h" in headers and "zdraw_hip_measure.h" in headers
    for h in headers:
        text = open(os.path.join(inc, h)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names |= set(re.findall(r"\b(zdraw_hip_[a-z0-9_]+)\s*\(", text))
    return sorted(names)


def test_library_exports_every_declared_symbol():
    L = hip.lib()
    declared = header_symbols()
    assert len(declared) >= 35
    for name in declared:
        assert hasattr(L, name), f"libzdraw_hip.so lacks {name}"
    # the Python binding table and the header agree
    assert sorted(hip.SYMBOLS) == declared


def test_abi_struct_sizes():
    L = hip.lib()
    # AttnParams must stay 24 bytes (runtime/abi_assert.zig:29)
    assert L.zdraw_hip_abi_sizeof(0) == 24 == C.sizeof(hip.AttnParams)
    assert L.zdraw_hip_abi_sizeof(1) == C.sizeof(hip.AttnExt) == 216
    assert L.zdraw_hip_abi_sizeof(2) == C.sizeof(hip.QkOperands) == 72
    # GemmParams keeps the reference's 32-byte layout (metal_c.zig:276-283)
    assert L.zdraw_hip_abi_sizeof(3) == C.sizeof(hip.GemmParams) == 32
    assert hip.GemmParams.weight_offset.offset == 24
    assert L.zdraw_hip_abi_sizeof(4) == C.sizeof(hip.GemmExt) == 48
    # QkNormParams keeps the reference's 80 bytes (metal_c.zig:258-274); in the chain
    # parameters qk follows three GemmParams and proj sits 104 bytes after qk, as in
    # ZdrawBlockChainParams (metal_api.m:6007-6008: qk at 128, proj at 232)
    assert L.zdraw_hip_abi_sizeof(5) == C.sizeof(hip.QkNormParams) == 80
    assert hip.QkNormParams.q_offset.offset == 40 and hip.QkNormParams.base0.offset == 56
    assert L.zdraw_hip_abi_sizeof(6) == C.sizeof(hip.ChainAttnBuffers) == 48
    assert L.zdraw_hip_abi_sizeof(7) == C.sizeof(hip.ChainAttnWeights) == 64
    assert L.zdraw_hip_abi_sizeof(8) == C.sizeof(hip.ChainAttnParams) == 240
    assert hip.ChainAttnParams.proj.offset - hip.ChainAttnParams.qk.offset == 232 - 128
    text = open(os.path.join(ROOT, "include", "zdraw_hip.h")).read()
    assert "#define ZDRAW_HIP_ABI_QK_NORM_PARAMS_SIZE 80" in text
    assert "#define ZDRAW_HIP_ABI_CHAIN_ATTN_PARAMS_SIZE 240" in text
    assert "#define ZDRAW_HIP_ABI_ATTN_PARAMS_SIZE 24" in text
    assert "#define ZDRAW_HIP_ABI_ATTN_EXT_SIZE 216" in text
    assert "#define ZDRAW_HIP_ABI_QK_OPERANDS_SIZE 72" in text
    assert "#define ZDRAW_HIP_ABI_GEMM_PARAMS_SIZE 32" in text
    assert "#define ZDRAW_HIP_ABI_GEMM_EXT_SIZE 48" in text


def test_gemm_tail_plan_of_the_projection_shapes():
    # 256 CUs, 256 x 256 tiles of C: which last rounds of the projections are split along k
    L = hip.lib()

    def plan(m, k, n, groups=1, cus=256):
        t, s = C.c_uint32(99), C.c_uint32(99)
        L.zdraw_hip_gemm_tail_plan(m, k, n, groups, cus, C.byref(t), C.byref(s))
        return t.value, s.value

    assert plan(4608, 3072, 9216) == (0, 1)          # Klein q/k/v: 648 tiles, a tail of 136 stays whole
    assert plan(4608, 3840, 3840, 3) == (42, 6)      # Z-Image q/k/v group: 810 tiles = 3 rounds + 42
    assert plan(4608, 3840, 3840) == (14, 8)         # Z-Image out projection: 270 tiles, never more than 8 parts
    assert plan(4608, 12288, 3072) == (0, 1)         # 216 tiles: one partly filled round, nothing before it to balance
    assert plan(512, 3072, 9216) == (0, 1)           # fewer than 160 tiles: the 128-tile build
    assert plan(4322, 1216, 4090) == (16, 4)         # 272 tiles, 19 slabs: at least four slabs per part
    assert plan(4322, 128, 4090) == (0, 1)           # two slabs: too short to split
    assert plan(4322, 1220, 4090) == (0, 1)          # k not a multiple of 64: another build
    assert plan(4608, 3840, 3840, 3, cus=0) == (0, 1) and plan(0, 64, 64) == (0, 1)
    for mt in range(10, 40):                         # invariants
        t, s = plan(mt * 256, 2048, 16 * 256)
        tiles = mt * 16
        assert (t == 0 and s == 1) or (tiles >= 160 and t == tiles % 256 and 2 <= s <= 8 and t * s <= 256 and 32 // s >= 4)


def test_tail_plan_of_the_baseline_shapes():
    # 256 CUs, one 256-row tile per workgroup: which last rounds are split along the keys
    L = hip.lib()

    def plan(tiles, key_blocks, cus=256):
        t, s = C.c_uint32(99), C.c_uint32(99)
        L.zdraw_hip_attention_tail_plan(tiles, cus, key_blocks, C.byref(t), C.byref(s))
        return t.value, s.value

    assert plan(18 * 24, 144) == (0, 1)        # Klein 1024^2: 432 tiles, a tail of 176 stays whole
    assert plan(18 * 30, 144) == (28, 9)       # Z-Image 1024^2: 540 tiles = 2 rounds + 28
    assert plan(6 * 24 * 4, 48) == (64, 4)     # Klein 512^2 x 4: 576 tiles = 2 rounds + 64
    assert plan(34 * 24 * 2, 272) == (96, 2)   # ragged edit: 1632 tiles = 6 rounds + 96
    assert plan(512, 144) == (0, 1)            # whole rounds
    assert plan(6, 10) == (0, 1)               # too few key blocks to split (8 per part)
    assert plan(6, 64) == (6, 8)               # a small launch spreads over the chip, 8 blocks per part
    assert plan(2, 1024) == (2, 16)            # never more than 16 parts
    assert plan(129, 144) == (0, 1)            # a tail above half the CUs stays whole
    assert plan(128, 144) == (128, 2)
    assert plan(0, 144) == (0, 1) and plan(10, 144, cus=0) == (0, 1)
    for tiles in range(1, 700, 7):             # invariants
        t, s = plan(tiles, 144)
        assert (t == 0 and s == 1) or (t == tiles % 256 and 2 <= s <= 16 and t * s <= 256 and 144 // s >= 8)


def test_zimage_axis_lens_are_the_positions_the_pair_table_holds():
    # what the kernels hold device-resident positions to (the reference refuses pos >= len
    # on the host, zimage/zrope.zig:48): for zrope.Cache's layout the counts are its lens
    L = hip.lib()

    def lens_of(table_pairs, bases, dims):
        out = (C.c_uint32 * 3)(7, 7, 7)
        rc = L.zdraw_hip_zimage_axis_lens(table_pairs * 8, (C.c_uint64 * 3)(*bases), (C.c_uint32 * 3)(*dims), out)
        return rc, tuple(out)

    cfg = zo.RopeConfig(wl.ZIMAGE_DIMS, wl.ZIMAGE_LENS, wl.ZIMAGE_THETA)
    bases = zo.zrope_axis_bases(cfg)
    pairs = zo.zrope_fill(cfg).shape[0]
    assert lens_of(pairs, bases, wl.ZIMAGE_DIMS) == (0, tuple(wl.ZIMAGE_LENS))
    # the last position of every axis ends inside the table, the one after it does not
    order = sorted(range(3), key=lambda a: bases[a])
    for a in range(3):
        per = wl.ZIMAGE_DIMS[a] // 2
        nxt = min([bases[b] for b in range(3) if bases[b] > bases[a]] + [pairs])
        assert bases[a] + wl.ZIMAGE_LENS[a] * per <= nxt < bases[a] + (wl.ZIMAGE_LENS[a] + 1) * per
    assert order == [0, 1, 2]
    # small cases by hand: axes of 2, 4, 4 pairs per position
    assert lens_of(2 * 3 + 4 * 5 + 4 * 2, (0, 6, 26), (4, 8, 8)) == (0, (3, 5, 2))
    assert lens_of(2 * 3 + 4 * 5 + 4 * 2 + 3, (0, 6, 26), (4, 8, 8)) == (0, (3, 5, 2))   # a partial position does not count
    assert lens_of(34, (26, 0, 20), (8, 8, 4)) == (0, (2, 5, 3))                          # axes in any order
    assert lens_of(29, (0, 6, 26), (4, 8, 8))[0] == hip.INVALID                           # last axis has no whole position
    assert lens_of(26, (0, 6, 26), (4, 8, 8))[0] == hip.INVALID                           # base at the end of the table
    assert lens_of(40, (0, 6, 26), (4, 0, 8))[0] == hip.INVALID                           # an axis without pairs
    assert L.zdraw_hip_zimage_axis_lens(64, None, None, None) == hip.ERR_HANDLE


def test_pipeline_lookup_without_device_is_null():
    L = hip.lib()
    err = C.create_string_buffer(128)
    assert not L.zdraw_hip_compile(None, None, b"attention_block_mfma", err, 128)


def _has_gpu():
    return os.path.exists("/dev/kfd")


@pytest.mark.skipif(_has_gpu(), reason="device present")
def test_context_init_reports_not_available_without_device():
    # mattn_test.zig:9-12: error.MetalNotAvailable is how "no device" surfaces
    with pytest.raises(host.NotAvailable):
        host.Context.init()


def _oracle_cpu(out, q, k, v, scratch, cfg):
    try:
        res = zo.attention_run(q, k, v, zo.Config(cfg.tokens, cfg.heads, cfg.kv_heads, cfg.head_dim,
                                                  cfg.causal, cfg.valid), scratch_len=scratch.size)
    except zo.OracleError:
        return 1
    out[:] = res.ravel()
    return 0


def test_attention_fast_without_backend_uses_callers_cpu_kernel():
    # runtime/attention_fast.zig:15-23: metal == null -> attention.run
    rng = np.random.default_rng(0)
    cfg = host.Config(5, 2, 1, 8, causal=True)
    q = rng.standard_normal((5, 2, 8), dtype=np.float32)
    k = rng.standard_normal((5, 1, 8), dtype=np.float32)
    v = rng.standard_normal((5, 1, 8), dtype=np.float32)
    got = host.attention_fast_run(None, q, k, v, cfg, cpu=_oracle_cpu)
    want = zo.attention_run(q, k, v, zo.Config(5, 2, 1, 8, True))
    assert np.array_equal(got, want)


def test_attention_fast_without_backend_and_without_cpu_fails_loudly():
    cfg = host.Config(4, 1, 1, 128)
    z = np.zeros((4, 1, 128), np.float32)
    with pytest.raises(host.NotAvailable):
        host.attention_fast_run(None, z, z, z, cfg, cpu=None)


def test_attention_fast_propagates_cpu_shape_error():
    cfg = host.Config(4, 1, 1, 8)
    z = np.zeros((4, 1, 8), np.float32)
    with pytest.raises(host.InvalidShape):
        host.attention_fast_run(None, z, z, z, cfg, cpu=_oracle_cpu, scratch_len=1)


def test_host_rope_tables_match_oracle_bitwise():
    c, s = host.klein_build_rope_ref(5, 7, 2, 3, theta=2000.0, txt_len=16)
    c2, s2 = zo.klein_build_rope_ref(5, 7, 2, 3, theta=2000.0, txt_len=16)
    assert np.array_equal(c, c2) and np.array_equal(s, s2)
    c, s = host.klein_build_rope_ref(64, 64, theta=10000.0)
    c2, s2 = zo.klein_build_rope_ref(64, 64, theta=10000.0)
    assert c.shape == (4608, 128) and np.array_equal(c, c2) and np.array_equal(s, s2)
    vals, bases = host.zimage_rope_fill(wl.ZIMAGE_DIMS, wl.ZIMAGE_LENS, wl.ZIMAGE_THETA)
    cfg = zo.RopeConfig(wl.ZIMAGE_DIMS, wl.ZIMAGE_LENS, wl.ZIMAGE_THETA)
    assert np.array_equal(vals, zo.zrope_fill(cfg)) and bases == zo.zrope_axis_bases(cfg)
    with pytest.raises(host.InvalidShape):
        host.zimage_rope_fill((2, 3, 2), (1, 1, 1), 10.0)
    with pytest.raises(host.InvalidShape):
        host.zimage_rope_fill((2, 2, 2), (1, 1, 1), 0.0)


def test_host_positions_follow_reference_sequence_order():
    pos = host.zimage_sequence_positions(64, 64, 512)
    assert pos.shape == (4608, 3)
    assert np.array_equal(pos[:4096], zo.zseq_grid((1, 64, 64), (513, 0, 0)))
    assert np.array_equal(pos[4096:], zo.zseq_grid((512, 1, 1), (1, 0, 0)))
    # padding: 7x9 image -> 64 slots, 33 caption tokens -> 64 slots
    pos = host.zimage_sequence_positions(7, 9, 33)
    assert pos.shape == (128, 3)
    assert pos[62].tolist() == [65, 6, 8] and pos[63].tolist() == [0, 0, 0]
    assert pos[64].tolist() == [1, 0, 0] and pos[127].tolist() == [64, 0, 0]


def test_bf16_rounding_helper_is_round_to_nearest_even():
    x = np.array([1.0, 1.00390625, 1.01171875, -3.0e-39, 3.3e38], np.float32)
    bits = host.f32_to_bf16_bits(x)
    back = host.bf16_bits_to_f32(bits)
    assert back[0] == 1.0
    assert back[1] == 1.0            # 1 + 2^-8 is a tie -> even mantissa (1.0)
    assert back[2] == 1.015625       # 1 + 3*2^-8 is a tie -> even mantissa (1 + 2^-6)
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(0)
    y = rng.standard_normal(10000).astype(np.float32) * 100
    want = torch.from_numpy(y).to(torch.bfloat16).float().numpy()
    assert np.array_equal(host.bf16_bits_to_f32(host.f32_to_bf16_bits(y)), want)


def test_workload_flops_match_the_published_work_figures():
    # 4 * S^2 * D * H (cmd/gemmbench.zig:5887): 260.92 GFLOP at Klein 1024^2
    def flops(tokens, heads, batch=1, keys=None):
        keys = [tokens] * batch if keys is None else keys
        return 4.0 * 128 * heads * sum(tokens * k for k in keys)
    assert abs(flops(4608, 24) / 1e9 - 260.92) < 0.01
    assert abs(flops(1536, 24, 4) / 1e9 - 115.96) < 0.01
    assert abs(flops(4608, 30) / 1e9 - 326.15) < 0.01
    assert abs(flops(8704, 24, 2, [8704 - 435, 8704 - 212]) / 1e9 - 1792.67) < 0.01
    w = wl.by_name("klein_edit_ragged", small=True)
    assert w.key_pad.shape == (2, w.tokens) and w.key_pad[0, 13:200].all() and not w.key_pad[0, :13].any()
    assert w.flops == 4.0 * 128 * w.heads * w.tokens * ((w.tokens - 187) + (w.tokens - 50))
    w1 = wl.by_name("klein_1024", seed=3, small=True)
    w2 = wl.by_name("klein_1024", seed=3, small=True)
    assert np.array_equal(w1.q, w2.q) and np.array_equal(w1.v, w2.v)
