"""Pins the oracle's QK-norm / rope / position helpers (oracle/klein_qk.c,
oracle/zimage_qk.c) against the reference's own known-answer tests, closed
forms and rotation identities."""
import numpy as np
import pytest

from oracle import zoracle as zo


# ======================================================================= Klein
def test_klein_rope_closed_form_and_structure():
    # klein/zflux2_dit.zig:125-170
    txt, gh, gw, rh, rw, theta = 8, 3, 5, 2, 4, 2000.0
    cos, sin = zo.klein_build_rope_ref(gh, gw, rh, rw, theta=theta, txt_len=txt)
    assert cos.shape == (txt + gh * gw + rh * rw, 128)
    # pair duplication
    assert np.array_equal(cos[:, 0::2], cos[:, 1::2]) and np.array_equal(sin[:, 0::2], sin[:, 1::2])
    freq = theta ** (-2.0 * np.arange(16) / 32.0)
    # text rows: axes 0..2 identity, axis 3 carries the token index
    for t in (0, 1, 7):
        assert np.all(cos[t, :96] == 1.0) and np.all(sin[t, :96] == 0.0)
        assert np.allclose(cos[t, 96::2], np.cos(t * freq), atol=1e-7)
        assert np.allclose(sin[t, 96::2], np.sin(t * freq), atol=1e-7)
    # image rows: axes 0 and 3 identity, axis 1 = row, axis 2 = column
    for p in (0, 4, 5, 14):
        t = txt + p
        r, c = divmod(p, gw)
        assert np.all(cos[t, :32] == 1.0) and np.all(cos[t, 96:] == 1.0)
        assert np.all(sin[t, :32] == 0.0) and np.all(sin[t, 96:] == 0.0)
        assert np.allclose(cos[t, 32:64:2], np.cos(r * freq), atol=1e-7)
        assert np.allclose(sin[t, 64:96:2], np.sin(c * freq), atol=1e-7)
    # reference-image rows: T axis id 10, own grid
    for p in (0, 3, 7):
        t = txt + gh * gw + p
        r, c = divmod(p, rw)
        assert np.allclose(cos[t, 0:32:2], np.cos(10 * freq), atol=1e-7)
        assert np.allclose(sin[t, 0:32:2], np.sin(10 * freq), atol=1e-7)
        assert np.allclose(sin[t, 32:64:2], np.sin(r * freq), atol=1e-7)
        assert np.allclose(cos[t, 64:96:2], np.cos(c * freq), atol=1e-7)
        assert np.all(cos[t, 96:] == 1.0)


def test_klein_rope_no_reference_grid_matches_build_rope():
    # buildRope == buildRopeRef(.., 0, 0, ..) (klein/zflux2_dit.zig:110-117)
    a = zo.klein_build_rope_ref(4, 4, 0, 0, theta=10000.0, txt_len=16)
    b = zo.klein_build_rope_ref(4, 4, 2, 2, theta=10000.0, txt_len=16)
    assert a[0].shape[0] == 32 and np.array_equal(a[0], b[0][:32]) and np.array_equal(a[1], b[1][:32])


def test_klein_f64_frequency_precision():
    # frequencies are evaluated in f64 then cast: compare a far position
    cos, sin = zo.klein_build_rope_ref(1, 1, theta=2000.0, txt_len=512)
    t = 511
    i = 15
    arg = np.float64(t) * (1.0 / np.power(np.float64(2000.0), np.float64(2 * i) / 32.0))
    assert cos[t, 96 + 2 * i] == np.float32(np.cos(arg))
    assert sin[t, 96 + 2 * i] == np.float32(np.sin(arg))


def test_klein_rms_norm_vector_and_invariants():
    # runtime/ops.zig:151-163: (3,4), gains (1,2), eps 0 -> (0.8485, 2.2627); the
    # 128-wide Klein form has the same mean square when the pair is tiled 64x
    # (eps 1e-6 against a mean square of 12.5 is below the tolerance).
    x = np.tile(np.array([3.0, 4.0], np.float32), 64).reshape(1, 1, 128)
    w = np.tile(np.array([1.0, 2.0], np.float32), 64)
    y = zo.klein_rms_norm_heads(x, w)
    assert np.abs(y[0, 0, 0::2] - 0.8485).max() < 1e-4 and np.abs(y[0, 0, 1::2] - 2.2627).max() < 1e-4
    rng = np.random.default_rng(0)
    x = rng.standard_normal((5, 3, 128), dtype=np.float32)
    y = zo.klein_rms_norm_heads(x, np.ones(128, np.float32))
    assert np.allclose(np.sqrt((y.astype(np.float64) ** 2).mean(-1)), 1.0, atol=1e-5)
    y2 = zo.klein_rms_norm_heads(x * 7.5, np.ones(128, np.float32))
    assert np.allclose(y, y2, atol=1e-5)
    # learned weight multiplies element-wise
    w = rng.standard_normal(128).astype(np.float32)
    assert np.allclose(zo.klein_rms_norm_heads(x, w), y * w, atol=1e-5)
    # eps 1e-6 matters for a tiny row: inv = 1/sqrt(ss/128 + 1e-6)
    tiny = np.full((1, 1, 128), 1e-4, np.float32)
    want = 1e-4 / np.sqrt(1e-8 + 1e-6)
    assert np.allclose(zo.klein_rms_norm_heads(tiny, np.ones(128, np.float32)), want, rtol=1e-5)


def test_klein_apply_rope_identities():
    rng = np.random.default_rng(1)
    txt, gh, gw = 4, 6, 7
    cos, sin = zo.klein_build_rope_ref(gh, gw, theta=10000.0, txt_len=txt)
    tokens = txt + gh * gw
    x = rng.standard_normal((tokens, 2, 128), dtype=np.float32)
    y = zo.klein_apply_rope(x, cos, sin)
    # position (0,0,0,0) is the identity: text token 0
    assert np.array_equal(y[0], x[0])
    # pair norms preserved
    nx = x[..., 0::2] ** 2 + x[..., 1::2] ** 2
    ny = y[..., 0::2] ** 2 + y[..., 1::2] ** 2
    assert np.allclose(nx, ny, rtol=1e-4, atol=1e-5)
    # explicit complex rotation: (x0 + i x1) * (c + i s)
    z = (x[..., 0::2] + 1j * x[..., 1::2]) * (cos[:, None, 0::2] + 1j * sin[:, None, 0::2])
    assert np.allclose(y[..., 0::2], z.real, atol=1e-5) and np.allclose(y[..., 1::2], z.imag, atol=1e-5)
    # relative-position property along the column axis: <R(p)q, R(p')k> depends on p - p'
    q = rng.standard_normal(128).astype(np.float32)
    k = rng.standard_normal(128).astype(np.float32)

    def rot(vec, tok):
        arr = np.zeros((tokens, 1, 128), np.float32)
        arr[tok, 0] = vec
        return zo.klein_apply_rope(arr, cos, sin)[tok, 0].astype(np.float64)

    row = txt + 2 * gw
    d1 = rot(q, row + 1) @ rot(k, row + 4)
    d2 = rot(q, row + 2) @ rot(k, row + 5)
    assert abs(d1 - d2) < 1e-3
    d3 = rot(q, row + 1) @ rot(k, row + 5)
    assert abs(d1 - d3) > 1e-3
    # a swapped-sign mistake (x0*c + x1*s) would turn the rotation into its inverse:
    zinv = (x[..., 0::2] + 1j * x[..., 1::2]) * (cos[:, None, 0::2] - 1j * sin[:, None, 0::2])
    assert np.abs(y[txt + 9:, :, 0::2] - zinv.real[txt + 9:]).max() > 1e-2


def test_klein_rope_uses_both_table_columns():
    # the reference reads c[i], s[i] for the even lane and c[i+1], s[i+1] for the odd
    x = np.ones((1, 1, 128), np.float32)
    cos = np.zeros((1, 128), np.float32)
    sin = np.zeros((1, 128), np.float32)
    cos[0, 0], cos[0, 1], sin[0, 0], sin[0, 1] = 2.0, 3.0, 5.0, 7.0
    y = zo.klein_apply_rope(x, cos, sin)
    assert y[0, 0, 0] == 2.0 - 5.0 and y[0, 0, 1] == 3.0 + 7.0


# ===================================================================== Z-Image
def test_zrope_position_zero_identity():
    # zimage/zrope.zig:142-151
    c = zo.RopeConfig((2, 2, 2), (2, 2, 2), 256.0)
    vals = zo.zrope_fill(c)
    vec = zo.zrope_apply(vals, c, [1, 2, 3, 4, 5, 6], (0, 0, 0))
    assert np.array_equal(vec, np.array([1, 2, 3, 4, 5, 6], np.float32))


def test_zrope_rotates_adjacent_pair_one_axis():
    # zimage/zrope.zig:153-165
    c = zo.RopeConfig((2, 2, 2), (3, 2, 2), 1.0)
    vals = zo.zrope_fill(c)
    vec = zo.zrope_apply(vals, c, [1, 2, 3, 4, 5, 6], (1, 0, 0))
    assert abs(vec[0] - (np.cos(1.0) - 2.0 * np.sin(1.0))) < 1e-4
    assert abs(vec[1] - (2.0 * np.cos(1.0) + np.sin(1.0))) < 1e-4
    assert np.array_equal(vec[2:], np.array([3, 4, 5, 6], np.float32))


def test_zrope_pair_frequency_exponent():
    # zimage/zrope.zig:167-180
    c = zo.RopeConfig((4, 2, 2), (3, 1, 1), 100.0)
    vals = zo.zrope_fill(c)
    vec = zo.zrope_apply(vals, c, [1, 0, 0, 1, 5, 6, 7, 8], (2, 0, 0))
    assert abs(vec[0] - np.cos(2.0)) < 1e-4 and abs(vec[1] - np.sin(2.0)) < 1e-4
    assert abs(vec[2] + np.sin(0.2)) < 1e-4 and abs(vec[3] - np.cos(0.2)) < 1e-4


def test_zrope_errors_and_layout():
    with pytest.raises(zo.OracleError) as e:
        zo.zrope_check(zo.RopeConfig((2, 3, 2), (1, 1, 1), 10.0))
    assert e.value.code == zo.INVALID_CONFIG
    with pytest.raises(zo.OracleError):
        zo.zrope_check(zo.RopeConfig((2, 2, 2), (1, 1, 1), 0.0))
    c = zo.RopeConfig((32, 48, 48), (1536, 512, 512), 256.0)
    vals = zo.zrope_fill(c)
    assert vals.shape == (1536 * 16 + 512 * 24 + 512 * 24, 2)
    assert zo.zrope_axis_bases(c) == (0, 1536 * 16, 1536 * 16 + 512 * 24)
    with pytest.raises(zo.OracleError) as e:
        zo.zrope_apply(vals, c, np.zeros(128), (1536, 0, 0))
    assert e.value.code == zo.BAD_POSITION
    with pytest.raises(zo.OracleError) as e:
        zo.zrope_apply(vals, c, np.zeros(127), (0, 0, 0))
    assert e.value.code == zo.INVALID_SHAPE
    # closed form of one entry: axis 1, pos 37, pair 5: angle = 37 * 256^(-10/48)
    b1 = 1536 * 16
    ang = np.float32(37.0) * np.exp(-np.log(np.float32(256.0)) * np.float32(10.0 / 48.0))
    assert np.allclose(vals[b1 + 37 * 24 + 5], [np.cos(ang), np.sin(ang)], atol=2e-6)


def test_zrope_full_head_matches_complex_rotation():
    rng = np.random.default_rng(3)
    c = zo.RopeConfig((32, 48, 48), (1536, 512, 512), 256.0)
    vals = zo.zrope_fill(c)
    vec = rng.standard_normal(128).astype(np.float32)
    pos = (513, 17, 63)
    got = zo.zrope_apply(vals, c, vec, pos)
    want = np.zeros(128)
    off = 0
    for ax, dim in enumerate(c.dims):
        pairs = np.arange(dim // 2)
        ang = pos[ax] * np.exp(-np.log(256.0) * 2.0 * pairs / dim)
        z = (vec[off:off + dim:2] + 1j * vec[off + 1:off + dim:2]) * np.exp(1j * ang)
        want[off:off + dim:2], want[off + 1:off + dim:2] = z.real, z.imag
        off += dim
    assert np.allclose(got, want, atol=5e-4)  # fp32 angle at pos 513


def test_rms_norm_reference_vector():
    # runtime/ops.zig:151-163
    out = zo.rms_norm([3.0, 4.0], [1.0, 2.0], 0.0)
    assert abs(out[0] - 0.8485) < 1e-4 and abs(out[1] - 2.2627) < 1e-4
    with pytest.raises(zo.OracleError):
        zo.rms_norm(np.zeros(0, np.float32), np.zeros(0, np.float32), 0.0)


def test_read_f32_decodes_reference_bytes():
    # runtime/ops.zig:137-149 and :165-174: f16 bytes 0x4200.. = 3,4,5,6; 0x3c00 = 1, 0x4000 = 2
    for raw, want in ((b"\x00\x42", 3.0), (b"\x00\x44", 4.0), (b"\x00\x45", 5.0), (b"\x00\x46", 6.0),
                      (b"\x00\x3c", 1.0), (b"\x00\x40", 2.0)):
        assert zo.read_f32(1, raw) == want
    assert zo.read_f32(3, b"\x07") == 7.0
    rng = np.random.default_rng(4)
    halfs = rng.integers(0, 1 << 16, 400, dtype=np.uint16)
    for h in halfs:
        want = np.array([h], np.uint16).view(np.float16)[0].astype(np.float32)
        got = np.float32(zo.read_f32(1, int(h).to_bytes(2, "little")))
        assert (np.isnan(want) and np.isnan(got)) or want == got
        wantb = np.array([int(h) << 16], np.uint32).view(np.float32)[0]
        gotb = np.float32(zo.read_f32(2, int(h).to_bytes(2, "little")))
        assert (np.isnan(wantb) and np.isnan(gotb)) or wantb == gotb
    assert zo.read_f32(0, np.float32(1.25).tobytes()) == 1.25


def test_zimage_attention_step_single_token():
    # zimage/zattn_test.zig:9-51 with identity projections: norm -> head norm ->
    # rope at pos 0 -> one-token attention returns V = normed input = ones.
    x = np.ones((1, 1, 6), np.float32)
    c = zo.RopeConfig((2, 2, 2), (1, 1, 1), 256.0)
    vals = zo.zrope_fill(c)
    normed = zo.zimage_norm_heads(x, np.ones(6, np.float32), 0.0)  # block RMSNorm, eps 0
    qk = zo.zimage_norm_heads(normed, np.ones(6, np.float32), 0.0)
    qk = zo.zimage_rotate(qk, vals, c, [(0, 0, 0)])
    out = zo.attention_run(qk, qk, normed, zo.Config(1, 1, 1, 6))
    assert np.array_equal(out.ravel(), np.ones(6, np.float32))


def test_zseq_helpers():
    # zimage/zseq.zig:94-133
    assert zo.zseq_pad_len(32) == 0 and zo.zseq_pad_len(2) == 30 and zo.zseq_padded_len(33) == 64
    ids = zo.zseq_grid((1, 2, 2), (5, 0, 0))
    assert ids.tolist() == [[5, 0, 0], [5, 0, 1], [5, 1, 0], [5, 1, 1]]
    with pytest.raises(zo.OracleError):
        zo.zseq_grid((1, 2, 2), (0, 0, 0), out_len=3)
    out, ids, mask, total = zo.zseq_pad_with_ids([1.0, 2.0, 3.0, 4.0], 2, (1, 1, 2), (7, 0, 0))
    assert total == 32
    assert out[:2].ravel().tolist() == [1, 2, 3, 4] and out[2].tolist() == [3, 4]
    assert ids[1].tolist() == [7, 0, 1] and ids[2].tolist() == [0, 0, 0]
    assert not mask[1] and mask[2]


def test_zunify_places_image_before_caption():
    # zimage/zunify.zig:47-66
    out, pos, span = zo.zunify_basic([1, 2, 3, 4], [(10, 0, 0), (11, 0, 0)], [5, 6], [(1, 0, 0)], 2)
    assert out.ravel().tolist() == [1, 2, 3, 4, 5, 6]
    assert pos[0].tolist() == [10, 0, 0] and pos[2].tolist() == [1, 0, 0]
    assert span["image_len"] == 2 and span["total"] == 3


def test_zimage_positions_for_the_1024_workload():
    # zimage/zstep_shape.zig:58-66: caption grid (cap_total,1,1) from (1,0,0);
    # image grid from (cap_total+1, 0, 0); sequence = image then caption.
    cap_total, gh, gw = 512, 64, 64
    img = zo.zseq_grid((1, gh, gw), (cap_total + 1, 0, 0))
    cap = zo.zseq_grid((cap_total, 1, 1), (1, 0, 0))
    assert img[0].tolist() == [513, 0, 0] and img[-1].tolist() == [513, 63, 63]
    assert cap[0].tolist() == [1, 0, 0] and cap[-1].tolist() == [512, 0, 0]
    assert img[:, 0].max() < 1536 and cap[:, 0].max() < 1536
