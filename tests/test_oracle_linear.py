"""The linear oracle (oracle/linear_ref.c) against the reference's own known
answers and against what the mathematics fixes. CPU only."""
import numpy as np
import pytest

from oracle import zoracle as zo

# metal/mlinear_test.zig:9-19: the reference's weight fixtures, as bytes
F16_WEIGHT_BYTES = bytes([0x00, 0x3C, 0x00, 0x40, 0x00, 0x42, 0x00, 0x44])
F32_WEIGHT_BYTES = bytes([0x00, 0x00, 0x80, 0x3F, 0x00, 0x00, 0x00, 0x40,
                          0x00, 0x00, 0x40, 0x40, 0x00, 0x00, 0x80, 0x40])


def _decode(dtype, raw, shape):
    width = {zo.DT_F32: 4, zo.DT_F16: 2, zo.DT_BF16: 2}[dtype]
    vals = [zo.read_f32(dtype, raw[i:i + width]) for i in range(0, len(raw), width)]
    return np.array(vals, np.float32).reshape(shape)


def test_small_f16_matrix_known_answer():
    # mlinear_test.zig:33-46: [[1,2],[3,4]] (f16) x [1,2] = [5, 11]
    w = _decode(zo.DT_F16, F16_WEIGHT_BYTES, (2, 2))
    assert w.tolist() == [[1.0, 2.0], [3.0, 4.0]]
    out = zo.linear_batch([[1.0, 2.0]], w)
    assert out.tolist() == [[5.0, 11.0]]


def test_batched_rows_known_answers():
    # mlinear_test.zig:48-65: five rows (1,2), (3,4), ... -> (x0 + 2 x1, 3 x0 + 4 x1)
    w = _decode(zo.DT_F16, F16_WEIGHT_BYTES, (2, 2))
    x = np.arange(1, 11, dtype=np.float32).reshape(5, 2)
    out = zo.linear_batch(x, w)
    for item in range(5):
        x0, x1 = x[item]
        assert out[item, 0] == x0 + 2.0 * x1 and out[item, 1] == 3.0 * x0 + 4.0 * x1


def test_f32_weights_known_answer():
    # mlinear_test.zig:67-80: the same matrix as f32, input (2, 3) -> (8, 18)
    w = _decode(zo.DT_F32, F32_WEIGHT_BYTES, (2, 2))
    assert zo.linear_batch([[2.0, 3.0]], w).tolist() == [[8.0, 18.0]]


def _bf16_case():
    # mlinear_test.zig:82-121: m=32, k=8, n=32; input (i % 7) * 0.1 - 0.3; weight = bf16
    # truncation (high 16 bits) of (i % 11) * 0.05 - 0.25
    m, k, n = 32, 8, 32
    x = (np.arange(m * k) % 7).astype(np.float32) * np.float32(0.1) - np.float32(0.3)
    raw = (np.arange(n * k) % 11).astype(np.float32) * np.float32(0.05) - np.float32(0.25)
    hi = (raw.view(np.uint32) >> 16).astype(np.uint16)
    return x.reshape(m, k), raw, hi.reshape(n, k)


def test_bf16_ffn_shaped_case_matches_the_reference_loop():
    x, raw, hi = _bf16_case()
    w = np.array([zo.read_f32(zo.DT_BF16, int(b).to_bytes(2, "little")) for b in hi.ravel()], np.float32).reshape(hi.shape)
    assert np.array_equal(w.view(np.uint32), (hi.astype(np.uint32) << 16))
    out = zo.linear_batch(x, w)
    # the reference's own check loop: ref += input * wvals, in k order, fp32
    ref = np.zeros_like(out)
    for kk in range(x.shape[1]):
        ref = (ref + x[:, kk:kk + 1] * w[None, :, kk]).astype(np.float32)
    assert np.array_equal(out, ref)


def test_against_float64_matmul_and_bias():
    rng = np.random.default_rng(0)
    x = rng.standard_normal((7, 96), dtype=np.float32)
    w = rng.standard_normal((13, 96), dtype=np.float32)
    b = rng.standard_normal(13, dtype=np.float32)
    want = x.astype(np.float64) @ w.astype(np.float64).T
    got = zo.linear_batch(x, w)
    assert np.abs(got - want).max() < 5e-5
    assert np.abs(zo.linear_batch(x, w, b) - (want + b)).max() < 5e-5
    # a transposed weight or swapped operands would not survive this:
    assert np.abs(got - (x.astype(np.float64)[:, :13] @ w.astype(np.float64)[:, :13].T)).max() > 1.0


def test_linearity_and_row_independence():
    rng = np.random.default_rng(1)
    x = rng.standard_normal((4, 32), dtype=np.float32)
    w = rng.standard_normal((5, 32), dtype=np.float32)
    full = zo.linear_batch(x, w)
    for i in range(4):
        assert np.array_equal(zo.linear_batch(x[i:i + 1], w), full[i:i + 1])
    e = np.eye(32, dtype=np.float32)
    assert np.array_equal(zo.linear_batch(e, w), w.T)  # unit inputs read out the weight columns


def test_shape_errors():
    with pytest.raises(zo.OracleError):
        zo.linear_batch(np.zeros((2, 3), np.float32), np.zeros((4, 5), np.float32))
    with pytest.raises(zo.OracleError):
        zo.linear_batch(np.zeros((0, 3), np.float32), np.zeros((4, 3), np.float32))
