"""ctypes loader for the CPU oracle (libzdraw_oracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the
benchmark's CPU-baseline leg. Nothing in the product package imports it.

The wrappers take and return numpy arrays and keep the reference's layouts:
token-major ``[tokens][heads][head_dim]`` fp32 (runtime/attention.zig:100-113).
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from concurrent.futures import ThreadPoolExecutor
from dataclasses import dataclass

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libzdraw_oracle.so")

OK, INVALID_SHAPE, INVALID_CONFIG, BAD_POSITION = 0, 1, 2, 3
DT_F32, DT_F16, DT_BF16 = 0, 1, 2  # dtype codes of read_f32 (pack/tensor.zig:108-115)


class OracleError(Exception):
    def __init__(self, code: int):
        self.code = code
        names = {1: "InvalidShape", 2: "InvalidConfig", 3: "BadPosition"}
        super().__init__(names.get(code, f"error {code}"))


class _AttnConfig(C.Structure):
    _fields_ = [
        ("tokens", C.c_size_t),
        ("heads", C.c_size_t),
        ("kv_heads", C.c_size_t),
        ("head_dim", C.c_size_t),
        ("causal", C.c_int),
        ("valid", C.c_size_t),
    ]


class _RopeConfig(C.Structure):
    _fields_ = [("dims", C.c_size_t * 3), ("lens", C.c_size_t * 3), ("theta", C.c_float)]


@dataclass
class Config:
    """runtime/attention.zig:9-19"""

    tokens: int
    heads: int
    kv_heads: int
    head_dim: int
    causal: bool = False
    valid: int = 0

    def c(self) -> _AttnConfig:
        return _AttnConfig(self.tokens, self.heads, self.kv_heads, self.head_dim,
                           1 if self.causal else 0, self.valid)


@dataclass
class RopeConfig:
    """zimage/zrope.zig:11-15"""

    dims: tuple
    lens: tuple
    theta: float

    def c(self) -> _RopeConfig:
        return _RopeConfig((C.c_size_t * 3)(*self.dims), (C.c_size_t * 3)(*self.lens), self.theta)


def build() -> str:
    """Compile the oracle with gcc (make -C oracle)."""
    subprocess.run(["make", "-C", _HERE, "-B"], check=True, capture_output=True)
    return _LIB_PATH


_lib = None
_fp = C.POINTER(C.c_float)
_sp = C.POINTER(C.c_size_t)
_bp = C.POINTER(C.c_uint8)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = C.CDLL(_LIB_PATH)
        L.zo_attention_run.restype = C.c_int
        L.zo_attention_run.argtypes = [_fp, C.c_size_t, _fp, C.c_size_t, _fp, C.c_size_t,
                                       _fp, C.c_size_t, _fp, C.c_size_t, C.POINTER(_AttnConfig)]
        L.zo_attention_rows.restype = C.c_int
        L.zo_attention_rows.argtypes = [_fp, _fp, _fp, _fp, _fp, C.POINTER(_AttnConfig),
                                        C.c_size_t, C.c_size_t]
        L.zo_attention_rows_masked.restype = C.c_int
        L.zo_attention_rows_masked.argtypes = [_fp, _fp, _fp, _fp, _fp, C.POINTER(_AttnConfig),
                                               _bp, C.c_size_t, C.c_size_t]
        L.zo_klein_build_rope_ref.restype = None
        L.zo_klein_build_rope_ref.argtypes = [_fp, _fp, C.c_size_t, C.c_size_t, C.c_size_t,
                                              C.c_size_t, C.c_size_t, C.c_double]
        L.zo_klein_rms_norm_heads.restype = None
        L.zo_klein_rms_norm_heads.argtypes = [_fp, _fp, C.c_size_t, C.c_size_t]
        L.zo_klein_apply_rope.restype = None
        L.zo_klein_apply_rope.argtypes = [_fp, _fp, _fp, C.c_size_t, C.c_size_t]
        L.zo_zrope_check.restype = C.c_int
        L.zo_zrope_check.argtypes = [C.POINTER(_RopeConfig)]
        L.zo_zrope_count.restype = C.c_size_t
        L.zo_zrope_count.argtypes = [C.POINTER(_RopeConfig)]
        L.zo_zrope_axis_base.restype = C.c_size_t
        L.zo_zrope_axis_base.argtypes = [C.POINTER(_RopeConfig), C.c_size_t]
        L.zo_zrope_fill.restype = None
        L.zo_zrope_fill.argtypes = [_fp, C.POINTER(_RopeConfig)]
        L.zo_zrope_apply.restype = C.c_int
        L.zo_zrope_apply.argtypes = [_fp, C.POINTER(_RopeConfig), _fp, C.c_size_t, _sp]
        L.zo_rms_norm.restype = C.c_int
        L.zo_rms_norm.argtypes = [_fp, _fp, _fp, C.c_size_t, C.c_float]
        L.zo_zimage_norm_heads.restype = C.c_int
        L.zo_zimage_norm_heads.argtypes = [_fp, _fp, C.c_size_t, C.c_size_t, C.c_size_t, C.c_float]
        L.zo_zimage_rotate.restype = C.c_int
        L.zo_zimage_rotate.argtypes = [_fp, _fp, C.POINTER(_RopeConfig), _sp, C.c_size_t, C.c_size_t]
        L.zo_zseq_pad_len.restype = C.c_size_t
        L.zo_zseq_pad_len.argtypes = [C.c_size_t]
        L.zo_zseq_padded_len.restype = C.c_size_t
        L.zo_zseq_padded_len.argtypes = [C.c_size_t]
        L.zo_zseq_grid.restype = C.c_int
        L.zo_zseq_grid.argtypes = [_sp, C.c_size_t, _sp, _sp]
        L.zo_zseq_pad_with_ids.restype = C.c_int
        L.zo_zseq_pad_with_ids.argtypes = [_fp, C.c_size_t, _sp, C.c_size_t, _bp, C.c_size_t,
                                           _fp, C.c_size_t, C.c_size_t, _sp, _sp, _sp]
        L.zo_zunify_basic.restype = C.c_int
        L.zo_zunify_basic.argtypes = [_fp, C.c_size_t, _sp, C.c_size_t, _fp, C.c_size_t, _sp,
                                      C.c_size_t, _fp, C.c_size_t, _sp, C.c_size_t, C.c_size_t]
        L.zo_read_f32.restype = C.c_float
        L.zo_read_f32.argtypes = [C.c_int, _bp]
        L.zo_linear_batch.restype = C.c_int
        L.zo_linear_batch.argtypes = [_fp, C.c_size_t, _fp, C.c_size_t, _fp, C.c_size_t, _fp,
                                      C.c_size_t, C.c_size_t, C.c_size_t]
        _lib = L
    return _lib


def _f(a: np.ndarray):
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(_fp)


def _s(a: np.ndarray):
    assert a.dtype == np.uintp and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(_sp)


def _check(rc: int):
    if rc != OK:
        raise OracleError(rc)


def f32(a) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(a, dtype=np.float32))


# ---------------------------------------------------------------- attention
def attention_run(q, k, v, cfg: Config, scratch_len: int | None = None,
                  out_len: int | None = None) -> np.ndarray:
    """attention.run with the reference's slice-length checks."""
    q, k, v = f32(q).ravel(), f32(k).ravel(), f32(v).ravel()
    out = np.zeros(q.size if out_len is None else out_len, dtype=np.float32)
    n = cfg.tokens if scratch_len is None else scratch_len
    scratch = np.zeros(max(n, 1), dtype=np.float32)
    c = cfg.c()
    _check(lib().zo_attention_run(_f(out), out.size, _f(q), q.size, _f(k), k.size,
                                  _f(v), v.size, _f(scratch), n, C.byref(c)))
    return out.reshape(cfg.tokens, cfg.heads, cfg.head_dim)


def attention_rows(q, k, v, cfg: Config, tok_begin: int, tok_end: int,
                   key_pad=None, out=None) -> np.ndarray:
    """Rows [tok_begin, tok_end) of attention.run; other rows stay zero."""
    q, k, v = f32(q).ravel(), f32(k).ravel(), f32(v).ravel()
    if out is None:
        out = np.zeros(cfg.tokens * cfg.heads * cfg.head_dim, dtype=np.float32)
    flat = out.reshape(-1)
    # score region (tokens floats, rounded up to even) + key list (tokens size_t)
    scratch = np.zeros(((cfg.tokens + 1) & ~1) + 2 * cfg.tokens + 2, dtype=np.float32)
    c = cfg.c()
    if key_pad is None:
        _check(lib().zo_attention_rows(_f(flat), _f(q), _f(k), _f(v), _f(scratch), C.byref(c),
                                       tok_begin, tok_end))
    else:
        kp = np.ascontiguousarray(np.asarray(key_pad, dtype=np.uint8))
        assert kp.size == cfg.tokens
        _check(lib().zo_attention_rows_masked(_f(flat), _f(q), _f(k), _f(v), _f(scratch),
                                              C.byref(c), kp.ctypes.data_as(_bp),
                                              tok_begin, tok_end))
    return out.reshape(cfg.tokens, cfg.heads, cfg.head_dim)


def attention_token_list(q, k, v, cfg: Config, tokens, key_pad=None, threads: int = 8) -> np.ndarray:
    """Rows for an explicit list of query tokens, spread over host threads
    (ctypes releases the GIL; rows are independent in the reference's loop).
    Returns [len(tokens)][heads][head_dim]."""
    q, k, v = f32(q), f32(k), f32(v)
    tokens = [int(t) for t in tokens]
    full = np.zeros((cfg.tokens, cfg.heads, cfg.head_dim), dtype=np.float32)

    def one(t):
        attention_rows(q, k, v, cfg, t, t + 1, key_pad=key_pad, out=full)

    with ThreadPoolExecutor(max_workers=threads) as ex:
        list(ex.map(one, tokens))
    return full[tokens]


# -------------------------------------------------------------------- Klein
def klein_build_rope_ref(grid_h, grid_w, ref_h=0, ref_w=0, theta=2000.0, txt_len=512):
    tokens = txt_len + grid_h * grid_w + ref_h * ref_w
    cos = np.zeros((tokens, 128), dtype=np.float32)
    sin = np.zeros((tokens, 128), dtype=np.float32)
    lib().zo_klein_build_rope_ref(_f(cos), _f(sin), txt_len, grid_h, grid_w, ref_h, ref_w, theta)
    return cos, sin


def klein_rms_norm_heads(x, w) -> np.ndarray:
    """x: [tokens][heads][128] -> normalised copy."""
    x = f32(x).copy()
    tokens, heads, d = x.shape
    assert d == 128
    w = f32(w)
    lib().zo_klein_rms_norm_heads(_f(x), _f(w), tokens, heads)
    return x


def klein_apply_rope(x, cos, sin) -> np.ndarray:
    x = f32(x).copy()
    tokens, heads, d = x.shape
    assert d == 128 and cos.shape == (tokens, 128)
    lib().zo_klein_apply_rope(_f(x), _f(f32(cos)), _f(f32(sin)), tokens, heads)
    return x


# ------------------------------------------------------------------ Z-Image
def zrope_check(cfg: RopeConfig):
    c = cfg.c()
    _check(lib().zo_zrope_check(C.byref(c)))


def zrope_fill(cfg: RopeConfig) -> np.ndarray:
    """Cache.init: [count][2] = (cos, sin)."""
    zrope_check(cfg)
    c = cfg.c()
    n = lib().zo_zrope_count(C.byref(c))
    values = np.zeros((n, 2), dtype=np.float32)
    lib().zo_zrope_fill(_f(values), C.byref(c))
    return values


def zrope_axis_bases(cfg: RopeConfig):
    c = cfg.c()
    return tuple(lib().zo_zrope_axis_base(C.byref(c), a) for a in range(3))


def zrope_apply(values, cfg: RopeConfig, vec, pos) -> np.ndarray:
    vec = f32(vec).copy()
    c = cfg.c()
    p = np.asarray(pos, dtype=np.uintp)
    _check(lib().zo_zrope_apply(_f(f32(values)), C.byref(c), _f(vec), vec.size, _s(p)))
    return vec


def rms_norm(x, w, eps) -> np.ndarray:
    x = f32(x)
    out = np.zeros_like(x)
    _check(lib().zo_rms_norm(_f(out), _f(x), _f(f32(w)), x.size, eps))
    return out


def zimage_norm_heads(x, w, eps) -> np.ndarray:
    x = f32(x).copy()
    tokens, heads, d = x.shape
    _check(lib().zo_zimage_norm_heads(_f(x), _f(f32(w)), tokens, heads, d, eps))
    return x


def zimage_rotate(x, values, cfg: RopeConfig, pos) -> np.ndarray:
    x = f32(x).copy()
    tokens, heads, _ = x.shape
    p = np.ascontiguousarray(np.asarray(pos, dtype=np.uintp))
    assert p.shape == (tokens, 3)
    c = cfg.c()
    _check(lib().zo_zimage_rotate(_f(x), _f(f32(values)), C.byref(c), _s(p), tokens, heads))
    return x


def zseq_pad_len(n: int) -> int:
    return lib().zo_zseq_pad_len(n)


def zseq_padded_len(n: int) -> int:
    return lib().zo_zseq_padded_len(n)


def zseq_grid(size, start, out_len=None) -> np.ndarray:
    n = size[0] * size[1] * size[2] if out_len is None else out_len
    out = np.zeros((n, 3), dtype=np.uintp)
    _check(lib().zo_zseq_grid(_s(out), n, _s(np.asarray(size, dtype=np.uintp)),
                              _s(np.asarray(start, dtype=np.uintp))))
    return out


def zseq_pad_with_ids(feat, dim, size, start):
    feat = f32(feat).ravel()
    span = size[0] * size[1] * size[2]
    total = zseq_padded_len(span)
    out = np.zeros(total * dim, dtype=np.float32)
    ids = np.full((total, 3), 9, dtype=np.uintp)
    mask = np.zeros(total, dtype=np.uint8)
    tot = C.c_size_t(0)
    _check(lib().zo_zseq_pad_with_ids(_f(out), out.size, _s(ids), total, mask.ctypes.data_as(_bp),
                                      total, _f(feat), feat.size, dim,
                                      _s(np.asarray(size, dtype=np.uintp)),
                                      _s(np.asarray(start, dtype=np.uintp)), C.byref(tot)))
    return out.reshape(total, dim), ids, mask.astype(bool), tot.value


def zunify_basic(image, image_pos, cap, cap_pos, hidden):
    image, cap = f32(image).ravel(), f32(cap).ravel()
    ip = np.ascontiguousarray(np.asarray(image_pos, dtype=np.uintp).reshape(-1, 3))
    cp = np.ascontiguousarray(np.asarray(cap_pos, dtype=np.uintp).reshape(-1, 3))
    total = ip.shape[0] + cp.shape[0]
    out = np.zeros(total * hidden, dtype=np.float32)
    pos = np.zeros((total, 3), dtype=np.uintp)
    _check(lib().zo_zunify_basic(_f(out), out.size, _s(pos), total, _f(image), image.size, _s(ip),
                                 ip.shape[0], _f(cap), cap.size, _s(cp), cp.shape[0], hidden))
    return out.reshape(total, hidden), pos, {"image_start": 0, "image_len": ip.shape[0], "total": total}


def read_f32(dtype: int, raw: bytes) -> float:
    buf = (C.c_uint8 * 4)(*(list(raw) + [0] * (4 - len(raw))))
    return float(lib().zo_read_f32(dtype, buf))


def linear_batch(x, weight, bias=None) -> np.ndarray:
    """runtime/ops.zig:37-60 over rows (metal/mgemm.zig:134-155): x [count][cols], weight [rows][cols]
    already decoded to fp32 -> [count][rows]."""
    x, weight = f32(x), f32(weight)
    if x.ndim != 2 or weight.ndim != 2:
        raise OracleError(INVALID_SHAPE)
    count, cols = x.shape
    rows = weight.shape[0]
    out = np.empty((count, rows), np.float32)
    b = f32(bias) if bias is not None else None
    _check(lib().zo_linear_batch(_f(out), out.size, _f(x), x.size, _f(weight), weight.size,
                                 _f(b) if b is not None else None, rows, weight.shape[1] if x.size else cols, count))
    return out
