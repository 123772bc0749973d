"""ctypes binding of the C++ host layer (libzdraw_host.so).

The classes keep the reference's names and call shapes so tests read like the
reference's own (`mattn.Context.init/run/pick`, `attention_fast.run`,
`attention.Config`): metal/mattn.zig, runtime/attention_fast.zig,
runtime/attention.zig.
"""
from __future__ import annotations

import ctypes as C
import os
from dataclasses import dataclass

import numpy as np

from . import hip

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libzdraw_host.so")


class ZdrawError(Exception):
    """One subclass per value of the host layer's Error enum."""
    code = -1


class UnsupportedShape(ZdrawError):
    code = 1


class InvalidShape(ZdrawError):
    code = 2


class NotAvailable(ZdrawError):
    code = 3


class QueueFailed(ZdrawError):
    code = 4


class CompileFailed(ZdrawError):
    code = 5


class DispatchFailed(ZdrawError):
    code = 6


class BadPosition(ZdrawError):
    code = 7


class OutOfMemory(ZdrawError):
    code = 8


_ERRORS = {c.code: c for c in (UnsupportedShape, InvalidShape, NotAvailable, QueueFailed, CompileFailed,
                               DispatchFailed, BadPosition, OutOfMemory)}


def _raise(code: int):
    if code != 0:
        raise _ERRORS.get(code, ZdrawError)(hip.last_error())


@dataclass
class Config:
    """runtime/attention.zig:9-19"""
    tokens: int
    heads: int
    kv_heads: int
    head_dim: int
    causal: bool = False
    valid: int = 0


class _ZhConfig(C.Structure):
    _fields_ = [("tokens", C.c_size_t), ("heads", C.c_size_t), ("kv_heads", C.c_size_t),
                ("head_dim", C.c_size_t), ("causal", C.c_int), ("valid", C.c_size_t)]


def _zc(cfg: Config) -> _ZhConfig:
    return _ZhConfig(cfg.tokens, cfg.heads, cfg.kv_heads, cfg.head_dim, 1 if cfg.causal else 0, cfg.valid)


class _Klein(C.Structure):
    _fields_ = [("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("o", C.c_void_p),
                ("in_dtype", C.c_uint32), ("out_dtype", C.c_uint32),
                ("tokens", C.c_size_t), ("heads", C.c_size_t), ("nb", C.c_size_t), ("txt_rows", C.c_size_t),
                ("norm_q", C.c_void_p), ("norm_k", C.c_void_p),
                ("norm_added_q", C.c_void_p), ("norm_added_k", C.c_void_p),
                ("rope_cos", C.c_void_p), ("rope_sin", C.c_void_p), ("rope_per_segment", C.c_bool),
                ("key_pad", C.c_void_p), ("out_row_stride", C.c_size_t), ("k_site", C.c_uint32),
                ("score_bound", C.c_float), ("staging", C.c_uint32)]


class _Zimage(C.Structure):
    _fields_ = [("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("o", C.c_void_p),
                ("in_dtype", C.c_uint32), ("out_dtype", C.c_uint32),
                ("tokens", C.c_size_t), ("heads", C.c_size_t),
                ("q_norm", C.c_void_p), ("k_norm", C.c_void_p), ("pos", C.c_void_p), ("rope_pairs", C.c_void_p),
                ("dims", C.c_size_t * 3), ("bases", C.c_size_t * 3), ("norm_eps", C.c_float),
                ("k_site", C.c_uint32), ("score_bound", C.c_float), ("staging", C.c_uint32)]


class _RopeCache(C.Structure):
    _fields_ = [("dims", C.c_size_t * 3), ("lens", C.c_size_t * 3), ("values", C.POINTER(C.c_float))]


CPU_RUN = C.CFUNCTYPE(C.c_int, C.POINTER(C.c_float), C.c_size_t, C.POINTER(C.c_float), C.c_size_t,
                      C.POINTER(C.c_float), C.c_size_t, C.POINTER(C.c_float), C.c_size_t,
                      C.POINTER(C.c_float), C.c_size_t, C.POINTER(_ZhConfig))

_fp = C.POINTER(C.c_float)
_lib = None


def lib():
    global _lib
    if _lib is None:
        hip.lib()  # libzdraw_host.so links against it
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: build it with `python -m zdraw_amd.build`")
        L = C.CDLL(LIB_PATH)
        vp, sz = C.c_void_p, C.c_size_t
        L.zh_context_init.restype = vp
        L.zh_context_init.argtypes = [C.POINTER(C.c_int)]
        L.zh_context_init_kernel.restype = vp
        L.zh_context_init_kernel.argtypes = [C.c_uint32, C.POINTER(C.c_int)]
        L.zh_context_deinit.restype = None
        L.zh_context_deinit.argtypes = [vp]
        for name in ("zh_context_device", "zh_context_queue", "zh_context_block_pipeline"):
            getattr(L, name).restype = vp
            getattr(L, name).argtypes = [vp]
        L.zh_context_pick.restype = C.c_int
        L.zh_context_pick.argtypes = [vp, sz, sz, C.POINTER(C.c_uint32), C.POINTER(sz)]
        run_args = [vp, _fp, sz, _fp, sz, _fp, sz, _fp, sz, C.POINTER(_ZhConfig)]
        L.zh_context_run.restype = C.c_int
        L.zh_context_run.argtypes = run_args
        L.zh_context_run_pooled.restype = C.c_int
        L.zh_context_run_pooled.argtypes = run_args
        L.zh_context_run_on_handles.restype = C.c_int
        L.zh_context_run_on_handles.argtypes = [vp, vp, vp, vp, vp, C.POINTER(_ZhConfig)]
        L.zh_attention_fast_run.restype = C.c_int
        L.zh_attention_fast_run.argtypes = [vp, _fp, sz, _fp, sz, _fp, sz, _fp, sz, _fp, sz,
                                            C.POINTER(_ZhConfig), CPU_RUN]
        L.zh_qk_run.restype = C.c_int
        L.zh_qk_run.argtypes = [vp, vp, vp, _fp, _fp, C.POINTER(sz), sz, C.POINTER(_RopeCache),
                                sz, sz, sz, sz, C.c_float]
        L.zh_joint_klein.restype = C.c_int
        L.zh_joint_klein.argtypes = [vp, C.POINTER(_Klein)]
        L.zh_joint_zimage.restype = C.c_int
        L.zh_joint_zimage.argtypes = [vp, C.POINTER(_Zimage)]
        L.zh_score_bound.restype = C.c_float
        L.zh_score_bound.argtypes = [_fp, _fp, _fp, _fp]
        L.zh_sizeof.restype = sz
        L.zh_sizeof.argtypes = [C.c_int]
        assert L.zh_sizeof(0) == C.sizeof(_ZhConfig)
        assert L.zh_sizeof(1) == C.sizeof(_Klein), (L.zh_sizeof(1), C.sizeof(_Klein))
        assert L.zh_sizeof(2) == C.sizeof(_Zimage), (L.zh_sizeof(2), C.sizeof(_Zimage))
        assert L.zh_sizeof(3) == C.sizeof(_RopeCache)
        _lib = L
    return _lib


# ------------------------------------------------------------- bf16 helpers
def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even fp32 -> bf16, returned as uint16 bit patterns."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    rounded = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    return rounded.astype(np.uint16)


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


# ----------------------------------------------------------- device buffers
class DeviceBuffer:
    """An owned device buffer created through the C ABI (mbuffer.Buffer, owned)."""

    def __init__(self, device, nbytes: int = 0, data: np.ndarray | None = None):
        L = hip.lib()
        if data is not None:
            data = np.ascontiguousarray(data)
            self.handle = L.zdraw_hip_create_buffer_with_data(device, data.ctypes.data_as(C.c_void_p), data.nbytes)
            self.nbytes = data.nbytes
        else:
            self.handle = L.zdraw_hip_create_buffer(device, nbytes)
            self.nbytes = nbytes
        if not self.handle:
            raise OutOfMemory(hip.last_error())

    def read(self, dtype, shape) -> np.ndarray:
        out = np.empty(shape, dtype=dtype)
        assert out.nbytes <= self.nbytes
        hip.lib().zdraw_hip_read_buffer(self.handle, out.ctypes.data_as(C.c_void_p), out.nbytes)
        return out

    def write(self, data: np.ndarray):
        data = np.ascontiguousarray(data)
        assert data.nbytes <= self.nbytes
        hip.lib().zdraw_hip_write_buffer(self.handle, data.ctypes.data_as(C.c_void_p), data.nbytes)

    def release(self):
        if self.handle:
            hip.lib().zdraw_hip_release_buffer(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.release()
        except Exception:
            pass


def _f(a: np.ndarray):
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(_fp)


class Context:
    """metal/mattn.zig:47-276 over HIP."""

    def __init__(self, ptr):
        self._ptr = ptr

    @classmethod
    def init(cls) -> "Context":
        err = C.c_int(0)
        ptr = lib().zh_context_init(C.byref(err))
        _raise(err.value)
        return cls(ptr)

    @classmethod
    def init_kernel(cls, kernel: int) -> "Context":
        err = C.c_int(0)
        ptr = lib().zh_context_init_kernel(kernel, C.byref(err))
        _raise(err.value)
        return cls(ptr)

    def deinit(self):
        if self._ptr:
            lib().zh_context_deinit(self._ptr)
            self._ptr = None

    @property
    def device(self):
        return lib().zh_context_device(self._ptr)

    @property
    def queue(self):
        return lib().zh_context_queue(self._ptr)

    @property
    def block_pipeline(self):
        return lib().zh_context_block_pipeline(self._ptr)

    def pick(self, tokens: int, head_dim: int):
        kernel, threads = C.c_uint32(0), C.c_size_t(0)
        if not lib().zh_context_pick(self._ptr, tokens, head_dim, C.byref(kernel), C.byref(threads)):
            return None
        return {"kernel": kernel.value, "threads": threads.value}

    def _run(self, fn, q, k, v, cfg: Config, out_len=None):
        q = np.ascontiguousarray(q, np.float32).ravel()
        k = np.ascontiguousarray(k, np.float32).ravel()
        v = np.ascontiguousarray(v, np.float32).ravel()
        out = np.zeros(q.size if out_len is None else out_len, np.float32)
        c = _zc(cfg)
        _raise(fn(self._ptr, _f(out), out.size, _f(q), q.size, _f(k), k.size, _f(v), v.size, C.byref(c)))
        return out.reshape(cfg.tokens, cfg.heads, cfg.head_dim)

    def run(self, q, k, v, cfg: Config, out_len=None) -> np.ndarray:
        return self._run(lib().zh_context_run, q, k, v, cfg, out_len)

    def run_pooled(self, q, k, v, cfg: Config) -> np.ndarray:
        return self._run(lib().zh_context_run_pooled, q, k, v, cfg)

    def run_on_handles(self, q_h, k_h, v_h, out_h, cfg: Config):
        c = _zc(cfg)
        _raise(lib().zh_context_run_on_handles(self._ptr, q_h, k_h, v_h, out_h, C.byref(c)))

    def buffer(self, data=None, nbytes=0) -> DeviceBuffer:
        return DeviceBuffer(self.device, nbytes=nbytes, data=data)

    # ---- fused joint attention (joint::Klein / joint::Zimage)
    def joint_klein(self, q, k, v, o, *, tokens, heads, nb=1, in_dtype=hip.BF16, out_dtype=hip.BF16,
                    norm_q, norm_k, norm_added_q=None, norm_added_k=None, txt_rows=0,
                    rope_cos, rope_sin, rope_per_segment=False, key_pad=None,
                    out_row_stride=0, k_site=hip.K_IN_TILE_LOAD, score_bound=0.0, staging=0):
        h = lambda b: b.handle if b is not None else None
        c = _Klein(h(q), h(k), h(v), h(o), in_dtype, out_dtype, tokens, heads, nb, txt_rows,
                   h(norm_q), h(norm_k), h(norm_added_q), h(norm_added_k), h(rope_cos), h(rope_sin),
                   rope_per_segment, h(key_pad), out_row_stride, k_site, score_bound, staging)
        _raise(lib().zh_joint_klein(self._ptr, C.byref(c)))

    def joint_zimage(self, q, k, v, o, *, tokens, heads, in_dtype=hip.BF16, out_dtype=hip.BF16,
                     q_norm, k_norm, pos, rope_pairs, dims, bases, norm_eps, k_site=hip.K_IN_TILE_LOAD,
                     score_bound=0.0, staging=0):
        c = _Zimage(q.handle, k.handle, v.handle, o.handle, in_dtype, out_dtype, tokens, heads,
                    q_norm.handle, k_norm.handle, pos.handle, rope_pairs.handle,
                    (C.c_size_t * 3)(*dims), (C.c_size_t * 3)(*bases), norm_eps, k_site, score_bound, staging)
        _raise(lib().zh_joint_zimage(self._ptr, C.byref(c)))

    def qk_run(self, q_buf, k_buf, q_weight, k_weight, pos, rope_values, dims, lens, *, tokens, heads,
               kv_heads, head_dim, norm_eps):
        """metal/mqk.zig:20-58"""
        qw = np.ascontiguousarray(q_weight, np.float32)
        kw = np.ascontiguousarray(k_weight, np.float32)
        p = np.ascontiguousarray(pos, np.uintp).reshape(-1)
        vals = np.ascontiguousarray(rope_values, np.float32)
        rc = _RopeCache((C.c_size_t * 3)(*dims), (C.c_size_t * 3)(*lens), _f(vals.reshape(-1)))
        _raise(lib().zh_qk_run(self._ptr, q_buf.handle, k_buf.handle, _f(qw), _f(kw),
                               p.ctypes.data_as(C.POINTER(C.c_size_t)), p.size // 3, C.byref(rc),
                               tokens, heads, kv_heads, head_dim, norm_eps))


def attention_fast_run(ctx: Context | None, q, k, v, cfg: Config, cpu=None, scratch_len=None) -> np.ndarray:
    """runtime/attention_fast.zig:6-24. `cpu(out, q, k, v, scratch, cfg) -> int` is the caller's CPU
    kernel (numpy views); None means the caller has none."""
    q = np.ascontiguousarray(q, np.float32).ravel()
    k = np.ascontiguousarray(k, np.float32).ravel()
    v = np.ascontiguousarray(v, np.float32).ravel()
    out = np.zeros(q.size, np.float32)
    n = cfg.tokens if scratch_len is None else scratch_len
    scratch = np.zeros(max(n, 1), np.float32)

    def tramp(o, ol, qq, ql, kk, kl, vv, vl, sc, sl, zc):
        as_np = lambda p, ln: np.ctypeslib.as_array(p, shape=(ln,))
        z = zc.contents
        return int(cpu(as_np(o, ol), as_np(qq, ql), as_np(kk, kl), as_np(vv, vl), as_np(sc, max(sl, 1))[:sl],
                       Config(z.tokens, z.heads, z.kv_heads, z.head_dim, bool(z.causal), z.valid)))

    cb = CPU_RUN(tramp) if cpu is not None else C.cast(None, CPU_RUN)
    c = _zc(cfg)
    _raise(lib().zh_attention_fast_run(ctx._ptr if ctx is not None else None, _f(out), out.size, _f(q), q.size,
                                       _f(k), k.size, _f(v), v.size, _f(scratch), n, C.byref(c), cb))
    return out.reshape(cfg.tokens, cfg.heads, cfg.head_dim)


# ------------------------------------------------- host-side tables / positions
_sp = C.POINTER(C.c_size_t)


def klein_build_rope_ref(grid_h, grid_w, ref_h=0, ref_w=0, theta=2000.0, txt_len=512):
    """klein/zflux2_dit.zig:125-170 -> (cos, sin) [tokens][128] f32."""
    L = lib()
    L.zh_klein_build_rope_ref.restype = None
    L.zh_klein_build_rope_ref.argtypes = [_fp, _fp] + [C.c_size_t] * 5 + [C.c_double]
    n = txt_len + grid_h * grid_w + ref_h * ref_w
    cos = np.zeros((n, 128), np.float32)
    sin = np.zeros((n, 128), np.float32)
    L.zh_klein_build_rope_ref(_f(cos.reshape(-1)), _f(sin.reshape(-1)), txt_len, grid_h, grid_w, ref_h, ref_w, theta)
    return cos, sin


def zimage_rope_fill(dims, lens, theta):
    """zimage/zrope.zig:29-106 -> (values [count][2], bases)."""
    L = lib()
    L.zh_zimage_rope_fill.restype = C.c_int
    L.zh_zimage_rope_fill.argtypes = [_fp, _sp, _sp, C.c_float]
    count = sum(l * (d // 2) for d, l in zip(dims, lens))
    vals = np.zeros((max(count, 1), 2), np.float32)
    _raise(L.zh_zimage_rope_fill(_f(vals.reshape(-1)), (C.c_size_t * 3)(*dims), (C.c_size_t * 3)(*lens), theta))
    bases, acc = [], 0
    for d, l in zip(dims, lens):
        bases.append(acc)
        acc += l * (d // 2)
    return vals, tuple(bases)


def zimage_sequence_positions(grid_h, grid_w, cap_tokens):
    """Positions of [image | caption] (zstep_shape.zig:58-66, zunify.zig:31-34) -> [total][3] uintp."""
    L = lib()
    L.zh_zseq_padded_len.restype = C.c_size_t
    L.zh_zseq_padded_len.argtypes = [C.c_size_t]
    L.zh_zimage_sequence_positions.restype = C.c_int
    L.zh_zimage_sequence_positions.argtypes = [_sp, C.c_size_t, C.c_size_t, C.c_size_t, C.c_size_t]
    total = L.zh_zseq_padded_len(grid_h * grid_w) + L.zh_zseq_padded_len(cap_tokens)
    pos = np.zeros((total, 3), np.uintp)
    _raise(L.zh_zimage_sequence_positions(pos.ctypes.data_as(_sp), total, grid_h, grid_w, cap_tokens))
    return pos


def score_bound(w_q, w_k, w_q_txt=None, w_k_txt=None) -> float:
    """joint::scoreBound: bound on |q'.k'|/sqrt(128) for RMS-normalised, rotated operands."""
    def ptr(w):
        if w is None:
            return None
        return _f(np.ascontiguousarray(w, np.float32))
    arrs = [None if w is None else np.ascontiguousarray(w, np.float32) for w in (w_q, w_k, w_q_txt, w_k_txt)]
    ptrs = [None if a is None else _f(a) for a in arrs]
    return float(lib().zh_score_bound(*ptrs))
