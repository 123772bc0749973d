"""ctypes binding of the C ABI in include/zdraw_hip.h and of the measurement aids in
include/zdraw_hip_measure.h (libzdraw_hip.so)."""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
# ZDRAW_HIP_LIB points the binding at an experimental build of the same C ABI
LIB_PATH = os.environ.get("ZDRAW_HIP_LIB") or os.path.join(HERE, "lib", "libzdraw_hip.so")

OK, ERR_HANDLE, ERR_DEVICE, UNAVAILABLE, INVALID = 0, -1, -2, 1, 2
K_ROWS, K_FLASH, K_BLOCK, K_WIDE = 0, 1, 2, 3
F32, F16, BF16 = 0, 1, 2
QK_NONE, QK_KLEIN, QK_ZIMAGE = 0, 1, 2
K_IN_TILE_LOAD, K_PREPASS = 0, 1
NOALLOC_SCRATCH_BYTES = 64 << 20  # ZDRAW_HIP_NOALLOC_SCRATCH_BYTES


class AttnParams(C.Structure):
    """ZdrawAttnParams (metal_c.zig:245-256)"""
    _fields_ = [("tokens", C.c_uint32), ("heads", C.c_uint32), ("kv_heads", C.c_uint32),
                ("head_dim", C.c_uint32), ("causal", C.c_uint32), ("valid", C.c_uint32)]


class AttnExt(C.Structure):
    """ZdrawHipAttnExt"""
    _fields_ = [
        ("q_off", C.c_uint64), ("k_off", C.c_uint64), ("v_off", C.c_uint64), ("out_off", C.c_uint64),
        ("q_stride", C.c_uint64 * 3), ("k_stride", C.c_uint64 * 3),
        ("v_stride", C.c_uint64 * 3), ("out_stride", C.c_uint64 * 3),
        ("rope_batch_rows", C.c_uint64), ("mask_batch_bytes", C.c_uint64),
        ("zimage_base", C.c_uint64 * 3), ("zimage_dims", C.c_uint32 * 3),
        ("batch", C.c_uint32), ("in_dtype", C.c_uint32), ("out_dtype", C.c_uint32),
        ("qk_mode", C.c_uint32), ("k_site", C.c_uint32), ("txt_rows", C.c_uint32), ("eps", C.c_float),
        ("score_bound", C.c_float), ("staging", C.c_uint32),
    ]


class QkOperands(C.Structure):
    """ZdrawHipQkOperands"""
    _fields_ = [(n, C.c_void_p) for n in ("q_weight", "k_weight", "q_weight_txt", "k_weight_txt",
                                          "rope_cos", "rope_sin", "pos", "rope_pairs", "key_pad")]


class GemmParams(C.Structure):
    """ZdrawGemmParams (metal_c.zig:276-283)"""
    _fields_ = [("m", C.c_uint32), ("k", C.c_uint32), ("n", C.c_uint32), ("dtype", C.c_uint32),
                ("mode", C.c_uint32), ("weight_offset", C.c_uint64)]


class GemmExt(C.Structure):
    """ZdrawHipGemmExt"""
    _fields_ = [("a_off", C.c_uint64), ("c_off", C.c_uint64), ("lda", C.c_uint64), ("ldw", C.c_uint64),
                ("ldc", C.c_uint64), ("a_dtype", C.c_uint32), ("c_dtype", C.c_uint32)]


class QkNormParams(C.Structure):
    """ZdrawQkNormParams (metal_c.zig:258-274)"""
    _fields_ = [("tokens", C.c_uint32), ("heads", C.c_uint32), ("kv_heads", C.c_uint32), ("head_dim", C.c_uint32),
                ("q_dtype", C.c_uint32), ("k_dtype", C.c_uint32),
                ("dim0", C.c_uint32), ("dim1", C.c_uint32), ("dim2", C.c_uint32), ("eps", C.c_float),
                ("q_offset", C.c_uint64), ("k_offset", C.c_uint64),
                ("base0", C.c_uint64), ("base1", C.c_uint64), ("base2", C.c_uint64)]


class ChainAttnBuffers(C.Structure):
    """ZdrawHipChainAttnBuffers"""
    _fields_ = [(n, C.c_void_p) for n in ("norm", "q", "k", "v", "mix", "attn")]


class ChainAttnWeights(C.Structure):
    """ZdrawHipChainAttnWeights"""
    _fields_ = [(n, C.c_void_p) for n in ("q", "k", "v", "q_norm", "k_norm", "pos", "rope", "proj")]


class ChainAttnParams(C.Structure):
    """ZdrawHipChainAttnParams"""
    _fields_ = [("q", GemmParams), ("k", GemmParams), ("v", GemmParams), ("qk", QkNormParams),
                ("attn", AttnParams), ("proj", GemmParams), ("act_dtype", C.c_uint32), ("score_bound", C.c_float)]


W_F16, W_BF16, W_F32 = 1, 2, 3     # weight dtype codes of GemmParams.dtype
GEMM_EXACT, GEMM_HALF = 1, 2       # GemmParams.mode

# every symbol include/*.h declares: name -> (restype, argtypes)
_vp, _sz, _u32, _u64, _int = C.c_void_p, C.c_size_t, C.c_uint32, C.c_uint64, C.c_int
_AP, _AX, _QO = C.POINTER(AttnParams), C.POINTER(AttnExt), C.POINTER(QkOperands)
_GP, _GX = C.POINTER(GemmParams), C.POINTER(GemmExt)
SYMBOLS = {
    "zdraw_hip_create_device": (_vp, []),
    "zdraw_hip_release_device": (None, [_vp]),
    "zdraw_hip_create_queue": (_vp, [_vp]),
    "zdraw_hip_release_queue": (None, [_vp]),
    "zdraw_hip_create_buffer": (_vp, [_vp, _sz]),
    "zdraw_hip_create_buffer_with_data": (_vp, [_vp, _vp, _sz]),
    "zdraw_hip_create_buffer_no_copy": (_vp, [_vp, _vp, _sz]),
    "zdraw_hip_wrap_device_memory": (_vp, [_vp, _vp, _sz]),
    "zdraw_hip_read_buffer_any": (_int, [_vp, _vp, _vp, _sz]),
    "zdraw_hip_release_weight_buffer": (None, [_vp]),
    "zdraw_hip_read_buffer": (None, [_vp, _vp, _sz]),
    "zdraw_hip_write_buffer": (None, [_vp, _vp, _sz]),
    "zdraw_hip_buffer_length": (_sz, [_vp]),
    "zdraw_hip_buffer_device_ptr": (_vp, [_vp]),
    "zdraw_hip_release_buffer": (None, [_vp]),
    "zdraw_hip_compile": (_vp, [_vp, C.c_char_p, C.c_char_p, C.c_char_p, _sz]),
    "zdraw_hip_release_pipeline": (None, [_vp]),
    "zdraw_hip_pipeline_threads": (_sz, [_vp]),
    "zdraw_hip_run_attention": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _AP, _u32, _sz]),
    "zdraw_hip_batch_begin": (_vp, [_vp]),
    "zdraw_hip_run_attention_enc": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _AP, _u32, _sz]),
    "zdraw_hip_run_attention_enc_off": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _AP, _u32, _sz, _u64, _u64]),
    "zdraw_hip_batch_end": (_int, [_vp]),
    "zdraw_hip_run_attention_fused_enc": (_int, [_vp, _vp, _vp, _vp, _vp, _AP, _AX, _QO]),
    "zdraw_hip_reserve_attention_fused": (_int, [_vp, _vp, _vp, _vp, _vp, _AP, _AX, _QO]),
    "zdraw_hip_run_attention_fused": (_int, [_vp, _vp, _vp, _vp, _vp, _AP, _AX, _QO]),
    "zdraw_hip_run_attention_fused_noalloc_enc": (_int, [_vp, _vp, _vp, _vp, _vp, _AP, _AX, _QO]),
    "zdraw_hip_run_qk_norm_rope_ext": (_int, [_vp, _vp, _vp, _vp, _AP, _AX, _QO]),
    "zdraw_hip_run_qk_norm_rope": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, C.POINTER(QkNormParams), _sz]),
    "zdraw_hip_attn_scratch": (_vp, [_vp, _int, _sz]),
    "zdraw_hip_metrics_reset": (None, []),
    "zdraw_hip_dispatch_count": (_u64, []),
    "zdraw_hip_command_count": (_u64, []),
    "zdraw_hip_attn_fallback_count": (_u64, []),
    "zdraw_hip_gpu_ns": (_u64, []),
    "zdraw_hip_trace_attention": (None, [_int]),
    "zdraw_hip_trace_attention_ns": (_u64, [C.POINTER(C.c_uint64)]),
    "zdraw_hip_run_gemm": (_int, [_vp, _vp, _vp, _vp, _vp, _GP]),
    "zdraw_hip_run_gemm_enc": (_int, [_vp, _vp, _vp, _vp, _vp, _GP]),
    "zdraw_hip_run_gemm_off_enc": (_int, [_vp, _vp, _vp, _vp, _vp, _GP, _u64, _u64]),
    "zdraw_hip_run_gemm_f16a_enc": (_int, [_vp, _vp, _vp, _vp, _GP, _u64, _u64]),
    "zdraw_hip_run_gemm_pair": (_int, [_vp, _vp, _vp, _vp, _vp, _GP, _vp, _vp, _GP]),
    "zdraw_hip_run_gemm_triple": (_int, [_vp, _vp, _vp, _vp, _vp, _GP, _vp, _vp, _GP, _vp, _vp, _GP]),
    "zdraw_hip_run_gemm_ext_enc": (_int, [_vp, _vp, _vp, _vp, _GP, _GX]),
    "zdraw_hip_run_gemm_group_ext_enc": (_int, [_vp, _vp, C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_GP), C.c_uint32, _GX]),
    "zdraw_hip_run_chain_attn_enc": (_int, [_vp, C.POINTER(ChainAttnBuffers), C.POINTER(ChainAttnWeights),
                                            C.POINTER(ChainAttnParams)]),
    "zdraw_hip_clock_probe": (None, [_int]),
    "zdraw_hip_clock_probe_read": (C.c_size_t, [C.POINTER(C.c_uint64), C.POINTER(C.c_uint64), C.c_size_t]),
    "zdraw_hip_event_create": (_vp, []),
    "zdraw_hip_event_record": (_int, [_vp, _vp]),
    "zdraw_hip_event_sync": (_int, [_vp]),
    "zdraw_hip_event_elapsed_ms": (C.c_float, [_vp, _vp]),
    "zdraw_hip_event_release": (None, [_vp]),
    "zdraw_hip_queue_sync": (_int, [_vp]),
    "zdraw_hip_set_attention_variant": (None, [_int]),
    "zdraw_hip_set_gemm_build": (None, [_int]),
    "zdraw_hip_create_queue_on_cus": (_vp, [_vp, _int]),
    "zdraw_hip_wide_redo_tiles": (_int, []),
    "zdraw_hip_attention_tail_plan": (None, [_u64, _u32, _u32, C.POINTER(C.c_uint32), C.POINTER(C.c_uint32)]),
    "zdraw_hip_gemm_tail_plan": (None, [_u32, _u32, _u32, _u32, _u32, C.POINTER(C.c_uint32), C.POINTER(C.c_uint32)]),
    "zdraw_hip_zimage_axis_lens": (_int, [_u64, C.POINTER(C.c_uint64), C.POINTER(C.c_uint32), C.POINTER(C.c_uint32)]),
    "zdraw_hip_abi_sizeof": (_sz, [_int]),
    "zdraw_hip_last_error": (C.c_char_p, []),
}

_lib = None


def lib():
    """Load libzdraw_hip.so; raises if it has not been built (python -m zdraw_amd.build)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: build it with `python -m zdraw_amd.build`")
        L = C.CDLL(LIB_PATH, mode=C.RTLD_GLOBAL)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(L, name)  # AttributeError if the library lacks a declared symbol
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def last_error() -> str:
    return (lib().zdraw_hip_last_error() or b"").decode()
