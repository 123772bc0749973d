// Device-side helpers shared by the gfx950 attention kernels: vector types,
// global-memory chunk loads, bf16 packing, lane-pair reductions and the
// QK-norm + rope arithmetic.
#pragma once

#include "attn_kernel.h"

#include <type_traits>

namespace zdraw {

typedef __bf16 bf16_t;
typedef _Float16 f16_t;
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));

constexpr int D = kHeadDim;

// ---------------------------------------------------------------- raw loads
// Eight consecutive head_dim elements as they come from memory.
template <typename T> struct Raw8;
template <> struct Raw8<float> { f32x4 a, b; };
template <> struct Raw8<bf16_t> { u32x4 r; };
template <> struct Raw8<f16_t> { u32x4 r; };

template <typename T>
__device__ __forceinline__ Raw8<T> ld_raw8(const T* p, bool ok) {
    Raw8<T> x;
    if constexpr (std::is_same<T, float>::value) {
        x.a = f32x4{0.f, 0.f, 0.f, 0.f};
        x.b = x.a;
        if (ok) {
            x.a = *reinterpret_cast<const f32x4*>(p);
            x.b = *reinterpret_cast<const f32x4*>(p + 4);
        }
    } else {
        x.r = u32x4{0u, 0u, 0u, 0u};
        if (ok) x.r = *reinterpret_cast<const u32x4*>(p);
    }
    return x;
}

// The same chunk through a buffer resource: the address is a wave-uniform
// descriptor (base in scalar registers) + a per-thread byte offset + a uniform
// byte offset, so a loop that walks blocks spends no vector ALU work on it.
typedef __amdgpu_buffer_rsrc_t rsrc_t;
__device__ __forceinline__ rsrc_t make_rsrc(const void* base, unsigned bytes) {
    // word 3: 32-bit data format, raw (unstrided) addressing
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}
template <typename T>
__device__ __forceinline__ Raw8<T> ld_raw8_buf(rsrc_t rsrc, unsigned thread_off, unsigned uniform_off) {
    Raw8<T> x;
    if constexpr (std::is_same<T, float>::value) {
        x.a = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)thread_off, (int)uniform_off, 0));
        x.b = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)(thread_off + 16), (int)uniform_off, 0));
    } else {
        x.r = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)thread_off, (int)uniform_off, 0));
    }
    return x;
}

// 16 bytes per lane from global memory straight into LDS: lane i's data lands at
// lds_addr + 16 i (lds_addr, the descriptor and uniform_off are wave-uniform). The
// instruction is written out so that the compiler does not make every later LDS
// read wait for it; the CALLER orders it against those reads (s_waitcnt vmcnt +
// barrier before the data is read, a barrier after the last read of what it overwrites).
__device__ __forceinline__ u32x4 make_rsrc_words(const void* base, unsigned bytes) {
    const unsigned long long p = reinterpret_cast<unsigned long long>(base);
    return u32x4{(unsigned)p, (unsigned)(p >> 32) & 0xffffu, bytes, 0x00020000u};
}
// LDS byte address of a __shared__ object (taken once; the cast carries a null check).
__device__ __forceinline__ unsigned lds_address(const void* p) {
    return (unsigned)(unsigned long long)(__attribute__((address_space(3))) const void*)p;
}
__device__ __forceinline__ void load_to_lds_16(u32x4 rsrc, unsigned lds_addr, unsigned thread_off, unsigned uniform_off) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :
                 : "s"(lds_addr), "v"(thread_off), "s"(rsrc), "s"(uniform_off)
                 : "memory", "m0");
}

// The same load in two parts, for runs of loads whose LDS targets differ by less than 4 KB:
// lds_dma_base sets M0 once, load_to_lds_16_at<IMM> adds IMM (< 4096) to it. The instruction's
// offset field moves the address in memory by IMM as well: the caller takes it off thread_off
// (biasing the descriptor's base downwards keeps that offset from going negative). M0 has to
// stay as it is between the parts; the compiler does not know that it is live, so a kernel that
// uses the pair may contain nothing else that writes M0 (zdraw_amd.build.m0_writes lists what a
// compiled file holds).
__device__ __forceinline__ void lds_dma_base(unsigned lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0" : : "s"(lds_addr) : "memory", "m0");
}
template <int IMM>
__device__ __forceinline__ void load_to_lds_16_at(u32x4 rsrc, unsigned thread_off, unsigned uniform_off) {
    static_assert(IMM >= 0 && IMM < 4096, "12-bit instruction offset");
    asm volatile("buffer_load_dwordx4 %0, %1, %2 offen offset:%3 lds" : : "v"(thread_off), "s"(rsrc), "s"(uniform_off), "n"(IMM) : "memory");
}

__device__ __forceinline__ void unpack8(const Raw8<float>& r, float (&x)[8]) {
#pragma unroll
    for (int i = 0; i < 4; i++) { x[i] = r.a[i]; x[4 + i] = r.b[i]; }
}
__device__ __forceinline__ void unpack8(const Raw8<bf16_t>& r, float (&x)[8]) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
        x[2 * i] = __uint_as_float(r.r[i] << 16);
        x[2 * i + 1] = __uint_as_float(r.r[i] & 0xffff0000u);
    }
}
__device__ __forceinline__ void unpack8(const Raw8<f16_t>& r, float (&x)[8]) {
    const f16x8 h = __builtin_bit_cast(f16x8, r.r);
#pragma unroll
    for (int i = 0; i < 8; i++) x[i] = (float)h[i];
}

// fp32 -> bf16, round to nearest even (v_cvt_pk_bf16_f32).
__device__ __forceinline__ u32x4 pack_bf16x8(const float (&x)[8]) {
    f32x8 v;
#pragma unroll
    for (int i = 0; i < 8; i++) v[i] = x[i];
    bf16x8 b = __builtin_convertvector(v, bf16x8);
    return __builtin_bit_cast(u32x4, b);
}
// fp32 -> IEEE half, round to nearest even. Values past the half range saturate at +-65504,
// as the reference's staging kernels clamp them (metal_api.m:6138).
__device__ __forceinline__ u32x4 pack_f16x8(const float (&x)[8]) {
    f16x8 h;
#pragma unroll
    for (int i = 0; i < 8; i++) h[i] = (f16_t)fminf(fmaxf(x[i], -65504.0f), 65504.0f);
    return __builtin_bit_cast(u32x4, h);
}
__device__ __forceinline__ u32x4 raw_to_bf16(const Raw8<bf16_t>& r) { return r.r; }
__device__ __forceinline__ u32x4 raw_to_bf16(const Raw8<float>& r) {
    float x[8];
    unpack8(r, x);
    return pack_bf16x8(x);
}

// Two consecutive elements of one V row as a packed bf16 pair.
__device__ __forceinline__ unsigned ld_pair_bf16(const bf16_t* p, bool ok) {
    return ok ? *reinterpret_cast<const unsigned*>(p) : 0u;
}
__device__ __forceinline__ unsigned ld_pair_bf16(const float* p, bool ok) {
    float x0 = 0.f, x1 = 0.f;
    if (ok) {
        const float2 t = *reinterpret_cast<const float2*>(p);
        x0 = t.x;
        x1 = t.y;
    }
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    f32x2 v = {x0, x1};
    return __builtin_bit_cast(unsigned, __builtin_convertvector(v, bf16x2));
}

// v_permlane32_swap with both operands = x returns, on every lane, the values
// held by lane (l % 32) and lane (l % 32) + 32: the two lanes that share a query.
__device__ __forceinline__ float pair_max(float x) {
    u32x2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float pair_sum(float x) {
    u32x2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// ------------------------------------------------------- QK-norm + rope math
// Rope/weight operands for one row; `row` indexes the rope table / positions,
// `tok` is the token index inside its segment (selects the text-row weights).
struct QkRow {
    const float* w;      // 128 weights for this row
    const float* cos_r;  // Klein: table row
    const float* sin_r;
    unsigned long long p0, p1, p2; // Z-Image position
};

__device__ __forceinline__ QkRow qk_row(const QkOps& a, int mode, const float* w, const float* wt, int seg, int tok,
                                        bool ok) {
    QkRow r;
    r.w = (wt != nullptr && tok < a.txt_rows) ? wt : w;
    r.cos_r = r.sin_r = nullptr;
    r.p0 = r.p1 = r.p2 = 0;
    if (mode == kQkKlein) {
        const int64_t row = ok ? (int64_t)seg * a.rope_bs + tok : 0;
        r.cos_r = a.rope_cos + row * D;
        r.sin_r = a.rope_sin + row * D;
    } else if (mode == kQkZimage) {
        const int64_t row = ok ? (int64_t)seg * a.rope_bs + tok : 0;
        const unsigned long long* p = a.pos + row * 3;
        r.p0 = p[0];
        r.p1 = p[1];
        r.p2 = p[2];
    }
    return r;
}

// Rope coefficients for the 8 elements starting at d0 (d0 % 8 == 0):
// Klein: c[i], s[i] straight from the table row (klein/zflux2_dit.zig:213-228
// reads both columns of a pair); Z-Image: 4 (cos,sin) pairs of the element's
// axis (metal/mqk_shader.zig:80-96).
struct Rope8 { f32x4 a, b, c, d; };

__device__ __forceinline__ Rope8 ld_rope8(const QkOps& a, int mode, const QkRow& r, int d0) {
    Rope8 t;
    if (mode == kQkKlein) {
        t.a = *reinterpret_cast<const f32x4*>(r.cos_r + d0);
        t.b = *reinterpret_cast<const f32x4*>(r.cos_r + d0 + 4);
        t.c = *reinterpret_cast<const f32x4*>(r.sin_r + d0);
        t.d = *reinterpret_cast<const f32x4*>(r.sin_r + d0 + 4);
    } else {
        // Every field is read before the choice by axis: a field read inside a conditional
        // becomes one load from a chosen address, which costs a memory round trip for the
        // launch arguments and parks the positions in scratch.
        const int dim0 = a.dim0, dim1 = a.dim1, dim2 = a.dim2;
        const unsigned base0 = a.base0, base1 = a.base1, base2 = a.base2;
        const unsigned len0 = a.len0, len1 = a.len1, len2 = a.len2;
        const unsigned long long q0 = r.p0, q1 = r.p1, q2 = r.p2;
        const int d01 = dim0 + dim1;
        const int axis = d0 < dim0 ? 0 : (d0 < d01 ? 1 : 2);
        const int axis_off = axis == 0 ? 0 : (axis == 1 ? dim0 : d01);
        const unsigned axis_pairs = (unsigned)(axis == 0 ? dim0 : (axis == 1 ? dim1 : dim2)) >> 1;
        const unsigned base = axis == 0 ? base0 : (axis == 1 ? base1 : base2);
        const unsigned long long p_raw = axis == 0 ? q0 : (axis == 1 ? q1 : q2);
        // zimage/zrope.zig:48 refuses pos >= len on the host; a device-resident position is
        // held to the table instead (the axis's last entry)
        const unsigned last = (axis == 0 ? len0 : (axis == 1 ? len1 : len2)) - 1u;
        const unsigned long long p = p_raw < (unsigned long long)last ? p_raw : (unsigned long long)last;
        const unsigned long long idx = base + p * axis_pairs + (unsigned)((d0 - axis_off) >> 1);
        const float* src = a.pairs + idx * 2;
        t.a = *reinterpret_cast<const f32x4*>(src);      // (c0,s0,c1,s1)
        t.b = *reinterpret_cast<const f32x4*>(src + 4);  // (c2,s2,c3,s3)
        t.c = t.a;
        t.d = t.b;
    }
    return t;
}

// x[0..7] (elements d0..d0+7 of a row) -> normalised, weighted (w0, w1 = the 8 norm
// weights of these elements), rotated.
__device__ __forceinline__ void qk_apply8(int mode, float (&x)[8], float inv, const f32x4& w0, const f32x4& w1, const Rope8& t) {
    float y[8];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        y[i] = x[i] * inv * w0[i];
        y[4 + i] = x[4 + i] * inv * w1[i];
    }
    if (mode == kQkKlein) {
        float c[8], s[8];
#pragma unroll
        for (int i = 0; i < 4; i++) { c[i] = t.a[i]; c[4 + i] = t.b[i]; s[i] = t.c[i]; s[4 + i] = t.d[i]; }
#pragma unroll
        for (int i = 0; i < 8; i += 2) {
            x[i] = y[i] * c[i] - y[i + 1] * s[i];
            x[i + 1] = y[i + 1] * c[i + 1] + y[i] * s[i + 1];
        }
    } else {
        const float c[4] = {t.a[0], t.a[2], t.b[0], t.b[2]};
        const float s[4] = {t.a[1], t.a[3], t.b[1], t.b[3]};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            x[2 * i] = y[2 * i] * c[i] - y[2 * i + 1] * s[i];
            x[2 * i + 1] = y[2 * i + 1] * c[i] + y[2 * i] * s[i];
        }
    }
}
// The same with the weights read from memory at w + d0.
__device__ __forceinline__ void qk_apply8(int mode, float (&x)[8], float inv, const float* w, int d0, const Rope8& t) {
    const f32x4 w0 = *reinterpret_cast<const f32x4*>(w + d0);
    const f32x4 w1 = *reinterpret_cast<const f32x4*>(w + d0 + 4);
    qk_apply8(mode, x, inv, w0, w1, t);
}

// Sum across the TPK adjacent lanes that share one K row (TPK = 4, 8 or 16).
template <int TPK>
__device__ __forceinline__ float row_group_sum(float v) {
    // quad_perm [1,0,3,2], quad_perm [2,3,0,1], then row_half_mirror for 8, row_mirror for 16
    v += __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(v), 0xB1, 0xF, 0xF, true));
    v += __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(v), 0x4E, 0xF, 0xF, true));
    if constexpr (TPK >= 8)
        v += __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(v), 0x141, 0xF, 0xF, true));
    if constexpr (TPK == 16) // row_mirror
        v += __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(v), 0x140, 0xF, 0xF, true));
    return v;
}

} // namespace zdraw
