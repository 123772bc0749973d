// gfx950 GEMM for the projections either side of attention:
//   C[m][n] = A[m][k] x W[n][k]^T, 16-bit MFMA, fp32 accumulation.
//
// What it replaces in the reference: the half-mode simdgroup GEMMs behind
// zdraw_metal_run_gemm_enc / _off_enc / _ours16_enc / _f16a_enc
// (metal/mgemm_shader.zig, metal_api.m) that produce Q, K, V from the block
// input and drain the attention output (klein/zflux2_resident.zig:1473-1513,
// 1986-1998). Both operands are K-major (activation rows and weight rows are
// contiguous in k), which is exactly the register layout of
// v_mfma_f32_32x32x16: a lane supplies 8 consecutive k of one row.
//
//   * workgroup tile 256 x 256, K slabs of 64, 8 waves as 4 (M) x 2 (N); a wave
//     owns 64 x 128 of C (2 x 4 MFMA tiles, 128 accumulator registers) and reads
//     6 fragments from LDS per 8 MFMAs;
//   * LDS rows are 144 bytes (64 elements + 8): 16-lane b128 fragment reads hit
//     16 distinct bank groups;
//   * two LDS stages: slab s+1 is written while slab s is computed on, one
//     barrier per slab; global loads (buffer loads, scalar slab offset) run
//     two slabs ahead in registers; with 16-bit activations and whole slabs the
//     loads go from global memory straight into a swizzled LDS layout instead;
//   * fp32 activations are rounded to the weight's 16-bit type on the way
//     into LDS (round to nearest even), so no conversion pass is needed;
//   * fixed summation order, no split-K, no atomics: bit-identical run to run.
#include "attn_device.hpp"
#include "gemm_kernel.h"

namespace zdraw {

namespace gemm {

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int NT = 512;
constexpr int PITCH = BK + 8;                  // elements per LDS row
constexpr int STAGE_ELEMS = (BM + BN) * PITCH; // A rows then W rows
constexpr size_t kLdsBytes = 2 * (size_t)STAGE_ELEMS * 2;

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));

// 8 consecutive k of one row as they come from memory.
template <typename T> struct Chunk { u32x4 r; };
template <> struct Chunk<float> { f32x4 a, b; };

template <typename T>
__device__ __forceinline__ Chunk<T> ld_chunk(rsrc_t rsrc, unsigned voff, unsigned soff) {
    Chunk<T> x;
    if constexpr (std::is_same<T, float>::value) {
        x.a = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)voff, (int)soff, 0));
        x.b = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)(voff + 16), (int)soff, 0));
    } else {
        x.r = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)voff, (int)soff, 0));
    }
    return x;
}

// The chunk as 8 packed 16-bit values of the compute type.
template <typename T, bool F16>
__device__ __forceinline__ u32x4 to_half8(const Chunk<T>& x, bool keep) {
    u32x4 r;
    if constexpr (std::is_same<T, float>::value) {
        f32x8 v;
#pragma unroll
        for (int i = 0; i < 4; i++) { v[i] = x.a[i]; v[4 + i] = x.b[i]; }
        if constexpr (F16) r = __builtin_bit_cast(u32x4, __builtin_convertvector(v, f16x8));
        else r = __builtin_bit_cast(u32x4, __builtin_convertvector(v, bf16x8));
    } else {
        r = x.r;
    }
    return keep ? r : u32x4{0u, 0u, 0u, 0u};
}

template <bool F16>
__device__ __forceinline__ f32x16 mfma(const u32x4& a, const u32x4& b, const f32x16& c) {
    if constexpr (F16)
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

// A wave's (32 TM) x (32 TN) block of C: lane holds column col0 + 32 j + l32, rows row0 + 32 i + 8 r + 4 h + jj.
template <bool F16, typename TC, int TM, int TN>
__device__ __forceinline__ void store_tile(const GemmArgs& g, void* c, const f32x16 (&acc)[TM][TN], int row0, int col0, int l32, int h) {
#pragma unroll
    for (int i = 0; i < TM; i++) {
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int col = col0 + j * 32 + l32;
#pragma unroll
            for (int r = 0; r < 4; r++) {
#pragma unroll
                for (int jj = 0; jj < 4; jj++) {
                    const int row = row0 + i * 32 + 8 * r + 4 * h + jj;
                    if (row < g.m && col < g.n) {
                        const float v = acc[i][j][4 * r + jj];
                        TC* dst = reinterpret_cast<TC*>(c) + (int64_t)row * g.ldc + col;
                        if constexpr (std::is_same<TC, float>::value) *dst = v;
                        else if constexpr (F16) *reinterpret_cast<_Float16*>(dst) = (_Float16)v;
                        else *reinterpret_cast<bf16_t*>(dst) = (bf16_t)v;
                    }
                }
            }
        }
    }
}

// XCD-aware tile id: consecutive logical tiles (one row of C tiles) share an XCD's L2
__device__ __forceinline__ int logical_tile() {
    const int nwg = gridDim.x;
    const int xcd = blockIdx.x & 7;
    const int idx = blockIdx.x >> 3;
    const int base = nwg >> 3;
    const int rem = nwg & 7;
    return idx + xcd * base + (xcd < rem ? xcd : rem);
}

// TA: float or a 16-bit type (then it is the compute type); F16: compute type is
// IEEE half instead of bf16; TC: float or a 16-bit type.
template <typename TA, bool F16, typename TC>
__global__ void __launch_bounds__(NT, 2) gemm_kernel(const GemmArgs g) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    unsigned short* const lds = reinterpret_cast<unsigned short*>(smem);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int l32 = lane & 31;
    const int h = lane >> 5;
    const int wm = wave >> 1, wn = wave & 1;

    const int logical = logical_tile();
    // the groups lie side by side along n: one row of tiles reads the same rows of A
    const int tiles_row = g.tiles_n * g.groups;
    const int tm = logical / tiles_row;
    int tn = logical - tm * tiles_row;
    const int grp = tn / g.tiles_n;
    tn -= grp * g.tiles_n;
    const void* const wp = grp == 0 ? g.w : g.w_more[grp - 1];
    void* const cp = grp == 0 ? g.c : g.c_more[grp - 1];
    const int m0 = tm * BM, n0 = tn * BN;

    // ---- staging: thread t owns 16-byte chunk t%8 of rows t/8 + 64 j (j < 4) of the A slab and of the W slab
    constexpr unsigned ea = sizeof(TA);
    const unsigned a_span = ((unsigned)(g.m - 1) * (unsigned)g.lda + (unsigned)g.k) * ea;
    const unsigned w_span = ((unsigned)(g.n - 1) * (unsigned)g.ldw + (unsigned)g.k) * 2u;
    const rsrc_t a_rsrc = make_rsrc(g.a, a_span);
    const rsrc_t w_rsrc = make_rsrc(wp, w_span);
    const int lr = tid >> 3;
    const int kc = tid & 7;
    unsigned a_off[4], w_off[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int ar = min(m0 + lr + 64 * j, g.m - 1); // rows past the edge re-read the last row; never stored
        const int wr = min(n0 + lr + 64 * j, g.n - 1);
        a_off[j] = ((unsigned)ar * (unsigned)g.lda + (unsigned)(kc * 8)) * ea;
        w_off[j] = ((unsigned)wr * (unsigned)g.ldw + (unsigned)(kc * 8)) * 2u;
    }
    const int nslab = (g.k + BK - 1) / BK;

    Chunk<TA> ra[4];
    Chunk<unsigned short> rw[4];
    auto load_slab = [&](int s) __attribute__((always_inline)) {
        const int ss = s < nslab ? s : nslab - 1; // past the end: a harmless re-read
#pragma unroll
        for (int j = 0; j < 4; j++) {
            ra[j] = ld_chunk<TA>(a_rsrc, a_off[j], (unsigned)ss * (BK * ea));
            rw[j] = ld_chunk<unsigned short>(w_rsrc, w_off[j], (unsigned)ss * (BK * 2u));
        }
    };
    auto store_slab = [&](int s) __attribute__((always_inline)) {
        unsigned short* st = lds + (s & 1) * STAGE_ELEMS;
        // chunks past k contribute zeros; only the last slab of a k that is not a multiple of 64 has any
        const bool ragged = (s + 1) * BK > g.k; // wave-uniform
        const bool keep = !ragged || s * BK + kc * 8 < g.k;
        if (ragged) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                *reinterpret_cast<u32x4*>(st + (lr + 64 * j) * PITCH + kc * 8) = to_half8<TA, F16>(ra[j], keep);
                *reinterpret_cast<u32x4*>(st + (BM + lr + 64 * j) * PITCH + kc * 8) = to_half8<unsigned short, F16>(rw[j], keep);
            }
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                *reinterpret_cast<u32x4*>(st + (lr + 64 * j) * PITCH + kc * 8) = to_half8<TA, F16>(ra[j], true);
                *reinterpret_cast<u32x4*>(st + (BM + lr + 64 * j) * PITCH + kc * 8) = to_half8<unsigned short, F16>(rw[j], true);
            }
        }
    };

    f32x16 acc[2][4];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    load_slab(0);
    store_slab(0);
    load_slab(1);
    __syncthreads();

    const int a_frag = (wm * 64 + l32) * PITCH + 8 * h;
    const int w_frag = (BM + wn * 128 + l32) * PITCH + 8 * h;
    for (int s = 0; s < nslab; s++) {
        const unsigned short* st = lds + (s & 1) * STAGE_ELEMS;
#pragma unroll
        for (int kk = 0; kk < BK / 16; kk++) {
            u32x4 af[2], wf[4];
#pragma unroll
            for (int i = 0; i < 2; i++) af[i] = *reinterpret_cast<const u32x4*>(st + a_frag + i * 32 * PITCH + kk * 16);
#pragma unroll
            for (int j = 0; j < 4; j++) wf[j] = *reinterpret_cast<const u32x4*>(st + w_frag + j * 32 * PITCH + kk * 16);
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 4; j++) acc[i][j] = mfma<F16>(af[i], wf[j], acc[i][j]);
            if (kk == 0) {
                // slab s+1 (in registers since the previous iteration) goes to the other stage,
                // whose readers finished before the last barrier; then slab s+2 starts loading.
                // The fences keep the loads here: sunk to the end of the iteration they would
                // be waited for as soon as they are issued.
                __builtin_amdgcn_sched_barrier(0);
                store_slab(s + 1);
                load_slab(s + 2);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        __syncthreads();
    }

    store_tile<F16, TC, 2, 4>(g, cp, acc, m0 + wm * 64, n0 + wn * 128, l32, h);
}

// The same tile with 16-bit activations and k a multiple of 64: both slabs go
// from global memory straight into LDS (buffer_load ... lds), no staging
// registers and no LDS store instructions. Such a load writes lane i's 16 bytes
// at (LDS base) + 16 i, so rows are 128 bytes with no padding and bank conflicts
// are avoided by a swizzle instead: the 16-byte chunk c of row r lives at chunk
// position c ^ ((r >> 1) & 7); the lane that fills position p of row r fetches
// logical chunk p ^ ((r >> 1) & 7) from memory. A 16-lane fragment read of one
// logical chunk over 16 consecutive rows then touches 16 distinct bank groups.
constexpr int DMA_STAGE_BYTES = (BM + BN) * BK * 2; // 64 KB
constexpr size_t kDmaLdsBytes = 2 * (size_t)DMA_STAGE_BYTES;

// WM x WN waves; a wave owns (256 / WM) x (256 / WN) of C. 4 x 2 waves run two per SIMD
// with 64 x 128 each; 2 x 2 waves run one per SIMD with 128 x 128 each (256 accumulator
// registers), which reads a third fewer LDS bytes per MFMA.
template <bool F16, typename TC, int WM, int WN>
__global__ void __launch_bounds__(WM * WN * 64, (WM * WN) / 4) gemm_dma_kernel(const GemmArgs g) {
    constexpr int NW = WM * WN;
    constexpr int TM = BM / WM / 32, TN = BN / WN / 32; // 32 x 32 MFMA tiles per wave
    constexpr int RW = BM / NW;                           // slab rows a wave fetches, of A and of W
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    typedef __attribute__((address_space(3))) void* lds_ptr_t;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int l32 = lane & 31;
    const int h = lane >> 5;
    const int wm = wave / WN, wn = wave % WN;
    const int logical = logical_tile();
    // the groups lie side by side along n: one row of tiles reads the same rows of A
    const int tiles_row = g.tiles_n * g.groups;
    const int tm = logical / tiles_row;
    int tn = logical - tm * tiles_row;
    const int grp = tn / g.tiles_n;
    tn -= grp * g.tiles_n;
    const void* const wp = grp == 0 ? g.w : g.w_more[grp - 1];
    void* const cp = grp == 0 ? g.c : g.c_more[grp - 1];
    const int m0 = tm * BM, n0 = tn * BN;

    const unsigned a_span = ((unsigned)(g.m - 1) * (unsigned)g.lda + (unsigned)g.k) * 2u;
    const unsigned w_span = ((unsigned)(g.n - 1) * (unsigned)g.ldw + (unsigned)g.k) * 2u;
    const rsrc_t a_rsrc = make_rsrc(g.a, a_span);
    const rsrc_t w_rsrc = make_rsrc(wp, w_span);
    // wave w fills rows RW w + 8 j + lane / 8 (j < RW / 8) of the A slab and of the W slab
    unsigned a_off[RW / 8], w_off[RW / 8];
#pragma unroll
    for (int j = 0; j < RW / 8; j++) {
        const int r = wave * RW + j * 8 + (lane >> 3);
        const int c = (lane & 7) ^ ((r >> 1) & 7);
        const int ar = min(m0 + r, g.m - 1); // rows past the edge re-read the last row; never stored
        const int wr = min(n0 + r, g.n - 1);
        a_off[j] = ((unsigned)ar * (unsigned)g.lda + (unsigned)(c * 8)) * 2u;
        w_off[j] = ((unsigned)wr * (unsigned)g.ldw + (unsigned)(c * 8)) * 2u;
    }
    const int nslab = g.k / BK;
    auto fetch_slab = [&](int s) __attribute__((always_inline)) {
        unsigned char* st = smem + (s & 1) * DMA_STAGE_BYTES + wave * (RW * BK * 2);
#pragma unroll
        for (int j = 0; j < RW / 8; j++) {
            __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, (lds_ptr_t)(st + j * (8 * BK * 2)), 16, (int)a_off[j],
                                                     (int)((unsigned)s * (BK * 2u)), 0, 0);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(w_rsrc, (lds_ptr_t)(st + BM * BK * 2 + j * (8 * BK * 2)), 16,
                                                     (int)w_off[j], (int)((unsigned)s * (BK * 2u)), 0, 0);
        }
    };

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    // fragment addresses: row (.. + l32), logical chunk 2 kk + h at position (2 kk + h) ^ ((l32 >> 1) & 7)
    const int sw = (l32 >> 1) & 7;
    const int a_row = (wm * (32 * TM) + l32) * (BK * 2);
    const int w_row = BM * BK * 2 + (wn * (32 * TN) + l32) * (BK * 2);
    struct Frag { u32x4 a[TM], w[TN]; };
    auto read_frag = [&](Frag& f, int s, int kk) __attribute__((always_inline)) {
        const unsigned char* st = smem + (s & 1) * DMA_STAGE_BYTES;
        const int pos = ((2 * kk + h) ^ sw) * 16;
#pragma unroll
        for (int i = 0; i < TM; i++) f.a[i] = *reinterpret_cast<const u32x4*>(st + a_row + i * 32 * (BK * 2) + pos);
#pragma unroll
        for (int j = 0; j < TN; j++) f.w[j] = *reinterpret_cast<const u32x4*>(st + w_row + j * 32 * (BK * 2) + pos);
    };
    auto mfma_frag = [&](const Frag& f) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++) acc[i][j] = mfma<F16>(f.a[i], f.w[j], acc[i][j]);
    };

    fetch_slab(0);
    __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0): this wave's part of slab 0 is in LDS
    __syncthreads();
    for (int s = 0; s < nslab; s++) {
        // slab s+1 into the other stage: its readers (iteration s-1) are behind the last barrier
        if (s + 1 < nslab) fetch_slab(s + 1);
#pragma unroll
        for (int kk = 0; kk < BK / 16; kk++) {
            Frag f;
            read_frag(f, s, kk);
            mfma_frag(f);
        }
        __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0): slab s+1 has landed
        __syncthreads();
    }
    store_tile<F16, TC, TM, TN>(g, cp, acc, m0 + wm * (32 * TM), n0 + wn * (32 * TN), l32, h);
}

// Measured on the Klein projections: 4 x 2 waves (two per SIMD, 64 x 128 each) 1090-1220
// TFLOP/s; 2 x 2 waves (one per SIMD, 128 x 128 each, fewer LDS reads) 960-1120.
constexpr int DMA_WM = 4, DMA_WN = 2;

template <typename TA, bool F16, typename TC>
static hipError_t launch_one(const GemmArgs& g, hipStream_t stream) {
    const int64_t tiles_m = (g.m + BM - 1) / BM;
    const int64_t nwg = tiles_m * g.tiles_n * g.groups;
    if (nwg <= 0 || nwg > 0x7fffffff) return hipErrorInvalidValue;
    if constexpr (!std::is_same<TA, float>::value) {
        if (g.k % BK == 0) { // whole slabs of 16-bit activations: the direct-to-LDS build
            gemm_dma_kernel<F16, TC, DMA_WM, DMA_WN><<<dim3((unsigned)nwg), dim3(DMA_WM * DMA_WN * 64), kDmaLdsBytes, stream>>>(g);
            return hipGetLastError();
        }
    }
    gemm_kernel<TA, F16, TC><<<dim3((unsigned)nwg), dim3(NT), kLdsBytes, stream>>>(g);
    return hipGetLastError();
}

template <typename TA, bool F16, typename TC>
static hipError_t raise_lds() {
    if constexpr (!std::is_same<TA, float>::value) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_dma_kernel<F16, TC, DMA_WM, DMA_WN>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)kDmaLdsBytes);
        if (e != hipSuccess) return e;
    }
    return hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_kernel<TA, F16, TC>),
                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsBytes);
}

} // namespace gemm

int gemm_tile_rows() { return gemm::BM; }
int gemm_tile_cols() { return gemm::BN; }

hipError_t launch_gemm(const GemmArgs& g, int a_dtype, int w_dtype, int c_dtype, hipStream_t stream) {
    using namespace gemm;
    typedef unsigned short h16; // a 16-bit operand in the compute type (bf16 or f16 per the weight)
    if (w_dtype == kBF16) {
        if (a_dtype == kF32 && c_dtype == kF32) return launch_one<float, false, float>(g, stream);
        if (a_dtype == kF32 && c_dtype == kBF16) return launch_one<float, false, h16>(g, stream);
        if (a_dtype == kBF16 && c_dtype == kF32) return launch_one<h16, false, float>(g, stream);
        if (a_dtype == kBF16 && c_dtype == kBF16) return launch_one<h16, false, h16>(g, stream);
    } else if (w_dtype == kF16) {
        if (a_dtype == kF32 && c_dtype == kF32) return launch_one<float, true, float>(g, stream);
        if (a_dtype == kF32 && c_dtype == kF16) return launch_one<float, true, h16>(g, stream);
        if (a_dtype == kF16 && c_dtype == kF32) return launch_one<h16, true, float>(g, stream);
        if (a_dtype == kF16 && c_dtype == kF16) return launch_one<h16, true, h16>(g, stream);
    }
    return hipErrorInvalidValue;
}

hipError_t gemm_setup() {
    using namespace gemm;
    typedef unsigned short h16;
    hipError_t e;
    if ((e = raise_lds<float, false, float>()) != hipSuccess) return e;
    if ((e = raise_lds<float, false, h16>()) != hipSuccess) return e;
    if ((e = raise_lds<h16, false, float>()) != hipSuccess) return e;
    if ((e = raise_lds<h16, false, h16>()) != hipSuccess) return e;
    if ((e = raise_lds<float, true, float>()) != hipSuccess) return e;
    if ((e = raise_lds<float, true, h16>()) != hipSuccess) return e;
    if ((e = raise_lds<h16, true, float>()) != hipSuccess) return e;
    if ((e = raise_lds<h16, true, h16>()) != hipSuccess) return e;
    return hipSuccess;
}

} // namespace zdraw
