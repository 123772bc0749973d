// gfx950 GEMM for the projections either side of attention:
//   C[m][n] = A[m][k] x W[n][k]^T, 16-bit MFMA, fp32 accumulation.
//
// What it replaces in the reference: the half-mode simdgroup GEMMs behind
// zdraw_metal_run_gemm_enc / _off_enc / _ours16_enc / _f16a_enc
// (metal/mgemm_shader.zig, metal_api.m) that produce Q, K, V from the block
// input and drain the attention output (klein/zflux2_resident.zig:1473-1513,
// 1986-1998). Both operands are K-major (activation rows and weight rows are
// contiguous in k), which is exactly the register layout of the 16-bit MFMAs
// (v_mfma_f32_16x16x32 in the direct-to-LDS builds, v_mfma_f32_32x32x16 in the
// register-staged one): a lane supplies 8 consecutive k of one row.
//
// Three builds share the tile walk, the operand layout and the epilogue:
//   * f32 activations, or k not a multiple of 64: workgroup tile 256 x 256, K slabs of
//     64, 8 waves as 4 (M) x 2 (N), a wave owns 64 x 128 of C; global loads (buffer
//     loads, scalar slab offset) run two slabs ahead in registers and are rounded to the
//     weight's 16-bit type on the way into padded LDS rows (144 bytes: 16-lane b128
//     fragment reads hit 16 distinct bank groups), so no conversion pass is needed;
//   * 16-bit activations, whole slabs, enough 256-tiles to fill the chip (the default for
//     the projections): 4 waves, one per SIMD, each owning 128 x 128 of C, slabs fetched
//     from global memory straight into swizzled, unpadded LDS rows (gemm_ring_kernel);
//     the same tile with 8 waves is kept behind a knob;
//   * the same with too few 256-tiles: 128 x 128 tiles, 4 waves, two workgroups per CU;
//   * two or three products of one A with equal shapes (q/k/v, gate/up) run as one launch
//     whose tiles cover all of them;
//   * fixed summation order and no atomics (a thinly filled last round is cut along k and
//     merged in part order): bit-identical run to run.
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

// v_mfma_f32_16x16x32: a lane supplies 8 consecutive k (chunk lane / 16 of the 32) of row lane % 16
// and receives, of the 16 x 16 result, row lane % 16 of the second operand against rows
// 4 (lane / 16) .. + 3 of the first. Per FLOP it moves half the accumulator bytes of the 32 x 32
// form through the register file, and at the board's power limit that is worth clock.
// Written as assembly with the accumulator tied to the result: given the builtin, the compiler
// picks the three-address form for these 64 four-register accumulators and then moves them
// around the accumulation file inside the loop (several copies per MFMA). The compiler inserts
// no hazard waits around assembly: the caller keeps dependent MFMAs apart (here 64 MFMAs) and
// calls mfma16_drain() in the same basic block as the last MFMA, before control can reach code
// the compiler may have placed on its own (copies or spills of the accumulators at a join): a
// result read within the MFMA's four passes is the old value.
template <bool F16>
__device__ __forceinline__ void mfma16(const u32x4& a, const u32x4& b, f32x4& c) {
    if constexpr (F16) asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
    else asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}
__device__ __forceinline__ void mfma16_drain() {
    asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");
}

// A wave's (32 TM) x (32 TN) block of C. The MFMAs take the W fragment as their first
// operand, so a lane holds row row0 + 32 i + l32 of C and, in register 4 r + jj of tile
// (i, j), column col0 + 32 j + 8 r + 4 h + jj: four consecutive columns per r, stored as
// one 8- or 16-byte vector where the row pitch and the base allow it.
template <bool F16, typename TC, int TM, int TN>
__device__ __forceinline__ void store_tile(const GemmArgs& g, void* c, const f32x16 (&acc)[TM][TN], int row0, int col0, int l32, int h) {
    // uniform over the launch: every group of four columns starts aligned for a vector store
    const bool vec = (g.ldc % 4 == 0) && ((reinterpret_cast<uintptr_t>(c) % (4 * sizeof(TC))) == 0);
#pragma unroll
    for (int i = 0; i < TM; i++) {
        const int row = row0 + i * 32 + l32;
        if (row >= g.m) continue;
        TC* const crow = reinterpret_cast<TC*>(c) + (int64_t)row * g.ldc;
#pragma unroll
        for (int j = 0; j < TN; j++) {
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int col = col0 + j * 32 + 8 * r + 4 * h;
                const f32x4 v = f32x4{acc[i][j][4 * r], acc[i][j][4 * r + 1], acc[i][j][4 * r + 2], acc[i][j][4 * r + 3]};
                if (vec && col + 3 < g.n) {
                    if constexpr (std::is_same<TC, float>::value) *reinterpret_cast<f32x4*>(crow + col) = v;
                    else if constexpr (F16) *reinterpret_cast<f16x4*>(crow + col) = __builtin_convertvector(v, f16x4);
                    else *reinterpret_cast<bf16x4*>(crow + col) = __builtin_convertvector(v, bf16x4);
                } else {
#pragma unroll
                    for (int jj = 0; jj < 4; jj++) {
                        if (col + jj < g.n) {
                            TC* dst = crow + col + jj;
                            if constexpr (std::is_same<TC, float>::value) *dst = v[jj];
                            else if constexpr (F16) *reinterpret_cast<_Float16*>(dst) = (_Float16)v[jj];
                            else *reinterpret_cast<bf16_t*>(dst) = (bf16_t)v[jj];
                        }
                    }
                }
            }
        }
    }
}

// A wave's (16 TI) x (16 TJ) block of C from 16 x 16 x 32 MFMAs. They take the W fragment as
// their first operand, so a lane (c = lane % 16, q = lane / 16) holds row row0 + 16 i + c of C
// and, in tile (i, j), columns col0 + 16 j + 4 q .. + 3: a store instruction covers 16 rows x 64
// contiguous bytes of f32.
template <bool F16, typename TC, int TI, int TJ>
__device__ __forceinline__ void store_tile16(const GemmArgs& g, void* c, const f32x4 (&acc)[TI][TJ], int row0, int col0, int lane) {
    const int c16 = lane & 15, q = lane >> 4;
    const bool vec = (g.ldc % 4 == 0) && ((reinterpret_cast<uintptr_t>(c) % (4 * sizeof(TC))) == 0);
#pragma unroll
    for (int i = 0; i < TI; i++) {
        const int row = row0 + 16 * i + c16;
        if (row >= g.m) continue;
        TC* const crow = reinterpret_cast<TC*>(c) + (int64_t)row * g.ldc;
#pragma unroll
        for (int j = 0; j < TJ; j++) {
            const int col = col0 + 16 * j + 4 * q;
            const f32x4 v = acc[i][j];
            if (vec && col + 4 <= g.n) {
                if constexpr (std::is_same<TC, float>::value) *reinterpret_cast<f32x4*>(crow + col) = v;
                else if constexpr (F16) *reinterpret_cast<u32x2*>(crow + col) = __builtin_bit_cast(u32x2, __builtin_convertvector(v, f16x4));
                else *reinterpret_cast<u32x2*>(crow + col) = __builtin_bit_cast(u32x2, __builtin_convertvector(v, bf16x4));
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    if (col + e >= g.n) break;
                    if constexpr (std::is_same<TC, float>::value) crow[col + e] = v[e];
                    else if constexpr (F16) { const _Float16 x = (_Float16)v[e]; crow[col + e] = __builtin_bit_cast(unsigned short, x); }
                    else { const bf16_t x = (bf16_t)v[e]; crow[col + e] = __builtin_bit_cast(unsigned short, x); }
                }
            }
        }
    }
}

// The same block for a 16-bit C, as whole rows of the block (32 TJ bytes: 256 for TJ = 8, 128
// for TJ = 4): the wave turns 32 rows at a time (two rows of tiles) through LDS of its own
// (32 x 32 TJ bytes at lds_wave), so it needs no barrier of its own; the caller sees to it that
// nobody else uses that LDS any more. Staged rows are unpadded; the 16-byte chunk c of row r
// sits at c ^ (r & 15) in 256-byte rows and at c ^ ((r >> 1) & 7) in 128-byte rows, which
// spreads both the 8-byte writes (16 rows x 2 halves per half wave) and the row-wise reads over
// all banks. A wave's LDS operations complete in order, so the reads of one pass see its
// writes and the next pass's writes follow its reads. Rows of C that do not start on 16 bytes,
// and the columns past n, are stored element by element.
constexpr int kEpiWaveBytes = 32 * 256;
template <bool F16, typename TC, int TI, int TJ>
__device__ __forceinline__ void store_tile_lds16(const GemmArgs& g, void* c, const f32x4 (&acc)[TI][TJ], unsigned lds_wave, int row0, int col0, int lane) {
    static_assert(sizeof(TC) == 2, "16-bit C only");
    static_assert((TJ == 8 || TJ == 4) && TI % 2 == 0, "blocks of 128 or 64 columns, rows in pairs of tiles");
    constexpr int ROWB = 32 * TJ;   // bytes per staged row
    constexpr int NCH = 2 * TJ;     // 16-byte chunks per row
    constexpr int RPI = 64 / NCH;   // rows per read-back instruction
    typedef __attribute__((address_space(3))) u32x2* lds_u32x2_t;
    typedef const __attribute__((address_space(3))) u32x4* lds_u32x4_t;
    auto swz = [](int r) { return TJ == 8 ? (r & 15) : ((r >> 1) & 7); };
    const int c16 = lane & 15, q = lane >> 4;
    // write: row 16 (i & 1) + c16, bytes 32 j + 8 q .. + 8 = chunk 2 j + q / 2, half q & 1
    const unsigned wbase = lds_wave + (unsigned)(c16 * ROWB + (q & 1) * 8);
    const unsigned wsw = (unsigned)(swz(c16) ^ (q >> 1)); // (2 j + q / 2) ^ s = (2 j) ^ (s ^ (q / 2))
    // read: row RPI p + lane / NCH (p < 32 / RPI), chunk lane % NCH
    const int rr = lane / NCH, ch = lane % NCH;
    const int col = col0 + 8 * ch;
    // (uniform over the launch: rows of C start on 16 bytes; otherwise element by element)
    const bool whole = col + 8 <= g.n && (g.ldc % 8 == 0) && (reinterpret_cast<uintptr_t>(c) % 16 == 0);
    unsigned short* const cbase = reinterpret_cast<unsigned short*>(c) + (int64_t)(row0 + rr) * g.ldc + col;
#pragma unroll
    for (int ip = 0; ip < TI / 2; ip++) {
#pragma unroll
        for (int ii = 0; ii < 2; ii++)
#pragma unroll
            for (int j = 0; j < TJ; j++) {
                const f32x4 v = acc[2 * ip + ii][j];
                u32x2 pk;
                if constexpr (F16) pk = __builtin_bit_cast(u32x2, __builtin_convertvector(v, f16x4));
                else pk = __builtin_bit_cast(u32x2, __builtin_convertvector(v, bf16x4));
                // (rows 16 .. 31 swizzle as rows 0 .. 15 do: both forms of swz ignore bit 4)
                *(lds_u32x2_t)(wbase + (unsigned)(ii * 16 * ROWB) + (((unsigned)(2 * j) ^ wsw) * 16u)) = pk;
            }
        __builtin_amdgcn_sched_barrier(0); // (keeps the scheduler from reading every accumulator out at once)
        u32x4 v[32 / RPI];
#pragma unroll
        for (int p2 = 0; p2 < 32 / RPI; p2++) {
            const int r = RPI * p2 + rr;
            v[p2] = *(lds_u32x4_t)(lds_wave + (unsigned)(r * ROWB) + (unsigned)((ch ^ swz(r)) * 16));
        }
#pragma unroll
        for (int p2 = 0; p2 < 32 / RPI; p2++) {
            const int row = row0 + 32 * ip + RPI * p2 + rr;
            if (row >= g.m) continue;
            unsigned short* const dst = cbase + (int64_t)(32 * ip + RPI * p2) * g.ldc;
            if (whole) {
                *reinterpret_cast<u32x4*>(dst) = v[p2];
            } else {
#pragma unroll
                for (int e = 0; e < 8; e++)
                    if (col + e < g.n) dst[e] = (unsigned short)(v[p2][e >> 1] >> (16 * (e & 1)));
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    }
}

// XCD-aware tile id: workgroups go to the XCDs in turn, so each XCD gets one contiguous
// run of the tile sequence
__device__ __forceinline__ int logical_tile(int wg, int nwg) {
    const int xcd = wg & 7;
    const int idx = wg >> 3;
    const int base = nwg >> 3;
    const int rem = nwg & 7;
    return idx + xcd * base + (xcd < rem ? xcd : rem);
}

// Order of the tiles within that sequence: strips of kStrip tile columns (the groups lie side
// by side along n), walked row by row. The 32 tiles an XCD works on at one time then cover
// about 4 x 8 tiles of C and share 12 row panels of A and W in its L2; in row-major order
// they are 1 x 32 and share 33 (measured on a 4608 x 3072 x 9216 product: 1.08 GB of L2
// misses per launch against 0.50 GB). The last strip takes the columns that are left.
constexpr int kStrip = 8;
__device__ __forceinline__ void tile_coords(int logical, int tiles_m, int tiles_row, int& tm, int& tn) {
    const int per_strip = kStrip * tiles_m;
    const int nfull = tiles_row / kStrip;
    int strip = logical / per_strip;
    int width = kStrip;
    if (strip >= nfull) {
        strip = nfull;
        width = tiles_row - nfull * kStrip;
    }
    const int r = logical - strip * per_strip;
    tm = r / width;
    tn = strip * kStrip + (r - tm * width);
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

    const int logical = logical_tile((int)blockIdx.x, (int)gridDim.x);
    const int tiles_row = g.tiles_n * g.groups;
    int tm, tn;
    tile_coords(logical, (g.m + BM - 1) / BM, tiles_row, tm, tn);
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
                for (int j = 0; j < 4; j++) acc[i][j] = mfma<F16>(wf[j], af[i], acc[i][j]);
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

// TB x TB tile of C, WM x WN waves, a wave owns (TB / WM) x (TB / WN). Built as 256 with
// 4 x 2 waves (two per SIMD, 64 x 128 each) and as 128 with 2 x 2 waves (64 x 64 each, 64 KB
// of LDS, two workgroups per CU) for problems with too few 256-tiles to fill the chip.
template <bool F16, typename TC, int WM, int WN, int TB>
__global__ void __launch_bounds__(WM * WN * 64, 2) gemm_dma_kernel(const GemmArgs g) {
    constexpr int STAGE_BYTES = 2 * TB * BK * 2; // A rows then W rows
    constexpr int NW = WM * WN;
    constexpr int TM = TB / WM / 16, TN = TB / WN / 16; // 16 x 16 MFMA tiles per wave
    constexpr int RW = TB / NW;                           // slab rows a wave fetches, of A and of W
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    typedef __attribute__((address_space(3))) void* lds_ptr_t;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int c16 = lane & 15;
    const int q4 = lane >> 4;
    const int wm = wave / WN, wn = wave % WN;
    const int logical = logical_tile((int)blockIdx.x, (int)gridDim.x);
    const int tiles_row = g.tiles_n * g.groups;
    int tm, tn;
    tile_coords(logical, (g.m + TB - 1) / TB, tiles_row, tm, tn);
    const int grp = tn / g.tiles_n;
    tn -= grp * g.tiles_n;
    const void* const wp = grp == 0 ? g.w : g.w_more[grp - 1];
    void* const cp = grp == 0 ? g.c : g.c_more[grp - 1];
    const int m0 = tm * TB, n0 = tn * TB;

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
        unsigned char* st = smem + (s & 1) * STAGE_BYTES + wave * (RW * BK * 2);
#pragma unroll
        for (int j = 0; j < RW / 8; j++) {
            __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, (lds_ptr_t)(st + j * (8 * BK * 2)), 16, (int)a_off[j],
                                                     (int)((unsigned)s * (BK * 2u)), 0, 0);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(w_rsrc, (lds_ptr_t)(st + TB * BK * 2 + j * (8 * BK * 2)), 16,
                                                     (int)w_off[j], (int)((unsigned)s * (BK * 2u)), 0, 0);
        }
    };

    f32x4 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    // fragment addresses: row (.. + c16), logical chunk 4 ks + q4 at position (4 ks + q4) ^ ((c16 >> 1) & 7)
    const int sw = (c16 >> 1) & 7;
    const int a_row = (wm * (16 * TM) + c16) * (BK * 2);
    const int w_row = TB * BK * 2 + (wn * (16 * TN) + c16) * (BK * 2);
    struct Frag { u32x4 a[TM], w[TN]; };
    auto read_frag = [&](Frag& f, int s, int ks) __attribute__((always_inline)) {
        const unsigned char* st = smem + (s & 1) * STAGE_BYTES;
        const int pos = ((4 * ks + q4) ^ sw) * 16;
#pragma unroll
        for (int i = 0; i < TM; i++) f.a[i] = *reinterpret_cast<const u32x4*>(st + a_row + i * 16 * (BK * 2) + pos);
#pragma unroll
        for (int j = 0; j < TN; j++) f.w[j] = *reinterpret_cast<const u32x4*>(st + w_row + j * 16 * (BK * 2) + pos);
    };
    // (The builtin form: with this few accumulators the compiler keeps them in place, and it
    // adds the wait states itself.)
    auto mfma_frag = [&](const Frag& f) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++) {
                if constexpr (F16)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, f.w[j]), __builtin_bit_cast(f16x8, f.a[i]), acc[i][j], 0, 0, 0);
                else
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, f.w[j]), __builtin_bit_cast(bf16x8, f.a[i]), acc[i][j], 0, 0, 0);
            }
    };

    fetch_slab(0);
    __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0): this wave's part of slab 0 is in LDS
    __syncthreads();
    for (int s = 0; s < nslab; s++) {
        // slab s+1 into the other stage: its readers (iteration s-1) are behind the last barrier.
        // (Spreading these loads over the four steps measured 9 % slower here: the compiler
        // then makes the fragment reads that follow each load wait for it.)
        if (s + 1 < nslab) fetch_slab(s + 1);
#pragma unroll
        for (int ks = 0; ks < BK / 32; ks++) {
            Frag f;
            read_frag(f, s, ks);
            mfma_frag(f);
        }
        __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0): slab s+1 has landed
        __syncthreads();
    }
    if constexpr (sizeof(TC) == 2 && TB == 128) {
        // the loop's last barrier has left the stages idle; each wave stages 32 rows of its block in them
        static_assert((size_t)WM * WN * 32 * (32 * TN) <= 2 * (size_t)(2 * TB * BK * 2), "staging exceeds the slab stages");
        store_tile_lds16<F16, TC, TM, TN>(g, cp, acc, lds_address(smem) + (unsigned)wave * (32 * 32 * TN),
                                          m0 + wm * (16 * TM), n0 + wn * (16 * TN), lane);
    } else {
        store_tile16<F16, TC, TM, TN>(g, cp, acc, m0 + wm * (16 * TM), n0 + wn * (16 * TN), lane);
    }
}

// ---------------------------------------------------------------------------
// Four-wave build: one wave per SIMD, each owning 128 x 128 of C as 8 x 8 tiles of
// v_mfma_f32_16x16x32 (256 accumulation registers; 16 fragment reads per 64 MFMAs, a third
// fewer LDS bytes per MFMA than the 8-wave builds). One wave per SIMD has no neighbour to hide
// its waits, so the schedule leaves none. A 64-wide slab is two 32-wide steps of 64 MFMAs; the
// 16 fragments of the next step are read one per two MFMAs under the first half of the current
// one. The slab's one barrier sits in its FIRST step, after the 40th MFMA, when the slab's last
// fragments are in registers: it both frees the slab's LDS stage for slab s + 2 and makes slab
// s + 1 visible, whose first fragments are read under the second step. The 16 loads of slab
// s + 2 follow the barrier one per four MFMAs (the CU's address unit takes 16 cycles per 1 KB
// load and the four waves issue in the same phase: 64 cycles per round of loads). The loop is
// unrolled over the two stages, so every LDS address is a pointer plus a constant. Same
// 128-byte swizzled rows and two 64 KB stages as the direct-to-LDS build above; behind them
// 8 KB per wave for the epilogue of a 16-bit C.
constexpr size_t kRingLdsBytes = 2 * (size_t)DMA_STAGE_BYTES + 4 * (size_t)kEpiWaveBytes; // 160 KB
template <bool F16, typename TC>
__global__ void __launch_bounds__(256, 1) gemm_ring_kernel(const GemmArgs g) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int c16 = lane & 15;
    const int q4 = lane >> 4;
    const int wm = wave >> 1, wn = wave & 1;
    // a tile of the split last round: workgroup = (tile, part), the part is a range of slabs
    int logical, part_id = 0, splits = 1;
    const int tiles_row = g.tiles_n * g.groups;
    const int tiles_m = (g.m + BM - 1) / BM;
    if ((int)blockIdx.x < g.part_wgs) {
        const int t = (int)blockIdx.x / g.splits;
        if (t >= tiles_m * tiles_row - g.tile_base) return; // padding up to a multiple of 8
        part_id = (int)blockIdx.x - t * g.splits;
        splits = g.splits;
        logical = g.tile_base + t;
    } else {
        // (part_wgs is a multiple of 8, so a workgroup's XCD is its id's low bits here too)
        logical = logical_tile((int)blockIdx.x - g.part_wgs, (int)gridDim.x - g.part_wgs);
    }
    int tm, tn;
    tile_coords(logical, tiles_m, tiles_row, tm, tn);
    const int grp = tn / g.tiles_n;
    tn -= grp * g.tiles_n;
    const void* const wp = grp == 0 ? g.w : g.w_more[grp - 1];
    void* const cp = grp == 0 ? g.c : g.c_more[grp - 1];
    const int m0 = tm * BM, n0 = tn * BN;

    const unsigned a_span = ((unsigned)(g.m - 1) * (unsigned)g.lda + (unsigned)g.k) * 2u;
    const unsigned w_span = ((unsigned)(g.n - 1) * (unsigned)g.ldw + (unsigned)g.k) * 2u;
    // The 16 loads of a slab go as four runs of four whose LDS targets lie 1 KB apart: M0 is set
    // once per run and the other three use the instruction's offset field, which also moves the
    // address in memory; that is taken off the lane's offset, and the descriptors start 3 KB
    // below the operands so that the offset stays positive.
    constexpr unsigned kBias = 3 * 1024;
    const u32x4 a_rsrc = make_rsrc_words(reinterpret_cast<const unsigned char*>(g.a) - kBias, a_span + kBias);
    const u32x4 w_rsrc = make_rsrc_words(reinterpret_cast<const unsigned char*>(wp) - kBias, w_span + kBias);
    const unsigned lds0 = lds_address(smem);
    // wave w fills rows 64 w + 8 j + lane / 8 (j < 8) of the A slab and of the W slab
    unsigned a_off[8], w_off[8];
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const int r = wave * 64 + j * 8 + (lane >> 3);
        const int c = (lane & 7) ^ ((r >> 1) & 7);
        const int ar = min(m0 + r, g.m - 1); // rows past the edge re-read the last row; never stored
        const int wr = min(n0 + r, g.n - 1);
        a_off[j] = ((unsigned)ar * (unsigned)g.lda + (unsigned)(c * 8)) * 2u + kBias - (unsigned)(j & 3) * 1024u;
        w_off[j] = ((unsigned)wr * (unsigned)g.ldw + (unsigned)(c * 8)) * 2u + kBias - (unsigned)(j & 3) * 1024u;
    }
    int nslab = g.k / BK, slab0 = 0;
    if (splits > 1) {
        const int per = (nslab + splits - 1) / splits;
        slab0 = part_id * per;
        nslab = max(min(nslab - slab0, per), 0);
    }
    const unsigned fetch_lds = __builtin_amdgcn_readfirstlane(lds0 + (unsigned)wave * (64 * BK * 2));
    // slabs past the end re-fetch the last slab into a stage nobody reads any more
    // the i-th (i < 16) of the loads that bring this wave's part of slab s in, in the order A rows
    // 0..31 of the wave's 64, W rows 0..31, A rows 32..63, W rows 32..63 (eight rows a load); the
    // loads of a run must be issued in order, the first sets M0 for the rest
    auto fetch_one = [&](int s, int i) __attribute__((always_inline)) {
        const unsigned uo = (unsigned)min(slab0 + max(s < nslab ? s : nslab - 1, 0), g.k / BK - 1) * (BK * 2u);
        const int run = i >> 2, jj = i & 3;
        const bool is_w = run & 1;
        const int j = (run >> 1) * 4 + jj;
        if (jj == 0) lds_dma_base(fetch_lds + (unsigned)(s & 1) * DMA_STAGE_BYTES + (is_w ? BM * BK * 2 : 0) + (unsigned)(run >> 1) * (32 * BK * 2));
        const u32x4& rsrc = is_w ? w_rsrc : a_rsrc;
        const unsigned off = is_w ? w_off[j] : a_off[j];
        if (jj == 0) load_to_lds_16_at<0>(rsrc, off, uo);
        if (jj == 1) load_to_lds_16_at<1024>(rsrc, off, uo);
        if (jj == 2) load_to_lds_16_at<2048>(rsrc, off, uo);
        if (jj == 3) load_to_lds_16_at<3072>(rsrc, off, uo);
    };
    auto fetch_slab = [&](int s) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 16; i++) fetch_one(s, i);
    };

    f32x4 acc[8][8];
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
        for (int j = 0; j < 8; j++) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    // fragment addresses: row (.. + c16), logical chunk 4 ks + q4 (ks < 2) at c ^ ((row >> 1) & 7);
    // a tile row adds 16 rows = 2 KB. (Pointers, so that the constant parts go into the
    // instruction's offset field; a stage is 64 KB, beyond that field: one pointer per stage.)
    typedef const __attribute__((address_space(3))) unsigned char* lds_byte_t;
    typedef const __attribute__((address_space(3))) u32x4* lds_u32x4_t;
    const lds_byte_t lds_base = (lds_byte_t)smem;
    const int sw = (c16 >> 1) & 7;
    lds_byte_t fa[2][2], fw[2][2]; // [stage][ks]
#pragma unroll
    for (int st = 0; st < 2; st++)
#pragma unroll
        for (int ks = 0; ks < 2; ks++) {
            const int pos = ((4 * ks + q4) ^ sw) * 16;
            fa[st][ks] = lds_base + (st * DMA_STAGE_BYTES + (wm * 128 + c16) * (BK * 2) + pos);
            fw[st][ks] = lds_base + (st * DMA_STAGE_BYTES + BM * BK * 2 + (wn * 128 + c16) * (BK * 2) + pos);
        }
    struct Frag { u32x4 a[8], w[8]; };
    // the r-th of the 16 reads of a fragment set
    auto read_one = [&](Frag& f, int st, int ks, int r) __attribute__((always_inline)) {
        if (r < 8) f.a[r] = *(lds_u32x4_t)(fa[st][ks] + r * 16 * (BK * 2));
        else f.w[r - 8] = *(lds_u32x4_t)(fw[st][ks] + (r - 8) * 16 * (BK * 2));
    };
    // One 32-wide step: 64 MFMAs on `cur`, the 16 reads of `nxt` under the first 32 of them.
    // FIRST (the slab's first step): the barrier after the 40th MFMA, then loads 0..5 of slab
    // s + 2, one per four MFMAs; the second step sends loads 6..15.
    auto mfma_step = [&](auto first_c, auto st_c, auto ks_c, const Frag& cur, Frag& nxt, int s) __attribute__((always_inline)) {
        constexpr bool FIRST = decltype(first_c)::value;
        constexpr int NST = decltype(st_c)::value, NKS = decltype(ks_c)::value; // where nxt is read from
#pragma unroll
        for (int t = 0; t < 64; t++) {
            if (FIRST && t >= 40 && (t & 3) == 0) fetch_one(s + 2, (t - 40) >> 2);
            if (!FIRST && (t & 3) == 1 && t < 40) fetch_one(s + 2, 6 + (t >> 2));
            if ((t & 1) == 0 && t < 32) read_one(nxt, NST, NKS, t >> 1);
            mfma16<F16>(cur.w[t & 7], cur.a[t >> 3], acc[t >> 3][t & 7]);
            __builtin_amdgcn_sched_barrier(0);
            if (FIRST && t == 39) {
                __builtin_amdgcn_s_waitcnt(0x0070); // vmcnt(0) lgkmcnt(0)
                asm volatile("" ::: "memory");
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };

    fetch_slab(0);
    fetch_slab(1);
    __builtin_amdgcn_s_waitcnt(0x4F70); // vmcnt(16): slab 0 has landed
    __syncthreads();
    Frag f0, f1;
#pragma unroll
    for (int r = 0; r < 16; r++) read_one(f0, 0, 0, r);
    typedef std::integral_constant<int, 0> I0;
    typedef std::integral_constant<int, 1> I1;
    int s = 0;
    for (; s + 1 < nslab; s += 2) {
        mfma_step(std::true_type{}, I0{}, I1{}, f0, f1, s);
        mfma_step(std::false_type{}, I1{}, I0{}, f1, f0, s);
        mfma_step(std::true_type{}, I1{}, I1{}, f0, f1, s + 1);
        mfma_step(std::false_type{}, I0{}, I0{}, f1, f0, s + 1);
        mfma16_drain(); // (24 cycles per two slabs: whatever follows the loop body may read the accumulators)
    }
    if (s < nslab) {
        mfma_step(std::true_type{}, I0{}, I1{}, f0, f1, s);
        mfma_step(std::false_type{}, I1{}, I0{}, f1, f0, s);
        mfma16_drain();
    }
    __builtin_amdgcn_s_waitcnt(0x0F70); // no direct load may outlive the workgroup's LDS
    if (splits > 1) {
        // partial tile in the accumulation layout: [tile][part][wave][i][j][lane] x 16 bytes,
        // every store instruction 1 KB in a row; the merge kernel reads it the same way
        f32x4* dst = reinterpret_cast<f32x4*>(g.part) +
                     ((((int64_t)(logical - g.tile_base) * g.splits + part_id) * 4 + wave) * 64) * 64 + lane;
#pragma unroll
        for (int i = 0; i < 8; i++)
#pragma unroll
            for (int j = 0; j < 8; j++) dst[(i * 8 + j) * 64] = acc[i][j];
        return;
    }
    if constexpr (sizeof(TC) == 2)
        store_tile_lds16<F16, TC, 8, 8>(g, cp, acc, lds0 + 2u * DMA_STAGE_BYTES + (unsigned)wave * kEpiWaveBytes, m0 + wm * 128, n0 + wn * 128, lane);
    else
        store_tile16<F16, TC, 8, 8>(g, cp, acc, m0 + wm * 128, n0 + wn * 128, lane);
}

// Adds the parts of the k-split tiles in part order and writes C. A workgroup takes the 32 x
// 128 block (tile, wave, i) of the four-wave build's accumulation layout: its wave j owns the
// 16 x 16 tiles (2 i + r / 2, 2 j + r % 2), r < 4; a lane holds row lane % 16 and columns
// 4 (lane / 16) .. + 4 of each. Every part's load (4 x splits of 16 bytes per lane) is sent
// before the first is used; the sums are turned through LDS so that C is stored as whole rows
// of the block.
constexpr int kMaxKSplits = 8;
template <bool F16, typename TC>
__global__ void __launch_bounds__(256) gemm_merge_kernel(const GemmArgs g) {
    constexpr int ES = (int)sizeof(TC);
    constexpr int PITCH = 128 * ES + 16; // bytes per staged row
    __shared__ __attribute__((aligned(16))) unsigned char stage[32 * PITCH];
    const int t = (int)blockIdx.x >> 4;
    const int wave = ((int)blockIdx.x >> 2) & 3, i = (int)blockIdx.x & 3;
    const int j = (int)threadIdx.x >> 6, lane = (int)threadIdx.x & 63;
    // quad (tile row 2 i + (r >> 1), tile column 2 j + (r & 1)) for r < 4
    const f32x4* src = reinterpret_cast<const f32x4*>(g.part) +
                       ((((int64_t)t * g.splits) * 4 + wave) * 64 + (16 * i + 2 * j)) * 64 + lane;
    f32x4 v[kMaxKSplits][4];
#pragma unroll
    for (int z = 0; z < kMaxKSplits; z++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
            v[z][r] = f32x4{0.f, 0.f, 0.f, 0.f};
            if (z < g.splits) v[z][r] = src[(int64_t)z * (4 * 64 * 64) + ((r >> 1) * 8 + (r & 1)) * 64];
        }
    const int c16 = lane & 15, q4 = lane >> 4;
#pragma unroll
    for (int r = 0; r < 4; r++) {
        f32x4 sum = v[0][r];
#pragma unroll
        for (int z = 1; z < kMaxKSplits; z++)
            if (z < g.splits) sum += v[z][r];
        unsigned char* dst = stage + (16 * (r >> 1) + c16) * PITCH + (32 * j + 16 * (r & 1) + 4 * q4) * ES;
        if constexpr (ES == 4) {
            *reinterpret_cast<f32x4*>(dst) = sum;
        } else {
            if constexpr (F16) *reinterpret_cast<u32x2*>(dst) = __builtin_bit_cast(u32x2, __builtin_convertvector(sum, f16x4));
            else *reinterpret_cast<u32x2*>(dst) = __builtin_bit_cast(u32x2, __builtin_convertvector(sum, bf16x4));
        }
    }
    __syncthreads();

    const int tiles_row = g.tiles_n * g.groups;
    int tm, tn;
    tile_coords(g.tile_base + t, (g.m + BM - 1) / BM, tiles_row, tm, tn);
    const int grp = tn / g.tiles_n;
    tn -= grp * g.tiles_n;
    void* const cp = grp == 0 ? g.c : g.c_more[grp - 1];
    const int row0 = tm * BM + (wave >> 1) * 128 + 32 * i;
    const int col0 = tn * BN + (wave & 1) * 128;
    constexpr int PER = 16 / ES;       // elements per 16-byte chunk
    constexpr int CH = 128 / PER;      // chunks per row of the block
    const bool vec = (g.ldc % PER == 0) && (reinterpret_cast<uintptr_t>(cp) % 16 == 0);
#pragma unroll
    for (int q = 0; q < 32 * CH / 256; q++) {
        const int c = (int)threadIdx.x + 256 * q;
        const int rr = c / CH, cc = c % CH;
        const int row = row0 + rr, col = col0 + PER * cc;
        if (row >= g.m || col >= g.n) continue;
        const u32x4 x = *reinterpret_cast<const u32x4*>(stage + rr * PITCH + cc * 16);
        TC* dst = reinterpret_cast<TC*>(cp) + (int64_t)row * g.ldc + col;
        if (vec && col + PER <= g.n) {
            *reinterpret_cast<u32x4*>(dst) = x;
        } else {
#pragma unroll
            for (int e = 0; e < PER; e++) {
                if (col + e >= g.n) break;
                if constexpr (ES == 4) reinterpret_cast<unsigned*>(dst)[e] = x[e];
                else reinterpret_cast<unsigned short*>(dst)[e] = (unsigned short)(x[e >> 1] >> (16 * (e & 1)));
            }
        }
    }
}

// f32 activations rounded to the weight's 16-bit type, once, into dense [m][k] rows: the
// products that follow then move their A slabs straight into LDS like 16-bit activations
// instead of rounding every slab of every tile (each row of A is read by every column tile).
template <bool F16>
__global__ void __launch_bounds__(256) gemm_round_kernel(const float* a, int64_t lda, unsigned short* out, int m, int k) {
    // grid x = row, grid y = 4096-element stretch of the row; a thread rounds two groups of 8
    const int row = (int)blockIdx.x;
    const int c0 = (int)blockIdx.y * 4096 + (int)threadIdx.x * 8;
    const float* src = a + (int64_t)row * lda;
    unsigned short* dst = out + (int64_t)row * k;
    f32x4 lo[2], hi[2];
#pragma unroll
    for (int u = 0; u < 2; u++) {
        const int c = min(c0 + u * 2048, k - 8); // past the end: re-read the last group, not stored
        lo[u] = *reinterpret_cast<const f32x4*>(src + c);
        hi[u] = *reinterpret_cast<const f32x4*>(src + c + 4);
    }
#pragma unroll
    for (int u = 0; u < 2; u++) {
        const int c = c0 + u * 2048;
        if (c >= k) continue;
        f32x8 v;
#pragma unroll
        for (int i = 0; i < 4; i++) { v[i] = lo[u][i]; v[4 + i] = hi[u][i]; }
        u32x4 r;
        if constexpr (F16) r = __builtin_bit_cast(u32x4, __builtin_convertvector(v, f16x8));
        else r = __builtin_bit_cast(u32x4, __builtin_convertvector(v, bf16x8));
        *reinterpret_cast<u32x4*>(dst + c) = r;
    }
}

// Measured on the Klein projections, same box, all with row-by-row stores and row-major tile
// order: eight waves (two per SIMD, 64 x 128 each) 1048-1217 TFLOP/s; four waves with the
// schedule above 1047-1248; four waves with the simple loop of the eight-wave build 960-1120.
constexpr int DMA_WM = 4, DMA_WN = 2;

static int g_gemm_build = 1; // 256-tiles of 16-bit activations: 1 = four-wave build (default), 0 = eight-wave build (measurement knob)

constexpr size_t kSmallLdsBytes = 2 * (size_t)(2 * 128 * BK * 2); // two stages of a 128-tile

template <typename TA, bool F16, typename TC>
static hipError_t launch_one(const GemmArgs& g0, hipStream_t stream) {
    GemmArgs g = g0;
    const int64_t tiles256 = (int64_t)((g.m + 255) / 256) * ((g.n + 255) / 256) * g.groups;
    if constexpr (!std::is_same<TA, float>::value) {
        // fewer 256-tiles than five eighths of the CUs: 128-tiles, two workgroups per CU
        if (g.k % BK == 0 && tiles256 < 160) {
            g.tiles_n = (g.n + 127) / 128;
            const int64_t nwg = (int64_t)((g.m + 127) / 128) * g.tiles_n * g.groups;
            if (nwg <= 0 || nwg > 0x7fffffff) return hipErrorInvalidValue;
            gemm_dma_kernel<F16, TC, 2, 2, 128><<<dim3((unsigned)nwg), dim3(256), kSmallLdsBytes, stream>>>(g);
            return hipGetLastError();
        }
    }
    g.tiles_n = (g.n + BN - 1) / BN;
    const int64_t nwg = tiles256;
    if (nwg <= 0 || nwg > 0x7fffffff) return hipErrorInvalidValue;
    if constexpr (!std::is_same<TA, float>::value) {
        if (g_gemm_build == 1 && g.k % BK == 0) {
            // one launch: (splits > 1) the tiles of the last round in parts, the whole tiles behind them; then the merge
            const int tail = g0.splits > 1 ? g0.tile_base : 0; // the planner leaves the tail size in tile_base
            if (tail < 0 || tail > nwg || g0.splits > kMaxKSplits || (tail > 0 && g0.part == nullptr)) return hipErrorInvalidValue;
            const int64_t whole = nwg - tail;
            g.tile_base = (int32_t)whole;
            g.splits = tail > 0 ? g0.splits : 1;
            g.part_wgs = tail > 0 ? (int32_t)(((int64_t)tail * g0.splits + 7) & ~(int64_t)7) : 0;
            if (whole + g.part_wgs > 0x7fffffff) return hipErrorInvalidValue;
            gemm_ring_kernel<F16, TC><<<dim3((unsigned)(whole + g.part_wgs)), dim3(256), kRingLdsBytes, stream>>>(g);
            if (tail > 0) {
                hipError_t e = hipGetLastError();
                if (e != hipSuccess) return e;
                gemm_merge_kernel<F16, TC><<<dim3((unsigned)tail * 16u), dim3(256), 0, stream>>>(g);
            }
            return hipGetLastError();
        }
        if (g.k % BK == 0) { // whole slabs of 16-bit activations: the direct-to-LDS build
            gemm_dma_kernel<F16, TC, DMA_WM, DMA_WN, 256><<<dim3((unsigned)nwg), dim3(DMA_WM * DMA_WN * 64), kDmaLdsBytes, stream>>>(g);
            return hipGetLastError();
        }
    }
    gemm_kernel<TA, F16, TC><<<dim3((unsigned)nwg), dim3(NT), kLdsBytes, stream>>>(g);
    return hipGetLastError();
}

template <typename TA, bool F16, typename TC>
static hipError_t raise_lds() {
    if constexpr (!std::is_same<TA, float>::value) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_dma_kernel<F16, TC, DMA_WM, DMA_WN, 256>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)kDmaLdsBytes);
        if (e != hipSuccess) return e;
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_dma_kernel<F16, TC, 2, 2, 128>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)kSmallLdsBytes);
        if (e != hipSuccess) return e;
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_ring_kernel<F16, TC>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)kRingLdsBytes);
        if (e != hipSuccess) return e;
    }
    return hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_kernel<TA, F16, TC>),
                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsBytes);
}

} // namespace gemm

int gemm_tile_rows() { return gemm::BM; }
int gemm_tile_cols() { return gemm::BN; }

// Only the four-wave build splits (16-bit activations, whole slabs, enough tiles for 256-tiles).
// A last round that fills at most half the CUs is cut along k so that it fills them: the round
// then costs 1 / splits of a tile's time plus the partial tiles' trip through memory (256 KB
// per part, which is why the number of parts is kept small and a fuller round is left whole).
void gemm_tail_plan(const GemmArgs& g, int a_dtype, int cus, int* tail_tiles, int* splits) {
    *tail_tiles = 0;
    *splits = 1;
    if (a_dtype == kF32 || gemm::g_gemm_build != 1 || g.k % gemm::BK != 0 || cus <= 0) return;
    const int64_t tiles = (int64_t)((g.m + 255) / 256) * ((g.n + 255) / 256) * g.groups;
    if (tiles < 160 || tiles > 0x7fffffff) return;
    const int tail = (int)(tiles % cus);
    if (tail == 0 || tail * 2 > cus) return;
    int s = cus / tail;
    if (s > gemm::kMaxKSplits) s = gemm::kMaxKSplits;
    const int nslab = g.k / gemm::BK;
    if (s > nslab / 4) s = nslab / 4; // at least four slabs per part
    if (s < 2) return;
    *tail_tiles = tail;
    *splits = s;
}
size_t gemm_part_bytes(int tail_tiles, int splits) {
    return (size_t)tail_tiles * splits * gemm::BM * gemm::BN * sizeof(float);
}

size_t gemm_round_bytes(const GemmArgs& g, int a_dtype) {
    // Whole slabs (the direct-to-LDS builds need them) and at least one full tile each way. The
    // pass moves 6 bytes per element of A through memory; measured at 4608 rows it pays at every
    // shape tried (n = 9216: 0.268 -> 0.263 ms with f32 C; k = 12288, n = 3072: 0.384 -> 0.372;
    // k = n = 3840: 0.225 -> 0.155, where it also opens the way to the k-split last round).
    if (a_dtype != kF32 || g.k % gemm::BK != 0 || g.m < 256 || g.n < 256) return 0;
    return (size_t)g.m * (size_t)g.k * 2;
}

hipError_t launch_gemm(const GemmArgs& g0, int a_dtype, int w_dtype, int c_dtype, hipStream_t stream) {
    using namespace gemm;
    typedef unsigned short h16; // a 16-bit operand in the compute type (bf16 or f16 per the weight)
    GemmArgs g = g0;
    if (a_dtype == kF32 && g.a16 != nullptr && gemm_round_bytes(g, a_dtype) != 0) {
        const dim3 grid((unsigned)g.m, (unsigned)((g.k + 4095) / 4096));
        if (w_dtype == kF16)
            gemm_round_kernel<true><<<grid, dim3(256), 0, stream>>>(static_cast<const float*>(g.a), g.lda, static_cast<h16*>(g.a16), g.m, g.k);
        else
            gemm_round_kernel<false><<<grid, dim3(256), 0, stream>>>(static_cast<const float*>(g.a), g.lda, static_cast<h16*>(g.a16), g.m, g.k);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
        g.a = g.a16;
        g.lda = g.k;
        a_dtype = w_dtype;
    }
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

void gemm_set_build(int build) { gemm::g_gemm_build = build == 1 ? 1 : 0; }

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
