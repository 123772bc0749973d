// gfx950 attention for one wide head (heads = 1, head_dim = 512): the VAE
// mid-block shape, 16384 tokens at 1024 px.
//
// What it replaces in the reference: attention_wide_mma
// (metal/mattn_shader.zig:225-390), reached through zdraw_metal_run_attention
// with kernel = wide (metal/mattn.zig:152-173, 261-275). The contract is the
// reference's: f32 token-major q, k, v, out [tokens][512], tokens % 64 == 0, no
// mask, not causal; anything else is refused on the host.
//
// Shape of the computation on this machine:
//   * a pre-pass rounds Q (times log2(e)/sqrt(512)), K and V to bf16 once, so the
//     main kernel moves half the bytes and fetches blocks straight into LDS;
//   * a workgroup is four waves, one per SIMD (512 registers each), and owns 128 query rows
//     and ALL 512 output dims over a range of the keys; a wave owns 32 of the rows: its O^T
//     accumulators (256 registers) fill the accumulation file and its Q fragments (128
//     registers) half the ordinary one. Nothing is exchanged between waves, the softmax runs
//     once per row, and no score is formed twice. The product's MFMAs are assembly statements
//     with the accumulator tied to the result, which is what keeps the 256 accumulation
//     registers where they are (given the builtin the compiler moves such tuples about and
//     spills); nothing else may touch those registers between such an MFMA and the wait that
//     ends the step (zdraw_amd.build.tied_mfma_hazards checks the compiled code);
//   * a query tile's keys are split over at least two workgroups (256 workgroups at 16384
//     tokens: one per CU), each leaving its unnormalised O and its (reference point, row sum)
//     in scratch; wide_merge_kernel combines the ranges in range order;
//   * per 32-key block a wave forms S^T = K Q^T (32 MFMAs; scores transposed, so a lane owns
//     one query and P^T is the next MFMA's B operand without an LDS round trip) with the online
//     softmax of the previous block in their shadow, then adds V^T P^T to O^T (32 MFMAs);
//   * K blocks (32 KB) cycle through three LDS slots, V blocks (32 KB) through two: all 160 KB,
//     filled by buffer_load ... lds in the swizzled 256-byte-row layout of the head_dim-128
//     kernel. K is requested three steps before it is used, V one; a wave's 16 loads per block
//     are issued a few MFMAs apart: the CU's address unit takes 16 cycles per load, and a burst
//     from four waves at once holds them at the memory queue;
//   * one barrier per block, placed after the 28th of the 32 S MFMAs, when the last K
//     fragments are in registers: the V fragments of the product are read under the rest;
//   * fixed block order and fixed summation order: bit-identical from run to run.
#include "attn_device.hpp"

namespace zdraw {

namespace wide {

constexpr int WD = 512;           // head_dim
constexpr int SL = 128;           // dims per LDS tile ("slice")
constexpr int NSL = WD / SL;
constexpr int KB = 32;            // keys per block
constexpr int NW = 4;
constexpr int NT = NW * 64;
constexpr int BQ = 128;           // query rows per workgroup
constexpr int TILE_BYTES = KB * SL * 2;        // 8 KB
constexpr int K_SLOT = NSL * TILE_BYTES;       // a K block: 32 KB
constexpr int V_SLOT = NSL * TILE_BYTES;       // a V block: 32 KB
constexpr int NSK = 3;                         // slots of the K ring
constexpr int NSV = 2;                         // slots of the V ring
constexpr int V_RING = NSK * K_SLOT;
constexpr size_t kLdsBytes = (size_t)NSK * K_SLOT + (size_t)NSV * V_SLOT; // 160 KB
constexpr float kTau = 8.0f;      // log2 headroom of the lazy softmax maximum (attn_wide_safe_kernel)
constexpr float kRowSumLimit = 0x1p90f; // a row sum past this flags its tile: a P beyond 2^90 may be on its way to overflow
constexpr int RA = 6;             // K fragments read ahead of their MFMA
constexpr int VA = 3;             // V fragment pairs read ahead
constexpr int kMaxSplits = 8;     // key ranges per query tile

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

// f32 -> bf16 with a scale, 8 elements per thread; blockIdx.y selects the operand.
__global__ void __launch_bounds__(256) wide_round_kernel(const WidePrepArgs p) {
    const int op = (int)blockIdx.y;
    // the launch that precedes every attention launch also clears its redo flags
    if (op == 0 && blockIdx.x == 0)
        for (int i = threadIdx.x; i < p.redo_tiles; i += blockDim.x) p.redo[i] = 0;
    const float* src = op == 0 ? p.q : op == 1 ? p.k : p.v;
    bf16_t* dst = reinterpret_cast<bf16_t*>(op == 0 ? p.qo : op == 1 ? p.ko : p.vo);
    const float scale = op == 0 ? p.q_scale : 1.0f;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < p.chunks; i += stride) {
        const f32x4 a = *reinterpret_cast<const f32x4*>(src + 8 * i);
        const f32x4 b = *reinterpret_cast<const f32x4*>(src + 8 * i + 4);
        const float x[8] = {a[0] * scale, a[1] * scale, a[2] * scale, a[3] * scale,
                            b[0] * scale, b[1] * scale, b[2] * scale, b[3] * scale};
        *reinterpret_cast<u32x4*>(dst + 8 * i) = pack_bf16x8(x);
    }
}

template <int N> using IC = std::integral_constant<int, N>;

__device__ __forceinline__ f32x16 zero16() {
    f32x16 z;
#pragma unroll
    for (int j = 0; j < 16; j++) z[j] = 0.f;
    return z;
}

// O^T += A B on the accumulation file, the accumulator tied to the result. The compiler adds no
// hazard waits around assembly: consecutive MFMAs on one accumulator are four MFMAs apart in the
// product's order, and acc_drain() ends every step in the basic block of its last MFMA, before
// anything else (the rescale, the epilogue, a copy the compiler placed at a join) can read the
// accumulation registers.
__device__ __forceinline__ void mfma_acc(f32x16& c, const bf16x8& x, const bf16x8& y) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(x), "v"(y));
}
// The same for the scores, in ordinary registers (the accumulation file is full): `first` starts
// the chain from zero. Dependent MFMAs of one shape issue back to back; the scores are first read
// by other instructions four product MFMAs after the chain's last.
template <bool FIRST>
__device__ __forceinline__ void mfma_score(f32x16& c, const bf16x8& x, const bf16x8& y) {
    if constexpr (FIRST) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(c) : "v"(x), "v"(y));
    else asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(x), "v"(y));
}
// c = 0 as an MFMA of zeros: the tuple is defined whole, never element by element. (An MFMA may
// not read a register in the two issue slots after an ordinary vector instruction wrote it; the
// compiler keeps that distance for its own MFMAs, not around assembly: z may just have been set.)
__device__ __forceinline__ void mfma_zero(f32x16& c, const bf16x8& z) {
    asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %1, 0" : "=&a"(c) : "v"(z));
}
__device__ __forceinline__ void acc_drain() {
    asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");
}

__global__ void __launch_bounds__(NT, 1) attn_wide_kernel(const WideArgs a) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int l32 = lane & 31;
    const int h = lane >> 5;
    // workgroup = (query tile, key range); a.splits is a power of two
    const int nsp = a.splits > 1 ? a.splits : 1;
    const int lg = __builtin_ctz((unsigned)nsp); // (shifts: an integer division would run on the vector unit)
    const int part = (int)blockIdx.x & (nsp - 1);
    const int q0 = ((int)blockIdx.x >> lg) * BQ + 32 * wave;        // this wave's query rows
    const int per = (a.tokens / KB + nsp - 1) >> lg;
    const int blk0 = part * per;                                    // this range's first key block
    const int nblk = max(min(a.tokens / KB - blk0, per), 1);        // and how many it has (the host gives every range some)

    const unsigned lds0 = lds_address(smem);

    // ---- Q fragments (B operand of S^T = K Q^T): query q0 + l32, dims 16 kk + 8 h .. +7
    bf16x8 qf[32];
    {
        // rows past the end read the last row and are never stored
        const bf16_t* qp = reinterpret_cast<const bf16_t*>(a.q) + (int64_t)min(q0 + l32, a.tokens - 1) * WD + 8 * h;
#pragma unroll
        for (int kk = 0; kk < 32; kk++) qf[kk] = *reinterpret_cast<const bf16x8*>(qp + 16 * kk);
    }

    // ---- block fetch. Wave w fills tile w (dims 128 w .. +127) of a K block and of a V block,
    // four rows per instruction. The lane that fills chunk position p of row r fetches the chunk
    // the swizzle places there: K chunk c of row r sits at c ^ (r & 15), V chunk c at
    // c ^ ((r & 3) << 2) (the same for every row a lane fills: one offset serves all eight loads).
    const unsigned span = (unsigned)a.tokens * (unsigned)(WD * 2);
    const u32x4 k_rsrc = make_rsrc_words(a.k, span);
    const u32x4 v_rsrc = make_rsrc_words(a.v, span);
    unsigned fk_off[4]; // K rows 4 j + 16 take the same chunks 16 rows further on
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int row = 4 * j + (lane >> 4);
        const unsigned kc = (unsigned)((lane & 15) ^ (row & 15));
        fk_off[j] = (unsigned)row * (WD * 2) + (unsigned)wave * (SL * 2) + kc * 16u;
    }
    const unsigned fv_off = (unsigned)(lane >> 4) * (WD * 2) + (unsigned)wave * (SL * 2) +
                            (unsigned)((lane & 15) ^ ((lane >> 4) << 2)) * 16u;
    const unsigned fetch_k_lds = __builtin_amdgcn_readfirstlane(lds0 + (unsigned)wave * TILE_BYTES);
    const unsigned fetch_v_lds = __builtin_amdgcn_readfirstlane(lds0 + V_RING + (unsigned)wave * TILE_BYTES);
    // the i-th (i < 8) load of K block kb into K slot ks / of V block vb into V slot vs; positions
    // past the range re-fetch its last block into a slot nobody reads any more
    auto fetch_k = [&](int kb, int ks, int i) __attribute__((always_inline)) {
        // (uniform, but the compiler may have formed it in a vector register)
        const unsigned uo = __builtin_amdgcn_readfirstlane((unsigned)(blk0 + (kb < nblk ? kb : nblk - 1)) * (unsigned)(KB * WD * 2) + (unsigned)(i >> 2) * (16 * WD * 2));
        load_to_lds_16(k_rsrc, fetch_k_lds + (unsigned)ks * K_SLOT + (unsigned)(4 * i) * (SL * 2), fk_off[i & 3], uo);
    };
    auto fetch_v = [&](int vb, int vs, int i) __attribute__((always_inline)) {
        const unsigned uo = __builtin_amdgcn_readfirstlane((unsigned)(blk0 + (vb < nblk ? vb : nblk - 1)) * (unsigned)(KB * WD * 2) + (unsigned)(4 * i) * (WD * 2));
        load_to_lds_16(v_rsrc, fetch_v_lds + (unsigned)vs * V_SLOT + (unsigned)(4 * i) * (SL * 2), fv_off, uo);
    };

    // ---- fragment addresses in slot 0 (a tile and a slot add constants)
    const int tr_row = (lane & 15) >> 2;
    const int tr_col = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
    // (pointers, so that the constant parts of an address go into the instruction's offset field)
    typedef __attribute__((address_space(3))) unsigned char* lds_byte_t;
    typedef const __attribute__((address_space(3))) bf16x8* lds_bf16x8_t;
    typedef __attribute__((address_space(3))) s16x4* lds_s16x4_t;
    const lds_byte_t lds_base = (lds_byte_t)smem;
    lds_byte_t kfo[8], vfo[4];
#pragma unroll
    for (int kk = 0; kk < 8; kk++) kfo[kk] = lds_base + ((l32 * SL + (((2 * kk + h) ^ (l32 & 15)) * 8)) * 2);
#pragma unroll
    for (int blk = 0; blk < 4; blk++)
        vfo[blk] = lds_base + V_RING + (((4 * h + tr_row) * SL + ((blk ^ tr_row) * 32) + tr_col) * 2);
    auto k_read = [&](int slot, int kk) __attribute__((always_inline)) {
        return *(lds_bf16x8_t)(kfo[kk & 7] + (slot * K_SLOT + (kk >> 3) * TILE_BYTES));
    };

    // O^T: lane = query l32, dims 32 blk + 8 i + 4 h + j. The tuples are only ever written whole
    // (by an MFMA), which is what lets them stay put in the accumulation file.
    f32x16 oacc[16];
    const bf16x8 zero_frag = __builtin_bit_cast(bf16x8, u32x4{0u, 0u, 0u, 0u});
    float l_run = 0.f;

    // ---- prologue: K(0..2), V(0) in; S(0)
#pragma unroll
    for (int i = 0; i < 8; i++) fetch_k(0, 0, i);
#pragma unroll
    for (int i = 0; i < 8; i++) fetch_v(0, 0, i);
#pragma unroll
    for (int i = 0; i < 8; i++) fetch_k(1, 1, i);
#pragma unroll
    for (int i = 0; i < 8; i++) fetch_k(2, 2, i);
    __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0)
    __syncthreads();
    f32x16 sv; // scores of the block the next step exponentiates: lane = query l32, element 4 i + j = key 8 i + 4 h + j
    {
        f32x16 s;
#pragma unroll
        for (int kk = 0; kk < 32; kk++) {
            if (kk == 0) mfma_score<true>(s, k_read(0, kk), qf[kk]);
            else mfma_score<false>(s, k_read(0, kk), qf[kk]);
        }
        acc_drain(); // the scores are read next
        sv = s;
    }
    // Softmax in the exp2 domain (the scale rides on Q) against ONE reference point per row: the
    // largest score of the range's first block. It never moves, so nothing is ever rescaled
    // (scaling 256 accumulation registers in place would have to change the tuples element by
    // element, and then the compiler no longer keeps them where they are; any branch that
    // touches them inside the loop costs hundreds of spills). fp32 and bf16 share one exponent
    // range, so a later score may lie far above the reference (P up to 2^kHeadroom and beyond)
    // or far below it without any loss; only a row whose scores climb more than kHeadroom above
    // its first block's is out of reach. Such a row shows in its row sum: the wave then flags the
    // query tile, and attn_wide_safe_kernel, which follows every launch, forms flagged tiles
    // again with a running maximum.
    float mc;
    {
        const float m0 = fmaxf(fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3])), fmaxf(fmaxf(sv[4], sv[5]), fmaxf(sv[6], sv[7])));
        const float m1 = fmaxf(fmaxf(fmaxf(sv[8], sv[9]), fmaxf(sv[10], sv[11])), fmaxf(fmaxf(sv[12], sv[13]), fmaxf(sv[14], sv[15])));
        mc = pair_max(fmaxf(m0, m1));
    }
    __syncthreads(); // K(0) has no reader left: the first step sends K(3) there
    bf16x8 kf[RA + 1]; // ring of fragments in flight
#pragma unroll
    for (int kk = 0; kk < RA; kk++) kf[kk] = k_read(1, kk);

    // One step b with K(b+1) in K slot KS = (b + 1) % 3 and V(b) in V slot VS = b % 2:
    //   S phase: the 32 MFMAs of S(b+1) = K(b+1) Q^T with the softmax of block b in their shadow,
    //            and the 8 loads of K(b+3) into the slot K(b) left (free since the last barrier);
    //   barrier: V(b) has landed (requested in the previous step's PV phase) and so has everything
    //            older (K(b+2)); K(b+1) and V(b-1) have no reader left;
    //   PV phase: O += V(b)^T P(b)^T (32 MFMAs), the 8 loads of V(b+1) into the slot V(b-1) left,
    //            the first fragments of K(b+2) read under the last MFMAs.
    auto step = [&](auto ks_c, auto vs_c, int b) __attribute__((always_inline)) {
        constexpr int KS = decltype(ks_c)::value;       // slot of K(b+1); K(b+2) is in (KS + 1) % 3, K(b+3) goes to (KS + 2) % 3
        constexpr int VS = decltype(vs_c)::value;       // slot of V(b); V(b+1) goes to the other
        constexpr int KN = (KS + 1) % 3;
        f32x16 s;
        float psum = 0.f, e_even = 0.f;
        unsigned pc[8];
        s16x4 vlo[VA + 1], vhi[VA + 1];
        // idx < 32: tile idx >> 3, key half (idx >> 2) & 1, 32-dim block idx & 3 of the tile
        auto v_read = [&](int idx) __attribute__((always_inline)) {
            const lds_byte_t va = vfo[idx & 3] + (VS * V_SLOT + (idx >> 3) * TILE_BYTES + (16 * ((idx >> 2) & 1)) * (SL * 2));
            vlo[idx % (VA + 1)] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_t)va);
            vhi[idx % (VA + 1)] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_t)(va + 8 * (SL * 2)));
        };
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < 32; t++) {
            if (t % 3 == 0 && t < 24) fetch_k(b + 3, (KS + 2) % 3, t / 3);
            if (t + RA < 32) kf[(t + RA) % (RA + 1)] = k_read(KS, t + RA);
            if (t >= 28 && t - 28 < VA) v_read(t - 28);
            if (t == 0) mfma_score<true>(s, kf[t % (RA + 1)], qf[t]);
            else mfma_score<false>(s, kf[t % (RA + 1)], qf[t]);
            // exponentials of block b against its reference, one per MFMA
            if (t >= 3 && t < 19) {
                const int e = t - 3;
                const float x = __builtin_amdgcn_exp2f(sv[e] - mc);
                psum += x;
                if (e & 1) {
                    f32x2 pp = {e_even, x};
                    pc[e >> 1] = __builtin_bit_cast(unsigned, __builtin_convertvector(pp, bf16x2));
                } else {
                    e_even = x;
                }
            } else if (t == 19) {
                l_run += psum;
            }
            __builtin_amdgcn_sched_barrier(0);
            if (t == 27) {
                // every fragment of K(b+1) is in registers; V(b) and all before it have landed:
                // everything but the 8 loads of K(b+3) sent in this phase
                __builtin_amdgcn_s_waitcnt(0x0078); // vmcnt(8) lgkmcnt(0)
                asm volatile("" ::: "memory");
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        const bf16x8 p0 = __builtin_bit_cast(bf16x8, u32x4{pc[0], pc[1], pc[2], pc[3]});
        const bf16x8 p1 = __builtin_bit_cast(bf16x8, u32x4{pc[4], pc[5], pc[6], pc[7]});
#pragma unroll
        for (int idx = 0; idx < 32; idx++) {
            if ((idx & 3) == 1) fetch_v(b + 1, VS ^ 1, idx >> 2);
            if (idx + VA < 32) v_read(idx + VA);
            if (idx >= 32 - RA) kf[(idx - (32 - RA)) % (RA + 1)] = k_read(KN, idx - (32 - RA));
            const bf16x8 vf = __builtin_bit_cast(bf16x8, (s16x8)__builtin_shufflevector(vlo[idx % (VA + 1)], vhi[idx % (VA + 1)], 0, 1, 2, 3, 4, 5, 6, 7));
            mfma_acc(oacc[(idx >> 3) * 4 + (idx & 3)], vf, ((idx >> 2) & 1) ? p1 : p0);
            if (idx == 4) sv = s; // the S MFMAs have drained by now
            __builtin_amdgcn_sched_barrier(0);
        }
        acc_drain();
    };
    // the K ring turns every three steps, the V ring every two: six steps per trip
#pragma unroll
    for (int blk = 0; blk < 16; blk++) mfma_zero(oacc[blk], zero_frag);
    acc_drain();
    int b = 0;
    for (; b + 5 < nblk; b += 6) {
        step(IC<1>{}, IC<0>{}, b);
        step(IC<2>{}, IC<1>{}, b + 1);
        step(IC<0>{}, IC<0>{}, b + 2);
        step(IC<1>{}, IC<1>{}, b + 3);
        step(IC<2>{}, IC<0>{}, b + 4);
        step(IC<0>{}, IC<1>{}, b + 5);
    }
    if (b < nblk) step(IC<1>{}, IC<0>{}, b);
    if (b + 1 < nblk) step(IC<2>{}, IC<1>{}, b + 1);
    if (b + 2 < nblk) step(IC<0>{}, IC<0>{}, b + 2);
    if (b + 3 < nblk) step(IC<1>{}, IC<1>{}, b + 3);
    if (b + 4 < nblk) step(IC<2>{}, IC<0>{}, b + 4);
    __builtin_amdgcn_s_waitcnt(0x0F70); // no direct load may outlive the workgroup's LDS

    // ---- epilogue: O = O^T / l, or the range's share as it stands
    const float l_tot = pair_sum(l_run);
    // a row sum past 2^kHeadroom (or not a number): some score left the reach of the fixed reference
    if (__any(!(l_tot <= kRowSumLimit)) && lane == 0) a.redo[(int)blockIdx.x >> lg] = 1;
    if (q0 + l32 >= a.tokens) return;
    if (nsp > 1) {
        float* op = a.part_o + ((int64_t)part * a.tokens + (q0 + l32)) * WD + 4 * h;
#pragma unroll
        for (int blk = 0; blk < 16; blk++)
#pragma unroll
            for (int i = 0; i < 4; i++)
                *reinterpret_cast<f32x4*>(op + 32 * blk + 8 * i) =
                    f32x4{oacc[blk][4 * i], oacc[blk][4 * i + 1], oacc[blk][4 * i + 2], oacc[blk][4 * i + 3]};
        if (h == 0) *reinterpret_cast<f32x2*>(a.part_ml + ((int64_t)part * a.tokens + (q0 + l32)) * 2) = f32x2{mc, l_tot};
        return;
    }
    const float inv_l = l_tot > 0.f ? 1.0f / l_tot : 0.f;
    float* op = a.o + (int64_t)(q0 + l32) * WD + 4 * h;
#pragma unroll
    for (int blk = 0; blk < 16; blk++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
            f32x4 v;
#pragma unroll
            for (int j = 0; j < 4; j++) v[j] = oacc[blk][4 * i + j] * inv_l;
            *reinterpret_cast<f32x4*>(op + 32 * blk + 8 * i) = v;
        }
}

// ---------------------------------------------------------------------------------------------
// The tiles that attn_wide_kernel flagged (a score more than 2^kHeadroom above its row's first
// block), formed again with a lazy running maximum. A workgroup is four waves and owns 128 query
// rows and HALF of the 512 output dims over all keys (both workgroups of a tile form the full
// scores: 48 MFMAs per wave and block where 32 would do); with 128 accumulation registers per
// wave the compiler has room to rescale O^T in place when a reference point moves. K blocks
// (32 KB) and V half-blocks (16 KB) cycle through three LDS slots each. Launched after every
// attn_wide_kernel launch; a workgroup whose tile is not flagged returns at once.
namespace safe {
constexpr int HALF = WD / 2;      // output dims per workgroup
constexpr int V_SLOT = (NSL / 2) * TILE_BYTES; // half the dims of a V block: 16 KB
constexpr int NS = 3;                          // slots per ring
constexpr int V_RING = NS * K_SLOT;
constexpr size_t kLdsBytes = (size_t)NS * (K_SLOT + V_SLOT); // 144 KB

__global__ void __launch_bounds__(NT, 1) attn_wide_safe_kernel(const WideArgs a) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int l32 = lane & 31;
    const int h = lane >> 5;
    // workgroup = (query tile, half of the output dims), over all keys; only flagged tiles run
    if (a.redo[(int)blockIdx.x >> 1] == 0) return; // uniform over the workgroup
    const int dh = (int)blockIdx.x & 1;
    constexpr int nsp = 1;
    const int q0 = ((int)blockIdx.x >> 1) * BQ + 32 * wave; // this wave's query rows
    const int blk0 = 0;
    const int nblk = a.tokens / KB;

    const unsigned lds0 = lds_address(smem);

    // ---- Q fragments (B operand of S^T = K Q^T): query q0 + l32, dims 16 kk + 8 h .. +7
    bf16x8 qf[32];
    {
        // rows past the end read the last row and are never stored
        const bf16_t* qp = reinterpret_cast<const bf16_t*>(a.q) + (int64_t)min(q0 + l32, a.tokens - 1) * WD + 8 * h;
#pragma unroll
        for (int kk = 0; kk < 32; kk++) qf[kk] = *reinterpret_cast<const bf16x8*>(qp + 16 * kk);
    }

    // ---- block fetch. K: wave w fills tile w (dims 128 w .. +127) of the block, four rows per
    // instruction. V: wave w fills rows 16 (w >> 1) .. +15 of tile (w & 1) of this workgroup's
    // half. The lane that fills chunk position p of row r fetches the chunk the swizzle places
    // there: K chunk c of row r sits at c ^ (r & 15), V chunk c at c ^ ((r & 3) << 2).
    const unsigned span = (unsigned)a.tokens * (unsigned)(WD * 2);
    const u32x4 k_rsrc = make_rsrc_words(a.k, span);
    const u32x4 v_rsrc = make_rsrc_words(a.v, span);
    unsigned fk_off[4], fv_off[4]; // K rows 4 j + 16 take the same chunks 16 rows further on
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int row = 4 * j + (lane >> 4);
        const unsigned kc = (unsigned)((lane & 15) ^ (row & 15));
        fk_off[j] = (unsigned)row * (WD * 2) + (unsigned)wave * (SL * 2) + kc * 16u;
    }
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int row = 16 * (wave >> 1) + 4 * j + (lane >> 4);
        const unsigned vc = (unsigned)((lane & 15) ^ ((row & 3) << 2));
        fv_off[j] = (unsigned)row * (WD * 2) + (unsigned)(2 * dh + (wave & 1)) * (SL * 2) + vc * 16u;
    }
    const unsigned fetch_k_lds = __builtin_amdgcn_readfirstlane(lds0 + (unsigned)wave * TILE_BYTES);
    const unsigned fetch_v_lds = __builtin_amdgcn_readfirstlane(lds0 + V_RING + (unsigned)(wave & 1) * TILE_BYTES + (unsigned)(16 * (wave >> 1)) * (SL * 2));
    // the i-th (i < 12) load of the group that brings K block kb into K slot ks and V block vb into V slot vs
    auto fetch_one = [&](int kb, int ks, int vb, int vs, int i) __attribute__((always_inline)) {
        if (i < 8) {
            // (uniform, but the compiler may have formed it in a vector register)
            const unsigned uo = __builtin_amdgcn_readfirstlane((unsigned)(blk0 + (kb < nblk ? kb : nblk - 1)) * (unsigned)(KB * WD * 2) + (unsigned)(i >> 2) * (16 * WD * 2));
            load_to_lds_16(k_rsrc, fetch_k_lds + (unsigned)ks * K_SLOT + (unsigned)(4 * i) * (SL * 2), fk_off[i & 3], uo);
        } else {
            const unsigned uo = __builtin_amdgcn_readfirstlane((unsigned)(blk0 + (vb < nblk ? vb : nblk - 1)) * (unsigned)(KB * WD * 2));
            load_to_lds_16(v_rsrc, fetch_v_lds + (unsigned)vs * V_SLOT + (unsigned)(4 * (i - 8)) * (SL * 2), fv_off[i - 8], uo);
        }
    };

    // ---- fragment addresses in slot 0 (a tile and a slot add constants)
    const int tr_row = (lane & 15) >> 2;
    const int tr_col = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
    // (pointers, so that the constant parts of an address go into the instruction's offset field)
    typedef __attribute__((address_space(3))) unsigned char* lds_byte_t;
    typedef const __attribute__((address_space(3))) bf16x8* lds_bf16x8_t;
    typedef __attribute__((address_space(3))) s16x4* lds_s16x4_t;
    const lds_byte_t lds_base = (lds_byte_t)smem;
    lds_byte_t kfo[8], vfo[4];
#pragma unroll
    for (int kk = 0; kk < 8; kk++) kfo[kk] = lds_base + ((l32 * SL + (((2 * kk + h) ^ (l32 & 15)) * 8)) * 2);
#pragma unroll
    for (int blk = 0; blk < 4; blk++)
        vfo[blk] = lds_base + V_RING + (((4 * h + tr_row) * SL + ((blk ^ tr_row) * 32) + tr_col) * 2);
    auto k_read = [&](int slot, int kk) __attribute__((always_inline)) {
        return *(lds_bf16x8_t)(kfo[kk & 7] + (slot * K_SLOT + (kk >> 3) * TILE_BYTES));
    };

    f32x16 oacc[8]; // O^T: lane = query l32, dims 256 dh + 32 blk + 8 i + 4 h + j
#pragma unroll
    for (int blk = 0; blk < 8; blk++)
#pragma unroll
        for (int j = 0; j < 16; j++) oacc[blk][j] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;

    // ---- prologue: K(0..2), V(0..1) in; S(0); then K(3) requested
#pragma unroll
    for (int i = 0; i < 12; i++) fetch_one(0, 0, 0, 0, i);
#pragma unroll
    for (int i = 0; i < 12; i++) fetch_one(1, 1, 1, 1, i);
#pragma unroll
    for (int i = 0; i < 8; i++) fetch_one(2, 2, 0, 0, i);
    __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0)
    __syncthreads();
    f32x16 sv; // scores of the block the next step exponentiates: lane = query l32, element 4 i + j = key 8 i + 4 h + j
    {
        f32x16 s = zero16();
#pragma unroll
        for (int kk = 0; kk < 32; kk++) s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(k_read(0, kk), qf[kk], s, 0, 0, 0);
        sv = s;
    }
    __syncthreads(); // K(0) has no reader left
#pragma unroll
    for (int i = 0; i < 4; i++) fetch_one(3, 0, 0, 0, i); // the first step sends the other eight of this group
    bf16x8 kf[RA + 1]; // ring of fragments in flight
#pragma unroll
    for (int kk = 0; kk < RA; kk++) kf[kk] = k_read(1, kk);

    // The running maximum moved (rare after the first blocks): O^T *= alpha, in place in the
    // accumulation file. Written out by hand: left to the compiler, the two versions of O that
    // meet after the branch cost more registers than there are.
    auto rescale = [&](float alpha) __attribute__((always_inline)) {
        asm volatile("s_nop 15\n\ts_nop 15" ::: "memory"); // MFMA results are read next
#pragma unroll
        for (int blk = 0; blk < 8; blk++)
#pragma unroll
            for (int j = 0; j < 16; j++) {
                float x = oacc[blk][j], t;
                asm volatile("v_accvgpr_read_b32 %1, %0\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 %0, %1" : "+a"(x), "=&v"(t) : "v"(alpha));
                oacc[blk][j] = x;
            }
        asm volatile("s_nop 7" ::: "memory"); // and feed the next MFMAs
    };

    // One step b with K(b+1) in K slot KS = (b + 1) % 3 and V(b) in V slot VS = b % 3:
    //   S phase: the 32 MFMAs of S(b+1) = K(b+1) Q^T with the softmax of block b in their shadow;
    //   barrier: K(b+2) and V(b) have landed (requested two steps ago), K(b+1) and V(b-1) have no
    //            reader left;
    //   PV phase: O += V(b)^T P(b)^T (16 MFMAs), the first fragments of K(b+2) read under them.
    // The 12 loads that bring K(b+4) and V(b+2) into the two freed slots follow the barrier, 4
    // under the PV phase and 8 under the next S phase.
    auto step = [&](auto ks_c, auto vs_c, int b) __attribute__((always_inline)) {
        constexpr int KS = decltype(ks_c)::value;       // slot of K(b+1); K(b+2) is in (KS + 1) % 3
        constexpr int VS = decltype(vs_c)::value;       // slot of V(b); V(b-1) was in (VS + 2) % 3
        constexpr int KN = (KS + 1) % 3;
        f32x16 s;
        float mloc = 0.f, mc = 0.f, alpha = 1.f, psum = 0.f, e_even = 0.f;
        bool up = false;
        unsigned pc[8];
        s16x4 vlo[VA + 1], vhi[VA + 1];
        // idx < 16: tile idx >> 3 of the half, key half (idx >> 2) & 1, 32-dim block idx & 3
        auto v_read = [&](int idx) __attribute__((always_inline)) {
            const lds_byte_t va = vfo[idx & 3] + (VS * V_SLOT + (idx >> 3) * TILE_BYTES + (16 * ((idx >> 2) & 1)) * (SL * 2));
            vlo[idx % (VA + 1)] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_t)va);
            vhi[idx % (VA + 1)] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_t)(va + 8 * (SL * 2)));
        };
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < 32; t++) {
            // the previous barrier's group: K(b+3) into the slot K(b) left, V(b+1) into V(b-2)'s
            if ((t & 3) == 0) fetch_one(b + 3, (KS + 2) % 3, b + 1, (VS + 1) % 3, 4 + (t >> 2));
            if (t + RA < 32) kf[(t + RA) % (RA + 1)] = k_read(KS, t + RA);
            if (t >= 28 && t - 28 < VA) v_read(t - 28);
            s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[t % (RA + 1)], qf[t], t == 0 ? zero16() : s, 0, 0, 0);
            // softmax of block b in the exp2 domain (the scale rides on Q) with a lazy maximum: the
            // reference point moves only when this block's maximum exceeds it by more than kTau
            if (t == 0) {
                mloc = fmaxf(fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3])), fmaxf(fmaxf(sv[4], sv[5]), fmaxf(sv[6], sv[7])));
            } else if (t == 1) {
                mloc = fmaxf(mloc, fmaxf(fmaxf(fmaxf(sv[8], sv[9]), fmaxf(sv[10], sv[11])), fmaxf(fmaxf(sv[12], sv[13]), fmaxf(sv[14], sv[15]))));
                const float mlc = pair_max(mloc);
                up = mlc > m_run + kTau;
                const float m_new = up ? mlc : m_run;
                mc = (m_new == -INFINITY) ? 0.f : m_new;
                alpha = __builtin_amdgcn_exp2f(m_run - mc);
                m_run = m_new;
            } else if (t >= 3 && t < 19) {
                const int e = t - 3; // one exponential per MFMA
                const float x = __builtin_amdgcn_exp2f(sv[e] - mc);
                psum += x;
                if (e & 1) {
                    f32x2 pp = {e_even, x};
                    pc[e >> 1] = __builtin_bit_cast(unsigned, __builtin_convertvector(pp, bf16x2));
                } else {
                    e_even = x;
                }
            } else if (t == 19) {
                l_run = l_run * alpha + psum;
                if (__any(up)) rescale(alpha);
            }
            __builtin_amdgcn_sched_barrier(0);
            if (t == 27) {
                // every fragment of K(b+1) is in registers; K(b+2), V(b) have landed: everything but
                // the 12 loads sent since the last barrier
                __builtin_amdgcn_s_waitcnt(0x007C); // vmcnt(12) lgkmcnt(0)
                asm volatile("" ::: "memory");
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        const bf16x8 p0 = __builtin_bit_cast(bf16x8, u32x4{pc[0], pc[1], pc[2], pc[3]});
        const bf16x8 p1 = __builtin_bit_cast(bf16x8, u32x4{pc[4], pc[5], pc[6], pc[7]});
#pragma unroll
        for (int idx = 0; idx < 16; idx++) {
            if ((idx & 3) == 1) fetch_one(b + 4, KS, b + 2, (VS + 2) % 3, idx >> 2);
            if (idx + VA < 16) v_read(idx + VA);
            if (idx >= 16 - RA) kf[(idx - (16 - RA)) % (RA + 1)] = k_read(KN, idx - (16 - RA));
            const bf16x8 vf = __builtin_bit_cast(bf16x8, (s16x8)__builtin_shufflevector(vlo[idx % (VA + 1)], vhi[idx % (VA + 1)], 0, 1, 2, 3, 4, 5, 6, 7));
            const int ob = (idx >> 3) * 4 + (idx & 3);
            oacc[ob] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, ((idx >> 2) & 1) ? p1 : p0, oacc[ob], 0, 0, 0);
            if (idx == 4) sv = s; // the S MFMAs have drained by now
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    int b = 0;
    for (; b + 2 < nblk; b += 3) {
        step(IC<1>{}, IC<0>{}, b);
        step(IC<2>{}, IC<1>{}, b + 1);
        step(IC<0>{}, IC<2>{}, b + 2);
    }
    if (b < nblk) step(IC<1>{}, IC<0>{}, b);
    if (b + 1 < nblk) step(IC<2>{}, IC<1>{}, b + 1);
    __builtin_amdgcn_s_waitcnt(0x0F70); // no direct load may outlive the workgroup's LDS

    // ---- epilogue: O = O^T / l, or the range's share as it stands
    const float l_tot = pair_sum(l_run);
    if (q0 + l32 >= a.tokens) return;
    const float inv_l = l_tot > 0.f ? 1.0f / l_tot : 0.f;
    float* op = a.o + (int64_t)(q0 + l32) * WD + HALF * dh;
#pragma unroll
    for (int blk = 0; blk < 8; blk++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
            f32x4 v;
#pragma unroll
            for (int j = 0; j < 4; j++) v[j] = oacc[blk][4 * i + j] * inv_l;
            *reinterpret_cast<f32x4*>(op + 32 * blk + 8 * i + 4 * h) = v;
        }
}

} // namespace safe

// Combines the key ranges of a split launch, in range order: with reference points m_p and row
// sums l_p, O = sum_p 2^(m_p - m) O_p / sum_p 2^(m_p - m) l_p, m = max_p m_p. A thread owns four
// dims of one row; NP = the number of ranges is the build's, so that every range's load is sent
// before the first is used, with no branch between them.
template <int NP>
__global__ void __launch_bounds__(256) wide_merge_kernel(const WideArgs a) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; // (row, dim / 4)
    const int64_t row = i / (WD / 4);
    if (row >= a.tokens) return;
    const int c4 = (int)(i - row * (WD / 4));
    f32x2 ml[NP];
    f32x4 o[NP];
#pragma unroll
    for (int p = 0; p < NP; p++) ml[p] = *reinterpret_cast<const f32x2*>(a.part_ml + ((int64_t)p * a.tokens + row) * 2);
#pragma unroll
    for (int p = 0; p < NP; p++) o[p] = *reinterpret_cast<const f32x4*>(a.part_o + ((int64_t)p * a.tokens + row) * WD + 4 * c4);
    float mm = -INFINITY;
#pragma unroll
    for (int p = 0; p < NP; p++) mm = fmaxf(mm, ml[p][0]);
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    float lt = 0.f;
#pragma unroll
    for (int p = 0; p < NP; p++) {
        const float w = (ml[p][0] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(ml[p][0] - mm);
        acc += o[p] * w;
        lt += ml[p][1] * w;
    }
    const float inv = lt > 0.f ? 1.0f / lt : 0.f;
    *reinterpret_cast<f32x4*>(a.o + row * WD + 4 * c4) = acc * inv;
}

} // namespace wide

int wide_head_dim() { return wide::WD; }
int wide_block_rows() { return 64; } // the reference's tokens % 64 == 0; a last tile may be half full

hipError_t launch_wide_round(const WidePrepArgs& p, hipStream_t stream) {
    if (p.chunks <= 0) return hipErrorInvalidValue;
    const int64_t want = (p.chunks + 255) / 256;
    const unsigned blocks = (unsigned)(want < 4096 ? want : 4096);
    wide::wide_round_kernel<<<dim3(blocks, 3), dim3(256), 0, stream>>>(p);
    return hipGetLastError();
}

// Key ranges per query tile (one workgroup each): doubled while the launch still fits the
// device's CUs once and every range keeps at least eight key blocks. 16384 tokens are 128 tiles
// of two ranges, one workgroup per CU; 4096 tokens (the mid-block at 512 px) 32 tiles of eight.
int wide_splits(int tokens, int cus) {
    const int tiles = (tokens + wide::BQ - 1) / wide::BQ;
    const int nblk = tokens / wide::KB;
    int s = 1;
    while (s < wide::kMaxSplits && tiles * (s * 2) <= cus && nblk / (s * 2) >= 8 && nblk % (s * 2) == 0) s *= 2;
    return s;
}
size_t wide_part_bytes(int tokens, int splits) {
    return splits > 1 ? (size_t)splits * (size_t)tokens * (wide::WD + 2) * sizeof(float) : 0;
}

hipError_t launch_wide_attention(const WideArgs& a, hipStream_t stream) {
    if (a.tokens <= 0 || a.tokens % wide_block_rows() != 0) return hipErrorInvalidValue;
    const int nsp = a.splits > 1 ? a.splits : 1;
    if (nsp > wide::kMaxSplits || (nsp & (nsp - 1)) != 0 || (a.tokens / wide::KB) % nsp != 0) return hipErrorInvalidValue;
    if (nsp > 1 && (a.part_o == nullptr || a.part_ml == nullptr)) return hipErrorInvalidValue;
    const unsigned tiles = (unsigned)((a.tokens + wide::BQ - 1) / wide::BQ);
    if (a.redo == nullptr) return hipErrorInvalidValue;
    wide::attn_wide_kernel<<<dim3(tiles * (unsigned)nsp), dim3(wide::NT), wide::kLdsBytes, stream>>>(a);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    if (nsp > 1) {
        const int64_t threads = (int64_t)a.tokens * (wide::WD / 4);
        const dim3 mgrid((unsigned)((threads + 255) / 256));
        if (nsp == 2) wide::wide_merge_kernel<2><<<mgrid, dim3(256), 0, stream>>>(a);
        else if (nsp == 4) wide::wide_merge_kernel<4><<<mgrid, dim3(256), 0, stream>>>(a);
        else wide::wide_merge_kernel<8><<<mgrid, dim3(256), 0, stream>>>(a);
        if ((e = hipGetLastError()) != hipSuccess) return e;
    }
    // flagged tiles (none on ordinary data) are formed again, over whatever the launches above left there
    wide::safe::attn_wide_safe_kernel<<<dim3(tiles * 2u), dim3(wide::NT), wide::safe::kLdsBytes, stream>>>(a);
    return hipGetLastError();
}

hipError_t wide_setup() {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&wide::attn_wide_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)wide::kLdsBytes);
    if (e != hipSuccess) return e;
    return hipFuncSetAttribute(reinterpret_cast<const void*>(&wide::safe::attn_wide_safe_kernel),
                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)wide::safe::kLdsBytes);
}
int wide_tiles(int tokens) { return (tokens + wide::BQ - 1) / wide::BQ; }

} // namespace zdraw
