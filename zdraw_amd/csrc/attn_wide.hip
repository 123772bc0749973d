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
//   * a workgroup of 8 waves owns 64 query rows: wave (g, s) owns query rows
//     32 g .. 32 g + 31 and the 128-wide slice s of the 512 dims, as the
//     reference's four simdgroups do. Every K/V byte is read once per workgroup;
//   * per 32-key block a wave forms its partial S^T = K_s Q_s^T (8 MFMAs), the
//     four partials of a query group are exchanged through LDS and summed in the
//     written-out order ((p0 + p1) + p2) + p3 by each of the four waves, which
//     then run the same online softmax redundantly (P must sit in every wave's
//     registers for its own V slice anyway) and add V_s^T P^T to their slice of
//     O^T (8 MFMAs). Scores are transposed (a lane owns one query), so P^T is
//     the MFMA's B operand without an LDS round trip;
//   * K/V blocks alternate between two LDS stages filled by buffer_load ... lds
//     with the swizzled 256-byte-row layout of the head_dim-128 kernel;
//   * fixed block order and fixed summation order: bit-identical from run to run.
#include "attn_device.hpp"

namespace zdraw {

namespace wide {

constexpr int WD = 512;           // head_dim
constexpr int SL = 128;           // dims per slice
constexpr int NSL = WD / SL;      // slices = waves per query group
constexpr int KB = 32;            // keys per block
constexpr int NW = 8;
constexpr int NT = NW * 64;
constexpr int BQ = 64;            // query rows per workgroup
constexpr int TILE_BYTES = KB * SL * 2;            // one slice of a K (or V) block: 8 KB
constexpr int RING_BYTES = NSL * TILE_BYTES;       // one K (or V) block, all slices: 32 KB
constexpr int V_RING = 2 * RING_BYTES;             // two K slots, then two V slots
constexpr int X_BYTES = 2 * NSL * 64 * 16 * 4;     // partial scores: [group][slice][4 x (lane x 16 B)]: 32 KB
constexpr size_t kLdsBytes = (size_t)4 * RING_BYTES + X_BYTES;
constexpr float kTau = 8.0f;      // log2 headroom of the lazy softmax maximum

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

// f32 -> bf16 with a scale, 8 elements per thread; blockIdx.y selects the operand.
__global__ void __launch_bounds__(256) wide_round_kernel(const WidePrepArgs p) {
    const int op = (int)blockIdx.y;
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

__global__ void __launch_bounds__(NT, 2) attn_wide_kernel(const WideArgs a) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int l32 = lane & 31;
    const int h = lane >> 5;
    const int grp = wave >> 2;  // query group
    const int sl = wave & 3;    // dim slice
    const int q0 = (int)blockIdx.x * BQ + 32 * grp;
    const int nblk = a.tokens / KB;

    const unsigned lds0 = lds_address(smem);
    const unsigned xbase = lds0 + 4 * RING_BYTES;

    // ---- Q fragments (B operand): query q0 + l32, dims 128 sl + 16 kk + 8 h .. +7
    bf16x8 qf[8];
    {
        const bf16_t* qp = reinterpret_cast<const bf16_t*>(a.q) + (int64_t)(q0 + l32) * WD + SL * sl + 8 * h;
#pragma unroll
        for (int kk = 0; kk < 8; kk++) qf[kk] = *reinterpret_cast<const bf16x8*>(qp + 16 * kk);
    }

    // ---- block fetch: wave w fills rows 16 (w >> 2) .. +15 of slice w & 3 of a K block or of a
    // V block, four rows per instruction. The lane that fills chunk position p of row r
    // fetches the chunk the swizzle places there: K chunk c of row r sits at c ^ (r & 15),
    // V chunk c at c ^ ((r & 3) << 2). Positions past the last block re-fetch the last block
    // into a slot nobody reads any more.
    const unsigned span = (unsigned)a.tokens * (unsigned)(WD * 2);
    const u32x4 k_rsrc = make_rsrc_words(a.k, span);
    const u32x4 v_rsrc = make_rsrc_words(a.v, span);
    unsigned fk_off[4], fv_off[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int row = 16 * grp + 4 * j + (lane >> 4);
        const unsigned kc = (unsigned)((lane & 15) ^ (row & 15));
        const unsigned vc = (unsigned)((lane & 15) ^ ((row & 3) << 2));
        fk_off[j] = (unsigned)row * (WD * 2) + (unsigned)sl * (SL * 2) + kc * 16u;
        fv_off[j] = (unsigned)row * (WD * 2) + (unsigned)sl * (SL * 2) + vc * 16u;
    }
    const unsigned fetch_lds = __builtin_amdgcn_readfirstlane(lds0 + (unsigned)sl * TILE_BYTES + (unsigned)(16 * grp) * (SL * 2));
    auto fetch_k = [&](int blk, int slot) __attribute__((always_inline)) {
        const unsigned uo = (unsigned)(blk < nblk ? blk : nblk - 1) * (unsigned)(KB * WD * 2);
        const unsigned base = fetch_lds + (unsigned)slot * RING_BYTES;
#pragma unroll
        for (int j = 0; j < 4; j++) load_to_lds_16(k_rsrc, base + (unsigned)(4 * j) * (SL * 2), fk_off[j], uo);
    };
    auto fetch_v = [&](int blk, int slot) __attribute__((always_inline)) {
        const unsigned uo = (unsigned)(blk < nblk ? blk : nblk - 1) * (unsigned)(KB * WD * 2);
        const unsigned base = fetch_lds + V_RING + (unsigned)slot * RING_BYTES;
#pragma unroll
        for (int j = 0; j < 4; j++) load_to_lds_16(v_rsrc, base + (unsigned)(4 * j) * (SL * 2), fv_off[j], uo);
    };

    // ---- fragment addresses in slot 0 of each ring (a slot adds a constant)
    const int tr_row = (lane & 15) >> 2;
    const int tr_col = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
    unsigned kfo[8], vfo[4];
#pragma unroll
    for (int kk = 0; kk < 8; kk++)
        kfo[kk] = lds0 + (unsigned)sl * TILE_BYTES + (unsigned)((l32 * SL + (((2 * kk + h) ^ (l32 & 15)) * 8)) * 2);
#pragma unroll
    for (int blk = 0; blk < 4; blk++)
        vfo[blk] = lds0 + V_RING + (unsigned)sl * TILE_BYTES +
                   (unsigned)(((4 * h + tr_row) * SL + ((blk ^ tr_row) * 32) + tr_col) * 2);
    typedef const __attribute__((address_space(3))) bf16x8* lds_bf16x8_t;
    typedef __attribute__((address_space(3))) s16x4* lds_s16x4_t;
    typedef __attribute__((address_space(3))) f32x4* lds_f32x4_t;

    // partial-score exchange: [group][slice][i < 4][lane] x 16 B
    const unsigned x_mine = xbase + (unsigned)(((grp * NSL + sl) * 4) * 64 + lane) * 16u;
    const unsigned x_group = xbase + (unsigned)((grp * NSL * 4) * 64 + lane) * 16u;
    auto x_write = [&](const f32x16& sp) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 4; i++)
            *(lds_f32x4_t)(x_mine + (unsigned)(i * 64 * 16)) = f32x4{sp[4 * i], sp[4 * i + 1], sp[4 * i + 2], sp[4 * i + 3]};
    };
    // full scores: ((p0 + p1) + p2) + p3, the same in each of the group's four waves
    auto x_sum = [&](f32x16& sv) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            f32x4 t = *(lds_f32x4_t)(x_group + (unsigned)((0 * 4 + i) * 64 * 16));
#pragma unroll
            for (int s = 1; s < NSL; s++) {
                const f32x4 u = *(lds_f32x4_t)(x_group + (unsigned)((s * 4 + i) * 64 * 16));
                t += u;
            }
#pragma unroll
            for (int j = 0; j < 4; j++) sv[4 * i + j] = t[j];
        }
    };

    f32x16 oacc[4]; // O^T slice: lane = query l32, dims 128 sl + 32 blk + 8 i + 4 h + j
#pragma unroll
    for (int blk = 0; blk < 4; blk++)
#pragma unroll
        for (int j = 0; j < 16; j++) oacc[blk][j] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;

    // ---- prologue: K(0), K(1), V(0) in; scores of block 0 exchanged; K(2), V(1) requested.
    // K runs one block ahead of V: step b multiplies by K(b+1) and by V(b).
    fetch_k(0, 0);
    fetch_v(0, 0);
    fetch_k(1, 1);
    __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0)
    __syncthreads();
    f32x16 sv; // scores of the block the next step exponentiates: lane = query l32, element 4 i + j = key 8 i + 4 h + j
    {
        f32x16 sp;
#pragma unroll
        for (int j = 0; j < 16; j++) sp[j] = 0.f;
#pragma unroll
        for (int kk = 0; kk < 8; kk++)
            sp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(lds_bf16x8_t)(kfo[kk]), qf[kk], sp, 0, 0, 0);
        x_write(sp);
        __syncthreads();
        x_sum(sv);
        __syncthreads();
    }
    fetch_k(2, 0);
    fetch_v(1, 1);

    // One step: the MFMAs of S(b+1) = K(b+1) Q^T (this wave's slice) run with the softmax of
    // block b in their shadow, then O += V(b)^T P(b)^T; the partial scores of block b+1 are
    // published between the two, and collected after the barrier that also says "block
    // b+2's K and block b+1's V have landed, K(b+1) and V(b) have no reader left".
    for (int b = 0; b < nblk; b++) {
        const unsigned kso = (unsigned)((b + 1) & 1) * RING_BYTES;
        const unsigned vso = (unsigned)(b & 1) * RING_BYTES;
        bf16x8 kf[8];
        s16x4 vlo[8], vhi[8];
#pragma unroll
        for (int kk = 0; kk < 8; kk++) kf[kk] = *(lds_bf16x8_t)(kfo[kk] + kso);
        auto v_read = [&](int idx) __attribute__((always_inline)) {
            const int kb = idx >> 2, blk = idx & 3;
            const unsigned va = vfo[blk] + vso + (unsigned)(16 * kb) * (SL * 2);
            vlo[idx] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_t)va);
            vhi[idx] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_t)(va + 8u * (SL * 2)));
        };
        f32x16 sp;
#pragma unroll
        for (int j = 0; j < 16; j++) sp[j] = 0.f;
        float mloc = 0.f, mc = 0.f, alpha = 1.f, psum = 0.f;
        bool up = false;
        unsigned pc[8];
        auto exp_pair = [&](int pr) __attribute__((always_inline)) {
            f32x2 pp;
            pp[0] = __builtin_amdgcn_exp2f(sv[2 * pr] - mc);
            pp[1] = __builtin_amdgcn_exp2f(sv[2 * pr + 1] - mc);
            psum += pp[0] + pp[1];
            pc[pr] = __builtin_bit_cast(unsigned, __builtin_convertvector(pp, bf16x2));
        };
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int g = 0; g < 8; g++) {
            sp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[g], qf[g], sp, 0, 0, 0);
            // softmax of block b in the exp2 domain (the scale rides on Q) with a lazy maximum:
            // the reference point moves only when this block's maximum exceeds it by more than kTau
            if (g == 0) {
                mloc = fmaxf(fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3])), fmaxf(fmaxf(sv[4], sv[5]), fmaxf(sv[6], sv[7])));
                v_read(0);
                v_read(1);
            } else if (g == 1) {
                mloc = fmaxf(mloc, fmaxf(fmaxf(fmaxf(sv[8], sv[9]), fmaxf(sv[10], sv[11])), fmaxf(fmaxf(sv[12], sv[13]), fmaxf(sv[14], sv[15]))));
                const float mlc = pair_max(mloc);
                up = mlc > m_run + kTau;
                const float m_new = up ? mlc : m_run;
                mc = (m_new == -INFINITY) ? 0.f : m_new;
                alpha = __builtin_amdgcn_exp2f(m_run - mc);
                m_run = m_new;
                v_read(2);
                v_read(3);
            } else if (g < 6) {
                exp_pair(2 * (g - 2));
                exp_pair(2 * (g - 2) + 1);
                if (g < 4) {
                    v_read(2 * g);
                    v_read(2 * g + 1);
                }
            } else if (g == 6) {
                l_run = l_run * alpha + psum;
                if (__any(up)) {
#pragma unroll
                    for (int blk = 0; blk < 4; blk++)
#pragma unroll
                        for (int j = 0; j < 16; j++) oacc[blk][j] *= alpha;
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        const bf16x8 p0 = __builtin_bit_cast(bf16x8, u32x4{pc[0], pc[1], pc[2], pc[3]});
        const bf16x8 p1 = __builtin_bit_cast(bf16x8, u32x4{pc[4], pc[5], pc[6], pc[7]});
        // O^T slice += V_s(b)^T . P^T; the transposing read delivers keys in P's order
#pragma unroll
        for (int idx = 0; idx < 8; idx++) {
            const bf16x8 vf = __builtin_bit_cast(bf16x8, (s16x8)__builtin_shufflevector(vlo[idx], vhi[idx], 0, 1, 2, 3, 4, 5, 6, 7));
            oacc[idx & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, idx < 4 ? p0 : p1, oacc[idx & 3], 0, 0, 0);
            if (idx == 1) x_write(sp); // the S MFMAs have drained by now
            __builtin_amdgcn_sched_barrier(0);
        }
        // every wave has seen its own part of K(b+2) and V(b+1) land (requested a step ago)
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();
        fetch_k(b + 3, (b + 1) & 1);
        fetch_v(b + 2, b & 1);
        x_sum(sv);
        __syncthreads(); // the exchange area is rewritten in the next step
    }
    __builtin_amdgcn_s_waitcnt(0x0F70); // no direct load may outlive the workgroup's LDS

    // ---- epilogue: O = O^T / l
    const float l_tot = pair_sum(l_run);
    const float inv_l = l_tot > 0.f ? 1.0f / l_tot : 0.f;
    float* op = a.o + (int64_t)(q0 + l32) * WD + SL * sl;
#pragma unroll
    for (int blk = 0; blk < 4; blk++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
            f32x4 v;
#pragma unroll
            for (int j = 0; j < 4; j++) v[j] = oacc[blk][4 * i + j] * inv_l;
            *reinterpret_cast<f32x4*>(op + 32 * blk + 8 * i + 4 * h) = v;
        }
}

} // namespace wide

int wide_head_dim() { return wide::WD; }
int wide_block_rows() { return wide::BQ; }

hipError_t launch_wide_round(const WidePrepArgs& p, hipStream_t stream) {
    if (p.chunks <= 0) return hipErrorInvalidValue;
    const int64_t want = (p.chunks + 255) / 256;
    const unsigned blocks = (unsigned)(want < 4096 ? want : 4096);
    wide::wide_round_kernel<<<dim3(blocks, 3), dim3(256), 0, stream>>>(p);
    return hipGetLastError();
}

hipError_t launch_wide_attention(const WideArgs& a, hipStream_t stream) {
    if (a.tokens <= 0 || a.tokens % wide::BQ != 0) return hipErrorInvalidValue;
    wide::attn_wide_kernel<<<dim3((unsigned)(a.tokens / wide::BQ)), dim3(wide::NT), wide::kLdsBytes, stream>>>(a);
    return hipGetLastError();
}

hipError_t wide_setup() {
    return hipFuncSetAttribute(reinterpret_cast<const void*>(&wide::attn_wide_kernel),
                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)wide::kLdsBytes);
}

} // namespace zdraw
