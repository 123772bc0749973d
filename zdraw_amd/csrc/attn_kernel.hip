// gfx950 flash-attention forward for zdraw's DiT joint self-attention.
//
// What it replaces in the reference: the Metal attention kernels behind
// zdraw_metal_run_attention* (metal/mattn_block_shader.zig:7-188, the steel
// route metal_api.m:6685-6815) together with the QK-norm + rope glue kernels
// that feed them (klein/zflux2_glue_shader.zig:61-122, metal/mqk_shader.zig:46-97).
// The design is MI355X-first, not a translation:
//
//   * one wave owns 32 query rows; a workgroup of NW waves shares each K/V tile;
//   * scores are computed TRANSPOSED (S^T = K . Q^T) with v_mfma_f32_32x32x16_bf16,
//     so every lane owns one query column: the online-softmax max/sum are
//     in-lane reductions plus one permlane32 swap, and the exponentiated tile
//     is already in the B-operand layout of the second MFMA (O^T = V^T . P^T),
//     no LDS round trip for P;
//   * K tiles sit in LDS row-major (padded pitch, conflict-free b128 reads);
//     V tiles are transposed in registers on the way in so the V^T operand is
//     one b128 read per MFMA;
//   * RMSNorm + rope are applied to the Q rows once in the prologue and to the
//     K rows between the global load and the LDS store of each tile;
//   * LDS is double buffered: tile i+1 is in flight in registers while tile i
//     is multiplied, one barrier per tile;
//   * the key-tile order is fixed and nothing is accumulated with atomics, so
//     the output is bit-identical from run to run.
#include "attn_device.hpp"

namespace zdraw {

constexpr int BK = kKeyTile;
constexpr int KPITCH = D + 8;   // bf16 elements per K row in LDS (272 B: b128 reads of 16 rows hit 16 bank groups)
constexpr int VPITCH = BK + 8;  // bf16 elements per V^T row in LDS (144 B)
constexpr int KS_ELEMS = BK * KPITCH;
constexpr int VT_ELEMS = D * VPITCH;

size_t attention_lds_bytes() {
    return (size_t)(2 * KS_ELEMS + 2 * VT_ELEMS) * sizeof(bf16_t) + (size_t)kMaxKeyTiles * sizeof(unsigned short);
}
int attention_block_rows(int nwaves) { return nwaves * 32; }

// ------------------------------------------------------------ the main kernel
template <typename TIn, int KMODE, int NW>
__global__ void __launch_bounds__(NW * 64) attn_fwd_kernel(const AttnArgs a) {
    constexpr int NT = NW * 64;
    constexpr int CPT = (BK * 16) / NT;  // 8-element K chunks per thread per tile
    constexpr int TPK = 16 / CPT;        // threads sharing one K row
    constexpr int VU = 512 / NT;         // V units (8 keys x 2 dims) per thread per tile
    static_assert(CPT * NT == BK * 16 && VU * NT == 512, "tile/thread mismatch");

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    bf16_t* const Ks = reinterpret_cast<bf16_t*>(smem);
    bf16_t* const Vt = Ks + 2 * KS_ELEMS;
    unsigned short* const tiles = reinterpret_cast<unsigned short*>(Vt + 2 * VT_ELEMS);
    __shared__ int s_ntiles;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int l32 = lane & 31;
    const int h = lane >> 5;

    // Workgroups are dealt round-robin to the 8 XCDs; remap so that consecutive
    // logical ids (same head, neighbouring query blocks) land on one XCD and
    // share its L2 copy of that head's K/V.
    int logical;
    {
        const int nwg = gridDim.x;
        const int xcd = blockIdx.x & 7;
        const int idx = blockIdx.x >> 3;
        const int base = nwg >> 3;
        const int rem = nwg & 7;
        logical = idx + xcd * base + (xcd < rem ? xcd : rem);
    }
    const int bh = logical / a.nqb;
    const int qb = logical - bh * a.nqb;
    const int seg = bh / a.heads;
    const int head = bh - seg * a.heads;
    const int q0 = qb * (NW * 32) + wave * 32;

    // ---- key-tile list: tiles with at least one admitted key, ascending
    const int nt_all = (a.key_limit + BK - 1) / BK;
    const unsigned char* const kp = a.key_pad ? a.key_pad + (int64_t)seg * a.mask_bs : nullptr;
    int ntiles = nt_all;
    if (kp) {
        if (wave == 0) {
            int count = 0;
            for (int base = 0; base < nt_all; base += 64) {
                const int t = base + lane;
                bool act = false;
                if (t < nt_all) {
                    const int k0 = t * BK;
                    const int k1 = min(k0 + BK, a.key_limit);
                    for (int j = k0; j < k1; j++) act |= (kp[j] == 0);
                }
                const unsigned long long m = __ballot(act);
                if (act) tiles[count + __popcll(m & ((1ull << lane) - 1ull))] = (unsigned short)t;
                count += __popcll(m);
            }
            if (lane == 0) s_ntiles = count;
        }
        __syncthreads();
        ntiles = s_ntiles;
    }

    // ---- Q rows -> B-operand registers (lane: query l32, dims 16s + 8h .. +7)
    bf16x8 qf[8];
    {
        const int qrow = q0 + l32;
        const bool ok = qrow < a.tokens;
        const TIn* qp = reinterpret_cast<const TIn*>(a.q) + (int64_t)seg * a.q_bs + (int64_t)(ok ? qrow : 0) * a.q_ts +
                        (int64_t)head * a.q_hs + 8 * h;
        float x[8][8];
#pragma unroll
        for (int s = 0; s < 8; s++) unpack8(ld_raw8<TIn>(qp + 16 * s, ok), x[s]);
        if (a.q_mode != kQkNone) {
            float ss = 0.f;
#pragma unroll
            for (int s = 0; s < 8; s++)
#pragma unroll
                for (int i = 0; i < 8; i++) ss += x[s][i] * x[s][i];
            ss = pair_sum(ss);
            const float inv = rsqrtf(ss * (1.0f / D) + a.qk.eps);
            const QkRow r = qk_row(a.qk, a.q_mode, a.q_w, a.q_w_txt, seg, qrow, ok);
#pragma unroll
            for (int s = 0; s < 8; s++) {
                const int d0 = 16 * s + 8 * h;
                const Rope8 t = ld_rope8(a.qk, a.q_mode, r, d0);
                qk_apply8(a.q_mode, x[s], inv, r.w, d0, t);
            }
        }
#pragma unroll
        for (int s = 0; s < 8; s++) qf[s] = __builtin_bit_cast(bf16x8, pack_bf16x8(x[s]));
    }

    // ---- tile staging (global -> registers -> LDS)
    const int lk_key = tid / TPK;          // K row inside the tile
    const int lk_d0 = (tid % TPK) * CPT * 8; // first dim of this thread's chunks
    const TIn* const kbase = reinterpret_cast<const TIn*>(a.k) + (int64_t)seg * a.k_bs + (int64_t)head * a.k_hs;
    const TIn* const vbase = reinterpret_cast<const TIn*>(a.v) + (int64_t)seg * a.v_bs + (int64_t)head * a.v_hs;

    Raw8<TIn> kraw[CPT];
    Rope8 krope[KMODE == kQkNone ? 1 : CPT];
    QkRow krow;
    unsigned vraw[VU][8];

    auto stage_load = [&](int tile) {
        const int key = tile * BK + lk_key;
        const bool ok = key < a.tokens;
        const TIn* p = kbase + (int64_t)(ok ? key : 0) * a.k_ts + lk_d0;
#pragma unroll
        for (int c = 0; c < CPT; c++) kraw[c] = ld_raw8<TIn>(p + 8 * c, ok);
        if constexpr (KMODE != kQkNone) {
            krow = qk_row(a.qk, KMODE, a.k_w, a.k_w_txt, seg, key, ok);
#pragma unroll
            for (int c = 0; c < CPT; c++) krope[c] = ld_rope8(a.qk, KMODE, krow, lk_d0 + 8 * c);
        }
#pragma unroll
        for (int u = 0; u < VU; u++) {
            const int unit = tid + u * NT;
            const int dc2 = unit & 63;   // dims 2*dc2, 2*dc2+1
            const int kg8 = unit >> 6;   // 8 keys: 16-block kg8/2, half kg8%2 -> keys {0..3, 8..11} + 4*half
            const int kb = tile * BK + (kg8 >> 1) * 16 + (kg8 & 1) * 4;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const int key_v = kb + (j & 3) + (j >> 2) * 8;
                const bool okv = key_v < a.tokens;
                vraw[u][j] = ld_pair_bf16(vbase + (int64_t)(okv ? key_v : 0) * a.v_ts + 2 * dc2, okv);
            }
        }
    };

    auto stage_store = [&](int buf) {
        bf16_t* kdst = Ks + buf * KS_ELEMS + lk_key * KPITCH + lk_d0;
        if constexpr (KMODE == kQkNone) {
#pragma unroll
            for (int c = 0; c < CPT; c++) *reinterpret_cast<u32x4*>(kdst + 8 * c) = raw_to_bf16(kraw[c]);
        } else {
            float x[CPT][8];
            float ss = 0.f;
#pragma unroll
            for (int c = 0; c < CPT; c++) {
                unpack8(kraw[c], x[c]);
#pragma unroll
                for (int i = 0; i < 8; i++) ss += x[c][i] * x[c][i];
            }
            ss = row_group_sum<TPK>(ss);
            const float inv = rsqrtf(ss * (1.0f / D) + a.qk.eps);
#pragma unroll
            for (int c = 0; c < CPT; c++) {
                qk_apply8(KMODE, x[c], inv, krow.w, lk_d0 + 8 * c, krope[c]);
                *reinterpret_cast<u32x4*>(kdst + 8 * c) = pack_bf16x8(x[c]);
            }
        }
#pragma unroll
        for (int u = 0; u < VU; u++) {
            const int unit = tid + u * NT;
            const int dc2 = unit & 63;
            const int kg8 = unit >> 6;
            // transpose 8 keys x 2 dims -> 2 rows of 8 keys (slot order = load order j)
            u32x4 lo, hi;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                lo[j] = __builtin_amdgcn_perm(vraw[u][2 * j + 1], vraw[u][2 * j], 0x05040100u);
                hi[j] = __builtin_amdgcn_perm(vraw[u][2 * j + 1], vraw[u][2 * j], 0x07060302u);
            }
            bf16_t* vdst = Vt + buf * VT_ELEMS + (2 * dc2) * VPITCH + kg8 * 8;
            *reinterpret_cast<u32x4*>(vdst) = lo;
            *reinterpret_cast<u32x4*>(vdst + VPITCH) = hi;
        }
    };

    // ---- running state: O^T accumulators (lane: query l32, dims 32*blk + 8i + 4h + j)
    f32x16 oacc[4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 16; j++) oacc[i][j] = 0.f;
    float m_run = -INFINITY; // running max of raw (unscaled) scores for this query
    float l_run = 0.f;       // this lane's half of the running denominator

    auto tile_of = [&](int i) -> int { return kp ? (int)tiles[i] : i; };

    if (ntiles > 0) {
        stage_load(tile_of(0));
        stage_store(0);
    }
    __syncthreads();

    for (int it = 0; it < ntiles; ++it) {
        const int cur = it & 1;
        const bool more = it + 1 < ntiles;
        const int tile = tile_of(it);
        if (more) stage_load(tile_of(it + 1));

        // S^T tile = K . Q^T: rows = 64 keys (2 blocks of 32), cols = 32 queries
        f32x16 sacc[2];
#pragma unroll
        for (int bb = 0; bb < 2; bb++)
#pragma unroll
            for (int j = 0; j < 16; j++) sacc[bb][j] = 0.f;
        {
            const bf16_t* kt = Ks + cur * KS_ELEMS + l32 * KPITCH + 8 * h;
#pragma unroll
            for (int s = 0; s < 8; s++) {
#pragma unroll
                for (int bb = 0; bb < 2; bb++) {
                    const bf16x8 kf = *reinterpret_cast<const bf16x8*>(kt + bb * 32 * KPITCH + 16 * s);
                    sacc[bb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[s], sacc[bb], 0, 0, 0);
                }
            }
        }

        // excluded keys (padding mask, key limit, tail of the last tile) -> -inf
        const int k0 = tile * BK;
        if (kp != nullptr || k0 + BK > a.key_limit) {
            const int key = k0 + lane;
            const bool bad = key >= a.key_limit || (kp != nullptr && kp[key] != 0);
            const unsigned long long badm = __ballot(bad);
            if (badm != 0ull) {
#pragma unroll
                for (int bb = 0; bb < 2; bb++)
#pragma unroll
                    for (int i = 0; i < 4; i++)
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            const int kk = 32 * bb + 8 * i + 4 * h + j;
                            if ((badm >> kk) & 1ull) sacc[bb][4 * i + j] = -INFINITY;
                        }
            }
        }

        // online softmax for this lane's query
        float mloc = sacc[0][0];
#pragma unroll
        for (int bb = 0; bb < 2; bb++)
#pragma unroll
            for (int j = 0; j < 16; j++) mloc = fmaxf(mloc, sacc[bb][j]);
        mloc = pair_max(mloc);
        const float m_new = fmaxf(m_run, mloc);
        const float mc = (m_new == -INFINITY) ? 0.f : m_new * a.scale_log2;
        const float alpha = __builtin_amdgcn_exp2f(m_run * a.scale_log2 - mc);
        const bool grew = m_new > m_run;
        m_run = m_new;
        float psum = 0.f;
#pragma unroll
        for (int bb = 0; bb < 2; bb++)
#pragma unroll
            for (int j = 0; j < 16; j++) {
                const float p = __builtin_amdgcn_exp2f(sacc[bb][j] * a.scale_log2 - mc);
                sacc[bb][j] = p;
                psum += p;
            }
        l_run = l_run * alpha + psum;
        if (__any(grew)) {
#pragma unroll
            for (int blk = 0; blk < 4; blk++)
#pragma unroll
                for (int j = 0; j < 16; j++) oacc[blk][j] *= alpha;
        }

        // O^T += V^T . P^T, 16 keys per MFMA; P^T comes straight from sacc
        {
            const bf16_t* vt = Vt + cur * VT_ELEMS + l32 * VPITCH + 8 * h;
#pragma unroll
            for (int kb = 0; kb < 4; kb++) {
                f32x8 pv;
#pragma unroll
                for (int j = 0; j < 8; j++) pv[j] = sacc[kb >> 1][8 * (kb & 1) + j];
                const bf16x8 pf = __builtin_convertvector(pv, bf16x8);
#pragma unroll
                for (int blk = 0; blk < 4; blk++) {
                    const bf16x8 vf = *reinterpret_cast<const bf16x8*>(vt + blk * 32 * VPITCH + 16 * kb);
                    oacc[blk] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf, oacc[blk], 0, 0, 0);
                }
            }
        }

        if (more) stage_store(cur ^ 1);
        __syncthreads();
    }

    // ---- epilogue: O = O^T / l
    const float l_tot = pair_sum(l_run);
    const float inv_l = l_tot > 0.f ? 1.0f / l_tot : 0.f;
    const int qrow = q0 + l32;
    if (qrow < a.tokens) {
        const int64_t off = (int64_t)seg * a.o_bs + (int64_t)qrow * a.o_ts + (int64_t)head * a.o_hs;
        if (a.out_dtype == kF32) {
            float* op = reinterpret_cast<float*>(a.o) + off;
#pragma unroll
            for (int blk = 0; blk < 4; blk++)
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    f32x4 v;
#pragma unroll
                    for (int j = 0; j < 4; j++) v[j] = oacc[blk][4 * i + j] * inv_l;
                    *reinterpret_cast<f32x4*>(op + 32 * blk + 8 * i + 4 * h) = v;
                }
        } else {
            bf16_t* op = reinterpret_cast<bf16_t*>(a.o) + off;
#pragma unroll
            for (int blk = 0; blk < 4; blk++)
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    f32x4 v;
#pragma unroll
                    for (int j = 0; j < 4; j++) v[j] = oacc[blk][4 * i + j] * inv_l;
                    *reinterpret_cast<bf16x4*>(op + 32 * blk + 8 * i + 4 * h) = __builtin_convertvector(v, bf16x4);
                }
        }
    }
}

// ------------------------------------------------ Q/K pre-pass (norm + rope)
// 16 lanes per row (8 dims each), 16 rows per workgroup. Rows are visited in
// (segment, head, token) order; input and output are addressed by strides, so
// the same kernel serves the bf16 head-major K pre-pass and the in-place f32
// token-major form. A lane reads and writes only its own 8 elements, so the
// output may alias the input.
template <typename TIn>
__global__ void __launch_bounds__(256) qk_prepass_kernel(const PrepArgs p) {
    const int64_t rows = (int64_t)p.batch * p.heads * p.tokens;
    const int64_t row = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 4);
    const bool ok = row < rows;
    const int d0 = (threadIdx.x & 15) * 8;
    const int64_t r = ok ? row : 0;
    const int tok = (int)(r % p.tokens);
    const int head = (int)((r / p.tokens) % p.heads);
    const int seg = (int)(r / ((int64_t)p.tokens * p.heads));
    const TIn* src = reinterpret_cast<const TIn*>(p.x) + (int64_t)seg * p.x_bs + (int64_t)tok * p.x_ts +
                     (int64_t)head * p.x_hs + d0;
    float x[8];
    unpack8(ld_raw8<TIn>(src, ok), x);
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 8; i++) ss += x[i] * x[i];
    // 16-lane sum: quad xor 1, xor 2, half mirror (8), row mirror (16)
    ss += __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(ss), 0xB1, 0xF, 0xF, true));
    ss += __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(ss), 0x4E, 0xF, 0xF, true));
    ss += __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(ss), 0x141, 0xF, 0xF, true));
    ss += __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(ss), 0x140, 0xF, 0xF, true));
    const float inv = rsqrtf(ss * (1.0f / D) + p.qk.eps);
    const QkRow qr = qk_row(p.qk, p.mode, p.w, p.w_txt, seg, tok, ok);
    const Rope8 t = ld_rope8(p.qk, p.mode, qr, d0);
    qk_apply8(p.mode, x, inv, qr.w, d0, t);
    if (ok) {
        const int64_t off = (int64_t)seg * p.y_bs + (int64_t)tok * p.y_ts + (int64_t)head * p.y_hs + d0;
        if (p.out_dtype == kF32) {
            float* dst = reinterpret_cast<float*>(p.y) + off;
            *reinterpret_cast<f32x4*>(dst) = f32x4{x[0], x[1], x[2], x[3]};
            *reinterpret_cast<f32x4*>(dst + 4) = f32x4{x[4], x[5], x[6], x[7]};
        } else {
            *reinterpret_cast<u32x4*>(reinterpret_cast<bf16_t*>(p.y) + off) = pack_bf16x8(x);
        }
    }
}

// ------------------------------------------------------------------- launch
template <typename TIn, int KMODE, int NW>
static hipError_t launch_one(const AttnArgs& a, hipStream_t stream) {
    const int64_t nwg = (int64_t)a.nqb * a.heads * a.batch;
    if (nwg <= 0 || nwg > 0x7fffffff) return hipErrorInvalidValue;
    attn_fwd_kernel<TIn, KMODE, NW><<<dim3((unsigned)nwg), dim3(NW * 64), attention_lds_bytes(), stream>>>(a);
    return hipGetLastError();
}

template <typename TIn, int NW>
static hipError_t launch_kmode(const AttnArgs& a, int k_mode, hipStream_t stream) {
    switch (k_mode) {
    case kQkNone: return launch_one<TIn, kQkNone, NW>(a, stream);
    case kQkKlein: return launch_one<TIn, kQkKlein, NW>(a, stream);
    case kQkZimage: return launch_one<TIn, kQkZimage, NW>(a, stream);
    default: return hipErrorInvalidValue;
    }
}

hipError_t launch_attention(const AttnArgs& a, int in_dtype, int k_mode, int nwaves, hipStream_t stream) {
    if (in_dtype == kF32) {
        return nwaves == 4 ? launch_kmode<float, 4>(a, k_mode, stream) : launch_kmode<float, 8>(a, k_mode, stream);
    } else if (in_dtype == kBF16) {
        return nwaves == 4 ? launch_kmode<bf16_t, 4>(a, k_mode, stream) : launch_kmode<bf16_t, 8>(a, k_mode, stream);
    }
    return hipErrorInvalidValue;
}

hipError_t launch_qk_prepass(const PrepArgs& p, int in_dtype, hipStream_t stream) {
    const int64_t rows = (int64_t)p.batch * p.heads * p.tokens;
    const int64_t nwg = (rows + 15) / 16;
    if (nwg <= 0 || nwg > 0x7fffffff) return hipErrorInvalidValue;
    if (in_dtype == kF32)
        qk_prepass_kernel<float><<<dim3((unsigned)nwg), dim3(256), 0, stream>>>(p);
    else if (in_dtype == kBF16)
        qk_prepass_kernel<bf16_t><<<dim3((unsigned)nwg), dim3(256), 0, stream>>>(p);
    else
        return hipErrorInvalidValue;
    return hipGetLastError();
}

template <typename TIn, int KMODE, int NW>
static hipError_t raise_lds() {
    return hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_fwd_kernel<TIn, KMODE, NW>),
                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)attention_lds_bytes());
}

hipError_t attention_setup() {
    hipError_t e;
#define ZD_RAISE(T, M, W) if ((e = raise_lds<T, M, W>()) != hipSuccess) return e;
    ZD_RAISE(float, kQkNone, 4) ZD_RAISE(float, kQkKlein, 4) ZD_RAISE(float, kQkZimage, 4)
    ZD_RAISE(float, kQkNone, 8) ZD_RAISE(float, kQkKlein, 8) ZD_RAISE(float, kQkZimage, 8)
    ZD_RAISE(bf16_t, kQkNone, 4) ZD_RAISE(bf16_t, kQkKlein, 4) ZD_RAISE(bf16_t, kQkZimage, 4)
    ZD_RAISE(bf16_t, kQkNone, 8) ZD_RAISE(bf16_t, kQkKlein, 8) ZD_RAISE(bf16_t, kQkZimage, 8)
#undef ZD_RAISE
    return hipSuccess;
}

} // namespace zdraw
