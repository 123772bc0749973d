// Role-split build of the attention forward kernel for prepared bf16 operands (gfx950).
// Included by attn_fwd.hip inside namespace zdraw::fwd; shares its constants and helpers.
//
// The single-role kernel gives every wave 32 query rows, so every wave reads every K and V
// fragment of a key block from LDS: 16 KB per 16 MFMAs, and those reads are a quarter of the
// kernel's energy on a chip that runs at its power limit. Here the two waves that share a SIMD
// share 64 query rows and split the WORK instead of the rows:
//
//   * the S-wave keeps the 64 query rows as B operands, forms S^T = K Q^T for both 32-row halves
//     from ONE read of each K fragment, runs the softmax and writes P^T (bf16, 4 KB per key
//     block) into a two-slot LDS mailbox;
//   * the O-wave keeps O^T for the 64 rows (128 accumulation registers), reads P^T back in the
//     very register image the second MFMA wants, and forms O^T += V^T P^T for both halves from
//     ONE read of each V fragment.
//
// Per 32 MFMAs the pair reads 8 KB of K, 8 KB of V and moves 4 KB of P in and out of LDS: 24 KB
// where two single-role waves read 32 KB. The register budget that made 64 rows per wave
// impossible at two waves per SIMD (128 accumulators + 64 of Q + scores) is split between the
// two roles. Everything else is the single-role design: transposed scores, the transposing LDS
// read for V, direct-to-LDS block loads in the swizzled layout, one lane per query column.
//
// Measured, it does not pay: the S-wave carries the whole softmax of 64 rows in ONE in-order
// instruction stream (two exponentials, two adds and a pack behind each of its MFMAs), which alone
// takes more cycles per MFMA than the pipe needs, and a wave priority either way only makes the
// two roles take turns; a key block takes 1650 cycles against 1270 in the single-role kernel. The
// chip then runs at 1.93 instead of 1.6 GHz (it draws less power), which does not make up for
// it. The build is kept behind the measurement knob and under the same tests.
//
// Pipeline, one workgroup barrier per 32-key step b (steps 0 .. nblk + 1):
//   S-wave: S(b+1) = K(b+1) Q^T on the MFMAs with the softmax of S(b) between them; P(b) -> slot b & 1
//   O-wave: O^T += V(b-2)^T P(b-2)^T from registers; meanwhile it reads P(b-1) from slot (b-1) & 1
//           and the first fragments of V(b-1) for the next step, so a step starts with its
//           operands in registers instead of waiting out an LDS round trip behind the barrier
//   every wave: requests its four rows of K(b + AK) and of V(b + AV); before the barrier it waits
//   until all but its last four loads have landed, so a block requested at step b is readable
//   from step b + 3 on.
// Ring depths follow: K(j) is requested at step j - AK and last read at step j - 1 (NK >= AK),
// V(j) is requested at step j - AV, first read at step j + 1 and last at step j + 2 (NV >= AV + 3).
#pragma once

namespace pairk {

constexpr int NK = 6;  // K ring stages
constexpr int NV = 8;  // V ring stages
constexpr int AK = 5;  // K(j) is requested AK steps before step j (its S is formed in step j - 1)
constexpr int AV = 2;  // V(j) is requested AV steps before step j (it is consumed in step j + 2)
constexpr int STAGE = KB * D;                       // elements per ring stage (unpadded rows)
constexpr int PSLOT = 4096 + 512 + 256;             // P^T of a step, the rows' rescale factors, a flag
constexpr size_t kRingBytes = (size_t)(NK + NV) * STAGE * sizeof(bf16_t);
constexpr size_t kMailBytes = (size_t)4 * 2 * PSLOT;
constexpr size_t kLdsBytes = kRingBytes + kMailBytes + kListBytes;
constexpr size_t kLdsAlloc = kLdsBytes;
static_assert(NK >= AK && NV >= AV + 3 && (NV & (NV - 1)) == 0, "ring depths");
static_assert(kLdsAlloc <= 160 * 1024, "LDS budget");

template <bool MASKED, bool BOUNDED>
__global__ void __launch_bounds__(512, 2) attn_pair_kernel(const AttnArgs a) {
    constexpr int NT = 512;
    constexpr int BQ = 256;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    bf16_t* const Ks = reinterpret_cast<bf16_t*>(smem);
    bf16_t* const Vs = Ks + NK * STAGE;
    unsigned char* const mail = reinterpret_cast<unsigned char*>(Vs + NV * STAGE);
    unsigned short* const blocks = reinterpret_cast<unsigned short*>(mail + kMailBytes);
    unsigned* const bmask = reinterpret_cast<unsigned*>(blocks + MAX_BLOCKS);
    __shared__ int s_nblocks;

    unsigned long long clk_c0 = 0, clk_r0 = 0;
    if (a.clock_probe) {
        clk_c0 = __builtin_readcyclecounter();
        clk_r0 = __builtin_amdgcn_s_memrealtime();
    }
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int pr_id = wave & 3;   // the pair: waves p and p + 4 share a SIMD and 64 query rows
    const bool o_role = wave >= 4;
    const int l32 = lane & 31;
    const int h = lane >> 5;

    // XCD-aware remap, as in the single-role kernel
    int logical;
    int split = 0;
    if (a.splits > 1) {
        const int t = (int)blockIdx.x / a.splits;
        split = (int)blockIdx.x - t * a.splits;
        logical = a.tile_base + t;
    } else {
        const int nwg = gridDim.x;
        const int xcd = blockIdx.x & 7;
        const int idx = blockIdx.x >> 3;
        const int base = nwg >> 3;
        const int rem = nwg & 7;
        logical = a.tile_base + idx + xcd * base + (xcd < rem ? xcd : rem);
    }
    const int bh = logical / a.nqb;
    const int qb = logical - bh * a.nqb;
    const int seg = bh / a.heads;
    const int head = bh - seg * a.heads;
    const int q0 = qb * BQ + pr_id * 64;

    // ---- key-block list (the masked build): exclusion mask per block, blocks that admit a key
    const int nb_all = (a.key_limit + KB - 1) / KB;
    const unsigned char* const kp = a.key_pad ? a.key_pad + (int64_t)seg * a.mask_bs : nullptr;
    int nblk = nb_all;
    if constexpr (MASKED) {
        for (int t2 = wave; 2 * t2 < nb_all; t2 += 8) {
            const int key = t2 * 64 + lane;
            const bool bad = key >= a.key_limit || (kp != nullptr && kp[key < a.key_limit ? key : 0] != 0);
            const unsigned long long m = __ballot(bad);
            if (lane == 0) {
                bmask[2 * t2] = (unsigned)m;
                if (2 * t2 + 1 < MAX_BLOCKS) bmask[2 * t2 + 1] = (unsigned)(m >> 32);
            }
        }
        __syncthreads();
        if (kp) {
            if (wave == 0) {
                int count = 0;
                for (int base = 0; base < nb_all; base += 64) {
                    const int t = base + lane;
                    const bool act = t < nb_all && bmask[t < nb_all ? t : 0] != 0xffffffffu;
                    const unsigned long long m = __ballot(act);
                    if (act) blocks[count + __popcll(m & ((1ull << lane) - 1ull))] = (unsigned short)t;
                    count += __popcll(m);
                }
                if (lane == 0) s_nblocks = count;
            }
            __syncthreads();
            nblk = __builtin_amdgcn_readfirstlane(s_nblocks);
        }
    }
    int i0 = 0;
    if (a.splits > 1) {
        const int per = (nblk + a.splits - 1) / a.splits;
        i0 = split * per;
        nblk = max(min(nblk - i0, per), 0);
    }
    auto block_of = [&](int i) -> int { return (MASKED && kp) ? __builtin_amdgcn_readfirstlane((int)blocks[i + i0]) : i + i0; };

    // ---- direct-to-LDS block loads: wave w moves rows 4 w + lane / 16 of a block (both roles load)
    const int last_row = a.tokens - 1;
    const int last_blk = last_row / KB;
    const unsigned k_span = ((unsigned)(a.tokens - 1) * (unsigned)a.k_ts + D) * 2u;
    const unsigned v_span = ((unsigned)(a.tokens - 1) * (unsigned)a.v_ts + D) * 2u;
    const unsigned k_blk_bytes = (unsigned)a.k_ts * (unsigned)(KB * 2);
    const unsigned v_blk_bytes = (unsigned)a.v_ts * (unsigned)(KB * 2);
    const int dma_row = 4 * wave + (lane >> 4);
    const unsigned dma_k_chunk = (unsigned)(((lane & 15) ^ (dma_row & 15)) * 8);
    const unsigned dma_v_chunk = (unsigned)(((lane & 15) ^ ((dma_row & 3) << 2)) * 8);
    const unsigned dma_k_off = ((unsigned)dma_row * (unsigned)a.k_ts + dma_k_chunk) * 2u;
    const unsigned dma_v_off = ((unsigned)dma_row * (unsigned)a.v_ts + dma_v_chunk) * 2u;
    const int dma_tail_row = min(dma_row, last_row - last_blk * KB);
    const unsigned dma_k_off_tail = ((unsigned)dma_tail_row * (unsigned)a.k_ts + dma_k_chunk) * 2u;
    const unsigned dma_v_off_tail = ((unsigned)dma_tail_row * (unsigned)a.v_ts + dma_v_chunk) * 2u;
    const u32x4 dma_k_rsrc = make_rsrc_words(reinterpret_cast<const bf16_t*>(a.k) + (int64_t)seg * a.k_bs + (int64_t)head * a.k_hs, k_span);
    const u32x4 dma_v_rsrc = make_rsrc_words(reinterpret_cast<const bf16_t*>(a.v) + (int64_t)seg * a.v_bs + (int64_t)head * a.v_hs, v_span);
    const unsigned dma_k_lds = __builtin_amdgcn_readfirstlane(lds_address(Ks) + (unsigned)(4 * wave * D * 2));
    const unsigned dma_v_lds = __builtin_amdgcn_readfirstlane(lds_address(Vs) + (unsigned)(4 * wave * D * 2));
    // Positions past the end of the list re-fetch the last block into a stage nobody reads any
    // more: the count of loads per step stays fixed, which the waits before the barriers rely on.
    auto fetch_k = [&](int i) __attribute__((always_inline)) {
        const int ii = i < nblk ? i : nblk - 1;
        const int blk = block_of(ii);
        unsigned ko = dma_k_off;
        if constexpr (MASKED) ko = blk >= last_blk ? dma_k_off_tail : dma_k_off;
        load_to_lds_16(dma_k_rsrc, dma_k_lds + (unsigned)(i % NK) * (STAGE * 2u), ko, (unsigned)blk * k_blk_bytes);
    };
    auto fetch_v = [&](int i) __attribute__((always_inline)) {
        const int ii = i < nblk ? i : nblk - 1;
        const int blk = block_of(ii);
        unsigned vo = dma_v_off;
        if constexpr (MASKED) vo = blk >= last_blk ? dma_v_off_tail : dma_v_off;
        load_to_lds_16(dma_v_rsrc, dma_v_lds + (unsigned)(i & (NV - 1)) * (STAGE * 2u), vo, (unsigned)blk * v_blk_bytes);
    };
    // the wait before a step's barrier: all but this wave's last four block loads have landed
    auto step_end = [&](bool last) __attribute__((always_inline)) {
        asm volatile("" ::: "memory");
        if (last) __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0)
        else __builtin_amdgcn_s_waitcnt(0x0074);       // vmcnt(4) lgkmcnt(0)
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    };

    // mailbox of this pair: two slots of P^T (register image: 16 bytes per lane and (half, key
    // half)), the rescale factors of the rows (the running-maximum build) and a flag
    const unsigned mail_lds = lds_address(mail) + (unsigned)(pr_id * 2 * PSLOT);
    typedef __attribute__((address_space(3))) u32x4* lds_w128_t;
    typedef const __attribute__((address_space(3))) u32x4* lds_r128_t;
    typedef __attribute__((address_space(3))) float* lds_wf_t;
    typedef const __attribute__((address_space(3))) float* lds_rf_t;
    typedef __attribute__((address_space(3))) unsigned* lds_wu_t;
    typedef const __attribute__((address_space(3))) unsigned* lds_ru_t;

    const int tr_row = (lane & 15) >> 2;
    const int tr_col = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
    typedef short s16x8 __attribute__((ext_vector_type(8)));

    if (nblk <= 0) {
        // no admitted key at all (a part of a key-split tile beyond the list, or every key masked)
        if (o_role) {
#pragma unroll
            for (int qi = 0; qi < 2; qi++) {
                const int qrow = q0 + 32 * qi + l32;
                if (a.splits > 1) {
                    const int64_t prow = ((int64_t)blockIdx.x * BQ + pr_id * 64 + 32 * qi + l32);
                    float* op = a.part_o + prow * D;
                    for (int c = 0; c < 16; c++) *reinterpret_cast<f32x4*>(op + 64 * h + 4 * c) = f32x4{0.f, 0.f, 0.f, 0.f};
                    if (h == 0) {
                        a.part_ml[prow * 2] = BOUNDED ? 0.f : -INFINITY;
                        a.part_ml[prow * 2 + 1] = 0.f;
                    }
                } else if (qrow < a.tokens) {
                    const int64_t off = (int64_t)seg * a.o_bs + (int64_t)qrow * a.o_ts + (int64_t)head * a.o_hs + 64 * h;
                    if (a.out_dtype == kF32) {
                        for (int c = 0; c < 16; c++) *reinterpret_cast<f32x4*>(reinterpret_cast<float*>(a.o) + off + 4 * c) = f32x4{0.f, 0.f, 0.f, 0.f};
                    } else {
                        for (int c = 0; c < 8; c++) *reinterpret_cast<u32x4*>(reinterpret_cast<unsigned short*>(a.o) + off + 8 * c) = u32x4{0u, 0u, 0u, 0u};
                    }
                }
            }
        }
        return;
    }

    // ---- prologue: the first AK blocks of K and AV blocks of V are requested by everybody
#pragma unroll
    for (int i = 0; i < AK; i++) fetch_k(i);
#pragma unroll
    for (int i = 0; i < AV; i++) fetch_v(i);

    if (!o_role) {
        // =============================================================== S-wave
        // Q rows -> B-operand registers: qf[qi][s], lane: query 32 qi + l32, dims 16 s + 8 h .. +7.
        // Each lane fetches the 16 pieces of its own two rows (prepared bf16, the softmax scale
        // folded in); all are in flight together with the block loads above.
        bf16x8 qf[2][8];
        {
            const bf16_t* const qbase = reinterpret_cast<const bf16_t*>(a.q) + (int64_t)seg * a.q_bs + (int64_t)head * a.q_hs + 8 * h;
#pragma unroll
            for (int qi = 0; qi < 2; qi++) {
                const int qrow = min(q0 + 32 * qi + l32, a.tokens - 1); // rows past the sequence re-read the last row (never stored)
                const bf16_t* const src = qbase + (int64_t)qrow * a.q_ts;
#pragma unroll
                for (int s = 0; s < 8; s++) qf[qi][s] = *reinterpret_cast<const bf16x8*>(src + 16 * s);
            }
            if (a.scale_log2 != 1.0f) {
#pragma unroll
                for (int qi = 0; qi < 2; qi++)
#pragma unroll
                    for (int s = 0; s < 8; s++) {
                        f32x8 x = __builtin_convertvector(qf[qi][s], f32x8);
                        x *= a.scale_log2;
                        qf[qi][s] = __builtin_convertvector(x, bf16x8);
                    }
            }
        }
        unsigned kfo[8];
#pragma unroll
        for (int s = 0; s < 8; s++) kfo[s] = lds_address(Ks) + (unsigned)((l32 * D + (((2 * s + h) ^ (l32 & 15)) * 8)) * 2);
        typedef const __attribute__((address_space(3))) bf16x8* lds_bf16x8_t;
        auto k_frag = [&](int stage, int s) __attribute__((always_inline)) -> bf16x8 {
            return *(lds_bf16x8_t)(kfo[s] + (unsigned)(stage * (STAGE * 2)));
        };

        float m_run[2], l_run[2];
#pragma unroll
        for (int qi = 0; qi < 2; qi++) {
            m_run[qi] = -INFINITY;
            l_run[qi] = 0.f;
        }
        unsigned badm_cur = 0;
        if constexpr (MASKED) badm_cur = bmask[block_of(0)];

        // everything requested so far has to land: the Q pieces (this wave) and the first blocks (all waves)
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(0x0070);
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");

        f32x16 s_a[2], s_b[2];
#pragma unroll
        for (int qi = 0; qi < 2; qi++)
#pragma unroll
            for (int j = 0; j < 16; j++) s_a[qi][j] = 0.f;
        bf16x8 kf[8];
#pragma unroll
        for (int s = 0; s < 8; s++) {
            kf[s] = k_frag(0, s);
#pragma unroll
            for (int qi = 0; qi < 2; qi++) s_a[qi] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[s], qf[qi][s], s_a[qi], 0, 0, 0);
        }
        constexpr int LAK = 2; // K fragments read ahead of the MFMA pair that consumes them
#pragma unroll
        for (int s = 0; s < LAK; s++) kf[s] = k_frag(1 % NK, s);

        // One step: consumes S(b) in s_cur, produces S(b+1) in s_next and P(b) in the mailbox.
        auto s_step = [&](int b, f32x16 (&s_cur)[2], f32x16 (&s_next)[2]) __attribute__((always_inline)) {
            // byte offsets of the stages that hold K(b+1) and K(b+2) (wave-uniform)
            const unsigned ks1 = (unsigned)((b + 1) % NK) * (STAGE * 2u);
            const unsigned ks2 = (unsigned)((b + 2) % NK) * (STAGE * 2u);
            if constexpr (MASKED) {
                const unsigned badm = __builtin_amdgcn_readfirstlane(badm_cur);
                if (badm != 0u) {
#pragma unroll
                    for (int qi = 0; qi < 2; qi++)
#pragma unroll
                        for (int i = 0; i < 4; i++)
#pragma unroll
                            for (int j = 0; j < 4; j++) {
                                const int kk = 8 * i + 4 * h + j;
                                s_cur[qi][4 * i + j] = ((badm >> kk) & 1u) ? -INFINITY : s_cur[qi][4 * i + j];
                            }
                }
            }
#pragma unroll
            for (int qi = 0; qi < 2; qi++)
#pragma unroll
                for (int j = 0; j < 16; j++) s_next[qi][j] = 0.f;
            float mc[2], psum[2];
            unsigned pc[2][8] = {};
#pragma unroll
            for (int qi = 0; qi < 2; qi++) {
                mc[qi] = (!BOUNDED && m_run[qi] != -INFINITY) ? m_run[qi] : 0.f;
                psum[qi] = 0.f;
            }
            // The exponentials of a pair are issued one slot before their sum and packing: a wave
            // that is alone with the softmax on its SIMD would otherwise wait out the latency of the
            // transcendental unit in every slot (the single-role kernel's second wave hides it).
            auto exp_issue = [&](int qi, int p2) __attribute__((always_inline)) -> f32x2 {
                f32x16& sv = s_cur[qi];
                f32x2 pp;
                if constexpr (BOUNDED) {
                    pp[0] = __builtin_amdgcn_exp2f(sv[2 * p2]);
                    pp[1] = __builtin_amdgcn_exp2f(sv[2 * p2 + 1]);
                } else {
                    pp[0] = __builtin_amdgcn_exp2f(sv[2 * p2] - mc[qi]);
                    pp[1] = __builtin_amdgcn_exp2f(sv[2 * p2 + 1] - mc[qi]);
                }
                return pp;
            };
            auto exp_finish = [&](int qi, int p2, f32x2 pp) __attribute__((always_inline)) {
                psum[qi] += pp[0] + pp[1];
                pc[qi][p2] = __builtin_bit_cast(unsigned, __builtin_convertvector(pp, bf16x2));
                pin(psum[qi]);
                pin(pc[qi][p2]);
            };
            auto exp_pair = [&](int qi, int p2) __attribute__((always_inline)) { exp_finish(qi, p2, exp_issue(qi, p2)); };
            const unsigned slot = mail_lds + (unsigned)((b & 1) * PSLOT);
            auto post_p = [&](int qi) __attribute__((always_inline)) {
                *(lds_w128_t)(slot + (unsigned)(((qi * 2 + 0) * 64 + lane) * 16)) = u32x4{pc[qi][0], pc[qi][1], pc[qi][2], pc[qi][3]};
                *(lds_w128_t)(slot + (unsigned)(((qi * 2 + 1) * 64 + lane) * 16)) = u32x4{pc[qi][4], pc[qi][5], pc[qi][6], pc[qi][7]};
            };
            f32x2 pp_pend = {0.f, 0.f};
#pragma unroll
            for (int g = 0; g < 16; g++) {
                // K fragment LAK ahead: fragments 0 .. 7 of K(b+1), then the first of K(b+2)
                if ((g & 1) == 0) {
                    const int f = (g >> 1) + LAK;
                    if (f < 8) kf[f] = *(lds_bf16x8_t)(kfo[f] + ks1);
                }
                {
                    const int s = g >> 1, qi = g & 1;
                    s_next[qi] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[s], qf[qi][s], s_next[qi], 0, 0, 0);
                }
                if ((g & 1) == 1) {
                    // the fragment just consumed twice frees its registers for K(b+2)'s first ones
                    const int f = (g >> 1) + LAK - 8;
                    if (f >= 0) kf[f] = *(lds_bf16x8_t)(kfo[f] + ks2);
                }
                // The 16 exponential pairs of the step are issued in slots 0 .. 11 (four per three
                // slots) and each is finished one issue later, so that P is posted by slot 12 and its
                // LDS writes are done when the step ends; the MFMAs of the last slots cover them.
                {
                    constexpr int kPairsAt[17] = {0, 2, 3, 4, 6, 7, 8, 10, 11, 12, 14, 15, 16, 16, 16, 16, 16};
                    for (int e = kPairsAt[g]; e < kPairsAt[g + 1]; e++) {
                        const f32x2 pp_new = exp_issue(e >> 3, e & 7);
                        if (e > 0) exp_finish((e - 1) >> 3, (e - 1) & 7, pp_pend);
                        pp_pend = pp_new;
                        pin(pp_pend);
                        if constexpr (BOUNDED) {
                            if (e == 8) post_p(0);
                        }
                    }
                    if (g == 12) {
                        exp_finish(1, 7, pp_pend);
                        if constexpr (BOUNDED) post_p(1);
                    }
                }
                if constexpr (MASKED) {
                    if (g == 10) badm_cur = bmask[block_of(b + 1 < nblk ? b + 1 : nblk - 1)];
                }
                if (g == 1) fetch_k(b + AK);
                if (g == 3) fetch_v(b + AV);
                __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr (BOUNDED) {
#pragma unroll
                for (int qi = 0; qi < 2; qi++) {
                    l_run[qi] += psum[qi];
                    pin(l_run[qi]);
                }
            } else {
                // Lazy running maximum, watched by the row sums (see the single-role kernel): the
                // exponentials above were taken against the reference point as it stood; a sum above
                // 16 * 2^kTau, a row without a reference, or a sum that is not a number redoes the block.
                bool redo = false;
#pragma unroll
                for (int qi = 0; qi < 2; qi++) redo |= !(psum[qi] <= 16.0f * 256.0f) || m_run[qi] == -INFINITY;
                float alpha[2] = {1.f, 1.f};
                const bool any_redo = __any(redo);
                if (any_redo) {
#pragma unroll
                    for (int qi = 0; qi < 2; qi++) {
                        f32x16& sv = s_cur[qi];
                        float t0 = fmaxf(fmaxf(sv[0], sv[1]), sv[2]);
                        float t1 = fmaxf(fmaxf(sv[3], sv[4]), sv[5]);
                        float t2 = fmaxf(fmaxf(sv[6], sv[7]), sv[8]);
                        float t3 = fmaxf(fmaxf(sv[9], sv[10]), sv[11]);
                        float t4 = fmaxf(fmaxf(sv[12], sv[13]), sv[14]);
                        t0 = fmaxf(fmaxf(t0, t1), t2);
                        t3 = fmaxf(fmaxf(t3, t4), sv[15]);
                        const float mlc = pair_max(fmaxf(t0, t3));
                        const bool up = mlc > m_run[qi] + kTau;
                        const float m_new = up ? mlc : m_run[qi];
                        mc[qi] = (m_new == -INFINITY) ? 0.f : m_new;
                        alpha[qi] = __builtin_amdgcn_exp2f(m_run[qi] - mc[qi]);
                        m_run[qi] = m_new;
                        psum[qi] = 0.f;
#pragma unroll
                        for (int p2 = 0; p2 < 8; p2++) exp_pair(qi, p2);
                        l_run[qi] *= alpha[qi];
                        // the O-wave rescales its rows before it adds this step's product
                        *(lds_wf_t)(slot + 4096u + (unsigned)((qi * 64 + lane) * 4)) = alpha[qi];
                    }
                }
                post_p(0);
                post_p(1);
                if (lane == 0) *(lds_wu_t)(slot + 4096u + 512u) = any_redo ? 1u : 0u;
#pragma unroll
                for (int qi = 0; qi < 2; qi++) {
                    l_run[qi] += psum[qi];
                    pin(l_run[qi]);
                }
            }
            step_end(false);
        };

        int b = 0;
        for (; b + 1 < nblk; b += 2) {
            s_step(b, s_a, s_b);
            s_step(b + 1, s_b, s_a);
        }
        if (b < nblk) s_step(b, s_a, s_b);
        // step nblk: the O-wave consumes P(nblk-1); this wave posts the denominators (and the
        // reference points, for the parts of a key-split tile) in the free slot
        {
            const unsigned slot = mail_lds + (unsigned)((nblk & 1) * PSLOT);
#pragma unroll
            for (int qi = 0; qi < 2; qi++) {
                const float l_tot = pair_sum(l_run[qi]);
                *(lds_wf_t)(slot + (unsigned)(((qi * 2 + 0) * 64 + lane) * 4)) = l_tot;
                *(lds_wf_t)(slot + (unsigned)(((qi * 2 + 1) * 64 + lane) * 4)) = BOUNDED ? 0.f : m_run[qi];
            }
            fetch_k(nblk + AK); // keeps the load count of the step (a dead stage)
            fetch_v(nblk + AV);
            step_end(false);
            // step nblk + 1: the O-wave's last product
            fetch_k(nblk + 1 + AK);
            fetch_v(nblk + 1 + AV);
            step_end(true);
        }
        // the O-waves may turn their tiles through the V ring now: nothing of this wave is in flight
    } else {
        // =============================================================== O-wave
        f32x16 oacc[2][4]; // O^T: lane query 32 qi + l32, dims 32 blk + 8 i + 4 h + j
#pragma unroll
        for (int qi = 0; qi < 2; qi++)
#pragma unroll
            for (int blk = 0; blk < 4; blk++)
#pragma unroll
                for (int j = 0; j < 16; j++) oacc[qi][blk][j] = 0.f;
        unsigned vfo[4];
#pragma unroll
        for (int blk = 0; blk < 4; blk++)
            vfo[blk] = lds_address(Vs) + (unsigned)(((4 * h + tr_row) * D + ((blk ^ tr_row) * 32) + tr_col) * 2);
        typedef __attribute__((address_space(3))) s16x4* lds_s16x4_t;
        auto v_frag = [&](int stage, int kb, int blk, int half) __attribute__((always_inline)) -> s16x4 {
            return __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                (lds_s16x4_t)(vfo[blk] + (unsigned)(stage * (STAGE * 2) + (16 * kb + 8 * half) * (D * 2))));
        };

        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(0x0070);
        __builtin_amdgcn_s_barrier(); // the prologue barrier of the S-waves
        asm volatile("" ::: "memory");

        // What the S-wave posted for one step, as the O-wave holds it in registers.
        struct PSet {
            bf16x8 pf[2][2]; // P^T, B operands: [query half][key half]
            float alpha[2];  // the rows' rescale factors (running-maximum build), valid when flag != 0
            unsigned flag;
        };
        PSet set_a, set_b;
        s16x4 vlo[8], vhi[8]; // V fragments; the first LAV are read one step ahead
        constexpr int LAV = 2;
        // One step: O^T += V(b-2)^T P(b-2)^T with P(b-2) in `use`; P(b-1) is read into `load`, and the
        // first fragments of V(b-1) at the end, for the next step. Steps 0 and 1 have no product yet.
        auto o_step = [&](int b, PSet& use, PSet& load) __attribute__((always_inline)) {
            const bool have_next = b >= 1 && b - 1 < nblk; // wave-uniform
            if (have_next) {
                const unsigned slot = mail_lds + (unsigned)(((b - 1) & 1) * PSLOT);
#pragma unroll
                for (int qi = 0; qi < 2; qi++)
#pragma unroll
                    for (int kb = 0; kb < 2; kb++)
                        load.pf[qi][kb] = __builtin_bit_cast(bf16x8, *(lds_r128_t)(slot + (unsigned)(((qi * 2 + kb) * 64 + lane) * 16)));
                if constexpr (!BOUNDED) {
                    load.flag = *(lds_ru_t)(slot + 4096u + 512u);
#pragma unroll
                    for (int qi = 0; qi < 2; qi++) load.alpha[qi] = *(lds_rf_t)(slot + 4096u + (unsigned)((qi * 64 + lane) * 4));
                }
            }
            if (b >= 2) {
                const int vstage = (b - 2) & (NV - 1);
                if constexpr (!BOUNDED) {
                    if (__builtin_amdgcn_readfirstlane(use.flag) != 0u) {
#pragma unroll
                        for (int qi = 0; qi < 2; qi++)
#pragma unroll
                            for (int blk = 0; blk < 4; blk++)
#pragma unroll
                                for (int j = 0; j < 16; j++) oacc[qi][blk][j] *= use.alpha[qi];
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int g = 0; g < 16; g++) {
                    if ((g & 1) == 0) {
                        const int f = (g >> 1) + LAV;
                        if (f < 8) {
                            vlo[f] = v_frag(vstage, f >> 2, f & 3, 0);
                            vhi[f] = v_frag(vstage, f >> 2, f & 3, 1);
                        }
                    }
                    const int f = g >> 1, kb = f >> 2, blk = f & 3, qi = g & 1;
                    const bf16x8 vf = __builtin_bit_cast(bf16x8, (s16x8)__builtin_shufflevector(vlo[f], vhi[f], 0, 1, 2, 3, 4, 5, 6, 7));
                    oacc[qi][blk] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, use.pf[qi][kb], oacc[qi][blk], 0, 0, 0);
                    if (g == 1) fetch_k(b + AK);
                    if (g == 3) fetch_v(b + AV);
                    if (g == 11 && have_next) {
                        // V(b-1) was requested at step b - 1 - AV and is readable since the last barrier;
                        // fragments 0 .. LAV-1 were consumed in slots 0 .. 2 LAV - 1
                        const int vnext = (b - 1) & (NV - 1);
#pragma unroll
                        for (int f = 0; f < LAV; f++) {
                            vlo[f] = v_frag(vnext, f >> 2, f & 3, 0);
                            vhi[f] = v_frag(vnext, f >> 2, f & 3, 1);
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            } else {
                fetch_k(b + AK);
                fetch_v(b + AV);
            }
            if (have_next && b < 2) {
                // V(b-1) was requested at step b - 1 - AV and is readable since the last barrier
                const int vnext = (b - 1) & (NV - 1);
#pragma unroll
                for (int f = 0; f < LAV; f++) {
                    vlo[f] = v_frag(vnext, f >> 2, f & 3, 0);
                    vhi[f] = v_frag(vnext, f >> 2, f & 3, 1);
                }
            }
        };
        {
            const int last = nblk + 1; // steps 0 .. nblk + 1
            int b = 0;
            for (; b + 1 <= last; b += 2) {
                o_step(b, set_a, set_b);
                step_end(false);
                o_step(b + 1, set_b, set_a);
                step_end(b + 1 == last);
            }
            if (b <= last) {
                o_step(b, set_a, set_b);
                step_end(true);
            }
        }

        // ---- epilogue: O = O^T / l
        const unsigned fin = mail_lds + (unsigned)((nblk & 1) * PSLOT);
#pragma unroll
        for (int qi = 0; qi < 2; qi++) {
            const float l_tot = *(lds_rf_t)(fin + (unsigned)(((qi * 2 + 0) * 64 + lane) * 4));
            const float inv_l = l_tot > 0.f ? 1.0f / l_tot : 0.f;
            const int qrow = q0 + 32 * qi + l32;
            if (a.splits > 1) {
                const float m_fin = *(lds_rf_t)(fin + (unsigned)(((qi * 2 + 1) * 64 + lane) * 4));
                const int64_t prow = ((int64_t)blockIdx.x * BQ + pr_id * 64 + 32 * qi + l32);
                float* op = a.part_o + prow * D;
#pragma unroll
                for (int blk = 0; blk < 4; blk++)
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        f32x4 v;
#pragma unroll
                        for (int j = 0; j < 4; j++) v[j] = oacc[qi][blk][4 * i + j];
                        *reinterpret_cast<f32x4*>(op + 32 * blk + 8 * i + 4 * h) = v;
                    }
                if (h == 0) {
                    a.part_ml[prow * 2] = m_fin;
                    a.part_ml[prow * 2 + 1] = l_tot;
                }
            } else if (a.out_dtype == kF32) {
                if (qrow < a.tokens) {
                    float* op = reinterpret_cast<float*>(a.o) + (int64_t)seg * a.o_bs + (int64_t)qrow * a.o_ts + (int64_t)head * a.o_hs;
#pragma unroll
                    for (int blk = 0; blk < 4; blk++)
#pragma unroll
                        for (int i = 0; i < 4; i++) {
                            f32x4 v;
#pragma unroll
                            for (int j = 0; j < 4; j++) v[j] = oacc[qi][blk][4 * i + j] * inv_l;
                            *reinterpret_cast<f32x4*>(op + 32 * blk + 8 * i + 4 * h) = v;
                        }
                }
            } else {
                // 16-bit output: the wave turns each 32 x 128 half through 8 KB of the idle V ring
                // (K layout: chunk c of row r at c ^ (r & 15)) and stores whole 256-byte rows
                typedef __attribute__((address_space(3))) u32x2* lds_u32x2_t;
                typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
                const unsigned o_lds = lds_address(Vs) + (unsigned)((pr_id * 2 + qi) * (STAGE * 2));
                const bool half = a.out_dtype == kF16;
#pragma unroll
                for (int blk = 0; blk < 4; blk++)
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        f32x4 v;
#pragma unroll
                        for (int j = 0; j < 4; j++) v[j] = oacc[qi][blk][4 * i + j] * inv_l;
                        const u32x2 bits = half ? __builtin_bit_cast(u32x2, __builtin_convertvector(v, f16x4))
                                                : __builtin_bit_cast(u32x2, __builtin_convertvector(v, bf16x4));
                        *(lds_u32x2_t)(o_lds + (unsigned)(l32 * (D * 2) + (((4 * blk + i) ^ (l32 & 15)) * 16) + 8 * h)) = bits;
                    }
                unsigned short* const obase = reinterpret_cast<unsigned short*>(a.o) + (int64_t)seg * a.o_bs + (int64_t)head * a.o_hs;
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    const int r = 4 * j + (lane >> 4);
                    const u32x4 row16 = *(lds_r128_t)(o_lds + (unsigned)(r * (D * 2) + (lane & 15) * 16));
                    const int orow = q0 + 32 * qi + r;
                    if (orow < a.tokens)
                        *reinterpret_cast<u32x4*>(obase + (int64_t)orow * a.o_ts + (((lane & 15) ^ (r & 15)) * 8)) = row16;
                }
            }
        }
    }
    if (a.clock_probe && tid == 256 && (int64_t)blockIdx.x < a.clock_cap) { // an O-wave: the last to finish
        a.clock_probe[2 * blockIdx.x] = __builtin_readcyclecounter() - clk_c0;
        a.clock_probe[2 * blockIdx.x + 1] = __builtin_amdgcn_s_memrealtime() - clk_r0;
    }
}

} // namespace pairk
