// gfx950 flash-attention forward for zdraw's DiT joint self-attention.
//
// What it replaces in the reference: the Metal attention kernels behind
// zdraw_metal_run_attention* (metal/mattn_block_shader.zig:7-188, the steel
// route metal_api.m:6685-6815) and, when K is prepared in the tile load, the
// QK-norm + rope glue kernels that feed them (klein/zflux2_glue_shader.zig:61-122,
// metal/mqk_shader.zig:46-97). The design is MI355X-first, not a translation:
//
//   * one wave owns 32 query rows; the waves of a workgroup share every K/V block;
//   * scores are computed TRANSPOSED (S^T = K . Q^T) with v_mfma_f32_32x32x16_bf16,
//     so every lane owns one query column: softmax reductions are in-lane plus
//     one permlane32 swap, and the exponentiated block is already the B operand
//     of the second MFMA (O^T = V^T . P^T): no LDS round trip for P;
//   * K and V blocks sit in LDS row-major; the V^T operand is built by the
//     transposing LDS read ds_read_b64_tr_b16, so staging V is a plain copy;
//   * Q and K normally arrive prepared (norm, rope, softmax scale: one pre-pass
//     kernel per call) as bf16, and then query rows and K/V blocks go from global
//     memory straight into LDS (buffer_load ... lds) in a swizzled, unpadded
//     layout; otherwise RMSNorm + rope are applied to the Q rows in the prologue
//     and to the K rows between the global load and the LDS store of each block
//     (registers, padded rows);
//   * keys are walked in blocks of 32 through an LDS ring; inside one wave the
//     MFMAs of S(b+1) = K(b+1) Q^T and O += V(b-1)^T P(b-1) are interleaved, slot
//     by slot, with the softmax VALU work of block b (the three are independent);
//   * blocks are requested five steps ahead (descriptor + scalar block offset, no
//     per-step address arithmetic); LDS fragment reads run ahead across step
//     boundaries; the main loop takes a whole turn of the ring per trip, so every
//     LDS address in it is a register plus an immediate;
//   * 16-bit outputs are turned through LDS and stored as whole rows; the tiles of
//     a thinly filled last round of workgroups are split along the keys and merged
//     by a small kernel in a fixed order;
//   * block order and merge order are fixed and nothing is accumulated with
//     atomics, so the output is bit-identical from run to run.
#include "attn_device.hpp"

namespace zdraw {

namespace fwd {

// Schedule constants of the pipelined step (the measured best of what was tried).
constexpr int kLdsLookahead = 4;   // slots between an LDS fragment read and the MFMA that consumes it
constexpr int kLdsLookaheadDirect = 6; // the same for the direct-to-LDS build (8 is 0.3 % better still where it does not spill)
constexpr int kReadBatch = 2;      // slots whose fragment reads are issued together (one wait per batch)
constexpr int kMfmaPrio = 1;       // wave priority while an MFMA is issued, builds that stage blocks through registers (0 = leave it alone)
constexpr int kMfmaPrioDirect = 0; // the same for the direct-to-LDS build
constexpr bool kDirectLds = true;  // prepared bf16 K/V blocks go from global memory straight into LDS
constexpr int kStoreSlot = 1;      // slot after which a step moves its staged block into the ring

constexpr int KB = 32;            // keys per block
constexpr int KPITCH = D + 8;     // 272 B rows: 16-lane b128 reads spread over all banks
constexpr int VPITCH = D + 32;    // 320 B rows: a 32-lane transposing read covers 4 rows x 64 B without overlap
constexpr int KS_ELEMS = KB * KPITCH;
constexpr int VS_ELEMS = KB * VPITCH;
constexpr int MAX_BLOCKS = 1024;  // key-block list capacity (tokens <= 32768)
constexpr float kTau = 8.0f;             // log2 headroom of the lazy softmax maximum

// Ring depth: 8 stages when one workgroup owns the CU (blocks are stored four
// steps ahead of their first use, so one barrier per two steps orders every
// write against its readers, including the reads a step issues for the next
// one), 4 stages when two workgroups share the CU's LDS (stored two steps
// ahead, one barrier per step).
constexpr int ring_stages(int qb, int nw) { return (qb == 2 || nw == 8) ? 8 : 4; }
constexpr size_t kListBytes = (size_t)MAX_BLOCKS * (sizeof(unsigned short) + sizeof(unsigned));
constexpr size_t lds_bytes(int nst) {
    // ring + key-block list (u16) + per-block exclusion masks (u32); the 8-stage build also
    // needs 24 KB behind the lists of its unpadded (direct-to-LDS) layout, where three waves
    // park their query rows (the padded layout's ring is the larger one, short by 4 KB)
    const size_t padded = (size_t)nst * (KS_ELEMS + VS_ELEMS) * sizeof(bf16_t) + kListBytes;
    const size_t direct = (size_t)nst * 2 * (KB * D) * sizeof(bf16_t) + kListBytes + 3 * (size_t)(KB * D) * sizeof(bf16_t);
    return nst == 8 && direct > padded ? direct : padded;
}

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

// Keeps a value's producer on this side of the point where it is called: the
// empty volatile asm "uses and redefines" the register, so the optimiser can
// neither sink the computation past it (into a later block) nor reorder it
// with the scheduling fences, which are ordered with volatile asm.
template <typename T>
__device__ __forceinline__ void pin(T& v) {
    asm volatile("" : "+v"(v));
}

// The transposing LDS read ds_read_b64_tr_b16 (used for V below): within each 16-lane
// group the hardware returns to lane i, element j, the value at (row of source lane
// (i>>2)+4j, column i&3 of that lane's 4-element chunk); a lane's address must point at
// row (lane&15)>>2, chunk lane&3 of the 4 x 16 patch.

// QB = 32-query blocks per wave, NW = waves per workgroup. Built shapes:
//   QB=1, NW=8: two waves per SIMD, 256 registers each (default);
//   QB=1, NW=4: two workgroups per CU, each with its own LDS ring.
// (QB=2, NW=4, one 64-query wave per SIMD, halves the LDS reads per MFMA but
// measured 8 % slower: one wave per SIMD cannot hide its own waits.)
//
// BOUNDED: the caller has promised that every scaled score fits comfortably in
// the fp32 exponent (QK-normalised operands: |q'.k'|/sqrt(D) <= sqrt(D) max|w_q| max|w_k|).
// Softmax is shift-invariant, so the kernel then exponentiates the scores as
// they are: no running maximum, no subtraction, no rescale of O. Otherwise a
// lazy running maximum is kept: S accumulates on top of minus the reference point
// (the MFMA's C operand), so the exponentials need no subtraction either, and the
// block's row sums, not a maximum per block, say when the reference must move.
//
// SF16: the prepared Q and K are IEEE half instead of bf16 (the staging type of the reference's
// own kernels, klein/zflux2_glue_shader.zig:95-122) and S = K Q^T runs on
// v_mfma_f32_32x32x16_f16: three more mantissa bits on every score at the same MFMA rate. P and
// V stay bf16 (P reaches 2^64 in the bounded form). Only for the direct-to-LDS build, where the
// operands' bits go from memory to the MFMA untouched.
template <typename TIn, int KMODE, bool MASKED, bool BOUNDED, int QB, int NW, bool SF16 = false>
__global__ void __launch_bounds__(NW * 64, (QB == 2 ? 1 : 2)) attn_fwd_kernel(const AttnArgs a) {
    constexpr int NT = NW * 64;
    constexpr int QR = 32 * QB;       // query rows per wave
    constexpr int BQ = NW * QR;       // query rows per workgroup
    constexpr int CPT = 512 / NT;     // 8-element chunks of K (and of V) per thread per block
    constexpr int TPK = 16 / CPT;     // threads sharing one key row
    constexpr int NST = ring_stages(QB, NW);
    constexpr bool XSTEP = NST == 8;          // fragment reads run ahead across step boundaries
    // Prepared bf16 operands (K pre-pass mode) skip the registers: each wave moves four K rows and four V rows of a block from global
    // memory straight into the ring (buffer_load ... lds). Such a load puts lane i's
    // 16 bytes at base + 16 i, so rows are 256 bytes without padding and bank
    // conflicts are avoided by swizzling the 16-byte chunk position instead:
    // K chunk c of row r sits at c ^ (r & 15), V chunk c of row r at c ^ ((r & 3) << 2).
    constexpr bool DMA = kDirectLds && std::is_same<TIn, bf16_t>::value && KMODE == kQkNone && NW == 8 && QB == 1;
    static_assert(!SF16 || DMA, "half-precision score operands exist for the direct-to-LDS build only");
    // The product O^T += V^T P^T on v_mfma_f32_16x16x32 (the scores keep the 32 x 32 x 16 form, in
    // which a lane owns one query). The 16 x 16 form moves half the accumulator bytes per FLOP
    // through the register file, and at the board's power limit that is worth clock: -2 % of the
    // kernel's time. It costs a few registers (the compiler writes these MFMAs' results to other
    // registers than their inputs) and four lane exchanges per block, so only the builds with
    // room take it: prepared operands, and not the running maximum together with a mask (that
    // build then spills inside the loop). (Giving the scores that form too would double the MFMA
    // instructions on a vector issue port that the softmax already half fills.)
    constexpr bool PV16 = DMA && (BOUNDED || !MASKED);
    constexpr int KSTAGE = DMA ? KB * D : KS_ELEMS; // elements per ring stage
    constexpr int VSTAGE = DMA ? KB * D : VS_ELEMS;
    // a block enters the ring AHEAD steps before S needs its K (direct loads: one more step, to land)
    constexpr int AHEAD = NST == 8 ? (DMA ? 5 : 4) : 2;
    constexpr int LA = DMA ? kLdsLookaheadDirect : kLdsLookahead; // slots between an LDS fragment read and its MFMA
    constexpr int RB = kReadBatch;      // slots whose reads are issued together (divides 16 and LA)
    // Wave priority while an MFMA is being issued. The register-staged builds gain from it (the
    // masked one loses 13 % without). The direct-to-LDS build runs 5 % fewer cycles per
    // workgroup without the two s_setprio per MFMA; the chip sits on its power limit, so the
    // clock gives part of that back and 2 % is left.
    constexpr int MFMA_PRIO = DMA ? kMfmaPrioDirect : kMfmaPrio;
    constexpr int STORE_SLOT = kStoreSlot; // slot after which the ring store is issued
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    bf16_t* const Ks = reinterpret_cast<bf16_t*>(smem);
    bf16_t* const Vs = Ks + NST * KSTAGE;
    unsigned short* const blocks = reinterpret_cast<unsigned short*>(Vs + NST * VSTAGE);
    unsigned* const bmask = reinterpret_cast<unsigned*>(blocks + MAX_BLOCKS); // bit j: key j of the block is excluded
    __shared__ int s_nblocks;

    unsigned long long clk_c0 = 0, clk_r0 = 0;
    if (a.clock_probe) {
        clk_c0 = __builtin_readcyclecounter();
        clk_r0 = __builtin_amdgcn_s_memrealtime();
    }
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int l32 = lane & 31;
    const int h = lane >> 5;

    // XCD-aware remap: consecutive logical ids (one head's query blocks) share an XCD's L2
    int logical;
    int split = 0;
    int splits = 1; // parts of this workgroup's tile
    if ((int)blockIdx.x < a.part_wgs) {
        // key-split tail: consecutive ids are the parts of one tile
        const int t = (int)blockIdx.x / a.splits;
        if (t >= a.nqb * a.heads * a.batch - a.tile_base) return; // padding up to a multiple of 8
        split = (int)blockIdx.x - t * a.splits;
        splits = a.splits;
        logical = a.tile_base + t;
    } else {
        // (part_wgs is a multiple of 8, so a workgroup's XCD is its id's low bits here too)
        const int w = (int)blockIdx.x - a.part_wgs;
        const int nwg = (int)gridDim.x - a.part_wgs;
        const int xcd = w & 7;
        const int idx = w >> 3;
        const int base = nwg >> 3;
        const int rem = nwg & 7;
        logical = idx + xcd * base + (xcd < rem ? xcd : rem);
    }
    const int bh = logical / a.nqb;
    const int qb = logical - bh * a.nqb;
    const int seg = bh / a.heads;
    const int head = bh - seg * a.heads;
    const int q0 = qb * BQ + wave * QR;

    // The pipeline's first O update multiplies P = 0 by the V stage of "block -1":
    // that stage must hold finite numbers, so it is zeroed. (The last S update
    // reads a K stage past the end; its result is discarded.)
    {
        u32x4* z = reinterpret_cast<u32x4*>(Vs + (NST - 1) * VSTAGE);
        constexpr int n16 = (int)(VSTAGE * sizeof(bf16_t) / 16);
        for (int i = tid; i < n16; i += NT) z[i] = u32x4{0u, 0u, 0u, 0u};
    }

    // ---- key-block list: blocks with at least one admitted key, ascending
    const int nb_all = (a.key_limit + KB - 1) / KB;
    const unsigned char* const kp = a.key_pad ? a.key_pad + (int64_t)seg * a.mask_bs : nullptr;
    int nblk = nb_all;
    if constexpr (MASKED) {
        // exclusion mask of every key block (padding mask, key limit, tail), two blocks per wave pass
        for (int t2 = wave; 2 * t2 < nb_all; t2 += NW) {
            const int key = t2 * 64 + lane;
            const bool bad = key >= a.key_limit || (kp != nullptr && kp[key < a.key_limit ? key : 0] != 0);
            const unsigned long long m = __ballot(bad);
            if (lane == 0) {
                bmask[2 * t2] = (unsigned)m;
                if (2 * t2 + 1 < MAX_BLOCKS) bmask[2 * t2 + 1] = (unsigned)(m >> 32);
            }
        }
        __syncthreads();
        if (kp) { // compact the blocks that admit at least one key
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
    // a key-split workgroup walks positions [i0, i0 + nblk) of the list
    int i0 = 0;
    if (splits > 1) {
        const int per = (nblk + splits - 1) / splits;
        i0 = split * per;
        nblk = max(min(nblk - i0, per), 0);
    }
    // wave-uniform by construction; readfirstlane lets the compiler keep it in scalar registers
    auto block_of = [&](int i) -> int { return (MASKED && kp) ? __builtin_amdgcn_readfirstlane((int)blocks[i + i0]) : i + i0; };

    // ---- Q rows -> B-operand registers: qf[qi][s], lane: query 32*qi + l32, dims 16s + 8h .. +7
    // The workgroup's query rows are prepared in the layout that coalesces: 16 lanes per
    // row (8 dims each, a row's 256 bytes and its rope row are contiguous), NT / 16 rows per
    // pass. Norm, rope and the softmax scale are applied there and the bf16 rows are parked
    // in LDS (the ring is not in use yet; 272-byte pitch, conflict-free b128 reads), from
    // where every lane then picks up the fragments of ITS query row. A lane fetching its
    // own row from memory would touch one cache line per lane and instruction.
    // log2(e)/sqrt(D) rides on Q, so the MFMA delivers scores in the exp2 domain.
    bf16x8 qf[QB][8];
    if constexpr (!DMA) {
        constexpr int QPITCH = D + 8;
        constexpr int RPP = NT / 16;      // rows per pass
        constexpr int PASSES = BQ / RPP;  // 8 QB
        constexpr int BATCH = 4;          // passes whose loads are in flight together
        bf16_t* const Qs = Ks;            // BQ x QPITCH elements at the start of the (idle) ring
        const int prr = tid >> 4;
        const int pd0 = (tid & 15) * 8;
        const TIn* const qbase = reinterpret_cast<const TIn*>(a.q) + (int64_t)seg * a.q_bs + (int64_t)head * a.q_hs + pd0;
#pragma unroll
        for (int p0 = 0; p0 < PASSES; p0 += BATCH) {
            Raw8<TIn> raw[BATCH];
            QkRow rows[BATCH];
            Rope8 rope[BATCH];
            f32x4 w0[BATCH], w1[BATCH];
#pragma unroll
            for (int j = 0; j < BATCH; j++) {
                // rows past the sequence work on the last row (their output is never stored)
                const int qrow_raw = qb * BQ + (p0 + j) * RPP + prr;
                const int qrow = qrow_raw < a.tokens ? qrow_raw : a.tokens - 1;
                raw[j] = ld_raw8<TIn>(qbase + (int64_t)qrow * a.q_ts, true);
                if (a.q_mode != kQkNone) {
                    rows[j] = qk_row(a.qk, a.q_mode, a.q_w, a.q_w_txt, seg, qrow, true);
                    rope[j] = ld_rope8(a.qk, a.q_mode, rows[j], pd0);
                    w0[j] = *reinterpret_cast<const f32x4*>(rows[j].w + pd0);
                    w1[j] = *reinterpret_cast<const f32x4*>(rows[j].w + pd0 + 4);
                }
            }
#pragma unroll
            for (int j = 0; j < BATCH; j++) {
                float x[8];
                unpack8(raw[j], x);
                if (a.q_mode != kQkNone) {
                    float ss = 0.f;
#pragma unroll
                    for (int i = 0; i < 8; i++) ss += x[i] * x[i];
                    ss = row_group_sum<16>(ss);
                    const float inv = rsqrtf(ss * (1.0f / D) + a.qk.eps);
                    qk_apply8(a.q_mode, x, inv, w0[j], w1[j], rope[j]);
                }
#pragma unroll
                for (int i = 0; i < 8; i++) x[i] *= a.scale_log2;
                *reinterpret_cast<u32x4*>(Qs + ((p0 + j) * RPP + prr) * QPITCH + pd0) = pack_bf16x8(x);
            }
        }
        __syncthreads();
#pragma unroll
        for (int qi = 0; qi < QB; qi++)
#pragma unroll
            for (int s = 0; s < 8; s++)
                qf[qi][s] = *reinterpret_cast<const bf16x8*>(Qs + (wave * QR + 32 * qi + l32) * QPITCH + 16 * s + 8 * h);
        __syncthreads(); // the ring may be filled from here on
    }
    // (The direct-to-LDS build fetches its query rows together with the first K/V blocks, below.)

    // ---- block staging: thread t owns key t/TPK of the block, CPT chunks of 8 dims of K and of V
    const int lk_key = tid / TPK;
    const int lk_d0 = (tid % TPK) * CPT * 8;
    // Addresses are a wave-uniform buffer descriptor (segment, head) + a uniform
    // byte offset (key block) + a 32-bit per-thread byte offset that never
    // changes (row within the block, column): the loop spends no vector ALU
    // work on them. The host checks that a head's rows span less than 4 GiB.
    const unsigned k_span = ((unsigned)(a.tokens - 1) * (unsigned)a.k_ts + D) * (unsigned)sizeof(TIn);
    const unsigned v_span = ((unsigned)(a.tokens - 1) * (unsigned)a.v_ts + D) * (unsigned)sizeof(TIn);
    const rsrc_t k_rsrc = make_rsrc(reinterpret_cast<const TIn*>(a.k) + (int64_t)seg * a.k_bs + (int64_t)head * a.k_hs, k_span);
    const rsrc_t v_rsrc = make_rsrc(reinterpret_cast<const TIn*>(a.v) + (int64_t)seg * a.v_bs + (int64_t)head * a.v_hs, v_span);
    const unsigned k_blk_bytes = (unsigned)a.k_ts * (unsigned)(KB * sizeof(TIn));
    const unsigned v_blk_bytes = (unsigned)a.v_ts * (unsigned)(KB * sizeof(TIn));
    const unsigned k_off = ((unsigned)lk_key * (unsigned)a.k_ts + (unsigned)lk_d0) * (unsigned)sizeof(TIn);
    const unsigned v_off = ((unsigned)lk_key * (unsigned)a.v_ts + (unsigned)lk_d0) * (unsigned)sizeof(TIn);
    // the block that holds the last row: its rows past the sequence re-read the last row
    const int last_row = a.tokens - 1;
    const int last_blk = last_row / KB;
    const int lk_tail = min(lk_key, last_row - last_blk * KB);
    const unsigned k_off_tail = ((unsigned)lk_tail * (unsigned)a.k_ts + (unsigned)lk_d0) * (unsigned)sizeof(TIn);
    const unsigned v_off_tail = ((unsigned)lk_tail * (unsigned)a.v_ts + (unsigned)lk_d0) * (unsigned)sizeof(TIn);

    // Two register sets alternate: a block's global loads are issued two steps
    // before the step that moves it into LDS, so a full step of work always
    // separates a load from its first use.
    struct StageRegs {
        Raw8<TIn> kraw[CPT], vraw[CPT];
        Rope8 krope[KMODE == kQkNone ? 1 : CPT];
        QkRow krow;
    };
    StageRegs sets[2];

    // i = position in the block list. Loads are unconditional (no branches in
    // the pipelined loop): positions past the end re-read the last block.
    // Neither those nor the rows past the sequence are ever used: the drained
    // ring stages feed only discarded MFMAs, and keys past the limit are
    // masked to -inf before the softmax. (The unmasked build only runs when
    // every block is full, so it needs no tail offsets.)
    auto stage_load = [&](StageRegs& r, int i) __attribute__((always_inline)) {
        const int ii = i < nblk ? i : nblk - 1;
        const int blk = block_of(ii);
        unsigned ko = k_off, vo = v_off;
        if constexpr (MASKED) {
            const bool tail = blk >= last_blk; // wave-uniform
            ko = tail ? k_off_tail : k_off;
            vo = tail ? v_off_tail : v_off;
        }
        const unsigned kb = (unsigned)blk * k_blk_bytes, vb = (unsigned)blk * v_blk_bytes;
#pragma unroll
        for (int c = 0; c < CPT; c++) {
            r.kraw[c] = ld_raw8_buf<TIn>(k_rsrc, ko + (unsigned)(8 * c * sizeof(TIn)), kb);
            r.vraw[c] = ld_raw8_buf<TIn>(v_rsrc, vo + (unsigned)(8 * c * sizeof(TIn)), vb);
        }
        if constexpr (KMODE != kQkNone) {
            int key = blk * KB + lk_key;
            key = key < last_row ? key : last_row;
            r.krow = qk_row(a.qk, KMODE, a.k_w, a.k_w_txt, seg, key, true);
#pragma unroll
            for (int c = 0; c < CPT; c++) r.krope[c] = ld_rope8(a.qk, KMODE, r.krow, lk_d0 + 8 * c);
        }
    };

    auto stage_store = [&](StageRegs& r, int stage) __attribute__((always_inline)) {
        bf16_t* kdst = Ks + stage * KS_ELEMS + lk_key * KPITCH + lk_d0;
        bf16_t* vdst = Vs + stage * VS_ELEMS + lk_key * VPITCH + lk_d0;
        if constexpr (KMODE == kQkNone) {
#pragma unroll
            for (int c = 0; c < CPT; c++) *reinterpret_cast<u32x4*>(kdst + 8 * c) = raw_to_bf16(r.kraw[c]);
        } else {
            float x[CPT][8];
            float ss = 0.f;
#pragma unroll
            for (int c = 0; c < CPT; c++) {
                unpack8(r.kraw[c], x[c]);
#pragma unroll
                for (int i = 0; i < 8; i++) ss += x[c][i] * x[c][i];
            }
            ss = row_group_sum<TPK>(ss);
            const float inv = rsqrtf(ss * (1.0f / D) + a.qk.eps);
#pragma unroll
            for (int c = 0; c < CPT; c++) {
                qk_apply8(KMODE, x[c], inv, r.krow.w, lk_d0 + 8 * c, r.krope[c]);
                *reinterpret_cast<u32x4*>(kdst + 8 * c) = pack_bf16x8(x[c]);
            }
        }
#pragma unroll
        for (int c = 0; c < CPT; c++) *reinterpret_cast<u32x4*>(vdst + 8 * c) = raw_to_bf16(r.vraw[c]);
    };

    // Direct path: wave w moves rows 4 w + lane / 16 of block position i into ring stage
    // i % NST; the lane that fills chunk position p of row r fetches the chunk that the
    // swizzle places there. In the block that holds the last row, rows past the sequence
    // re-read the last row (they are masked before the softmax).
    const int dma_row = 4 * wave + (lane >> 4);
    const unsigned dma_k_chunk = (unsigned)(((lane & 15) ^ (dma_row & 15)) * 8);
    // (PV16: a row's 16-dim halves also swap with bit 4 of the row, so that the lane groups that
    // read rows 16 apart hit different banks)
    const unsigned dma_v_chunk = (unsigned)(((lane & 15) ^ ((dma_row & 3) << 2) ^ (PV16 ? (((dma_row >> 4) & 1) << 1) : 0)) * 8);
    const unsigned dma_k_off = ((unsigned)dma_row * (unsigned)a.k_ts + dma_k_chunk) * 2u;
    const unsigned dma_v_off = ((unsigned)dma_row * (unsigned)a.v_ts + dma_v_chunk) * 2u;
    const int dma_tail_row = min(dma_row, last_row - last_blk * KB);
    const unsigned dma_k_off_tail = ((unsigned)dma_tail_row * (unsigned)a.k_ts + dma_k_chunk) * 2u;
    const unsigned dma_v_off_tail = ((unsigned)dma_tail_row * (unsigned)a.v_ts + dma_v_chunk) * 2u;
    const u32x4 dma_k_rsrc = make_rsrc_words(reinterpret_cast<const TIn*>(a.k) + (int64_t)seg * a.k_bs + (int64_t)head * a.k_hs, k_span);
    const u32x4 dma_v_rsrc = make_rsrc_words(reinterpret_cast<const TIn*>(a.v) + (int64_t)seg * a.v_bs + (int64_t)head * a.v_hs, v_span);
    // LDS byte addresses of this wave's four rows in stage 0 of the K ring and of the V ring
    const unsigned dma_k_lds = __builtin_amdgcn_readfirstlane(lds_address(Ks) + (unsigned)(4 * wave * D * 2));
    const unsigned dma_v_lds = __builtin_amdgcn_readfirstlane(lds_address(Vs) + (unsigned)(4 * wave * D * 2));
    // which: 1 = the K block, 2 = the V block, 3 = both
    auto dma_fetch_part = [&](int i, int stage, int which) __attribute__((always_inline)) {
        const int ii = i < nblk ? i : nblk - 1; // past the end: a harmless re-fetch into a dead stage
        const int blk = block_of(ii);
        unsigned ko = dma_k_off, vo = dma_v_off;
        if constexpr (MASKED) {
            const bool tail = blk >= last_blk; // wave-uniform
            ko = tail ? dma_k_off_tail : dma_k_off;
            vo = tail ? dma_v_off_tail : dma_v_off;
        }
        if (which & 1) load_to_lds_16(dma_k_rsrc, dma_k_lds + (unsigned)stage * (KSTAGE * 2u), ko, (unsigned)blk * k_blk_bytes);
        if (which & 2) load_to_lds_16(dma_v_rsrc, dma_v_lds + (unsigned)stage * (VSTAGE * 2u), vo, (unsigned)blk * v_blk_bytes);
    };
    auto dma_fetch = [&](int i, int stage) __attribute__((always_inline)) { dma_fetch_part(i, stage, 3); };

    // ---- running state
    f32x16 oacc[QB][4]; // O^T: lane query 32*qi + l32, dims 32*blk + 8i + 4h + j
#pragma unroll
    for (int qi = 0; qi < QB; qi++)
#pragma unroll
        for (int blk = 0; blk < 4; blk++)
#pragma unroll
            for (int j = 0; j < 16; j++) oacc[qi][blk][j] = 0.f;
    // PV16: O^T as 8 x 2 tiles of 16 x 16: with c16 = lane % 16 and g4 = lane / 16 the lane holds query
    // 16 r + c16, dims 16 dt + 4 g4 + j of tile oacc16[dt][r] (and oacc above stays unused)
    static_assert(!PV16 || QB == 1, "the 16 x 16 product is written for one 32-query block per wave");
    const int c16 = lane & 15;
    const int g4 = lane >> 4;
    f32x4 oacc16[8][2];
#pragma unroll
    for (int dt = 0; dt < 8; dt++)
#pragma unroll
        for (int r = 0; r < 2; r++) oacc16[dt][r] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m_run[QB], l_run[QB]; // running maximum (already multiplied by scale_log2) and denominator half
#pragma unroll
    for (int qi = 0; qi < QB; qi++) {
        m_run[qi] = -INFINITY;
        l_run[qi] = 0.f;
    }
    // Running-maximum build: minus the reference point of each query column, in the shape of an
    // MFMA accumulator. The first MFMA of a block's S takes it as its C operand, so scores arrive
    // relative to the reference and the exponentials need no subtraction.
    // (Only the builds with registers to spare: prepared 16-bit operands. The others subtract.)
    constexpr bool REFACC = !BOUNDED && KMODE == kQkNone && std::is_same<TIn, bf16_t>::value && NW == 8 && QB == 1;
    float negm[QB]; // (one value per lane: every element of the accumulator starts from it)
#pragma unroll
    for (int qi = 0; qi < QB; qi++) negm[qi] = 0.f;

    // LDS byte addresses of this lane's fragments in ring stage 0; a stage, a key half (kb)
    // and a row half add constants. K: key row l32, dims 16 s + 8 h .. +7 (8 addresses, the
    // swizzle makes them differ by more than a constant). V: the 4 x 16 patch of the
    // transposing read, row 16 kb + 8 half + 4 h + tr_row, one address per output block.
    const int tr_row = (lane & 15) >> 2;
    const int tr_col = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
    constexpr int KROW = DMA ? D : KPITCH, VROW = DMA ? D : VPITCH; // elements per LDS row
    unsigned kfo[8], vfo[4];
#pragma unroll
    for (int s = 0; s < 8; s++) {
        const int col = DMA ? (((2 * s + h) ^ (l32 & 15)) * 8) : (8 * h + 16 * s);
        kfo[s] = lds_address(Ks) + (unsigned)((l32 * KROW + col) * 2);
    }
#pragma unroll
    for (int blk = 0; blk < 4; blk++) {
        const int col = (DMA ? ((blk ^ tr_row) * 32) : (32 * blk)) + tr_col; // (4 h + tr_row) & 3 == tr_row
        vfo[blk] = lds_address(Vs) + (unsigned)(((4 * h + tr_row) * VROW + col) * 2);
    }
    // PV16: the patch for output tile dt = 2 blk + x: the 16 lanes of group g4 take keys vkey0 + 8
    // half + tr_row (vkey0 = 0, 16, 4, 20: the keys whose probabilities the group holds as the
    // product's B operand, see the exchange in valu_slice), dims 16 dt .. + 15
    const int vkey0 = 16 * (g4 & 1) + 4 * (g4 >> 1);
    unsigned vfo16[4][2];
#pragma unroll
    for (int blk = 0; blk < 4; blk++)
#pragma unroll
        for (int x = 0; x < 2; x++) {
            const int col = (blk ^ tr_row) * 32 + (x ^ (g4 & 1)) * 16 + 4 * (lane & 3); // (vkey0 + tr_row) & 3 == tr_row
            vfo16[blk][x] = lds_address(Vs) + (unsigned)(((vkey0 + tr_row) * VROW + col) * 2);
        }
    typedef const __attribute__((address_space(3))) bf16x8* lds_bf16x8_t;
    typedef __attribute__((address_space(3))) s16x4* lds_s16x4_t;
    auto k_frag = [&](int stage, int s) __attribute__((always_inline)) -> bf16x8 {
        return *(lds_bf16x8_t)(kfo[s] + (unsigned)(stage * (KSTAGE * 2)));
    };
    auto v_frag = [&](int stage, int kb, int blk, int half) __attribute__((always_inline)) -> s16x4 {
        return __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (lds_s16x4_t)(vfo[blk] + (unsigned)(stage * (VSTAGE * 2) + (16 * kb + 8 * half) * (VROW * 2))));
    };

    auto v_frag16 = [&](int stage, int dt, int half) __attribute__((always_inline)) -> s16x4 {
        return __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (lds_s16x4_t)(vfo16[dt >> 1][dt & 1] + (unsigned)(stage * (VSTAGE * 2) + (8 * half) * (VROW * 2))));
    };

    // one 32 x 32 x 16 step of S^T += K Q^T on the operands' element type
    auto score_mfma = [&](const bf16x8& kfrag, const bf16x8& qfrag, const f32x16& c) __attribute__((always_inline)) -> f32x16 {
        if constexpr (SF16)
            return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, kfrag), __builtin_bit_cast(f16x8, qfrag), c, 0, 0, 0);
        else
            return __builtin_amdgcn_mfma_f32_32x32x16_bf16(kfrag, qfrag, c, 0, 0, 0);
    };

    // S^T block = K(block) . Q^T for both query blocks
    auto qk_block = [&](int stage, f32x16 (&s_out)[QB]) {
#pragma unroll
        for (int qi = 0; qi < QB; qi++)
#pragma unroll
            for (int j = 0; j < 16; j++) s_out[qi][j] = 0.f;
#pragma unroll
        for (int s = 0; s < 8; s++) {
            const bf16x8 kf = k_frag(stage, s);
#pragma unroll
            for (int qi = 0; qi < QB; qi++)
                s_out[qi] = score_mfma(kf, qf[qi][s], s_out[qi]);
        }
    };

    // O^T += V(block)^T . P^T
    auto pv_block = [&](int stage, const bf16x8 (&p)[QB][2]) {
        if constexpr (PV16) { // p[0][r] is the B operand of query tile r
#pragma unroll
            for (int dt = 0; dt < 8; dt++) {
                const s16x4 lo = v_frag16(stage, dt, 0);
                const s16x4 hi = v_frag16(stage, dt, 1);
                typedef short s16x8 __attribute__((ext_vector_type(8)));
                const bf16x8 vf = __builtin_bit_cast(bf16x8, (s16x8)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
#pragma unroll
                for (int r = 0; r < 2; r++)
                    oacc16[dt][r] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, p[0][r], oacc16[dt][r], 0, 0, 0);
            }
            return;
        }
#pragma unroll
        for (int kb = 0; kb < 2; kb++) {
#pragma unroll
            for (int blk = 0; blk < 4; blk++) {
                const s16x4 lo = v_frag(stage, kb, blk, 0);
                const s16x4 hi = v_frag(stage, kb, blk, 1);
                typedef short s16x8 __attribute__((ext_vector_type(8)));
                const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                const bf16x8 vf = __builtin_bit_cast(bf16x8, both);
#pragma unroll
                for (int qi = 0; qi < QB; qi++)
                    oacc[qi][blk] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, p[qi][kb], oacc[qi][blk], 0, 0, 0);
            }
        }
    };

    // Fragment registers of the software pipeline; they live across steps because the
    // first reads of a step are issued at the end of the step before it.
    typedef short s16x8 __attribute__((ext_vector_type(8)));
    bf16x8 kf[8];
    s16x4 vlo[8], vhi[8];
    // LDS fragment read for slot `slot` of step `bb`: even slots read K(bb+1) dims
    // 16*(slot/2).., odd slots read the V(bb-1) patch for output block (slot/2)%4, keys 16*(slot/8)..
    // (k_stage holds K(bb+1), v_stage holds V(bb-1))
    auto frag_read = [&](int k_stage, int v_stage, int slot) __attribute__((always_inline)) {
        if (slot & 1) {
            const int idx = slot >> 1, kb = idx >> 2, blk = idx & 3;
            if constexpr (PV16) { // the two patches of output tile idx
                vlo[idx] = v_frag16(v_stage, idx, 0);
                vhi[idx] = v_frag16(v_stage, idx, 1);
            } else {
                vlo[idx] = v_frag(v_stage, kb, blk, 0);
                vhi[idx] = v_frag(v_stage, kb, blk, 1);
            }
        } else {
            kf[slot >> 1] = k_frag(k_stage, slot >> 1);
        }
    };

    unsigned badm_cur = 0; // exclusion mask of the block whose scores the next step exponentiates
    if constexpr (MASKED) {
        if (nblk > 0) badm_cur = bmask[block_of(0)];
    }

    // One pipeline step for list position b: consumes S(b) and P(b-1),
    // produces S(b+1) and P(b). The three streams are independent, so the
    // step is laid out by hand as 16 slots, each fenced from the next:
    //   LDS reads for the MFMA LA slots ahead | one MFMA per query block |
    //   one slice of the softmax VALU work, which runs in the MFMA's shadow.
    // Even slots extend S(b+1) = K(b+1) Q^T, odd slots add V(b-1)^T P(b-1)^T to O^T.
    // With the 8-stage ring the reads for the first LA slots of step b+1 are
    // issued in the last LA slots of step b, so no step starts by waiting on LDS.
    // `phase` is b modulo the ring depth as a compile-time constant (every LDS address of
    // the step is then a register plus an immediate), or -1 when only b itself is known.
    auto step = [&](auto phase, int b, StageRegs& regs, bool sync, f32x16 (&s_cur)[QB], f32x16 (&s_next)[QB],
                    const bf16x8 (&p_prev)[QB][2], bf16x8 (&p_cur)[QB][2]) __attribute__((always_inline)) {
        constexpr int J = decltype(phase)::value;
        auto stage_of = [&](int off) __attribute__((always_inline)) -> int {
            if constexpr (J >= 0) return (J + off) & (NST - 1);
            else return (b + off) & (NST - 1);
        };
        if constexpr (J >= 0) {
            // the fragment addresses are "redefined" here so that address + constant is formed
            // inside the step (and folded into the read's immediate) instead of being hoisted
            // out of the loop into one register per stage and fragment
#pragma unroll
            for (int i = 0; i < 8; i++) pin(kfo[i]);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                if constexpr (PV16) {
                    pin(vfo16[i][0]);
                    pin(vfo16[i][1]);
                } else {
                    pin(vfo[i]);
                }
            }
        }
        auto mfma_slot = [&](int slot) __attribute__((always_inline)) {
            if (MFMA_PRIO) __builtin_amdgcn_s_setprio(MFMA_PRIO);
            if (slot & 1) {
                const int idx = slot >> 1, kb = idx >> 2, blk = idx & 3;
                const bf16x8 vf =
                    __builtin_bit_cast(bf16x8, (s16x8)__builtin_shufflevector(vlo[idx], vhi[idx], 0, 1, 2, 3, 4, 5, 6, 7));
                if constexpr (PV16) {
#pragma unroll
                    for (int r = 0; r < 2; r++)
                        oacc16[idx][r] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, p_prev[0][r], oacc16[idx][r], 0, 0, 0);
                } else {
#pragma unroll
                    for (int qi = 0; qi < QB; qi++)
                        oacc[qi][blk] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, p_prev[qi][kb], oacc[qi][blk], 0, 0, 0);
                }
            } else {
                const int st = slot >> 1;
#pragma unroll
                for (int qi = 0; qi < QB; qi++)
                    s_next[qi] = score_mfma(kf[st], qf[qi][st], s_next[qi]);
            }
            if (MFMA_PRIO) __builtin_amdgcn_s_setprio(0);
        };

        if constexpr (MASKED) {
            // excluded keys (padding mask, key limit, tail) -> -inf; bit kk of badm = key kk of the block
            const unsigned badm = __builtin_amdgcn_readfirstlane(badm_cur); // fetched from LDS during the previous step
            if (badm != 0u) { // wave-uniform: most blocks exclude nothing
#pragma unroll
                for (int qi = 0; qi < QB; qi++)
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
        for (int qi = 0; qi < QB; qi++)
#pragma unroll
            for (int j = 0; j < 16; j++) s_next[qi][j] = REFACC ? negm[qi] : 0.f;

        float mc[QB], alpha[QB], psum[QB];
        unsigned pc[QB][8] = {}; // P as packed bf16 pairs
        u32x4 pb[2] = {};        // PV16: the same after the exchange between lane rows
#pragma unroll
        for (int qi = 0; qi < QB; qi++) {
            mc[qi] = (!BOUNDED && !REFACC && m_run[qi] != -INFINITY) ? m_run[qi] : 0.f;
            alpha[qi] = 1.f;
            psum[qi] = 0.f;
        }
        // exponentials of elements 2*pr, 2*pr+1 of this lane's 16 scores
        // (`shifted`: the scores still have mc to lose; not so for bounded scores, nor for scores
        // that arrived relative to the reference point)
        auto exp_pair = [&](int qi, int pr, auto shifted) __attribute__((always_inline)) {
            f32x16& sv = s_cur[qi];
            f32x2 pp;
            if constexpr (BOUNDED || !decltype(shifted)::value) {
                pp[0] = __builtin_amdgcn_exp2f(sv[2 * pr]);
                pp[1] = __builtin_amdgcn_exp2f(sv[2 * pr + 1]);
            } else {
                pp[0] = __builtin_amdgcn_exp2f(sv[2 * pr] - mc[qi]);
                pp[1] = __builtin_amdgcn_exp2f(sv[2 * pr + 1] - mc[qi]);
            }
            psum[qi] += pp[0] + pp[1];
            pc[qi][pr] = __builtin_bit_cast(unsigned, __builtin_convertvector(pp, bf16x2));
            pin(psum[qi]);
            pin(pc[qi][pr]);
        };
        // softmax of S(b) in 16 slices (per query block), spread so that every
        // MFMA has about the same amount of VALU work behind it
        auto valu_slice = [&](int c) __attribute__((always_inline)) {
#pragma unroll
            for (int qi = 0; qi < QB; qi++) {
                f32x16& sv = s_cur[qi];
                if constexpr (BOUNDED) {
                    if ((c & 1) == 0) exp_pair(qi, c >> 1, std::false_type{});
                    if (c == 15) {
                        l_run[qi] += psum[qi];
                        pin(l_run[qi]);
                    }
                } else {
                    // running-maximum build: the same slices, against the reference point as it
                    // stands (the scores arrive relative to it, or it is subtracted here); the
                    // watch after the slots adds the denominator
                    if ((c & 1) == 0) exp_pair(qi, c >> 1, std::integral_constant<bool, !REFACC>{});
                }
                if constexpr (PV16) {
                    // The exponentiated block as the product's B operands. pc[k] packs this lane's
                    // scores 2 k and 2 k + 1 of its query (keys 8 (k / 2) + 4 h + 2 (k % 2) .. + 1).
                    // v_permlane16_swap of pc[k] and pc[k + 4] returns [a.row0, b.row0, a.row2, b.row2]
                    // and [a.row1, b.row1, a.row3, b.row3] (rows of 16 lanes): the first holds queries
                    // 0..15 on every lane row, the second queries 16..31, and lane row g4 holds keys
                    // vkey0 + {0..3, 8..11}: eight of the block's 32 keys per group, as the 16 x 16 x
                    // 32 MFMA's B operand wants them. One pair per odd slice, as soon as both exist.
                    if (c >= 9 && (c & 1)) {
                        const int k = (c - 9) >> 1;
                        const u32x2 r = __builtin_amdgcn_permlane16_swap(pc[qi][k], pc[qi][k + 4], false, false);
                        pb[0][k] = r[0];
                        pb[1][k] = r[1];
                    }
                    if (c == 15) {
                        p_cur[qi][0] = __builtin_bit_cast(bf16x8, pb[0]);
                        p_cur[qi][1] = __builtin_bit_cast(bf16x8, pb[1]);
                    }
                } else if (c == 15) {
                    p_cur[qi][0] = __builtin_bit_cast(bf16x8, u32x4{pc[qi][0], pc[qi][1], pc[qi][2], pc[qi][3]});
                    p_cur[qi][1] = __builtin_bit_cast(bf16x8, u32x4{pc[qi][4], pc[qi][5], pc[qi][6], pc[qi][7]});
                }
            }
        };

        if constexpr (!XSTEP) {
#pragma unroll
            for (int g = 0; g < LA; g++) frag_read(stage_of(1), stage_of(NST - 1), g);
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int g = 0; g < 16; g++) {
            // reads are issued RB slots' worth at a time, so one wait covers RB MFMAs
            if (g % RB == 0) {
#pragma unroll
                for (int j = 0; j < RB; j++) {
                    const int slot = g + LA + j;
                    if (slot < 16) frag_read(stage_of(1), stage_of(NST - 1), slot);
                    else if constexpr (XSTEP) frag_read(stage_of(2), stage_of(0), slot - 16);
                }
            }
            mfma_slot(g);
            valu_slice(g);
            // ring: block b+AHEAD (in this register set since two steps ago) goes to its stage,
            // whose previous tenant's last reader (V, NST-AHEAD-1 steps back) is at least one
            // barrier behind; then the set starts loading block b+AHEAD+2
            if constexpr (MASKED) {
                if (g == 10) badm_cur = bmask[block_of(b + 1 < nblk ? b + 1 : nblk - 1)];
            }
            if constexpr (DMA) {
                if (g == STORE_SLOT) dma_fetch(b + AHEAD, stage_of(AHEAD));
            } else {
                if (g == STORE_SLOT) stage_store(regs, stage_of(AHEAD));
                if (g == STORE_SLOT + 1) stage_load(regs, b + AHEAD + 2);
            }
            __builtin_amdgcn_sched_barrier(0);
        }

        if constexpr (!BOUNDED) {
            // Lazy running maximum without a maximum per block. The exponentials above were taken
            // against the reference point m_run as it stood (the scores arrived relative to it,
            // negm being their accumulator's starting value, or it was subtracted). A lane's 16 of them add up
            // to more than 16 * 2^kTau only if one of its scores lies more than kTau above the
            // reference (then, or for a row that has no reference yet, or when the sum is not a
            // number, the block is redone below); otherwise every P is at most 2^(kTau+4) and
            // the block stands. The redo forms the row maxima, moves the reference of the rows
            // whose maximum exceeds it by more than kTau (both lanes of a row decide alike),
            // takes the exponentials again and rescales O and the denominator.
            bool redo = false;
#pragma unroll
            for (int qi = 0; qi < QB; qi++) redo |= !(psum[qi] <= 16.0f * 256.0f) || m_run[qi] == -INFINITY;
            static_assert(kTau == 8.0f, "the watch threshold is 16 * 2^kTau");
            if (__any(redo)) {
#pragma unroll
                for (int qi = 0; qi < QB; qi++) {
                    f32x16& sv = s_cur[qi];
                    float t0 = fmaxf(fmaxf(sv[0], sv[1]), sv[2]);
                    float t1 = fmaxf(fmaxf(sv[3], sv[4]), sv[5]);
                    float t2 = fmaxf(fmaxf(sv[6], sv[7]), sv[8]);
                    float t3 = fmaxf(fmaxf(sv[9], sv[10]), sv[11]);
                    float t4 = fmaxf(fmaxf(sv[12], sv[13]), sv[14]);
                    t0 = fmaxf(fmaxf(t0, t1), t2);
                    t3 = fmaxf(fmaxf(t3, t4), sv[15]);
                    // the scores are relative to `ref` (the reference point, 0 before the first)
                    const float ref = (REFACC && m_run[qi] != -INFINITY) ? m_run[qi] : 0.f;
                    const float mlc = pair_max(fmaxf(t0, t3)) + ref;
                    const bool up = mlc > m_run[qi] + kTau;
                    const float m_new = up ? mlc : m_run[qi];
                    const float ref_new = (m_new == -INFINITY) ? 0.f : m_new;
                    mc[qi] = ref_new - ref;
                    alpha[qi] = __builtin_amdgcn_exp2f(m_run[qi] - ref_new);
                    m_run[qi] = m_new;
                    psum[qi] = 0.f;
#pragma unroll
                    for (int pr = 0; pr < 8; pr++) exp_pair(qi, pr, std::true_type{});
                    if constexpr (REFACC) {
                        // the next block's scores were formed against the old reference
#pragma unroll
                        for (int j = 0; j < 16; j++) {
                            s_next[qi][j] -= mc[qi];
                            negm[qi] = -ref_new;
                        }
                    }
                    l_run[qi] *= alpha[qi];
                    if constexpr (PV16) {
                        // O^T holds other queries on this lane than the scores do: the factor of
                        // query 16 r + c16 comes from the lane that owns that query's scores
#pragma unroll
                        for (int r = 0; r < 2; r++) {
                            const float ar = __uint_as_float((unsigned)__builtin_amdgcn_ds_bpermute(4 * (16 * r + c16), (int)__float_as_uint(alpha[qi])));
#pragma unroll
                            for (int dt = 0; dt < 8; dt++) oacc16[dt][r] *= ar;
                        }
                    } else {
#pragma unroll
                        for (int blk = 0; blk < 4; blk++)
#pragma unroll
                            for (int j = 0; j < 16; j++) oacc[qi][blk][j] *= alpha[qi];
                    }
                    if constexpr (PV16) { // the exchange of valu_slice, on the pairs taken again
#pragma unroll
                        for (int k = 0; k < 4; k++) {
                            const u32x2 r = __builtin_amdgcn_permlane16_swap(pc[qi][k], pc[qi][k + 4], false, false);
                            pb[0][k] = r[0];
                            pb[1][k] = r[1];
                        }
                        p_cur[qi][0] = __builtin_bit_cast(bf16x8, pb[0]);
                        p_cur[qi][1] = __builtin_bit_cast(bf16x8, pb[1]);
                    } else {
                        p_cur[qi][0] = __builtin_bit_cast(bf16x8, u32x4{pc[qi][0], pc[qi][1], pc[qi][2], pc[qi][3]});
                        p_cur[qi][1] = __builtin_bit_cast(bf16x8, u32x4{pc[qi][4], pc[qi][5], pc[qi][6], pc[qi][7]});
                    }
                }
            }
#pragma unroll
            for (int qi = 0; qi < QB; qi++) {
                l_run[qi] += psum[qi];
                pin(l_run[qi]);
            }
        }
        if (sync) {
            if constexpr (XSTEP) {
                // Only the next step's first fragment reads are outstanding here and they
                // touch stages no one writes before the next barrier. LDS operations of a
                // wave complete in order and every read of this step has been consumed, so
                // this step's ring writes are complete: the bare barrier orders them.
                asm volatile("" ::: "memory");
                // direct loads: all but this step's two must have landed (vmcnt(2)); a block is
                // first read two barriers after it was requested
                if constexpr (DMA) __builtin_amdgcn_s_waitcnt(0x0F72);
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
            } else {
                __syncthreads();
            }
        }
    };

    if (nblk > 0) {
        // prologue: blocks 0 .. AHEAD-1 into the ring, blocks AHEAD and AHEAD+1 in flight
        if constexpr (DMA) {
            // The wave's 32 prepared query rows (bf16, scale folded in) and the first AHEAD K/V
            // blocks are requested together: one memory latency for all of it. Each wave parks
            // its rows in 8 KB that the ring does not use yet (K stages 5-7, V stages 5-6, and
            // the area behind the lists), in the K layout (chunk c of row r at c ^ (r & 15)),
            // and is their only reader, so it needs no barrier for them, only its own vmcnt.
            const unsigned q_span = ((unsigned)(a.tokens - 1) * (unsigned)a.q_ts + D) * 2u;
            const u32x4 q_rsrc = make_rsrc_words(reinterpret_cast<const bf16_t*>(a.q) + (int64_t)seg * a.q_bs + (int64_t)head * a.q_hs, q_span);
            const unsigned q_lds = __builtin_amdgcn_readfirstlane(
                wave < 3   ? lds_address(Ks) + (unsigned)((5 + wave) * (KSTAGE * 2))
                : wave < 5 ? lds_address(Vs) + (unsigned)((5 + wave - 3) * (VSTAGE * 2))
                           : lds_address(Vs) + (unsigned)(NST * (VSTAGE * 2) + (int)kListBytes + (wave - 5) * (KB * D * 2)));
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const int r = 4 * j + (lane >> 4);
                const int qrow = min(q0 + r, a.tokens - 1); // rows past the sequence re-read the last row (never stored)
                const unsigned off = ((unsigned)qrow * (unsigned)a.q_ts + (unsigned)(((lane & 15) ^ (r & 15)) * 8)) * 2u;
                load_to_lds_16(q_rsrc, q_lds + (unsigned)(j * 1024), off, 0u);
            }
            // what the first two steps read before their barrier (K blocks 0..3, V blocks 0 and 1:
            // step 1 already reads the first fragments of step 2) is requested first and waited
            // for here; the rest of the first AHEAD blocks (4 loads) is covered by the wait before
            // the barrier that ends step 1. Every workgroup of a round starts at once, so these
            // first loads arrive at the rate of memory, not at its latency.
            static_assert(AHEAD == 5, "the prologue's load count assumes five blocks ahead");
            dma_fetch_part(0, 0, 3);
            dma_fetch_part(1, 1, 3);
            dma_fetch_part(2, 2, 1);
            dma_fetch_part(3, 3, 1);
            dma_fetch_part(2, 2, 2);
            dma_fetch_part(3, 3, 2);
            dma_fetch_part(4, 4, 3);
            __builtin_amdgcn_s_waitcnt(0x0F74); // vmcnt(4)
            asm volatile("" ::: "memory");
            typedef const __attribute__((address_space(3))) bf16x8* lds_q_t;
#pragma unroll
            for (int s = 0; s < 8; s++)
                qf[0][s] = *(lds_q_t)(q_lds + (unsigned)(l32 * (D * 2) + (((2 * s + h) ^ (l32 & 15)) * 16)));
            // rows that did not pass the pre-pass (operands used as given) still need the softmax
            // scale that the exp2-domain scores ride on (wave-uniform branch)
            if (a.scale_log2 != 1.0f) {
#pragma unroll
                for (int s = 0; s < 8; s++) {
                    f32x8 x = __builtin_convertvector(qf[0][s], f32x8);
                    x *= a.scale_log2;
                    qf[0][s] = __builtin_convertvector(x, bf16x8);
                }
            }
        } else {
            StageRegs pre[AHEAD];
#pragma unroll
            for (int i = 0; i < AHEAD; i++) stage_load(pre[i], i);
            stage_load(sets[0], AHEAD);
            stage_load(sets[1], AHEAD + 1);
            __syncthreads(); // ring zeroing complete
#pragma unroll
            for (int i = 0; i < AHEAD; i++) stage_store(pre[i], i);
        }
        __syncthreads();

        f32x16 s_a[QB], s_b[QB];
        bf16x8 p_a[QB][2], p_b[QB][2];
#pragma unroll
        for (int qi = 0; qi < QB; qi++)
#pragma unroll
            for (int kb = 0; kb < 2; kb++)
#pragma unroll
                for (int j = 0; j < 8; j++) p_a[qi][kb][j] = (bf16_t)0.0f;
        qk_block(0, s_a);
        if constexpr (XSTEP) {
#pragma unroll
            for (int g = 0; g < LA; g++) frag_read(1, NST - 1, g);
        }

        // Steps alternate the roles of the S and P buffers; with the 8-stage ring only odd
        // steps end in a barrier. The main loop takes one full turn of the ring per trip
        // with the ring phase a constant in every step; the remainder runs step by step.
        typedef std::integral_constant<int, -1> Dyn;
        int b = 0;
        // (builds that prepare K inside the block load carry too much state for a full turn)
        for (; KMODE == kQkNone && b + NST <= nblk; b += NST) {
            step(std::integral_constant<int, 0>{}, b, sets[0], NST != 8, s_a, s_b, p_a, p_b);
            step(std::integral_constant<int, 1>{}, b + 1, sets[1], true, s_b, s_a, p_b, p_a);
            step(std::integral_constant<int, 2>{}, b + 2, sets[0], NST != 8, s_a, s_b, p_a, p_b);
            step(std::integral_constant<int, 3>{}, b + 3, sets[1], true, s_b, s_a, p_b, p_a);
            if constexpr (NST == 8) {
                step(std::integral_constant<int, 4>{}, b + 4, sets[0], false, s_a, s_b, p_a, p_b);
                step(std::integral_constant<int, 5>{}, b + 5, sets[1], true, s_b, s_a, p_b, p_a);
                step(std::integral_constant<int, 6>{}, b + 6, sets[0], false, s_a, s_b, p_a, p_b);
                step(std::integral_constant<int, 7>{}, b + 7, sets[1], true, s_b, s_a, p_b, p_a);
            }
        }
        for (; b + 1 < nblk; b += 2) {
            step(Dyn{}, b, sets[0], NST != 8, s_a, s_b, p_a, p_b);
            step(Dyn{}, b + 1, sets[1], true, s_b, s_a, p_b, p_a);
        }
        if (b < nblk) {
            step(Dyn{}, b, sets[0], true, s_a, s_b, p_a, p_b);
            pv_block((nblk - 1) & (NST - 1), p_b);
        } else {
            pv_block((nblk - 1) & (NST - 1), p_a);
        }
        if constexpr (DMA) __builtin_amdgcn_s_waitcnt(0x0F70); // no direct load may outlive the workgroup's LDS
    }

    // ---- epilogue: O = O^T / l
    if constexpr (PV16) {
        // The denominator lives with the scores (lane = query l32); the lane that holds query
        // 16 r + c16 of O^T fetches it from there.
        const float l_tot = pair_sum(l_run[0]);
        const float inv_l = l_tot > 0.f ? 1.0f / l_tot : 0.f;
        float inv_r[2];
#pragma unroll
        for (int r = 0; r < 2; r++)
            inv_r[r] = __uint_as_float((unsigned)__builtin_amdgcn_ds_bpermute(4 * (16 * r + c16), (int)__float_as_uint(inv_l)));
        if (splits > 1) {
            // unnormalised rows, reference point and denominator of this part
            const int64_t prow0 = (int64_t)blockIdx.x * BQ + wave * QR;
#pragma unroll
            for (int r = 0; r < 2; r++) {
                float* op = a.part_o + (prow0 + 16 * r + c16) * D + 4 * g4;
#pragma unroll
                for (int dt = 0; dt < 8; dt++) *reinterpret_cast<f32x4*>(op + 16 * dt) = oacc16[dt][r];
            }
            if (h == 0) {
                a.part_ml[(prow0 + l32) * 2] = BOUNDED ? 0.f : m_run[0];
                a.part_ml[(prow0 + l32) * 2 + 1] = l_tot;
            }
        } else if (a.out_dtype == kF32) {
#pragma unroll
            for (int r = 0; r < 2; r++) {
                const int qrow = q0 + 16 * r + c16;
                if (qrow < a.tokens) {
                    float* op = reinterpret_cast<float*>(a.o) + (int64_t)seg * a.o_bs + (int64_t)qrow * a.o_ts + (int64_t)head * a.o_hs + 4 * g4;
#pragma unroll
                    for (int dt = 0; dt < 8; dt++) *reinterpret_cast<f32x4*>(op + 16 * dt) = oacc16[dt][r] * inv_r[r];
                }
            }
        } else {
            // 16-bit output: a lane holds 8-byte pieces of two rows, which would leave the chip as
            // 16 thirty-two-byte segments per store instruction. The wave turns its 32 x 128 tile
            // through 8 KB of LDS (its own stage of the idle K ring, K layout: chunk c of row r
            // at c ^ (r & 15)) and stores whole 256-byte rows, four per instruction.
            __syncthreads(); // every wave is done with the ring
            typedef __attribute__((address_space(3))) u32x2* lds_u32x2_t;
            typedef const __attribute__((address_space(3))) u32x4* lds_u32x4_t;
            typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
            const unsigned o_lds = lds_address(Ks) + (unsigned)(wave * (KSTAGE * 2));
            const bool half = a.out_dtype == kF16;
#pragma unroll
            for (int r = 0; r < 2; r++)
#pragma unroll
                for (int dt = 0; dt < 8; dt++) {
                    // row 16 r + c16, dims 16 dt + 4 g4 .. + 3: chunk 2 dt + g4 / 2, half g4 % 2
                    const f32x4 v = oacc16[dt][r] * inv_r[r];
                    const u32x2 bits = half ? __builtin_bit_cast(u32x2, __builtin_convertvector(v, f16x4))
                                            : __builtin_bit_cast(u32x2, __builtin_convertvector(v, bf16x4));
                    *(lds_u32x2_t)(o_lds + (unsigned)((16 * r + c16) * (D * 2) + (((2 * dt + (g4 >> 1)) ^ c16) * 16) + 8 * (g4 & 1))) = bits;
                }
            unsigned short* const obase = reinterpret_cast<unsigned short*>(a.o) + (int64_t)seg * a.o_bs + (int64_t)head * a.o_hs;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const int r = 4 * j + (lane >> 4);
                const u32x4 row16 = *(lds_u32x4_t)(o_lds + (unsigned)(r * (D * 2) + (lane & 15) * 16));
                const int orow = q0 + r;
                if (orow < a.tokens)
                    *reinterpret_cast<u32x4*>(obase + (int64_t)orow * a.o_ts + (((lane & 15) ^ (r & 15)) * 8)) = row16;
            }
        }
    } else {
#pragma unroll
        for (int qi = 0; qi < QB; qi++) {
            const float l_tot = pair_sum(l_run[qi]);
            const float inv_l = l_tot > 0.f ? 1.0f / l_tot : 0.f;
            const int qrow = q0 + 32 * qi + l32;
            if (splits > 1) {
                // unnormalised rows, reference point and denominator of this part
                const int64_t prow = ((int64_t)blockIdx.x * BQ + wave * QR + 32 * qi + l32);
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
                    a.part_ml[prow * 2] = BOUNDED ? 0.f : m_run[qi];
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
                // 16-bit output: a lane holds one row in 8-byte pieces, which would leave the chip as
                // 32 sixteen-byte segments per store instruction. The wave turns its 32 x 128 tile
                // through 8 KB of LDS (its own stage of the idle K ring, K layout: chunk c of row r
                // at c ^ (r & 15)) and stores whole 256-byte rows, four per instruction.
                __syncthreads(); // every wave is done with the ring
                typedef __attribute__((address_space(3))) u32x2* lds_u32x2_t;
                typedef const __attribute__((address_space(3))) u32x4* lds_u32x4_t;
                typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
                const unsigned o_lds = lds_address(Ks) + (unsigned)((wave * QB + qi) * (KSTAGE * 2));
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
                    const u32x4 row16 = *(lds_u32x4_t)(o_lds + (unsigned)(r * (D * 2) + (lane & 15) * 16));
                    const int orow = q0 + 32 * qi + r;
                    if (orow < a.tokens)
                        *reinterpret_cast<u32x4*>(obase + (int64_t)orow * a.o_ts + (((lane & 15) ^ (r & 15)) * 8)) = row16;
                }
            }
        }
    }
    // (whole tiles only: the parts carry no probe)
    const int64_t probe_slot = (int64_t)blockIdx.x - a.part_wgs;
    if (a.clock_probe && tid == 0 && probe_slot >= 0 && probe_slot < a.clock_cap) {
        a.clock_probe[2 * probe_slot] = __builtin_readcyclecounter() - clk_c0;
        a.clock_probe[2 * probe_slot + 1] = __builtin_amdgcn_s_memrealtime() - clk_r0;
    }
}

constexpr int kMaxSplits = 16; // parts per key-split tile

// Combines the parts of the key-split tiles: out[row] = sum_z O_z 2^(m_z - M) / sum_z l_z 2^(m_z - M),
// M = max_z m_z, z ascending (l_z = 0: an empty part, weight 0). 32 lanes per row, 4 dims each.
// NZ >= splits is the build's bound on the parts: every load of the lane (reference point and
// denominator, then the rows, of all parts) is sent before the first is used, so the kernel
// pays one memory round trip instead of one per part.
template <int NZ>
__global__ void __launch_bounds__(256) attn_merge_kernel(const AttnArgs a, int block_rows) {
    const int r = (int)blockIdx.x * 8 + (int)(threadIdx.x >> 5); // row among tail_tiles x block_rows
    const int t = r / block_rows;
    const int rr = r - t * block_rows;
    const int logical = a.tile_base + t;
    const int bh = logical / a.nqb;
    const int qb = logical - bh * a.nqb;
    const int seg = bh / a.heads;
    const int head = bh - seg * a.heads;
    const int qrow = qb * block_rows + rr;
    if (qrow >= a.tokens) return;
    const int d0 = (threadIdx.x & 31) * 4;
    const int64_t prow0 = (int64_t)t * a.splits * block_rows + rr;
    f32x2 ml[NZ];
    f32x4 x[NZ];
#pragma unroll
    for (int z = 0; z < NZ; z++) {
        ml[z] = f32x2{0.f, 0.f};
        if (z < a.splits) ml[z] = *reinterpret_cast<const f32x2*>(a.part_ml + (prow0 + (int64_t)z * block_rows) * 2);
    }
#pragma unroll
    for (int z = 0; z < NZ; z++) {
        x[z] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (z < a.splits) x[z] = *reinterpret_cast<const f32x4*>(a.part_o + (prow0 + (int64_t)z * block_rows) * D + d0);
    }
    float M = -INFINITY;
#pragma unroll
    for (int z = 0; z < NZ; z++) M = (ml[z][1] > 0.f) ? fmaxf(M, ml[z][0]) : M;
    f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
    float l = 0.f;
#pragma unroll
    for (int z = 0; z < NZ; z++) {
        // past the last part, or a part that admitted no key: weight 0 (its row is all zeros)
        const float w = (ml[z][1] > 0.f) ? __builtin_amdgcn_exp2f(ml[z][0] - M) : 0.f;
        l += ml[z][1] * w;
        acc += x[z] * w;
    }
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    acc *= inv;
    const int64_t off = (int64_t)seg * a.o_bs + (int64_t)qrow * a.o_ts + (int64_t)head * a.o_hs + d0;
    if (a.out_dtype == kF32) {
        *reinterpret_cast<f32x4*>(reinterpret_cast<float*>(a.o) + off) = acc;
    } else if (a.out_dtype == kF16) {
        typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
        *reinterpret_cast<f16x4*>(reinterpret_cast<_Float16*>(a.o) + off) = __builtin_convertvector(acc, f16x4);
    } else {
        *reinterpret_cast<bf16x4*>(reinterpret_cast<bf16_t*>(a.o) + off) = __builtin_convertvector(acc, bf16x4);
    }
}

// One launch: the tiles of the last round in parts (tail.splits > 1), the whole tiles behind them; then the merge.
template <typename TIn, int KMODE, bool MASKED, bool BOUNDED, int QB, int NW>
static void launch_kernel(const AttnArgs& a, unsigned grid, hipStream_t stream) {
    if constexpr (std::is_same<TIn, bf16_t>::value && KMODE == kQkNone && QB == 1 && NW == 8) {
        if (a.score_f16) {
            attn_fwd_kernel<TIn, KMODE, MASKED, BOUNDED, QB, NW, true>
                <<<dim3(grid), dim3(NW * 64), lds_bytes(ring_stages(QB, NW)), stream>>>(a);
            return;
        }
    }
    attn_fwd_kernel<TIn, KMODE, MASKED, BOUNDED, QB, NW>
        <<<dim3(grid), dim3(NW * 64), lds_bytes(ring_stages(QB, NW)), stream>>>(a);
}

template <typename TIn, int KMODE, bool MASKED, bool BOUNDED, int QB, int NW>
static hipError_t launch_one(const AttnArgs& a0, hipStream_t stream) {
    const int64_t nwg = (int64_t)a0.nqb * a0.heads * a0.batch;
    if (nwg <= 0 || nwg > 0x7fffffff) return hipErrorInvalidValue;
    const int tail = a0.splits > 1 ? a0.tile_base : 0; // the planner leaves the tail size in tile_base
    AttnArgs a = a0;
    const int64_t whole = nwg - tail;
    a.tile_base = (int32_t)whole;
    a.splits = tail > 0 ? a0.splits : 1;
    a.part_wgs = tail > 0 ? (int32_t)(((int64_t)tail * a0.splits + 7) & ~(int64_t)7) : 0;
    if (whole + a.part_wgs > 0x7fffffff) return hipErrorInvalidValue;
    launch_kernel<TIn, KMODE, MASKED, BOUNDED, QB, NW>(a, (unsigned)(whole + a.part_wgs), stream);
    {
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    if (tail > 0) {
        const int rows = tail * NW * 32 * QB;
        const dim3 mgrid((unsigned)((rows + 7) / 8));
        if (a.splits <= 4) attn_merge_kernel<4><<<mgrid, dim3(256), 0, stream>>>(a, NW * 32 * QB);
        else if (a.splits <= 8) attn_merge_kernel<8><<<mgrid, dim3(256), 0, stream>>>(a, NW * 32 * QB);
        else if (a.splits <= kMaxSplits) attn_merge_kernel<kMaxSplits><<<mgrid, dim3(256), 0, stream>>>(a, NW * 32 * QB);
        else return hipErrorInvalidValue;
        return hipGetLastError();
    }
    return hipSuccess;
}

template <typename TIn, bool MASKED, bool BOUNDED, int QB, int NW>
static hipError_t launch_kmode(const AttnArgs& a, int k_mode, hipStream_t stream) {
    switch (k_mode) {
    case kQkNone: return launch_one<TIn, kQkNone, MASKED, BOUNDED, QB, NW>(a, stream);
    case kQkKlein: return launch_one<TIn, kQkKlein, MASKED, BOUNDED, QB, NW>(a, stream);
    case kQkZimage: return launch_one<TIn, kQkZimage, MASKED, BOUNDED, QB, NW>(a, stream);
    default: return hipErrorInvalidValue;
    }
}

template <typename TIn, int QB, int NW>
static hipError_t launch_flags(const AttnArgs& a, int k_mode, hipStream_t stream) {
    // Q and K are prepared at the same site: the builds rely on it
    if ((k_mode == kQkNone) != (a.q_mode == kQkNone)) return hipErrorInvalidValue;
    // half-precision score operands: prepared 16-bit rows on the eight-wave shape, scale already applied
    if (a.score_f16 && !(std::is_same<TIn, bf16_t>::value && k_mode == kQkNone && QB == 1 && NW == 8 && a.scale_log2 == 1.0f))
        return hipErrorInvalidValue;
    // the masked build is only needed when some key of some block is excluded
    const bool masked = a.key_pad != nullptr || (a.key_limit % KB) != 0;
    const bool bounded = a.bounded != 0;
    if (masked)
        return bounded ? launch_kmode<TIn, true, true, QB, NW>(a, k_mode, stream)
                       : launch_kmode<TIn, true, false, QB, NW>(a, k_mode, stream);
    return bounded ? launch_kmode<TIn, false, true, QB, NW>(a, k_mode, stream)
                   : launch_kmode<TIn, false, false, QB, NW>(a, k_mode, stream);
}

template <int QB, int NW>
static hipError_t launch_shape(const AttnArgs& a, int in_dtype, int k_mode, hipStream_t stream) {
    if (in_dtype == kF32) return launch_flags<float, QB, NW>(a, k_mode, stream);
    if (in_dtype == kBF16) return launch_flags<bf16_t, QB, NW>(a, k_mode, stream);
    return hipErrorInvalidValue;
}

template <typename TIn, int KMODE, bool MASKED, bool BOUNDED, int QB, int NW>
static hipError_t raise_lds() {
    if constexpr (std::is_same<TIn, bf16_t>::value && KMODE == kQkNone && QB == 1 && NW == 8) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_fwd_kernel<TIn, KMODE, MASKED, BOUNDED, QB, NW, true>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes(ring_stages(QB, NW)));
        if (e != hipSuccess) return e;
    }
    return hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_fwd_kernel<TIn, KMODE, MASKED, BOUNDED, QB, NW>),
                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes(ring_stages(QB, NW)));
}

template <int QB, int NW>
static hipError_t raise_shape() {
    hipError_t e;
#define ZD_RAISE(T, M) \
    if ((e = raise_lds<T, M, false, false, QB, NW>()) != hipSuccess) return e; \
    if ((e = raise_lds<T, M, true, false, QB, NW>()) != hipSuccess) return e; \
    if ((e = raise_lds<T, M, false, true, QB, NW>()) != hipSuccess) return e; \
    if ((e = raise_lds<T, M, true, true, QB, NW>()) != hipSuccess) return e;
    ZD_RAISE(float, kQkNone) ZD_RAISE(float, kQkKlein) ZD_RAISE(float, kQkZimage)
    ZD_RAISE(bf16_t, kQkNone) ZD_RAISE(bf16_t, kQkKlein) ZD_RAISE(bf16_t, kQkZimage)
#undef ZD_RAISE
    return hipSuccess;
}

} // namespace fwd

int attention_block_rows(int shape) { return shape == 1 ? 128 : 256; }

void attention_tail_plan(int64_t tiles, int cus, int key_blocks, int* tail_tiles, int* splits) {
    *tail_tiles = 0;
    *splits = 1;
    if (tiles <= 0 || cus <= 0) return;
    const int tail = (int)(tiles % cus);
    // a last round that fills at most half the CUs: split its tiles along the keys so that it
    // fills them all; each part keeps at least 8 key blocks
    if (tail == 0 || tail * 2 > cus) return;
    int s = cus / tail;
    if (s > fwd::kMaxSplits) s = fwd::kMaxSplits;
    if (s > key_blocks / 8) s = key_blocks / 8;
    if (s < 2) return;
    *tail_tiles = tail;
    *splits = s;
}
size_t attention_part_o_bytes(int tail_tiles, int splits, int shape) {
    return (size_t)tail_tiles * splits * attention_block_rows(shape) * D * sizeof(float);
}
size_t attention_part_ml_bytes(int tail_tiles, int splits, int shape) {
    return (size_t)tail_tiles * splits * attention_block_rows(shape) * 2 * sizeof(float);
}
int attention_key_block() { return fwd::KB; }
int attention_max_tokens() { return fwd::MAX_BLOCKS * fwd::KB; }

hipError_t launch_attention(const AttnArgs& a, int in_dtype, int k_mode, int shape, hipStream_t stream) {
    switch (shape) {
    case 0: return fwd::launch_shape<1, 8>(a, in_dtype, k_mode, stream);
    case 1: return fwd::launch_shape<1, 4>(a, in_dtype, k_mode, stream);
    default: return hipErrorInvalidValue;
    }
}

hipError_t attention_setup() {
    hipError_t e;
    if ((e = fwd::raise_shape<1, 8>()) != hipSuccess) return e;
    if ((e = fwd::raise_shape<1, 4>()) != hipSuccess) return e;
    return hipSuccess;
}

} // namespace zdraw
