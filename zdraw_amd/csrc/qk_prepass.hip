// Standalone QK-norm + rope over the rows of one operand (gfx950).
//
// Replaces krms_rope / krms_rope_hm (klein/zflux2_glue_shader.zig:61-122) and
// qk_norm_rope / qk_norm_rope_hm_f16 (metal/mqk_shader.zig:46-97,
// metal_api.m:6215-6265): used as the optional Q/K pre-pass of the fused
// attention entry and as the in-place f32 form behind zdraw_hip_run_qk_norm_rope.
#include "attn_device.hpp"

namespace zdraw {

// ------------------------------------------------ Q/K pre-pass (norm + rope)
// 16 lanes per row (8 dims each). A wave covers one token: its four 16-lane
// groups take four heads at a time (1 KB contiguous in a token-major operand)
// and walk G such groups of heads, keeping the token's rope coefficients and
// norm weights in registers, so the rope table is read once per token. All G
// loads of a lane are issued before the first is used. Input and output are
// addressed by strides, so the same kernel serves the 16-bit Q/K pre-pass and the
// in-place f32 token-major form. A lane reads and writes only its own 8
// elements, so the output may alias the input.
constexpr int kPrepTokens = 4; // tokens (waves) per workgroup

// G = groups of four heads walked by one lane: 6 (24 heads per pass: Klein) or 8 (32 heads
// per pass: Z-Image's 30 heads in one pass instead of two)
template <typename TIn, int MODE, int G>
__global__ void __launch_bounds__(kPrepTokens * 64) qk_prepass_kernel(const PrepPair pair) {
    // grid z = operand * batch + segment; the choice is uniform over the workgroup
    const int op = (int)blockIdx.z / pair.op[0].batch;
    const PrepArgs& p = pair.op[op];
    const int tok_raw = (int)blockIdx.x * kPrepTokens + (int)(threadIdx.x >> 6);
    const bool tok_ok = tok_raw < p.tokens;
    const int tok = tok_ok ? tok_raw : p.tokens - 1; // lanes past the end work on the last token and store nothing
    const int h0 = (int)blockIdx.y * (4 * G) + (int)((threadIdx.x >> 4) & 3);
    const int seg = (int)blockIdx.z - op * pair.op[0].batch;
    const int d0 = (threadIdx.x & 15) * 8;
    // Every load of the lane is issued before the first is used, with clamped addresses
    // instead of predicates: no branch, so nothing waits for an earlier load to come back
    // before the next is sent.
    if (p.mode == kQkNone) {
        // rows that are only rounded and re-laid (V beside a prepared Q and K)
        const TIn* src = reinterpret_cast<const TIn*>(p.x) + (int64_t)seg * p.x_bs + (int64_t)tok * p.x_ts + d0;
        Raw8<TIn> raw[G];
#pragma unroll
        for (int g = 0; g < G; g++) {
            const int head = h0 + 4 * g;
            raw[g] = ld_raw8<TIn>(src + (int64_t)(head < p.heads ? head : p.heads - 1) * p.x_hs, true);
        }
        __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0), once: see below
#pragma unroll
        for (int g = 0; g < G; g++) {
            const int head = h0 + 4 * g;
            float x[8];
            unpack8(raw[g], x);
#pragma unroll
            for (int i = 0; i < 8; i++) x[i] *= p.scale; // 1, or the softmax scale on un-normalised query rows
            if (tok_ok && head < p.heads) {
                const int64_t off = (int64_t)seg * p.y_bs + (int64_t)tok * p.y_ts + (int64_t)head * p.y_hs + d0;
                if (p.out_dtype == kF32) {
                    float* dst = reinterpret_cast<float*>(p.y) + off;
                    *reinterpret_cast<f32x4*>(dst) = f32x4{x[0], x[1], x[2], x[3]};
                    *reinterpret_cast<f32x4*>(dst + 4) = f32x4{x[4], x[5], x[6], x[7]};
                } else {
                    *reinterpret_cast<u32x4*>(reinterpret_cast<bf16_t*>(p.y) + off) = p.out_dtype == kF16 ? pack_f16x8(x) : pack_bf16x8(x);
                }
            }
        }
        return;
    }
    // Order of the loads: the token's position (Z-Image) first, because the address of its
    // rope coefficients depends on it and loads come back in the order they were sent; then
    // the norm weights, the rows, the rope coefficients. Nothing is used before all are sent.
    const QkRow qr = qk_row(p.qk, MODE, nullptr, nullptr, seg, tok, true);
    // weights of this lane's 8 dims: two 16-byte loads whatever the type (no branch between
    // loads); for 16-bit weights the second repeats the first
    const void* wsel = (p.w_txt != nullptr && tok < p.qk.txt_rows) ? p.w_txt : p.w;
    const bool w_f32 = p.w_dtype == kF32;
    const char* wsrc = static_cast<const char*>(wsel) + d0 * (w_f32 ? 4 : 2);
    const u32x4 wr0 = *reinterpret_cast<const u32x4*>(wsrc);
    const u32x4 wr1 = *reinterpret_cast<const u32x4*>(wsrc + (w_f32 ? 16 : 0));
    const TIn* src = reinterpret_cast<const TIn*>(p.x) + (int64_t)seg * p.x_bs + (int64_t)tok * p.x_ts + d0;
    Raw8<TIn> raw[G];
#pragma unroll
    for (int g = 0; g < G; g++) {
        const int head = h0 + 4 * g;
        raw[g] = ld_raw8<TIn>(src + (int64_t)(head < p.heads ? head : p.heads - 1) * p.x_hs, true);
    }
    const Rope8 t = ld_rope8(p.qk, MODE, qr, d0);
    // One wait for everything: the stores below sit under a predicate, and past a branch the
    // compiler no longer knows how many stores are younger than a load it waits for, so it
    // would wait for the previous heads' stores as well.
    // (Z-Image only: its coefficients are the last load to come back anyway. Klein's heads are
    // worked on as their rows arrive, which measured 5 % faster than one wait.)
    if constexpr (MODE != kQkKlein) __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0)
    // the token's weights and rope row stay in registers across its heads
    f32x4 w0, w1;
    if (w_f32) {
        w0 = __builtin_bit_cast(f32x4, wr0);
        w1 = __builtin_bit_cast(f32x4, wr1);
    } else {
        float wv[8];
        if (p.w_dtype == kBF16) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                wv[2 * i] = __builtin_bit_cast(float, wr0[i] << 16);
                wv[2 * i + 1] = __builtin_bit_cast(float, wr0[i] & 0xffff0000u);
            }
        } else {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                wv[2 * i] = (float)__builtin_bit_cast(_Float16, (unsigned short)(wr0[i] & 0xffffu));
                wv[2 * i + 1] = (float)__builtin_bit_cast(_Float16, (unsigned short)(wr0[i] >> 16));
            }
        }
        w0 = f32x4{wv[0], wv[1], wv[2], wv[3]};
        w1 = f32x4{wv[4], wv[5], wv[6], wv[7]};
    }
#pragma unroll
    for (int g = 0; g < G; g++) {
        const int head = h0 + 4 * g;
        float x[8];
        unpack8(raw[g], x);
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) ss += x[i] * x[i];
        ss = row_group_sum<16>(ss);
        const float inv = rsqrtf(ss * (1.0f / D) + p.qk.eps);
        qk_apply8(MODE, x, inv, w0, w1, t);
#pragma unroll
        for (int i = 0; i < 8; i++) x[i] *= p.scale;
        if (tok_ok && head < p.heads) {
            const int64_t off = (int64_t)seg * p.y_bs + (int64_t)tok * p.y_ts + (int64_t)head * p.y_hs + d0;
            if (p.out_dtype == kF32) {
                float* dst = reinterpret_cast<float*>(p.y) + off;
                *reinterpret_cast<f32x4*>(dst) = f32x4{x[0], x[1], x[2], x[3]};
                *reinterpret_cast<f32x4*>(dst + 4) = f32x4{x[4], x[5], x[6], x[7]};
            } else {
                *reinterpret_cast<u32x4*>(reinterpret_cast<bf16_t*>(p.y) + off) = p.out_dtype == kF16 ? pack_f16x8(x) : pack_bf16x8(x);
            }
        }
    }
}

// Norm weights as a checkpoint view hands them over (metal/mqk.zig:77-102: a type per
// operand, a file offset that is only element-aligned), copied one element per thread to
// f32 where the pre-pass reads them with 16-byte loads.
__global__ void __launch_bounds__(2 * D) norm_weight_stage_kernel(const WeightStageArgs a) {
    const int i = (int)threadIdx.x & (D - 1);
    const bool is_k = (int)threadIdx.x >= D;
    const void* src = is_k ? a.k : a.q;
    const int dt = is_k ? a.k_dtype : a.q_dtype;
    float v;
    if (dt == kF32) {
        v = static_cast<const float*>(src)[i];
    } else {
        const unsigned short h = static_cast<const unsigned short*>(src)[i];
        v = dt == kBF16 ? __uint_as_float((unsigned)h << 16) : (float)__builtin_bit_cast(_Float16, h);
    }
    a.out[threadIdx.x] = v;
}

hipError_t launch_weight_stage(const WeightStageArgs& a, hipStream_t stream) {
    if (!a.q || !a.k || !a.out) return hipErrorInvalidValue;
    for (int dt : {a.q_dtype, a.k_dtype})
        if (dt != kF32 && dt != kF16 && dt != kBF16) return hipErrorInvalidValue;
    norm_weight_stage_kernel<<<dim3(1), dim3(2 * D), 0, stream>>>(a);
    return hipGetLastError();
}

// One launch covers `count` operands (1 to 3) of equal tokens/heads/batch: the first two are
// normalised and rotated (same mode), a third is only rounded and re-laid (mode kQkNone).
hipError_t launch_qk_prepass(const PrepArgs* ops, int count, int in_dtype, hipStream_t stream) {
    if (count < 1 || count > 3) return hipErrorInvalidValue;
    const PrepArgs& p = ops[0];
    if (p.batch <= 0 || p.heads <= 0 || p.tokens <= 0 || p.batch * count > 65535) return hipErrorInvalidValue;
    // all operands round-only (plain attention on f32 rows), or Q and K prepared and a third round-only
    const bool plain = p.mode == kQkNone;
    for (int i = 1; i < count; i++) {
        if (ops[i].batch != p.batch || ops[i].heads != p.heads || ops[i].tokens != p.tokens) return hipErrorInvalidValue;
        if (ops[i].mode != ((i == 2 || plain) ? (int32_t)kQkNone : p.mode)) return hipErrorInvalidValue;
    }
    PrepPair pair;
    for (int i = 0; i < 3; i++) pair.op[i] = ops[i < count ? i : count - 1];
    pair.count = count;
    pair.pad0 = 0;
    const bool wide_pass = (p.heads + 31) / 32 < (p.heads + 23) / 24; // fewer passes over the heads with 32 per pass
    const int per_pass = wide_pass ? 32 : 24;
    const dim3 grid((unsigned)((p.tokens + kPrepTokens - 1) / kPrepTokens), (unsigned)((p.heads + per_pass - 1) / per_pass),
                    (unsigned)(p.batch * count));
    const dim3 block(kPrepTokens * 64);
    const bool klein = p.mode == kQkKlein || plain; // round-only operands never reach the mode's code
    if (!klein && p.mode != kQkZimage) return hipErrorInvalidValue;
#define ZD_PREP(T, M) \
    do { \
        if (wide_pass) qk_prepass_kernel<T, M, 8><<<grid, block, 0, stream>>>(pair); \
        else qk_prepass_kernel<T, M, 6><<<grid, block, 0, stream>>>(pair); \
    } while (0)
    if (in_dtype == kF32) {
        if (klein) ZD_PREP(float, kQkKlein);
        else ZD_PREP(float, kQkZimage);
    } else if (in_dtype == kBF16) {
        if (klein) ZD_PREP(bf16_t, kQkKlein);
        else ZD_PREP(bf16_t, kQkZimage);
    } else if (in_dtype == kF16) {
        if (klein) ZD_PREP(f16_t, kQkKlein);
        else ZD_PREP(f16_t, kQkZimage);
    } else {
        return hipErrorInvalidValue;
    }
#undef ZD_PREP
    return hipGetLastError();
}

} // namespace zdraw
