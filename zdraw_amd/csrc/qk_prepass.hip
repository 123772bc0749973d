// Standalone QK-norm + rope over the rows of one operand (gfx950).
//
// Replaces krms_rope / krms_rope_hm (klein/zflux2_glue_shader.zig:61-122) and
// qk_norm_rope / qk_norm_rope_hm_f16 (metal/mqk_shader.zig:46-97,
// metal_api.m:6215-6265): used as the optional K pre-pass of the fused
// attention entry and as the in-place f32 form behind zdraw_hip_run_qk_norm_rope.
#include "attn_device.hpp"

namespace zdraw {

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

} // namespace zdraw
