// Fused QK-norm + rope + attention calls and the standalone Z-Image QK step,
// as the Klein and Z-Image block code issues them.
#include "zdraw_host.hpp"

#include <cstring>
#include <vector>

namespace zdraw {

namespace hqk {

size_t RopeCache::count() const {
    size_t total = 0;
    for (int a = 0; a < 3; a++) total += lens[a] * (dims[a] / 2);
    return total;
}
size_t RopeCache::axisBase(size_t axis) const {
    size_t base = 0;
    for (size_t a = 0; a < axis; a++) base += lens[a] * (dims[a] / 2);
    return base;
}

// metal/mqk.zig:60-75 (check) plus zrope.zig:48's position bound, which the
// reference applies on its CPU path and which protects the table gather here.
static Error check(const size_t* pos, size_t pos_len, const RopeCache& rope, const Config& cfg) {
    if (pos_len != cfg.tokens || cfg.head_dim == 0) return Error::InvalidShape;
    if (cfg.head_dim != rope.dims[0] + rope.dims[1] + rope.dims[2]) return Error::InvalidShape;
    for (size_t t = 0; t < pos_len; t++)
        for (int a = 0; a < 3; a++)
            if (pos[3 * t + a] >= rope.lens[a]) return Error::BadPosition;
    return Error::Ok;
}

Error run(hattn::Context* ctx, void* q_h, void* k_h, const float* q_weight, const float* k_weight,
          const size_t* pos, size_t pos_len, const RopeCache& rope, const Config& cfg) {
    if (!ctx || !ctx->qk_pipeline) return Error::NotAvailable; // mqk.zig:31 (error.GemmUnavailable)
    Error e = check(pos, pos_len, rope, cfg);
    if (e != Error::Ok) return e;
    std::vector<uint64_t> pos64(pos_len * 3);
    for (size_t i = 0; i < pos_len * 3; i++) pos64[i] = pos[i];
    hattn::Buffer qw = hattn::Buffer::fromBytes(ctx->device, q_weight, cfg.head_dim * sizeof(float));
    hattn::Buffer kw = hattn::Buffer::fromBytes(ctx->device, k_weight, cfg.head_dim * sizeof(float));
    hattn::Buffer pb = hattn::Buffer::fromBytes(ctx->device, pos64.data(), pos64.size() * sizeof(uint64_t));
    hattn::Buffer rb = hattn::Buffer::fromBytes(ctx->device, rope.values, rope.count() * 2 * sizeof(float));
    Error result = Error::OutOfMemory;
    if (qw.handle && kw.handle && pb.handle && rb.handle) {
        // mqk.zig:77-102 (makeParams): the weights are f32 views at offset 0 here
        ZdrawQkNormParams p{};
        p.tokens = (uint32_t)cfg.tokens;
        p.heads = (uint32_t)cfg.heads;
        p.kv_heads = (uint32_t)cfg.kv_heads;
        p.head_dim = (uint32_t)cfg.head_dim;
        p.q_dtype = p.k_dtype = ZDRAW_HIP_W_F32;
        p.dim0 = (uint32_t)rope.dims[0];
        p.dim1 = (uint32_t)rope.dims[1];
        p.dim2 = (uint32_t)rope.dims[2];
        p.eps = cfg.norm_eps;
        p.q_offset = p.k_offset = 0;
        p.base0 = rope.axisBase(0);
        p.base1 = rope.axisBase(1);
        p.base2 = rope.axisBase(2);
        result = fromCode(zdraw_hip_run_qk_norm_rope(ctx->queue, ctx->qk_pipeline, q_h, k_h, qw.handle, kw.handle,
                                                     pb.handle, rb.handle, &p, ctx->qk_threads));
    }
    qw.deinit();
    kw.deinit();
    pb.deinit();
    rb.deinit();
    return result;
}

} // namespace hqk

namespace joint {

float scoreBound(const float* w_q, const float* w_k, const float* w_q_txt, const float* w_k_txt) {
    auto amax = [](const float* w) {
        float m = 0.f;
        if (w)
            for (size_t i = 0; i < hattn::flash_head_dim; i++) {
                const float v = w[i] < 0 ? -w[i] : w[i];
                m = v > m ? v : m;
            }
        return m;
    };
    const float mq = amax(w_q) > amax(w_q_txt) ? amax(w_q) : amax(w_q_txt);
    const float mk = amax(w_k) > amax(w_k_txt) ? amax(w_k) : amax(w_k_txt);
    // |q'| <= sqrt(128) mq, |k'| <= sqrt(128) mk, divided by sqrt(128); 2% slack for
    // the rounding of the normalisation and of the bf16 operands
    return 11.313708498984761f * mq * mk * 1.02f;
}

static void fill_strides(uint64_t* s, size_t tokens, size_t row_stride, size_t nb) {
    s[0] = nb > 1 ? (uint64_t)tokens * row_stride : 0;
    s[1] = row_stride;
    s[2] = hattn::flash_head_dim;
}

Error run(hattn::Context* ctx, const Klein& c) {
    if (!ctx) return Error::NotAvailable;
    if (c.tokens == 0) return Error::UnsupportedShape;
    if (c.heads == 0 || c.nb == 0) return Error::InvalidShape;
    if (c.tokens > 0xffffffffu || c.heads > 0xffffffffu || c.nb > 0xffffffffu) return Error::InvalidShape;
    const size_t hidden = c.heads * hattn::flash_head_dim;
    ZdrawAttnParams p{};
    p.tokens = (uint32_t)c.tokens;
    p.heads = p.kv_heads = (uint32_t)c.heads;
    p.head_dim = (uint32_t)hattn::flash_head_dim;
    ZdrawHipAttnExt x;
    memset(&x, 0, sizeof(x));
    fill_strides(x.q_stride, c.tokens, hidden, c.nb);
    fill_strides(x.k_stride, c.tokens, hidden, c.nb);
    fill_strides(x.v_stride, c.tokens, hidden, c.nb);
    fill_strides(x.out_stride, c.tokens, c.out_row_stride ? c.out_row_stride : hidden, c.nb);
    x.batch = (uint32_t)c.nb;
    x.in_dtype = c.in_dtype;
    x.out_dtype = c.out_dtype;
    x.qk_mode = ZDRAW_HIP_QK_KLEIN;
    x.k_site = (uint32_t)c.k_site;
    x.txt_rows = (uint32_t)c.txt_rows;
    x.eps = 1e-6f; // klein/zflux2.zig:70 (rms_eps)
    x.rope_batch_rows = c.rope_per_segment ? c.tokens : 0;
    x.mask_batch_bytes = c.key_pad ? c.tokens : 0;
    x.score_bound = c.score_bound;
    x.staging = c.staging;
    ZdrawHipQkOperands ops;
    memset(&ops, 0, sizeof(ops));
    ops.q_weight = c.norm_q;
    ops.k_weight = c.norm_k;
    ops.q_weight_txt = c.norm_added_q;
    ops.k_weight_txt = c.norm_added_k;
    ops.rope_cos = c.rope_cos;
    ops.rope_sin = c.rope_sin;
    ops.key_pad = c.key_pad;
    return fromCode(zdraw_hip_run_attention_fused(ctx->queue, c.q, c.k, c.v, c.o, &p, &x, &ops));
}

Error run(hattn::Context* ctx, const Zimage& c) {
    if (!ctx) return Error::NotAvailable;
    if (c.tokens == 0) return Error::UnsupportedShape;
    if (c.heads == 0) return Error::InvalidShape;
    if (c.tokens > 0xffffffffu || c.heads > 0xffffffffu) return Error::InvalidShape;
    const size_t hidden = c.heads * hattn::flash_head_dim;
    ZdrawAttnParams p{};
    p.tokens = (uint32_t)c.tokens;
    p.heads = p.kv_heads = (uint32_t)c.heads;
    p.head_dim = (uint32_t)hattn::flash_head_dim;
    ZdrawHipAttnExt x;
    memset(&x, 0, sizeof(x));
    fill_strides(x.q_stride, c.tokens, hidden, 1);
    fill_strides(x.k_stride, c.tokens, hidden, 1);
    fill_strides(x.v_stride, c.tokens, hidden, 1);
    fill_strides(x.out_stride, c.tokens, hidden, 1);
    x.batch = 1;
    x.in_dtype = c.in_dtype;
    x.out_dtype = c.out_dtype;
    x.qk_mode = ZDRAW_HIP_QK_ZIMAGE;
    x.k_site = (uint32_t)c.k_site;
    x.eps = c.norm_eps;
    x.score_bound = c.score_bound;
    x.staging = c.staging;
    for (int a = 0; a < 3; a++) {
        x.zimage_dims[a] = (uint32_t)c.dims[a];
        x.zimage_base[a] = c.bases[a];
    }
    ZdrawHipQkOperands ops;
    memset(&ops, 0, sizeof(ops));
    ops.q_weight = c.q_norm;
    ops.k_weight = c.k_norm;
    ops.pos = c.pos;
    ops.rope_pairs = c.rope_pairs;
    return fromCode(zdraw_hip_run_attention_fused(ctx->queue, c.q, c.k, c.v, c.o, &p, &x, &ops));
}

} // namespace joint
} // namespace zdraw
