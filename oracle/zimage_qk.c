/*
 * CPU oracle (test infrastructure, never linked into the product library):
 * Z-Image complex-pair rope cache, RMSNorm, sequence/position helpers and
 * the f16/bf16 weight decode, restating zimage/zrope.zig, runtime/ops.zig,
 * zimage/zattn.zig, zimage/zseq.zig, zimage/zunify.zig, pack/tensor.zig.
 */
#include "zdraw_oracle.h"

#include <math.h>
#include <string.h>

/* zimage/zrope.zig:134-136 */
static size_t pair_count(size_t dim) { return dim / 2; }

/* zimage/zrope.zig:82-87 */
int zo_zrope_check(const ZoRopeConfig* cfg) {
    if (cfg->theta <= 0.0f) return ZO_INVALID_CONFIG;
    for (int a = 0; a < 3; a++) {
        if (cfg->dims[a] == 0 || cfg->lens[a] == 0 || cfg->dims[a] % 2 != 0)
            return ZO_INVALID_CONFIG;
    }
    return ZO_OK;
}

/* zimage/zrope.zig:118-122 */
size_t zo_zrope_count(const ZoRopeConfig* cfg) {
    size_t total = 0;
    for (int a = 0; a < 3; a++) total += cfg->lens[a] * pair_count(cfg->dims[a]);
    return total;
}

/* zimage/zrope.zig:124-128 */
size_t zo_zrope_axis_base(const ZoRopeConfig* cfg, size_t axis) {
    size_t base = 0;
    for (size_t a = 0; a < axis; a++) base += cfg->lens[a] * pair_count(cfg->dims[a]);
    return base;
}

/* zimage/zrope.zig:138-140 (power): 2*pair/dim in fp32. */
static float power(size_t pair, size_t dim) {
    return 2.0f * (float)pair / (float)dim;
}

/* zimage/zrope.zig:97-106 (fillAxis): angle = pos * exp(-ln(theta) * power),
 * all fp32; entry = (cos, sin). */
static void fill_axis(float* values, size_t n_pairs_total, size_t dim, float theta) {
    size_t pairs = pair_count(dim);
    for (size_t pos = 0; pos < n_pairs_total / pairs; pos++) {
        float fpos = (float)pos;
        for (size_t pair = 0; pair < pairs; pair++) {
            float freq = fpos * expf(-logf(theta) * power(pair, dim));
            values[2 * (pos * pairs + pair)] = cosf(freq);
            values[2 * (pos * pairs + pair) + 1] = sinf(freq);
        }
    }
}

/* zimage/zrope.zig:89-95 (fill) */
void zo_zrope_fill(float* values, const ZoRopeConfig* cfg) {
    size_t off = 0;
    for (int a = 0; a < 3; a++) {
        size_t n = cfg->lens[a] * pair_count(cfg->dims[a]);
        fill_axis(values + 2 * off, n, cfg->dims[a], cfg->theta);
        off += n;
    }
}

/* zimage/zrope.zig:108-116 (applyAxis) */
static void apply_axis(float* vec, const float* pairs, size_t n_pairs) {
    for (size_t pair = 0; pair < n_pairs; pair++) {
        float c = pairs[2 * pair];
        float s = pairs[2 * pair + 1];
        size_t i = pair * 2;
        float a = vec[i];
        float b = vec[i + 1];
        vec[i] = a * c - b * s;
        vec[i + 1] = b * c + a * s;
    }
}

/* zimage/zrope.zig:44-55 (apply), :76-80 (axis) */
int zo_zrope_apply(const float* values, const ZoRopeConfig* cfg,
                   float* vec, size_t vec_len, const size_t pos[3]) {
    if (vec_len != cfg->dims[0] + cfg->dims[1] + cfg->dims[2]) return ZO_INVALID_SHAPE;
    size_t vpos = 0;
    for (size_t ax = 0; ax < 3; ax++) {
        if (pos[ax] >= cfg->lens[ax]) return ZO_BAD_POSITION;
        size_t dim = cfg->dims[ax];
        size_t pairs = pair_count(dim);
        size_t base = zo_zrope_axis_base(cfg, ax) + pos[ax] * pairs;
        apply_axis(vec + vpos, values + 2 * base, pairs);
        vpos += dim;
    }
    return ZO_OK;
}

/* runtime/ops.zig:62-79 (rmsNorm): fp32 sum in ascending order,
 * scale = 1/sqrt(mean + eps), out = value * scale * gain (left to right). */
int zo_rms_norm(float* out, const float* in, const float* w, size_t n, float eps) {
    if (n == 0) return ZO_INVALID_SHAPE;
    float mean = 0.0f;
    for (size_t i = 0; i < n; i++) mean += in[i] * in[i];
    float count = (float)n;
    float scale = 1.0f / sqrtf(mean / count + eps);
    for (size_t i = 0; i < n; i++) out[i] = in[i] * scale * w[i];
    return ZO_OK;
}

/* zimage/zattn.zig:140-151 (normHeads): norm into a temporary, copy back. */
int zo_zimage_norm_heads(float* data, const float* w, size_t tokens, size_t heads,
                         size_t head_dim, float eps) {
    float buf[1024];
    if (head_dim == 0 || head_dim > 1024) return ZO_INVALID_SHAPE;
    for (size_t tok = 0; tok < tokens; tok++) {
        for (size_t head = 0; head < heads; head++) {
            float* vec = data + (tok * heads + head) * head_dim;
            int rc = zo_rms_norm(buf, vec, w, head_dim, eps);
            if (rc != ZO_OK) return rc;
            memcpy(vec, buf, head_dim * sizeof(float));
        }
    }
    return ZO_OK;
}

/* zimage/zattn.zig:153-164 (rotate) */
int zo_zimage_rotate(float* data, const float* values, const ZoRopeConfig* cfg,
                     const size_t* pos, size_t tokens, size_t heads) {
    size_t head_dim = cfg->dims[0] + cfg->dims[1] + cfg->dims[2];
    for (size_t tok = 0; tok < tokens; tok++) {
        for (size_t head = 0; head < heads; head++) {
            int rc = zo_zrope_apply(values, cfg, data + (tok * heads + head) * head_dim,
                                    head_dim, pos + tok * 3);
            if (rc != ZO_OK) return rc;
        }
    }
    return ZO_OK;
}

/* zimage/zseq.zig:9,15-21 */
#define ZSEQ_MULTI 32
size_t zo_zseq_pad_len(size_t len) { return (ZSEQ_MULTI - len % ZSEQ_MULTI) % ZSEQ_MULTI; }
size_t zo_zseq_padded_len(size_t len) { return len + zo_zseq_pad_len(len); }

static size_t grid_len(const size_t size[3]) { return size[0] * size[1] * size[2]; }

/* zimage/zseq.zig:23-34 (grid): frame, row, column order. */
int zo_zseq_grid(size_t* out, size_t out_len, const size_t size[3], const size_t start[3]) {
    if (out_len != grid_len(size)) return ZO_INVALID_SHAPE;
    size_t p = 0;
    for (size_t f = 0; f < size[0]; f++)
        for (size_t h = 0; h < size[1]; h++)
            for (size_t w = 0; w < size[2]; w++) {
                out[3 * p + 0] = start[0] + f;
                out[3 * p + 1] = start[1] + h;
                out[3 * p + 2] = start[2] + w;
                p++;
            }
    return ZO_OK;
}

/* zimage/zseq.zig:36-71 (padWithIds) */
int zo_zseq_pad_with_ids(float* out, size_t out_len, size_t* pos_ids, size_t pos_len,
                         uint8_t* mask, size_t mask_len,
                         const float* feat, size_t feat_len, size_t dim,
                         const size_t size[3], const size_t start[3], size_t* total_out) {
    if (dim == 0) return ZO_INVALID_SHAPE;
    size_t span = grid_len(size);
    size_t total = zo_zseq_padded_len(span);
    if (span == 0 || feat_len % dim != 0) return ZO_INVALID_SHAPE;
    size_t real = feat_len / dim;
    if (real == 0 || real > total) return ZO_INVALID_SHAPE;
    if (out_len != total * dim || pos_len != total || mask_len != total) return ZO_INVALID_SHAPE;
    int rc = zo_zseq_grid(pos_ids, span, size, start);
    if (rc != ZO_OK) return rc;
    for (size_t t = span; t < total; t++) pos_ids[3 * t] = pos_ids[3 * t + 1] = pos_ids[3 * t + 2] = 0;
    memcpy(out, feat, real * dim * sizeof(float));
    const float* last = feat + (real - 1) * dim;
    for (size_t t = real; t < total; t++) memcpy(out + t * dim, last, dim * sizeof(float));
    for (size_t t = 0; t < real; t++) mask[t] = 0;
    for (size_t t = real; t < total; t++) mask[t] = 1;
    *total_out = total;
    return ZO_OK;
}

/* zimage/zunify.zig:16-37 (basic) */
int zo_zunify_basic(float* out, size_t out_len, size_t* pos_out, size_t pos_out_len,
                    const float* image, size_t image_len, const size_t* image_pos, size_t image_pos_len,
                    const float* cap, size_t cap_len, const size_t* cap_pos, size_t cap_pos_len,
                    size_t hidden) {
    if (hidden == 0) return ZO_INVALID_SHAPE;
    if (image_pos_len * hidden != image_len) return ZO_INVALID_SHAPE;
    if (cap_pos_len * hidden != cap_len) return ZO_INVALID_SHAPE;
    size_t total = image_pos_len + cap_pos_len;
    if (out_len != total * hidden || pos_out_len != total) return ZO_INVALID_SHAPE;
    memcpy(out, image, image_len * sizeof(float));
    memcpy(out + image_len, cap, cap_len * sizeof(float));
    memcpy(pos_out, image_pos, image_pos_len * 3 * sizeof(size_t));
    memcpy(pos_out + image_pos_len * 3, cap_pos, cap_pos_len * 3 * sizeof(size_t));
    return ZO_OK;
}

/* pack/tensor.zig:125-147 (fromBits): IEEE half decode via sign, exponent,
 * mantissa with ldexp; subnormals, inf and nan handled as the reference does. */
static float from_bits(uint32_t bits, unsigned exp_bits, unsigned mant_bits, int bias) {
    uint32_t sign_mask = 1u << (exp_bits + mant_bits);
    uint32_t exp_mask = (1u << exp_bits) - 1;
    uint32_t mant_mask = (1u << mant_bits) - 1;
    uint32_t exp_raw = (bits >> mant_bits) & exp_mask;
    uint32_t mant = bits & mant_mask;
    float sign = (bits & sign_mask) == 0 ? 1.0f : -1.0f;
    float fr = (float)mant / (float)(1u << mant_bits);
    if (exp_raw == exp_mask) {
        if (mant != 0) return NAN;
        return sign * INFINITY;
    }
    if (exp_raw == 0) {
        if (mant == 0) return sign * 0.0f;
        return sign * ldexpf(fr, 1 - bias);
    }
    return sign * ldexpf(1.0f + fr, (int)exp_raw - bias);
}

/* pack/tensor.zig:108-115 (readF32), little-endian. */
float zo_read_f32(int dtype, const uint8_t* bytes) {
    switch (dtype) {
    case 0: {
        uint32_t b = (uint32_t)bytes[0] | ((uint32_t)bytes[1] << 8) |
                     ((uint32_t)bytes[2] << 16) | ((uint32_t)bytes[3] << 24);
        float f;
        memcpy(&f, &b, 4);
        return f;
    }
    case 1:
        return from_bits((uint32_t)bytes[0] | ((uint32_t)bytes[1] << 8), 5, 10, 15);
    case 2: {
        uint32_t b = ((uint32_t)bytes[0] | ((uint32_t)bytes[1] << 8)) << 16;
        float f;
        memcpy(&f, &b, 4);
        return f;
    }
    default:
        return (float)bytes[0];
    }
}
