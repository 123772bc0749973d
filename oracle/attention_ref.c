/*
 * CPU oracle (test infrastructure, never linked into the product library):
 * scalar scaled dot-product attention restating runtime/attention.zig.
 *
 * Loop nest, arithmetic type (fp32) and summation order are the reference's:
 * token (outer) -> head -> score all keys -> 3-pass softmax -> mix.
 */
#include "zdraw_oracle.h"

#include <math.h>
#include <string.h>

/* runtime/attention.zig:94-98 (dot): ascending d, fp32 accumulator. */
static float dot(const float* a, const float* b, size_t n) {
    float sum = 0.0f;
    for (size_t i = 0; i < n; i++) sum += a[i] * b[i];
    return sum;
}

/* runtime/attention.zig:100-113 (qVec/outVec/kvVec): token-major
 * [tok][head][dim]. */
static size_t vec_start(size_t heads, size_t head_dim, size_t tok, size_t head) {
    return (tok * heads + head) * head_dim;
}

/* runtime/attention.zig:62-73 (score): key j gets dot(q, k_j) * scale, the
 * scale multiplied after the dot. `keys[j]` maps slot j to a key token
 * (identity in the reference; a compacted list for the masked extension). */
static void score(const float* qv, const float* k, float* out, size_t count,
                  const size_t* keys, const ZoAttnConfig* cfg, size_t kv_head, float scale) {
    for (size_t j = 0; j < count; j++) {
        size_t tok = keys ? keys[j] : j;
        out[j] = dot(qv, k + vec_start(cfg->kv_heads, cfg->head_dim, tok, kv_head), cfg->head_dim) * scale;
    }
}

/* runtime/attention.zig:75-85 (softmax): max from -inf, exp and sum in one
 * pass, divide in a third. */
static void softmax(float* values, size_t count) {
    float max = -INFINITY;
    for (size_t j = 0; j < count; j++) max = values[j] > max ? values[j] : max;
    float sum = 0.0f;
    for (size_t j = 0; j < count; j++) {
        values[j] = expf(values[j] - max);
        sum += values[j];
    }
    for (size_t j = 0; j < count; j++) values[j] /= sum;
}

/* runtime/attention.zig:87-93 (mix): zero, then ascending key accumulate. */
static void mix(float* out, const float* v, const float* weights, size_t count,
                const size_t* keys, const ZoAttnConfig* cfg, size_t kv_head) {
    memset(out, 0, cfg->head_dim * sizeof(float));
    for (size_t j = 0; j < count; j++) {
        size_t tok = keys ? keys[j] : j;
        const float* vv = v + vec_start(cfg->kv_heads, cfg->head_dim, tok, kv_head);
        for (size_t d = 0; d < cfg->head_dim; d++) out[d] += weights[j] * vv[d];
    }
}

/* runtime/attention.zig:45-60 (check). */
static int check(size_t out_len, size_t q_len, size_t k_len, size_t v_len,
                 size_t scratch_len, const ZoAttnConfig* cfg) {
    if (cfg->tokens == 0 || cfg->heads == 0 || cfg->kv_heads == 0) return ZO_INVALID_SHAPE;
    if (cfg->head_dim == 0 || cfg->heads % cfg->kv_heads != 0) return ZO_INVALID_SHAPE;
    size_t ql = cfg->tokens * cfg->heads * cfg->head_dim;
    size_t kvl = cfg->tokens * cfg->kv_heads * cfg->head_dim;
    if (out_len != ql || q_len != ql) return ZO_INVALID_SHAPE;
    if (k_len != kvl || v_len != kvl) return ZO_INVALID_SHAPE;
    if (scratch_len < cfg->tokens) return ZO_INVALID_SHAPE;
    return ZO_OK;
}

static int check_cfg_only(const ZoAttnConfig* cfg, size_t tok_begin, size_t tok_end) {
    if (cfg->tokens == 0 || cfg->heads == 0 || cfg->kv_heads == 0) return ZO_INVALID_SHAPE;
    if (cfg->head_dim == 0 || cfg->heads % cfg->kv_heads != 0) return ZO_INVALID_SHAPE;
    if (tok_begin > tok_end || tok_end > cfg->tokens) return ZO_INVALID_SHAPE;
    return ZO_OK;
}

/* runtime/attention.zig:21-43 (run), restricted to a token range. */
static void run_range(float* out, const float* q, const float* k, const float* v,
                      float* scratch, const ZoAttnConfig* cfg,
                      size_t tok_begin, size_t tok_end) {
    const float scale = 1.0f / sqrtf((float)cfg->head_dim);
    for (size_t tok = tok_begin; tok < tok_end; tok++) {
        size_t limit = cfg->causal ? tok + 1 : cfg->tokens;
        if (cfg->valid != 0 && limit > cfg->valid) limit = cfg->valid;
        for (size_t head = 0; head < cfg->heads; head++) {
            size_t kv_head = head * cfg->kv_heads / cfg->heads;
            size_t qs = vec_start(cfg->heads, cfg->head_dim, tok, head);
            score(q + qs, k, scratch, limit, NULL, cfg, kv_head, scale);
            softmax(scratch, limit);
            mix(out + qs, v, scratch, limit, NULL, cfg, kv_head);
        }
    }
}

int zo_attention_run(float* out, size_t out_len,
                     const float* q, size_t q_len,
                     const float* k, size_t k_len,
                     const float* v, size_t v_len,
                     float* scratch, size_t scratch_len,
                     const ZoAttnConfig* cfg) {
    int rc = check(out_len, q_len, k_len, v_len, scratch_len, cfg);
    if (rc != ZO_OK) return rc;
    run_range(out, q, k, v, scratch, cfg, 0, cfg->tokens);
    return ZO_OK;
}

int zo_attention_rows(float* out, const float* q, const float* k, const float* v,
                      float* scratch, const ZoAttnConfig* cfg,
                      size_t tok_begin, size_t tok_end) {
    int rc = check_cfg_only(cfg, tok_begin, tok_end);
    if (rc != ZO_OK) return rc;
    run_range(out, q, k, v, scratch, cfg, tok_begin, tok_end);
    return ZO_OK;
}

/* EXTENSION. scratch must hold 2*tokens floats worth of storage when a mask
 * is given: the first `tokens` floats are the scores, the key list lives in
 * a size_t array carved from the caller's second region (see below). To keep
 * the ABI simple the key list is built in a local heap-free way: two passes
 * over key_pad. */
int zo_attention_rows_masked(float* out, const float* q, const float* k, const float* v,
                             float* scratch, const ZoAttnConfig* cfg,
                             const uint8_t* key_pad,
                             size_t tok_begin, size_t tok_end) {
    int rc = check_cfg_only(cfg, tok_begin, tok_end);
    if (rc != ZO_OK) return rc;
    if (!key_pad) {
        run_range(out, q, k, v, scratch, cfg, tok_begin, tok_end);
        return ZO_OK;
    }
    /* The masked extension is defined for the bidirectional DiT call only. */
    if (cfg->causal) return ZO_INVALID_SHAPE;
    size_t limit_all = cfg->tokens;
    if (cfg->valid != 0 && limit_all > cfg->valid) limit_all = cfg->valid;
    /* Key list stored after the score region: caller provides
     * scratch of at least tokens floats + tokens size_t (documented in the
     * Python loader, which allocates it). */
    size_t* keys = (size_t*)(void*)(scratch + ((cfg->tokens + 1) & ~(size_t)1));
    size_t count = 0;
    for (size_t j = 0; j < limit_all; j++)
        if (!key_pad[j]) keys[count++] = j;
    const float scale = 1.0f / sqrtf((float)cfg->head_dim);
    for (size_t tok = tok_begin; tok < tok_end; tok++) {
        for (size_t head = 0; head < cfg->heads; head++) {
            size_t kv_head = head * cfg->kv_heads / cfg->heads;
            size_t qs = vec_start(cfg->heads, cfg->head_dim, tok, head);
            score(q + qs, k, scratch, count, keys, cfg, kv_head, scale);
            softmax(scratch, count);
            mix(out + qs, v, scratch, count, keys, cfg, kv_head);
        }
    }
    return ZO_OK;
}
