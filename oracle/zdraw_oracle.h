/*
 * CPU oracle for zdraw's DiT joint-attention path.
 *
 * TEST INFRASTRUCTURE ONLY. This is a plain-C restatement of the reference's
 * scalar CPU algorithm, used as the checker in tests, in the smoke check and
 * as the timed CPU baseline of the benchmark. The product library
 * (libzdraw_hip.so) never links, loads or calls anything in this directory.
 *
 * Every function cites the reference file:line it restates (paths relative to
 * the reference tree). Arithmetic type, evaluation order and rounding points
 * follow the reference: fp32 everywhere except where the reference itself
 * uses f64 (the Klein rope table and the Klein head RMS sum).
 *
 * Two entry points are extensions that the reference does not have; both are
 * restrictions/loops of reference math and are marked EXTENSION below:
 *   - zo_attention_rows_masked: a boolean key-padding mask (a masked key is
 *     dropped from the key set; a suffix mask equals Config.valid);
 *   - callers loop zo_attention_* over batch segments (no function needed).
 *
 * Parity pinning status (what checks each function beyond retyping it):
 *   zo_attention_run / rows       pinned: reference known-answer tests
 *                                 (attention.zig:115-156, mattn_test.zig:15-31),
 *                                 fp64 brute force, torch CPU SDPA, invariants.
 *   zo_attention_rows_masked      pinned: equals deletion of masked keys
 *                                 (bit-exact), suffix mask equals `valid`.
 *   zo_klein_build_rope_ref       pinned: closed forms + structural identities.
 *   zo_klein_rms_norm_heads       pinned: ops.zig:151-163 vector, invariants.
 *   zo_klein_apply_rope           pinned: rotation identities (norm, compose,
 *                                 relative-position property).
 *   zo_zrope_*                    pinned: zrope.zig:142-180 known answers.
 *   zo_rms_norm                   pinned: ops.zig:151-163 vector.
 *   zo_zseq_*, zo_zunify_basic    pinned: zseq.zig:94-133, zunify.zig:47-66.
 *   zo_read_f32 (f16/bf16 decode) pinned: ops.zig:137-174 byte vectors and
 *                                 numpy's float16 / bit-shifted bf16 decode.
 *   zo_linear_batch               pinned: mlinear_test.zig:33-80 known answers,
 *                                 the bf16 case of mlinear_test.zig:82-121,
 *                                 numpy float64 matmul, linearity.
 */
#ifndef ZDRAW_ORACLE_H
#define ZDRAW_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Error codes (reference: `error.InvalidShape` etc.). */
enum {
    ZO_OK = 0,
    ZO_INVALID_SHAPE = 1,   /* attention.zig:5-7, zrope.zig:17-21, zseq.zig:11-13 */
    ZO_INVALID_CONFIG = 2,  /* zrope.zig:18 */
    ZO_BAD_POSITION = 3     /* zrope.zig:20 */
};

/* runtime/attention.zig:9-19 */
typedef struct ZoAttnConfig {
    size_t tokens;
    size_t heads;
    size_t kv_heads;
    size_t head_dim;
    int causal;
    size_t valid; /* 0 = no right-padding limit */
} ZoAttnConfig;

/* runtime/attention.zig:21-43 (run) with :45-60 (check). Lengths are element
 * counts of the caller's slices, checked exactly as the reference does. */
int zo_attention_run(float* out, size_t out_len,
                     const float* q, size_t q_len,
                     const float* k, size_t k_len,
                     const float* v, size_t v_len,
                     float* scratch, size_t scratch_len,
                     const ZoAttnConfig* cfg);

/* Same loops, restricted to query tokens [tok_begin, tok_end): rows of the
 * reference's outer loop are independent, so this is the reference's result
 * for those rows. Used to check samples of full-size workloads. */
int zo_attention_rows(float* out, const float* q, const float* k, const float* v,
                      float* scratch, const ZoAttnConfig* cfg,
                      size_t tok_begin, size_t tok_end);

/* EXTENSION (not in the reference): key_pad[j] != 0 removes key j for every
 * query. Implemented as the reference's score/softmax/mix over the surviving
 * keys in ascending order. key_pad may be NULL. */
int zo_attention_rows_masked(float* out, const float* q, const float* k, const float* v,
                             float* scratch, const ZoAttnConfig* cfg,
                             const uint8_t* key_pad,
                             size_t tok_begin, size_t tok_end);

/* klein/zflux2_dit.zig:125-170 (buildRopeRef); txt_len is zflux2.zig:68 (512
 * in the reference, a parameter here so tests can use small cases).
 * cos/sin: [txt_len + grid_h*grid_w + ref_h*ref_w][128]. */
void zo_klein_build_rope_ref(float* cos_out, float* sin_out,
                             size_t txt_len, size_t grid_h, size_t grid_w,
                             size_t ref_h, size_t ref_w, double theta);

/* klein/zflux2_dit.zig:203-211 (rmsNormHeads): in place, f64 sum, eps 1e-6,
 * head_dim 128, w = 128 f32 weights. */
void zo_klein_rms_norm_heads(float* x, const float* w, size_t tokens, size_t heads);

/* klein/zflux2_dit.zig:213-228 (applyRope): in place, head_dim 128. */
void zo_klein_apply_rope(float* x, const float* cos_t, const float* sin_t,
                         size_t tokens, size_t heads);

/* zimage/zrope.zig:11-15 */
typedef struct ZoRopeConfig {
    size_t dims[3];
    size_t lens[3];
    float theta;
} ZoRopeConfig;

/* zimage/zrope.zig:82-87 (checkConfig) */
int zo_zrope_check(const ZoRopeConfig* cfg);
/* zimage/zrope.zig:118-122 (count): number of (cos,sin) pairs in the cache. */
size_t zo_zrope_count(const ZoRopeConfig* cfg);
/* zimage/zrope.zig:124-128 (axisBase) */
size_t zo_zrope_axis_base(const ZoRopeConfig* cfg, size_t axis);
/* zimage/zrope.zig:89-106 (fill, fillAxis): values = count() x {cos, sin}. */
void zo_zrope_fill(float* values, const ZoRopeConfig* cfg);
/* zimage/zrope.zig:44-55,108-116 (apply, applyAxis) on one head vector. */
int zo_zrope_apply(const float* values, const ZoRopeConfig* cfg,
                   float* vec, size_t vec_len, const size_t pos[3]);

/* runtime/ops.zig:62-79 (rmsNorm; rmsNormView :81-101 is the same arithmetic
 * with the weight decoded to f32 first). */
int zo_rms_norm(float* out, const float* in, const float* w, size_t n, float eps);

/* zimage/zattn.zig:140-151 (normHeads): every head vector, in place. */
int zo_zimage_norm_heads(float* data, const float* w, size_t tokens, size_t heads,
                         size_t head_dim, float eps);
/* zimage/zattn.zig:153-164 (rotate): pos = [tokens][3]. */
int zo_zimage_rotate(float* data, const float* values, const ZoRopeConfig* cfg,
                     const size_t* pos, size_t tokens, size_t heads);

/* zimage/zseq.zig:15-21 */
size_t zo_zseq_pad_len(size_t len);
size_t zo_zseq_padded_len(size_t len);
/* zimage/zseq.zig:23-34 (grid): out = [size0*size1*size2][3]. */
int zo_zseq_grid(size_t* out, size_t out_len, const size_t size[3], const size_t start[3]);
/* zimage/zseq.zig:36-71 (padWithIds). mask: 1 = pad slot. Returns total via *total_out. */
int zo_zseq_pad_with_ids(float* out, size_t out_len, size_t* pos_ids, size_t pos_len,
                         uint8_t* mask, size_t mask_len,
                         const float* feat, size_t feat_len, size_t dim,
                         const size_t size[3], const size_t start[3], size_t* total_out);
/* zimage/zunify.zig:16-37 (basic): image tokens then caption tokens. */
int zo_zunify_basic(float* out, size_t out_len, size_t* pos_out, size_t pos_out_len,
                    const float* image, size_t image_len, const size_t* image_pos, size_t image_pos_len,
                    const float* cap, size_t cap_len, const size_t* cap_pos, size_t cap_pos_len,
                    size_t hidden);

/* pack/tensor.zig:108-147 (readF32 / fromBits): dtype 0=f32, 1=f16, 2=bf16, 3=u8. */
float zo_read_f32(int dtype, const uint8_t* bytes);

/* ---- dense projection (runtime/ops.zig:37-60, metal/mgemm.zig:134-155) -------
 * out [count][rows] = input [count][cols] x weight[rows][cols]^T (+ bias[rows]),
 * fp32, columns accumulated in order. bias may be NULL. */
int zo_linear_batch(float *out, size_t out_len, const float *input, size_t input_len, const float *weight,
                    size_t weight_len, const float *bias, size_t rows, size_t cols, size_t count);

#ifdef __cplusplus
}
#endif
#endif
