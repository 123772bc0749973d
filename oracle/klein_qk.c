/*
 * CPU oracle (test infrastructure, never linked into the product library):
 * Klein rope table, per-head RMSNorm and rope rotation, restating
 * klein/zflux2_dit.zig:102-228.
 */
#include "zdraw_oracle.h"

#include <math.h>

#define KLEIN_HEAD_DIM 128 /* klein/zflux2.zig:67 */

/* klein/zflux2_dit.zig:125-170. ids per token: text (0,0,0,t); image
 * (0, p/grid_w, p%grid_w, 0); reference image (10, p/ref_w, p%ref_w, 0).
 * Four axes of 32 dims: 16 frequencies each, computed in f64, cast to f32 and
 * written to both elements of the pair. */
void zo_klein_build_rope_ref(float* cos_out, float* sin_out,
                             size_t txt_len, size_t grid_h, size_t grid_w,
                             size_t ref_h, size_t ref_w, double theta) {
    const size_t img = grid_h * grid_w;
    const size_t tokens = txt_len + img + ref_h * ref_w;
    for (size_t t = 0; t < tokens; t++) {
        double ids[4] = {0, 0, 0, 0};
        if (t < txt_len) {
            ids[3] = (double)t;
        } else if (t < txt_len + img) {
            size_t p = t - txt_len;
            ids[1] = (double)(p / grid_w);
            ids[2] = (double)(p % grid_w);
        } else {
            size_t p = t - txt_len - img;
            ids[0] = 10;
            ids[1] = (double)(p / ref_w);
            ids[2] = (double)(p % ref_w);
        }
        for (size_t ax = 0; ax < 4; ax++) {
            for (size_t i = 0; i < 16; i++) {
                double exponent = (double)(2 * i) / 32.0;
                double freq = 1.0 / pow(theta, exponent);
                double arg = ids[ax] * freq;
                float c = (float)cos(arg);
                float s = (float)sin(arg);
                size_t base = t * KLEIN_HEAD_DIM + ax * 32 + 2 * i;
                cos_out[base] = c;
                cos_out[base + 1] = c;
                sin_out[base] = s;
                sin_out[base + 1] = s;
            }
        }
    }
}

/* klein/zflux2_dit.zig:203-211: f64 sum of squares, inv = 1/sqrt(ss/128+1e-6)
 * in f64, each element computed in f64 and cast to f32. */
void zo_klein_rms_norm_heads(float* x, const float* w, size_t tokens, size_t heads) {
    for (size_t th = 0; th < tokens * heads; th++) {
        float* row = x + th * KLEIN_HEAD_DIM;
        double ss = 0;
        for (size_t j = 0; j < KLEIN_HEAD_DIM; j++) ss += (double)row[j] * row[j];
        double inv = 1.0 / sqrt(ss / KLEIN_HEAD_DIM + 1e-6);
        for (size_t j = 0; j < KLEIN_HEAD_DIM; j++)
            row[j] = (float)((double)row[j] * inv * w[j]);
    }
}

/* klein/zflux2_dit.zig:213-228: adjacent-pair rotation in fp32, one table
 * row per token shared by all heads. */
void zo_klein_apply_rope(float* x, const float* cos_t, const float* sin_t,
                         size_t tokens, size_t heads) {
    for (size_t t = 0; t < tokens; t++) {
        for (size_t h = 0; h < heads; h++) {
            float* row = x + (t * heads + h) * KLEIN_HEAD_DIM;
            const float* c = cos_t + t * KLEIN_HEAD_DIM;
            const float* s = sin_t + t * KLEIN_HEAD_DIM;
            for (size_t i = 0; i < KLEIN_HEAD_DIM; i += 2) {
                float x0 = row[i];
                float x1 = row[i + 1];
                row[i] = x0 * c[i] - x1 * s[i];
                row[i + 1] = x1 * c[i + 1] + x0 * s[i + 1];
            }
        }
    }
}
