/*
 * CPU oracle, part 4: the dense projection either side of attention.
 * TEST INFRASTRUCTURE ONLY (see zdraw_oracle.h).
 *
 * Restates the reference's scalar linear kernel, runtime/ops.zig:37-60
 * (linearView): out[row] = sum over col, in column order, of
 * input[col] * weight[row][col], accumulated in fp32, plus bias[row].
 * The batched form applies it to `count` input rows (metal/mgemm.zig:134-155,
 * runtime/linear_fast.zig:31-45): out is [count][rows], input [count][cols].
 * The weight arrives decoded to fp32: f16 and bf16 decode exactly
 * (zo_read_f32), so this is the reference's weight.atF32Unchecked().
 */
#include "zdraw_oracle.h"

int zo_linear_batch(float *out, size_t out_len, const float *input, size_t input_len, const float *weight,
                    size_t weight_len, const float *bias, size_t rows, size_t cols, size_t count) {
    /* ops.zig:43-49, mgemm.zig:141-145 */
    if (rows == 0 || cols == 0 || count == 0) return ZO_INVALID_SHAPE;
    if (weight_len != rows * cols) return ZO_INVALID_SHAPE;
    if (out_len != rows * count || input_len != cols * count) return ZO_INVALID_SHAPE;
    for (size_t item = 0; item < count; item++) {
        const float *x = input + item * cols;
        float *y = out + item * rows;
        for (size_t row = 0; row < rows; row++) { /* ops.zig:51-59 */
            float sum = 0.0f;
            const float *w = weight + row * cols;
            for (size_t col = 0; col < cols; col++) sum += x[col] * w[col];
            y[row] = sum;
            if (bias) y[row] += bias[row];
        }
    }
    return ZO_OK;
}
