// Internal interface of the 16-bit MFMA GEMM that feeds and drains attention.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace zdraw {

// C[m][n] = A[m][k] x W[n][k]^T, fp32 accumulation, operands rounded to the
// weight's 16-bit type. Leading dimensions are in elements.
struct GemmArgs {
    const void* a;   // activations, row-major [m][lda]
    const void* w;   // weights, row-major [n][ldw]
    void* c;         // output, row-major [m][ldc]
    int32_t m, n, k;
    int32_t pad0;
    int64_t lda, ldw, ldc;
    int32_t tiles_n; // column tiles of one group (grid = tiles_m * tiles_n * groups)
    int32_t groups;  // 1..3 products sharing A and every dimension: group i > 0 uses w_more[i-1], c_more[i-1]
    const void* w_more[2];
    void* c_more[2];
    // Tiles of a partly filled last round, split along k (set by the caller from gemm_tail_plan;
    // splits <= 1: none). On entry tile_base holds the NUMBER of tail tiles; the launcher puts
    // the tail tiles, in `splits` parts each (fp32 partial tiles to `part`), at the head of the
    // one launch (part_wgs workgroups, a multiple of 8; ids past the last part return at once)
    // with the whole tiles behind them, which cover the parts' waits as they follow them onto
    // the CUs; then the kernel that adds the parts in part order and writes C.
    int32_t tile_base;
    int32_t splits;
    float* part;
    int32_t part_wgs; // set by the launcher
    int32_t pad1;
    // f32 activations: room for A rounded to the weight's type, [m][k] 16-bit (gemm_round_bytes
    // says how much; null: A is rounded block by block on its way into LDS instead)
    void* a16;
};

int gemm_tile_rows();
int gemm_tile_cols();
// a_dtype: kF32 or the weight's type; w_dtype: kF16 or kBF16; c_dtype: kF32 or the weight's type.
hipError_t launch_gemm(const GemmArgs& args, int a_dtype, int w_dtype, int c_dtype, hipStream_t stream);
hipError_t gemm_setup();
// How launch_gemm would split the last round of this product on a device with `cus` compute
// units: *tail_tiles tiles in *splits parts each (splits 1: no split), and the bytes of fp32
// partial tiles that needs.
void gemm_tail_plan(const GemmArgs& args, int a_dtype, int cus, int* tail_tiles, int* splits);
size_t gemm_part_bytes(int tail_tiles, int splits);
// Bytes of scratch launch_gemm wants for rounding f32 activations once, ahead of the product
// (0: not worth it or not possible for this shape).
size_t gemm_round_bytes(const GemmArgs& args, int a_dtype);
void gemm_set_build(int build); // 256-tiles of 16-bit activations: 1 = four-wave build (default), 0 = eight-wave build

} // namespace zdraw
