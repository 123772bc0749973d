// Internal launch interface between the C-ABI bridge and the gfx950 kernels.
// Not part of the public ABI (that is include/zdraw_hip.h).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace zdraw {

constexpr int kHeadDim = 128;      // the only head width the MFMA kernel is built for

enum QkMode : int {
    kQkNone = 0,   // operands are used as given
    kQkKlein = 1,  // RMSNorm(eps, learned weight) then table rope (cos/sin [rows][128])
    kQkZimage = 2, // RMSNorm then 3-axis complex-pair rope from pos[rows][3] and a pair table
};

enum DType : int { kF32 = 0, kF16 = 1, kBF16 = 2 };

// Side operands of the QK-norm + rope step, shared by the attention kernel
// and the standalone pre-pass.
struct QkOps {
    // Klein rope table rows, [rows][128] f32; row = segment * rope_bs + token
    const float* rope_cos;
    const float* rope_sin;
    // Z-Image: positions u64[rows][3] and (cos,sin) pair table
    const unsigned long long* pos;
    const float* pairs;
    int64_t rope_bs;    // table / position rows between segments (0 = shared)
    uint32_t base0, base1, base2; // Z-Image axis bases in pairs
    int32_t dim0, dim1, dim2;     // Z-Image axis widths
    // Z-Image: positions the pair table holds per axis (>= 1); a position at or past its
    // axis's count reads the axis's last entry, so no position can index outside the table
    uint32_t len0, len1, len2;
    int32_t txt_rows;   // tokens < txt_rows use the *_txt weights when given
    float eps;
};

// Everything one attention launch needs, passed by value as the kernel argument.
// Strides are in elements; the head_dim axis is contiguous.
struct AttnArgs {
    const void* q;
    const void* k;
    const void* v;
    void* o;
    int64_t q_bs, q_ts, q_hs;
    int64_t k_bs, k_ts, k_hs;
    int64_t v_bs, v_ts, v_hs;
    int64_t o_bs, o_ts, o_hs;
    int32_t tokens;     // S: queries and keys per segment
    int32_t heads;      // H
    int32_t batch;      // independent segments
    int32_t key_limit;  // keys >= key_limit are excluded (min(S, valid))
    int32_t nqb;        // query blocks per (segment, head)
    int32_t q_mode;     // QkMode applied to Q rows at load
    int32_t out_dtype;  // kF32, kF16 or kBF16
    float scale_log2;   // log2(e) / sqrt(head_dim)
    int32_t bounded;    // 1: scaled scores are known to fit the fp32 exponent with room to spare
    int32_t score_f16;  // 1: q and k hold IEEE half (prepared operands only): S = K Q^T runs on the f16 MFMA; v stays bf16
    QkOps qk;
    // QK-norm weights (f32[128]); *_txt used for tokens < qk.txt_rows when non-null
    const float* q_w;
    const float* k_w;
    const float* q_w_txt;
    const float* k_w_txt;
    // key-padding mask, u8 [segment][tokens], nonzero = key excluded; may be null
    const unsigned char* key_pad;
    int64_t mask_bs;    // bytes between segments (0 = shared)
    // clock probe (null = off): workgroup i stores its run time as shader-clock
    // cycles at [2i] and as ticks of the fixed 100 MHz reference at [2i+1], i < clock_cap
    unsigned long long* clock_probe;
    int64_t clock_cap;
    // One launch holds the tiles of the last, thinly filled round in parts (splits > 1) and the
    // whole tiles behind them: workgroups below part_wgs are parts, id = (tile - tile_base) *
    // splits + z (ids from (tiles - tile_base) * splits up to part_wgs are padding and return at
    // once); part z walks the z-th share of the tile's key-block list and writes its
    // unnormalised O^T rows, reference point and denominator, and attn_merge_kernel combines
    // them in z order. Workgroups from part_wgs on take the whole tiles 0 .. tile_base - 1. The
    // parts come first: they are short and mostly wait on memory, which the whole tiles that
    // follow them onto the CUs cover.
    int32_t tile_base;  // first logical tile (segment, head, query block) that is split
    int32_t splits;     // 0 or 1 = none
    int32_t part_wgs;   // workgroups at the head of the grid that are parts (a multiple of 8), or 0
    int32_t pad2;
    float* part_o;      // f32 [tile - tile_base][splits][block rows][128]
    float* part_ml;     // f32 [tile - tile_base][splits][block rows][2]
};

// Standalone norm + rope over rows of one operand (Q or K): the pre-pass for
// K and the in-place qk_norm_rope entry. Output may alias the input.
struct PrepArgs {
    const void* x;
    void* y;
    int64_t x_bs, x_ts, x_hs;
    int64_t y_bs, y_ts, y_hs;
    int32_t tokens, heads, batch;
    int32_t mode;       // QkMode; kQkNone = the rows are only rounded and re-laid (V beside a prepared Q and K)
    int32_t out_dtype;  // kF32, kF16 or kBF16 (per operand: a launch may write Q and K as f16 and V as bf16)
    float scale;        // multiplies the result (1 for K; log2(e)/sqrt(head_dim) when Q is prepared for attention)
    QkOps qk;
    const void* w;      // 128 norm weights, element type w_dtype
    const void* w_txt;
    int32_t w_dtype;    // kF32, kF16 or kBF16
    int32_t pad0;
};

struct PrepPair {
    PrepArgs op[3]; // Q, K and, when the launch has a third operand, rows that are only rounded (mode kQkNone)
    int32_t count;
    int32_t pad0;
};

// Norm weights that the pre-pass cannot take as they lie (two element types, or off a
// 16-byte boundary): 128 weights of Q and of K, each of its own type (kF32, kF16, kBF16)
// at an element-aligned address, copied as f32 to out[0..127] and out[128..255].
struct WeightStageArgs {
    const void* q;
    const void* k;
    float* out;
    int32_t q_dtype, k_dtype;
};
hipError_t launch_weight_stage(const WeightStageArgs& args, hipStream_t stream);

// Kernel shape: 0 = 8 waves x 32 query rows (one workgroup per CU, 8-stage LDS
// ring), 1 = 4 waves x 32 query rows (two workgroups per CU, 4-stage rings).
int attention_block_rows(int shape);
int attention_key_block();
int attention_max_tokens();
// One wide head (heads = 1, head_dim = 512), dense token-major rows.
struct WideArgs {
    const void* q; // bf16 [tokens][512], already multiplied by log2(e)/sqrt(512)
    const void* k; // bf16 [tokens][512]
    const void* v; // bf16 [tokens][512]
    float* o;      // f32 [tokens][512]
    int32_t tokens; // multiple of 64
    int32_t splits; // key ranges per query tile (wide_splits; 0 or 1: none); > 1 needs the two buffers below
    float* part_o;  // f32 [splits][tokens][512]: unnormalised O of each key range
    float* part_ml; // f32 [splits][tokens][2]: its reference point and row sum
    int* redo;      // [wide_tiles(tokens)]: set by the kernel for a query tile (128 rows) whose scores outgrew the
                    // fixed reference point; such tiles are formed again by the running-maximum kernel that follows
};
// f32 -> bf16 rounding of the three operands (Q with its scale) in one launch.
struct WidePrepArgs {
    const float* q; const float* k; const float* v;
    void* qo; void* ko; void* vo;
    int64_t chunks; // 8-element chunks per operand
    float q_scale;
    int32_t redo_tiles; // entries of redo that the launch clears
    int* redo;
};
int wide_head_dim();
int wide_block_rows();
// Key ranges per query tile that fill a device of `cus` compute units (1: no split), and the
// bytes of part_o followed by part_ml they need.
int wide_splits(int tokens, int cus);
int wide_tiles(int tokens); // query tiles (128 rows) = entries of WideArgs::redo
size_t wide_part_bytes(int tokens, int splits);
hipError_t launch_wide_round(const WidePrepArgs& args, hipStream_t stream);
hipError_t launch_wide_attention(const WideArgs& args, hipStream_t stream);
hipError_t wide_setup();

// Launch one attention forward. in_dtype is kF32 or kBF16; k_mode is the
// QkMode applied to K rows inside the K-block load. Returns a hipError_t.
hipError_t launch_attention(const AttnArgs& args, int in_dtype, int k_mode, int shape, hipStream_t stream);
// Tail plan for a launch of `tiles` workgroup tiles on `cus` compute units: how many tiles of
// the last, partly filled round are better split along the keys, and into how many parts
// (0 tiles = run everything whole). key_blocks = 32-key blocks per tile.
void attention_tail_plan(int64_t tiles, int cus, int key_blocks, int* tail_tiles, int* splits);
// Bytes of part_o and part_ml that `tail_tiles` x `splits` need for the kernel shape.
size_t attention_part_o_bytes(int tail_tiles, int splits, int shape);
size_t attention_part_ml_bytes(int tail_tiles, int splits, int shape);
// Normalise + rotate `count` (1 or 2) operands of equal shape in one launch.
hipError_t launch_qk_prepass(const PrepArgs* ops, int count, int in_dtype, hipStream_t stream);
// One-time per-device setup (raises the dynamic LDS limit on every instantiation).
hipError_t attention_setup();

} // namespace zdraw
