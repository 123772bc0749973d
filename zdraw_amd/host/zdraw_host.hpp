// Host layer above the C ABI: the C++ counterpart of the reference's Zig
// operator interface for the attention path. Names, argument meaning and
// error behaviour follow the reference so that call sites and tests read the
// same:
//   attention::Config          runtime/attention.zig:9-19
//   attention_fast::run        runtime/attention_fast.zig:6-24
//   hattn::Context             metal/mattn.zig:47-276 (Context, Kernel, Pick)
//   hqk::run / hqk::Config     metal/mqk.zig:12-60
//   joint::Klein / joint::Zimage  the rmsRopeHm + runAttnHm sequences of
//                              klein/zflux2_resident.zig:1515-1571, 1956-2063
//                              and qk-norm + attention of metal/mres.zig:47-80
// Zig error unions become the Error enum; `Ok` is success.
#pragma once

#include <cstddef>
#include <cstdint>

#include "zdraw_hip.h"

namespace zdraw {

enum class Error : int {
    Ok = 0,
    UnsupportedShape = 1,  // error.UnsupportedShape: the caller falls back to its CPU kernel
    InvalidShape = 2,      // error.InvalidShape
    NotAvailable = 3,      // error.MetalNotAvailable: no gfx950 device
    QueueFailed = 4,       // error.MetalQueueFailed
    CompileFailed = 5,     // error.MetalCompileFailed
    DispatchFailed = 6,    // error.MetalDispatchFailed
    BadPosition = 7,       // zrope error.BadPosition
    OutOfMemory = 8,
};

namespace attention {
// runtime/attention.zig:9-19
struct Config {
    size_t tokens;
    size_t heads;
    size_t kv_heads;
    size_t head_dim;
    bool causal;
    size_t valid = 0;
};
// Signature of the caller's CPU kernel (runtime/attention.zig:21-28). This
// library ships none: zdraw keeps its own attention.run, and tests pass the
// oracle's.
using CpuRun = int (*)(float* out, size_t out_len, const float* q, size_t q_len, const float* k, size_t k_len,
                       const float* v, size_t v_len, float* scratch, size_t scratch_len, const Config* cfg,
                       void* user);
} // namespace attention

namespace hattn {

constexpr size_t max_tokens = 32768;    // key-block list capacity of the kernel (mattn.zig:15 is 6144 for `rows`)
constexpr size_t flash_head_dim = 128;  // mattn.zig:16
constexpr size_t wide_head_dim = 512;   // mattn.zig:17

// mattn.zig:19. Only `block` (the bf16-MFMA flash kernel) exists on gfx950.
enum class Kernel : uint32_t { rows = 0, flash = 1, block = 2, wide = 3 };

struct Pick {
    Kernel kernel;
    void* pipeline;
    size_t threads;
};

// A device buffer with the reference's owned/borrowed tag (metal/mbuffer.zig:140-186).
struct Buffer {
    void* handle = nullptr;
    bool owned = false;
    static Buffer fromBytes(void* device, const void* data, size_t size);
    static Buffer empty(void* device, size_t size);
    static Buffer borrow(void* handle);
    void deinit();
};

// mattn.zig:47-276
struct Context {
    void* device = nullptr;
    void* queue = nullptr;
    void* block_pipeline = nullptr;
    void* qk_pipeline = nullptr;
    void* wide_pipeline = nullptr; // one head of width 512 (the VAE mid-block), mattn.zig:53
    size_t wide_threads = 0;
    Kernel kernel = Kernel::block;
    size_t threads = 0;
    size_t qk_threads = 0;
    // grow-only activation pool for runPooled (q, k, v, mix slots)
    void* pool[4] = {nullptr, nullptr, nullptr, nullptr};
    size_t pool_bytes[4] = {0, 0, 0, 0};

    static Error init(Context* out);                       // mattn.zig:65-67
    static Error initKernel(Kernel kernel, Context* out);  // mattn.zig:69-118
    void deinit();                                         // mattn.zig:120-130
    bool pick(size_t tokens, size_t head_dim, Pick* out) const; // mattn.zig:134-150; false = no kernel for the shape
    bool widePick(const attention::Config& cfg, Pick* out) const; // mattn.zig:261-275

    // mattn.zig:152-173: host f32 token-major slices in, out.
    Error run(float* out, size_t out_len, const float* q, size_t q_len, const float* k, size_t k_len,
              const float* v, size_t v_len, const attention::Config& cfg);
    // mattn.zig:183-218: same through the context's reusable device pool.
    Error runPooled(float* out, size_t out_len, const float* q, size_t q_len, const float* k, size_t k_len,
                    const float* v, size_t v_len, const attention::Config& cfg);
    // mattn.zig:228-250: caller-owned device handles, no upload or readback.
    Error runOnHandles(void* q_h, void* k_h, void* v_h, void* out_h, const attention::Config& cfg);
};

} // namespace hattn

namespace attention_fast {
// runtime/attention_fast.zig:6-24. `hip` may be null (no backend). On
// UnsupportedShape, or without a backend, the caller's CPU kernel runs if one
// is given; with none, UnsupportedShape / NotAvailable is returned: this
// library never computes attention on the CPU itself.
Error run(hattn::Context* hip, float* out, size_t out_len, const float* q, size_t q_len, const float* k,
          size_t k_len, const float* v, size_t v_len, float* scratch, size_t scratch_len,
          const attention::Config& cfg, attention::CpuRun cpu, void* cpu_user);
} // namespace attention_fast

namespace hqk {
// metal/mqk.zig:12-18
struct Config {
    size_t tokens;
    size_t heads;
    size_t kv_heads;
    size_t head_dim;
    float norm_eps;
};
// zimage/zrope.zig:11-15 + Cache (values are (cos,sin) pairs, axis-major)
struct RopeCache {
    size_t dims[3];
    size_t lens[3];
    const float* values; // host pointer, count() pairs
    size_t count() const;
    size_t axisBase(size_t axis) const;
};
// metal/mqk.zig:20-58: Z-Image QK-norm + rope in place on device buffers
// q [tokens][heads][128], k [tokens][kv_heads][128] (f32). Weights are host
// f32[head_dim]; pos is host [tokens][3].
Error run(hattn::Context* ctx, void* q_h, void* k_h, const float* q_weight, const float* k_weight,
          const size_t* pos, size_t pos_len, const RopeCache& rope, const Config& cfg);
} // namespace hqk

namespace joint {

enum class KSite : uint32_t { tile_load = ZDRAW_HIP_K_IN_TILE_LOAD, prepass = ZDRAW_HIP_K_PREPASS };

// One Klein joint-attention call over `nb` image segments laid out
// [txt_0 | img_0 | txt_1 | img_1 | ...] (klein/zflux2_resident.zig:1407-1411):
// q, k, v, o are [nb*tokens][heads*128]. Double blocks pass the text-row
// weights (norm_added_q/k) with txt_rows = 512; single blocks pass null.
struct Klein {
    void* q; void* k; void* v; void* o;  // device buffer handles
    uint32_t in_dtype;                   // ZDRAW_HIP_F32 / ZDRAW_HIP_BF16
    uint32_t out_dtype;
    size_t tokens;                       // per segment (text + image + reference image)
    size_t heads;
    size_t nb;
    size_t txt_rows;
    void* norm_q; void* norm_k;          // f32[128] device buffers
    void* norm_added_q; void* norm_added_k; // or null
    void* rope_cos; void* rope_sin;      // f32 [rows][128]
    bool rope_per_segment;               // table has nb*tokens rows (forwardBatch duplicates it) or tokens rows
    void* key_pad;                       // u8 [nb][tokens] or null
    size_t out_row_stride;               // elements between output token rows; 0 = heads*128
    KSite k_site;
    float score_bound;                   // see scoreBound(); 0 = unknown (running-maximum softmax)
    uint32_t staging;                    // 0 = bf16 copies of the prepared Q and K; ZDRAW_HIP_F16 = IEEE half (needs the pre-pass)
};
Error run(hattn::Context* ctx, const Klein& c);

// Upper bound on |q'.k'| / sqrt(128) after RMSNorm with the given weights and a
// rope that rotates pairs (both table builders of the reference do): each
// normalised row has norm <= sqrt(128) * max|w|. Pass null for weight sets that
// are not in use. Valid only when the rope tables are rotations.
float scoreBound(const float* w_q, const float* w_k, const float* w_q_txt, const float* w_k_txt);

// One Z-Image single-stream attention call (zimage/zattn.zig:45-82 after the
// projections): q, k, v, o are [tokens][heads*128].
struct Zimage {
    void* q; void* k; void* v; void* o;
    uint32_t in_dtype;
    uint32_t out_dtype;
    size_t tokens;
    size_t heads;
    void* q_norm; void* k_norm;          // f32[128] device buffers
    void* pos;                           // u64 [tokens][3] device buffer
    void* rope_pairs;                    // (cos,sin) f32 pairs device buffer
    size_t dims[3];
    size_t bases[3];
    float norm_eps;
    KSite k_site;
    float score_bound;                   // see scoreBound(); 0 = unknown
    uint32_t staging;                    // as Klein::staging
};
Error run(hattn::Context* ctx, const Zimage& c);

} // namespace joint

Error fromCode(int rc);

} // namespace zdraw
