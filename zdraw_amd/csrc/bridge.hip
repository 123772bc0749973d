// C-ABI bridge of the gfx950 attention backend (include/zdraw_hip.h).
//
// Replaces the attention slice of the reference's Objective-C Metal bridge
// (metal/metal_api.m: device/queue/buffer lifecycle :536-576, standalone and
// batch attention encode :2976-3125, scratch slots :6147-6191, the steel route
// :6772-6815, batch begin/end :1084-1114, counters :333-353). Handles are
// heap structs behind void*; every entry validates its operands on the host
// before a kernel is launched, because a kernel that reads out of bounds can
// take the whole device down.
#include "../../include/zdraw_hip.h"
#include "../../include/zdraw_hip_measure.h"
#include "attn_kernel.h"
#include "gemm_kernel.h"

#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

using namespace zdraw;

// Scratch of zdraw_hip_run_attention_fused_noalloc_enc: the prepared Q and K (and the bf16 copy
// of an f32 V, and the parts of key-split tiles) of ONE call. Every GPU the library runs on holds
// its own copy of the array until the process ends; host code never uses the array's name as an
// address, only what hipGetSymbolAddress returned for the device in question.
constexpr size_t kNoallocScratchBytes = (size_t)ZDRAW_HIP_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kNoallocScratchBytes];
constexpr int kMaxDevices = 16;
static void* g_noalloc_scratch[kMaxDevices] = {};

static_assert(sizeof(ZdrawAttnParams) == ZDRAW_HIP_ABI_ATTN_PARAMS_SIZE, "AttnParams ABI drift");
static_assert(sizeof(ZdrawHipAttnExt) == ZDRAW_HIP_ABI_ATTN_EXT_SIZE, "AttnExt ABI drift");
static_assert(sizeof(ZdrawHipQkOperands) == ZDRAW_HIP_ABI_QK_OPERANDS_SIZE, "QkOperands ABI drift");
static_assert(sizeof(ZdrawGemmParams) == ZDRAW_HIP_ABI_GEMM_PARAMS_SIZE, "GemmParams ABI drift");
static_assert(sizeof(ZdrawHipGemmExt) == ZDRAW_HIP_ABI_GEMM_EXT_SIZE, "GemmExt ABI drift");
static_assert(sizeof(ZdrawQkNormParams) == ZDRAW_HIP_ABI_QK_NORM_PARAMS_SIZE, "QkNormParams ABI drift");
static_assert(sizeof(ZdrawHipChainAttnBuffers) == ZDRAW_HIP_ABI_CHAIN_ATTN_BUFFERS_SIZE, "ChainAttnBuffers ABI drift");
static_assert(sizeof(ZdrawHipChainAttnWeights) == ZDRAW_HIP_ABI_CHAIN_ATTN_WEIGHTS_SIZE, "ChainAttnWeights ABI drift");
static_assert(sizeof(ZdrawHipChainAttnParams) == ZDRAW_HIP_ABI_CHAIN_ATTN_PARAMS_SIZE, "ChainAttnParams ABI drift");

namespace {

struct Device {
    int ordinal;
    int cus; // compute units: workgroup slots of the one-workgroup-per-CU kernels
};
struct Buffer {
    void* ptr;
    size_t len;
    bool owned;
    // The bytes can only change through zdraw_hip_write_buffer: memory this library allocated,
    // whose address was never handed out and which no kernel was ever asked to write. Only
    // such buffers have anything read from them cached (the norm weights' maximum).
    bool stable;
};
constexpr int kScratchSlots = 8; // per queue: slots 0-6 as below, 7 = staged norm weights
constexpr int kCallerSlots = 7;  // zdraw_hip_attn_scratch hands these out (metal_api.m:6147-6191)
struct Queue {
    Device* dev;
    hipStream_t stream;
    // The library's own scratch (prepared operands, parts of split tiles, rounded activations):
    // grow-only slots owned by the queue whose work uses them, so that two queues never share a
    // byte of it; freed with the queue.
    Buffer* scratch[kScratchSlots] = {};
};
struct Pipeline {
    int kind; // 0 = attention_block_mfma, 1 = qk_norm_rope, 2 = gemm_half
};
struct Batch {
    Queue* queue;
    hipEvent_t start;
    hipEvent_t stop;
};
struct Event {
    hipEvent_t ev;
};

// Single-threaded counters, as in the reference bridge (metal_api.m:333-353).
uint64_t g_dispatch = 0;
uint64_t g_command = 0;
uint64_t g_fallback = 0;
uint64_t g_gpu_ns = 0;
int g_variant = 0; // bit 0: kernel shape, 0 = 8 waves per workgroup, 1 = 4 waves (two workgroups per CU); bit 1: never split tail tiles
bool g_setup_done = false;
bool g_gemm_setup_done = false;

// Attention-kernel trace (the reference's ZDRAW_KLEIN_TRACE attention bucket,
// klein/zflux2_resident.zig:443-467): when on, every attention launch is
// bracketed by its own pair of events on the launch stream.
bool g_trace = false;
struct TracePair {
    hipEvent_t a, b;
};
std::vector<TracePair> g_trace_open;
uint64_t g_trace_ns = 0;
uint64_t g_trace_launches = 0;

// Clock probe: per-workgroup run time of the last traced attention launch in
// shader-clock cycles and in 100 MHz reference ticks (their ratio is the clock
// the kernel actually ran at, which under load is set by the power limit).
constexpr int64_t kClockCap = 4096;
bool g_clock_on = false;
unsigned long long* g_clock_buf = nullptr;
int64_t g_clock_wgs = 0;
hipStream_t g_clock_stream = nullptr;

thread_local char g_err[512] = "";

void set_err(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int hip_fail(hipError_t e, const char* what) {
    set_err("%s: %s", what, hipGetErrorString(e));
    return ZDRAW_HIP_ERR_DEVICE;
}

int unavailable(const char* why) {
    g_fallback++;
    set_err("unavailable: %s", why);
    return ZDRAW_HIP_UNAVAILABLE;
}

int invalid(const char* why) {
    set_err("invalid: %s", why);
    return ZDRAW_HIP_INVALID;
}

size_t elem_size(uint32_t dtype) { return dtype == ZDRAW_HIP_F32 ? 4 : 2; }

// One strided activation operand checked against its buffer.
struct Operand {
    const Buffer* buf;
    uint64_t off;          // bytes
    uint64_t bs, ts, hs;   // elements
};

// Returns nullptr if fine, else a reason. The kernel issues 16-byte loads of
// 8 (bf16) or 4 (f32) consecutive elements, and 8/16-byte stores of 4.
const char* check_operand(const Operand& o, uint32_t dtype, uint32_t batch, uint32_t tokens, uint32_t heads,
                          const char* name) {
    static thread_local char why[128];
    if (!o.buf || !o.buf->ptr) {
        snprintf(why, sizeof(why), "%s: null buffer", name);
        return why;
    }
    const size_t es = elem_size(dtype);
    const uint64_t align_elems = 16 / es;
    if (o.off % 16 != 0 || o.ts % align_elems != 0 || o.hs % align_elems != 0 || (batch > 1 && o.bs % align_elems != 0)) {
        snprintf(why, sizeof(why), "%s: offset/strides must keep rows 16-byte aligned", name);
        return why;
    }
    if (((uintptr_t)o.buf->ptr) % 16 != 0) {
        snprintf(why, sizeof(why), "%s: device pointer not 16-byte aligned", name);
        return why;
    }
    // the kernel addresses the rows of one head with 32-bit byte offsets from the head's first row
    if (o.ts >= (1ull << 31) || ((uint64_t)(tokens - 1) * o.ts + kHeadDim) * es >= (1ull << 32)) {
        snprintf(why, sizeof(why), "%s: one head's rows span 4 GiB or more", name);
        return why;
    }
    if (o.ts < kHeadDim && tokens > 1) {
        snprintf(why, sizeof(why), "%s: token stride smaller than head_dim", name);
        return why;
    }
    const uint64_t last = (uint64_t)(batch - 1) * o.bs + (uint64_t)(tokens - 1) * o.ts + (uint64_t)(heads - 1) * o.hs +
                          kHeadDim;
    if (o.off > o.buf->len || last * es > o.buf->len - o.off) {
        snprintf(why, sizeof(why), "%s: buffer too small for the declared shape", name);
        return why;
    }
    return nullptr;
}

const void* at(const Buffer* b, uint64_t off) { return static_cast<const char*>(b->ptr) + off; }

bool need(const void* handle, size_t bytes) {
    const Buffer* b = static_cast<const Buffer*>(handle);
    return b && b->ptr && b->len >= bytes && ((uintptr_t)b->ptr % 16) == 0;
}

bool scratch_poisoned(int slot);

// (Re)allocation of a grow-only scratch slot. `wait` drains whatever may still read the old
// allocation before it is freed; the new one is filled (0x00, or 0xFF under
// ZDRAW_SCRATCH_POISON) so that a read that precedes its write sees the same bytes on every
// run (metal_api.m:6160-6181).
template <typename Wait>
Buffer* grow_slot(Buffer** slot_ptr, int slot, size_t bytes, Wait wait) {
    Buffer* cur = *slot_ptr;
    if (cur && cur->len >= bytes) return cur;
    wait();
    void* p = nullptr;
    if (hipMalloc(&p, bytes) != hipSuccess) {
        set_err("scratch hipMalloc(%zu) failed", bytes);
        return nullptr;
    }
    (void)hipMemset(p, scratch_poisoned(slot) ? 0xFF : 0x00, bytes);
    (void)hipDeviceSynchronize();
    if (cur) {
        (void)hipFree(cur->ptr);
        cur->ptr = p;
        cur->len = bytes;
        return cur;
    }
    *slot_ptr = new Buffer{p, bytes, true, false};
    return *slot_ptr;
}

// A queue's own slot: only work enqueued on this queue can be reading the old allocation.
Buffer* queue_scratch(Queue* q, int slot, size_t bytes) {
    if (!q || slot < 0 || slot >= kScratchSlots || bytes == 0) return nullptr;
    return grow_slot(&q->scratch[slot], slot, bytes, [q] { (void)hipStreamSynchronize(q->stream); });
}

// Where a call's scratch comes from: the grow-only slots of the queue the call runs on,
// or a caller-supplied span handed out piece by piece in 256-byte steps (the entry that
// allocates nothing), or nowhere (a plan that is only validated).
struct ScratchSource {
    Queue* queue;
    bool dry;
    char* span = nullptr; // bump allocation over [span, span + cap)
    size_t cap = 0, used = 0;
    bool over = false;    // the span was too small for what the call needs
    ScratchSource(Queue* q, bool dry_run = false) : queue(q), dry(dry_run) {}
    ScratchSource(Queue* q, void* base, size_t bytes) : queue(q), dry(false), span(static_cast<char*>(base)), cap(bytes) {}
    void* get(int slot, size_t bytes);
};

constexpr uint32_t kRoundPlainTokens = 1024; // plain f32 attention from this length on rounds its operands once, ahead of the kernel

struct FusedPlan {
    AttnArgs args;
    int in_dtype;
    int k_mode;
    bool prepass;
    PrepArgs prep;   // K pre-pass
    PrepArgs prep_q; // Q pre-pass (same launch condition)
    PrepArgs prep_v; // f32 operands only: V rounded to bf16 by the same launch
    bool round_v = false;
    int prep_in_dtype = kF32; // element type the pre-pass reads
    int w_dtype = kF32; // element type of the norm weights as the kernels read them (16-bit only with the pre-pass)
    bool stage_w = false;  // the norm weights are first copied as f32 into scratch (two types, or off a 16-byte boundary)
    WeightStageArgs stage;
};

// Norm weights as QkNormParams describes them (metal_c.zig:258-274): element
// type in the weight coding (1 f16, 2 bf16, 3 f32) and a byte offset into the buffer.
struct NormWeights {
    uint32_t q_dtype, k_dtype;
    uint64_t q_off, k_off;
};

int norm_weight_dtype(uint32_t coded) {
    return coded == ZDRAW_HIP_W_F32 ? (int)kF32 : coded == ZDRAW_HIP_W_F16 ? (int)kF16 : coded == ZDRAW_HIP_W_BF16 ? (int)kBF16 : -1;
}

// max |w| over the 128 norm weights at `off` in `b`, element type `dtype` (kF32, kF16, kBF16).
// Only for buffers whose bytes cannot change behind the library's back (Buffer::stable): those
// are read back once per (address, type) and the figure is kept until the buffer is written
// through this library or released. +inf for any other buffer, and when the weights cannot be
// read or hold a NaN (the caller then gets the running-maximum softmax).
struct WeightMax {
    const void* ptr;
    int dtype;
    float amax;
};
std::vector<WeightMax> g_weight_max;

// A buffer that a kernel is about to write, or whose address leaves the library: nothing read
// from it is cached from here on.
void forget_weight_max(const Buffer* b);
void mark_unstable(void* handle) {
    Buffer* b = static_cast<Buffer*>(handle);
    if (!b || !b->stable) return;
    b->stable = false;
    if (b->ptr) forget_weight_max(b);
}

void forget_weight_max(const Buffer* b) {
    const char* lo = static_cast<const char*>(b->ptr);
    const char* hi = lo + b->len;
    for (size_t i = 0; i < g_weight_max.size();) {
        const char* p = static_cast<const char*>(g_weight_max[i].ptr);
        if (p >= lo && p < hi) {
            g_weight_max[i] = g_weight_max.back();
            g_weight_max.pop_back();
        } else {
            i++;
        }
    }
}

float weight_abs_max(const Buffer* b, uint64_t off, int dtype) {
    if (!b->stable) return INFINITY;
    const void* src = static_cast<const char*>(b->ptr) + off;
    for (const WeightMax& w : g_weight_max)
        if (w.ptr == src && w.dtype == dtype) return w.amax;
    unsigned char raw[kHeadDim * 4];
    const size_t bytes = (size_t)kHeadDim * (dtype == kF32 ? 4 : 2);
    if (hipMemcpy(raw, src, bytes, hipMemcpyDeviceToHost) != hipSuccess) return INFINITY;
    float m = 0.f;
    for (int i = 0; i < kHeadDim; i++) {
        float v;
        if (dtype == kF32) {
            memcpy(&v, raw + 4 * i, 4);
        } else {
            uint16_t h;
            memcpy(&h, raw + 2 * i, 2);
            if (dtype == kBF16) {
                const uint32_t u = (uint32_t)h << 16;
                memcpy(&v, &u, 4);
            } else {
                v = (float)__builtin_bit_cast(_Float16, h);
            }
        }
        v = fabsf(v);
        if (!(v <= m)) m = v; // a NaN sticks
    }
    if (!(m >= 0.0f)) m = INFINITY;
    if (g_weight_max.size() >= 256) g_weight_max.clear();
    g_weight_max.push_back(WeightMax{src, dtype, m});
    return m;
}

// How many positions of each Z-Image rope axis lie inside a (cos,sin) pair table of
// `table_bytes` bytes: axis i holds dims[i] / 2 pairs per position from pair base[i] up to the
// next axis base above it (or the end of the table). The layout of zrope.Cache
// (zimage/zrope.zig:29-42, 118-140) gives back its `lens`. False when an axis has no whole
// position inside the table.
bool zimage_axis_lens(uint64_t table_bytes, const uint64_t base[3], const uint32_t dims[3], uint32_t lens[3]) {
    const uint64_t total = table_bytes / 8; // pairs
    for (int i = 0; i < 3; i++) {
        const uint64_t per = dims[i] / 2;
        if (per == 0 || base[i] >= total) return false;
        uint64_t end = total;
        for (int j = 0; j < 3; j++)
            if (base[j] > base[i] && base[j] < end) end = base[j];
        const uint64_t n = (end - base[i]) / per;
        if (n == 0) return false;
        lens[i] = n > 0xffffffffull ? 0xffffffffu : (uint32_t)n;
    }
    return true;
}

// Shared validation + argument assembly. Returns 0 or an ABI return code.
// nw == nullptr: norm weights are f32[128] at offset 0.
int scratch_failed(const ScratchSource* src) {
    if (src->over) {
        g_fallback++;
        set_err("unavailable: the call needs more than the %zu bytes of scratch this entry holds", src->cap);
        return ZDRAW_HIP_UNAVAILABLE;
    }
    set_err("scratch allocation failed");
    return ZDRAW_HIP_ERR_HANDLE;
}

int plan_attention(Device* dev, void* q, void* k, void* v, void* out, const ZdrawAttnParams* p,
                   const ZdrawHipAttnExt* x, const ZdrawHipQkOperands* ops, FusedPlan* plan,
                   ScratchSource* src, const NormWeights* nw = nullptr) {
    if (!p || !x) {
        set_err("null params");
        return ZDRAW_HIP_ERR_HANDLE;
    }
    // shape classes, in the order mattn.zig:376-408 checks them
    if (p->tokens == 0) return unavailable("tokens == 0");
    if (p->heads == 0 || p->kv_heads == 0 || p->head_dim == 0) return invalid("zero dimension");
    if (p->heads % p->kv_heads != 0) return invalid("heads % kv_heads != 0");
    if (p->head_dim != (uint32_t)kHeadDim) return unavailable("head_dim != 128");
    if (p->causal != 0) return unavailable("causal attention");
    if (p->kv_heads != p->heads) return unavailable("grouped-query attention");
    if (x->batch == 0) return invalid("batch == 0");
    const uint64_t max_tokens = (uint64_t)attention_max_tokens();
    if ((uint64_t)p->tokens > max_tokens) return unavailable("too many tokens");
    if ((x->in_dtype != ZDRAW_HIP_F32 && x->in_dtype != ZDRAW_HIP_BF16 && x->in_dtype != ZDRAW_HIP_F16) ||
        (x->out_dtype != ZDRAW_HIP_F32 && x->out_dtype != ZDRAW_HIP_BF16 && x->out_dtype != ZDRAW_HIP_F16))
        return unavailable("activation dtype");
    if (x->qk_mode > ZDRAW_HIP_QK_ZIMAGE) return invalid("qk_mode");
    if (x->staging != 0 && x->staging != ZDRAW_HIP_BF16 && x->staging != ZDRAW_HIP_F16) return invalid("staging");
    // IEEE-half score operands (the reference's staging type): where the library writes the
    // staged copies of Q and K itself, on the eight-wave kernel shape
    const bool stage_f16 = x->in_dtype == ZDRAW_HIP_F16 || x->staging == ZDRAW_HIP_F16;
    if (stage_f16) {
        if (x->qk_mode != ZDRAW_HIP_QK_NONE && x->k_site != ZDRAW_HIP_K_PREPASS)
            return unavailable("IEEE-half staging needs the pre-pass (k_site)");
        if (x->qk_mode == ZDRAW_HIP_QK_NONE && x->in_dtype == ZDRAW_HIP_BF16)
            return unavailable("IEEE-half staging of operands that arrive as bf16 and are used as given");
        if (g_variant & 1) return unavailable("IEEE-half staging on the four-wave kernel shape");
    }

    const Operand oq{static_cast<Buffer*>(q), x->q_off, x->q_stride[0], x->q_stride[1], x->q_stride[2]};
    const Operand ok{static_cast<Buffer*>(k), x->k_off, x->k_stride[0], x->k_stride[1], x->k_stride[2]};
    const Operand ov{static_cast<Buffer*>(v), x->v_off, x->v_stride[0], x->v_stride[1], x->v_stride[2]};
    const Operand oo{static_cast<Buffer*>(out), x->out_off, x->out_stride[0], x->out_stride[1], x->out_stride[2]};
    const char* why;
    if ((why = check_operand(oq, x->in_dtype, x->batch, p->tokens, p->heads, "q"))) return invalid(why);
    if ((why = check_operand(ok, x->in_dtype, x->batch, p->tokens, p->heads, "k"))) return invalid(why);
    if ((why = check_operand(ov, x->in_dtype, x->batch, p->tokens, p->heads, "v"))) return invalid(why);
    if ((why = check_operand(oo, x->out_dtype, x->batch, p->tokens, p->heads, "out"))) return invalid(why);
    mark_unstable(out); // a kernel is about to write it

    AttnArgs a;
    memset(&a, 0, sizeof(a));
    a.q = at(oq.buf, oq.off);
    a.k = at(ok.buf, ok.off);
    a.v = at(ov.buf, ov.off);
    a.o = const_cast<void*>(at(oo.buf, oo.off));
    a.q_bs = (int64_t)oq.bs; a.q_ts = (int64_t)oq.ts; a.q_hs = (int64_t)oq.hs;
    a.k_bs = (int64_t)ok.bs; a.k_ts = (int64_t)ok.ts; a.k_hs = (int64_t)ok.hs;
    a.v_bs = (int64_t)ov.bs; a.v_ts = (int64_t)ov.ts; a.v_hs = (int64_t)ov.hs;
    a.o_bs = (int64_t)oo.bs; a.o_ts = (int64_t)oo.ts; a.o_hs = (int64_t)oo.hs;
    a.tokens = (int32_t)p->tokens;
    a.heads = (int32_t)p->heads;
    a.batch = (int32_t)x->batch;
    a.key_limit = (int32_t)((p->valid != 0 && p->valid < p->tokens) ? p->valid : p->tokens);
    const int rows = attention_block_rows(g_variant & 1);
    a.nqb = (int32_t)((p->tokens + rows - 1) / rows);
    a.q_mode = (int32_t)x->qk_mode;
    a.out_dtype = (int32_t)x->out_dtype;
    a.scale_log2 = 1.4426950408889634f / sqrtf((float)kHeadDim);
    if (!(x->score_bound >= 0.0f)) return invalid("score_bound");
    float bound = x->score_bound; // raised below to what the norm weights themselves allow
    if ((int64_t)a.nqb * a.heads * a.batch > 0x7fffffffLL) return unavailable("grid too large");

    const uint64_t rows_needed = (uint64_t)(x->batch - 1) * x->rope_batch_rows + p->tokens;
    if (x->qk_mode != ZDRAW_HIP_QK_NONE) {
        if (!ops) return invalid("qk_mode set without operands");
        int qwd = kF32, kwd = kF32;
        uint64_t qwo = 0, kwo = 0;
        bool stage = false;
        if (nw) {
            qwd = norm_weight_dtype(nw->q_dtype);
            kwd = norm_weight_dtype(nw->k_dtype);
            qwo = nw->q_off;
            kwo = nw->k_off;
            if (qwd < 0 || kwd < 0) return unavailable("norm weight dtype");
            if (qwo % (qwd == kF32 ? 4 : 2) != 0 || kwo % (kwd == kF32 ? 4 : 2) != 0)
                return invalid("norm weight offset is not a multiple of the element size");
            if (ops->q_weight_txt || ops->k_weight_txt) return invalid("text norm weights with typed norm weights");
        }
        const size_t qwbytes = (size_t)kHeadDim * (qwd == kF32 ? 4 : 2), kwbytes = (size_t)kHeadDim * (kwd == kF32 ? 4 : 2);
        const Buffer* qwb = static_cast<Buffer*>(ops->q_weight);
        const Buffer* kwb = static_cast<Buffer*>(ops->k_weight);
        if (!qwb || !kwb || !qwb->ptr || !kwb->ptr || qwo > qwb->len || kwo > kwb->len || qwb->len - qwo < qwbytes ||
            kwb->len - kwo < kwbytes)
            return invalid("norm weights must be [128] buffers (f32 unless the caller states a type)");
        const bool q_al = ((uintptr_t)qwb->ptr + qwo) % 16 == 0, k_al = ((uintptr_t)kwb->ptr + kwo) % 16 == 0;
        if (nw) {
            // The kernels read the weights with 16-byte loads and one type for both operands
            // (16-bit types only in the pre-pass). What a checkpoint view hands over instead (a
            // type per operand, a file offset) is first copied as f32 into scratch.
            stage = qwd != kwd || !q_al || !k_al || (qwd != kF32 && x->k_site != ZDRAW_HIP_K_PREPASS);
        } else if (!q_al || !k_al) {
            return invalid("norm weights must be 16-byte aligned");
        }
        plan->w_dtype = stage ? (int)kF32 : qwd;
        if ((ops->q_weight_txt && !need(ops->q_weight_txt, kHeadDim * 4)) ||
            (ops->k_weight_txt && !need(ops->k_weight_txt, kHeadDim * 4)))
            return invalid("text norm weights must be f32[128] buffers");
        if (!(x->eps >= 0.0f)) return invalid("eps");
        a.q_w = reinterpret_cast<const float*>(static_cast<const char*>(qwb->ptr) + qwo);
        a.k_w = reinterpret_cast<const float*>(static_cast<const char*>(kwb->ptr) + kwo);
        if (stage) {
            float* staged = static_cast<float*>(src->get(7, 2 * kHeadDim * sizeof(float)));
            if (!staged) return scratch_failed(src);
            plan->stage_w = true;
            plan->stage = WeightStageArgs{a.q_w, a.k_w, staged, qwd, kwd};
            a.q_w = staged;
            a.k_w = staged + kHeadDim;
        }
        a.q_w_txt = ops->q_weight_txt ? static_cast<const float*>(static_cast<Buffer*>(ops->q_weight_txt)->ptr) : nullptr;
        a.k_w_txt = ops->k_weight_txt ? static_cast<const float*>(static_cast<Buffer*>(ops->k_weight_txt)->ptr) : nullptr;
        a.qk.txt_rows = (int32_t)x->txt_rows;
        a.qk.eps = x->eps;
        a.qk.rope_bs = (int64_t)x->rope_batch_rows;
        if (bound > 0.0f) {
            // The caller asks for the form without a running maximum. Whether the scores allow it
            // is a function of the norm weights alone (rows normalised to sqrt(128) max|w|, a rope
            // that rotates): the library forms that bound itself, so a caller's figure that is too
            // small cannot make the exponentials overflow. (Weight buffers that can change behind
            // the library's back give +inf: the running-maximum form.)
            float mq = weight_abs_max(qwb, qwo, qwd);
            float mk = weight_abs_max(kwb, kwo, kwd);
            if (ops->q_weight_txt) mq = fmaxf(mq, weight_abs_max(static_cast<Buffer*>(ops->q_weight_txt), 0, kF32));
            if (ops->k_weight_txt) mk = fmaxf(mk, weight_abs_max(static_cast<Buffer*>(ops->k_weight_txt), 0, kF32));
            const float own = sqrtf((float)kHeadDim) * mq * mk * 1.02f; // 2 % for the roundings of norm and operands
            bound = (own >= bound) ? own : bound;                       // a NaN or infinite weight: no bound
            if (!(own >= 0.0f)) bound = INFINITY;
        }
        if (x->qk_mode == ZDRAW_HIP_QK_KLEIN) {
            const size_t bytes = (size_t)rows_needed * kHeadDim * 4;
            if (!need(ops->rope_cos, bytes) || !need(ops->rope_sin, bytes))
                return invalid("rope cos/sin tables too small for [rows][128] f32");
            a.qk.rope_cos = static_cast<const float*>(static_cast<Buffer*>(ops->rope_cos)->ptr);
            a.qk.rope_sin = static_cast<const float*>(static_cast<Buffer*>(ops->rope_sin)->ptr);
        } else {
            const uint32_t* d = x->zimage_dims;
            if (d[0] + d[1] + d[2] != (uint32_t)kHeadDim) return invalid("zimage dims must sum to head_dim");
            if (d[0] % 8 != 0 || d[1] % 8 != 0 || d[2] % 8 != 0 || d[0] == 0 || d[1] == 0 || d[2] == 0)
                return unavailable("zimage axis widths must be non-zero multiples of 8");
            for (int i = 0; i < 3; i++)
                if (x->zimage_base[i] % 2 != 0 || x->zimage_base[i] > 0xffffffffull)
                    return unavailable("zimage axis bases must be even and fit 32 bits");
            if (!need(ops->pos, (size_t)rows_needed * 24)) return invalid("positions too small for [rows][3] u64");
            if (!need(ops->rope_pairs, 16)) return invalid("rope pair table missing");
            // positions per axis that lie inside the table: the kernels hold every position to them
            const Buffer* pt = static_cast<Buffer*>(ops->rope_pairs);
            uint32_t lens[3];
            if (!zimage_axis_lens(pt->len, x->zimage_base, d, lens)) return invalid("rope pair table smaller than an axis base");
            a.qk.len0 = lens[0]; a.qk.len1 = lens[1]; a.qk.len2 = lens[2];
            a.qk.pos = static_cast<const unsigned long long*>(static_cast<Buffer*>(ops->pos)->ptr);
            a.qk.pairs = static_cast<const float*>(pt->ptr);
            a.qk.dim0 = (int32_t)d[0]; a.qk.dim1 = (int32_t)d[1]; a.qk.dim2 = (int32_t)d[2];
            a.qk.base0 = (uint32_t)x->zimage_base[0];
            a.qk.base1 = (uint32_t)x->zimage_base[1];
            a.qk.base2 = (uint32_t)x->zimage_base[2];
        }
    }
    // exp2 of a scaled score must stay far from the fp32 exponent limits: 2^64 times
    // tokens (<= 2^15) times |v| still fits, 2^-64 does not underflow
    a.bounded = (bound > 0.0f && bound * 1.4426950408889634f <= 64.0f) ? 1 : 0;
    if (ops && ops->key_pad) {
        const Buffer* m = static_cast<Buffer*>(ops->key_pad);
        const uint64_t mbytes = (uint64_t)(x->batch - 1) * x->mask_batch_bytes + p->tokens;
        if (!m->ptr || m->len < mbytes) return invalid("key_pad smaller than [segments][tokens]");
        a.key_pad = static_cast<const unsigned char*>(m->ptr);
        a.mask_bs = (int64_t)x->mask_batch_bytes;
    }

    // A last round of workgroups that fills at most half the CUs is split along the keys so
    // that it fills them all (its parts are merged by a small kernel, in a fixed order).
    if ((g_variant & 2) == 0) {
        int tail = 0, splits = 1;
        attention_tail_plan((int64_t)a.nqb * a.heads * a.batch, dev->cus, (a.key_limit + attention_key_block() - 1) / attention_key_block(),
                            &tail, &splits);
        if (splits > 1) {
            void* po = src->get(3, attention_part_o_bytes(tail, splits, g_variant & 1));
            void* pm = src->get(4, attention_part_ml_bytes(tail, splits, g_variant & 1));
            if (!po || !pm) return scratch_failed(src);
            a.splits = splits;
            a.tile_base = tail; // launch_attention reads the tail size here
            a.part_o = static_cast<float*>(po);
            a.part_ml = static_cast<float*>(pm);
        }
    }
    plan->args = a;
    plan->in_dtype = (int)x->in_dtype;
    plan->k_mode = (int)x->qk_mode;
    plan->prepass = false;
    if (x->qk_mode != ZDRAW_HIP_QK_NONE && x->k_site == ZDRAW_HIP_K_PREPASS) {
        // Q and K are normalised and rotated once into scratch slots 0 and 1, head-major,
        // as bf16; the attention kernel then reads them as they are. One
        // pass over the rows reads a token's rope row once for all its heads; inside the
        // attention kernel every (head, query block) workgroup would fetch its own copy.
        // Q also takes the softmax scale (in the exp2 domain) here, before the rounding.
        // f32 operands (the reference's resident layout, zflux2_resident.zig:1642-1669, writes
        // half-precision head-major copies the same way): the pre-pass rounds Q and K to bf16
        // and the same launch rounds V into slot 2, so the attention kernel runs its
        // direct-to-LDS build on 16-bit rows instead of rounding every block it loads.
        // f32 and f16 operands: V needs a bf16 copy as well
        const bool to_bf16 = x->in_dtype != ZDRAW_HIP_BF16;
        const uint32_t prep_out = stage_f16 ? (uint32_t)ZDRAW_HIP_F16 : (uint32_t)ZDRAW_HIP_BF16;
        const size_t bytes = (size_t)x->batch * p->heads * p->tokens * kHeadDim * 2;
        void* sq = src->get(0, bytes);
        void* sk = src->get(1, bytes);
        if (!sq || !sk) return scratch_failed(src);
        PrepArgs pr;
        memset(&pr, 0, sizeof(pr));
        pr.y_bs = (int64_t)p->heads * p->tokens * kHeadDim;
        pr.y_ts = kHeadDim;
        pr.y_hs = (int64_t)p->tokens * kHeadDim;
        pr.tokens = a.tokens; pr.heads = a.heads; pr.batch = a.batch;
        pr.mode = (int32_t)x->qk_mode;
        pr.out_dtype = (int32_t)prep_out;
        pr.qk = a.qk;
        pr.w_dtype = plan->w_dtype;
        PrepArgs pq = pr;
        pr.x = a.k;
        pr.y = sk;
        pr.x_bs = a.k_bs; pr.x_ts = a.k_ts; pr.x_hs = a.k_hs;
        pr.w = a.k_w;
        pr.w_txt = a.k_w_txt;
        pr.scale = 1.0f;
        pq.x = a.q;
        pq.y = sq;
        pq.x_bs = a.q_bs; pq.x_ts = a.q_ts; pq.x_hs = a.q_hs;
        pq.w = a.q_w;
        pq.w_txt = a.q_w_txt;
        pq.scale = a.scale_log2;
        plan->prep = pr;
        plan->prep_q = pq;
        plan->prepass = true;
        plan->k_mode = kQkNone;
        plan->args.k = sk;
        plan->args.k_bs = pr.y_bs; plan->args.k_ts = pr.y_ts; plan->args.k_hs = pr.y_hs;
        plan->args.q = sq;
        plan->args.q_bs = pr.y_bs; plan->args.q_ts = pr.y_ts; plan->args.q_hs = pr.y_hs;
        plan->args.q_mode = kQkNone;
        plan->args.scale_log2 = 1.0f;
        plan->args.score_f16 = stage_f16 ? 1 : 0;
        plan->prep_in_dtype = (int)x->in_dtype;
        plan->in_dtype = kBF16; // the kernel's 16-bit build (its score operands' type is args.score_f16)
        if (to_bf16) {
            void* sv = src->get(2, bytes);
            if (!sv) return scratch_failed(src);
            PrepArgs pv = pr;
            pv.mode = kQkNone;
            pv.out_dtype = kBF16;
            pv.x = a.v;
            pv.y = sv;
            pv.x_bs = a.v_bs; pv.x_ts = a.v_ts; pv.x_hs = a.v_hs;
            pv.w = pv.w_txt = nullptr;
            pv.scale = 1.0f;
            plan->prep_v = pv;
            plan->round_v = true;
            plan->args.v = sv;
            plan->args.v_bs = pr.y_bs; plan->args.v_ts = pr.y_ts; plan->args.v_hs = pr.y_hs;
            plan->in_dtype = kBF16;
        }
    }
    if (x->qk_mode == ZDRAW_HIP_QK_NONE &&
        ((x->in_dtype == ZDRAW_HIP_F32 && p->tokens >= kRoundPlainTokens) || stage_f16)) {
        // Plain attention on f32 rows (the reference's base entry, metal_c.zig:286-299, takes
        // them): Q (with the softmax scale), K and V are rounded to bf16 once, head-major, into
        // slots 0-2 by one launch, and the kernel is the direct-to-LDS build, as for prepared
        // operands. Short sequences stay on the build that rounds in its tile load. IEEE-half
        // staging (f16 operands, or asked for on f32 ones) takes this way at any length: Q with
        // its scale and K become f16 copies, V a bf16 one.
        const size_t bytes = (size_t)x->batch * p->heads * p->tokens * kHeadDim * 2;
        void* sc[3];
        for (int i = 0; i < 3; i++) {
            sc[i] = src->get(i, bytes);
            if (!sc[i]) return scratch_failed(src);
        }
        PrepArgs pr;
        memset(&pr, 0, sizeof(pr));
        pr.y_bs = (int64_t)p->heads * p->tokens * kHeadDim;
        pr.y_ts = kHeadDim;
        pr.y_hs = (int64_t)p->tokens * kHeadDim;
        pr.tokens = a.tokens; pr.heads = a.heads; pr.batch = a.batch;
        pr.mode = kQkNone;
        pr.out_dtype = kBF16;
        pr.scale = 1.0f;
        PrepArgs pq = pr, pk = pr, pv = pr;
        pq.out_dtype = pk.out_dtype = stage_f16 ? (int32_t)kF16 : (int32_t)kBF16;
        pq.x = a.q; pq.y = sc[0]; pq.x_bs = a.q_bs; pq.x_ts = a.q_ts; pq.x_hs = a.q_hs; pq.scale = a.scale_log2;
        pk.x = a.k; pk.y = sc[1]; pk.x_bs = a.k_bs; pk.x_ts = a.k_ts; pk.x_hs = a.k_hs;
        pv.x = a.v; pv.y = sc[2]; pv.x_bs = a.v_bs; pv.x_ts = a.v_ts; pv.x_hs = a.v_hs;
        plan->prep_q = pq;
        plan->prep = pk;
        plan->prep_v = pv;
        plan->round_v = true;
        plan->prepass = true;
        plan->prep_in_dtype = (int)x->in_dtype;
        plan->in_dtype = kBF16;
        plan->args.score_f16 = stage_f16 ? 1 : 0;
        plan->args.q = sc[0];
        plan->args.k = sc[1];
        plan->args.v = sc[2];
        plan->args.q_bs = plan->args.k_bs = plan->args.v_bs = pr.y_bs;
        plan->args.q_ts = plan->args.k_ts = plan->args.v_ts = pr.y_ts;
        plan->args.q_hs = plan->args.k_hs = plan->args.v_hs = pr.y_hs;
        plan->args.scale_log2 = 1.0f;
    }
    return ZDRAW_HIP_OK;
}

// no_alloc: the call may not allocate: no clock probe buffer, no trace events, and the
// kernels' one-time setup must already have happened (zdraw_hip_create_device does it).
int enqueue(const FusedPlan& plan, hipStream_t stream, bool no_alloc = false) {
    if (!g_setup_done) {
        if (no_alloc) {
            set_err("attention kernels not set up: create the device first");
            return ZDRAW_HIP_ERR_HANDLE;
        }
        hipError_t e = attention_setup();
        if (e != hipSuccess) {
            set_err("attention_setup: %s", hipGetErrorString(e));
            return ZDRAW_HIP_ERR_HANDLE;
        }
        g_setup_done = true;
    }
    if (plan.stage_w) {
        hipError_t e = launch_weight_stage(plan.stage, stream);
        if (e != hipSuccess) {
            set_err("norm weight staging launch: %s", hipGetErrorString(e));
            return ZDRAW_HIP_ERR_HANDLE;
        }
        g_dispatch++;
    }
    if (plan.prepass) {
        const PrepArgs ops[3] = {plan.prep_q, plan.prep, plan.prep_v};
        hipError_t e = launch_qk_prepass(ops, plan.round_v ? 3 : 2, plan.prep_in_dtype, stream);
        if (e != hipSuccess) {
            set_err("qk pre-pass launch: %s", hipGetErrorString(e));
            return ZDRAW_HIP_ERR_HANDLE;
        }
        g_dispatch++;
    }
    AttnArgs args = plan.args;
    if (g_clock_on && !no_alloc) {
        if (!g_clock_buf && hipMalloc(&g_clock_buf, sizeof(unsigned long long) * 2 * kClockCap) != hipSuccess) g_clock_buf = nullptr;
        if (g_clock_buf) {
            args.clock_probe = g_clock_buf;
            args.clock_cap = kClockCap;
            // key-split tail tiles carry no probe
            g_clock_wgs = (int64_t)args.nqb * args.heads * args.batch - (args.splits > 1 ? args.tile_base : 0);
            g_clock_stream = stream;
        }
    }
    TracePair tp{nullptr, nullptr};
    if (g_trace && !no_alloc && hipEventCreate(&tp.a) == hipSuccess && hipEventCreate(&tp.b) == hipSuccess)
        (void)hipEventRecord(tp.a, stream);
    hipError_t e = launch_attention(args, plan.in_dtype, plan.k_mode, g_variant & 1, stream);
    if (e != hipSuccess) {
        set_err("attention launch: %s", hipGetErrorString(e));
        return ZDRAW_HIP_ERR_HANDLE;
    }
    if (tp.a && tp.b) {
        (void)hipEventRecord(tp.b, stream);
        g_trace_open.push_back(tp);
    }
    g_dispatch++;
    return ZDRAW_HIP_OK;
}

// Token-major f32 [tokens][heads][128] operands of the reference's standalone
// entry (runtime/attention.zig:100-113), one segment at byte offsets.
void standalone_ext(const ZdrawAttnParams* p, uint64_t in_off, uint64_t out_off, ZdrawHipAttnExt* x) {
    memset(x, 0, sizeof(*x));
    x->q_off = x->k_off = x->v_off = in_off;
    x->out_off = out_off;
    const uint64_t ts = (uint64_t)p->heads * p->head_dim;
    uint64_t* strides[4] = {x->q_stride, x->k_stride, x->v_stride, x->out_stride};
    for (auto* s : strides) {
        s[0] = 0;
        s[1] = ts;
        s[2] = p->head_dim;
    }
    x->batch = 1;
    x->in_dtype = ZDRAW_HIP_F32;
    x->out_dtype = ZDRAW_HIP_F32;
    x->qk_mode = ZDRAW_HIP_QK_NONE;
}

int check_pipeline(void* pipeline, uint32_t kernel, int want_kind) {
    Pipeline* pl = static_cast<Pipeline*>(pipeline);
    if (!pl) {
        set_err("null pipeline");
        return ZDRAW_HIP_ERR_HANDLE;
    }
    if (pl->kind != want_kind) {
        set_err("pipeline of the wrong kind");
        return ZDRAW_HIP_ERR_HANDLE;
    }
    if (want_kind == 0 && kernel != ZDRAW_HIP_K_BLOCK) return unavailable("only the block (MFMA) kernel exists");
    if (want_kind == 3 && kernel != ZDRAW_HIP_K_WIDE) return unavailable("the wide pipeline runs the wide kernel only");
    return ZDRAW_HIP_OK;
}

bool g_wide_setup_done = false;
// the redo flags of the last wide-head launch (measurement aid: how many tiles took the safe kernel)
int* g_last_wide_redo = nullptr;
int g_last_wide_tiles = 0;
hipStream_t g_last_wide_stream = nullptr;

// One wide head (metal/mattn.zig:261-275 widePick, :280-283 sdpaShape): f32 token-major
// q, k, v, out [tokens][512] at byte offsets; rounds the operands into scratch slots 0-2,
// then runs the wide kernel.
int enqueue_wide(Queue* queue, void* q, void* k, void* v, void* out, const ZdrawAttnParams* p, uint64_t in_off,
                 uint64_t out_off) {
    hipStream_t stream = queue->stream;
    if (p->tokens == 0) return unavailable("tokens == 0");
    if (p->heads != 1 || p->kv_heads != 1) return unavailable("the wide kernel runs one head");
    if (p->head_dim != (uint32_t)wide_head_dim()) return unavailable("the wide kernel runs head_dim 512");
    if (p->causal != 0) return unavailable("causal attention");
    if (p->valid != 0 && p->valid != p->tokens) return unavailable("the wide kernel has no key limit");
    if (p->tokens % (uint32_t)wide_block_rows() != 0) return unavailable("tokens % 64 != 0");
    if (p->tokens > (1u << 20)) return unavailable("too many tokens");
    const uint64_t n = (uint64_t)p->tokens * p->head_dim;
    const Buffer* bs[4] = {static_cast<Buffer*>(q), static_cast<Buffer*>(k), static_cast<Buffer*>(v), static_cast<Buffer*>(out)};
    for (int i = 0; i < 4; i++) {
        const uint64_t off = i == 3 ? out_off : in_off;
        if (!bs[i] || !bs[i]->ptr) return invalid("null buffer");
        if (off % 16 != 0 || ((uintptr_t)bs[i]->ptr % 16) != 0) return invalid("operand not 16-byte aligned");
        if (off > bs[i]->len || n * 4 > bs[i]->len - off) return invalid("buffer smaller than [tokens][512] f32");
    }
    mark_unstable(out);
    Buffer* sc[3];
    for (int i = 0; i < 3; i++) {
        sc[i] = queue_scratch(queue, i, (size_t)n * 2);
        if (!sc[i]) {
            set_err("scratch allocation failed");
            return ZDRAW_HIP_ERR_HANDLE;
        }
    }
    if (!g_wide_setup_done) {
        hipError_t e = wide_setup();
        if (e != hipSuccess) {
            set_err("wide_setup: %s", hipGetErrorString(e));
            return ZDRAW_HIP_ERR_HANDLE;
        }
        g_wide_setup_done = true;
    }
    // one flag per query tile (scratch slot 4): set by the kernel where a row's scores outgrow its
    // fixed reference point, cleared by the rounding launch, read by the kernel that forms such
    // tiles again
    Buffer* redo = queue_scratch(queue, 4, (size_t)wide_tiles((int)p->tokens) * sizeof(int));
    if (!redo) {
        set_err("scratch allocation failed");
        return ZDRAW_HIP_ERR_HANDLE;
    }
    WidePrepArgs pr;
    memset(&pr, 0, sizeof(pr));
    pr.redo = static_cast<int*>(redo->ptr);
    pr.redo_tiles = wide_tiles((int)p->tokens);
    pr.q = reinterpret_cast<const float*>(static_cast<const char*>(bs[0]->ptr) + in_off);
    pr.k = reinterpret_cast<const float*>(static_cast<const char*>(bs[1]->ptr) + in_off);
    pr.v = reinterpret_cast<const float*>(static_cast<const char*>(bs[2]->ptr) + in_off);
    pr.qo = sc[0]->ptr; pr.ko = sc[1]->ptr; pr.vo = sc[2]->ptr;
    pr.chunks = (int64_t)(n / 8);
    pr.q_scale = 1.4426950408889634f / sqrtf((float)p->head_dim);
    hipError_t e = launch_wide_round(pr, stream);
    if (e != hipSuccess) {
        set_err("wide rounding launch: %s", hipGetErrorString(e));
        return ZDRAW_HIP_ERR_HANDLE;
    }
    g_dispatch++;
    WideArgs a;
    memset(&a, 0, sizeof(a));
    a.q = sc[0]->ptr; a.k = sc[1]->ptr; a.v = sc[2]->ptr;
    a.o = reinterpret_cast<float*>(static_cast<char*>(bs[3]->ptr) + out_off);
    a.tokens = (int32_t)p->tokens;
    a.redo = static_cast<int*>(redo->ptr);
    a.splits = wide_splits(a.tokens, queue->dev->cus);
    if (a.splits > 1) {
        // a short sequence runs as key ranges whose shares go through scratch slot 3
        Buffer* part = queue_scratch(queue, 3, wide_part_bytes(a.tokens, a.splits));
        if (!part) {
            set_err("scratch allocation failed");
            return ZDRAW_HIP_ERR_HANDLE;
        }
        a.part_o = static_cast<float*>(part->ptr);
        a.part_ml = a.part_o + (size_t)a.splits * (size_t)a.tokens * (size_t)wide_head_dim();
    }
    TracePair tp{nullptr, nullptr};
    if (g_trace && hipEventCreate(&tp.a) == hipSuccess && hipEventCreate(&tp.b) == hipSuccess)
        (void)hipEventRecord(tp.a, stream);
    e = launch_wide_attention(a, stream);
    if (e != hipSuccess) {
        set_err("wide attention launch: %s", hipGetErrorString(e));
        return ZDRAW_HIP_ERR_HANDLE;
    }
    if (tp.a && tp.b) {
        (void)hipEventRecord(tp.b, stream);
        g_trace_open.push_back(tp);
    }
    g_dispatch++;
    g_last_wide_redo = a.redo;
    g_last_wide_tiles = wide_tiles(a.tokens);
    g_last_wide_stream = stream;
    return ZDRAW_HIP_OK;
}

int finish_blocking(Queue* qu, hipEvent_t start, hipEvent_t stop) {
    hipError_t e = hipEventRecord(stop, qu->stream);
    if (e == hipSuccess) e = hipEventSynchronize(stop);
    if (e != hipSuccess) return hip_fail(e, "wait");
    float ms = 0.f;
    if (hipEventElapsedTime(&ms, start, stop) == hipSuccess && ms > 0.f) g_gpu_ns += (uint64_t)((double)ms * 1e6);
    g_command++;
    return ZDRAW_HIP_OK;
}

Buffer* g_scratch[kCallerSlots] = {};

void* ScratchSource::get(int slot, size_t bytes) {
    // a plan of which only the pre-pass arguments are used: its operand slots are never
    // dereferenced, the staged norm weights (slot 7) are
    if (dry && slot != 7) return reinterpret_cast<void*>(uintptr_t{256});
    if (span) {
        const size_t at = (used + 255) & ~size_t{255};
        if (bytes > cap || at > cap - bytes) {
            over = true;
            return nullptr;
        }
        used = at + bytes;
        return span + at;
    }
    Buffer* b = queue_scratch(queue, slot, bytes);
    return b ? b->ptr : nullptr;
}

bool scratch_poisoned(int slot) {
    // ZDRAW_SCRATCH_POISON: "1" every slot, "attn" the group, "attn:2" one slot
    const char* raw = getenv("ZDRAW_SCRATCH_POISON");
    if (!raw || !*raw) return false;
    if (strcmp(raw, "1") == 0) return true;
    if (strncmp(raw, "attn", 4) != 0) return false;
    if (raw[4] == '\0') return true;
    if (raw[4] == ':') return atoi(raw + 5) == slot;
    return false;
}

// C = A x W^T (metal_api.m gemm encode paths). Validates, then launches on `stream`.
// One launch for `groups` (1..3) products that share A, every dimension and the
// extension block: group i multiplies by ws[i] at byte offset w_offs[i] into cs[i].
int enqueue_gemm_group(void* a, void* const* ws, void* const* cs, const uint64_t* w_offs, int groups,
                       const ZdrawGemmParams* p, const ZdrawHipGemmExt* x, Queue* queue) {
    if (!p || !x || !queue || groups < 1 || groups > 3) {
        set_err("null params");
        return ZDRAW_HIP_ERR_HANDLE;
    }
    if (p->m == 0 || p->k == 0 || p->n == 0) return invalid("zero dimension");
    if (p->mode != ZDRAW_HIP_GEMM_HALF) return unavailable("only the half-precision GEMM mode exists");
    if (p->dtype != ZDRAW_HIP_W_F16 && p->dtype != ZDRAW_HIP_W_BF16) return unavailable("weight dtype");
    if (p->k % 8 != 0) return unavailable("k % 8 != 0");
    const uint32_t wt = p->dtype == ZDRAW_HIP_W_F16 ? (uint32_t)ZDRAW_HIP_F16 : (uint32_t)ZDRAW_HIP_BF16;
    if ((x->a_dtype != ZDRAW_HIP_F32 && x->a_dtype != wt) || (x->c_dtype != ZDRAW_HIP_F32 && x->c_dtype != wt))
        return invalid("activation / output dtype must be f32 or the weight's type");
    const Buffer* ab = static_cast<const Buffer*>(a);
    if (!ab || !ab->ptr) return invalid("null buffer");
    const uint64_t lda = x->lda ? x->lda : p->k, ldw = x->ldw ? x->ldw : p->k, ldc = x->ldc ? x->ldc : p->n;
    if (lda < p->k || ldw < p->k || ldc < p->n) return invalid("leading dimension smaller than the row");
    const uint64_t ea = elem_size(x->a_dtype), ec = elem_size(x->c_dtype);
    // 16-byte loads of 8 (16-bit) or 4 (f32) elements: rows must start 16-byte aligned
    if (x->a_off % 16 != 0 || (lda * ea) % 16 != 0 || ((uintptr_t)ab->ptr % 16) != 0) return invalid("A rows not 16-byte aligned");
    if (x->c_off % ec != 0) return invalid("C offset not element aligned");
    const uint64_t a_bytes = ((uint64_t)(p->m - 1) * lda + p->k) * ea;
    const uint64_t w_bytes = ((uint64_t)(p->n - 1) * ldw + p->k) * 2;
    const uint64_t c_bytes = ((uint64_t)(p->m - 1) * ldc + p->n) * ec;
    if (x->a_off > ab->len || a_bytes > ab->len - x->a_off) return invalid("A buffer too small");
    // the kernel addresses A and W with 32-bit byte offsets from their first element
    if (a_bytes >= (1ull << 32) || w_bytes >= (1ull << 32)) return unavailable("operand spans 4 GiB or more");
    for (int i = 0; i < groups; i++) {
        const Buffer* wb = static_cast<const Buffer*>(ws[i]);
        const Buffer* cb = static_cast<const Buffer*>(cs[i]);
        if (!wb || !cb || !wb->ptr || !cb->ptr) return invalid("null buffer");
        if (w_offs[i] % 16 != 0 || (ldw * 2) % 16 != 0 || ((uintptr_t)wb->ptr % 16) != 0) return invalid("W rows not 16-byte aligned");
        if (w_offs[i] > wb->len || w_bytes > wb->len - w_offs[i]) return invalid("W buffer too small");
        if (x->c_off > cb->len || c_bytes > cb->len - x->c_off) return invalid("C buffer too small");
    }
    for (int i = 0; i < groups; i++) mark_unstable(cs[i]); // kernels are about to write them
    if (!g_gemm_setup_done) {
        hipError_t e = gemm_setup();
        if (e != hipSuccess) {
            set_err("gemm_setup: %s", hipGetErrorString(e));
            return ZDRAW_HIP_ERR_HANDLE;
        }
        g_gemm_setup_done = true;
    }
    GemmArgs g;
    memset(&g, 0, sizeof(g));
    g.a = static_cast<const char*>(ab->ptr) + x->a_off;
    g.w = static_cast<const char*>(static_cast<const Buffer*>(ws[0])->ptr) + w_offs[0];
    g.c = static_cast<char*>(static_cast<const Buffer*>(cs[0])->ptr) + x->c_off;
    g.groups = groups;
    for (int i = 1; i < groups; i++) {
        g.w_more[i - 1] = static_cast<const char*>(static_cast<const Buffer*>(ws[i])->ptr) + w_offs[i];
        g.c_more[i - 1] = static_cast<char*>(static_cast<const Buffer*>(cs[i])->ptr) + x->c_off;
    }
    g.m = (int32_t)p->m; g.n = (int32_t)p->n; g.k = (int32_t)p->k;
    g.lda = (int64_t)lda; g.ldw = (int64_t)ldw; g.ldc = (int64_t)ldc;
    g.tiles_n = (int32_t)((p->n + (uint32_t)gemm_tile_cols() - 1) / (uint32_t)gemm_tile_cols());
    if ((uint64_t)g.tiles_n * (uint64_t)groups * ((p->m + (uint32_t)gemm_tile_rows() - 1) / (uint32_t)gemm_tile_rows()) > 0x7fffffffull)
        return unavailable("grid too large");
    int a_eff = (int)x->a_dtype;
    if (const size_t rb = gemm_round_bytes(g, (int)x->a_dtype)) {
        // f32 activations are rounded to the weight's type once, into scratch slot 6, and the
        // product then runs as for 16-bit activations
        Buffer* a16 = queue_scratch(queue, 6, rb);
        if (!a16) {
            set_err("scratch allocation failed");
            return ZDRAW_HIP_ERR_HANDLE;
        }
        g.a16 = a16->ptr;
        a_eff = (int)wt;
    }
    {
        // a last round of tiles that fills at most half the CUs runs split along k; its fp32
        // partial tiles go through scratch slot 5
        int tail = 0, splits = 1;
        gemm_tail_plan(g, a_eff, queue->dev->cus, &tail, &splits);
        if (splits > 1) {
            Buffer* part = queue_scratch(queue, 5, gemm_part_bytes(tail, splits));
            if (!part) {
                set_err("scratch allocation failed");
                return ZDRAW_HIP_ERR_HANDLE;
            }
            g.splits = splits;
            g.tile_base = tail; // launch_gemm reads the tail size here
            g.part = static_cast<float*>(part->ptr);
        }
    }
    hipError_t e = launch_gemm(g, (int)x->a_dtype, (int)wt, (int)x->c_dtype, queue->stream);
    if (e != hipSuccess) {
        set_err("gemm launch: %s", hipGetErrorString(e));
        return ZDRAW_HIP_ERR_HANDLE;
    }
    g_dispatch++;
    return ZDRAW_HIP_OK;
}

int enqueue_gemm(void* a, void* w, void* c, const ZdrawGemmParams* p, const ZdrawHipGemmExt* x, Queue* queue) {
    if (!p) {
        set_err("null params");
        return ZDRAW_HIP_ERR_HANDLE;
    }
    return enqueue_gemm_group(a, &w, &c, &p->weight_offset, 1, p, x, queue);
}

} // namespace

extern "C" {

// ---------------------------------------------------------------- lifecycle
void* zdraw_hip_create_device(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || n <= 0) {
        set_err("no HIP device");
        return nullptr;
    }
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, 0) != hipSuccess) {
        set_err("hipGetDeviceProperties failed");
        return nullptr;
    }
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        set_err("device 0 is %s; this library is built for gfx950 only", prop.gcnArchName);
        return nullptr;
    }
    if (hipSetDevice(0) != hipSuccess) return nullptr;
    // One-time setup with the device current: the attention kernels' LDS limits (this also loads
    // their code), and this device's address of the no-allocation entry's scratch array.
    if (!g_setup_done) {
        hipError_t e = attention_setup();
        if (e != hipSuccess) {
            set_err("attention_setup: %s", hipGetErrorString(e));
            return nullptr;
        }
        g_setup_done = true;
    }
    const int ordinal = 0;
    if (!g_noalloc_scratch[ordinal]) {
        void* ptr = nullptr;
        hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr) {
            set_err("hipGetSymbolAddress(scratch): %s", hipGetErrorString(e));
            return nullptr;
        }
        g_noalloc_scratch[ordinal] = ptr;
    }
    g_weight_max.reserve(256); // no host allocation when a call notes a weight buffer's maximum
    Device* d = new Device{ordinal, prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256};
    return d;
}

void zdraw_hip_release_device(void* device) { delete static_cast<Device*>(device); }

void* zdraw_hip_create_queue(void* device) {
    Device* d = static_cast<Device*>(device);
    if (!d) return nullptr;
    hipStream_t s;
    if (hipStreamCreateWithFlags(&s, hipStreamNonBlocking) != hipSuccess) {
        set_err("hipStreamCreate failed");
        return nullptr;
    }
    Queue* nq = new Queue;
    nq->dev = d;
    nq->stream = s;
    return nq;
}

// Measurement aid (include/zdraw_hip_measure.h): a queue whose stream is confined to `cu_count`
// compute units (mask bit i set for i < cu_count; the driver deals the bits out over the XCDs
// in turn). It answers "does the kernel's time depend on how many CUs it has, or on the
// board's power limit".
void* zdraw_hip_create_queue_on_cus(void* device, int cu_count) {
    Device* d = static_cast<Device*>(device);
    if (!d) return nullptr;
    if (cu_count <= 0 || cu_count >= d->cus) return zdraw_hip_create_queue(device);
    hipStream_t s;
    std::vector<uint32_t> mask((size_t)(d->cus + 31) / 32, 0u);
    for (int i = 0; i < cu_count; i++) mask[(size_t)i >> 5] |= 1u << (i & 31);
    if (hipExtStreamCreateWithCUMask(&s, (uint32_t)mask.size(), mask.data()) != hipSuccess) {
        set_err("hipExtStreamCreateWithCUMask failed");
        return nullptr;
    }
    Queue* nq = new Queue;
    nq->dev = d;
    nq->stream = s;
    return nq;
}

void zdraw_hip_release_queue(void* queue) {
    Queue* q = static_cast<Queue*>(queue);
    if (!q) return;
    (void)hipStreamSynchronize(q->stream);
    for (Buffer*& b : q->scratch) {
        if (b) {
            if (b->ptr) (void)hipFree(b->ptr);
            delete b;
            b = nullptr;
        }
    }
    (void)hipStreamDestroy(q->stream);
    delete q;
}

// ------------------------------------------------------------------ buffers
void* zdraw_hip_create_buffer(void* device, size_t size) {
    if (!device || size == 0) return nullptr;
    void* p = nullptr;
    if (hipMalloc(&p, size) != hipSuccess) {
        set_err("hipMalloc(%zu) failed", size);
        return nullptr;
    }
    return new Buffer{p, size, true, true};
}

void* zdraw_hip_create_buffer_with_data(void* device, const uint8_t* data, size_t size) {
    if (!data) return nullptr;
    Buffer* b = static_cast<Buffer*>(zdraw_hip_create_buffer(device, size));
    if (!b) return nullptr;
    if (hipMemcpy(b->ptr, data, size, hipMemcpyHostToDevice) != hipSuccess) {
        zdraw_hip_release_buffer(b);
        set_err("upload failed");
        return nullptr;
    }
    return b;
}

// metal_api.m:601-638 wraps the caller's host pages (unified memory). A discrete GPU reads its
// own memory: the bytes are uploaded once and the caller keeps owning the source.
void* zdraw_hip_create_buffer_no_copy(void* device, const uint8_t* data, size_t size) {
    return zdraw_hip_create_buffer_with_data(device, data, size);
}

void* zdraw_hip_wrap_device_memory(void* device, void* device_ptr, size_t size) {
    Device* d = static_cast<Device*>(device);
    if (!d || !device_ptr || size == 0) return nullptr;
    // only memory the runtime knows as a device allocation on this device, and only a range
    // that lies inside that allocation, may reach a kernel
    hipPointerAttribute_t attr;
    memset(&attr, 0, sizeof(attr));
    if (hipPointerGetAttributes(&attr, device_ptr) != hipSuccess) {
        (void)hipGetLastError(); // a plain host pointer is reported as an error: clear it
        set_err("wrap_device_memory: not memory the HIP runtime knows");
        return nullptr;
    }
    if (attr.type != hipMemoryTypeDevice || attr.device != d->ordinal) {
        set_err("wrap_device_memory: not device memory of device %d", d->ordinal);
        return nullptr;
    }
    hipDeviceptr_t base = nullptr;
    size_t span = 0;
    if (hipMemGetAddressRange(&base, &span, device_ptr) != hipSuccess) {
        (void)hipGetLastError();
        set_err("wrap_device_memory: no allocation around the pointer");
        return nullptr;
    }
    const uintptr_t lo = (uintptr_t)base, p = (uintptr_t)device_ptr;
    if (p < lo || size > span || p - lo > span - size) {
        set_err("wrap_device_memory: %zu bytes do not fit the allocation", size);
        return nullptr;
    }
    return new Buffer{device_ptr, size, false, false};
}

void zdraw_hip_read_buffer(void* buffer, uint8_t* dst, size_t size) {
    Buffer* b = static_cast<Buffer*>(buffer);
    if (!b || !dst || size > b->len) return;
    (void)hipMemcpy(dst, b->ptr, size, hipMemcpyDeviceToHost);
}

void zdraw_hip_write_buffer(void* buffer, const uint8_t* src, size_t size) {
    Buffer* b = static_cast<Buffer*>(buffer);
    if (!b || !src || size > b->len) return;
    forget_weight_max(b);
    (void)hipMemcpy(b->ptr, src, size, hipMemcpyHostToDevice);
}

size_t zdraw_hip_buffer_length(void* buffer) {
    Buffer* b = static_cast<Buffer*>(buffer);
    return b ? b->len : 0;
}

void* zdraw_hip_buffer_device_ptr(void* buffer) {
    Buffer* b = static_cast<Buffer*>(buffer);
    if (!b) return nullptr;
    mark_unstable(b); // whoever holds the address can write the bytes
    return b->ptr;
}

int zdraw_hip_read_buffer_any(void* queue, void* buffer, uint8_t* dst, size_t size) {
    Queue* q = static_cast<Queue*>(queue);
    Buffer* b = static_cast<Buffer*>(buffer);
    if (!q || !b || !b->ptr || !dst || size > b->len) return ZDRAW_HIP_ERR_HANDLE;
    hipError_t e = hipStreamSynchronize(q->stream);
    if (e == hipSuccess) e = hipMemcpy(dst, b->ptr, size, hipMemcpyDeviceToHost);
    return e == hipSuccess ? ZDRAW_HIP_OK : hip_fail(e, "read_buffer_any");
}

void zdraw_hip_release_buffer(void* buffer) {
    Buffer* b = static_cast<Buffer*>(buffer);
    if (!b) return;
    if (b->ptr) forget_weight_max(b);
    if (b->owned && b->ptr) (void)hipFree(b->ptr);
    delete b;
}

void zdraw_hip_release_weight_buffer(void* buffer) { zdraw_hip_release_buffer(buffer); }

// ---------------------------------------------------------------- pipelines
void* zdraw_hip_compile(void* device, const char* source, const char* entry, char* error_buf, size_t error_len) {
    (void)source; // the kernels were compiled ahead of time; the reference's call sites pass their shader text here
    if (error_buf && error_len) error_buf[0] = '\0';
    if (!device || !entry) return nullptr;
    if (strcmp(entry, "attention_block_mfma") == 0) return new Pipeline{0};
    if (strcmp(entry, "qk_norm_rope") == 0) return new Pipeline{1};
    if (strcmp(entry, "gemm_half") == 0) return new Pipeline{2};
    if (strcmp(entry, "attention_wide_mfma") == 0) return new Pipeline{3};
    if (error_buf && error_len) snprintf(error_buf, error_len, "no gfx950 kernel named '%s'", entry);
    return nullptr;
}

void zdraw_hip_release_pipeline(void* pipeline) { delete static_cast<Pipeline*>(pipeline); }

size_t zdraw_hip_pipeline_threads(void* pipeline) {
    Pipeline* p = static_cast<Pipeline*>(pipeline);
    if (!p) return 0;
    if (p->kind == 2 || p->kind == 3) return 512;
    return p->kind == 0 ? ((g_variant & 1) == 0 ? 512 : 256) : 256;
}

// ---------------------------------------------------------------- attention
int zdraw_hip_run_attention(void* queue, void* pipeline, void* q, void* k, void* v, void* output,
                            const ZdrawAttnParams* params, uint32_t kernel, size_t thread_count) {
    (void)thread_count;
    Queue* qu = static_cast<Queue*>(queue);
    if (!qu || !params) {
        set_err("null queue or params");
        return ZDRAW_HIP_ERR_HANDLE;
    }
    const bool wide = pipeline && static_cast<Pipeline*>(pipeline)->kind == 3;
    int rc = check_pipeline(pipeline, kernel, wide ? 3 : 0);
    if (rc != ZDRAW_HIP_OK) return rc;
    ZdrawHipAttnExt x;
    FusedPlan plan;
    if (!wide) {
        standalone_ext(params, 0, 0, &x);
        ScratchSource slots(qu);
        rc = plan_attention(qu->dev, q, k, v, output, params, &x, nullptr, &plan, &slots);
        if (rc != ZDRAW_HIP_OK) return rc;
    }
    hipEvent_t start, stop;
    if (hipEventCreate(&start) != hipSuccess || hipEventCreate(&stop) != hipSuccess) return ZDRAW_HIP_ERR_HANDLE;
    (void)hipEventRecord(start, qu->stream);
    rc = wide ? enqueue_wide(qu, q, k, v, output, params, 0, 0) : enqueue(plan, qu->stream);
    if (rc == ZDRAW_HIP_OK) rc = finish_blocking(qu, start, stop);
    (void)hipEventDestroy(start);
    (void)hipEventDestroy(stop);
    return rc;
}

void* zdraw_hip_batch_begin(void* queue) {
    Queue* qu = static_cast<Queue*>(queue);
    if (!qu) return nullptr;
    Batch* b = new Batch{qu, nullptr, nullptr};
    if (hipEventCreate(&b->start) != hipSuccess || hipEventCreate(&b->stop) != hipSuccess ||
        hipEventRecord(b->start, qu->stream) != hipSuccess) {
        delete b;
        return nullptr;
    }
    return b;
}

int zdraw_hip_run_attention_enc_off(void* batch, void* pipeline, void* q, void* k, void* v, void* o,
                                    const ZdrawAttnParams* params, uint32_t kernel, size_t thread_count,
                                    uint64_t in_off, uint64_t out_off) {
    (void)thread_count;
    Batch* b = static_cast<Batch*>(batch);
    if (!b || !params) {
        set_err("null batch or params");
        return ZDRAW_HIP_ERR_HANDLE;
    }
    const bool wide = pipeline && static_cast<Pipeline*>(pipeline)->kind == 3;
    int rc = check_pipeline(pipeline, kernel, wide ? 3 : 0);
    if (rc != ZDRAW_HIP_OK) return rc;
    if (wide) return enqueue_wide(b->queue, q, k, v, o, params, in_off, out_off);
    ZdrawHipAttnExt x;
    standalone_ext(params, in_off, out_off, &x);
    FusedPlan plan;
    ScratchSource slots(b->queue);
    rc = plan_attention(b->queue->dev, q, k, v, o, params, &x, nullptr, &plan, &slots);
    if (rc != ZDRAW_HIP_OK) return rc;
    return enqueue(plan, b->queue->stream);
}

int zdraw_hip_run_attention_enc(void* batch, void* pipeline, void* q, void* k, void* v, void* o,
                                const ZdrawAttnParams* params, uint32_t kernel, size_t thread_count) {
    return zdraw_hip_run_attention_enc_off(batch, pipeline, q, k, v, o, params, kernel, thread_count, 0, 0);
}

int zdraw_hip_batch_end(void* batch) {
    Batch* b = static_cast<Batch*>(batch);
    if (!b) return ZDRAW_HIP_ERR_HANDLE;
    int rc = finish_blocking(b->queue, b->start, b->stop);
    (void)hipEventDestroy(b->start);
    (void)hipEventDestroy(b->stop);
    delete b;
    return rc;
}

int zdraw_hip_run_attention_fused_enc(void* batch, void* q, void* k, void* v, void* out,
                                      const ZdrawAttnParams* params, const ZdrawHipAttnExt* ext,
                                      const ZdrawHipQkOperands* ops) {
    Batch* b = static_cast<Batch*>(batch);
    if (!b) {
        set_err("null batch");
        return ZDRAW_HIP_ERR_HANDLE;
    }
    FusedPlan plan;
    ScratchSource slots(b->queue);
    int rc = plan_attention(b->queue->dev, q, k, v, out, params, ext, ops, &plan, &slots);
    if (rc != ZDRAW_HIP_OK) return rc;
    return enqueue(plan, b->queue->stream);
}

int zdraw_hip_reserve_attention_fused(void* queue, void* q, void* k, void* v, void* out, const ZdrawAttnParams* params,
                                      const ZdrawHipAttnExt* ext, const ZdrawHipQkOperands* ops) {
    Queue* qu = static_cast<Queue*>(queue);
    if (!qu) {
        set_err("null queue");
        return ZDRAW_HIP_ERR_HANDLE;
    }
    // planning grows the queue's scratch slots to what the call needs (and reads the norm
    // weights back for the score bound); nothing is enqueued
    FusedPlan plan;
    ScratchSource slots(qu);
    return plan_attention(qu->dev, q, k, v, out, params, ext, ops, &plan, &slots);
}

int zdraw_hip_run_attention_fused_noalloc_enc(void* batch, void* q, void* k, void* v, void* out,
                                              const ZdrawAttnParams* params, const ZdrawHipAttnExt* ext,
                                              const ZdrawHipQkOperands* ops) {
    Batch* b = static_cast<Batch*>(batch);
    if (!b) {
        set_err("null batch");
        return ZDRAW_HIP_ERR_HANDLE;
    }
    Device* dev = b->queue->dev;
    void* base = (dev->ordinal >= 0 && dev->ordinal < kMaxDevices) ? g_noalloc_scratch[dev->ordinal] : nullptr;
    if (!base) {
        set_err("no scratch array address for this device");
        return ZDRAW_HIP_ERR_HANDLE;
    }
    // The array keeps the previous call's contents. Nothing in it has to start at zero: the
    // pre-pass writes every prepared row before the attention kernel reads it, and the key-split
    // parts write every row of every part before the merge reads them, in stream order.
    ScratchSource span(b->queue, base, kNoallocScratchBytes);
    FusedPlan plan;
    int rc = plan_attention(dev, q, k, v, out, params, ext, ops, &plan, &span);
    if (rc != ZDRAW_HIP_OK) return rc;
    return enqueue(plan, b->queue->stream, /*no_alloc=*/true);
}

int zdraw_hip_run_attention_fused(void* queue, void* q, void* k, void* v, void* out,
                                  const ZdrawAttnParams* params, const ZdrawHipAttnExt* ext,
                                  const ZdrawHipQkOperands* ops) {
    void* b = zdraw_hip_batch_begin(queue);
    if (!b) {
        set_err("null queue");
        return ZDRAW_HIP_ERR_HANDLE;
    }
    int rc = zdraw_hip_run_attention_fused_enc(b, q, k, v, out, params, ext, ops);
    int rc2 = zdraw_hip_batch_end(b);
    return rc != ZDRAW_HIP_OK ? rc : rc2;
}

namespace {
// In-place norm + rope of q (then k) on f32 token-major rows: one pre-pass launch each.
// nw == nullptr: norm weights are f32[128] at offset 0.
int run_qk_norm_rope_impl(void* queue, void* pipeline, void* q, void* k, const ZdrawAttnParams* p,
                          const ZdrawHipAttnExt* x, const ZdrawHipQkOperands* ops, const NormWeights* nw) {
    Queue* qu = static_cast<Queue*>(queue);
    if (!qu || !p || !x || !ops) {
        set_err("null argument");
        return ZDRAW_HIP_ERR_HANDLE;
    }
    int rc = check_pipeline(pipeline, 0, 1);
    if (rc != ZDRAW_HIP_OK) return rc;
    if (p->tokens == 0) return unavailable("tokens == 0");
    if (p->heads == 0 || p->kv_heads == 0) return invalid("zero dimension");
    if (p->head_dim != (uint32_t)kHeadDim) return unavailable("head_dim != 128");
    if (x->qk_mode != ZDRAW_HIP_QK_KLEIN && x->qk_mode != ZDRAW_HIP_QK_ZIMAGE) return invalid("qk_mode");
    // Reuse the attention planner's operand validation by planning a
    // same-shape launch over q (then k); nothing is enqueued from the plan
    // except the pre-pass arguments assembled below. Both operands are checked
    // before the first launch, so a refused call leaves q untouched.
    PrepArgs prs[2];
    bool stage_w = false;
    WeightStageArgs stage;
    for (int which = 0; which < 2; which++) {
        ZdrawAttnParams sp = *p;
        sp.heads = sp.kv_heads = which == 0 ? p->heads : p->kv_heads;
        sp.causal = 0;
        sp.valid = 0;
        ZdrawHipAttnExt sx;
        standalone_ext(&sp, 0, 0, &sx);
        sx.qk_mode = x->qk_mode;
        sx.k_site = ZDRAW_HIP_K_PREPASS; // typed norm weights are the pre-pass kernel's
        sx.eps = x->eps;
        sx.txt_rows = x->txt_rows;
        sx.rope_batch_rows = x->rope_batch_rows;
        memcpy(sx.zimage_dims, x->zimage_dims, sizeof(sx.zimage_dims));
        memcpy(sx.zimage_base, x->zimage_base, sizeof(sx.zimage_base));
        void* buf = which == 0 ? q : k;
        FusedPlan plan;
        ScratchSource none(qu, /*dry=*/true);
        rc = plan_attention(qu->dev, buf, buf, buf, buf, &sp, &sx, ops, &plan, &none, nw);
        if (rc != ZDRAW_HIP_OK) return rc;
        // the plan's pre-pass describes the in-place form: same strides in and out, f32 out, no scale
        PrepArgs pr = which == 0 ? plan.prep_q : plan.prep;
        pr.y = const_cast<void*>(pr.x);
        pr.y_bs = pr.x_bs; pr.y_ts = pr.x_ts; pr.y_hs = pr.x_hs;
        pr.batch = 1;
        pr.out_dtype = kF32;
        pr.scale = 1.0f;
        prs[which] = pr;
        // both plans stage the same two weight vectors into the same place: one launch serves both
        stage_w = plan.stage_w;
        stage = plan.stage;
    }
    if (stage_w) {
        hipError_t e = launch_weight_stage(stage, qu->stream);
        if (e != hipSuccess) {
            set_err("norm weight staging launch: %s", hipGetErrorString(e));
            return ZDRAW_HIP_ERR_HANDLE;
        }
        g_dispatch++;
    }
    for (int which = 0; which < 2; which++) {
        hipError_t e = launch_qk_prepass(&prs[which], 1, kF32, qu->stream);
        if (e != hipSuccess) {
            set_err("qk_norm_rope launch: %s", hipGetErrorString(e));
            return ZDRAW_HIP_ERR_HANDLE;
        }
        g_dispatch++;
    }
    hipError_t e = hipStreamSynchronize(qu->stream);
    if (e != hipSuccess) return hip_fail(e, "qk_norm_rope wait");
    g_command++;
    return ZDRAW_HIP_OK;
}
} // namespace

int zdraw_hip_run_qk_norm_rope_ext(void* queue, void* pipeline, void* q, void* k, const ZdrawAttnParams* p,
                                   const ZdrawHipAttnExt* x, const ZdrawHipQkOperands* ops) {
    return run_qk_norm_rope_impl(queue, pipeline, q, k, p, x, ops, nullptr);
}

// metal_c.zig:148-159, the dispatch behind mqk.run (metal/mqk.zig:20-58; kernel
// metal/mqk_shader.zig:46-97, encode metal_api.m:6215-6265).
int zdraw_hip_run_qk_norm_rope(void* queue, void* pipeline, void* q, void* k, void* q_weight, void* k_weight,
                               void* pos, void* rope, const ZdrawQkNormParams* qp, size_t thread_count) {
    (void)thread_count;
    if (!qp) {
        set_err("null params");
        return ZDRAW_HIP_ERR_HANDLE;
    }
    ZdrawAttnParams p;
    memset(&p, 0, sizeof(p));
    p.tokens = qp->tokens;
    p.heads = qp->heads;
    p.kv_heads = qp->kv_heads;
    p.head_dim = qp->head_dim;
    ZdrawHipAttnExt x;
    memset(&x, 0, sizeof(x));
    x.qk_mode = ZDRAW_HIP_QK_ZIMAGE;
    x.eps = qp->eps;
    x.zimage_dims[0] = qp->dim0; x.zimage_dims[1] = qp->dim1; x.zimage_dims[2] = qp->dim2;
    x.zimage_base[0] = qp->base0; x.zimage_base[1] = qp->base1; x.zimage_base[2] = qp->base2;
    ZdrawHipQkOperands ops;
    memset(&ops, 0, sizeof(ops));
    ops.q_weight = q_weight;
    ops.k_weight = k_weight;
    ops.pos = pos;
    ops.rope_pairs = rope;
    const NormWeights nw{qp->q_dtype, qp->k_dtype, qp->q_offset, qp->k_offset};
    return run_qk_norm_rope_impl(queue, pipeline, q, k, &p, &x, &ops, &nw);
}

// --------------------------------------------------------------------- gemm
int zdraw_hip_run_gemm_ext_enc(void* batch, void* a, void* w, void* c, const ZdrawGemmParams* params,
                               const ZdrawHipGemmExt* ext) {
    Batch* b = static_cast<Batch*>(batch);
    if (!b) {
        set_err("null batch");
        return ZDRAW_HIP_ERR_HANDLE;
    }
    return enqueue_gemm(a, w, c, params, ext, b->queue);
}

int zdraw_hip_run_gemm_off_enc(void* batch, void* pipeline, void* a, void* w, void* c,
                               const ZdrawGemmParams* params, uint64_t a_offset, uint64_t c_offset) {
    int rc = check_pipeline(pipeline, 0, 2);
    if (rc != ZDRAW_HIP_OK) return rc;
    ZdrawHipGemmExt x;
    memset(&x, 0, sizeof(x));
    x.a_off = a_offset;
    x.c_off = c_offset;
    x.a_dtype = ZDRAW_HIP_F32;
    x.c_dtype = ZDRAW_HIP_F32;
    return zdraw_hip_run_gemm_ext_enc(batch, a, w, c, params, &x);
}

int zdraw_hip_run_gemm_enc(void* batch, void* pipeline, void* a, void* w, void* c, const ZdrawGemmParams* params) {
    return zdraw_hip_run_gemm_off_enc(batch, pipeline, a, w, c, params, 0, 0);
}

int zdraw_hip_run_gemm_f16a_enc(void* batch, void* a, void* w, void* c, const ZdrawGemmParams* params,
                                uint64_t a_offset, uint64_t c_offset) {
    if (!params) {
        set_err("null params");
        return ZDRAW_HIP_ERR_HANDLE;
    }
    ZdrawHipGemmExt x;
    memset(&x, 0, sizeof(x));
    x.a_off = a_offset;
    x.c_off = c_offset;
    x.a_dtype = params->dtype == ZDRAW_HIP_W_F16 ? ZDRAW_HIP_F16 : ZDRAW_HIP_BF16;
    x.c_dtype = ZDRAW_HIP_F32;
    return zdraw_hip_run_gemm_ext_enc(batch, a, w, c, params, &x);
}

int zdraw_hip_run_gemm(void* queue, void* pipeline, void* a, void* w, void* c, const ZdrawGemmParams* params) {
    void* b = zdraw_hip_batch_begin(queue);
    if (!b) {
        set_err("null queue");
        return ZDRAW_HIP_ERR_HANDLE;
    }
    int rc = zdraw_hip_run_gemm_enc(b, pipeline, a, w, c, params);
    int rc2 = zdraw_hip_batch_end(b);
    return rc != ZDRAW_HIP_OK ? rc : rc2;
}

namespace {
// Two or three products of the same f32 A (metal_api.m zdraw_metal_run_gemm_pair / _triple):
// one grouped launch when the shapes and weight types agree, one launch each otherwise.
// `count` products of one A into an open batch: one grouped launch when shapes and weight
// types agree, else one launch each; a product this backend does not run refuses the call
// before anything is enqueued.
int enqueue_gemm_several(Batch* b, void* a, void* const* ws, void* const* cs, const ZdrawGemmParams* const* ps, int count,
                         const ZdrawHipGemmExt* x) {
    for (int i = 0; i < count; i++) {
        if (ps[i]->mode != ZDRAW_HIP_GEMM_HALF || (ps[i]->dtype != ZDRAW_HIP_W_F16 && ps[i]->dtype != ZDRAW_HIP_W_BF16) ||
            (ps[i]->k % 8 != 0 && ps[i]->m != 0 && ps[i]->k != 0 && ps[i]->n != 0))
            return unavailable("a product of the group is not a 16-bit-weight half-mode GEMM with k % 8 == 0");
    }
    bool same = true;
    for (int i = 1; i < count; i++)
        same = same && ps[i]->m == ps[0]->m && ps[i]->k == ps[0]->k && ps[i]->n == ps[0]->n &&
               ps[i]->dtype == ps[0]->dtype && ps[i]->mode == ps[0]->mode;
    int rc = ZDRAW_HIP_OK;
    if (same) {
        uint64_t offs[3];
        for (int i = 0; i < count; i++) offs[i] = ps[i]->weight_offset;
        rc = enqueue_gemm_group(a, ws, cs, offs, count, ps[0], x, b->queue);
    } else {
        for (int i = 0; i < count && rc == ZDRAW_HIP_OK; i++) rc = enqueue_gemm(a, ws[i], cs[i], ps[i], x, b->queue);
    }
    return rc;
}

int run_gemm_several(void* queue, void* pipeline, void* a, void* const* ws, void* const* cs,
                     const ZdrawGemmParams* const* ps, int count) {
    int rc = check_pipeline(pipeline, 0, 2);
    if (rc != ZDRAW_HIP_OK) return rc;
    for (int i = 0; i < count; i++)
        if (!ps[i]) {
            set_err("null params");
            return ZDRAW_HIP_ERR_HANDLE;
        }
    Batch* b = static_cast<Batch*>(zdraw_hip_batch_begin(queue));
    if (!b) {
        set_err("null queue");
        return ZDRAW_HIP_ERR_HANDLE;
    }
    ZdrawHipGemmExt x;
    memset(&x, 0, sizeof(x));
    x.a_dtype = ZDRAW_HIP_F32;
    x.c_dtype = ZDRAW_HIP_F32;
    rc = enqueue_gemm_several(b, a, ws, cs, ps, count, &x);
    const int rc2 = zdraw_hip_batch_end(b);
    return rc != ZDRAW_HIP_OK ? rc : rc2;
}
} // namespace

int zdraw_hip_run_gemm_group_ext_enc(void* batch, void* a, void* const* ws, void* const* cs,
                                     const ZdrawGemmParams* const* params, uint32_t count, const ZdrawHipGemmExt* ext) {
    Batch* b = static_cast<Batch*>(batch);
    if (!b || !ws || !cs || !params || !ext || count < 1 || count > 3) {
        set_err("null batch, arrays or ext, or count outside 1..3");
        return ZDRAW_HIP_ERR_HANDLE;
    }
    for (uint32_t i = 0; i < count; i++)
        if (!params[i]) {
            set_err("null params");
            return ZDRAW_HIP_ERR_HANDLE;
        }
    return enqueue_gemm_several(b, a, ws, cs, params, (int)count, ext);
}

int zdraw_hip_run_gemm_pair(void* queue, void* pipeline, void* a, void* w0, void* c0, const ZdrawGemmParams* params0,
                            void* w1, void* c1, const ZdrawGemmParams* params1) {
    void* const ws[2] = {w0, w1};
    void* const cs[2] = {c0, c1};
    const ZdrawGemmParams* const ps[2] = {params0, params1};
    return run_gemm_several(queue, pipeline, a, ws, cs, ps, 2);
}

int zdraw_hip_run_gemm_triple(void* queue, void* pipeline, void* a, void* w0, void* c0, const ZdrawGemmParams* params0,
                              void* w1, void* c1, const ZdrawGemmParams* params1, void* w2, void* c2,
                              const ZdrawGemmParams* params2) {
    void* const ws[3] = {w0, w1, w2};
    void* const cs[3] = {c0, c1, c2};
    const ZdrawGemmParams* const ps[3] = {params0, params1, params2};
    return run_gemm_several(queue, pipeline, a, ws, cs, ps, 3);
}

// ------------------------------------------------ Z-Image layer, attention segment
int zdraw_hip_run_chain_attn_enc(void* batch, const ZdrawHipChainAttnBuffers* bufs,
                                 const ZdrawHipChainAttnWeights* w, const ZdrawHipChainAttnParams* p) {
    Batch* b = static_cast<Batch*>(batch);
    if (!b || !bufs || !w || !p) {
        set_err("null argument");
        return ZDRAW_HIP_ERR_HANDLE;
    }
    const ZdrawAttnParams& at = p->attn;
    const uint64_t inner = (uint64_t)at.heads * at.head_dim;
    // the segment's shapes must agree with each other before anything is enqueued
    if (at.tokens == 0) return unavailable("tokens == 0");
    if (p->q.m != at.tokens || p->k.m != at.tokens || p->v.m != at.tokens || p->proj.m != at.tokens)
        return invalid("projection rows != attention tokens");
    if (p->q.n != inner || p->k.n != (uint64_t)at.kv_heads * at.head_dim || p->v.n != p->k.n || p->proj.k != inner)
        return invalid("projection widths != heads * head_dim");
    if (p->k.k != p->q.k || p->v.k != p->q.k) return invalid("q/k/v projections read different widths");
    if (p->qk.tokens != at.tokens || p->qk.heads != at.heads || p->qk.kv_heads != at.kv_heads || p->qk.head_dim != at.head_dim)
        return invalid("QkNormParams shape != AttnParams shape");
    if (p->act_dtype != ZDRAW_HIP_F32 && p->act_dtype != ZDRAW_HIP_BF16) return unavailable("activation dtype");
    const ZdrawGemmParams* gs[4] = {&p->q, &p->k, &p->v, &p->proj};
    for (const ZdrawGemmParams* g : gs) {
        if (g->mode != ZDRAW_HIP_GEMM_HALF) return unavailable("only the half-precision GEMM mode exists");
        if (g->dtype != ZDRAW_HIP_W_F16 && g->dtype != ZDRAW_HIP_W_BF16) return unavailable("weight dtype");
        if (p->act_dtype == ZDRAW_HIP_BF16 && g->dtype != ZDRAW_HIP_W_BF16) return unavailable("bf16 activations need bf16 weights");
        if (g->k % 8 != 0) return unavailable("k % 8 != 0");
    }

    ZdrawHipAttnExt x;
    memset(&x, 0, sizeof(x));
    const uint64_t row = inner;
    x.q_stride[0] = x.k_stride[0] = x.v_stride[0] = x.out_stride[0] = (uint64_t)at.tokens * row;
    x.q_stride[1] = x.k_stride[1] = x.v_stride[1] = x.out_stride[1] = row;
    x.q_stride[2] = x.k_stride[2] = x.v_stride[2] = x.out_stride[2] = at.head_dim;
    x.batch = 1;
    x.in_dtype = x.out_dtype = p->act_dtype;
    x.qk_mode = ZDRAW_HIP_QK_ZIMAGE;
    x.k_site = ZDRAW_HIP_K_PREPASS;
    x.eps = p->qk.eps;
    x.score_bound = p->score_bound;
    x.zimage_dims[0] = p->qk.dim0; x.zimage_dims[1] = p->qk.dim1; x.zimage_dims[2] = p->qk.dim2;
    x.zimage_base[0] = p->qk.base0; x.zimage_base[1] = p->qk.base1; x.zimage_base[2] = p->qk.base2;
    ZdrawHipQkOperands ops;
    memset(&ops, 0, sizeof(ops));
    ops.q_weight = w->q_norm;
    ops.k_weight = w->k_norm;
    ops.pos = w->pos;
    ops.rope_pairs = w->rope;
    const NormWeights nw{p->qk.q_dtype, p->qk.k_dtype, p->qk.q_offset, p->qk.k_offset};
    FusedPlan plan;
    ScratchSource slots(b->queue);
    int rc = plan_attention(b->queue->dev, bufs->q, bufs->k, bufs->v, bufs->mix, &at, &x, &ops, &plan, &slots, &nw);
    if (rc != ZDRAW_HIP_OK) return rc;

    ZdrawHipGemmExt gx;
    memset(&gx, 0, sizeof(gx));
    gx.a_dtype = gx.c_dtype = p->act_dtype;
    hipStream_t st = b->queue->stream;
    // a projection that is refused leaves nothing half-written that a later step
    // reads: the caller re-runs the whole segment on its own path
    // q, k and v read the same rows and have the same shape (kv_heads == heads was checked):
    // one launch whose tiles cover all three, so the last partly filled round of workgroups
    // is paid once instead of three times
    if (p->k.dtype == p->q.dtype && p->v.dtype == p->q.dtype) {
        void* const wsv[3] = {w->q, w->k, w->v};
        void* const csv[3] = {bufs->q, bufs->k, bufs->v};
        const uint64_t offs[3] = {p->q.weight_offset, p->k.weight_offset, p->v.weight_offset};
        if ((rc = enqueue_gemm_group(bufs->norm, wsv, csv, offs, 3, &p->q, &gx, b->queue)) != ZDRAW_HIP_OK) return rc;
    } else {
        if ((rc = enqueue_gemm(bufs->norm, w->q, bufs->q, &p->q, &gx, b->queue)) != ZDRAW_HIP_OK) return rc;
        if ((rc = enqueue_gemm(bufs->norm, w->k, bufs->k, &p->k, &gx, b->queue)) != ZDRAW_HIP_OK) return rc;
        if ((rc = enqueue_gemm(bufs->norm, w->v, bufs->v, &p->v, &gx, b->queue)) != ZDRAW_HIP_OK) return rc;
    }
    if ((rc = enqueue(plan, st)) != ZDRAW_HIP_OK) return rc;
    return enqueue_gemm(bufs->mix, w->proj, bufs->attn, &p->proj, &gx, b->queue);
}

// ------------------------------------------------------------------ scratch
void* zdraw_hip_attn_scratch(void* device, int slot, size_t bytes) {
    if (!device || slot < 0 || slot >= kCallerSlots || bytes == 0) return nullptr;
    // The caller's slots (the reference's process-static set, metal_api.m:6147-6191). The
    // library's own scratch lives with its queues, so nothing of the library reads these.
    return grow_slot(&g_scratch[slot], slot, bytes, [] { (void)hipDeviceSynchronize(); });
}

// --------------------------------------------------------- counters, timing
void zdraw_hip_metrics_reset(void) {
    (void)zdraw_hip_trace_attention_ns(nullptr);
    g_dispatch = g_command = g_fallback = g_gpu_ns = 0;
    g_trace_ns = g_trace_launches = 0;
}
uint64_t zdraw_hip_dispatch_count(void) { return g_dispatch; }
uint64_t zdraw_hip_command_count(void) { return g_command; }
uint64_t zdraw_hip_attn_fallback_count(void) { return g_fallback; }
uint64_t zdraw_hip_gpu_ns(void) { return g_gpu_ns; }

void* zdraw_hip_event_create(void) {
    hipEvent_t e;
    if (hipEventCreate(&e) != hipSuccess) return nullptr;
    return new Event{e};
}
int zdraw_hip_event_record(void* event, void* queue) {
    Event* e = static_cast<Event*>(event);
    Queue* q = static_cast<Queue*>(queue);
    if (!e || !q) return ZDRAW_HIP_ERR_HANDLE;
    return hipEventRecord(e->ev, q->stream) == hipSuccess ? ZDRAW_HIP_OK : ZDRAW_HIP_ERR_DEVICE;
}
int zdraw_hip_event_sync(void* event) {
    Event* e = static_cast<Event*>(event);
    if (!e) return ZDRAW_HIP_ERR_HANDLE;
    return hipEventSynchronize(e->ev) == hipSuccess ? ZDRAW_HIP_OK : ZDRAW_HIP_ERR_DEVICE;
}
float zdraw_hip_event_elapsed_ms(void* start, void* stop) {
    Event* a = static_cast<Event*>(start);
    Event* b = static_cast<Event*>(stop);
    float ms = -1.f;
    if (!a || !b || hipEventElapsedTime(&ms, a->ev, b->ev) != hipSuccess) return -1.f;
    return ms;
}
void zdraw_hip_event_release(void* event) {
    Event* e = static_cast<Event*>(event);
    if (!e) return;
    (void)hipEventDestroy(e->ev);
    delete e;
}
int zdraw_hip_queue_sync(void* queue) {
    Queue* q = static_cast<Queue*>(queue);
    if (!q) return ZDRAW_HIP_ERR_HANDLE;
    hipError_t e = hipStreamSynchronize(q->stream);
    return e == hipSuccess ? ZDRAW_HIP_OK : hip_fail(e, "queue sync");
}

void zdraw_hip_trace_attention(int on) { g_trace = on != 0; }

uint64_t zdraw_hip_trace_attention_ns(uint64_t* launches) {
    // fold every finished pair into the totals (waits for pairs still in flight)
    for (TracePair& tp : g_trace_open) {
        float ms = 0.f;
        if (hipEventSynchronize(tp.b) == hipSuccess && hipEventElapsedTime(&ms, tp.a, tp.b) == hipSuccess) {
            g_trace_ns += (uint64_t)((double)ms * 1e6);
            g_trace_launches++;
        }
        (void)hipEventDestroy(tp.a);
        (void)hipEventDestroy(tp.b);
    }
    g_trace_open.clear();
    if (launches) *launches = g_trace_launches;
    return g_trace_ns;
}

void zdraw_hip_clock_probe(int on) { g_clock_on = on != 0; }

size_t zdraw_hip_clock_probe_read(uint64_t* cycles, uint64_t* ref_ticks, size_t capacity) {
    if (!g_clock_buf || g_clock_wgs <= 0) return 0;
    if (hipStreamSynchronize(g_clock_stream) != hipSuccess) return 0;
    const size_t n = (size_t)(g_clock_wgs < kClockCap ? g_clock_wgs : kClockCap);
    std::vector<unsigned long long> host(2 * n);
    if (hipMemcpy(host.data(), g_clock_buf, sizeof(unsigned long long) * 2 * n, hipMemcpyDeviceToHost) != hipSuccess) return 0;
    const size_t m = n < capacity ? n : capacity;
    for (size_t i = 0; i < m; i++) {
        if (cycles) cycles[i] = host[2 * i];
        if (ref_ticks) ref_ticks[i] = host[2 * i + 1];
    }
    return m;
}

void zdraw_hip_set_attention_variant(int variant) { g_variant = variant & 3; }

void zdraw_hip_set_gemm_build(int build) { gemm_set_build(build); }

int zdraw_hip_wide_redo_tiles(void) {
    if (!g_last_wide_redo || g_last_wide_tiles <= 0) return -1;
    if (hipStreamSynchronize(g_last_wide_stream) != hipSuccess) return -1;
    std::vector<int> flags((size_t)g_last_wide_tiles);
    if (hipMemcpy(flags.data(), g_last_wide_redo, flags.size() * sizeof(int), hipMemcpyDeviceToHost) != hipSuccess) return -1;
    int n = 0;
    for (int f : flags) n += f != 0;
    return n;
}

void zdraw_hip_gemm_tail_plan(uint32_t m, uint32_t k, uint32_t n, uint32_t groups, uint32_t cus, uint32_t* tail_tiles,
                              uint32_t* splits) {
    GemmArgs g;
    memset(&g, 0, sizeof(g));
    g.m = (int32_t)m; g.k = (int32_t)k; g.n = (int32_t)n;
    g.groups = (int32_t)groups;
    int t = 0, s = 1;
    if (m && k && n && groups >= 1 && groups <= 3 && m <= 0x7fffffffu && k <= 0x7fffffffu && n <= 0x7fffffffu)
        gemm_tail_plan(g, (int)ZDRAW_HIP_BF16, (int)cus, &t, &s);
    if (tail_tiles) *tail_tiles = (uint32_t)t;
    if (splits) *splits = (uint32_t)s;
}

void zdraw_hip_attention_tail_plan(uint64_t tiles, uint32_t cus, uint32_t key_blocks, uint32_t* tail_tiles,
                                   uint32_t* splits) {
    int t = 0, s = 1;
    if (tiles <= 0x7fffffffull && cus <= 0x7fffffffu && key_blocks <= 0x7fffffffu)
        attention_tail_plan((int64_t)tiles, (int)cus, (int)key_blocks, &t, &s);
    if (tail_tiles) *tail_tiles = (uint32_t)t;
    if (splits) *splits = (uint32_t)s;
}

int zdraw_hip_zimage_axis_lens(uint64_t table_bytes, const uint64_t* base, const uint32_t* dims, uint32_t* lens) {
    if (!base || !dims || !lens) return ZDRAW_HIP_ERR_HANDLE;
    return zimage_axis_lens(table_bytes, base, dims, lens) ? ZDRAW_HIP_OK : ZDRAW_HIP_INVALID;
}

size_t zdraw_hip_abi_sizeof(int which) {
    switch (which) {
    case 0: return sizeof(ZdrawAttnParams);
    case 1: return sizeof(ZdrawHipAttnExt);
    case 2: return sizeof(ZdrawHipQkOperands);
    case 3: return sizeof(ZdrawGemmParams);
    case 4: return sizeof(ZdrawHipGemmExt);
    case 5: return sizeof(ZdrawQkNormParams);
    case 6: return sizeof(ZdrawHipChainAttnBuffers);
    case 7: return sizeof(ZdrawHipChainAttnWeights);
    case 8: return sizeof(ZdrawHipChainAttnParams);
    default: return 0;
    }
}

const char* zdraw_hip_last_error(void) { return g_err; }

} // extern "C"
