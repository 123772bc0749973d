// hattn::Context: the HIP-backed counterpart of metal/mattn.zig's Context.
#include "zdraw_host.hpp"

#include <cstring>

namespace zdraw {

Error fromCode(int rc) {
    switch (rc) {
    case ZDRAW_HIP_OK: return Error::Ok;
    case ZDRAW_HIP_UNAVAILABLE: return Error::UnsupportedShape;
    case ZDRAW_HIP_INVALID: return Error::InvalidShape;
    default: return Error::DispatchFailed; // mattn.zig:214: `if (code != 0) return error.MetalDispatchFailed`
    }
}

namespace hattn {

Buffer Buffer::fromBytes(void* device, const void* data, size_t size) {
    Buffer b;
    b.handle = zdraw_hip_create_buffer_with_data(device, static_cast<const uint8_t*>(data), size);
    b.owned = b.handle != nullptr;
    return b;
}
Buffer Buffer::empty(void* device, size_t size) {
    Buffer b;
    b.handle = zdraw_hip_create_buffer(device, size);
    b.owned = b.handle != nullptr;
    return b;
}
Buffer Buffer::borrow(void* handle) {
    Buffer b;
    b.handle = handle;
    b.owned = false;
    return b;
}
void Buffer::deinit() {
    if (owned && handle) zdraw_hip_release_buffer(handle);
    handle = nullptr;
    owned = false;
}

Error Context::init(Context* out) { return initKernel(Kernel::block, out); }

// mattn.zig:69-118 hands zdraw_metal_compile the shader text of each kernel; the gfx950
// kernels are compiled ahead of time, so there is no text to hand over.
static const char* const kNoSource = "";

Error Context::initKernel(Kernel kernel, Context* out) {
    Context c;
    c.device = zdraw_hip_create_device();
    if (!c.device) return Error::NotAvailable;
    c.queue = zdraw_hip_create_queue(c.device);
    if (!c.queue) {
        zdraw_hip_release_device(c.device);
        return Error::QueueFailed;
    }
    char err[256];
    c.block_pipeline = zdraw_hip_compile(c.device, kNoSource, "attention_block_mfma", err, sizeof(err));
    if (!c.block_pipeline) {
        zdraw_hip_release_queue(c.queue);
        zdraw_hip_release_device(c.device);
        return Error::CompileFailed;
    }
    c.qk_pipeline = zdraw_hip_compile(c.device, kNoSource, "qk_norm_rope", err, sizeof(err)); // optional, like mattn.zig:86
    c.wide_pipeline = zdraw_hip_compile(c.device, kNoSource, "attention_wide_mfma", err, sizeof(err)); // optional, mattn.zig:83-85
    c.wide_threads = c.wide_pipeline ? zdraw_hip_pipeline_threads(c.wide_pipeline) : 0;
    c.kernel = kernel;
    c.threads = zdraw_hip_pipeline_threads(c.block_pipeline);
    c.qk_threads = c.qk_pipeline ? zdraw_hip_pipeline_threads(c.qk_pipeline) : 0;
    *out = c;
    return Error::Ok;
}

void Context::deinit() {
    for (int i = 0; i < 4; i++) {
        if (pool[i]) zdraw_hip_release_buffer(pool[i]);
        pool[i] = nullptr;
        pool_bytes[i] = 0;
    }
    if (wide_pipeline) zdraw_hip_release_pipeline(wide_pipeline);
    if (qk_pipeline) zdraw_hip_release_pipeline(qk_pipeline);
    if (block_pipeline) zdraw_hip_release_pipeline(block_pipeline);
    if (queue) zdraw_hip_release_queue(queue);
    if (device) zdraw_hip_release_device(device);
    *this = Context{};
}

bool Context::pick(size_t tokens, size_t head_dim, Pick* out) const {
    (void)tokens;
    // mattn.zig:134-150 routes by head_dim and token count between three
    // kernels; here one kernel covers every token count at head_dim 128 and
    // there is none for other widths.
    if (head_dim != flash_head_dim || !block_pipeline) return false;
    *out = Pick{Kernel::block, block_pipeline, threads};
    return true;
}

// mattn.zig:261-275 (widePick): one head of width 512 in whole 64-row blocks. The
// reference keeps its wide kernel behind an opt-in switch because it lost to the
// system's graph route there; here it is the only route for the shape, at any length.
bool Context::widePick(const attention::Config& cfg, Pick* out) const {
    if (!wide_pipeline || cfg.heads != 1 || cfg.kv_heads != 1 || cfg.causal) return false;
    if (cfg.head_dim != wide_head_dim || cfg.tokens == 0 || cfg.tokens % 64 != 0 || cfg.valid != 0) return false;
    *out = Pick{Kernel::wide, wide_pipeline, wide_threads};
    return true;
}

namespace {

// mattn.zig:396-411 (checkLens)
Error checkLens(size_t out_len, size_t q_len, size_t k_len, size_t v_len, const attention::Config& cfg) {
    if (cfg.heads == 0 || cfg.kv_heads == 0 || cfg.head_dim == 0) return Error::InvalidShape;
    if (cfg.heads % cfg.kv_heads != 0) return Error::InvalidShape;
    const size_t ql = cfg.tokens * cfg.heads * cfg.head_dim;
    const size_t kvl = cfg.tokens * cfg.kv_heads * cfg.head_dim;
    if (out_len != ql || q_len != ql) return Error::InvalidShape;
    if (k_len != kvl || v_len != kvl) return Error::InvalidShape;
    return Error::Ok;
}

// mattn.zig:376-394 (check) for the one kernel this backend has
Error check(size_t out_len, size_t q_len, size_t k_len, size_t v_len, const attention::Config& cfg) {
    if (cfg.tokens == 0) return Error::UnsupportedShape;
    if (cfg.head_dim != flash_head_dim) return Error::UnsupportedShape; // mattn.zig:388 (.block)
    if (cfg.heads == 0 || cfg.kv_heads == 0 || cfg.head_dim == 0) return Error::InvalidShape;
    return checkLens(out_len, q_len, k_len, v_len, cfg);
}

// mattn.zig:413-422 (paramsFor): every field must fit u32
bool paramsFor(const attention::Config& cfg, ZdrawAttnParams* p) {
    const size_t lim = 0xffffffffu;
    if (cfg.tokens > lim || cfg.heads > lim || cfg.kv_heads > lim || cfg.head_dim > lim || cfg.valid > lim)
        return false;
    p->tokens = (uint32_t)cfg.tokens;
    p->heads = (uint32_t)cfg.heads;
    p->kv_heads = (uint32_t)cfg.kv_heads;
    p->head_dim = (uint32_t)cfg.head_dim;
    p->causal = cfg.causal ? 1u : 0u;
    p->valid = (uint32_t)cfg.valid;
    return true;
}

} // namespace

Error Context::run(float* out, size_t out_len, const float* q, size_t q_len, const float* k, size_t k_len,
                   const float* v, size_t v_len, const attention::Config& cfg) {
    Pick picked;
    const bool wide = widePick(cfg, &picked);
    // mattn.zig:320-331 (checkWide) adds nothing to widePick but the length check; every other shape
    // takes check()
    Error e = wide ? checkLens(out_len, q_len, k_len, v_len, cfg) : check(out_len, q_len, k_len, v_len, cfg);
    if (e != Error::Ok) return e;
    if (!wide && !pick(cfg.tokens, cfg.head_dim, &picked)) return Error::UnsupportedShape;
    // Causal and grouped-query shapes belong to the text encoder; the backend
    // refuses them before anything is uploaded.
    if (cfg.causal || cfg.kv_heads != cfg.heads) return Error::UnsupportedShape;
    ZdrawAttnParams params;
    if (!paramsFor(cfg, &params)) return Error::InvalidShape;
    // mattn.zig:349-374 (runFresh): upload q/k/v, one dispatch, read back.
    Buffer qb = Buffer::fromBytes(device, q, q_len * sizeof(float));
    Buffer kb = Buffer::fromBytes(device, k, k_len * sizeof(float));
    Buffer vb = Buffer::fromBytes(device, v, v_len * sizeof(float));
    Buffer ob = Buffer::empty(device, out_len * sizeof(float));
    Error result = Error::OutOfMemory;
    if (qb.handle && kb.handle && vb.handle && ob.handle) {
        const int code = zdraw_hip_run_attention(queue, picked.pipeline, qb.handle, kb.handle, vb.handle, ob.handle,
                                                 &params, (uint32_t)picked.kernel, picked.threads);
        result = fromCode(code);
        if (result == Error::Ok)
            zdraw_hip_read_buffer(ob.handle, reinterpret_cast<uint8_t*>(out), out_len * sizeof(float));
    }
    qb.deinit();
    kb.deinit();
    vb.deinit();
    ob.deinit();
    return result;
}

Error Context::runPooled(float* out, size_t out_len, const float* q, size_t q_len, const float* k, size_t k_len,
                         const float* v, size_t v_len, const attention::Config& cfg) {
    Pick picked;
    const bool wide = widePick(cfg, &picked);
    // mattn.zig:320-331 (checkWide) adds nothing to widePick but the length check; every other shape
    // takes check()
    Error e = wide ? checkLens(out_len, q_len, k_len, v_len, cfg) : check(out_len, q_len, k_len, v_len, cfg);
    if (e != Error::Ok) return e;
    if (!wide && !pick(cfg.tokens, cfg.head_dim, &picked)) return Error::UnsupportedShape;
    if (cfg.causal || cfg.kv_heads != cfg.heads) return Error::UnsupportedShape;
    ZdrawAttnParams params;
    if (!paramsFor(cfg, &params)) return Error::InvalidShape;
    const size_t want[4] = {q_len * sizeof(float), k_len * sizeof(float), v_len * sizeof(float),
                            out_len * sizeof(float)};
    for (int i = 0; i < 4; i++) {
        if (pool_bytes[i] < want[i]) {
            if (pool[i]) zdraw_hip_release_buffer(pool[i]);
            pool[i] = zdraw_hip_create_buffer(device, want[i]);
            pool_bytes[i] = pool[i] ? want[i] : 0;
            if (!pool[i]) return Error::OutOfMemory;
        }
    }
    zdraw_hip_write_buffer(pool[0], reinterpret_cast<const uint8_t*>(q), want[0]);
    zdraw_hip_write_buffer(pool[1], reinterpret_cast<const uint8_t*>(k), want[1]);
    zdraw_hip_write_buffer(pool[2], reinterpret_cast<const uint8_t*>(v), want[2]);
    const int code = zdraw_hip_run_attention(queue, picked.pipeline, pool[0], pool[1], pool[2], pool[3], &params,
                                             (uint32_t)picked.kernel, picked.threads);
    if (code != 0) return fromCode(code);
    zdraw_hip_read_buffer(pool[3], reinterpret_cast<uint8_t*>(out), want[3]);
    return Error::Ok;
}

Error Context::runOnHandles(void* q_h, void* k_h, void* v_h, void* out_h, const attention::Config& cfg) {
    ZdrawAttnParams params;
    if (!paramsFor(cfg, &params)) return Error::InvalidShape;
    Pick picked;
    if (!widePick(cfg, &picked) && !pick(cfg.tokens, cfg.head_dim, &picked)) return Error::UnsupportedShape;
    const int code = zdraw_hip_run_attention(queue, picked.pipeline, q_h, k_h, v_h, out_h, &params,
                                             (uint32_t)picked.kernel, picked.threads);
    return fromCode(code);
}

} // namespace hattn

namespace attention_fast {

Error run(hattn::Context* hip, float* out, size_t out_len, const float* q, size_t q_len, const float* k,
          size_t k_len, const float* v, size_t v_len, float* scratch, size_t scratch_len,
          const attention::Config& cfg, attention::CpuRun cpu, void* cpu_user) {
    Error backend = Error::NotAvailable;
    if (hip) {
        backend = hip->run(out, out_len, q, q_len, k, k_len, v, v_len, cfg);
        if (backend == Error::Ok) return Error::Ok;           // the backend handled the shape
        if (backend != Error::UnsupportedShape) return backend; // every other error propagates
    }
    if (!cpu) return backend;
    const int rc = cpu(out, out_len, q, q_len, k, k_len, v, v_len, scratch, scratch_len, &cfg, cpu_user);
    return rc == 0 ? Error::Ok : Error::InvalidShape;
}

} // namespace attention_fast

} // namespace zdraw
