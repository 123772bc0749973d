// Flat C exports of the host layer so that tests and the benchmark can drive
// it through ctypes. Error values are zdraw::Error as int.
#include "zdraw_host.hpp"

using namespace zdraw;

extern "C" {

struct ZhConfig {
    size_t tokens, heads, kv_heads, head_dim;
    int causal;
    size_t valid;
};

static attention::Config cfgOf(const ZhConfig* c) {
    return attention::Config{c->tokens, c->heads, c->kv_heads, c->head_dim, c->causal != 0, c->valid};
}

void* zh_context_init(int* err) {
    hattn::Context* c = new hattn::Context();
    Error e = hattn::Context::init(c);
    if (err) *err = (int)e;
    if (e != Error::Ok) {
        delete c;
        return nullptr;
    }
    return c;
}
void* zh_context_init_kernel(uint32_t kernel, int* err) {
    hattn::Context* c = new hattn::Context();
    Error e = hattn::Context::initKernel((hattn::Kernel)kernel, c);
    if (err) *err = (int)e;
    if (e != Error::Ok) {
        delete c;
        return nullptr;
    }
    return c;
}
void zh_context_deinit(void* ctx) {
    hattn::Context* c = static_cast<hattn::Context*>(ctx);
    if (!c) return;
    c->deinit();
    delete c;
}
void* zh_context_device(void* ctx) { return static_cast<hattn::Context*>(ctx)->device; }
void* zh_context_queue(void* ctx) { return static_cast<hattn::Context*>(ctx)->queue; }
void* zh_context_block_pipeline(void* ctx) { return static_cast<hattn::Context*>(ctx)->block_pipeline; }

int zh_context_pick(void* ctx, size_t tokens, size_t head_dim, uint32_t* kernel, size_t* threads) {
    hattn::Pick p;
    if (!static_cast<hattn::Context*>(ctx)->pick(tokens, head_dim, &p)) return 0;
    if (kernel) *kernel = (uint32_t)p.kernel;
    if (threads) *threads = p.threads;
    return 1;
}
int zh_context_run(void* ctx, float* out, size_t out_len, const float* q, size_t q_len, const float* k, size_t k_len,
                   const float* v, size_t v_len, const ZhConfig* cfg) {
    return (int)static_cast<hattn::Context*>(ctx)->run(out, out_len, q, q_len, k, k_len, v, v_len, cfgOf(cfg));
}
int zh_context_run_pooled(void* ctx, float* out, size_t out_len, const float* q, size_t q_len, const float* k,
                          size_t k_len, const float* v, size_t v_len, const ZhConfig* cfg) {
    return (int)static_cast<hattn::Context*>(ctx)->runPooled(out, out_len, q, q_len, k, k_len, v, v_len, cfgOf(cfg));
}
int zh_context_run_on_handles(void* ctx, void* q, void* k, void* v, void* out, const ZhConfig* cfg) {
    return (int)static_cast<hattn::Context*>(ctx)->runOnHandles(q, k, v, out, cfgOf(cfg));
}

// The CPU kernel arrives as a C callback taking the flat config.
typedef int (*ZhCpuRun)(float*, size_t, const float*, size_t, const float*, size_t, const float*, size_t, float*,
                        size_t, const ZhConfig*);

static int cpuTrampoline(float* out, size_t out_len, const float* q, size_t q_len, const float* k, size_t k_len,
                         const float* v, size_t v_len, float* scratch, size_t scratch_len,
                         const attention::Config* cfg, void* user) {
    ZhConfig c{cfg->tokens, cfg->heads, cfg->kv_heads, cfg->head_dim, cfg->causal ? 1 : 0, cfg->valid};
    return reinterpret_cast<ZhCpuRun>(user)(out, out_len, q, q_len, k, k_len, v, v_len, scratch, scratch_len, &c);
}

int zh_attention_fast_run(void* ctx, float* out, size_t out_len, const float* q, size_t q_len, const float* k,
                          size_t k_len, const float* v, size_t v_len, float* scratch, size_t scratch_len,
                          const ZhConfig* cfg, ZhCpuRun cpu) {
    return (int)attention_fast::run(static_cast<hattn::Context*>(ctx), out, out_len, q, q_len, k, k_len, v, v_len,
                                    scratch, scratch_len, cfgOf(cfg), cpu ? cpuTrampoline : nullptr,
                                    reinterpret_cast<void*>(cpu));
}

struct ZhRopeCache {
    size_t dims[3];
    size_t lens[3];
    const float* values;
};

int zh_qk_run(void* ctx, void* q_h, void* k_h, const float* q_weight, const float* k_weight, const size_t* pos,
              size_t pos_len, const ZhRopeCache* rope, size_t tokens, size_t heads, size_t kv_heads, size_t head_dim,
              float norm_eps) {
    hqk::RopeCache rc;
    for (int a = 0; a < 3; a++) {
        rc.dims[a] = rope->dims[a];
        rc.lens[a] = rope->lens[a];
    }
    rc.values = rope->values;
    return (int)hqk::run(static_cast<hattn::Context*>(ctx), q_h, k_h, q_weight, k_weight, pos, pos_len, rc,
                         hqk::Config{tokens, heads, kv_heads, head_dim, norm_eps});
}

int zh_joint_klein(void* ctx, const joint::Klein* c) { return (int)joint::run(static_cast<hattn::Context*>(ctx), *c); }
int zh_joint_zimage(void* ctx, const joint::Zimage* c) { return (int)joint::run(static_cast<hattn::Context*>(ctx), *c); }

float zh_score_bound(const float* wq, const float* wk, const float* wqt, const float* wkt) {
    return joint::scoreBound(wq, wk, wqt, wkt);
}

size_t zh_sizeof(int which) {
    switch (which) {
    case 0: return sizeof(ZhConfig);
    case 1: return sizeof(joint::Klein);
    case 2: return sizeof(joint::Zimage);
    case 3: return sizeof(ZhRopeCache);
    default: return 0;
    }
}

} // extern "C"
