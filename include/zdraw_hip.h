/*
 * zdraw_hip.h: C ABI of the MI355X (gfx950) attention backend.
 *
 * This is the drop-in boundary for zdraw's DiT joint self-attention. It
 * replaces the attention slice of the reference's Metal bridge
 * (src/metal/metal_c.zig, implemented by src/metal/metal_api.m): opaque
 * pointer handles, plain-old-data parameter structs passed by const pointer,
 * int return codes. Each declaration cites the reference declaration it
 * replaces (paths relative to the reference tree).
 *
 * Return-code convention (metal_api.m:3072-3079, 1103-1113, 6604-6607):
 *    0  success
 *   -1  no usable handle / launch could not be issued
 *   -2  the device reported an error when the work completed
 *    1  "unavailable": the shape or operands are outside what this backend
 *       computes; NOTHING was enqueued and the caller takes its own fallback
 *       (zdraw's attention_fast.run falls through to its CPU kernel on
 *       error.UnsupportedShape, runtime/attention_fast.zig:16-23). The
 *       fallback counter is bumped.
 *    2  the operands are malformed for the declared shape (buffer too small,
 *       misaligned offset, zero dimension): the caller's error.InvalidShape.
 *
 * Threading: one host thread per queue, as in the reference (counters are
 * plain integers, metal_api.m:333). Work on one queue executes in order.
 */
#ifndef ZDRAW_HIP_H
#define ZDRAW_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ZDRAW_HIP_OK 0
#define ZDRAW_HIP_ERR_HANDLE (-1)
#define ZDRAW_HIP_ERR_DEVICE (-2)
#define ZDRAW_HIP_UNAVAILABLE 1
#define ZDRAW_HIP_INVALID 2

/* metal_c.zig:245-256 (AttnParams), 24 bytes, same field order. */
typedef struct ZdrawAttnParams {
    uint32_t tokens;
    uint32_t heads;
    uint32_t kv_heads;
    uint32_t head_dim;
    uint32_t causal;
    uint32_t valid; /* keys >= valid are masked for every query; 0 = none */
} ZdrawAttnParams;

/* mattn.Kernel order (metal/mattn.zig:19, metal_api.m:2983). Only BLOCK is
 * implemented by this backend: the bf16-MFMA flash kernel for head_dim 128. */
enum { ZDRAW_HIP_K_ROWS = 0, ZDRAW_HIP_K_FLASH = 1, ZDRAW_HIP_K_BLOCK = 2, ZDRAW_HIP_K_WIDE = 3 };

/* Element types of activations. */
enum { ZDRAW_HIP_F32 = 0, ZDRAW_HIP_F16 = 1, ZDRAW_HIP_BF16 = 2 };

/* What is applied to Q and K rows as they are loaded. */
enum {
    ZDRAW_HIP_QK_NONE = 0,  /* operands used as given (standalone attention) */
    ZDRAW_HIP_QK_KLEIN = 1, /* krms_rope: klein/zflux2_glue_shader.zig:61-83 */
    ZDRAW_HIP_QK_ZIMAGE = 2 /* qk_norm_rope: metal/mqk_shader.zig:46-97 */
};

/* Where norm+rope happens for the fused entry. */
enum {
    ZDRAW_HIP_K_IN_TILE_LOAD = 0, /* inside the attention kernel: Q in its prologue, K per tile */
    ZDRAW_HIP_K_PREPASS = 1       /* one pre-pass kernel prepares Q and K as bf16 in library scratch (f32 operands:
                                   * the same launch also rounds V, as krms_rope_hm / to_headmajor_f16 write half
                                   * copies, zflux2_glue_shader.zig:95-122), then attention on 16-bit rows */
};

/*
 * Extension block for the fused entry (no counterpart struct in the
 * reference: it gathers what RopeHmParams (klein/zflux2_glue_shader.zig:87-93),
 * QkNormParams (metal_c.zig:258-274) and the in_off/out_off arguments of
 * zdraw_metal_run_attention_steel_route_enc (metal_c.zig:339-349) carry).
 * Strides are in ELEMENTS: [0]=between batch segments, [1]=between tokens,
 * [2]=between heads; head_dim is contiguous.
 */
typedef struct ZdrawHipAttnExt {
    uint64_t q_off, k_off, v_off, out_off; /* byte offsets into the buffers */
    uint64_t q_stride[3];
    uint64_t k_stride[3];
    uint64_t v_stride[3];
    uint64_t out_stride[3];
    uint64_t rope_batch_rows;  /* rope-table / position rows between segments; 0 = shared */
    uint64_t mask_batch_bytes; /* key_pad bytes between segments; 0 = shared */
    uint64_t zimage_base[3];   /* Z-Image axis bases in pairs (zrope.Cache.axisBases) */
    uint32_t zimage_dims[3];   /* Z-Image axis widths, sum = head_dim */
    uint32_t batch;            /* independent segments, >= 1 */
    uint32_t in_dtype;         /* ZDRAW_HIP_F32, ZDRAW_HIP_F16 or ZDRAW_HIP_BF16 (F16: with the pre-pass, or qk_mode NONE) */
    uint32_t out_dtype;        /* ZDRAW_HIP_F32, ZDRAW_HIP_F16 or ZDRAW_HIP_BF16 */
    uint32_t qk_mode;          /* ZDRAW_HIP_QK_* */
    uint32_t k_site;           /* ZDRAW_HIP_K_IN_TILE_LOAD or ZDRAW_HIP_K_PREPASS */
    uint32_t txt_rows;         /* tokens < txt_rows use the *_txt weights (Klein double block) */
    float eps;                 /* RMSNorm epsilon */
    /* Caller's upper bound on |q'.k'|/sqrt(head_dim) over all rows AFTER norm and
     * rope, or 0 if unknown. With RMS-normalised Q and K and rope tables that are
     * rotations it is sqrt(head_dim) * max|w_q| * max|w_k|. A bound of at most 44
     * lets the kernel exponentiate scores without tracking a running maximum
     * (softmax is shift-invariant); 0 or a larger bound selects the running-maximum
     * form. When the call carries norm weights (qk_mode != NONE) the library forms
     * sqrt(head_dim) * max|w_q| * max|w_k| from the weight buffers itself and decides on
     * the larger of the two values: the caller's figure can only make the choice more
     * cautious, a figure that is too small cannot overflow. It does so only for weight
     * buffers whose bytes cannot change behind its back: memory the library allocated
     * (create_buffer, _with_data, _no_copy), whose device address was never handed out
     * (buffer_device_ptr) and which no kernel of this library was ever asked to write;
     * their 128 weights are read back once and the figure kept until write_buffer or
     * release. With any other weight buffer (wrap_device_memory, an exposed or
     * kernel-written buffer) the call takes the running-maximum form whatever the
     * caller's figure says. With qk_mode NONE there are no weights to check and the
     * caller's figure stands.
     * Accuracy: Q' and K' are rounded to 16 bits before the product, so a score of s
     * nats carries an absolute error of about s * 2^-8 (bf16 operands) or s * 2^-11
     * (ZDRAW_HIP_F16 staging, see `staging`); scores reach sqrt(head_dim) * max|w_q| *
     * max|w_k| = 11.3 nats with unit weights and grow with the product of the weights. */
    float score_bound;
    /* Element type in which the prepared Q and K are staged for the score product: 0 (or
     * ZDRAW_HIP_BF16) = bf16, ZDRAW_HIP_F16 = IEEE half, the staging type of the reference's
     * own kernels (klein/zflux2_glue_shader.zig:95-122, metal_api.m:6124-6145), values past
     * +-65504 saturating as there: three more mantissa bits on every score at the same MFMA
     * rate. It applies where the library writes the staged copies (qk_mode != NONE with
     * k_site PREPASS, or f32 / f16 operands with qk_mode NONE); elsewhere F16 returns 1.
     * in_dtype F16 implies it. P and V are bf16 in either case. */
    uint32_t staging;
} ZdrawHipAttnExt;

/* Buffer handles for the fused entry's side operands (NULL where unused). */
typedef struct ZdrawHipQkOperands {
    void* q_weight;     /* f32[128]  (norm_q) */
    void* k_weight;     /* f32[128]  (norm_k) */
    void* q_weight_txt; /* f32[128]  (norm_added_q) or NULL */
    void* k_weight_txt; /* f32[128]  (norm_added_k) or NULL */
    void* rope_cos;     /* Klein: f32 [rows][128] */
    void* rope_sin;     /* Klein: f32 [rows][128] */
    void* pos;          /* Z-Image: u64 [rows][3] (zrope.Pos) */
    void* rope_pairs;   /* Z-Image: f32 (cos,sin) pairs (zrope.Cache.pairBytes) */
    void* key_pad;      /* u8 [segments][tokens], nonzero = key excluded; NULL = no mask */
} ZdrawHipQkOperands;

/* ---- device / queue lifecycle ------------------------------------------ */
/* metal_c.zig:8-11. NULL when no gfx950 device is usable
 * (the caller's error.MetalNotAvailable). */
void* zdraw_hip_create_device(void);
void zdraw_hip_release_device(void* device);
/* One HIP stream, default priority. */
void* zdraw_hip_create_queue(void* device);
void zdraw_hip_release_queue(void* queue);

/* ---- buffers (metal_c.zig:12-33) ----------------------------------------- */
void* zdraw_hip_create_buffer(void* device, size_t size);
void* zdraw_hip_create_buffer_with_data(void* device, const uint8_t* data, size_t size);
/* metal_c.zig:18-22, metal_api.m:601-638: a buffer over `size` bytes of HOST memory that the
 * caller keeps owning (mbuffer.Cache.trySliceBind / sourceBuffer hand it a slice of the mmapped
 * checkpoint, metal/mbuffer.zig:88, 129). Unified memory lets Metal wrap those pages; a discrete
 * GPU cannot read them at speed, so the bytes are uploaded once here, when the buffer is
 * created (the sources are immutable weights), and the kernels read the device copy. Any
 * address and length is accepted (the Metal call returns NULL for a pointer that is not
 * page-aligned and its caller then binds the whole mapping at an offset: both bindings work
 * here). `data` is not read again after the call returns; release_buffer /
 * release_weight_buffer free the device copy only. NULL when the allocation or upload fails. */
void* zdraw_hip_create_buffer_no_copy(void* device, const uint8_t* data, size_t size);
/* No counterpart in the reference (interop with memory another runtime already holds on the
 * GPU, e.g. a tensor): a buffer handle over `size` bytes of DEVICE memory at device_ptr, never
 * freed by release_buffer. The pointer is checked with the runtime (hipPointerGetAttributes,
 * hipMemGetAddressRange): NULL unless [device_ptr, device_ptr + size) lies inside one device
 * allocation on this device, so host memory cannot reach a kernel through this call. The
 * library never caches anything it read from such memory (see score_bound above). */
void* zdraw_hip_wrap_device_memory(void* device, void* device_ptr, size_t size);
void zdraw_hip_read_buffer(void* buffer, uint8_t* dst, size_t size);
/* metal_c.zig:24-29, metal_api.m:647-665: the readback that works for every buffer and is
 * ordered after the work enqueued on `queue` (waits for the queue, then copies).
 * 0, -1 for a null or short buffer, -2 when the device reports an error. */
int zdraw_hip_read_buffer_any(void* queue, void* buffer, uint8_t* dst, size_t size);
void zdraw_hip_write_buffer(void* buffer, const uint8_t* src, size_t size);
size_t zdraw_hip_buffer_length(void* buffer);
/* No reference counterpart: interop. A buffer whose device address has been handed out may
 * change behind the library's back; from then on nothing read from it is cached. */
void* zdraw_hip_buffer_device_ptr(void* buffer);
void zdraw_hip_release_buffer(void* buffer);
/* metal_c.zig:32, metal_api.m:686-692: release of a buffer made by create_buffer_no_copy (the
 * reference keeps a separate weight-footprint ledger); the same as release_buffer here. */
void zdraw_hip_release_weight_buffer(void* buffer);

/* ---- pipelines (metal_c.zig:99-107) -------------------------------------- */
/* Same argument list as zdraw_metal_compile (metal_c.zig:99-105). The kernels are
 * compiled ahead of time for gfx950, so `source` is not read (NULL is accepted) and
 * "compile" is a lookup by entry name: "attention_block_mfma", "attention_wide_mfma",
 * "qk_norm_rope" and "gemm_half". Unknown names return NULL and write a message. */
void* zdraw_hip_compile(void* device, const char* source, const char* entry, char* error_buf, size_t error_len);
void zdraw_hip_release_pipeline(void* pipeline);
size_t zdraw_hip_pipeline_threads(void* pipeline);

/* ---- standalone attention (metal_c.zig:137-147) -------------------------- */
/* q, k, v, output: f32 token-major [tokens][heads][head_dim] buffers, as the
 * reference's. Blocks until the result is in `output`. */
int zdraw_hip_run_attention(void* queue, void* pipeline, void* q, void* k, void* v, void* output,
                            const ZdrawAttnParams* params, uint32_t kernel, size_t thread_count);

/* ---- resident batch (metal_c.zig:286-311, 350) --------------------------- */
void* zdraw_hip_batch_begin(void* queue);
int zdraw_hip_run_attention_enc(void* batch, void* pipeline, void* q, void* k, void* v, void* o,
                                const ZdrawAttnParams* params, uint32_t kernel, size_t thread_count);
int zdraw_hip_run_attention_enc_off(void* batch, void* pipeline, void* q, void* k, void* v, void* o,
                                    const ZdrawAttnParams* params, uint32_t kernel, size_t thread_count,
                                    uint64_t in_off, uint64_t out_off);
/* Waits for everything enqueued since batch_begin and frees the batch. */
int zdraw_hip_batch_end(void* batch);

/* ---- fused QK-norm + rope + attention ------------------------------------ */
/* Replaces the rmsRopeHm x2..4 + zdraw_metal_run_attention_steel_route_enc
 * sequence (klein/zflux2_resident.zig:1547-1550, 1673-1710; metal_c.zig:339-349)
 * and mqk.run + attention for Z-Image (metal/mres.zig:47-80): Q and K arrive
 * un-normalised, V as is; one launch (or pre-pass + launch) writes O. */
int zdraw_hip_run_attention_fused_enc(void* batch, void* q, void* k, void* v, void* out,
                                      const ZdrawAttnParams* params, const ZdrawHipAttnExt* ext,
                                      const ZdrawHipQkOperands* ops);
/* Same, on a queue, blocking until complete. */
int zdraw_hip_run_attention_fused(void* queue, void* q, void* k, void* v, void* out,
                                  const ZdrawAttnParams* params, const ZdrawHipAttnExt* ext,
                                  const ZdrawHipQkOperands* ops);

/* Sizes the queue's private scratch for a later zdraw_hip_run_attention_fused_enc with the same
 * arguments (no counterpart in the reference, whose slots are sized by their first use too): the
 * fused call then finds its scratch in place and neither waits for the queue nor allocates inside
 * an open batch. Enqueues nothing; returns what the fused call would return for these arguments. */
int zdraw_hip_reserve_attention_fused(void* queue, void* q, void* k, void* v, void* out,
                                      const ZdrawAttnParams* params, const ZdrawHipAttnExt* ext,
                                      const ZdrawHipQkOperands* ops);

/* The fused entry for callers that cannot allocate (no counterpart in the reference: it is
 * for code under HIP graph capture, tight serving loops and harnesses that forbid hipMalloc).
 * Same arguments, results bit-identical to zdraw_hip_run_attention_fused_enc, but the prepared
 * Q and K (the bf16 copy of an f32 V, the parts of key-split tiles) live in an array inside the
 * library's device code instead of the grow-only slots: ZDRAW_HIP_NOALLOC_SCRATCH_BYTES per GPU,
 * held until the process ends. A call that needs more (with bf16 operands:
 * batch x heads x tokens x 512 bytes, plus 256 KiB per key-split tile part) returns 1 and
 * enqueues nothing; the message says so. The call itself performs no device allocation and
 * creates no events (it is left out of the attention trace and the clock probe). One array per
 * GPU: calls that overlap on one GPU (two queues) race, calls on one queue are ordered. The
 * first call that meets a norm-weight buffer reads its 128 weights back once (a blocking copy of
 * 512 bytes) to form the score bound: make that call before a capture starts. */
#define ZDRAW_HIP_NOALLOC_SCRATCH_BYTES (64u << 20)
int zdraw_hip_run_attention_fused_noalloc_enc(void* batch, void* q, void* k, void* v, void* out,
                                              const ZdrawAttnParams* params, const ZdrawHipAttnExt* ext,
                                              const ZdrawHipQkOperands* ops);

/* ---- standalone QK-norm + rope --------------------------------------------
 * The general form (no counterpart declaration in the reference; it also serves the
 * in-place Klein krms_rope dispatches, klein/zflux2_resident.zig:1573-1579). In place on
 * f32 token-major q [tokens][heads][128] and k [tokens][kv_heads][128]. Only
 * ext->qk_mode, eps, txt_rows, zimage_* and rope_batch_rows are read. Blocks until done. */
int zdraw_hip_run_qk_norm_rope_ext(void* queue, void* pipeline, void* q, void* k,
                                   const ZdrawAttnParams* params, const ZdrawHipAttnExt* ext,
                                   const ZdrawHipQkOperands* ops);

/* metal_c.zig:148-159 with QkNormParams (metal_c.zig:258-274), argument for argument: the
 * Z-Image qk_norm_rope dispatch behind mqk.run (metal/mqk.zig:20-58). In place on f32
 * token-major q [tokens][heads][head_dim] and k [tokens][kv_heads][head_dim]; q_weight /
 * k_weight hold head_dim norm weights of type params->q_dtype / k_dtype (each f16, bf16 or
 * f32, independently) at byte offsets params->q_offset / k_offset, which need only be
 * multiples of the element size (mbuffer.Cache.bindView hands over file offsets,
 * metal/mqk.zig:97-98); weights of two types or off a 16-byte boundary are first copied as
 * f32 into 1 KiB of the queue's scratch by a small launch. pos is u64 [tokens][3]; rope the
 * (cos,sin) f32 pair table (zrope.Cache.pairBytes) whose axes start at params->base0..2
 * pairs. thread_count is accepted and not used. A position past its axis
 * (zimage/zrope.zig:48 refuses those on the host) reads the axis's last table entry
 * instead of memory outside the table. Blocks until done; returns 0, or 1 / 2 / negative
 * as above. */
typedef struct ZdrawQkNormParams { /* metal_c.zig:258-274, 80 bytes */
    uint32_t tokens, heads, kv_heads, head_dim;
    uint32_t q_dtype, k_dtype; /* element type of q_norm / k_norm: 1 f16, 2 bf16, 3 f32 */
    uint32_t dim0, dim1, dim2; /* rope axis widths, sum = head_dim */
    float eps;
    uint64_t q_offset, k_offset; /* byte offsets of the norm weights in their buffers */
    uint64_t base0, base1, base2; /* axis bases in (cos,sin) pairs */
} ZdrawQkNormParams;
int zdraw_hip_run_qk_norm_rope(void* queue, void* pipeline, void* q, void* k, void* q_weight, void* k_weight,
                               void* pos, void* rope, const ZdrawQkNormParams* params, size_t thread_count);

/* ---- projections either side of attention: C = A x W^T ----------------------
 * metal_c.zig:276-283 (GemmParams), same field order, 32 bytes. dtype is the
 * WEIGHT's type in the reference's coding (metal/mres_util.zig:11-18): 1 = f16,
 * 2 = bf16, 3 = f32; mode is metal/mgemm.zig:225-233: 2 = half (operands
 * rounded to the weight's 16-bit type, fp32 accumulation), 1 = exact f32.
 * This backend computes mode 2 with 16-bit weights; everything else (exact
 * mode, f32 or packed W8/W6/W4 weights, k % 8 != 0) returns 1 = unavailable
 * and the caller keeps its own path (runtime/linear_fast.zig:14-29). */
typedef struct ZdrawGemmParams {
    uint32_t m;  /* rows of A and C */
    uint32_t k;  /* columns of A and of W */
    uint32_t n;  /* rows of W, columns of C */
    uint32_t dtype;
    uint32_t mode;
    uint64_t weight_offset; /* byte offset of W in its buffer */
} ZdrawGemmParams;
enum { ZDRAW_HIP_W_F16 = 1, ZDRAW_HIP_W_BF16 = 2, ZDRAW_HIP_W_F32 = 3 };
enum { ZDRAW_HIP_GEMM_EXACT = 1, ZDRAW_HIP_GEMM_HALF = 2 };

/* What the reference passes as byte offsets only, plus leading dimensions and
 * 16-bit activations / outputs (no counterpart struct in the reference).
 * Leading dimensions are in elements; 0 means dense (k, k, n). */
typedef struct ZdrawHipGemmExt {
    uint64_t a_off, c_off; /* byte offsets into the A and C buffers */
    uint64_t lda, ldw, ldc;
    uint32_t a_dtype;      /* ZDRAW_HIP_F32, or the weight's type (ZDRAW_HIP_F16 / ZDRAW_HIP_BF16) */
    uint32_t c_dtype;      /* ZDRAW_HIP_F32, or the weight's type */
} ZdrawHipGemmExt;

/* metal_c.zig:160-167: A f32 [m][k], W [n][k], C f32 [m][n]; blocks until done.
 * pipeline is zdraw_hip_compile(device, "gemm_half", ...). */
int zdraw_hip_run_gemm(void* queue, void* pipeline, void* a, void* w, void* c, const ZdrawGemmParams* params);
/* metal_c.zig:357-364, 368-377: the same inside a batch, and with A / C byte offsets. */
int zdraw_hip_run_gemm_enc(void* batch, void* pipeline, void* a, void* w, void* c, const ZdrawGemmParams* params);
int zdraw_hip_run_gemm_off_enc(void* batch, void* pipeline, void* a, void* w, void* c,
                               const ZdrawGemmParams* params, uint64_t a_offset, uint64_t c_offset);
/* metal_c.zig:425-433 (and :378-386): A already in the weight's 16-bit type, C f32. */
int zdraw_hip_run_gemm_f16a_enc(void* batch, void* a, void* w, void* c, const ZdrawGemmParams* params,
                                uint64_t a_offset, uint64_t c_offset);
/* metal_c.zig:175-198: two or three products of the same A (f32 in, f32 out), blocking.
 * Products of equal shape and weight type run as one launch whose tiles cover all
 * of them; otherwise one launch each. */
int zdraw_hip_run_gemm_pair(void* queue, void* pipeline, void* a, void* w0, void* c0, const ZdrawGemmParams* params0,
                            void* w1, void* c1, const ZdrawGemmParams* params1);
int zdraw_hip_run_gemm_triple(void* queue, void* pipeline, void* a, void* w0, void* c0, const ZdrawGemmParams* params0,
                              void* w1, void* c1, const ZdrawGemmParams* params1, void* w2, void* c2,
                              const ZdrawGemmParams* params2);
/* General form: leading dimensions and 16-bit output, e.g. Q/K/V written as
 * bf16 token-major rows for the attention entry, or the attention output read
 * from the concat operand at its row pitch. */
int zdraw_hip_run_gemm_ext_enc(void* batch, void* a, void* w, void* c, const ZdrawGemmParams* params,
                               const ZdrawHipGemmExt* ext);
/* The general form for `count` (1..3) products of one A that share `ext` (gate/up, q/k/v of
 * the resident 16-bit path; the pair/triple of metal_c.zig:175-198 with the options of the
 * entry above): equal shapes and weight types run as one launch whose tiles cover all of
 * them, otherwise one launch each. params[i]->weight_offset selects each W; ext->c_off
 * applies to every C. A product this backend does not run refuses the whole call (1)
 * before anything is enqueued. */
int zdraw_hip_run_gemm_group_ext_enc(void* batch, void* a, void* const* ws, void* const* cs,
                                     const ZdrawGemmParams* const* params, uint32_t count, const ZdrawHipGemmExt* ext);

/* ---- Z-Image layer, attention segment --------------------------------------
 * The q/k/v projections, QK-norm + rope, attention and output projection of one
 * Z-Image layer as metal_api.m:7134-7212 (encode_chain_layer_ours16) and
 * :7103-7108 (encode_chain_layer) encode them:
 *   q = norm x Wq^T, k = norm x Wk^T, v = norm x Wv^T      (GemmParams q, k, v)
 *   qk_norm_rope(q, k; q_norm, k_norm, pos, rope)           (QkNormParams qk)
 *   mix = attention(q, k, v)                                (AttnParams attn)
 *   attn = mix x Wproj^T                                    (GemmParams proj)
 * The structs carry the fields of ZdrawBlockBuffers / ZdrawBlockWeights /
 * ZdrawBlockChainParams (metal_api.m:5961-5987) that this segment reads, in the
 * reference's order. Rows padded to a multiple of 32 (zimage/zseq.zig:23-34) are
 * ordinary rows here, as they are there. */

typedef struct ZdrawHipChainAttnBuffers {
    void* norm; /* [tokens][hidden] layer input after its norm (activation dtype) */
    void* q;    /* [tokens][heads*128]; holds the raw projection afterwards */
    void* k;
    void* v;
    void* mix;  /* [tokens][heads*128] attention output */
    void* attn; /* [tokens][hidden] projected output */
} ZdrawHipChainAttnBuffers;

typedef struct ZdrawHipChainAttnWeights {
    void* q; void* k; void* v; /* [heads*128][hidden], 16-bit */
    void* q_norm; void* k_norm; /* [128] */
    void* pos;  /* u64 [tokens][3] */
    void* rope; /* (cos,sin) f32 pairs */
    void* proj; /* [hidden][heads*128], 16-bit */
} ZdrawHipChainAttnWeights;

typedef struct ZdrawHipChainAttnParams {
    ZdrawGemmParams q, k, v;
    ZdrawQkNormParams qk;
    ZdrawAttnParams attn;
    ZdrawGemmParams proj;
    /* no counterpart in the reference (its chain buffers are f32): element type of
     * every buffer in ZdrawHipChainAttnBuffers, ZDRAW_HIP_F32 or ZDRAW_HIP_BF16
     * (the latter needs bf16 weights). */
    uint32_t act_dtype;
    float score_bound; /* as ZdrawHipAttnExt.score_bound; 0 = unknown */
} ZdrawHipChainAttnParams;

/* Enqueues the launches (q/k/v projections as one, pre-pass, attention, projection) on the batch's stream. 0 = enqueued; 1 = a shape or
 * weight form this backend does not run (nothing enqueued, the caller keeps its
 * own path); negative = invalid arguments. */
int zdraw_hip_run_chain_attn_enc(void* batch, const ZdrawHipChainAttnBuffers* buffers,
                                 const ZdrawHipChainAttnWeights* weights,
                                 const ZdrawHipChainAttnParams* params);

/* ---- scratch slots (metal_c.zig:321-325) ----------------------------------
 * The reference's process-lifetime, grow-only slots, for callers that keep their own
 * intermediates in them: (re)allocated only to grow, filled at (re)allocation with 0x00
 * (0xFF when ZDRAW_SCRATCH_POISON is set, metal_api.m:6147-6181). slot in [0, 7).
 * The library's OWN scratch (prepared Q and K, V's bf16 copy, the parts of key-split
 * attention tiles and of k-split GEMM tiles, rounded f32 activations) does not live here:
 * every queue owns a private set of such slots, grown on the first call of a size on that
 * queue (which waits for that queue's earlier work, then allocates; zdraw_hip_reserve_attention_fused
 * does that ahead of time) and freed with the queue, so work on two queues never shares scratch. */
void* zdraw_hip_attn_scratch(void* device, int slot, size_t bytes);

/* ---- counters and timing (metal_api.m:333-353, 420-433) ------------------- */
void zdraw_hip_metrics_reset(void);
uint64_t zdraw_hip_dispatch_count(void);
uint64_t zdraw_hip_command_count(void);
uint64_t zdraw_hip_attn_fallback_count(void);
uint64_t zdraw_hip_gpu_ns(void); /* device time summed over completed batches / blocking runs */

/* Attention-kernel trace (the attention bucket of ZDRAW_KLEIN_TRACE,
 * klein/zflux2_resident.zig:443-467): when on, each attention kernel launch is
 * bracketed by its own HIP events on the stream it is launched on (a pre-pass
 * kernel is outside the bracket). trace_attention_ns waits for the bracketed
 * launches, returns their summed device time and stores their count. */
void zdraw_hip_trace_attention(int on);
uint64_t zdraw_hip_trace_attention_ns(uint64_t* launches);

/* HIP events on a queue's stream, for measuring kernels where they run. */
void* zdraw_hip_event_create(void);
int zdraw_hip_event_record(void* event, void* queue);
int zdraw_hip_event_sync(void* event);
float zdraw_hip_event_elapsed_ms(void* start, void* stop); /* negative on error */
void zdraw_hip_event_release(void* event);
int zdraw_hip_queue_sync(void* queue);

/* How a launch of `tiles` workgroup tiles (segments x heads x query blocks) is laid on `cus`
 * compute units (no reference counterpart: scheduling, exposed so that it can be checked
 * without a device). A last round that fills at most half the CUs is split along the keys:
 * *tail_tiles tiles (the last ones) run as *splits parts each, at least 8 key blocks per part,
 * at most 16 parts; *tail_tiles = 0 and *splits = 1 when everything runs whole. */
void zdraw_hip_attention_tail_plan(uint64_t tiles, uint32_t cus, uint32_t key_blocks, uint32_t* tail_tiles,
                                   uint32_t* splits);

/* The same for `groups` (1..3) side-by-side products C[m][n] = A[m][k] x W[n][k]^T of 16-bit
 * activations: the tiles are 256 x 256; a last round that fills at most half the CUs runs as
 * *splits ranges of k per tile (at most 8, at least four 64-wide slabs each) whose fp32
 * partial tiles are added in range order; nothing is split when k is not a multiple of 64,
 * when fewer than 160 tiles exist, or under the eight-wave build. */
void zdraw_hip_gemm_tail_plan(uint32_t m, uint32_t k, uint32_t n, uint32_t groups, uint32_t cus, uint32_t* tail_tiles,
                              uint32_t* splits);

/* Positions per Z-Image rope axis that lie inside a (cos,sin) pair table of `table_bytes`
 * bytes whose axes start at base[0..2] pairs and are dims[0..2] wide (no reference
 * counterpart: zimage/zrope.zig:48 refuses pos >= len on the host; positions that are only
 * known on the device are held to these counts by the kernels, so that none indexes outside
 * the table). For the layout of zrope.Cache the counts are its `lens`. Host arithmetic only.
 * 0, or 2 when an axis has no whole position inside the table. */
int zdraw_hip_zimage_axis_lens(uint64_t table_bytes, const uint64_t* base, const uint32_t* dims, uint32_t* lens);

/* ABI drift guard (src/abi_gen.zig, runtime/abi_assert.zig:29): sizeof of the
 * shared structs as this library was compiled. which: 0 = ZdrawAttnParams,
 * 1 = ZdrawHipAttnExt, 2 = ZdrawHipQkOperands, 3 = ZdrawGemmParams,
 * 4 = ZdrawHipGemmExt, 5 = ZdrawQkNormParams, 6 = ZdrawHipChainAttnBuffers,
 * 7 = ZdrawHipChainAttnWeights, 8 = ZdrawHipChainAttnParams. */
size_t zdraw_hip_abi_sizeof(int which);
/* Last error text of this thread's most recent failing call ("" if none). */
const char* zdraw_hip_last_error(void);

#define ZDRAW_HIP_ABI_ATTN_PARAMS_SIZE 24
#define ZDRAW_HIP_ABI_ATTN_EXT_SIZE 216
#define ZDRAW_HIP_ABI_QK_OPERANDS_SIZE 72
#define ZDRAW_HIP_ABI_GEMM_PARAMS_SIZE 32
#define ZDRAW_HIP_ABI_GEMM_EXT_SIZE 48
#define ZDRAW_HIP_ABI_QK_NORM_PARAMS_SIZE 80
#define ZDRAW_HIP_ABI_CHAIN_ATTN_BUFFERS_SIZE 48
#define ZDRAW_HIP_ABI_CHAIN_ATTN_WEIGHTS_SIZE 64
#define ZDRAW_HIP_ABI_CHAIN_ATTN_PARAMS_SIZE 240

#ifdef __cplusplus
}
#endif
#endif
