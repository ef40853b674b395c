/*
 * argus_hip.h -- C ABI of the MI355X (gfx950) attention backend for the Argus engine.
 *
 * Every entry point is `extern "C"`, takes plain pointers / integers, returns an
 * `int` (0 = ok, negative = error, never throws or aborts: the engine's release
 * profile is panic=abort, crates/argus-extension-api/src/lib.rs:1680) and runs on
 * the single in-order stream the engine lends (NULL = the default stream,
 * engine/src/kv/quant_window_cuda.rs:38-46).  A context serves ONE stream at a time: its split-KV
 * workspace is handed to every attention call, so calls issued on different streams without
 * ordering between them race on the partial results (the reference backends are single-stream too,
 * engine/src/backend/cuda_pc/gpu_score.rs:40-50).  The engine owns every Q / KV / out /
 * score buffer and lends raw device pointers for the duration of one call; the
 * library never frees or retains them (crates/argus-extension-api/src/lib.rs:1593).
 *
 * Each declaration cites the reference interface it stands in for; paths are
 * relative to the reference repository root.
 */
#ifndef ARGUS_HIP_H
#define ARGUS_HIP_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ARGUS_HIP_ABI_VERSION 2

/* Return codes. */
#define ARGUS_HIP_OK 0
#define ARGUS_HIP_ERR_INVALID (-1)     /* bad argument (null pointer, non-dividing heads, ...) */
#define ARGUS_HIP_ERR_UNSUPPORTED (-2) /* shape / dtype outside the kernels' coverage */
#define ARGUS_HIP_ERR_RUNTIME (-3)     /* HIP runtime error; see argus_hip_last_error */
#define ARGUS_HIP_ERR_NOMEM (-4)       /* workspace allocation failed */

/* DType subset of engine/src/buffer.rs:25-47 that the attention path touches. */
#define ARGUS_HIP_F32 0
#define ARGUS_HIP_F16 1
/* Block-quantised cache rows, 32 elements per block (DType::Q4_0 of the reference,
 * engine/src/backend/cpu/common.rs:676-690, and the `--kv-format` descriptors q4_0 / q4_1 / q8_0 /
 * q2_0, engine/src/format/dtype_layout.rs:102-166): [f16 d][16 nibble bytes] = 18 bytes,
 * [f16 d][f16 m][16 nibble bytes] = 20 bytes, [f16 d][32 int8] = 34 bytes,
 * [f16 d][f16 m][8 bytes of four 2-bit codes] = 12 bytes.  attention_gen only. */
#define ARGUS_HIP_Q4_0 2
#define ARGUS_HIP_Q4_1 3
#define ARGUS_HIP_Q8_0 4
#define ARGUS_HIP_Q2_0 5

/* KVLayout, engine/src/kv/kv_cache_ops.rs:18-21. */
#define ARGUS_HIP_HEAD_MAJOR 0 /* [batch, kv_heads, capacity, head_dim] */
#define ARGUS_HIP_SEQ_MAJOR 1  /* [batch, seq, kv_heads, head_dim]     */

typedef struct argus_hip_ctx argus_hip_ctx;

/* ---- context: what `HipBackend::new` / `Drop` bind -------------------------------------- */
/* Counterpart of CudaBackend construction in engine/src/session/init.rs:351-428: selects the
 * device, reads its CU count and allocates the split-KV partial workspace.  Fails with
 * ARGUS_HIP_ERR_RUNTIME (and *out = NULL) when no HIP device is present. */
int argus_hip_create(int device, argus_hip_ctx **out);
/* The reference pre-allocates every buffer at max_seq_len and lends it for the session, with no
 * allocator callback into the engine (crates/argus-extension-api/src/lib.rs:1903-1907).  The one
 * buffer this library owns is the split-KV workspace; create_ex sizes it once for the largest call
 * the caller will issue (zero fields / NULL opts: 8 MiB), so that no attention call allocates.  A
 * call beyond the hint still works: it grows the workspace, which synchronises the device.
 * The environment switches ARGUS_HIP_DECODE / ARGUS_HIP_SCORES / ARGUS_HIP_KIVI are read here. */
typedef struct argus_hip_create_opts {
  int32_t max_batch;    /* sequences (or KIVI caches) per attention call */
  int32_t max_heads_q;  /* query heads */
  int32_t max_head_dim; /* 64, 128 or 256 */
  int32_t max_seq_len;  /* informational: the split count is bounded whatever the length */
} argus_hip_create_opts;
int argus_hip_create_ex(int device, const argus_hip_create_opts *opts, argus_hip_ctx **out);
int argus_hip_reserve_workspace(argus_hip_ctx *ctx, size_t bytes);
int argus_hip_destroy(argus_hip_ctx *ctx);
int argus_hip_abi_version(void);
/* Last error text of this context (single inference thread, like the reference backends). */
const char *argus_hip_last_error(const argus_hip_ctx *ctx);

typedef struct argus_hip_device_info {
  int32_t compute_units;
  int32_t clock_mhz;
  int32_t wavefront_size;
  int32_t lds_bytes_per_block;
  int64_t hbm_bytes;
  char name[128];
  char gcn_arch[64];
} argus_hip_device_info;
int argus_hip_get_device_info(const argus_hip_ctx *ctx, argus_hip_device_info *info);

/* ---- per-kernel event timing ------------------------------------------------------------- */
/* Counterpart of the event-based GPU profiling switch Backend::profile_events_enabled /
 * set_op_label (engine/src/backend.rs:1296-1306).  Between _begin and _end the dominant kernel
 * of every attention call (decode split pass, prefill, KIVI decode) is bracketed by a HIP event
 * pair recorded on the stream it is launched on; _end waits for the last one and returns the
 * per-launch durations in milliseconds (at most `capacity`; *n_out = launches recorded). */
int argus_hip_kernel_timing_begin(argus_hip_ctx *ctx, int32_t max_launches);
int argus_hip_kernel_timing_end(argus_hip_ctx *ctx, float *ms_out, int32_t capacity, int32_t *n_out);
/* Same, and in tail_ms_out (may be NULL) the time from the end of the dominant kernel to the end of
 * the call's last launch: the combine pass of a split-KV decode, zero for single-kernel calls. */
int argus_hip_kernel_timing_end2(argus_hip_ctx *ctx, float *ms_out, float *tail_ms_out, int32_t capacity,
                                 int32_t *n_out);

/* ---- memory helpers for the Rust `Memory` / `Buffer` impls ------------------------------- */
/* Backend::{read_buffer, write_buffer, write_buffer_range, copy_slice, buffer_shift,
 * synchronize}: engine/src/backend.rs:610, 710, 736, 1085, 1119, 762. */
int argus_hip_malloc(argus_hip_ctx *ctx, size_t bytes, void **dev_ptr);
int argus_hip_free(argus_hip_ctx *ctx, void *dev_ptr);
int argus_hip_write_buffer(argus_hip_ctx *ctx, void *stream, void *dst_dev, const void *src_host, size_t bytes);
int argus_hip_read_buffer(argus_hip_ctx *ctx, void *stream, void *dst_host, const void *src_dev, size_t bytes);
int argus_hip_copy_slice(argus_hip_ctx *ctx, void *stream, void *dst_dev, const void *src_dev, size_t bytes);
/* Backend::write_buffer_range (engine/src/backend.rs:736): host bytes into dst_dev + dst_offset. */
int argus_hip_write_buffer_range(argus_hip_ctx *ctx, void *stream, void *dst_dev, size_t dst_offset,
                                 const void *src_host, size_t bytes);
/* Backend::buffer_shift (engine/src/backend.rs:1085-1112): std::ptr::copy inside one buffer, i.e.
 * memmove -- the ranges may overlap in either direction (prefix prune; the KIVI residual ring moving
 * its remaining rows to the front, engine/src/kv/quant_window_cache.rs:1820-1841).  Uses the
 * context workspace as staging when the ranges lie less than 1 MiB apart. */
int argus_hip_buffer_shift(argus_hip_ctx *ctx, void *stream, void *dst_dev, const void *src_dev, size_t bytes);
int argus_hip_synchronize(argus_hip_ctx *ctx, void *stream);

/* ---- (a-1) single-query GQA decode attention ---------------------------------------------- */
/* Backend::attention_gen, engine/src/backend.rs:284-295 (CPU: backend/cpu/x86.rs:178-357,
 * backend/cpu/common.rs:359-675; CUDA host: backend/cuda_pc.rs:1693-1885).
 *   s_t = (q . k_t) * scale;  [soft-cap];  p = softmax_t(s);  out = sum_t p_t v_t
 * Layout rule of x86.rs:195-198: HeadMajor offset (kv_h*capacity + t)*d, SeqMajor
 * (t*Hkv + kv_h)*d.  `scores_out[h*score_stride + t] = p_t` like x86.rs:302-310, but the
 * pointer is a DEVICE pointer here (the host-slice contract of the trait, with its
 * synchronize + copy-back, lives in the host mirror `HipBackend::attention_gen`).
 * NaN logits count as -inf and an all -inf row falls back to uniform weights, as in
 * common.rs:555-584.
 * Beyond the reference trait (all default to the reference behaviour when zero / NULL):
 *   batch / *_batch_stride : `batch` independent sequences in one launch (the reference
 *                            loops, engine/src/backend.rs:277-295);
 *   kv_start               : first attended slot (windowed layers pass cache_len - window);
 *   kv_index               : logical token t lives in slot kv_index[t]
 *                            (SelectiveRead gather, engine/src/kv/standard_format.rs:2052-2184);
 *                            `capacity` (> 0, both layouts) bounds the slots: an entry outside
 *                            [0, capacity) never reaches memory outside the head's rows (it reads
 *                            zeros or the last slot; the result for such a list is unspecified);
 *   softcap                : cap*tanh(s/cap) after scaling
 *                            (engine/kernels/flash_attn_f32_f16.cl:563-565; host passes 0);
 *   scale                  : 0 selects 1/sqrt(head_dim) (x86.rs:192);
 *   score_stats            : opt-in score form for consumers that reduce the scores on the device
 *                            (argus_hip_score_reduce_ex): `scores_out` then keeps the LOGITS s_t (after
 *                            scale and soft-cap, NaN as -inf) and score_stats[h*2 .. +1] = (max_t s_t,
 *                            sum_t exp(s_t - max)), so that p_t = exp(s_t - max) / sum -- the call does
 *                            not read the row again to rewrite it.  NULL: probabilities, as the trait says.
 * Block-quantised caches (kv_dtype ARGUS_HIP_Q4_0 / Q4_1 / Q8_0 / Q2_0): the Q4_0 arm of the reference
 * (common.rs:676-850, rows dequantised on the fly) and the in-kernel form of the `--kv-format`
 * attention whose reference floor decodes the whole cache to F32 first
 * (engine/src/kv/standard_format.rs:538-643).  Rows are head_dim/32 blocks; capacity, kv_start and
 * the strides stay in elements (multiples of 32).  softcap and kv_index apply as for F16 caches;
 * up to 16 query heads per KV head (8 at head_dim 256), else ARGUS_HIP_ERR_UNSUPPORTED (decode with
 * argus_hip_kv_decode_descriptor and attend the F16 copy). */
typedef struct argus_hip_attention_gen_args {
  void *stream;
  const float *q;       /* [batch, num_heads_q, head_dim] F32 */
  const void *k_cache;  /* F16, F32 or blocks, layout per `layout` */
  const void *v_cache;
  float *out;           /* [batch, num_heads_q, head_dim] F32 */
  float *scores_out;    /* device, [batch, num_heads_q, score_stride] F32, or NULL */
  const int32_t *kv_index; /* device, [cache_seq_len] (per sequence if index_batch_stride != 0), or NULL */
  int32_t num_heads_q;
  int32_t num_heads_kv;
  int32_t head_dim;      /* 64, 128 or 256 */
  int32_t cache_seq_len; /* valid tokens attended */
  int32_t capacity;      /* HeadMajor rows per head; ignored for SeqMajor */
  int32_t kv_start;
  int32_t layout;        /* ARGUS_HIP_HEAD_MAJOR / ARGUS_HIP_SEQ_MAJOR */
  int32_t kv_dtype;      /* ARGUS_HIP_F16 / ARGUS_HIP_F32 / ARGUS_HIP_Q4_0 / _Q4_1 / _Q8_0 / _Q2_0 */
  int32_t batch;         /* >= 1 */
  int32_t score_stride;  /* floats per head row of scores_out, >= cache_seq_len */
  int64_t q_batch_stride;     /* elements; 0 = num_heads_q*head_dim */
  int64_t out_batch_stride;   /* elements; 0 = num_heads_q*head_dim */
  int64_t kv_batch_stride;    /* elements between consecutive sequences' caches */
  int64_t score_batch_stride; /* elements; 0 = num_heads_q*score_stride */
  int64_t index_batch_stride; /* elements; 0 = one index list shared by the batch */
  float softcap;
  float scale;
  float *score_stats;         /* device, [batch, num_heads_q, 2] F32 (max, sum), or NULL; needs scores_out */
  int64_t stats_batch_stride; /* elements; 0 = num_heads_q*2 */
} argus_hip_attention_gen_args;
int argus_hip_attention_gen(argus_hip_ctx *ctx, const argus_hip_attention_gen_args *args);

/* No counterpart in the reference.  For callers that cannot allocate device memory: code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  Same arguments, kernels and
 * results as argus_hip_attention_gen, but the split-KV partials live in a 16 MiB static device array
 * of the library (one copy per GPU, held until the process ends) and the call makes no hipMalloc /
 * hipFree / allocating library call.  A call whose partials exceed the array -- batch * num_heads_q
 * * splits * (head_dim + 2) * 4 bytes, e.g. more than ~250 sequences of the Llama-3-8B head shape
 * without scores -- returns ARGUS_HIP_ERR_NOMEM with the sizes in argus_hip_last_error.  Every call
 * on a GPU shares that GPU's array: calls that overlap on one GPU (different streams or contexts)
 * race; nothing in the array needs clearing between calls.  Kernels are loaded on their first
 * launch, so issue one call of each shape class before capturing. */
int argus_hip_attention_gen_noalloc(argus_hip_ctx *ctx, const argus_hip_attention_gen_args *args);

/* How the last attention_gen / attention_gen_quant call on this context was cut along the KV length
 * (diagnostics for benchmarks and tests; the reference has no split-KV on this path outside
 * engine/src/backend/cpu/neon.rs:261-300). */
typedef struct argus_hip_decode_plan {
  int32_t nsplit;        /* workgroups per (sequence, KV head) */
  int32_t chunk;         /* tokens per split */
  int32_t wgs_per_cu;    /* resident workgroups per compute unit the plan assumed */
  int32_t lds_bytes;     /* dynamic LDS of the launch */
  int32_t launches;      /* kernels launched by the call (1 = no combine pass) */
  int32_t kernel;        /* 0 vector-ALU, 1 matrix-core F16, 2 block formats, 3 KIVI matrix-core, 4 KIVI vector-ALU */
  int32_t staged_scores; /* 1: the logits of a chunk waited in LDS; 0: stored from inside the token loop (or no scores) */
} argus_hip_decode_plan;
int argus_hip_last_decode_plan(const argus_hip_ctx *ctx, argus_hip_decode_plan *plan);

/* ---- (a-2) causal GQA flash-attention prefill ---------------------------------------------- */
/* Backend::flash_attention_prefill, engine/src/backend.rs:1011-1027 (CUDA host
 * backend/cuda_pc.rs:830-926, CPU layers/attention.rs:78-351).  Key c is visible to query
 * row r iff c <= r + q_start_pos (and c + window > r + q_start_pos when window > 0), with
 * q_start_pos = cache_seq_len - seq_len; fully masked rows give zeros.
 * Returns 1 when dispatched (trait: Ok(true)), 0 when declined so the caller runs its CPU
 * path (Ok(false): SeqMajor, head_dim outside {64,128,256}, unsupported dtype -- the same
 * cases cuda_pc.rs:851-860 declines), negative on error.
 * Q/out [batch, seq_len, n_heads_q, head_dim], K/V HeadMajor [batch, n_heads_kv, capacity,
 * head_dim].  The reference shape is F32 Q/out with F16 KV; F16 Q/out is the all-f16 form. */
typedef struct argus_hip_prefill_args {
  void *stream;
  const void *q;
  const void *k_cache;
  const void *v_cache;
  void *out;
  int32_t n_heads_q;
  int32_t n_heads_kv;
  int32_t seq_len;
  int32_t cache_seq_len;
  int32_t head_dim;
  int32_t kv_capacity;
  int32_t batch_size;
  int32_t is_head_major;
  int32_t q_dtype;   /* ARGUS_HIP_F32 / ARGUS_HIP_F16 */
  int32_t kv_dtype;  /* ARGUS_HIP_F16 / ARGUS_HIP_F32 */
  int32_t out_dtype; /* ARGUS_HIP_F32 / ARGUS_HIP_F16 */
  int32_t window;    /* 0 = none */
} argus_hip_prefill_args;
int argus_hip_flash_attention_prefill(argus_hip_ctx *ctx, const argus_hip_prefill_args *args);

/* ---- (a-3) KIVI fused dequant + decode attention ------------------------------------------- */
/* Field-for-field twin of CudaQuantAttnArgs, crates/argus-extension-api/src/lib.rs:3000-3026,
 * so the Rust side is a cast.  `scores_out` is a HOST pointer filled by a blocking copy, as in
 * crates/techniques/kivi/src/gpu_kivi_cuda.rs:204-212.  Block layouts and index math:
 * crates/techniques/kivi/src/kivi_attn.cu:71-82, 256-262 (K per channel), 173-177, 357-361
 * (V per token); codec crates/argus-kv-codec/src/lib.rs:26-203. */
typedef struct argus_hip_quant_attn_args {
  void *stream;
  uint64_t q_mem;     /* [num_heads_q, head_dim] F32 */
  uint64_t qk_mem;    /* quantised key blocks, per channel, flush-interleaved */
  uint64_t qv_mem;    /* quantised value blocks, per token, flush-interleaved */
  uint64_t res_k_mem; /* residual keys [kv_heads, res_cap, head_dim] */
  uint64_t res_v_mem;
  uint64_t out_mem;   /* [num_heads_q, head_dim] F32 */
  float *scores_out;  /* host, may be NULL */
  size_t scores_len;
  size_t num_heads_q;
  size_t num_heads_kv;
  size_t head_dim;
  size_t q_tokens;
  size_t res_tokens;
  size_t res_cap;
  float scale;
  uint8_t bits; /* 2, 4 or 8 */
} argus_hip_quant_attn_args;

/* Optional extras that have no field in the reference POD. */
typedef struct argus_hip_quant_attn_ext {
  uint64_t scores_dev;   /* device score buffer [num_heads_q, score_stride]; 0 = none */
  size_t score_stride;
  int32_t res_dtype;     /* ARGUS_HIP_F32 (reference, engine/src/kv/quant_window_cache.rs:171-177) or ARGUS_HIP_F16 */
  float softcap;
  /* `batch` > 1: that many independent caches (sequences or layers) of identical geometry in one
   * launch; Q / out are [batch, num_heads_q, head_dim], block streams and residual windows sit at
   * the strides below.  The reference issues one call per cache. */
  int32_t batch;
  int64_t block_batch_stride_bytes; /* between consecutive qk (and qv) block streams */
  int64_t res_batch_stride;         /* elements between consecutive residual windows */
  int64_t score_batch_stride;       /* elements; 0 = num_heads_q * score_stride */
  /* Opt-in score form of argus_hip_attention_gen_args::score_stats: scores_dev keeps the logits and
   * (max, sum) per head go here ([batch, num_heads_q, 2] F32, device); 0 = probabilities. */
  uint64_t score_stats_dev;
} argus_hip_quant_attn_ext;

/* CudaQuantAttnBackend::{has_quant_attn_kernel, attention_gen_quant, gather_update_quant},
 * crates/argus-extension-api/src/lib.rs:3087-3104. */
int argus_hip_has_quant_attn_kernel(const argus_hip_ctx *ctx, uint8_t bits);
int argus_hip_attention_gen_quant(argus_hip_ctx *ctx, const argus_hip_quant_attn_args *args);
int argus_hip_attention_gen_quant_ex(argus_hip_ctx *ctx, const argus_hip_quant_attn_args *args,
                                     const argus_hip_quant_attn_ext *ext);

/* Twin of CudaQuantAttnGatherArgs, crates/argus-extension-api/src/lib.rs:3031-3046; kernel
 * semantics crates/techniques/kivi/src/kivi_q2.cu:117-138 (residual ring append). */
typedef struct argus_hip_quant_gather_args {
  void *stream;
  uint64_t input_mem;    /* [seq_len, kv_heads, head_dim] F32 */
  uint64_t residual_mem; /* [kv_heads, res_cap, head_dim] F32, written */
  size_t kv_heads;
  size_t res_cap;
  size_t head_dim;
  size_t seq_len;
  size_t res_pos;
} argus_hip_quant_gather_args;
int argus_hip_gather_update_quant(argus_hip_ctx *ctx, const argus_hip_quant_gather_args *args);

/* On-device quantise-at-flush: the CPU loop of QuantizedRecentWindowCache::flush_residual,
 * engine/src/kv/quant_window_cache.rs:919-946, producing bit-identical blocks appended at
 * block offsets k_block_start / v_block_start (the reference quantises on the CPU even in GPU
 * mode, quant_window_cache.rs:1700-1722). */
typedef struct argus_hip_quant_flush_args {
  void *stream;
  uint64_t res_k_mem; /* [kv_heads, res_cap, head_dim] F32 */
  uint64_t res_v_mem;
  uint64_t qk_mem;    /* destination block stream */
  uint64_t qv_mem;
  size_t kv_heads;
  size_t res_cap;
  size_t head_dim;
  size_t flush_tokens; /* multiple of 32, <= res_cap */
  size_t k_block_start;
  size_t v_block_start;
  uint8_t bits;
  /* 0: the blocks of this call form one flush (order h -> group -> ch / h -> token -> block, as the
   * CPU loop pushes them).  Otherwise a multiple of 32 that divides flush_tokens: the blocks are laid
   * out as flush_tokens / out_res_cap consecutive flushes of a ring of that capacity, the order every
   * reader assumes for a cache whose res_cap is out_res_cap (kivi_attn.cu:71-77, 173-177;
   * quant_window_cache.rs:1463-1540).  Used by the 16 -> Q transition of the container, which
   * quantises a residual of many groups in one go and continues with a ring of 32. */
  size_t out_res_cap;
} argus_hip_quant_flush_args;
int argus_hip_quant_flush(argus_hip_ctx *ctx, const argus_hip_quant_flush_args *args);

/* Bit-width transition of a block stream on the device: the block loop of
 * QuantizedRecentWindowCache::transition_bits between two quantised widths,
 * engine/src/kv/quant_window_cache.rs:1308-1372 (each block dequantised to f32 and quantised again
 * at the new width; the reference reads the streams back, does it on the CPU and uploads the result).
 * Same blocks bit for bit.  `n_blocks` blocks from src_mem to dst_mem, which must not overlap. */
typedef struct argus_hip_quant_requant_args {
  void *stream;
  uint64_t src_mem;
  uint64_t dst_mem;
  size_t n_blocks;
  uint8_t old_bits; /* 2, 4 or 8 */
  uint8_t new_bits;
} argus_hip_quant_requant_args;
int argus_hip_quant_requant(argus_hip_ctx *ctx, const argus_hip_quant_requant_args *args);

/* Dequantise flushed blocks into the F16 attention view [max_seq, kv_heads, head_dim] (sequence
 * major).  Field-for-field twin of CudaQuantDequantFlushArgs,
 * crates/argus-extension-api/src/lib.rs:3045-3063; CudaQuantAttnBackend::dequant_flush 3096-3099;
 * kernels crates/techniques/kivi/src/kivi_q2.cu:18-92 (keys: block (h, g, ch) = 32 tokens of one
 * channel, n_groups_or_tokens = groups per flush; values: block (h, t, b) = 32 channels of one
 * token, n_groups_or_tokens = flush tokens).  The reference serves bits == 2 only
 * (gpu_kivi_cuda.rs:251-254); 2, 4 and 8 are served here.  attn_mem 16-byte aligned. */
typedef struct argus_hip_quant_dequant_flush_args {
  void *stream;
  uint64_t q_blocks_mem;
  uint64_t attn_mem;
  size_t kv_heads;
  size_t head_dim;
  size_t n_groups_or_tokens;
  size_t tok_base;
  size_t block_start; /* index of the first block in q_blocks_mem */
  uint8_t bits;
  uint8_t is_key; /* Rust bool */
} argus_hip_quant_dequant_flush_args;
int argus_hip_quant_dequant_flush(argus_hip_ctx *ctx, const argus_hip_quant_dequant_flush_args *args);

/* Copy the first res_pos rows of the F32 residual ring [kv_heads, res_cap, head_dim] to rows
 * tok_base.. of the F16 attention view.  Twin of CudaQuantScatterResidualArgs, lib.rs:3065-3081;
 * CudaQuantAttnBackend::scatter_residual 3100-3103; kernel kivi_q2.cu:94-116. */
typedef struct argus_hip_quant_scatter_residual_args {
  void *stream;
  uint64_t res_mem;
  uint64_t attn_mem;
  size_t kv_heads;
  size_t res_cap;
  size_t head_dim;
  size_t res_pos;
  size_t tok_base;
} argus_hip_quant_scatter_residual_args;
int argus_hip_quant_scatter_residual(argus_hip_ctx *ctx, const argus_hip_quant_scatter_residual_args *args);

/* ---- CACHE-category capability: the KIVI container behind the reference's plugin vtable ------
 * QuantCacheBackend / QuantCacheVTable, crates/argus-extension-api/src/lib.rs:1932-2090: a stateful
 * per-layer quantised cache (F32 residual ring + the two block streams) with `make`, `current_pos`,
 * `capacity`, `current_bits`, `update`, `flush_if_full`, `assemble_view`, `get_raw_buffers`,
 * `transition_bits`, `drop`.  The structs are field-for-field twins of QuantCacheMakeArgs (1932-1955),
 * QuantCacheUpdateArgs (1957-1970), QuantCacheViewOut (1972-1986) and QuantCacheRawBuffersOut
 * (1988-2012) with the OpenCL handles replaced by their HIP counterparts, and
 * argus_hip_quant_cache_vtable lists the functions in QuantCacheVTable's order (2068-2090), so the Rust
 * side registers `argus_hip_quant_cache_get_vtable()` as the vtable of a BACKEND_CAP_CATEGORY_CACHE
 * entry.  Behaviour is the GPU mode of QuantizedRecentWindowCache
 * (engine/src/kv/quant_window_cache.rs:1563-1848, 2518-2562, 741-760, 2248-2475, 1308-1448), every
 * step on the device.  A handle allocates its ring and streams at `make` (sized for max_seq_len),
 * the F16 view at the first assemble_view, and new streams at a width transition; nothing else.
 * Work functions return 0 or a negative ARGUS_HIP_ERR_* (text in argus_hip_last_error of the context
 * given at make).
 * bits = 16 is the unquantised mode of the reference container (quant_window_cache.rs:292-300, 410-446,
 * 2417-2429): the residual covers max_seq_len tokens, nothing is flushed, the view IS the residual
 * (F32, [kv_heads, max_seq_len, head_dim], layout tag ARGUS_HIP_VIEW_HEADS_TOKENS_DIM) and there is no
 * raw-buffer set.  transition_bits(16 -> b) quantises every full group of 32 on the device and
 * continues with a ring of 32 tokens (quant_window_cache.rs:1140-1306; the block streams come out in
 * the order a ring of 32 produces, which is what the readers assume -- the reference pushes h -> group
 * -> ch over all groups at once, the same order only for one KV head); transition_bits(b -> 16)
 * refills the residual from the F16 view, as the reference's GPU mode does (988-1034), and releases
 * the view and the block streams.
 * The context given at make must outlive the handle; `make` checks that the pointer is an
 * argus_hip_ctx (a tag word at its head) and returns NULL for anything else -- a host that fills the
 * slot with a context of its own kind passes NULL instead and the handle creates one. */
#define ARGUS_HIP_VIEW_TOKENS_HEADS_DIM 0u /* ViewLayoutTag::HeadMajor of lib.rs:1917-1926: [tokens, kv_heads, head_dim] */
#define ARGUS_HIP_VIEW_HEADS_TOKENS_DIM 1u /* ViewLayoutTag::SeqMajor: [kv_heads, tokens, head_dim]; bits = 16 only */
typedef struct argus_hip_quant_cache_make_args {
  void *ctx;              /* cl_ctx slot: the argus_hip_ctx the cache allocates from and launches on; NULL: a
                             context of its own on the current device, destroyed with the handle */
  void *device;           /* cl_device_id slot: unused */
  void *stream;           /* cl_queue slot: the stream of every call of the handle (NULL = default) */
  const char *build_opts; /* unused */
  size_t kv_heads;
  size_t head_dim;      /* multiple of 32 */
  size_t max_seq_len;
  size_t residual_size; /* positive multiple of 32 (not used while bits = 16) */
  uint8_t bits;         /* 2, 4, 8 or 16 */
} argus_hip_quant_cache_make_args;
typedef struct argus_hip_quant_cache_update_args {
  void *stream;   /* NULL or the stream given at make (the handle works on one stream) */
  void *k_in_mem; /* device F32 [seq_len, kv_heads, head_dim] */
  void *v_in_mem;
  size_t seq_len; /* 1 = decode, > 1 = prefill batch */
} argus_hip_quant_cache_update_args;
typedef struct argus_hip_quant_cache_view_out {
  void *k_mem; /* F16 [max_seq_len, kv_heads, head_dim], rows [0, tokens) valid; bits = 16: the F32 residual */
  void *v_mem;
  size_t tokens;
  uint32_t layout; /* ARGUS_HIP_VIEW_TOKENS_HEADS_DIM, or ARGUS_HIP_VIEW_HEADS_TOKENS_DIM while bits = 16 */
} argus_hip_quant_cache_view_out;
typedef struct argus_hip_quant_cache_raw_buffers_out {
  void *qk_mem;
  void *qv_mem;
  void *res_k_mem;
  void *res_v_mem;
  size_t q_tokens;
  size_t res_tokens;
  size_t res_cap;
  uint8_t bits;
} argus_hip_quant_cache_raw_buffers_out;
void *argus_hip_quant_cache_make(const argus_hip_quant_cache_make_args *args); /* NULL on failure */
size_t argus_hip_quant_cache_current_pos(void *handle);
size_t argus_hip_quant_cache_capacity(void *handle);
uint8_t argus_hip_quant_cache_current_bits(void *handle);
int32_t argus_hip_quant_cache_update(void *handle, const argus_hip_quant_cache_update_args *args);
int32_t argus_hip_quant_cache_flush_if_full(void *handle);
int32_t argus_hip_quant_cache_assemble_view(void *handle, argus_hip_quant_cache_view_out *out);
/* false (out untouched) when there is no native-consumable set: an empty cache, or bits = 16. */
bool argus_hip_quant_cache_get_raw_buffers(void *handle, argus_hip_quant_cache_raw_buffers_out *out);
int32_t argus_hip_quant_cache_transition_bits(void *handle, uint8_t target_bits);
void argus_hip_quant_cache_drop(void *handle);
typedef struct argus_hip_quant_cache_vtable {
  void *(*make)(const argus_hip_quant_cache_make_args *);
  size_t (*current_pos)(void *);
  size_t (*capacity)(void *);
  uint8_t (*current_bits)(void *);
  int32_t (*update)(void *, const argus_hip_quant_cache_update_args *);
  int32_t (*flush_if_full)(void *);
  int32_t (*assemble_view)(void *, argus_hip_quant_cache_view_out *);
  bool (*get_raw_buffers)(void *, argus_hip_quant_cache_raw_buffers_out *);
  int32_t (*transition_bits)(void *, uint8_t);
  void (*drop)(void *);
} argus_hip_quant_cache_vtable;
const argus_hip_quant_cache_vtable *argus_hip_quant_cache_get_vtable(void);

/* ---- the reference's dlopen plugin protocol -----------------------------------------------------
 * A capability plugin is a shared library that exports `register_backend_caps_v2`, returning by
 * value the envelope BackendCapExportAbi { abi_version, count, vtables } of entries
 * BackendCapVTableAbi { name, category, vtable } (crates/argus-extension-api/src/lib.rs:1752-1782,
 * BACKEND_CAP_ABI_VERSION = 2 at 1574, categories ATTENTION = 1 at 1578 and CACHE = 2 at 1914; loaded by
 * engine/src/capability/dynamic_backend_registry.rs:50-160 and resolved by `--backend-cap <name>`).
 * This library is such a plugin: it registers the fused dequant + attention capability as
 * "kivi_hip" (QuantAttnVTable, lib.rs:1726-1746: make, has_quant_attn_kernel, is_nosub_device,
 * attention_gen_quant, gather_update_quant, dequant_flush, scatter_residual, drop) and the container
 * above as "kivi_cache_hip".  The ATTENTION handle owns a context on the device that is current when
 * `make` is called and ignores the OpenCL handles of QuantAttnMakeArgs (lib.rs:1583-1592); the `*_mem`
 * slots of the argument structs carry HIP device pointers and the `cl_queue` slot the HIP stream, as
 * in the entry points of the same names above.  A CACHE `make` with a NULL `ctx` slot does the same. */
#define ARGUS_BACKEND_CAP_ABI_VERSION 2u
#define ARGUS_BACKEND_CAP_CATEGORY_ATTENTION 1u
#define ARGUS_BACKEND_CAP_CATEGORY_CACHE 2u
#define ARGUS_HIP_CAP_NAME_ATTENTION "kivi_hip"
#define ARGUS_HIP_CAP_NAME_CACHE "kivi_cache_hip"
typedef struct argus_hip_quant_attn_make_args {
  void *cl_ctx;
  void *device;
  const char *build_opts;
} argus_hip_quant_attn_make_args;
typedef struct argus_hip_quant_attn_vtable {
  void *(*make)(const argus_hip_quant_attn_make_args *);
  bool (*has_quant_attn_kernel)(void *, uint8_t);
  bool (*is_nosub_device)(void *);
  int32_t (*attention_gen_quant)(void *, const argus_hip_quant_attn_args *);
  int32_t (*gather_update_quant)(void *, const argus_hip_quant_gather_args *);
  int32_t (*dequant_flush)(void *, const argus_hip_quant_dequant_flush_args *);
  int32_t (*scatter_residual)(void *, const argus_hip_quant_scatter_residual_args *);
  void (*drop)(void *);
} argus_hip_quant_attn_vtable;
void *argus_hip_quant_attn_cap_make(const argus_hip_quant_attn_make_args *args); /* NULL on failure */
bool argus_hip_quant_attn_cap_has_kernel(void *handle, uint8_t bits);
bool argus_hip_quant_attn_cap_is_nosub_device(void *handle);
int32_t argus_hip_quant_attn_cap_attention_gen_quant(void *handle, const argus_hip_quant_attn_args *args);
int32_t argus_hip_quant_attn_cap_gather_update_quant(void *handle, const argus_hip_quant_gather_args *args);
int32_t argus_hip_quant_attn_cap_dequant_flush(void *handle, const argus_hip_quant_dequant_flush_args *args);
int32_t argus_hip_quant_attn_cap_scatter_residual(void *handle, const argus_hip_quant_scatter_residual_args *args);
void argus_hip_quant_attn_cap_drop(void *handle);
const argus_hip_quant_attn_vtable *argus_hip_quant_attn_get_vtable(void);
typedef struct argus_backend_cap_vtable_abi {
  const char *name;
  uint32_t category;
  const void *vtable;
} argus_backend_cap_vtable_abi;
typedef struct argus_backend_cap_export_abi {
  uint32_t abi_version;
  size_t count;
  const argus_backend_cap_vtable_abi *vtables;
} argus_backend_cap_export_abi;
argus_backend_cap_export_abi register_backend_caps_v2(void);

/* ---- (a-6) PFA side channel: prefill attention scores on the device --------------------------
 * Stands in for the host mirror prefill_attention_scores, engine/src/kv/standard_format.rs:
 * 1400-1510 (arguments in the same order and meaning; PerRowScores { out, per_head } becomes
 * per_row_out / per_row_per_head), which the reference can only run after reading K back from
 * VRAM (standard_format.rs:1137-1173).  q: device F32 [seq_len, n_heads_q, head_dim]; k: device
 * F32 or F16 addressed as k[key * k_pos_stride + kv_head * kv_head_stride + d] (elements), so both
 * cache layouts work.  sum_out [n_heads_q, cache_seq_len] is accumulated in place (+=);
 * per_row_out is [q_window, n_heads_q, cache_seq_len] written (per head) or
 * [q_window, cache_seq_len] accumulated with 1/n_heads_q (head mean).  Either may be NULL.
 * Single sequence, like the reference. */
typedef struct argus_hip_pfa_args {
  void *stream;
  const void *q;
  const void *k;
  int32_t k_dtype; /* ARGUS_HIP_F32 / ARGUS_HIP_F16 */
  int32_t n_heads_q;
  int32_t n_heads_kv;
  int32_t head_dim;
  int32_t seq_len;
  int32_t cache_seq_len;
  int64_t k_pos_stride;
  int64_t kv_head_stride;
  int32_t q_start_pos;
  int32_t q_window;
  int32_t has_window; /* Option<usize>: 0 = None */
  int32_t window;
  void *sum_out;
  void *per_row_out;
  int32_t per_row_per_head;
} argus_hip_pfa_args;
int argus_hip_prefill_attention_scores(argus_hip_ctx *ctx, const argus_hip_pfa_args *args);

/* ---- (f-4) descriptor-driven block formats: the device-side floor of --kv-format -------------
 * KVLayoutDesc twin (crates/argus-extension-api/src/lib.rs:1111-1159): scale_layout 0 None,
 * 1 PerBlockF16, 2 PerBlockF16WithMin; packing 0 Dense, 1 Nibble, 2 Byte, 3 Quad.
 * kv_decode_descriptor = decode_via_descriptor / unpack_block_via_descriptor
 * (engine/src/format/dtype_layout.rs:102-166, 285-300) into F32 or F16, bit-identical;
 * kv_encode_descriptor = encode_via_descriptor (302-396), q4_0- and q2_0-style only, other
 * descriptors return ARGUS_HIP_ERR_UNSUPPORTED like the reference's Err.  n_elems is a multiple of
 * block_elems (<= 64); block buffers are 2-byte aligned.  They replace the host dequant-to-F32 of
 * standard_format.rs:538-643 by a device pass followed by the F16/F32 attention entry points. */
typedef struct argus_hip_kv_layout_desc {
  uint32_t block_elems;
  uint8_t bits;
  uint32_t scale_layout;
  uint32_t packing;
} argus_hip_kv_layout_desc;
int argus_hip_kv_decode_descriptor(argus_hip_ctx *ctx, void *stream, const argus_hip_kv_layout_desc *desc, const void *src,
                                   void *dst, int32_t dst_dtype, int64_t n_elems);
int argus_hip_kv_encode_descriptor(argus_hip_ctx *ctx, void *stream, const argus_hip_kv_layout_desc *desc, const void *src,
                                   void *dst, int64_t n_elems);
/* Backend::attention_gen over a cache whose rows are blocks of `desc`: what StandardFormat computes for
 * an opaque --kv-format cache after decoding it whole (engine/src/kv/standard_format.rs:538-643 with
 * engine/src/format/dtype_layout.rs:102-166), without the decoded copy.  `args` as for
 * argus_hip_attention_gen (kv_dtype ignored; capacity, kv_start and strides in elements, whole blocks;
 * caches 2-byte aligned).  Any PerBlockF16 / PerBlockF16WithMin x Nibble / Byte / Quad descriptor whose
 * block_elems is a multiple of 8, at most 64 and divides head_dim is attended in-kernel: q4_0 / q4_1 /
 * q8_0 / q2_0 on the matrix cores, every other one by the vector-ALU kernel (each lane decodes its 8
 * channels from the row's blocks), any GQA ratio.  Every other descriptor (Dense packing, no scale,
 * shared exponents, codebooks, ...) is DECLINED: ARGUS_HIP_ERR_UNSUPPORTED, nothing launched, and the
 * caller takes the floor (argus_hip_kv_decode_descriptor or its CPU decode, then the F16 / F32 call). */
int argus_hip_attention_gen_desc(argus_hip_ctx *ctx, const argus_hip_attention_gen_args *args,
                                 const argus_hip_kv_layout_desc *desc);

/* ---- (a-4) attention-score reduce for H2O / D2O --------------------------------------------- */
/* Field-for-field twin of CudaScoreReduceArgs, crates/argus-extension-api/src/lib.rs:2909-2933;
 * CudaScoreReduceBackend::{reduce, reduce_per_layer} 2938-2948; kernel semantics
 * crates/techniques/attn-score/src/score_reduce.cu:13-62, 64-91. */
typedef struct argus_hip_score_reduce_args {
  void *stream;
  uint64_t score_buf;       /* [n_layers, n_heads_q, score_stride] F32 */
  uint64_t importance;      /* [max_seq_len] F32, in place */
  uint64_t head_importance; /* [n_kv_heads * max_seq_len] F32, in place */
  float decay_factor;
  size_t n_layers;
  size_t n_heads_q;
  size_t n_kv_heads; /* <= 16 */
  size_t cache_seq_len;
  size_t score_stride;
  size_t max_seq_len;
  uint64_t layer_flat_importance; /* [n_layers * max_seq_len] or 0 */
} argus_hip_score_reduce_args;
int argus_hip_score_reduce(argus_hip_ctx *ctx, const argus_hip_score_reduce_args *args);
int argus_hip_score_reduce_per_layer(argus_hip_ctx *ctx, const argus_hip_score_reduce_args *args);
/* The same reduces over a score buffer in the logits + (max, sum) form (argus_hip_attention_gen_args::
 * score_stats): `stats` is [n_layers, n_heads_q, 2] F32 on the device and every score is taken as
 * exp(s - max) / sum while it is read -- the arithmetic of the rewrite the attention call skipped, so the
 * results equal those of the probability form bit for bit.  The reference reduce
 * (crates/techniques/attn-score/src/score_reduce.cu:13-91) reads probabilities only; this form exists
 * because the rewrite of a 32K-token score buffer costs as much as the reduce itself.  stats == 0:
 * identical to the calls above. */
typedef struct argus_hip_score_reduce_ext {
  uint64_t stats;
} argus_hip_score_reduce_ext;
int argus_hip_score_reduce_ex(argus_hip_ctx *ctx, const argus_hip_score_reduce_args *args,
                              const argus_hip_score_reduce_ext *ext);
int argus_hip_score_reduce_per_layer_ex(argus_hip_ctx *ctx, const argus_hip_score_reduce_args *args,
                                        const argus_hip_score_reduce_ext *ext);

/* ---- (f-1) KV write path ---------------------------------------------------------------------- */
/* Backend::kv_scatter_f32_to_f16 / _batch / _f32_batch, engine/src/backend.rs:425-545; device
 * semantics engine/src/backend/cuda_pc/kernels.cu:305-360.  src [seq_len, kv_heads, head_dim]
 * F32 -> dst HeadMajor [kv_heads, capacity, head_dim] at rows write_pos_start + s. */
int argus_hip_kv_scatter_f32_to_f16(argus_hip_ctx *ctx, void *stream, const float *k_src,
                                    const float *v_src, void *k_dst, void *v_dst, int32_t kv_heads,
                                    int32_t head_dim, int32_t capacity, int32_t write_pos);
int argus_hip_kv_scatter_f32_to_f16_batch(argus_hip_ctx *ctx, void *stream, const float *k_src,
                                          const float *v_src, void *k_dst, void *v_dst,
                                          int32_t kv_heads, int32_t head_dim, int32_t capacity,
                                          int32_t write_pos_start, int32_t seq_len);
int argus_hip_kv_scatter_f32_batch(argus_hip_ctx *ctx, void *stream, const float *k_src,
                                   const float *v_src, float *k_dst, float *v_dst, int32_t kv_heads,
                                   int32_t head_dim, int32_t capacity, int32_t write_pos_start,
                                   int32_t seq_len);

#ifdef __cplusplus
}
#endif
#endif /* ARGUS_HIP_H */
