// The KIVI container as a C ABI: the CACHE-category capability of the reference's plugin interface
// (QuantCacheBackend / QuantCacheVTable, crates/argus-extension-api/src/lib.rs:1932-2090) served by the
// GPU mode of QuantizedRecentWindowCache (engine/src/kv/quant_window_cache.rs:380-586 new_gpu,
// 2518-2562 update, 1563-1686 update_gpu, 1688-1848 flush_residual_gpu, 741-760 get_raw_gpu_buffers,
// 2248-2475 assemble_view_gpu, 1308-1448 transition_bits between quantised widths) with every step on
// the device: append = the gather kernel, flush = quantise-at-flush, the tokens a flush leaves behind
// move down with the overlap-safe shift, a width transition requantises both block streams in place
// of the reference's read-back / CPU loop / upload.  bits = 16 is the unquantised mode (292-300,
// 410-446): the residual spans max_seq_len tokens and doubles as the view; the transitions to and from
// it (975-1306) quantise the whole residual on the device, or refill it from the F16 view.  Host code
// apart from one copy kernel; the other kernels are those of kivi_attn.hip and kivi_view.hip behind
// their own entry points.
#include "argus_hip_internal.hpp"

#include <algorithm>
#include <new>

namespace {

constexpr size_t kGroup = 32;  // QKKV: tokens per key block, channels per value block

struct QuantCache {
  argus_hip_ctx *ctx = nullptr;
  bool owns_ctx = false;  // made without a context: one of its own, destroyed with the handle
  void *stream = nullptr;
  size_t kv_heads = 0, head_dim = 0, max_seq_len = 0, res_cap = 0;  // res_cap: max_seq_len while bits = 16
  uint8_t bits = 0;
  size_t q_tokens = 0, res_pos = 0, deq_tokens = 0;
  void *res_k = nullptr, *res_v = nullptr, *qk = nullptr, *qv = nullptr, *attn_k = nullptr, *attn_v = nullptr;

  size_t block_bytes(uint8_t b) const { return 4 + kGroup * b / 8; }
  // blocks one stream can come to hold: whole groups of max_seq_len tokens
  size_t stream_blocks() const { return (max_seq_len / kGroup + 1) * kv_heads * head_dim; }
  size_t blocks_held() const { return q_tokens * kv_heads * head_dim / kGroup; }
  void release() {
    for (void **p : {&res_k, &res_v, &qk, &qv, &attn_k, &attn_v}) {
      if (*p) argus_hip_free(ctx, *p);
      *p = nullptr;
    }
  }
};

// F16 view rows [tokens, kv_heads, D] -> F32 residual [kv_heads, res_cap, D] (transition to bits = 16)
__global__ __launch_bounds__(256) void view_to_residual_kernel(const _Float16 *__restrict__ view, float *__restrict__ res, int kv_heads,
                                                               int64_t res_cap, int D, int64_t tokens) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int cpr = D / 8;
  if (idx >= tokens * kv_heads * cpr) return;
  const int c = (int)(idx % cpr);
  const int h = (int)((idx / cpr) % kv_heads);
  const int64_t t = idx / ((int64_t)cpr * kv_heads);
  const half8_t v = *(const half8_t *)(view + (t * kv_heads + h) * D + 8 * c);
  float *dst = res + ((int64_t)h * res_cap + t) * D + 8 * c;
  *(float4_t *)dst = float4_t{(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
  *(float4_t *)(dst + 4) = float4_t{(float)v[4], (float)v[5], (float)v[6], (float)v[7]};
}

// flush_residual_gpu: whole groups of the ring become blocks, the remainder moves to the ring's start.
int flush_residual(QuantCache *c, void *stream) {
  if (c->bits == 16) return ARGUS_HIP_OK;  // residual-only mode: nothing is ever quantised (845-848)
  const size_t flush_tokens = c->res_pos / kGroup * kGroup;
  if (flush_tokens == 0) return ARGUS_HIP_OK;
  argus_hip_quant_flush_args f{};
  f.stream = stream;
  f.res_k_mem = (uint64_t)c->res_k; f.res_v_mem = (uint64_t)c->res_v;
  f.qk_mem = (uint64_t)c->qk; f.qv_mem = (uint64_t)c->qv;
  f.kv_heads = c->kv_heads; f.res_cap = c->res_cap; f.head_dim = c->head_dim; f.flush_tokens = flush_tokens;
  f.k_block_start = f.v_block_start = c->blocks_held();
  f.bits = c->bits;
  int rc = argus_hip_quant_flush(c->ctx, &f);
  if (rc != ARGUS_HIP_OK) return rc;
  c->q_tokens += flush_tokens;
  const size_t remaining = c->res_pos - flush_tokens;
  if (remaining > 0) {
    for (void *ring : {c->res_k, c->res_v})
      for (size_t h = 0; h < c->kv_heads; ++h) {
        float *base = (float *)ring + h * c->res_cap * c->head_dim;
        rc = argus_hip_buffer_shift(c->ctx, stream, base, base + flush_tokens * c->head_dim, remaining * c->head_dim * sizeof(float));
        if (rc != ARGUS_HIP_OK) return rc;
      }
  }
  c->res_pos = remaining;
  return ARGUS_HIP_OK;
}

}  // namespace

ARGUS_API void *argus_hip_quant_cache_make(const argus_hip_quant_cache_make_args *a) {
  if (!a) return nullptr;
  argus_hip_ctx *ctx = (argus_hip_ctx *)a->ctx;
  // The slot is untyped (the reference's cl_context): anything that is not one of this library's
  // contexts is refused rather than written through.
  if (ctx && ctx->tag != kArgusCtxTag) return nullptr;
  const bool owns_ctx = ctx == nullptr;
  if (owns_ctx) {
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess) {
      (void)hipGetLastError();
      return nullptr;
    }
    if (argus_hip_create(device, &ctx) != ARGUS_HIP_OK) return nullptr;
  }
  struct CtxGuard {  // a refused make gives the context back
    argus_hip_ctx *ctx;
    bool armed;
    ~CtxGuard() {
      if (armed) argus_hip_destroy(ctx);
    }
  } guard{ctx, owns_ctx};
  // the reference asserts these (quant_window_cache.rs:283-295)
  if (a->bits != 2 && a->bits != 4 && a->bits != 8 && a->bits != 16) {
    argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "quant_cache_make: bits %d (2, 4, 8 or 16)", (int)a->bits);
    return nullptr;
  }
  if (a->kv_heads == 0 || a->head_dim == 0 || a->head_dim % kGroup || a->residual_size == 0 || a->residual_size % kGroup ||
      a->max_seq_len == 0) {
    argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "quant_cache_make: kv_heads %zu head_dim %zu residual_size %zu max_seq_len %zu", a->kv_heads,
               a->head_dim, a->residual_size, a->max_seq_len);
    return nullptr;
  }
  QuantCache *c = new (std::nothrow) QuantCache();
  if (!c) return nullptr;  // (the guard returns an owned context)
  c->ctx = ctx; c->owns_ctx = owns_ctx; c->stream = a->stream;
  c->kv_heads = a->kv_heads; c->head_dim = a->head_dim; c->max_seq_len = a->max_seq_len; c->bits = a->bits;
  // bits = 16: the residual covers the full sequence and no block stream exists (297-300, 410)
  c->res_cap = a->bits == 16 ? a->max_seq_len : a->residual_size;
  const size_t res_bytes = c->kv_heads * c->res_cap * c->head_dim * sizeof(float);
  const size_t stream_bytes = c->stream_blocks() * c->block_bytes(c->bits);
  bool ok = argus_hip_malloc(ctx, res_bytes, &c->res_k) == ARGUS_HIP_OK && argus_hip_malloc(ctx, res_bytes, &c->res_v) == ARGUS_HIP_OK;
  if (ok && a->bits != 16)
    ok = argus_hip_malloc(ctx, stream_bytes, &c->qk) == ARGUS_HIP_OK && argus_hip_malloc(ctx, stream_bytes, &c->qv) == ARGUS_HIP_OK;
  if (!ok) {
    c->release();
    delete c;
    return nullptr;
  }
  guard.armed = false;
  return c;
}

ARGUS_API void argus_hip_quant_cache_drop(void *handle) {
  QuantCache *c = (QuantCache *)handle;
  if (!c) return;
  c->release();
  if (c->owns_ctx) argus_hip_destroy(c->ctx);
  delete c;
}

ARGUS_API size_t argus_hip_quant_cache_current_pos(void *handle) {
  const QuantCache *c = (const QuantCache *)handle;
  return c ? c->q_tokens + c->res_pos : 0;
}
ARGUS_API size_t argus_hip_quant_cache_capacity(void *handle) {
  const QuantCache *c = (const QuantCache *)handle;
  return c ? c->max_seq_len : 0;
}
ARGUS_API uint8_t argus_hip_quant_cache_current_bits(void *handle) {
  const QuantCache *c = (const QuantCache *)handle;
  return c ? c->bits : 0;
}

ARGUS_API int32_t argus_hip_quant_cache_update(void *handle, const argus_hip_quant_cache_update_args *a) {
  QuantCache *c = (QuantCache *)handle;
  if (!c || !a) return ARGUS_HIP_ERR_INVALID;
  if (a->seq_len == 0) return ARGUS_HIP_OK;
  if (!a->k_in_mem || !a->v_in_mem) return argus_fail(c->ctx, ARGUS_HIP_ERR_INVALID, "quant_cache_update: null input");
  if (c->q_tokens + c->res_pos + a->seq_len > c->max_seq_len)
    return argus_fail(c->ctx, ARGUS_HIP_ERR_INVALID, "QuantWindowCache overflow: %zu + %zu > %zu", c->q_tokens + c->res_pos, a->seq_len,
                      c->max_seq_len);
  // One stream per handle: the flush, view and transition calls carry no stream of their own, so an
  // update on another queue would race them.
  if (a->stream && a->stream != c->stream)
    return argus_fail(c->ctx, ARGUS_HIP_ERR_INVALID, "quant_cache_update: the stream differs from the one given at make");
  void *stream = c->stream;
  size_t written = 0;
  while (written < a->seq_len) {
    if (c->res_pos >= c->res_cap) {
      const int rc = flush_residual(c, stream);
      if (rc != ARGUS_HIP_OK) return rc;
    }
    const size_t batch = std::min(a->seq_len - written, c->res_cap - c->res_pos);
    const size_t off = written * c->kv_heads * c->head_dim * sizeof(float);
    for (int which = 0; which < 2; ++which) {
      argus_hip_quant_gather_args g{stream, (uint64_t)((const char *)(which ? a->v_in_mem : a->k_in_mem) + off),
                                    (uint64_t)(which ? c->res_v : c->res_k), c->kv_heads, c->res_cap, c->head_dim, batch, c->res_pos};
      const int rc = argus_hip_gather_update_quant(c->ctx, &g);
      if (rc != ARGUS_HIP_OK) return rc;
    }
    c->res_pos += batch;
    written += batch;
  }
  return ARGUS_HIP_OK;
}

ARGUS_API int32_t argus_hip_quant_cache_flush_if_full(void *handle) {
  QuantCache *c = (QuantCache *)handle;
  if (!c) return ARGUS_HIP_ERR_INVALID;
  if (c->res_pos < c->res_cap) return ARGUS_HIP_OK;
  return flush_residual(c, c->stream);
}

ARGUS_API int32_t argus_hip_quant_cache_assemble_view(void *handle, argus_hip_quant_cache_view_out *out) {
  QuantCache *c = (QuantCache *)handle;
  if (!c || !out) return ARGUS_HIP_ERR_INVALID;
  if (c->bits == 16) {  // the residual is the view (2417-2429)
    out->k_mem = c->res_k;
    out->v_mem = c->res_v;
    out->tokens = c->res_pos;
    out->layout = ARGUS_HIP_VIEW_HEADS_TOKENS_DIM;
    return ARGUS_HIP_OK;
  }
  // the view is allocated once, at max_seq_len, the first time it is asked for
  const size_t view_bytes = c->max_seq_len * c->kv_heads * c->head_dim * 2;
  for (void **p : {&c->attn_k, &c->attn_v})
    if (!*p) {
      const int rc = argus_hip_malloc(c->ctx, view_bytes, p);
      if (rc != ARGUS_HIP_OK) return rc;
    }
  while (c->deq_tokens < c->q_tokens) {
    // one flush of the streams at a time: key blocks are grouped per flush
    const size_t flush_tokens = std::min(c->res_cap, c->q_tokens - c->deq_tokens);
    const size_t block_start = c->deq_tokens * c->kv_heads * c->head_dim / kGroup;
    argus_hip_quant_dequant_flush_args dk{c->stream, (uint64_t)c->qk, (uint64_t)c->attn_k, c->kv_heads, c->head_dim, flush_tokens / kGroup,
                                          c->deq_tokens, block_start, c->bits, 1};
    argus_hip_quant_dequant_flush_args dv{c->stream, (uint64_t)c->qv, (uint64_t)c->attn_v, c->kv_heads, c->head_dim, flush_tokens,
                                          c->deq_tokens, block_start, c->bits, 0};
    int rc = argus_hip_quant_dequant_flush(c->ctx, &dk);
    if (rc == ARGUS_HIP_OK) rc = argus_hip_quant_dequant_flush(c->ctx, &dv);
    if (rc != ARGUS_HIP_OK) return rc;
    c->deq_tokens += flush_tokens;
  }
  if (c->res_pos > 0) {
    argus_hip_quant_scatter_residual_args sk{c->stream, (uint64_t)c->res_k, (uint64_t)c->attn_k, c->kv_heads, c->res_cap, c->head_dim,
                                             c->res_pos, c->q_tokens};
    argus_hip_quant_scatter_residual_args sv = sk;
    sv.res_mem = (uint64_t)c->res_v;
    sv.attn_mem = (uint64_t)c->attn_v;
    int rc = argus_hip_quant_scatter_residual(c->ctx, &sk);
    if (rc == ARGUS_HIP_OK) rc = argus_hip_quant_scatter_residual(c->ctx, &sv);
    if (rc != ARGUS_HIP_OK) return rc;
  }
  out->k_mem = c->attn_k;
  out->v_mem = c->attn_v;
  out->tokens = c->q_tokens + c->res_pos;
  out->layout = ARGUS_HIP_VIEW_TOKENS_HEADS_DIM;
  return ARGUS_HIP_OK;
}

ARGUS_API bool argus_hip_quant_cache_get_raw_buffers(void *handle, argus_hip_quant_cache_raw_buffers_out *out) {
  const QuantCache *c = (const QuantCache *)handle;
  if (!c || !out || c->bits == 16 || c->q_tokens + c->res_pos == 0) return false;  // no native-consumable set (742-744)
  out->qk_mem = c->qk; out->qv_mem = c->qv; out->res_k_mem = c->res_k; out->res_v_mem = c->res_v;
  out->q_tokens = c->q_tokens; out->res_tokens = c->res_pos; out->res_cap = c->res_cap; out->bits = c->bits;
  return true;
}

namespace {

// 2/4/8 -> 16 (quant_window_cache.rs:988-1130): every token goes back into an F32 residual of
// max_seq_len rows per head, through the F16 view as in the reference's GPU mode; the view and the
// block streams are released.
int transition_to_unquantised(QuantCache *c) {
  const size_t total = c->q_tokens + c->res_pos;
  argus_hip_quant_cache_view_out view{};
  int rc = total > 0 ? argus_hip_quant_cache_assemble_view(c, &view) : ARGUS_HIP_OK;
  if (rc != ARGUS_HIP_OK) return rc;
  const size_t res_bytes = c->kv_heads * c->max_seq_len * c->head_dim * sizeof(float);
  void *nk = nullptr, *nv = nullptr;
  rc = argus_hip_malloc(c->ctx, res_bytes, &nk);
  if (rc == ARGUS_HIP_OK) rc = argus_hip_malloc(c->ctx, res_bytes, &nv);
  if (rc == ARGUS_HIP_OK && total > 0) {
    const int64_t n = (int64_t)total * c->kv_heads * (c->head_dim / 8);
    for (int which = 0; which < 2; ++which)
      hipLaunchKernelGGL(view_to_residual_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)c->stream,
                         (const _Float16 *)(which ? view.v_mem : view.k_mem), (float *)(which ? nv : nk), (int)c->kv_heads,
                         (int64_t)c->max_seq_len, (int)c->head_dim, (int64_t)total);
    if (hipGetLastError() != hipSuccess) rc = argus_fail(c->ctx, ARGUS_HIP_ERR_RUNTIME, "quant_cache_transition_bits: launch failed");
    // everything the copies read is freed below
    if (rc == ARGUS_HIP_OK) rc = argus_hip_synchronize(c->ctx, c->stream);
  }
  if (rc != ARGUS_HIP_OK) {
    if (nk) argus_hip_free(c->ctx, nk);
    if (nv) argus_hip_free(c->ctx, nv);
    return rc;
  }
  c->release();
  c->res_k = nk;
  c->res_v = nv;
  c->res_cap = c->max_seq_len;
  c->res_pos = total;
  c->q_tokens = c->deq_tokens = 0;
  c->bits = 16;
  return ARGUS_HIP_OK;
}

// 16 -> 2/4/8 (quant_window_cache.rs:1137-1306): every full group of the residual is quantised, the
// rest moves into a ring of 32 tokens, which is the cache's residual from then on.
int transition_from_unquantised(QuantCache *c, uint8_t bits) {
  const size_t new_cap = kGroup;
  const size_t flush_tokens = c->res_pos / kGroup * kGroup, remaining = c->res_pos - flush_tokens;
  const size_t stream_bytes = c->stream_blocks() * c->block_bytes(bits);
  const size_t ring_bytes = c->kv_heads * new_cap * c->head_dim * sizeof(float);
  void *qk = nullptr, *qv = nullptr, *rk = nullptr, *rv = nullptr;
  int rc = argus_hip_malloc(c->ctx, stream_bytes, &qk);
  if (rc == ARGUS_HIP_OK) rc = argus_hip_malloc(c->ctx, stream_bytes, &qv);
  if (rc == ARGUS_HIP_OK) rc = argus_hip_malloc(c->ctx, ring_bytes, &rk);
  if (rc == ARGUS_HIP_OK) rc = argus_hip_malloc(c->ctx, ring_bytes, &rv);
  if (rc == ARGUS_HIP_OK && flush_tokens > 0) {
    argus_hip_quant_flush_args f{};
    f.stream = c->stream;
    f.res_k_mem = (uint64_t)c->res_k; f.res_v_mem = (uint64_t)c->res_v;
    f.qk_mem = (uint64_t)qk; f.qv_mem = (uint64_t)qv;
    f.kv_heads = c->kv_heads; f.res_cap = c->res_cap; f.head_dim = c->head_dim; f.flush_tokens = flush_tokens;
    f.bits = bits;
    f.out_res_cap = new_cap;  // the order a ring of 32 would have produced, flush by flush
    rc = argus_hip_quant_flush(c->ctx, &f);
  }
  for (size_t h = 0; rc == ARGUS_HIP_OK && remaining > 0 && h < c->kv_heads; ++h) {
    const size_t src = (h * c->res_cap + flush_tokens) * c->head_dim, dst = h * new_cap * c->head_dim;
    rc = argus_hip_copy_slice(c->ctx, c->stream, (float *)rk + dst, (const float *)c->res_k + src, remaining * c->head_dim * sizeof(float));
    if (rc == ARGUS_HIP_OK)
      rc = argus_hip_copy_slice(c->ctx, c->stream, (float *)rv + dst, (const float *)c->res_v + src, remaining * c->head_dim * sizeof(float));
  }
  // the old residual is freed below: every kernel that reads it must have finished
  if (rc == ARGUS_HIP_OK) rc = argus_hip_synchronize(c->ctx, c->stream);
  if (rc != ARGUS_HIP_OK) {
    for (void *p : {qk, qv, rk, rv})
      if (p) argus_hip_free(c->ctx, p);
    return rc;
  }
  c->release();
  c->qk = qk; c->qv = qv; c->res_k = rk; c->res_v = rv;
  c->res_cap = new_cap;
  c->res_pos = remaining;
  c->q_tokens = flush_tokens;
  c->deq_tokens = 0;
  c->bits = bits;
  return ARGUS_HIP_OK;
}

}  // namespace

ARGUS_API int32_t argus_hip_quant_cache_transition_bits(void *handle, uint8_t target_bits) {
  QuantCache *c = (QuantCache *)handle;
  if (!c) return ARGUS_HIP_ERR_INVALID;
  if (target_bits == c->bits) return ARGUS_HIP_OK;
  if (target_bits != 2 && target_bits != 4 && target_bits != 8 && target_bits != 16)
    return argus_fail(c->ctx, ARGUS_HIP_ERR_UNSUPPORTED, "quant_cache_transition_bits: %d -> %d (widths 2, 4, 8, 16)", (int)c->bits,
                      (int)target_bits);
  if (target_bits == 16) return transition_to_unquantised(c);
  if (c->bits == 16) return transition_from_unquantised(c, target_bits);
  // Both streams are rewritten at the new block size into fresh buffers (the one allocation this
  // handle makes after `make`; a transition is a rare, policy-driven event), then the old ones go.
  const size_t new_bytes = c->stream_blocks() * c->block_bytes(target_bits);
  void *nk = nullptr, *nv = nullptr;
  int rc = argus_hip_malloc(c->ctx, new_bytes, &nk);
  if (rc == ARGUS_HIP_OK) rc = argus_hip_malloc(c->ctx, new_bytes, &nv);
  if (rc == ARGUS_HIP_OK && c->q_tokens > 0) {
    argus_hip_quant_requant_args r{c->stream, (uint64_t)c->qk, (uint64_t)nk, c->blocks_held(), c->bits, target_bits};
    rc = argus_hip_quant_requant(c->ctx, &r);
    if (rc == ARGUS_HIP_OK) {
      r.src_mem = (uint64_t)c->qv;
      r.dst_mem = (uint64_t)nv;
      rc = argus_hip_quant_requant(c->ctx, &r);
    }
    // the old streams are freed below: every kernel that reads them must have finished
    if (rc == ARGUS_HIP_OK) rc = argus_hip_synchronize(c->ctx, c->stream);
  }
  if (rc != ARGUS_HIP_OK) {
    if (nk) argus_hip_free(c->ctx, nk);
    if (nv) argus_hip_free(c->ctx, nv);
    return rc;
  }
  argus_hip_free(c->ctx, c->qk);
  argus_hip_free(c->ctx, c->qv);
  c->qk = nk;
  c->qv = nv;
  c->bits = target_bits;
  c->deq_tokens = 0;  // the F16 view is rebuilt from the new blocks
  return ARGUS_HIP_OK;
}

ARGUS_API const argus_hip_quant_cache_vtable *argus_hip_quant_cache_get_vtable(void) {
  static const argus_hip_quant_cache_vtable vt = {
      argus_hip_quant_cache_make,          argus_hip_quant_cache_current_pos,   argus_hip_quant_cache_capacity,
      argus_hip_quant_cache_current_bits,  argus_hip_quant_cache_update,        argus_hip_quant_cache_flush_if_full,
      argus_hip_quant_cache_assemble_view, argus_hip_quant_cache_get_raw_buffers, argus_hip_quant_cache_transition_bits,
      argus_hip_quant_cache_drop};
  return &vt;
}
