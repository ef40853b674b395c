// Host-side mirror of the engine interfaces the attention path goes through, written above the
// C ABI of include/argus_hip.h.  Same method names, argument meaning and error behaviour as the
// reference traits, so a test written against the reference reads the same here:
//   HipBackend             ~ `trait Backend`            engine/src/backend.rs:127-1360 (hot-path subset)
//   HipQuantAttnBackend    ~ `CudaQuantAttnBackend`     crates/argus-extension-api/src/lib.rs:3087-3104
//   HipScoreReduceBackend  ~ `CudaScoreReduceBackend`   crates/argus-extension-api/src/lib.rs:2938-2948
//   HipGpuScoreAccumulator ~ `CudaGpuScoreAccumulator`  engine/src/backend/cuda_pc/gpu_score.rs:72-403
// `Result<T>` stands in for anyhow::Result<T>: ok() / value() / error().
// Everything runs on the single inference thread and the single in-order stream (null = default),
// like the reference backends.  Header-only; links against libargus_hip.so.
#pragma once

#include <algorithm>
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <limits>
#include <memory>
#include <string>
#include <utility>
#include <vector>

#include "../../include/argus_hip.h"

namespace argus {

template <typename T>
class Result {
 public:
  static Result Ok(T v) { Result r; r.ok_ = true; r.value_ = std::move(v); return r; }
  static Result Err(std::string msg) { Result r; r.ok_ = false; r.error_ = std::move(msg); return r; }
  bool ok() const { return ok_; }
  const T &value() const { return value_; }
  T &value() { return value_; }
  const std::string &error() const { return error_; }

 private:
  bool ok_ = false;
  T value_{};
  std::string error_;
};
struct Unit {};
using Status = Result<Unit>;
inline Status OkStatus() { return Status::Ok(Unit{}); }

// DType subset of engine/src/buffer.rs:25-47.
enum class DType { F32 = ARGUS_HIP_F32, F16 = ARGUS_HIP_F16, Q4_0 = ARGUS_HIP_Q4_0 };

// A tensor is a shape over a lent buffer (engine/src/tensor.rs:8-58); `device` tells whether the
// pointer is a device pointer of this backend (a `Buffer` of another backend has none).
struct Tensor {
  void *ptr = nullptr;
  DType dtype = DType::F32;
  std::vector<size_t> dims;
  bool device = true;
};

class HipGpuScoreAccumulator;

class HipBackend {
 public:
  // Counterpart of the "hip" arm of engine/src/session/init.rs:203-468.
  // `max_*`: the largest attention call the session will issue (the engine knows them from the model
  // config and --max-seq-len, and pre-allocates its own buffers from the same numbers,
  // crates/argus-extension-api/src/lib.rs:1903-1907); the split-KV workspace is sized once from
  // them so that no call allocates.
  static Result<std::shared_ptr<HipBackend>> create(int device = 0, int max_batch = 0, int max_heads_q = 0, int max_head_dim = 0,
                                                    int max_seq_len = 0) {
    argus_hip_ctx *ctx = nullptr;
    const argus_hip_create_opts opts = {max_batch, max_heads_q, max_head_dim, max_seq_len};
    const int rc = argus_hip_create_ex(device, &opts, &ctx);
    if (rc != ARGUS_HIP_OK) return Result<std::shared_ptr<HipBackend>>::Err("argus_hip_create failed: code " + std::to_string(rc));
    return Result<std::shared_ptr<HipBackend>>::Ok(std::shared_ptr<HipBackend>(new HipBackend(ctx)));
  }
  ~HipBackend();
  HipBackend(const HipBackend &) = delete;
  HipBackend &operator=(const HipBackend &) = delete;

  const char *name() const { return "HIP"; }
  bool is_gpu() const { return true; }
  bool is_discrete_gpu() const { return true; }
  bool is_nosub_device() const { return true; }
  bool supports_kv_scatter_batch() const { return true; }
  argus_hip_ctx *ctx() const { return ctx_; }

  // ---- memory (Backend::{read_buffer, write_buffer, write_buffer_range, copy_slice, buffer_shift,
  //      synchronize}, engine/src/backend.rs:610, 710, 736, 1085, 1119, 762) ---------------------
  Result<void *> alloc(size_t bytes) {
    void *p = nullptr;
    if (argus_hip_malloc(ctx_, bytes, &p) != ARGUS_HIP_OK) return Result<void *>::Err(last_error());
    return Result<void *>::Ok(p);
  }
  Status free(void *p) { return wrap(argus_hip_free(ctx_, p)); }
  Status write_buffer(void *dst_dev, const void *src_host, size_t bytes) { return wrap(argus_hip_write_buffer(ctx_, nullptr, dst_dev, src_host, bytes)); }
  Status read_buffer(void *dst_host, const void *src_dev, size_t bytes) { return wrap(argus_hip_read_buffer(ctx_, nullptr, dst_host, src_dev, bytes)); }
  Status copy_slice(void *dst_dev, const void *src_dev, size_t bytes) { return wrap(argus_hip_copy_slice(ctx_, nullptr, dst_dev, src_dev, bytes)); }
  // Backend::write_buffer_range(t, src, dst_offset): bounds-checked like the trait default
  // (engine/src/backend.rs:736-757).
  Status write_buffer_range(void *dst_dev, size_t dst_size, const void *src_host, size_t bytes, size_t dst_offset) {
    if (dst_offset + bytes < dst_offset) return Status::Err("write_buffer_range: offset+len overflow");
    if (dst_offset + bytes > dst_size)
      return Status::Err("write_buffer_range: out of bounds (" + std::to_string(dst_offset) + " + " + std::to_string(bytes) + " > " +
                         std::to_string(dst_size) + ")");
    return wrap(argus_hip_write_buffer_range(ctx_, nullptr, dst_dev, dst_offset, src_host, bytes));
  }
  // Backend::buffer_shift(tensor, src_offset, dst_offset, count): offsets and count in elements of
  // the tensor's dtype, overlap-safe like memmove (engine/src/backend.rs:1082-1112).
  Status buffer_shift(Tensor &t, size_t src_offset, size_t dst_offset, size_t count) {
    if (!t.ptr) return Status::Err("Null pointer in buffer_shift");
    const size_t ts = t.dtype == DType::F32 ? 4 : t.dtype == DType::F16 ? 2 : t.dtype == DType::Q4_0 ? 18 : 1;
    return wrap(argus_hip_buffer_shift(ctx_, nullptr, (char *)t.ptr + dst_offset * ts, (const char *)t.ptr + src_offset * ts, count * ts));
  }
  Status synchronize() { return wrap(argus_hip_synchronize(ctx_, nullptr)); }

  // ---- Backend::attention_gen (engine/src/backend.rs:284-295) ---------------------------------
  // `scores_out` is a HOST slice of `scores_len` floats or null; stride = scores_len / num_heads_q;
  // on return the slice is valid (explicit synchronize + copy-back, cuda_pc.rs:1861-1880).  When the
  // GPU score accumulator is active its per-layer device slice takes precedence and nothing is
  // copied back (cuda_pc.rs:1750-1766).  A malformed slice (stride < cache_seq_len) disables the
  // export instead of failing (cuda_pc.rs:1776-1779).
  Status attention_gen(const Tensor &q, const Tensor &k_cache, const Tensor &v_cache, Tensor &out,
                       size_t num_heads_q, size_t num_heads_kv, size_t head_dim, size_t cache_seq_len,
                       float *scores_out, size_t scores_len) {
    return attention_gen_indexed(q, k_cache, v_cache, out, num_heads_q, num_heads_kv, head_dim, cache_seq_len, nullptr, scores_out, scores_len);
  }

  // ---- SelectiveRead::attention_into_selected (engine/src/kv/standard_format.rs:2043-2184) ------
  // Attention over the selected cache positions only, the softmax normalised over that subset.
  // `page_size` 0 = ReadGranularity::Token (select holds positions), else ::Page (select holds page
  // indices, expanded by page_indices_to_positions, standard_format.rs:1924-1938, clamped to
  // current_pos).  An empty cache or selection zeroes `out`.  The reference gathers the rows on the
  // host (for a device cache: snapshot, CPU attention, upload); here the positions go to the device
  // as an index list and the decode kernel reads the rows in place.  scores_out[h * stride + i] is
  // the weight of the i-th selected position.
  Status attention_into_selected(const Tensor &q, const Tensor &k_cache, const Tensor &v_cache, Tensor &out, size_t num_heads_q,
                                 size_t num_heads_kv, size_t head_dim, size_t current_pos, const std::vector<size_t> &select,
                                 size_t page_size, float *scores_out, size_t scores_len) {
    std::vector<int32_t> positions;
    if (current_pos != 0) {
      if (page_size == 0) {
        positions.assign(select.begin(), select.end());
      } else {
        for (size_t pi : select)
          for (size_t pos = pi * page_size, end = std::min(pi * page_size + page_size, current_pos); pos < end; ++pos) positions.push_back((int32_t)pos);
      }
    }
    if (positions.empty()) {
      const std::vector<float> zeros(num_heads_q * head_dim, 0.0f);
      return write_buffer(out.ptr, zeros.data(), zeros.size() * sizeof(float));
    }
    const std::vector<size_t> &kd = k_cache.dims;
    const bool head_major = kd.size() >= 3 && kd[1] == num_heads_kv && kd[1] != kd[2];
    const size_t slots = kd.size() >= 3 ? (head_major ? kd[2] : kd[1]) : 0;
    for (int32_t pos : positions)
      if (pos < 0 || (size_t)pos >= slots) return Status::Err("attention_into_selected: position " + std::to_string(pos) + " outside the cache (" + std::to_string(slots) + " slots)");
    const size_t need = positions.size() * sizeof(int32_t);
    if (need > index_tmp_bytes_) {
      if (index_tmp_) argus_hip_free(ctx_, index_tmp_);
      index_tmp_ = nullptr;
      index_tmp_bytes_ = 0;
      if (argus_hip_malloc(ctx_, need, &index_tmp_) != ARGUS_HIP_OK) return Status::Err("index list: " + last_error());
      index_tmp_bytes_ = need;
    }
    Status st = write_buffer(index_tmp_, positions.data(), need);
    if (!st.ok()) return st;
    return attention_gen_indexed(q, k_cache, v_cache, out, num_heads_q, num_heads_kv, head_dim, positions.size(), (const int32_t *)index_tmp_, scores_out,
                                 scores_len);
  }

  // ---- attention over an opaque --kv-format cache ----------------------------------------------
  // What StandardFormat::attention_into does in its opaque arm (engine/src/kv/standard_format.rs:
  // 538-643): the cache rows are blocks of the format plugin's KVLayoutDesc.  Ok(true): attended on
  // the device without a decoded copy.  Ok(false): the descriptor is outside what the kernels decode
  // -- the caller takes the floor (decode_via_descriptor, then attention_gen on the F32 copy), as it
  // does for every backend today.  `capacity`: rows per KV head of the HeadMajor cache.
  Result<bool> attention_gen_opaque(const Tensor &q, const Tensor &k_cache, const Tensor &v_cache, Tensor &out, const argus_hip_kv_layout_desc &desc,
                                    size_t num_heads_q, size_t num_heads_kv, size_t head_dim, size_t cache_seq_len, size_t capacity) {
    if (!q.device || !k_cache.device || !v_cache.device || !out.device) return Result<bool>::Ok(false);
    argus_hip_attention_gen_args a{};
    a.q = (const float *)q.ptr; a.k_cache = k_cache.ptr; a.v_cache = v_cache.ptr; a.out = (float *)out.ptr;
    a.num_heads_q = (int32_t)num_heads_q; a.num_heads_kv = (int32_t)num_heads_kv; a.head_dim = (int32_t)head_dim;
    a.cache_seq_len = (int32_t)cache_seq_len; a.capacity = (int32_t)capacity; a.layout = ARGUS_HIP_HEAD_MAJOR; a.batch = 1;
    const int rc = argus_hip_attention_gen_desc(ctx_, &a, &desc);
    if (rc == ARGUS_HIP_ERR_UNSUPPORTED) return Result<bool>::Ok(false);
    if (rc != ARGUS_HIP_OK) return Result<bool>::Err("attention_gen_desc failed: " + last_error());
    return Result<bool>::Ok(true);
  }

  // ---- Backend::flash_attention_prefill (engine/src/backend.rs:1011-1027) --------------------
  // Ok(true) = dispatched, Ok(false) = not handled, caller uses its CPU path.
  Result<bool> flash_attention_prefill(const Tensor &q, const Tensor &k_cache, const Tensor &v_cache, Tensor &out,
                                       size_t n_heads_q, size_t n_heads_kv, size_t seq_len, size_t cache_seq_len,
                                       size_t head_dim, size_t kv_capacity, size_t batch_size, bool is_head_major) {
    if (!q.device || !k_cache.device || !v_cache.device || !out.device) return Result<bool>::Ok(false);
    if (k_cache.dtype == DType::Q4_0) return Result<bool>::Ok(false);
    argus_hip_prefill_args a{};
    a.q = q.ptr; a.k_cache = k_cache.ptr; a.v_cache = v_cache.ptr; a.out = out.ptr;
    a.n_heads_q = (int32_t)n_heads_q; a.n_heads_kv = (int32_t)n_heads_kv; a.seq_len = (int32_t)seq_len;
    a.cache_seq_len = (int32_t)cache_seq_len; a.head_dim = (int32_t)head_dim; a.kv_capacity = (int32_t)kv_capacity;
    a.batch_size = (int32_t)batch_size; a.is_head_major = is_head_major ? 1 : 0;
    a.q_dtype = (int32_t)q.dtype; a.kv_dtype = (int32_t)k_cache.dtype; a.out_dtype = (int32_t)out.dtype;
    const int rc = argus_hip_flash_attention_prefill(ctx_, &a);
    if (rc < 0) return Result<bool>::Err("flash_attn_prefill launch failed: " + last_error());
    return Result<bool>::Ok(rc == 1);
  }

  // ---- PFA side channel (prefill_attention_scores, engine/src/kv/standard_format.rs:1400-1510) ----
  // Same argument order as the host mirror; q and k are device tensors, sum_out / per_row device F32
  // buffers (nullptr = not armed).  has_window mirrors Option<usize>.
  Status prefill_attention_scores(const Tensor &q, const Tensor &k, size_t n_heads_q, size_t n_heads_kv, size_t head_dim,
                                  size_t seq_len, size_t cache_seq_len, size_t k_pos_stride, size_t kv_head_stride,
                                  size_t q_start_pos, size_t q_window, bool has_window, size_t window, float *sum_out,
                                  float *per_row_out, bool per_row_per_head) {
    argus_hip_pfa_args a{};
    a.q = q.ptr; a.k = k.ptr; a.k_dtype = (int32_t)k.dtype;
    a.n_heads_q = (int32_t)n_heads_q; a.n_heads_kv = (int32_t)n_heads_kv; a.head_dim = (int32_t)head_dim;
    a.seq_len = (int32_t)seq_len; a.cache_seq_len = (int32_t)cache_seq_len;
    a.k_pos_stride = (int64_t)k_pos_stride; a.kv_head_stride = (int64_t)kv_head_stride;
    a.q_start_pos = (int32_t)q_start_pos; a.q_window = (int32_t)q_window;
    a.has_window = has_window ? 1 : 0; a.window = (int32_t)window;
    a.sum_out = sum_out; a.per_row_out = per_row_out; a.per_row_per_head = per_row_per_head ? 1 : 0;
    return wrap(argus_hip_prefill_attention_scores(ctx_, &a));
  }

  // ---- Backend::kv_scatter_f32_to_f16 / _batch (engine/src/backend.rs:425-545) ----------------
  Status kv_scatter_f32_to_f16(const Tensor &k_src, const Tensor &v_src, Tensor &k_dst, Tensor &v_dst,
                               size_t head_dim, size_t capacity, size_t write_pos) {
    const size_t kv_heads = k_dst.dims.size() >= 3 ? k_dst.dims[k_dst.dims.size() - 3] : 0;
    return wrap(argus_hip_kv_scatter_f32_to_f16(ctx_, nullptr, (const float *)k_src.ptr, (const float *)v_src.ptr, k_dst.ptr,
                                                v_dst.ptr, (int32_t)kv_heads, (int32_t)head_dim, (int32_t)capacity, (int32_t)write_pos));
  }
  Status kv_scatter_f32_to_f16_batch(const Tensor &k_src, const Tensor &v_src, Tensor &k_dst, Tensor &v_dst,
                                     size_t kv_heads, size_t head_dim, size_t capacity, size_t write_pos_start, size_t seq_len) {
    if (k_dst.dtype == DType::F32)
      return wrap(argus_hip_kv_scatter_f32_batch(ctx_, nullptr, (const float *)k_src.ptr, (const float *)v_src.ptr, (float *)k_dst.ptr,
                                                 (float *)v_dst.ptr, (int32_t)kv_heads, (int32_t)head_dim, (int32_t)capacity,
                                                 (int32_t)write_pos_start, (int32_t)seq_len));
    return wrap(argus_hip_kv_scatter_f32_to_f16_batch(ctx_, nullptr, (const float *)k_src.ptr, (const float *)v_src.ptr, k_dst.ptr,
                                                      v_dst.ptr, (int32_t)kv_heads, (int32_t)head_dim, (int32_t)capacity,
                                                      (int32_t)write_pos_start, (int32_t)seq_len));
  }

  // ---- GPU score accumulator (Backend::gpu_score_acc[_mut], engine/src/backend.rs:1312-1322) --
  Status init_gpu_score_acc(size_t n_layers, size_t n_heads_q, size_t n_kv_heads, size_t max_seq_len, float decay);
  HipGpuScoreAccumulator *gpu_score_acc() { return acc_.get(); }

  std::string last_error() const { return argus_hip_last_error(ctx_); }
  Status wrap(int rc) const { return rc == ARGUS_HIP_OK ? OkStatus() : Status::Err(last_error() + " (code " + std::to_string(rc) + ")"); }

 private:
  explicit HipBackend(argus_hip_ctx *ctx) : ctx_(ctx) {}
  argus_hip_ctx *ctx_;
  Status attention_gen_indexed(const Tensor &q, const Tensor &k_cache, const Tensor &v_cache, Tensor &out, size_t num_heads_q, size_t num_heads_kv,
                               size_t head_dim, size_t cache_seq_len, const int32_t *kv_index_dev, float *scores_out, size_t scores_len);
  void *score_tmp_ = nullptr;  // reusable device score scratch (cuda_pc.rs `score_tmp_buf`)
  size_t score_tmp_bytes_ = 0;
  void *index_tmp_ = nullptr;  // reusable device index list of attention_into_selected
  size_t index_tmp_bytes_ = 0;
  std::unique_ptr<HipGpuScoreAccumulator> acc_;
};

// CudaScoreReduceBackend twin: the args struct is the reference POD field for field.
// The compaction executor of the KV container on device buffers: KVCache::shift_positions,
// shift_positions_for_head, compact_keep_positions and compact_keep_positions_for_head
// (engine/src/kv/kv_cache.rs:1002-1100, 1266-1350), which is what a committed keep-list turns into
// (engine/src/kv/cache_handle.rs:154-210).  Every move is Backend::buffer_shift, overlap-safe; the
// caller sets current_pos afterwards, as in the reference.  F16 / F32 caches of either layout; the
// per-head variants need HeadMajor.
struct HipKvCache {
  HipBackend *be = nullptr;
  Tensor k, v;  // HeadMajor [kv_heads, capacity, head_dim] or SeqMajor [capacity, kv_heads, head_dim]
  size_t kv_heads = 0, capacity = 0, head_dim = 0, current_pos = 0;
  bool head_major = true;

  Status shift_positions(size_t src_pos, size_t dst_pos, size_t count) {
    if (count == 0 || src_pos == dst_pos) return OkStatus();
    if (!head_major) {
      const size_t epp = kv_heads * head_dim;
      Status s = be->buffer_shift(k, src_pos * epp, dst_pos * epp, count * epp);
      return s.ok() ? be->buffer_shift(v, src_pos * epp, dst_pos * epp, count * epp) : s;
    }
    for (size_t h = 0; h < kv_heads; ++h) {
      Status s = shift_positions_for_head(h, src_pos, dst_pos, count);
      if (!s.ok()) return s;
    }
    return OkStatus();
  }
  Status shift_positions_for_head(size_t head, size_t src_pos, size_t dst_pos, size_t count) {
    if (!head_major) return Status::Err("shift_positions_for_head requires HeadMajor layout");
    if (count == 0 || src_pos == dst_pos) return OkStatus();
    const size_t base = head * capacity * head_dim;
    Status s = be->buffer_shift(k, base + src_pos * head_dim, base + dst_pos * head_dim, count * head_dim);
    return s.ok() ? be->buffer_shift(v, base + src_pos * head_dim, base + dst_pos * head_dim, count * head_dim) : s;
  }
  // `keep` ascending.  Consecutive source positions merge into one shift; a run already in place
  // is skipped.  head < 0: every head.
  Status compact_keep(const std::vector<size_t> &keep, size_t write_start, long head) {
    if (keep.empty()) return OkStatus();
    auto flush = [&](size_t src, size_t dst, size_t count) {
      if (src == dst) return OkStatus();
      return head < 0 ? shift_positions(src, dst, count) : shift_positions_for_head((size_t)head, src, dst, count);
    };
    size_t write_pos = write_start, src0 = keep[0], dst0 = write_pos, count = 1;
    ++write_pos;
    for (size_t i = 1; i < keep.size(); ++i) {
      if (keep[i] == src0 + count) {
        ++count;
      } else {
        Status s = flush(src0, dst0, count);
        if (!s.ok()) return s;
        src0 = keep[i];
        dst0 = write_pos;
        count = 1;
      }
      ++write_pos;
    }
    return flush(src0, dst0, count);
  }
  Status compact_keep_positions(const std::vector<size_t> &keep, size_t write_start) { return compact_keep(keep, write_start, -1); }
  Status compact_keep_positions_for_head(size_t head, const std::vector<size_t> &keep, size_t write_start) {
    return compact_keep(keep, write_start, (long)head);
  }
};

class HipScoreReduceBackend {
 public:
  explicit HipScoreReduceBackend(argus_hip_ctx *ctx) : ctx_(ctx) {}
  const char *name() const { return "attn_score"; }
  int reduce(const argus_hip_score_reduce_args &a) const { return ctx_ ? argus_hip_score_reduce(ctx_, &a) : -1; }
  int reduce_per_layer(const argus_hip_score_reduce_args &a) const { return ctx_ ? argus_hip_score_reduce_per_layer(ctx_, &a) : -1; }
  // score buffers in the logits + (max, sum) form
  int reduce_ex(const argus_hip_score_reduce_args &a, const argus_hip_score_reduce_ext &e) const { return ctx_ ? argus_hip_score_reduce_ex(ctx_, &a, &e) : -1; }
  int reduce_per_layer_ex(const argus_hip_score_reduce_args &a, const argus_hip_score_reduce_ext &e) const { return ctx_ ? argus_hip_score_reduce_per_layer_ex(ctx_, &a, &e) : -1; }

 private:
  argus_hip_ctx *ctx_;
};

// CudaQuantAttnBackend twin.  A handle built without a context is *degraded*: every op returns -1
// without crashing (engine/tests/gate_c_kivi_backend_cap.rs:90-146).
class HipQuantAttnBackend {
 public:
  explicit HipQuantAttnBackend(argus_hip_ctx *ctx) : ctx_(ctx) {}
  bool has_quant_attn_kernel(uint8_t bits) const { return ctx_ && argus_hip_has_quant_attn_kernel(ctx_, bits) == 1; }
  bool is_nosub_device() const { return true; }
  int attention_gen_quant(const argus_hip_quant_attn_args &a) const { return ctx_ ? argus_hip_attention_gen_quant(ctx_, &a) : -1; }
  int gather_update_quant(const argus_hip_quant_gather_args &a) const { return ctx_ ? argus_hip_gather_update_quant(ctx_, &a) : -1; }
  // F16-view helpers (lib.rs:3096-3103): negative on failure like the reference (-1 .. -4).
  int dequant_flush(const argus_hip_quant_dequant_flush_args &a) const { return ctx_ ? argus_hip_quant_dequant_flush(ctx_, &a) : -1; }
  int scatter_residual(const argus_hip_quant_scatter_residual_args &a) const { return ctx_ ? argus_hip_quant_scatter_residual(ctx_, &a) : -1; }

 private:
  argus_hip_ctx *ctx_;
};

// QuantWindowRawBuffers (engine/src/kv/kv_cache_ops.rs:39-56): what the fused kernel is handed.
struct QuantWindowRawBuffers {
  void *qk_buf, *qv_buf, *res_k, *res_v;
  size_t q_tokens, res_tokens, res_cap;
  uint8_t bits;
};

// The GPU mode of QuantizedRecentWindowCache (engine/src/kv/quant_window_cache.rs:380-586 new_gpu,
// 2518-2562 update, 1688-1848 flush_residual_gpu, 741-760 get_raw_gpu_buffers, 2248-2475
// get_view_gpu, 973-1448 transition_bits, 810-843 reset) for one layer, over the library's
// CACHE-category handle (argus_hip_quant_cache_*, the C form of QuantCacheBackend,
// crates/argus-extension-api/src/lib.rs:2017-2035): an F32 residual ring that new tokens are
// appended to and the two block streams it is quantised into when full, every step on the device.
// bits = 16 is the unquantised mode (residual of max_seq_len rows, which is also the view) with the
// transitions to and from the quantised widths.  Flush metrics (QCF / AWQE proxies) are host
// bookkeeping of the reference with no device part and are not mirrored.
class HipQuantWindowCache {
 public:
  static Result<std::unique_ptr<HipQuantWindowCache>> new_gpu(HipBackend *be, size_t kv_heads, size_t head_dim, size_t max_seq_len,
                                                              size_t residual_size, uint8_t bits) {
    using R = Result<std::unique_ptr<HipQuantWindowCache>>;
    if (!be) return R::Err("quant-window GPU mode needs a backend");
    argus_hip_quant_cache_make_args a{};
    a.ctx = be->ctx(); a.kv_heads = kv_heads; a.head_dim = head_dim; a.max_seq_len = max_seq_len; a.residual_size = residual_size; a.bits = bits;
    void *h = argus_hip_quant_cache_make(&a);
    if (!h) return R::Err("quant-window cache: " + be->last_error());
    std::unique_ptr<HipQuantWindowCache> c(new HipQuantWindowCache());
    c->be_ = be; c->h_ = h; c->kv_heads_ = kv_heads; c->head_dim_ = head_dim; c->max_seq_len_ = max_seq_len; c->res_cap_ = residual_size;
    return R::Ok(std::move(c));
  }
  ~HipQuantWindowCache() { argus_hip_quant_cache_drop(h_); }
  HipQuantWindowCache(const HipQuantWindowCache &) = delete;
  HipQuantWindowCache &operator=(const HipQuantWindowCache &) = delete;

  bool is_gpu() const { return true; }
  uint8_t bits() const { return argus_hip_quant_cache_current_bits(h_); }
  size_t current_pos() const { return argus_hip_quant_cache_current_pos(h_); }
  size_t capacity() const { return argus_hip_quant_cache_capacity(h_); }
  size_t kv_heads() const { return kv_heads_; }
  size_t head_dim() const { return head_dim_; }

  // update(new_k, new_v): device F32 [1, seq_len, kv_heads, head_dim]; flushes whenever the ring is full.
  Status update(const Tensor &new_k, const Tensor &new_v) {
    if (new_k.dims.size() != 4 || new_k.dims != new_v.dims || new_k.dims[2] != kv_heads_ || new_k.dims[3] != head_dim_)
      return Status::Err("QuantWindowCache update: expected [1, seq_len, kv_heads, head_dim]");
    if (new_k.dtype != DType::F32 || new_v.dtype != DType::F32 || !new_k.device || !new_v.device)
      return Status::Err("QuantWindowCache update: device F32 tensors expected");
    argus_hip_quant_cache_update_args a{nullptr, new_k.ptr, new_v.ptr, new_k.dims[1]};
    return wrap(argus_hip_quant_cache_update(h_, &a));
  }
  Status flush_if_full() { return wrap(argus_hip_quant_cache_flush_if_full(h_)); }
  Status transition_bits(uint8_t new_bits) { return wrap(argus_hip_quant_cache_transition_bits(h_, new_bits)); }

  // None (ok() false) for an empty cache, like the reference for a cache with no native set.
  Result<QuantWindowRawBuffers> get_raw_gpu_buffers() const {
    argus_hip_quant_cache_raw_buffers_out o{};
    if (!argus_hip_quant_cache_get_raw_buffers(h_, &o)) return Result<QuantWindowRawBuffers>::Err("no raw buffers");
    return Result<QuantWindowRawBuffers>::Ok(QuantWindowRawBuffers{o.qk_mem, o.qv_mem, o.res_k_mem, o.res_v_mem, o.q_tokens, o.res_tokens, o.res_cap, o.bits});
  }

  // QuantWindowFormat::attention_native (engine/src/kv/quant_window_format.rs:258-330): fused
  // dequant + attention over the raw buffers; `scores` (host, [n_heads_q, current_pos]) optional.
  Status attention_native(const Tensor &q, Tensor &out, size_t n_heads_q, float *scores, size_t scores_len) const {
    auto got = get_raw_gpu_buffers();
    if (!got.ok()) return Status::Err("attention_native: empty cache");
    const QuantWindowRawBuffers &raw = got.value();
    HipQuantAttnBackend cap(be_->ctx());
    if (!cap.has_quant_attn_kernel(raw.bits)) return Status::Err("no fused kernel for these bits");
    argus_hip_quant_attn_args a{};
    a.q_mem = (uint64_t)q.ptr; a.qk_mem = (uint64_t)raw.qk_buf; a.qv_mem = (uint64_t)raw.qv_buf;
    a.res_k_mem = (uint64_t)raw.res_k; a.res_v_mem = (uint64_t)raw.res_v; a.out_mem = (uint64_t)out.ptr;
    a.scores_out = scores; a.scores_len = scores ? scores_len : 0;
    a.num_heads_q = n_heads_q; a.num_heads_kv = kv_heads_; a.head_dim = head_dim_;
    a.q_tokens = raw.q_tokens; a.res_tokens = raw.res_tokens; a.res_cap = raw.res_cap;
    a.scale = 1.0f / std::sqrt((float)head_dim_); a.bits = raw.bits;
    const int rc = cap.attention_gen_quant(a);
    return rc == 0 ? OkStatus() : Status::Err("attention_gen_quant failed (rc=" + std::to_string(rc) + "): " + be_->last_error());
  }

  // get_view_gpu: F16 [max_seq_len, kv_heads, head_dim] views covering [0, current_pos); while bits = 16
  // the F32 residual itself, [1, kv_heads, max_seq_len, head_dim] (quant_window_cache.rs:2417-2429).
  Result<std::pair<Tensor, Tensor>> get_view_gpu() {
    using R = Result<std::pair<Tensor, Tensor>>;
    argus_hip_quant_cache_view_out o{};
    const int rc = argus_hip_quant_cache_assemble_view(h_, &o);
    if (rc != 0) return R::Err("assemble_view failed (rc=" + std::to_string(rc) + "): " + be_->last_error());
    const bool residual = o.layout == ARGUS_HIP_VIEW_HEADS_TOKENS_DIM;
    Tensor tk{o.k_mem, residual ? DType::F32 : DType::F16,
              residual ? std::vector<size_t>{1, kv_heads_, max_seq_len_, head_dim_} : std::vector<size_t>{1, max_seq_len_, kv_heads_, head_dim_}, true};
    Tensor tv = tk;
    tv.ptr = o.v_mem;
    return R::Ok(std::make_pair(tk, tv));
  }

  // reset(): a fresh handle of the same geometry and width (the reference keeps its buffers and
  // zeroes its counters; the vtable has no such call)
  Status reset() {
    argus_hip_quant_cache_make_args a{};
    a.ctx = be_->ctx(); a.kv_heads = kv_heads_; a.head_dim = head_dim_; a.max_seq_len = max_seq_len_; a.residual_size = res_cap_; a.bits = bits();
    void *h = argus_hip_quant_cache_make(&a);
    if (!h) return Status::Err("quant-window cache: " + be_->last_error());
    argus_hip_quant_cache_drop(h_);
    h_ = h;
    return OkStatus();
  }

 private:
  HipQuantWindowCache() = default;
  Status wrap(int rc) const { return rc == 0 ? OkStatus() : Status::Err(be_->last_error() + " (code " + std::to_string(rc) + ")"); }
  HipBackend *be_ = nullptr;
  void *h_ = nullptr;
  size_t kv_heads_ = 0, head_dim_ = 0, max_seq_len_ = 0, res_cap_ = 0;
};

// CudaGpuScoreAccumulator twin (engine/src/backend/cuda_pc/gpu_score.rs:72-403): persistent device
// buffers [n_layers, n_heads_q, max_seq_len] scores + cumulative flat / per-head importance; the
// attention kernel writes each layer's slice, end_step() folds them with the fused reducer.
// The slices are kept in the library's logits + (max, sum) form (argus_hip_attention_gen_args::
// score_stats, a [n_layers, n_heads_q, 2] buffer beside the scores): the reducer normalises while it
// reads, with the arithmetic the attention call would have used to rewrite the rows, so the cumulative
// buffers come out bit for bit as from probabilities, and no layer's row is read twice.
class HipGpuScoreAccumulator {
 public:
  static Result<std::unique_ptr<HipGpuScoreAccumulator>> create(HipBackend *be, size_t n_layers, size_t n_heads_q,
                                                                size_t n_kv_heads, size_t max_seq_len, float decay) {
    using R = Result<std::unique_ptr<HipGpuScoreAccumulator>>;
    if (n_kv_heads > 16) return R::Err("n_kv_heads exceeds the fused kernel limit of 16");
    std::unique_ptr<HipGpuScoreAccumulator> a(new HipGpuScoreAccumulator(be));
    a->n_layers_ = n_layers; a->n_heads_q_ = n_heads_q; a->n_kv_heads_ = n_kv_heads;
    a->max_seq_len_ = max_seq_len; a->score_stride_ = max_seq_len;
    const float f = 1.0f - decay;
    a->decay_factor_ = f < 0.0f ? 0.0f : (f > 1.0f ? 1.0f : f);
    auto alloc_zeroed = [&](size_t elems, void **out) -> bool {
      auto r = be->alloc(elems * sizeof(float));
      if (!r.ok()) return false;
      *out = r.value();
      std::vector<float> z(elems, 0.0f);
      return be->write_buffer(*out, z.data(), elems * sizeof(float)).ok();
    };
    if (!alloc_zeroed(n_layers * n_heads_q * max_seq_len, &a->score_buf_) || !alloc_zeroed(max_seq_len, &a->importance_) ||
        !alloc_zeroed(n_kv_heads * max_seq_len, &a->head_importance_) || !alloc_zeroed(n_layers * max_seq_len, &a->layer_flat_))
      return R::Err("score buffer allocation failed: " + be->last_error());
    // (max, sum) = (+inf, 1): a layer no call has written yet reads as all-zero probabilities
    std::vector<float> st(n_layers * n_heads_q * 2);
    for (size_t i = 0; i < st.size(); i += 2) { st[i] = std::numeric_limits<float>::infinity(); st[i + 1] = 1.0f; }
    auto r = be->alloc(st.size() * sizeof(float));
    if (!r.ok()) return R::Err("score statistics allocation failed: " + be->last_error());
    a->stats_ = r.value();
    if (!be->write_buffer(a->stats_, st.data(), st.size() * sizeof(float)).ok()) return R::Err(be->last_error());
    return R::Ok(std::move(a));
  }
  ~HipGpuScoreAccumulator() {
    for (void *p : {score_buf_, importance_, head_importance_, layer_flat_, stats_})
      if (p) be_->free(p);
  }

  uint64_t score_buf_device_ptr() const { return (uint64_t)score_buf_; }
  // statistics rows of a layer's heads, or null while the buffer holds probabilities (debug fill)
  float *layer_stats_ptr(size_t layer_idx) const { return logits_form_ ? (float *)stats_ + layer_idx * n_heads_q_ * 2 : nullptr; }
  size_t score_stride() const { return score_stride_; }
  size_t layer_offset_elems(size_t layer_idx) const { return layer_idx * n_heads_q_ * score_stride_; }
  size_t current_layer_idx() const { return current_layer_idx_; }
  void set_current_layer_idx(size_t i) { current_layer_idx_ = i; }
  bool is_active() const { return active_; }
  void set_active(bool a) { active_ = a; }
  void enable_per_layer_flat() { per_layer_flat_ = true; }
  size_t steps_accumulated() const { return steps_; }

  Status end_step(void *stream, size_t cache_seq_len) {
    if (!active_ || cache_seq_len == 0) return OkStatus();
    argus_hip_score_reduce_args a{};
    a.stream = stream;
    a.score_buf = (uint64_t)score_buf_; a.importance = (uint64_t)importance_; a.head_importance = (uint64_t)head_importance_;
    a.decay_factor = decay_factor_; a.n_layers = n_layers_; a.n_heads_q = n_heads_q_; a.n_kv_heads = n_kv_heads_;
    a.cache_seq_len = cache_seq_len; a.score_stride = score_stride_; a.max_seq_len = max_seq_len_;
    a.layer_flat_importance = (uint64_t)layer_flat_;
    HipScoreReduceBackend reducer(be_->ctx());
    argus_hip_score_reduce_ext ext{};
    ext.stats = logits_form_ ? (uint64_t)stats_ : 0;
    int ret = reducer.reduce_ex(a, ext);
    if (ret != 0) return Status::Err("attn_score HIP reduce failed: code " + std::to_string(ret));
    if (per_layer_flat_) {
      ret = reducer.reduce_per_layer_ex(a, ext);
      if (ret != 0) return Status::Err("attn_score HIP per-layer reduce failed: code " + std::to_string(ret));
    }
    steps_ += 1;
    current_layer_idx_ = 0;
    return OkStatus();
  }

  // seed_prefill_importance[_dual] (engine/src/inference/attention_scores.rs:249-322) without the
  // host fold: `pfa_dev` holds the per-layer column sums of prefill_attention_scores on the device,
  // [n_layers, n_heads_q, prefix_len] F32, and one synthetic step folds them into the cumulative
  // buffers exactly as the reference's accumulate_layer_gqa + end_step does on the host
  // (importance += layer-MAX of the head sums, head_importance += GQA average), with the PFA layout's
  // stride = cache_seq_len = prefix_len.  The reference folds on the CPU and uploads the result
  // through seed_cumulative, because its PFA runs on the host.
  Status seed_prefill_importance_device(void *stream, const void *pfa_dev, size_t prefix_len) {
    if (!active_ || prefix_len == 0 || n_heads_q_ == 0) return OkStatus();
    if (prefix_len > max_seq_len_) return Status::Err("seed_prefill_importance: prefix_len exceeds max_seq_len");
    argus_hip_score_reduce_args a{};
    a.stream = stream;
    a.score_buf = (uint64_t)pfa_dev; a.importance = (uint64_t)importance_; a.head_importance = (uint64_t)head_importance_;
    a.decay_factor = decay_factor_; a.n_layers = n_layers_; a.n_heads_q = n_heads_q_; a.n_kv_heads = n_kv_heads_;
    a.cache_seq_len = prefix_len; a.score_stride = prefix_len; a.max_seq_len = max_seq_len_;
    a.layer_flat_importance = (uint64_t)layer_flat_;
    HipScoreReduceBackend reducer(be_->ctx());
    int ret = reducer.reduce(a);
    if (ret != 0) return Status::Err("attn_score HIP prefill seed failed: code " + std::to_string(ret));
    if (per_layer_flat_) {
      ret = reducer.reduce_per_layer(a);
      if (ret != 0) return Status::Err("attn_score HIP per-layer prefill seed failed: code " + std::to_string(ret));
    }
    steps_ += 1;
    return OkStatus();
  }

  Result<std::pair<std::vector<float>, std::vector<float>>> sync_to_cpu() const {
    using R = Result<std::pair<std::vector<float>, std::vector<float>>>;
    std::vector<float> flat(max_seq_len_), head(n_kv_heads_ * max_seq_len_);
    if (!be_->read_buffer(flat.data(), importance_, flat.size() * 4).ok() ||
        !be_->read_buffer(head.data(), head_importance_, head.size() * 4).ok())
      return R::Err(be_->last_error());
    return R::Ok({std::move(flat), std::move(head)});
  }
  Result<std::vector<float>> sync_layer_flat_to_cpu() const {
    std::vector<float> lf(n_layers_ * max_seq_len_);
    if (!be_->read_buffer(lf.data(), layer_flat_, lf.size() * 4).ok()) return Result<std::vector<float>>::Err(be_->last_error());
    return Result<std::vector<float>>::Ok(std::move(lf));
  }
  Status seed_cumulative(const std::vector<float> &flat, const std::vector<float> &head) {
    if (flat.size() != max_seq_len_) return Status::Err("seed_cumulative: flat.len() != max_seq_len");
    if (head.size() != n_kv_heads_ * max_seq_len_) return Status::Err("seed_cumulative: head.len() != n_kv_heads*max_seq_len");
    Status s = be_->write_buffer(importance_, flat.data(), flat.size() * 4);
    if (!s.ok()) return s;
    return be_->write_buffer(head_importance_, head.data(), head.size() * 4);
  }
  // gpu_score.rs:340-363
  Status seed_layer_flat_cumulative(const std::vector<float> &layer_flat) {
    if (layer_flat.size() != n_layers_ * max_seq_len_)
      return Status::Err("seed_layer_flat_cumulative: layer_flat.len()=" + std::to_string(layer_flat.size()) + " != n_layers*max_seq_len=" +
                         std::to_string(n_layers_ * max_seq_len_));
    return be_->write_buffer(layer_flat_, layer_flat.data(), layer_flat.size() * 4);
  }
  Status reset_layer_flat() {
    const std::vector<float> z(n_layers_ * max_seq_len_, 0.0f);
    return be_->write_buffer(layer_flat_, z.data(), z.size() * 4);
  }
  Status reset() {
    std::vector<float> z(n_layers_ * max_seq_len_ > n_kv_heads_ * max_seq_len_ ? n_layers_ * max_seq_len_ : n_kv_heads_ * max_seq_len_, 0.0f);
    Status s = be_->write_buffer(importance_, z.data(), max_seq_len_ * 4);
    if (s.ok()) s = be_->write_buffer(head_importance_, z.data(), n_kv_heads_ * max_seq_len_ * 4);
    if (s.ok()) s = be_->write_buffer(layer_flat_, z.data(), n_layers_ * max_seq_len_ * 4);
    steps_ = 0;
    current_layer_idx_ = 0;
    return s;
  }
  // Test-only, like the reference's debug_fill_score_buf.
  Status debug_fill_score_buf(const std::vector<float> &scores) {
    if (scores.size() != n_layers_ * n_heads_q_ * score_stride_) return Status::Err("debug_fill_score_buf: wrong length");
    logits_form_ = false;  // the values given are probabilities
    return be_->write_buffer(score_buf_, scores.data(), scores.size() * 4);
  }

 private:
  explicit HipGpuScoreAccumulator(HipBackend *be) : be_(be) {}
  HipBackend *be_;
  void *score_buf_ = nullptr, *importance_ = nullptr, *head_importance_ = nullptr, *layer_flat_ = nullptr, *stats_ = nullptr;
  bool logits_form_ = true;
  size_t n_layers_ = 0, n_heads_q_ = 0, n_kv_heads_ = 0, max_seq_len_ = 0, score_stride_ = 0;
  float decay_factor_ = 1.0f;
  bool active_ = false, per_layer_flat_ = false;
  size_t steps_ = 0, current_layer_idx_ = 0;
};

inline HipBackend::~HipBackend() {
  acc_.reset();
  if (score_tmp_) argus_hip_free(ctx_, score_tmp_);
  if (index_tmp_) argus_hip_free(ctx_, index_tmp_);
  argus_hip_destroy(ctx_);
}

inline Status HipBackend::init_gpu_score_acc(size_t n_layers, size_t n_heads_q, size_t n_kv_heads, size_t max_seq_len, float decay) {
  auto r = HipGpuScoreAccumulator::create(this, n_layers, n_heads_q, n_kv_heads, max_seq_len, decay);
  if (!r.ok()) return Status::Err(r.error());
  acc_ = std::move(r.value());
  return OkStatus();
}

inline Status HipBackend::attention_gen_indexed(const Tensor &q, const Tensor &k_cache, const Tensor &v_cache, Tensor &out,
                                                size_t num_heads_q, size_t num_heads_kv, size_t head_dim, size_t cache_seq_len,
                                                const int32_t *kv_index_dev, float *scores_out, size_t scores_len) {
  // The reference falls back to its CPU companion for non-device buffers and Q4_0 KV
  // (cuda_pc.rs:1716-1729); this mirror has no CPU companion, so it reports the former.  Q4_0
  // caches are attended on the device (BlockQ4_0 rows, common.rs:676-850).
  if (!q.device || !k_cache.device || !v_cache.device || !out.device)
    return Status::Err("attention_gen: not a device call; route to the CPU companion");
  const std::vector<size_t> &kd = k_cache.dims;
  // Layout rule of x86.rs:195-198.
  const bool head_major = kd.size() >= 3 && kd[1] == num_heads_kv && kd[1] != kd[2];
  argus_hip_attention_gen_args a{};
  a.q = (const float *)q.ptr; a.k_cache = k_cache.ptr; a.v_cache = v_cache.ptr; a.out = (float *)out.ptr;
  a.num_heads_q = (int32_t)num_heads_q; a.num_heads_kv = (int32_t)num_heads_kv; a.head_dim = (int32_t)head_dim;
  a.cache_seq_len = (int32_t)cache_seq_len;
  a.capacity = head_major ? (int32_t)kd[2] : (kv_index_dev && kd.size() >= 3 ? (int32_t)kd[1] : 0);
  a.layout = head_major ? ARGUS_HIP_HEAD_MAJOR : ARGUS_HIP_SEQ_MAJOR;
  a.kv_dtype = (int32_t)k_cache.dtype;
  a.batch = 1;
  a.kv_index = kv_index_dev;

  size_t stride = 0;
  bool copy_back = false;
  if (acc_ && acc_->is_active()) {
    a.scores_out = (float *)acc_->score_buf_device_ptr() + acc_->layer_offset_elems(acc_->current_layer_idx());
    a.score_stride = (int32_t)acc_->score_stride();
    a.score_stats = acc_->layer_stats_ptr(acc_->current_layer_idx());
  } else if (scores_out && num_heads_q > 0) {
    stride = scores_len / num_heads_q;
    if (stride != 0 && stride >= cache_seq_len) {
      const size_t need = num_heads_q * stride * sizeof(float);
      if (need > score_tmp_bytes_) {
        if (score_tmp_) argus_hip_free(ctx_, score_tmp_);
        score_tmp_ = nullptr;
        score_tmp_bytes_ = 0;
        if (argus_hip_malloc(ctx_, need, &score_tmp_) != ARGUS_HIP_OK) return Status::Err("score buffer: " + last_error());
        score_tmp_bytes_ = need;
      }
      a.scores_out = (float *)score_tmp_;
      a.score_stride = (int32_t)stride;
      copy_back = true;
    }
  }
  const int rc = argus_hip_attention_gen(ctx_, &a);
  if (rc != ARGUS_HIP_OK) return Status::Err("attention_gen kernel launch failed: " + last_error());
  if (copy_back) {
    // The caller expects the slice to be valid on return: synchronising read-back of the rows.
    const size_t total = num_heads_q * stride;
    const size_t n = scores_len < total ? scores_len : total;
    Status s = read_buffer(scores_out, score_tmp_, n * sizeof(float));
    if (!s.ok()) return s;
  }
  return OkStatus();
}

}  // namespace argus
