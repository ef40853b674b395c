// Device tests of the C++ host mirror (argus-engine_amd/host/argus_hip_backend.hpp), written the way
// the reference's own device tests are: drive the backend through its trait-shaped methods and
// compare with a host computation.
//   * score accumulator flow      engine/src/bin/test_cuda_gpu_score_device.rs (cases 1-3)
//   * attention_gen unit shape    engine/src/backend/cpu/x86.rs:1811-1973 (LCG seeds 42/137/53)
//   * KIVI residual-only pattern  engine/src/bin/test_cuda_quant_attn_device.rs:108-178 (Test A)
//   * degraded capability handle  engine/tests/gate_c_kivi_backend_cap.rs:90-146
// The CPU oracle (test infrastructure) supplies the expected values.
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "../../argus-engine_amd/host/argus_hip_backend.hpp"

extern "C" {
void oracle_gen_data(float *dst, int64_t n, uint32_t seed);
void oracle_f32_to_f16(const float *src, uint16_t *dst, int64_t n);
int oracle_attention_gen_scalar(const float *q, const void *k, const void *v, float *out, int hq, int hkv, int d, int len,
                                int capacity, int head_major, int kv_dtype, float *scores, int64_t stride, float softcap,
                                const int32_t *kv_index);
int oracle_prefill_attention(const float *q, const void *k, const void *v, float *out, int hq, int hkv, int seq_len,
                             int cache_len, int d, int capacity, int batch, int kv_dtype, int window, int n_threads);
int oracle_score_fused_reduce(const float *scores, float *imp, float *himp, float decay_factor, int n_layers, int hq,
                              int hkv, int len, int64_t stride, int max_seq);
int oracle_decode_via_descriptor(int block_elems, int bits, int scale_layout, int packing, const uint8_t *src, float *dst,
                                 int64_t n_elems);
int oracle_encode_via_descriptor(int block_elems, int bits, int scale_layout, int packing, const float *src, uint8_t *dst,
                                 int64_t n_elems);
int oracle_kivi_build(const float *k_in, const float *v_in, int n_tokens, int kv_heads, int head_dim, int res_cap, int bits, uint8_t *qk,
                      uint8_t *qv, float *res_k, float *res_v, int *q_tokens_out, int *res_tokens_out);
int oracle_kivi_assemble_view(const uint8_t *qk, const uint8_t *qv, const float *res_k, const float *res_v, int q_tokens, int res_tokens,
                              int kv_heads, int head_dim, int res_cap, int bits, float *attn_k, float *attn_v);
int oracle_kivi_attention(const float *q, const uint8_t *qk, const uint8_t *qv, const float *res_k, const float *res_v, float *out,
                          float *scores, int64_t score_stride, int num_heads_q, int num_heads_kv, int head_dim, int q_tokens, int res_tokens,
                          int res_cap, float scale, int bits);
int oracle_prefill_attention_scores(const float *q, const float *k, int n_heads_q, int n_heads_kv, int head_dim, int seq_len, int cache_seq_len,
                                    int64_t k_pos_stride, int64_t kv_head_stride, int q_start_pos, int q_window, int window, float *sum_out,
                                    float *per_row_out, int per_row_per_head);
void oracle_kv_scatter(const float *k_src, const float *v_src, void *k_dst, void *v_dst, int kv_heads, int head_dim,
                       int capacity, int write_pos_start, int seq_len, int dst_f16);
}

using namespace argus;

static int g_fail = 0;
#define CHECK(cond, ...)                                       \
  do {                                                         \
    if (!(cond)) {                                             \
      printf("FAIL %s:%d: ", __FILE__, __LINE__);              \
      printf(__VA_ARGS__);                                     \
      printf("\n");                                            \
      ++g_fail;                                                \
    }                                                          \
  } while (0)

static float max_abs_diff(const std::vector<float> &a, const std::vector<float> &b) {
  float m = 0;
  for (size_t i = 0; i < a.size(); ++i) m = fmaxf(m, fabsf(a[i] - b[i]));
  return m;
}

struct DevBuf {
  HipBackend *be;
  void *p = nullptr;
  DevBuf(HipBackend *b, size_t bytes, const void *host = nullptr) : be(b) {
    p = be->alloc(bytes).value();
    if (host) be->write_buffer(p, host, bytes);
  }
  ~DevBuf() { be->free(p); }
};

static void test_score_accumulator(HipBackend &be) {
  const size_t n_layers = 2, hq = 2, hkv = 1, max_seq = 8, len = 3;
  CHECK(be.init_gpu_score_acc(n_layers, hq, hkv, max_seq, 0.0f).ok(), "init");
  be.gpu_score_acc()->set_active(true);
  std::vector<float> scores(n_layers * hq * max_seq, 0.0f);
  auto set = [&](size_t l, size_t h, float a, float b, float c) {
    float *p = &scores[l * hq * max_seq + h * max_seq];
    p[0] = a; p[1] = b; p[2] = c;
  };
  set(0, 0, 0.1f, 0.2f, 0.7f); set(0, 1, 0.3f, 0.3f, 0.4f); set(1, 0, 0.5f, 0.4f, 0.1f); set(1, 1, 0.2f, 0.2f, 0.6f);
  CHECK(be.gpu_score_acc()->debug_fill_score_buf(scores).ok(), "fill");
  CHECK(be.gpu_score_acc()->end_step(nullptr, len).ok(), "end_step");
  CHECK(be.synchronize().ok(), "sync");
  auto r = be.gpu_score_acc()->sync_to_cpu();
  CHECK(r.ok(), "sync_to_cpu");
  const float exp_flat[3] = {0.7f, 0.6f, 1.1f}, exp_head[3] = {0.35f, 0.30f, 0.55f};
  for (size_t t = 0; t < len; ++t) {
    CHECK(fabsf(r.value().first[t] - exp_flat[t]) < 1e-5f, "case1 flat[%zu]=%g", t, r.value().first[t]);
    CHECK(fabsf(r.value().second[t] - exp_head[t]) < 1e-5f, "case1 head[%zu]=%g", t, r.value().second[t]);
  }
  CHECK(be.gpu_score_acc()->steps_accumulated() == 1, "steps");
  // case 2: decay 0.5, two identical steps -> 1.5 x
  CHECK(be.init_gpu_score_acc(n_layers, hq, hkv, max_seq, 0.5f).ok(), "init2");
  be.gpu_score_acc()->set_active(true);
  be.gpu_score_acc()->debug_fill_score_buf(scores);
  be.gpu_score_acc()->end_step(nullptr, len);
  be.gpu_score_acc()->end_step(nullptr, len);
  be.synchronize();
  auto r2 = be.gpu_score_acc()->sync_to_cpu();
  for (size_t t = 0; t < len; ++t) CHECK(fabsf(r2.value().first[t] - 1.5f * exp_flat[t]) < 1e-5f, "case2 flat[%zu]", t);
  // case 3: seed round trip, then reset
  CHECK(be.init_gpu_score_acc(n_layers, hq, hkv, max_seq, 0.0f).ok(), "init3");
  std::vector<float> sf(max_seq), sh(hkv * max_seq);
  for (size_t i = 0; i < max_seq; ++i) sf[i] = (float)i + 1.0f;
  for (size_t i = 0; i < sh.size(); ++i) sh[i] = 0.25f * (float)i;
  CHECK(be.gpu_score_acc()->seed_cumulative(sf, sh).ok(), "seed");
  auto r3 = be.gpu_score_acc()->sync_to_cpu();
  CHECK(r3.value().first == sf && r3.value().second == sh, "case3 seed round trip");
  CHECK(!be.gpu_score_acc()->seed_cumulative(std::vector<float>(3), sh).ok(), "seed length check");
  // per-layer flat cumulative: seed, read back, clear alone (gpu_score.rs:329-363)
  std::vector<float> lf(n_layers * max_seq);
  for (size_t i = 0; i < lf.size(); ++i) lf[i] = 0.5f * (float)i;
  CHECK(be.gpu_score_acc()->seed_layer_flat_cumulative(lf).ok(), "seed_layer_flat_cumulative");
  CHECK(!be.gpu_score_acc()->seed_layer_flat_cumulative(std::vector<float>(5)).ok(), "layer_flat length check");
  CHECK(be.gpu_score_acc()->sync_layer_flat_to_cpu().value() == lf, "layer_flat round trip");
  CHECK(be.gpu_score_acc()->reset_layer_flat().ok(), "reset_layer_flat");
  auto cleared = be.gpu_score_acc()->sync_layer_flat_to_cpu();
  for (float x : cleared.value()) CHECK(x == 0.0f, "reset_layer_flat clears");
  CHECK(be.gpu_score_acc()->sync_to_cpu().value().first == sf, "reset_layer_flat leaves the collapsed buffers");
  CHECK(be.gpu_score_acc()->reset().ok(), "reset");
  auto r4 = be.gpu_score_acc()->sync_to_cpu();
  for (float x : r4.value().first) CHECK(x == 0.0f, "reset clears");
  printf("[score] accumulator cases 1-3 ok\n");
}

static void test_attention_gen(HipBackend &be) {
  const int hq = 4, hkv = 2, d = 64, len = 16, cap = 32;
  std::vector<float> q(hq * d), kf(hkv * cap * d), vf(hkv * cap * d);
  oracle_gen_data(q.data(), q.size(), 42); oracle_gen_data(kf.data(), kf.size(), 137); oracle_gen_data(vf.data(), vf.size(), 53);
  std::vector<uint16_t> kh(kf.size()), vh(vf.size());
  oracle_f32_to_f16(kf.data(), kh.data(), kf.size()); oracle_f32_to_f16(vf.data(), vh.data(), vf.size());
  for (int f16 = 0; f16 < 2; ++f16) {
    const void *kp = f16 ? (const void *)kh.data() : (const void *)kf.data();
    const void *vp = f16 ? (const void *)vh.data() : (const void *)vf.data();
    const size_t kvb = kf.size() * (f16 ? 2 : 4);
    DevBuf dq(&be, q.size() * 4, q.data()), dk(&be, kvb, kp), dv(&be, kvb, vp), dout(&be, q.size() * 4);
    Tensor tq{dq.p, DType::F32, {(size_t)hq, (size_t)d}}, tout{dout.p, DType::F32, {(size_t)hq, (size_t)d}};
    Tensor tk{dk.p, f16 ? DType::F16 : DType::F32, {1, (size_t)hkv, (size_t)cap, (size_t)d}}, tv = tk;
    tv.ptr = dv.p;
    // scores at stride `cap` (> cache_seq_len): rows beyond len keep their sentinel
    std::vector<float> sc(hq * cap, -7.0f), ref(hq * d), ref_sc(hq * cap, -7.0f), got(hq * d);
    CHECK(be.attention_gen(tq, tk, tv, tout, hq, hkv, d, len, sc.data(), sc.size()).ok(), "attention_gen");
    be.read_buffer(got.data(), dout.p, got.size() * 4);
    oracle_attention_gen_scalar(q.data(), kp, vp, ref.data(), hq, hkv, d, len, cap, 1, f16, ref_sc.data(), cap, 0.0f, nullptr);
    CHECK(max_abs_diff(got, ref) < (f16 ? 1e-3f : 1e-4f), "attention_gen out diff %g", max_abs_diff(got, ref));
    float worst = 0;
    for (int h = 0; h < hq; ++h)
      for (int t = 0; t < len; ++t) worst = fmaxf(worst, fabsf(sc[h * cap + t] - ref_sc[h * cap + t]) / ref_sc[h * cap + t]);
    CHECK(worst < 1e-4f, "scores rel diff %g", worst);
    // a malformed score slice (stride < cache_seq_len) disables the export, the call still succeeds
    std::vector<float> small(hq * 4, -7.0f);
    CHECK(be.attention_gen(tq, tk, tv, tout, hq, hkv, d, len, small.data(), small.size()).ok(), "malformed slice");
    for (float x : small) CHECK(x == -7.0f, "malformed slice untouched");
    // SelectiveRead (standard_format.rs:2043-2184): a token selection, the same as pages, an empty one
    {
      const std::vector<size_t> sel = {0, 1, 2, 3, 6, 9, 10, 11, (size_t)len - 2, (size_t)len - 1};
      std::vector<int32_t> idx(sel.begin(), sel.end());
      std::vector<float> ssc(hq * sel.size(), -7.0f), sref(hq * d), sref_sc(hq * sel.size(), -7.0f);
      CHECK(be.attention_into_selected(tq, tk, tv, tout, hq, hkv, d, len, sel, 0, ssc.data(), ssc.size()).ok(), "attention_into_selected");
      be.read_buffer(got.data(), dout.p, got.size() * 4);
      oracle_attention_gen_scalar(q.data(), kp, vp, sref.data(), hq, hkv, d, (int)sel.size(), cap, 1, f16, sref_sc.data(), (int64_t)sel.size(), 0.0f, idx.data());
      CHECK(max_abs_diff(got, sref) < (f16 ? 1e-3f : 1e-4f), "selected out diff %g", max_abs_diff(got, sref));
      CHECK(max_abs_diff(ssc, sref_sc) < 1e-5f, "selected scores diff %g", max_abs_diff(ssc, sref_sc));
      // pages of 4: page 0 = positions 0..3, the last page clamped to current_pos
      const std::vector<size_t> pages = {0, (size_t)(len - 1) / 4};
      std::vector<int32_t> pidx = {0, 1, 2, 3};
      for (int pos = (len - 1) / 4 * 4; pos < len; ++pos) pidx.push_back(pos);
      CHECK(be.attention_into_selected(tq, tk, tv, tout, hq, hkv, d, len, pages, 4, nullptr, 0).ok(), "attention_into_selected pages");
      be.read_buffer(got.data(), dout.p, got.size() * 4);
      oracle_attention_gen_scalar(q.data(), kp, vp, sref.data(), hq, hkv, d, (int)pidx.size(), cap, 1, f16, nullptr, 0, 0.0f, pidx.data());
      CHECK(max_abs_diff(got, sref) < (f16 ? 1e-3f : 1e-4f), "paged out diff %g", max_abs_diff(got, sref));
      // select = every position: the full read
      std::vector<size_t> all(len);
      for (int t = 0; t < len; ++t) all[t] = t;
      CHECK(be.attention_into_selected(tq, tk, tv, tout, hq, hkv, d, len, all, 0, nullptr, 0).ok(), "select all");
      be.read_buffer(got.data(), dout.p, got.size() * 4);
      CHECK(max_abs_diff(got, ref) < (f16 ? 1e-3f : 1e-4f), "select-all equals the full read (%g)", max_abs_diff(got, ref));
      CHECK(be.attention_into_selected(tq, tk, tv, tout, hq, hkv, d, len, {}, 0, nullptr, 0).ok(), "empty selection");
      be.read_buffer(got.data(), dout.p, got.size() * 4);
      for (float x : got) CHECK(x == 0.0f, "empty selection zeroes out");
      CHECK(!be.attention_into_selected(tq, tk, tv, tout, hq, hkv, d, len, {(size_t)cap + 3}, 0, nullptr, 0).ok(), "position outside the cache refused");
    }
    // SeqMajor-shaped tensor ([len, hkv, d]) is detected from the shape
    Tensor host_q = tq;
    host_q.device = false;
    CHECK(!be.attention_gen(host_q, tk, tv, tout, hq, hkv, d, len, nullptr, 0).ok(), "host tensor is refused");
  }
  {
    // Q4_0 cache (BlockQ4_0 rows, common.rs:676-850): blocks made by the q4_0 encoder, reference =
    // the same blocks decoded to F32 and attended by the scalar oracle.
    std::vector<uint8_t> kq(kf.size() / 32 * 18), vq(kq.size());
    CHECK(oracle_encode_via_descriptor(32, 4, 1, 1, kf.data(), kq.data(), kf.size()) == 0, "encode K");
    CHECK(oracle_encode_via_descriptor(32, 4, 1, 1, vf.data(), vq.data(), vf.size()) == 0, "encode V");
    std::vector<float> kd(kf.size()), vd(vf.size());
    oracle_decode_via_descriptor(32, 4, 1, 1, kq.data(), kd.data(), kd.size());
    oracle_decode_via_descriptor(32, 4, 1, 1, vq.data(), vd.data(), vd.size());
    DevBuf dq(&be, q.size() * 4, q.data()), dk(&be, kq.size(), kq.data()), dv(&be, vq.size(), vq.data()), dout(&be, q.size() * 4);
    Tensor tq{dq.p, DType::F32, {(size_t)hq, (size_t)d}}, tout{dout.p, DType::F32, {(size_t)hq, (size_t)d}};
    Tensor tk{dk.p, DType::Q4_0, {1, (size_t)hkv, (size_t)cap, (size_t)d}}, tv = tk;
    tv.ptr = dv.p;
    std::vector<float> sc(hq * len), ref(hq * d), ref_sc(hq * len), got(hq * d);
    CHECK(be.attention_gen(tq, tk, tv, tout, hq, hkv, d, len, sc.data(), sc.size()).ok(), "attention_gen q4_0: %s", be.last_error().c_str());
    be.read_buffer(got.data(), dout.p, got.size() * 4);
    oracle_attention_gen_scalar(q.data(), kd.data(), vd.data(), ref.data(), hq, hkv, d, len, cap, 1, 0, ref_sc.data(), len, 0.0f, nullptr);
    CHECK(max_abs_diff(got, ref) < 1e-3f, "attention_gen q4_0 out diff %g", max_abs_diff(got, ref));
    float worst = 0;
    for (size_t i = 0; i < sc.size(); ++i) worst = fmaxf(worst, fabsf(sc[i] - ref_sc[i]) / ref_sc[i]);
    CHECK(worst < 1e-4f, "q4_0 scores rel diff %g", worst);
  }
  printf("[attention_gen] unit shape f32/f16/q4_0 + host score slice + selective read (tokens, pages, all, none) ok\n");
}

static void test_accumulator_binding(HipBackend &be) {
  // With the accumulator active the kernel writes the layer's slice of the persistent score buffer
  // and the host slice is left alone (cuda_pc.rs:1750-1766); end_step then reduces on the device.
  const int n_layers = 3, hq = 8, hkv = 4, d = 128, len = 300, max_seq = 512;
  CHECK(be.init_gpu_score_acc(n_layers, hq, hkv, max_seq, 0.0f).ok(), "init");
  be.gpu_score_acc()->set_active(true);
  std::vector<float> all_scores((size_t)n_layers * hq * max_seq, 0.0f);
  for (int l = 0; l < n_layers; ++l) {
    std::vector<float> q(hq * d), kf(hkv * max_seq * d), vf(kf.size());
    oracle_gen_data(q.data(), q.size(), 100 + l); oracle_gen_data(kf.data(), kf.size(), 200 + l); oracle_gen_data(vf.data(), vf.size(), 300 + l);
    for (auto &x : q) x *= 4.0f;
    std::vector<uint16_t> kh(kf.size()), vh(vf.size());
    oracle_f32_to_f16(kf.data(), kh.data(), kf.size()); oracle_f32_to_f16(vf.data(), vh.data(), vf.size());
    DevBuf dq(&be, q.size() * 4, q.data()), dk(&be, kh.size() * 2, kh.data()), dv(&be, vh.size() * 2, vh.data()), dout(&be, q.size() * 4);
    Tensor tq{dq.p, DType::F32, {(size_t)hq, (size_t)d}}, tout = tq, tk{dk.p, DType::F16, {1, (size_t)hkv, (size_t)max_seq, (size_t)d}}, tv = tk;
    tout.ptr = dout.p; tv.ptr = dv.p;
    be.gpu_score_acc()->set_current_layer_idx(l);
    std::vector<float> host_sc(hq * len, -7.0f);
    CHECK(be.attention_gen(tq, tk, tv, tout, hq, hkv, d, len, host_sc.data(), host_sc.size()).ok(), "attention_gen layer %d", l);
    for (float x : host_sc) CHECK(x == -7.0f, "host slice untouched while the accumulator is armed");
    std::vector<float> ref(hq * d);
    oracle_attention_gen_scalar(q.data(), kh.data(), vh.data(), ref.data(), hq, hkv, d, len, max_seq, 1, 1,
                                &all_scores[(size_t)l * hq * max_seq], max_seq, 0.0f, nullptr);
  }
  CHECK(be.gpu_score_acc()->end_step(nullptr, len).ok(), "end_step");
  be.synchronize();
  auto r = be.gpu_score_acc()->sync_to_cpu();
  std::vector<float> imp(max_seq, 0.0f), himp(hkv * max_seq, 0.0f);
  oracle_score_fused_reduce(all_scores.data(), imp.data(), himp.data(), 1.0f, n_layers, hq, hkv, len, max_seq, max_seq);
  float worst = 0;
  for (int t = 0; t < len; ++t) worst = fmaxf(worst, fabsf(r.value().first[t] - imp[t]) / imp[t]);
  for (size_t i = 0; i < himp.size(); ++i)
    if (himp[i] > 0) worst = fmaxf(worst, fabsf(r.value().second[i] - himp[i]) / himp[i]);
  CHECK(worst < 1e-4f, "importance rel diff %g", worst);
  be.gpu_score_acc()->set_active(false);
  printf("[score] attention -> accumulator slice -> fused reduce ok (rel %.2e)\n", worst);
}

static void test_prefill_and_scatter(HipBackend &be) {
  const int hq = 8, hkv = 2, d = 64, s = 100, cap = 128;
  std::vector<float> q((size_t)s * hq * d), ksrc((size_t)s * hkv * d), vsrc(ksrc.size());
  oracle_gen_data(q.data(), q.size(), 1); oracle_gen_data(ksrc.data(), ksrc.size(), 2); oracle_gen_data(vsrc.data(), vsrc.size(), 3);
  // write path: scatter the prompt's K/V rows into the HeadMajor F16 cache (supports_kv_scatter_batch)
  DevBuf dq(&be, q.size() * 4, q.data()), dks(&be, ksrc.size() * 4, ksrc.data()), dvs(&be, vsrc.size() * 4, vsrc.data());
  std::vector<uint16_t> zero((size_t)hkv * cap * d, 0), kc = zero, vc = zero;
  DevBuf dk(&be, zero.size() * 2, zero.data()), dv(&be, zero.size() * 2, zero.data()), dout(&be, q.size() * 4);
  Tensor tks{dks.p, DType::F32, {(size_t)s, (size_t)hkv, (size_t)d}}, tvs = tks;
  tvs.ptr = dvs.p;
  Tensor tk{dk.p, DType::F16, {1, (size_t)hkv, (size_t)cap, (size_t)d}}, tv = tk;
  tv.ptr = dv.p;
  CHECK(be.supports_kv_scatter_batch(), "scatter batch");
  CHECK(be.kv_scatter_f32_to_f16_batch(tks, tvs, tk, tv, hkv, d, cap, 0, s).ok(), "kv_scatter batch");
  oracle_kv_scatter(ksrc.data(), vsrc.data(), kc.data(), vc.data(), hkv, d, cap, 0, s, 1);
  std::vector<uint16_t> got_k(zero.size());
  be.read_buffer(got_k.data(), dk.p, got_k.size() * 2);
  CHECK(memcmp(got_k.data(), kc.data(), kc.size() * 2) == 0, "scattered K cache bit-exact");
  CHECK(!be.kv_scatter_f32_to_f16_batch(tks, tvs, tk, tv, hkv, d, cap, cap - 1, s).ok(), "scatter beyond capacity fails");
  // prefill over the scattered cache
  Tensor tq{dq.p, DType::F32, {1, (size_t)s, (size_t)hq, (size_t)d}}, tout = tq;
  tout.ptr = dout.p;
  auto r = be.flash_attention_prefill(tq, tk, tv, tout, hq, hkv, s, s, d, cap, 1, true);
  CHECK(r.ok() && r.value(), "prefill dispatched");
  std::vector<float> got(q.size()), ref(q.size());
  be.read_buffer(got.data(), dout.p, got.size() * 4);
  oracle_prefill_attention(q.data(), kc.data(), vc.data(), ref.data(), hq, hkv, s, s, d, cap, 1, 1, 0, 0);
  CHECK(max_abs_diff(got, ref) < 2e-3f, "prefill diff %g", max_abs_diff(got, ref));
  // Ok(false): SeqMajor and unsupported head_dim are declined, the caller keeps its CPU path
  auto r2 = be.flash_attention_prefill(tq, tk, tv, tout, hq, hkv, s, s, d, cap, 1, false);
  CHECK(r2.ok() && !r2.value(), "SeqMajor declined");
  auto r3 = be.flash_attention_prefill(tq, tk, tv, tout, hq, hkv, s, s, 96, cap, 1, true);
  CHECK(r3.ok() && !r3.value(), "head_dim 96 declined");
  auto r4 = be.flash_attention_prefill(tq, tk, tv, tout, hq, 3, s, s, d, cap, 1, true);
  CHECK(!r4.ok(), "bad head counts are an error");
  printf("[prefill] kv_scatter -> flash_attention_prefill ok, declines reported as Ok(false)\n");
}

static void test_quant_attn(HipBackend &be) {
  HipQuantAttnBackend degraded(nullptr);
  argus_hip_quant_attn_args za{};
  argus_hip_quant_gather_args zg{};
  argus_hip_quant_dequant_flush_args zd{};
  argus_hip_quant_scatter_residual_args zs{};
  CHECK(!degraded.has_quant_attn_kernel(2) && degraded.attention_gen_quant(za) == -1 && degraded.gather_update_quant(zg) == -1 &&
            degraded.dequant_flush(zd) == -1 && degraded.scatter_residual(zs) == -1,
        "degraded handle returns -1 everywhere");
  HipQuantAttnBackend cap(be.ctx());
  CHECK(cap.has_quant_attn_kernel(2) && cap.has_quant_attn_kernel(4) && cap.has_quant_attn_kernel(8) && !cap.has_quant_attn_kernel(3), "kernels present");
  // Test A of the reference device test at head_dim 64: residual-only attention with host score read-back.
  const size_t nhq = 2, nhkv = 1, hd = 64, res_cap = 32, r = 20;
  const float scale = 1.0f / sqrtf((float)hd);
  std::vector<float> q(nhq * hd), rk(nhkv * res_cap * hd, 0.0f), rv(rk.size(), 0.0f);
  for (size_t h = 0; h < nhq; ++h)
    for (size_t d = 0; d < hd; ++d) q[h * hd + d] = 0.1f * (float)((h * 7 + d) % 5) - 0.2f;
  for (size_t t = 0; t < r; ++t)
    for (size_t d = 0; d < hd; ++d) {
      rk[t * hd + d] = 0.05f * (float)((t * 3 + d) % 7) - 0.15f;
      rv[t * hd + d] = 0.03f * (float)((t + d * 2) % 9);
    }
  DevBuf dq(&be, q.size() * 4, q.data()), drk(&be, rk.size() * 4, rk.data()), drv(&be, rv.size() * 4, rv.data()), dummy(&be, 16), dout(&be, q.size() * 4);
  // gather_update_quant appends a token row to the residual ring
  std::vector<float> tok(nhkv * hd, 0.5f);
  DevBuf dtok(&be, tok.size() * 4, tok.data());
  argus_hip_quant_gather_args g{nullptr, (uint64_t)dtok.p, (uint64_t)drk.p, nhkv, res_cap, hd, 1, r};
  CHECK(cap.gather_update_quant(g) == 0, "gather_update_quant");
  std::vector<float> rk_back(rk.size());
  be.read_buffer(rk_back.data(), drk.p, rk_back.size() * 4);
  CHECK(rk_back[r * hd + 3] == 0.5f && rk_back[(r - 1) * hd + 3] == rk[(r - 1) * hd + 3], "residual row appended at res_pos");
  std::vector<float> scores_host(nhq * r, 0.0f);
  argus_hip_quant_attn_args a{};
  a.q_mem = (uint64_t)dq.p; a.qk_mem = (uint64_t)dummy.p; a.qv_mem = (uint64_t)dummy.p;
  a.res_k_mem = (uint64_t)drk.p; a.res_v_mem = (uint64_t)drv.p; a.out_mem = (uint64_t)dout.p;
  a.scores_out = scores_host.data(); a.scores_len = scores_host.size();
  a.num_heads_q = nhq; a.num_heads_kv = nhkv; a.head_dim = hd; a.q_tokens = 0; a.res_tokens = r; a.res_cap = res_cap;
  a.scale = scale; a.bits = 2;
  CHECK(cap.attention_gen_quant(a) == 0, "attention_gen_quant residual rc");
  std::vector<float> o(nhq * hd);
  be.read_buffer(o.data(), dout.p, o.size() * 4);
  for (size_t h = 0; h < nhq; ++h) {
    // host f64 textbook attention, as in the reference test
    std::vector<double> s(r);
    double mx = -1e300, sum = 0;
    for (size_t t = 0; t < r; ++t) {
      double acc = 0;
      for (size_t d = 0; d < hd; ++d) acc += (double)q[h * hd + d] * (double)rk[t * hd + d];
      s[t] = acc * (double)scale;
      mx = fmax(mx, s[t]);
    }
    for (size_t t = 0; t < r; ++t) { s[t] = exp(s[t] - mx); sum += s[t]; }
    double wsum = 0;
    for (size_t t = 0; t < r; ++t) {
      CHECK(fabs(scores_host[h * r + t] - s[t] / sum) < 1e-4, "A: weight[h%zu,t%zu]", h, t);
      wsum += scores_host[h * r + t];
    }
    CHECK(fabs(wsum - 1.0) < 1e-4, "A: weights sum %g", wsum);
    for (size_t d = 0; d < hd; ++d) {
      double od = 0;
      for (size_t t = 0; t < r; ++t) od += s[t] / sum * (double)rv[t * hd + d];
      CHECK(fabs(o[h * hd + d] - od) < 1e-4, "A: O[h%zu,d%zu]", h, d);
    }
  }
  a.bits = 3;
  CHECK(cap.attention_gen_quant(a) < 0, "unsupported bits return a negative code");
  printf("[kivi] degraded handle, gather_update, residual-only attention + host score read-back ok\n");
}

// Faithful-H2O seed on the device: the PFA column sums of every layer are produced on the device
// into one [n_layers, n_heads_q, prefix] buffer and folded into the cumulative importance by one
// synthetic reduce step (attention_scores.rs:249-276), with no host round trip.  Expected values:
// the oracle's PFA per layer folded by the oracle's reduce.
static void test_prefill_seed(HipBackend &be) {
  const size_t n_layers = 3, hq = 8, hkv = 2, hd = 64, prefix = 96, seq = 40, qwin = 16, max_seq = 128;
  CHECK(be.init_gpu_score_acc(n_layers, hq, hkv, max_seq, 0.0f).ok(), "init");
  be.gpu_score_acc()->set_active(true);
  std::vector<float> ref_pfa(n_layers * hq * prefix, 0.0f);
  DevBuf dpfa(&be, ref_pfa.size() * 4, ref_pfa.data());  // zeroed: the side channel accumulates
  for (size_t l = 0; l < n_layers; ++l) {
    std::vector<float> q(seq * hq * hd), k(hkv * prefix * hd);
    oracle_gen_data(q.data(), q.size(), 700 + l); oracle_gen_data(k.data(), k.size(), 800 + l);
    DevBuf dq(&be, q.size() * 4, q.data()), dk(&be, k.size() * 4, k.data());
    Tensor tq{dq.p, DType::F32, {seq, hq, hd}, true}, tk{dk.p, DType::F32, {1, hkv, prefix, hd}, true};
    // HeadMajor K: key stride hd, head stride prefix * hd; chunked prefill: q_start_pos = prefix - seq
    CHECK(be.prefill_attention_scores(tq, tk, hq, hkv, hd, seq, prefix, hd, prefix * hd, prefix - seq, qwin, false, 0,
                                      (float *)dpfa.p + l * hq * prefix, nullptr, false).ok(), "pfa layer %zu", l);
    oracle_prefill_attention_scores(q.data(), k.data(), hq, hkv, hd, seq, prefix, hd, prefix * hd, prefix - seq, qwin, -1,
                                    ref_pfa.data() + l * hq * prefix, nullptr, 0);
  }
  CHECK(be.gpu_score_acc()->seed_prefill_importance_device(nullptr, dpfa.p, prefix).ok(), "seed");
  std::vector<float> imp(max_seq, 0.0f), himp(hkv * max_seq, 0.0f);
  oracle_score_fused_reduce(ref_pfa.data(), imp.data(), himp.data(), 1.0f, n_layers, hq, hkv, prefix, prefix, max_seq);
  auto got = be.gpu_score_acc()->sync_to_cpu();
  CHECK(got.ok(), "sync");
  float worst = 0, total = 0;
  for (size_t t = 0; t < prefix; ++t) {
    worst = fmaxf(worst, fabsf(got.value().first[t] - imp[t]) / fmaxf(imp[t], 1e-30f));
    total += got.value().first[t];
  }
  for (size_t i = 0; i < himp.size(); ++i)
    if (i % max_seq < prefix) worst = fmaxf(worst, fabsf(got.value().second[i] - himp[i]) / fmaxf(himp[i], 1e-30f));
  CHECK(worst < 1e-4f, "seeded importance rel diff %g", worst);
  for (size_t t = prefix; t < max_seq; ++t) CHECK(got.value().first[t] == 0.0f, "positions past the prefix untouched");
  CHECK(total > 0.0f, "seed is not empty");
  CHECK(be.gpu_score_acc()->steps_accumulated() == 1, "one synthetic step");
  printf("[score] PFA on the device -> one-step prefill seed of the cumulative importance ok (rel %.3g)\n", worst);
}

// The KIVI container in GPU mode, driven the way the layer loop drives it: a multi-token prefill
// update that crosses a flush, then one token per step; at checkpoints the device blocks must be
// the CPU container's bit for bit, the fused attention and its host scores must match the oracle's
// attention over that container, and the F16 view must be the dequantised cache.
static float f16_bits_to_f32(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000) << 16, exp = (h >> 10) & 31, man = h & 1023;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) bits = sign;
    else {
      int e = -1;
      uint32_t m = man;
      do { ++e; m <<= 1; } while (!(m & 1024));
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((m & 1023) << 13);
    }
  } else if (exp == 31) bits = sign | 0x7f800000u | (man << 13);
  else bits = sign | ((exp + 112) << 23) | (man << 13);
  float f;
  memcpy(&f, &bits, 4);
  return f;
}
static void test_quant_window_cache(HipBackend &be) {
  const size_t hq = 8, hkv = 2, hd = 128, res_cap = 64, max_seq = 320, total = 3 * res_cap + 37;
  std::vector<float> k(total * hkv * hd), v(k.size()), q(hq * hd);
  oracle_gen_data(k.data(), k.size(), 501); oracle_gen_data(v.data(), v.size(), 502); oracle_gen_data(q.data(), q.size(), 503);
  for (size_t t = 0; t < total; ++t) k[(t * hkv + 1) * hd + 7] *= 12.0f;  // an outlier channel
  DevBuf dk(&be, k.size() * 4, k.data()), dv(&be, v.size() * 4, v.data()), dq(&be, q.size() * 4, q.data()), dout(&be, q.size() * 4);
  CHECK(!HipQuantWindowCache::new_gpu(&be, hkv, hd, max_seq, 48, 4).ok(), "residual_size must be a multiple of 32");
  CHECK(!HipQuantWindowCache::new_gpu(&be, hkv, hd, max_seq, res_cap, 3).ok(), "bits 3 refused");
  for (int bits : {2, 4, 8}) {
    auto made = HipQuantWindowCache::new_gpu(&be, hkv, hd, max_seq, res_cap, (uint8_t)bits);
    CHECK(made.ok(), "new_gpu bits %d: %s", bits, made.error().c_str());
    if (!made.ok()) return;
    HipQuantWindowCache &c = *made.value();
    const size_t bb = 4 + 32 * bits / 8;
    auto tokens = [&](void *base, size_t first, size_t n) {
      return Tensor{(char *)base + first * hkv * hd * 4, DType::F32, {1, n, hkv, hd}, true};
    };
    auto check_at = [&](size_t n) {
      CHECK(c.current_pos() == n, "current_pos %zu != %zu", c.current_pos(), n);
      const size_t max_blocks = (n / res_cap + 1) * hkv * res_cap * hd / 32;
      std::vector<uint8_t> rqk(max_blocks * bb, 0), rqv(max_blocks * bb, 0);
      std::vector<float> rrk(hkv * res_cap * hd, 0.0f), rrv(rrk.size(), 0.0f);
      int qt = 0, rt = 0;
      CHECK(oracle_kivi_build(k.data(), v.data(), (int)n, hkv, hd, res_cap, bits, rqk.data(), rqv.data(), rrk.data(), rrv.data(), &qt, &rt) == 0, "oracle build");
      auto raw_r = c.get_raw_gpu_buffers();
      CHECK(raw_r.ok(), "raw buffers");
      if (!raw_r.ok()) return;
      const QuantWindowRawBuffers raw = raw_r.value();
      CHECK(raw.q_tokens == (size_t)qt && raw.res_tokens == (size_t)rt && raw.bits == bits, "q_tokens %zu/%d res_tokens %zu/%d", raw.q_tokens, qt, raw.res_tokens, rt);
      const size_t used = (size_t)qt * hkv * hd / 32 * bb;
      std::vector<uint8_t> gk(used), gv(used);
      if (used) {
        be.read_buffer(gk.data(), raw.qk_buf, used);
        be.read_buffer(gv.data(), raw.qv_buf, used);
        CHECK(memcmp(gk.data(), rqk.data(), used) == 0, "bits %d n %zu: key blocks differ from the CPU container", bits, n);
        CHECK(memcmp(gv.data(), rqv.data(), used) == 0, "bits %d n %zu: value blocks differ from the CPU container", bits, n);
      }
      std::vector<float> grk(rrk.size());
      be.read_buffer(grk.data(), raw.res_k, grk.size() * 4);
      bool same = true;
      for (size_t h = 0; h < hkv; ++h)
        for (size_t i = 0; i < (size_t)rt * hd; ++i) same = same && grk[h * res_cap * hd + i] == rrk[h * res_cap * hd + i];
      CHECK(same, "bits %d n %zu: residual ring differs", bits, n);
      // fused attention + host scores
      std::vector<float> ref(hq * hd), ref_sc(hq * n), got(hq * hd), sc(hq * n, -1.0f);
      const float scale = 1.0f / sqrtf((float)hd);
      oracle_kivi_attention(q.data(), rqk.data(), rqv.data(), rrk.data(), rrv.data(), ref.data(), ref_sc.data(), (int64_t)n, hq, hkv, hd, qt, rt, res_cap, scale, bits);
      Tensor tq{dq.p, DType::F32, {hq, hd}, true}, tout{dout.p, DType::F32, {hq, hd}, true};
      auto st = c.attention_native(tq, tout, hq, sc.data(), sc.size());
      CHECK(st.ok(), "attention_native: %s", st.error().c_str());
      be.read_buffer(got.data(), dout.p, got.size() * 4);
      CHECK(max_abs_diff(got, ref) < 2e-3f, "bits %d n %zu: attention out diff %g", bits, n, max_abs_diff(got, ref));
      float worst = 0;
      for (size_t i = 0; i < sc.size(); ++i) worst = fmaxf(worst, fabsf(sc[i] - ref_sc[i]) / fmaxf(ref_sc[i], 1e-30f));
      CHECK(worst < 1e-4f, "bits %d n %zu: scores rel diff %g", bits, n, worst);
      // F16 view = dequantised blocks + residual rows
      std::vector<float> vk(n * hkv * hd), vv(vk.size());
      oracle_kivi_assemble_view(rqk.data(), rqv.data(), rrk.data(), rrv.data(), qt, rt, hkv, hd, res_cap, bits, vk.data(), vv.data());
      auto view = c.get_view_gpu();
      CHECK(view.ok(), "get_view_gpu: %s", view.error().c_str());
      if (!view.ok()) return;
      std::vector<uint16_t> hk(vk.size()), hv(vk.size());
      be.read_buffer(hk.data(), view.value().first.ptr, hk.size() * 2);
      be.read_buffer(hv.data(), view.value().second.ptr, hv.size() * 2);
      float wk = 0, wv = 0;
      for (size_t i = 0; i < vk.size(); ++i) {
        wk = fmaxf(wk, fabsf(f16_bits_to_f32(hk[i]) - vk[i]) / (1.0f + fabsf(vk[i])));
        wv = fmaxf(wv, fabsf(f16_bits_to_f32(hv[i]) - vv[i]) / (1.0f + fabsf(vv[i])));
      }
      CHECK(wk < 1e-3f && wv < 1e-3f, "bits %d n %zu: F16 view differs (%g, %g)", bits, n, wk, wv);
    };
    // prefill of 100 tokens: fills the ring, flushes 64, leaves 36
    CHECK(c.update(tokens(dk.p, 0, 100), tokens(dv.p, 0, 100)).ok(), "prefill update");
    check_at(100);
    for (size_t t = 100; t < total; ++t) {
      auto st = c.update(tokens(dk.p, t, 1), tokens(dv.p, t, 1));
      CHECK(st.ok(), "update token %zu: %s", t, st.error().c_str());
      if (t + 1 == 128 || t + 1 == 129 || t + 1 == 3 * res_cap) check_at(t + 1);
    }
    check_at(total);
    CHECK(!c.update(tokens(dk.p, 0, max_seq), tokens(dv.p, 0, max_seq)).ok(), "overflow refused");
    // a width transition keeps the token count and serves attention at the new width
    const uint8_t other = bits == 4 ? 8 : 4;
    CHECK(c.transition_bits(other).ok() && c.bits() == other && c.current_pos() == total, "transition_bits");
    {
      std::vector<float> got(hq * hd);
      Tensor tq{dq.p, DType::F32, {hq, hd}, true}, tout{dout.p, DType::F32, {hq, hd}, true};
      CHECK(c.attention_native(tq, tout, hq, nullptr, 0).ok(), "attention after the transition");
      be.read_buffer(got.data(), dout.p, got.size() * 4);
      bool finite = true;
      for (float x : got) finite = finite && std::isfinite(x);
      CHECK(finite, "attention after the transition is finite");
    }
    // up to the unquantised mode and down again: positions kept, raw buffers only while quantised
    CHECK(c.transition_bits(16).ok() && c.bits() == 16 && c.current_pos() == total && !c.get_raw_gpu_buffers().ok(), "transition to bits 16");
    {
      auto view = c.get_view_gpu();
      CHECK(view.ok() && view.value().first.dtype == DType::F32 && view.value().first.dims[1] == hkv, "bits 16: the residual is the view");
    }
    CHECK(c.transition_bits(bits).ok() && c.bits() == bits && c.current_pos() == total, "transition back from bits 16");
    {
      auto raw = c.get_raw_gpu_buffers();
      CHECK(raw.ok() && raw.value().res_cap == 32 && raw.value().q_tokens == total / 32 * 32, "ring of 32 after the transition");
    }
    CHECK(!c.transition_bits(5).ok(), "width 5 refused");
    CHECK(c.reset().ok() && c.current_pos() == 0 && !c.get_raw_gpu_buffers().ok(), "reset");
  }
  printf("[kivi] quant-window container on the device: update / flush / raw buffers / fused attention / F16 view ok (bits 2, 4, 8)\n");
}

// A committed keep-list on a device cache: compaction through overlapping buffer_shift runs must
// equal the gather cache[:, keep] (engine/src/kv/naive_reference.rs), per layer and per head; then
// write_buffer_range into the freed tail.
static void test_compaction_and_memory(HipBackend &be) {
  const size_t hkv = 3, cap = 64, hd = 64, cur = 50;
  std::vector<float> host_k(hkv * cap * hd), host_v(hkv * cap * hd);
  for (size_t i = 0; i < host_k.size(); ++i) {
    host_k[i] = (float)(i % 977) * 0.25f;
    host_v[i] = -(float)(i % 613);
  }
  DevBuf dk(&be, host_k.size() * 4, host_k.data()), dv(&be, host_v.size() * 4, host_v.data());
  HipKvCache c;
  c.be = &be;
  c.k = Tensor{dk.p, DType::F32, {1, hkv, cap, hd}, true};
  c.v = Tensor{dv.p, DType::F32, {1, hkv, cap, hd}, true};
  c.kv_heads = hkv; c.capacity = cap; c.head_dim = hd; c.current_pos = cur; c.head_major = true;
  // sinks 0..3, two heavy runs, the recent window: runs overlap their destinations
  std::vector<size_t> keep = {0, 1, 2, 3, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15, 16, 30, 31, 40, 41, 42, 43, 44, 45, 46, 47, 48, 49};
  CHECK(c.compact_keep_positions(keep, 0).ok(), "compact_keep_positions");
  std::vector<float> got(host_k.size());
  be.read_buffer(got.data(), dk.p, got.size() * 4);
  bool same = true;
  for (size_t h = 0; h < hkv; ++h)
    for (size_t i = 0; i < keep.size(); ++i)
      for (size_t d = 0; d < hd; ++d) same = same && got[(h * cap + i) * hd + d] == host_k[(h * cap + keep[i]) * hd + d];
  CHECK(same, "compacted K rows equal the gather");
  be.read_buffer(got.data(), dv.p, got.size() * 4);
  same = true;
  for (size_t h = 0; h < hkv; ++h)
    for (size_t i = 0; i < keep.size(); ++i)
      for (size_t d = 0; d < hd; ++d) same = same && got[(h * cap + i) * hd + d] == host_v[(h * cap + keep[i]) * hd + d];
  CHECK(same, "compacted V rows equal the gather");
  // per head: head 1 of a fresh copy only
  be.write_buffer(dk.p, host_k.data(), host_k.size() * 4);
  std::vector<size_t> keep1 = {2, 3, 4, 20, 21, 22, 23, 49};
  CHECK(c.compact_keep_positions_for_head(1, keep1, 0).ok(), "compact_keep_positions_for_head");
  be.read_buffer(got.data(), dk.p, got.size() * 4);
  same = true;
  for (size_t i = 0; i < keep1.size(); ++i)
    for (size_t d = 0; d < hd; ++d) same = same && got[(1 * cap + i) * hd + d] == host_k[(1 * cap + keep1[i]) * hd + d];
  for (size_t i = 0; i < cap * hd; ++i) same = same && got[i] == host_k[i] && got[2 * cap * hd + i] == host_k[2 * cap * hd + i];
  CHECK(same, "per-head compaction moves that head only");
  // write_buffer_range: bounds-checked upload into the tail
  std::vector<float> patch(hd, 7.5f);
  CHECK(be.write_buffer_range(dk.p, host_k.size() * 4, patch.data(), hd * 4, (cap - 1) * hd * 4).ok(), "write_buffer_range");
  CHECK(!be.write_buffer_range(dk.p, host_k.size() * 4, patch.data(), hd * 4, host_k.size() * 4 - 8).ok(), "write_buffer_range out of bounds");
  be.read_buffer(got.data(), dk.p, got.size() * 4);
  CHECK(got[(cap - 1) * hd] == 7.5f && got[(cap - 1) * hd + hd - 1] == 7.5f && got[(cap - 1) * hd - 1] == host_k[(cap - 1) * hd - 1],
        "write_buffer_range landed at the offset");
  printf("[kv] compaction through buffer_shift (layer and per head), write_buffer_range ok\n");
}

// What one attention_gen call costs a compiled caller (no interpreter in the loop): calls issued back to
// back on the default stream, wall time per call with one synchronisation at the end.  Printed, not
// asserted: the figure depends on the host.
static void report_call_cost(HipBackend &be) {
  const size_t hq = 32, hkv = 8, d = 128, cap = 4096;
  if (be.gpu_score_acc()) be.gpu_score_acc()->set_active(false);  // no score slice: the plain decode call
  std::vector<uint16_t> kv(hkv * cap * d, 0x3c00);  // 1.0
  std::vector<float> q(hq * d, 0.01f);
  DevBuf dk(&be, kv.size() * 2, kv.data()), dv(&be, kv.size() * 2, kv.data()), dq(&be, q.size() * 4, q.data()), dout(&be, q.size() * 4);
  Tensor tq{dq.p, DType::F32, {hq, d}, true}, tout{dout.p, DType::F32, {hq, d}, true};
  Tensor tk{dk.p, DType::F16, {1, hkv, cap, d}, true}, tv = tk;
  tv.ptr = dv.p;
  for (size_t len : {(size_t)512, (size_t)4096}) {
    auto first = be.attention_gen(tq, tk, tv, tout, hq, hkv, d, len, nullptr, 0);
    CHECK(first.ok(), "attention_gen: %s", first.error().c_str());
    for (int i = 0; i < 50; ++i) be.attention_gen(tq, tk, tv, tout, hq, hkv, d, len, nullptr, 0);
    be.synchronize();
    const int n = 2000;
    const auto t0 = std::chrono::steady_clock::now();
    for (int i = 0; i < n; ++i) be.attention_gen(tq, tk, tv, tout, hq, hkv, d, len, nullptr, 0);
    const auto t1 = std::chrono::steady_clock::now();
    be.synchronize();
    const auto t2 = std::chrono::steady_clock::now();
    argus_hip_decode_plan plan{};
    argus_hip_last_decode_plan(be.ctx(), &plan);
    printf("[cost] attention_gen Hq32 Hkv8 d128 L%zu, one sequence, %d launch(es) per call: %.2f us per call to issue, %.2f us per call end to end\n",
           len, plan.launches, std::chrono::duration<double, std::micro>(t1 - t0).count() / n,
           std::chrono::duration<double, std::micro>(t2 - t0).count() / n);
  }
}

int main() {
  auto r = HipBackend::create(0, 16, 32, 128, 32768);
  if (!r.ok()) {
    printf("no HIP device: %s\n", r.error().c_str());
    return 77;
  }
  HipBackend &be = *r.value();
  CHECK(std::string(be.name()) == "HIP" && be.is_gpu() && be.is_discrete_gpu() && be.is_nosub_device(), "identity");
  test_score_accumulator(be);
  test_attention_gen(be);
  test_accumulator_binding(be);
  test_prefill_and_scatter(be);
  test_prefill_seed(be);
  test_quant_attn(be);
  test_quant_window_cache(be);
  test_compaction_and_memory(be);
  report_call_cost(be);
  if (g_fail) {
    printf("%d check(s) FAILED\n", g_fail);
    return 1;
  }
  printf("ALL PASS: host mirror verified on-device\n");
  return 0;
}
