// torch op registrations of the layer-list models' kernels (namespace torch.ops.rfq_mix).
//
// Every op launches on the caller's current HIP stream, allocates nothing and never
// synchronises, so a decode step can be captured into a hipGraph.  Shapes are checked on the
// host against what the kernels index before anything is launched.
#include <torch/library.h>
#include <ATen/ATen.h>
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../kernels/mix_linrec.h"

namespace rfqmix {
void launch_embed_sinusoid(bool, const int32_t*, const int32_t*, const void*, const float*, float,
                           float*, int, int, int, hipStream_t);
void launch_sandwich_norm(bool, const void*, int64_t, float*, const float*, const float*,
                          const float*, float*, int, int, float, hipStream_t);
void launch_canon_conv(bool, const float*, const float*, float*, const int32_t*, const int32_t*,
                       const int32_t*, const int32_t*, void*, int, int, int, int, hipStream_t);
void launch_head_norm_append(bool, const void*, int64_t, const float*, const float*, float,
                             const int32_t*, void*, void*, int, int, int, int, int, int, float*,
                             const float*, float*, int, hipStream_t);
void launch_glu_clamped(bool, const void*, int64_t, void*, int64_t, int, int, float, float,
                        hipStream_t);
int launch_attn_talk_decode(bool, const float*, const void*, const void*, const int32_t*, int,
                            const int32_t*, const int32_t*, const int32_t*, void*, int64_t,
                            const float*, const float*, const float*, float, int, int, int, int,
                            int, int, int, int, hipStream_t);
bool launch_attn_mixq_prefill(bool, const float*, const void*, const void*, const int32_t*, int,
                              const int32_t*, const int32_t*, const int32_t*, const int32_t*,
                              const int32_t*, int, void*, int64_t, const float*, const float*, int,
                              int, int, int, int, int, hipStream_t);
bool launch_attn_mixq_prefill_mfma(const float*, const float*, const void*, const void*, const int32_t*, int,
                                   const int32_t*, const int32_t*, const int32_t*, const int32_t*,
                                   const int32_t*, int, void*, int64_t, const float*, const float*,
                                   int, int, int, int, int, int, bool, hipStream_t);
bool mixq_mfma_ok(int, int, int, int, int);
void launch_embed_rows(bool, const int32_t*, const void*, float*, int, int, int, float,
                       hipStream_t);
void launch_post_norm_add(bool, const void*, int64_t, float*, const float*, float, float, void*,
                          int, int, hipStream_t);
void launch_rms_norm_rows(bool, bool, const void*, int64_t, const float*, float, float, void*, int,
                          int, hipStream_t);
void launch_latent_norm_append(bool, const void*, int64_t, const float*, float, const int32_t*,
                               void*, int, int, int64_t, hipStream_t);
void launch_silu_mul_any(bool, const void*, int64_t, void*, int, int, hipStream_t);
void launch_softcap(float*, float, int64_t, hipStream_t);
void launch_token_shift_mix(bool, const float*, const float*, float*, const int32_t*,
                            const int32_t*, const int32_t*, const int32_t*, void*, int, int, int,
                            int, hipStream_t);
bool wkv_ok(int);
bool latent_mfma_ok(int, int);
bool launch_attn_latent_mfma(const void*, int64_t, int64_t, const void*, const int32_t*, int,
                             const int32_t*, const int32_t*, const int32_t*, const int32_t*,
                             const int32_t*, int, void*, int64_t, const float*, float, int, int, int,
                             hipStream_t);
void launch_wkv_recurrence(bool, const void*, const void*, const void*, const void*, const void*,
                           int64_t, int64_t, int64_t, int64_t, int64_t, const float*, const float*,
                           const float*, float, float*, const int32_t*, const int32_t*,
                           const int32_t*, const int32_t*, const int32_t*, int, void*, int, int, int,
                           int, hipStream_t);
void launch_moe_route_grouped(const float*, const float*, int, int, int, int, int, int32_t*, float*,
                              hipStream_t);
void launch_moe_pair_up(bool, const void*, int64_t, const int32_t*, const void*, void*, int, int,
                        int, int, int, hipStream_t);
void launch_moe_pair_down(bool, const void*, const int32_t*, const float*, const void*, const void*,
                          int64_t, float*, int, int, int, int, int, hipStream_t);
void launch_residual_add_norm(bool, float*, const void*, int64_t, bool, const void*, int64_t, bool,
                              const float*, const float*, float, float, void*, int, int, float,
                              hipStream_t);
bool launch_qk_norm_rotary_append(bool, const void*, int64_t, const float*, const float*,
                                  const float*, bool, int, float, const int32_t*, const float*, int,
                                  float, int, int, const int32_t*, void*, void*, int, int, int, int,
                                  int, int, int, int, int64_t, float*, hipStream_t);
bool launch_attn_keep_window(bool, const float*, const void*, const void*, int64_t, const int32_t*,
                             int, const int32_t*, const int32_t*, const int32_t*, const int32_t*,
                             const int32_t*, int, const float*, const void*, int64_t, void*,
                             int64_t, float, int, int, bool, int, int, int, int, int, hipStream_t);
int launch_attn_keep_decode(bool, const float*, const void*, const void*, int64_t, const int32_t*,
                            int, const int32_t*, const int32_t*, const int32_t*, int, int,
                            const float*, const void*, int64_t, void*, int64_t, float, int, int,
                            bool, int, int, int, int, int, hipStream_t);
bool keep_mfma_ok(int, int, int, bool);
bool launch_attn_keep_mfma(const float*, const void*, const void*, int64_t, const int32_t*, int,
                           const int32_t*, const int32_t*, const int32_t*, const int32_t*,
                           const int32_t*, int, const float*, const void*, int64_t, void*, int64_t,
                           float, int, int, bool, int, int, int, int, int, bool, int, int,
                           hipStream_t);
void launch_xielu_rows(bool, const void*, int64_t, void*, int64_t, int, int, float, float,
                       hipStream_t);
void launch_rotary_append(bool, const void*, int64_t, const int32_t*, const float*, int,
                          const int32_t*, void*, void*, int, int, int, int, int, int, int, int64_t,
                          float*, hipStream_t);
void launch_conv_act_heads(bool, const void*, int64_t, const float*, float*, const int32_t*,
                           const int32_t*, const int32_t*, const int32_t*, float*, int, int, int,
                           int, int, int, float, hipStream_t);
void launch_moe_route_topk(const float*, const float*, int, int, int, int32_t*, float*, hipStream_t);
void launch_gelu_rows(bool, const void*, int64_t, void*, int64_t, int, int, hipStream_t);
bool diff_mfma_ok(int, int, int);
bool launch_attn_diff_mfma(const float*, const void*, const void*, const int32_t*, int,
                           const int32_t*, const int32_t*, const int32_t*, const int32_t*,
                           const int32_t*, int, const void*, int64_t, void*, int64_t, float, int,
                           float, float, float, int, int, int, int, int, hipStream_t);
int launch_attn_diff_decode(bool, const float*, const void*, const void*, const int32_t*, int,
                            const int32_t*, const int32_t*, const int32_t*, int, int, const void*,
                            int64_t, void*, int64_t, float, int, float, float, float, int, int, int,
                            int, int, hipStream_t);
bool launch_attn_diff_window(bool, const float*, const void*, const void*, const int32_t*, int,
                             const int32_t*, const int32_t*, const int32_t*, const int32_t*,
                             const int32_t*, int, const void*, int64_t, void*, int64_t, float, int,
                             float, float, float, int, int, int, int, int, hipStream_t);
}  // namespace rfqmix

namespace {

using at::Tensor;
using OptT = c10::optional<Tensor>;

hipStream_t stream() { return c10::hip::getCurrentHIPStream().stream(); }

bool act_f32(const Tensor& t, const char* what) {
  TORCH_CHECK(t.is_cuda(), what, ": not a GPU tensor");
  TORCH_CHECK(t.scalar_type() == at::kFloat || t.scalar_type() == at::kBFloat16, what,
              ": float32 or bfloat16 expected");
  return t.scalar_type() == at::kFloat;
}

const float* f32p(const Tensor& t, const char* what, int64_t numel = -1) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == at::kFloat && t.is_contiguous(), what,
              ": contiguous float32 GPU tensor expected");
  TORCH_CHECK(numel < 0 || t.numel() == numel, what, ": wrong size");
  return t.data_ptr<float>();
}

const int32_t* i32p(const Tensor& t, const char* what, int64_t min_numel) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == at::kInt && t.is_contiguous(), what,
              ": contiguous int32 GPU tensor expected");
  TORCH_CHECK(t.numel() >= min_numel, what, ": too short");
  return t.data_ptr<int32_t>();
}

const float* optf(const OptT& t, const char* what, int64_t numel) {
  return t.has_value() ? f32p(*t, what, numel) : nullptr;
}

void embed_sinusoid(const Tensor& ids, const Tensor& pos, const Tensor& table,
                    const Tensor& inv_freq, double scale, const Tensor& out) {
  const bool f32 = act_f32(table, "embed_sinusoid table");
  const int T = (int)ids.numel(), d = (int)table.size(1);
  TORCH_CHECK(table.dim() == 2 && table.is_contiguous(), "embed_sinusoid: table [V, d]");
  TORCH_CHECK(out.dim() == 2 && out.size(0) == T && out.size(1) == d, "embed_sinusoid: out [T, d]");
  rfqmix::launch_embed_sinusoid(f32, i32p(ids, "ids", T), i32p(pos, "positions", T),
                                table.data_ptr(), f32p(inv_freq, "inv_freq", (d + 1) / 2),
                                (float)scale, const_cast<float*>(f32p(out, "out")), T, d,
                                (int)table.size(0), stream());
}

void sandwich_norm(const OptT& y, const Tensor& residual, const OptT& w_post, const OptT& gain,
                   const Tensor& w_pre, double eps, const Tensor& out) {
  TORCH_CHECK(residual.dim() == 2, "sandwich_norm: residual [T, d]");
  const int T = (int)residual.size(0), d = (int)residual.size(1);
  bool f32 = true;
  const void* yp = nullptr;
  int64_t ys = 0;
  if (y.has_value()) {
    f32 = act_f32(*y, "sandwich_norm y");
    TORCH_CHECK(y->dim() == 2 && y->size(0) == T && y->size(1) == d && y->stride(1) == 1,
                "sandwich_norm: y [T, d]");
    TORCH_CHECK(w_post.has_value() && gain.has_value(), "sandwich_norm: y needs w_post and gain");
    yp = y->data_ptr();
    ys = y->stride(0);
  }
  TORCH_CHECK(out.sizes() == residual.sizes(), "sandwich_norm: out [T, d]");
  rfqmix::launch_sandwich_norm(f32, yp, ys, const_cast<float*>(f32p(residual, "residual")),
                               y.has_value() ? f32p(*w_post, "w_post", d) : nullptr,
                               y.has_value() ? f32p(*gain, "gain", d) : nullptr,
                               f32p(w_pre, "w_pre", d), const_cast<float*>(f32p(out, "out")), T, d,
                               (float)eps, stream());
}

void canon_conv(const Tensor& h, const Tensor& w, const Tensor& state, const Tensor& row_state,
                const Tensor& row_back, const Tensor& row_fwd, const Tensor& pos,
                const Tensor& out) {
  TORCH_CHECK(h.dim() == 2 && w.dim() == 2 && state.dim() == 3, "canon_conv: h [T, d], w [d, taps], state [2S, taps-1, d]");
  const int T = (int)h.size(0), d = (int)h.size(1), taps = (int)w.size(1);
  TORCH_CHECK(w.size(0) == d && taps >= 1, "canon_conv: w [d, taps]");
  TORCH_CHECK(state.size(1) == taps - 1 && state.size(2) == d && state.size(0) % 2 == 0,
              "canon_conv: state [2 * slots, taps - 1, d]");
  const bool f32 = act_f32(out, "canon_conv out");
  TORCH_CHECK(out.is_contiguous() && out.size(0) == T && out.size(1) == d, "canon_conv: out [T, d]");
  rfqmix::launch_canon_conv(f32, f32p(h, "h"), f32p(w, "w"), const_cast<float*>(f32p(state, "state")),
                            i32p(row_state, "row_state", T), i32p(row_back, "row_back", T),
                            i32p(row_fwd, "row_fwd", T), i32p(pos, "positions", T), out.data_ptr(),
                            T, d, taps, (int)state.size(0) / 2, stream());
}

void head_norm_append(const Tensor& qkv, const Tensor& q_w, const Tensor& k_w, double eps,
                      const Tensor& slots, const Tensor& k_cache, const Tensor& v_cache, int64_t H,
                      int64_t G, int64_t dim, int64_t vdim, const Tensor& qn, const OptT& ts,
                      const OptT& qmix, int64_t mix_from) {
  const bool f32 = act_f32(qkv, "head_norm_append qkv");
  const int T = (int)qkv.size(0);
  TORCH_CHECK(qkv.dim() == 2 && qkv.stride(1) == 1 && qkv.size(1) == H * dim + G * (dim + vdim),
              "head_norm_append: qkv [T, H dim + G (dim + vdim)]");
  TORCH_CHECK(H % G == 0 && H * dim * 4 <= 64 * 1024, "head_norm_append: heads do not fit");
  TORCH_CHECK(k_cache.scalar_type() == qkv.scalar_type() && v_cache.scalar_type() == qkv.scalar_type(),
              "head_norm_append: cache dtype");
  TORCH_CHECK(k_cache.dim() == 4 && k_cache.is_contiguous() && k_cache.size(1) == G &&
              k_cache.size(3) == dim, "head_norm_append: k_cache [blocks, G, BS, dim]");
  TORCH_CHECK(v_cache.dim() == 4 && v_cache.is_contiguous() && v_cache.size(1) == G &&
              v_cache.size(3) == vdim && v_cache.size(2) == k_cache.size(2) &&
              v_cache.size(0) == k_cache.size(0), "head_norm_append: v_cache [blocks, G, BS, vdim]");
  float* qm = nullptr;
  if (qmix.has_value() && mix_from < T) {
    TORCH_CHECK(ts.has_value(), "head_norm_append: mixing needs the matrix");
    qm = const_cast<float*>(f32p(*qmix, "qmix", (int64_t)(T - mix_from) * H * G * dim));
  }
  rfqmix::launch_head_norm_append(
      f32, qkv.data_ptr(), qkv.stride(0), f32p(q_w, "q_w", dim), f32p(k_w, "k_w", dim), (float)eps,
      i32p(slots, "slot_mapping", T), k_cache.data_ptr(), v_cache.data_ptr(), T, (int)H, (int)G,
      (int)dim, (int)vdim, (int)k_cache.size(2), const_cast<float*>(f32p(qn, "qn", (int64_t)T * H * dim)),
      optf(ts, "talk_scaled", H * H), qm, (int)mix_from, stream());
}

void attn_talk_decode(const Tensor& qn, const Tensor& k_cache, const Tensor& v_cache,
                      const Tensor& bt, const Tensor& q_start, const Tensor& q_len,
                      const Tensor& kv_len, const Tensor& out, const Tensor& slopes,
                      const OptT& talk, const OptT& sink, double scale, int64_t chunk,
                      int64_t max_rows) {
  const bool f32 = act_f32(k_cache, "attn_talk_decode k_cache");
  TORCH_CHECK(qn.dim() == 3, "attn_talk_decode: qn [T, H, dim]");
  const int H = (int)qn.size(1), dim = (int)qn.size(2), G = (int)k_cache.size(1);
  const int vdim = (int)v_cache.size(3), BS = (int)k_cache.size(2), NA = (int)q_len.numel();
  TORCH_CHECK(k_cache.dim() == 4 && v_cache.dim() == 4 && k_cache.is_contiguous() &&
              v_cache.is_contiguous() && k_cache.size(3) == dim && v_cache.size(1) == G &&
              v_cache.size(2) == BS && v_cache.scalar_type() == k_cache.scalar_type() && H % G == 0,
              "attn_talk_decode: caches [blocks, G, BS, dim | vdim]");
  TORCH_CHECK(out.scalar_type() == k_cache.scalar_type() && out.dim() == 2 &&
              out.size(0) == qn.size(0) && out.size(1) == (int64_t)H * vdim && out.stride(1) == 1,
              "attn_talk_decode: out [T, H vdim]");
  TORCH_CHECK(bt.dim() == 2 && bt.size(0) == NA, "attn_talk_decode: block_tables [NA, maxb]");
  TORCH_CHECK(max_rows >= 1 && max_rows <= 65535, "attn_talk_decode: max_rows");
  const int kt = rfqmix::launch_attn_talk_decode(
      f32, f32p(qn, "qn"), k_cache.data_ptr(), v_cache.data_ptr(), i32p(bt, "block_tables", 0),
      (int)bt.size(1), i32p(q_start, "q_start", NA), i32p(q_len, "q_len", NA),
      i32p(kv_len, "kv_len", NA), out.data_ptr(), out.stride(0), f32p(slopes, "slopes", H),
      optf(talk, "talk", (int64_t)H * H), optf(sink, "sink", H), (float)scale, (int)chunk, NA,
      (int)max_rows, H, G, dim, vdim, BS, stream());
  TORCH_CHECK(kt > 0, "attn_talk_decode: head sizes do not fit the LDS");
}

void attn_mixq_prefill(const Tensor& qmix, const Tensor& k_cache, const Tensor& v_cache,
                       const Tensor& bt, const Tensor& q_start, const Tensor& q_len,
                       const Tensor& kv_len, const Tensor& work_seq, const Tensor& work_qblk,
                       const Tensor& out, const Tensor& slopes, const OptT& sink, int64_t chunk,
                       int64_t qblk) {
  const bool f32 = act_f32(k_cache, "attn_mixq_prefill k_cache");
  TORCH_CHECK(qmix.dim() == 3, "attn_mixq_prefill: qmix [T, H, G dim]");
  const int H = (int)qmix.size(1), G = (int)k_cache.size(1), dim = (int)k_cache.size(3);
  const int vdim = (int)v_cache.size(3), BS = (int)k_cache.size(2), NB = (int)q_len.numel();
  const int W = (int)work_seq.numel();
  TORCH_CHECK(qblk == 32, "attn_mixq_prefill: 32 queries per work item");
  TORCH_CHECK(k_cache.dim() == 4 && v_cache.dim() == 4 && k_cache.is_contiguous() &&
              v_cache.is_contiguous() && qmix.size(2) == (int64_t)G * dim && v_cache.size(1) == G &&
              v_cache.size(2) == BS && v_cache.scalar_type() == k_cache.scalar_type() && H % G == 0,
              "attn_mixq_prefill: caches [blocks, G, BS, dim | vdim], qmix [T, H, G dim]");
  TORCH_CHECK(out.scalar_type() == k_cache.scalar_type() && out.dim() == 2 &&
              out.size(0) == qmix.size(0) && out.size(1) == (int64_t)H * vdim && out.stride(1) == 1,
              "attn_mixq_prefill: out [T, H vdim]");
  TORCH_CHECK(bt.dim() == 2 && bt.size(0) == NB, "attn_mixq_prefill: block_tables [NB, maxb]");
  const float* sk = optf(sink, "sink", H);
  const bool ok = rfqmix::launch_attn_mixq_prefill(
      f32, f32p(qmix, "qmix"), k_cache.data_ptr(), v_cache.data_ptr(), i32p(bt, "block_tables", 0),
      (int)bt.size(1), i32p(q_start, "q_start", NB), i32p(q_len, "q_len", NB),
      i32p(kv_len, "kv_len", NB), i32p(work_seq, "work_seq", W), i32p(work_qblk, "work_qblk", W), W,
      out.data_ptr(), out.stride(0), f32p(slopes, "slopes", H), sk, (int)chunk, H, G, dim, vdim, BS,
      stream());
  TORCH_CHECK(ok, "attn_mixq_prefill: value size does not fit the LDS");
}

// The same attention on MFMA tiles (bf16 caches): takes the normed queries [T, H, dim] and the
// scaled mixing matrix [H, H]; the mixed queries are formed in registers.
void attn_mix_mfma(const Tensor& qn, const Tensor& ts, const Tensor& k_cache, const Tensor& v_cache,
                   const Tensor& bt, const Tensor& q_start, const Tensor& q_len,
                   const Tensor& kv_len, const Tensor& work_seq, const Tensor& work_qblk,
                   const Tensor& out, const Tensor& slopes, const OptT& sink, int64_t chunk,
                   bool grouped) {
  TORCH_CHECK(!act_f32(k_cache, "attn_mix_mfma k_cache"), "attn_mix_mfma: bf16 caches");
  TORCH_CHECK(qn.dim() == 3 && k_cache.dim() == 4 && v_cache.dim() == 4, "attn_mix_mfma: qn [T, H, dim]");
  const int H = (int)qn.size(1), G = (int)k_cache.size(1), dim = (int)k_cache.size(3);
  const int vdim = (int)v_cache.size(3), BS = (int)k_cache.size(2), NB = (int)q_len.numel();
  const int W = (int)work_seq.numel();
  TORCH_CHECK(k_cache.is_contiguous() && v_cache.is_contiguous() && qn.size(2) == dim &&
              v_cache.size(1) == G && v_cache.size(2) == BS &&
              v_cache.scalar_type() == at::kBFloat16 && v_cache.size(0) == k_cache.size(0),
              "attn_mix_mfma: caches [blocks, G, BS, dim | vdim]");
  TORCH_CHECK(rfqmix::mixq_mfma_ok(H, G, dim, vdim, BS), "attn_mix_mfma: sizes outside the tiles");
  TORCH_CHECK(out.scalar_type() == at::kBFloat16 && out.dim() == 2 && out.size(0) == qn.size(0) &&
              out.size(1) == (int64_t)H * vdim && out.stride(1) == 1 && out.stride(0) % 4 == 0,
              "attn_mix_mfma: out [T, H vdim]");
  TORCH_CHECK(bt.dim() == 2 && bt.size(0) == NB, "attn_mix_mfma: block_tables [NB, maxb]");
  TORCH_CHECK(work_qblk.numel() >= W, "attn_mix_mfma: work lists");
  const bool ok = rfqmix::launch_attn_mixq_prefill_mfma(
      f32p(qn, "qn"), f32p(ts, "talk_scaled", (int64_t)H * H), k_cache.data_ptr(),
      v_cache.data_ptr(), i32p(bt, "block_tables", 0), (int)bt.size(1),
      i32p(q_start, "q_start", NB), i32p(q_len, "q_len", NB), i32p(kv_len, "kv_len", NB),
      i32p(work_seq, "work_seq", W), i32p(work_qblk, "work_qblk", W), W, out.data_ptr(),
      out.stride(0), f32p(slopes, "slopes", H), optf(sink, "sink", H), (int)chunk, H, G, dim, vdim,
      BS, grouped, stream());
  TORCH_CHECK(ok, "attn_mix_mfma: no tile for these sizes");
}

bool mixq_mfma_ok(int64_t H, int64_t G, int64_t dim, int64_t vdim, int64_t BS) {
  return rfqmix::mixq_mfma_ok((int)H, (int)G, (int)dim, (int)vdim, (int)BS);
}

void glu_clamped(const Tensor& gu, double limit, double alpha, const Tensor& out) {
  const bool f32 = act_f32(gu, "glu_clamped gate_up");
  const int T = (int)gu.size(0), F = (int)out.size(1);
  TORCH_CHECK(gu.dim() == 2 && out.dim() == 2 && gu.size(1) == 2 * F && out.size(0) == T &&
              gu.stride(1) == 1 && out.stride(1) == 1 && out.scalar_type() == gu.scalar_type(),
              "glu_clamped: gate_up [T, 2F], out [T, F]");
  TORCH_CHECK((F + 255) / 256 <= 65535, "glu_clamped: F too large");
  rfqmix::launch_glu_clamped(f32, gu.data_ptr(), gu.stride(0), out.data_ptr(), out.stride(0), T, F,
                             (float)limit, (float)alpha, stream());
}


// ---- post-norm residual layers, latent norm, wkv, grouped sigmoid routing ----
bool rows2d(const Tensor& t, int64_t T, int64_t n) {
  return t.dim() == 2 && t.size(0) == T && t.size(1) == n && t.stride(1) == 1;
}

void embed_rows(const Tensor& ids, const Tensor& table, const Tensor& out, double scale) {
  const bool f32 = act_f32(table, "embed_rows table");
  const int T = (int)ids.numel(), d = (int)table.size(1);
  TORCH_CHECK(table.dim() == 2 && table.is_contiguous(), "embed_rows: table [V, d]");
  TORCH_CHECK(out.dim() == 2 && out.size(0) == T && out.size(1) == d, "embed_rows: out [T, d]");
  rfqmix::launch_embed_rows(f32, i32p(ids, "ids", T), table.data_ptr(),
                            const_cast<float*>(f32p(out, "out")), T, d, (int)table.size(0),
                            (float)scale, stream());
}

void post_norm_add(const Tensor& y, const Tensor& residual, const Tensor& w, double mult, double eps,
                   const OptT& copy) {
  const bool f32 = act_f32(y, "post_norm_add y");
  TORCH_CHECK(residual.dim() == 2, "post_norm_add: residual [T, d]");
  const int T = (int)residual.size(0), d = (int)residual.size(1);
  TORCH_CHECK(rows2d(y, T, d), "post_norm_add: y [T, d]");
  void* cp = nullptr;
  if (copy.has_value()) {
    TORCH_CHECK(copy->is_cuda() && copy->scalar_type() == at::kBFloat16 && copy->is_contiguous() &&
                rows2d(*copy, T, d), "post_norm_add: copy [T, d] bfloat16");
    cp = copy->data_ptr();
  }
  rfqmix::launch_post_norm_add(f32, y.data_ptr(), y.stride(0),
                               const_cast<float*>(f32p(residual, "residual")), f32p(w, "w", d),
                               (float)mult, (float)eps, cp, T, d, stream());
}

void rms_norm_rows(const Tensor& x, const Tensor& w, double eps, double offset, const Tensor& out) {
  const bool fi = act_f32(x, "rms_norm_rows x"), fo = act_f32(out, "rms_norm_rows out");
  TORCH_CHECK(x.dim() == 2 && x.stride(1) == 1, "rms_norm_rows: x [T, n]");
  const int T = (int)x.size(0), n = (int)x.size(1);
  TORCH_CHECK(rows2d(out, T, n) && out.is_contiguous(), "rms_norm_rows: out [T, n]");
  rfqmix::launch_rms_norm_rows(fi, fo, x.data_ptr(), x.stride(0), f32p(w, "w", n), (float)eps,
                               (float)offset, out.data_ptr(), T, n, stream());
}

void latent_norm_append(const Tensor& x, const Tensor& w, double eps, const Tensor& slots,
                        const Tensor& pool) {
  const bool f32 = act_f32(x, "latent_norm_append x");
  TORCH_CHECK(x.dim() == 2 && x.stride(1) == 1, "latent_norm_append: x [T, R]");
  const int T = (int)x.size(0), R = (int)x.size(1);
  TORCH_CHECK(pool.is_cuda() && pool.dim() == 4 && pool.is_contiguous() && pool.size(1) == 1 &&
              pool.size(3) == R && pool.scalar_type() == x.scalar_type(),
              "latent_norm_append: pool [blocks, 1, BS, R] of x's dtype");
  rfqmix::launch_latent_norm_append(f32, x.data_ptr(), x.stride(0), f32p(w, "w", R), (float)eps,
                                    i32p(slots, "slot_mapping", T), pool.data_ptr(), T, R,
                                    pool.size(0) * pool.size(2), stream());
}

void silu_mul_any(const Tensor& gu, const Tensor& out) {
  const bool f32 = act_f32(gu, "silu_mul_any gate_up");
  const int T = (int)gu.size(0), F = (int)out.size(1);
  TORCH_CHECK(gu.dim() == 2 && gu.size(1) == 2 * F && gu.stride(1) == 1 && rows2d(out, T, F) &&
              out.is_contiguous() && out.scalar_type() == gu.scalar_type(),
              "silu_mul_any: gate_up [T, 2F], out [T, F]");
  rfqmix::launch_silu_mul_any(f32, gu.data_ptr(), gu.stride(0), out.data_ptr(), T, F, stream());
}

void softcap(const Tensor& x, double cap) {
  TORCH_CHECK(cap > 0, "softcap: cap > 0");
  rfqmix::launch_softcap(const_cast<float*>(f32p(x, "logits")), (float)cap, x.numel(), stream());
}

void token_shift_mix(const Tensor& x, const Tensor& mu, const Tensor& prev, const Tensor& row_state,
                     const Tensor& row_back, const Tensor& row_fwd, const Tensor& pos,
                     const Tensor& out) {
  TORCH_CHECK(x.dim() == 2 && mu.dim() == 2 && prev.dim() == 2, "token_shift_mix: x [T, d], mu [S, d], prev [2 slots, d]");
  const int T = (int)x.size(0), d = (int)x.size(1), NS = (int)mu.size(0);
  TORCH_CHECK(mu.size(1) == d && prev.size(1) == d && prev.size(0) % 2 == 0, "token_shift_mix: widths");
  const bool fo = act_f32(out, "token_shift_mix out");
  TORCH_CHECK(out.dim() == 3 && out.is_contiguous() && out.size(0) == NS && out.size(1) == T &&
              out.size(2) == d, "token_shift_mix: out [S, T, d]");
  rfqmix::launch_token_shift_mix(fo, f32p(x, "x"), f32p(mu, "mu"),
                                 const_cast<float*>(f32p(prev, "prev")),
                                 i32p(row_state, "row_state", T), i32p(row_back, "row_back", T),
                                 i32p(row_fwd, "row_fwd", T), i32p(pos, "positions", T),
                                 out.data_ptr(), T, d, NS, (int)prev.size(0) / 2, stream());
}

void wkv_recurrence(const Tensor& r, const Tensor& k, const Tensor& v, const Tensor& zw,
                    const Tensor& w0, const Tensor& u, const Tensor& gate, const Tensor& norm_w,
                    double eps, const Tensor& state, const Tensor& row_state,
                    const Tensor& row_back, const Tensor& row_fwd, const Tensor& pos,
                    const OptT& run_rows, const Tensor& out) {
  const bool f32 = act_f32(r, "wkv_recurrence r");
  TORCH_CHECK(u.dim() == 2, "wkv_recurrence: u [H, N]");
  const int H = (int)u.size(0), N = (int)u.size(1), T = (int)r.size(0);
  const int64_t HN = (int64_t)H * N;
  for (const Tensor* t : {&r, &k, &v, &zw, &gate})
    TORCH_CHECK(t->is_cuda() && rows2d(*t, T, HN) && t->scalar_type() == r.scalar_type(),
                "wkv_recurrence: r, k, v, zw, gate [T, H N] of one dtype");
  TORCH_CHECK(rows2d(out, T, HN) && out.is_contiguous() && out.scalar_type() == r.scalar_type(),
              "wkv_recurrence: out [T, H N]");
  TORCH_CHECK(state.dim() == 4 && state.size(0) % 2 == 0 && state.size(1) == H &&
              state.size(2) == N && state.size(3) == N, "wkv_recurrence: state [2 slots, H, N, N]");
  TORCH_CHECK(rfqmix::wkv_ok(N) && H <= 65535, "wkv_recurrence: head size outside the kernel's range");
  rfqmix::launch_wkv_recurrence(
      f32, r.data_ptr(), k.data_ptr(), v.data_ptr(), zw.data_ptr(), gate.data_ptr(), r.stride(0),
      k.stride(0), v.stride(0), zw.stride(0), gate.stride(0), f32p(w0, "w0", HN), f32p(u, "u", HN),
      f32p(norm_w, "norm_w", HN), (float)eps, const_cast<float*>(f32p(state, "state")),
      i32p(row_state, "row_state", T), i32p(row_back, "row_back", T), i32p(row_fwd, "row_fwd", T),
      i32p(pos, "positions", T), run_rows.has_value() ? i32p(*run_rows, "run_rows", 0) : nullptr,
      run_rows.has_value() ? (int)run_rows->numel() : 0, out.data_ptr(), T, H, N,
      (int)state.size(0) / 2, stream());
}

// Latent attention on MFMA tiles: q [T, H, R] bf16 (the queries carried into the latent space;
// any row and head strides that are multiples of 8), pool [blocks, 1, 32, R] bf16 = keys and
// values, out [T, H R] bf16.
void attn_latent_mfma(const Tensor& q, const Tensor& pool, const Tensor& bt, const Tensor& q_start,
                      const Tensor& q_len, const Tensor& kv_len, const Tensor& work_seq,
                      const Tensor& work_qblk, const Tensor& out, const OptT& sink, double scale) {
  TORCH_CHECK(q.is_cuda() && q.scalar_type() == at::kBFloat16 && q.dim() == 3 && q.stride(2) == 1,
              "attn_latent_mfma: q [T, H, R] bfloat16");
  const int T = (int)q.size(0), H = (int)q.size(1), R = (int)q.size(2);
  TORCH_CHECK(q.stride(0) % 8 == 0 && q.stride(1) % 8 == 0 &&
              reinterpret_cast<uintptr_t>(q.data_ptr()) % 16 == 0, "attn_latent_mfma: q alignment");
  TORCH_CHECK(pool.is_cuda() && pool.scalar_type() == at::kBFloat16 && pool.dim() == 4 &&
              pool.is_contiguous() && pool.size(1) == 1 && pool.size(3) == R,
              "attn_latent_mfma: pool [blocks, 1, BS, R] bfloat16");
  const int BS = (int)pool.size(2), NB = (int)q_len.numel(), W = (int)work_seq.numel();
  TORCH_CHECK(rfqmix::latent_mfma_ok(R, BS), "attn_latent_mfma: sizes outside the tiles");
  TORCH_CHECK(out.is_cuda() && out.scalar_type() == at::kBFloat16 && out.dim() == 2 &&
              out.size(0) == T && out.size(1) == (int64_t)H * R && out.stride(1) == 1 &&
              out.stride(0) % 4 == 0 && reinterpret_cast<uintptr_t>(out.data_ptr()) % 8 == 0,
              "attn_latent_mfma: out [T, H R] bfloat16");
  TORCH_CHECK(bt.dim() == 2 && bt.size(0) == NB, "attn_latent_mfma: block_tables [NB, maxb]");
  TORCH_CHECK(work_qblk.numel() >= W, "attn_latent_mfma: work lists");
  const bool ok = rfqmix::launch_attn_latent_mfma(
      q.data_ptr(), q.stride(0), q.stride(1), pool.data_ptr(), i32p(bt, "block_tables", 0),
      (int)bt.size(1), i32p(q_start, "q_start", NB), i32p(q_len, "q_len", NB),
      i32p(kv_len, "kv_len", NB), i32p(work_seq, "work_seq", W), i32p(work_qblk, "work_qblk", W), W,
      out.data_ptr(), out.stride(0), optf(sink, "sink", H), (float)scale, H, R, BS, stream());
  TORCH_CHECK(ok, "attn_latent_mfma: no tile for these sizes");
}

bool latent_mfma_ok(int64_t R, int64_t BS) { return rfqmix::latent_mfma_ok((int)R, (int)BS); }

void moe_route_grouped(const Tensor& z, const Tensor& corr, int64_t top, int64_t groups,
                       int64_t keep, const Tensor& ids, const Tensor& weights) {
  TORCH_CHECK(z.dim() == 2, "moe_route_grouped: z [T, E]");
  const int T = (int)z.size(0), E = (int)z.size(1);
  TORCH_CHECK(top >= 1 && top <= E, "moe_route_grouped: top");
  TORCH_CHECK(groups == 0 || (groups <= 64 && E % groups == 0 && keep >= 1 && keep <= groups &&
                              top <= keep * (E / groups)), "moe_route_grouped: groups");
  TORCH_CHECK(ids.is_cuda() && ids.scalar_type() == at::kInt && ids.is_contiguous() &&
              ids.numel() == (int64_t)T * top, "moe_route_grouped: ids [T, top] int32");
  rfqmix::launch_moe_route_grouped(f32p(z, "z"), f32p(corr, "correction", E), T, E, (int)top,
                                   (int)groups, (int)keep, ids.data_ptr<int32_t>(),
                                   const_cast<float*>(f32p(weights, "weights", (int64_t)T * top)),
                                   stream());
}

void moe_pair_up(const Tensor& h, const Tensor& ids, const Tensor& w13, const Tensor& act) {
  const bool f32 = act_f32(h, "moe_pair_up h");
  TORCH_CHECK(h.dim() == 2 && h.stride(1) == 1 && w13.dim() == 3 && w13.is_contiguous() &&
              w13.is_cuda() && w13.scalar_type() == h.scalar_type() && w13.size(2) == h.size(1) &&
              w13.size(1) % 2 == 0, "moe_pair_up: h [T, d], w13 [E, 2F, d]");
  const int T = (int)h.size(0), d = (int)h.size(1), E = (int)w13.size(0), F = (int)w13.size(1) / 2;
  const int pairs = (int)ids.numel();
  TORCH_CHECK(T > 0 ? pairs % T == 0 : pairs == 0, "moe_pair_up: ids [T, top]");
  TORCH_CHECK(rows2d(act, pairs, F) && act.is_contiguous() && act.scalar_type() == h.scalar_type(),
              "moe_pair_up: act [T top, F]");
  TORCH_CHECK((int64_t)d * 4 <= 64 * 1024 && (F + 63) / 64 <= 65535, "moe_pair_up: sizes");
  rfqmix::launch_moe_pair_up(f32, h.data_ptr(), h.stride(0), i32p(ids, "ids", pairs), w13.data_ptr(),
                             act.data_ptr(), pairs, T > 0 ? pairs / T : 1, d, F, E, stream());
}

void moe_pair_down(const Tensor& act, const Tensor& ids, const Tensor& weights, const Tensor& w2,
                   const OptT& base, const Tensor& out) {
  const bool f32 = act_f32(act, "moe_pair_down act");
  TORCH_CHECK(out.dim() == 2 && w2.dim() == 3 && w2.is_contiguous() && w2.is_cuda() &&
              w2.scalar_type() == act.scalar_type() && w2.size(1) == out.size(1),
              "moe_pair_down: w2 [E, d, F], out [T, d]");
  const int T = (int)out.size(0), d = (int)out.size(1), E = (int)w2.size(0), F = (int)w2.size(2);
  const int pairs = (int)ids.numel(), top = T > 0 ? pairs / T : 1;
  TORCH_CHECK(pairs == T * top && rows2d(act, pairs, F) && act.is_contiguous(), "moe_pair_down: act [T top, F]");
  TORCH_CHECK((int64_t)top * F * 4 <= 160 * 1024 - 256 && (d + 63) / 64 <= 65535, "moe_pair_down: sizes");
  const void* bp = nullptr;
  int64_t bs = 0;
  if (base.has_value()) {
    TORCH_CHECK(base->is_cuda() && rows2d(*base, T, d) && base->scalar_type() == act.scalar_type(),
                "moe_pair_down: base [T, d]");
    bp = base->data_ptr();
    bs = base->stride(0);
  }
  rfqmix::launch_moe_pair_down(f32, act.data_ptr(), i32p(ids, "ids", pairs),
                               f32p(weights, "weights", pairs), w2.data_ptr(), bp, bs,
                               const_cast<float*>(f32p(out, "out")), T, top, d, F, E, stream());
}

// ---- parallel-sublayer layers: residual, rotary differential attention, linear recurrences
void residual_add_norm(const Tensor& x, const OptT& y1, const OptT& y2, const OptT& shift,
                       const OptT& w, double eps, double offset, const OptT& out, double mult) {
  TORCH_CHECK(x.dim() == 2, "residual_add_norm: x [T, d]");
  const int T = (int)x.size(0), d = (int)x.size(1);
  const void* yp[2] = {nullptr, nullptr};
  int64_t ys[2] = {0, 0};
  bool yf[2] = {true, true};
  const OptT* yy[2] = {&y1, &y2};
  for (int i = 0; i < 2; ++i)
    if (yy[i]->has_value()) {
      const Tensor& y = **yy[i];
      yf[i] = act_f32(y, "residual_add_norm y");
      TORCH_CHECK(rows2d(y, T, d), "residual_add_norm: y [T, d]");
      yp[i] = y.data_ptr();
      ys[i] = y.stride(0);
    }
  bool of32 = true;
  void* op = nullptr;
  if (w.has_value()) {
    TORCH_CHECK(out.has_value(), "residual_add_norm: a norm weight needs out");
    of32 = act_f32(*out, "residual_add_norm out");
    TORCH_CHECK(rows2d(*out, T, d) && out->is_contiguous(), "residual_add_norm: out [T, d]");
    op = out->data_ptr();
  }
  rfqmix::launch_residual_add_norm(of32, const_cast<float*>(f32p(x, "x")), yp[0], ys[0], yf[0],
                                   yp[1], ys[1], yf[1], optf(shift, "shift", d), optf(w, "w", d),
                                   (float)eps, (float)offset, op, T, d, (float)mult, stream());
}

void rotary_append(const Tensor& qkv, const Tensor& pos, const Tensor& inv_freq,
                   const Tensor& slots, const Tensor& k_cache, const Tensor& v_cache, int64_t H,
                   int64_t G, int64_t maps, int64_t dim, int64_t vdim, const Tensor& q_out) {
  const bool f32 = act_f32(qkv, "rotary_append qkv");
  TORCH_CHECK(qkv.dim() == 2 && qkv.stride(1) == 1, "rotary_append: qkv [T, N]");
  const int T = (int)qkv.size(0);
  const int64_t kw = maps * dim;
  TORCH_CHECK(H >= 1 && G >= 1 && maps >= 1 && dim >= 1 && vdim >= 1 &&
              qkv.size(1) >= (H + G) * kw + G * vdim, "rotary_append: qkv narrower than q | k | v");
  TORCH_CHECK(k_cache.is_cuda() && v_cache.is_cuda() && k_cache.scalar_type() == qkv.scalar_type() &&
              v_cache.scalar_type() == qkv.scalar_type() && k_cache.is_contiguous() &&
              v_cache.is_contiguous() && k_cache.dim() == 4 && v_cache.dim() == 4 &&
              k_cache.size(1) == G && k_cache.size(3) == kw && v_cache.size(1) == G &&
              v_cache.size(3) == vdim && v_cache.size(0) == k_cache.size(0) &&
              v_cache.size(2) == k_cache.size(2),
              "rotary_append: k_cache [blocks, G, BS, maps dim], v_cache [blocks, G, BS, vdim]");
  const int nrot = (int)inv_freq.numel();
  TORCH_CHECK(2 * nrot <= dim && dim <= 8192, "rotary_append: more rotated dimensions than a map has");
  TORCH_CHECK(q_out.dim() == 3 && q_out.size(0) == T && q_out.size(1) == H && q_out.size(2) == kw,
              "rotary_append: q_out [T, H, maps dim]");
  const float* fr = nrot > 0 ? f32p(inv_freq, "inv_freq") : nullptr;
  rfqmix::launch_rotary_append(f32, qkv.data_ptr(), qkv.stride(0), i32p(pos, "positions", T), fr,
                               nrot, i32p(slots, "slots", T), k_cache.data_ptr(),
                               v_cache.data_ptr(), T, (int)H, (int)G, (int)maps, (int)dim,
                               (int)vdim, (int)k_cache.size(2),
                               k_cache.size(0) * k_cache.size(2),
                               const_cast<float*>(f32p(q_out, "q_out")), stream());
}

void attn_diff_window(const Tensor& q, const Tensor& k_cache, const Tensor& v_cache,
                      const Tensor& bt, const Tensor& q_start, const Tensor& q_len,
                      const Tensor& kv_len, const Tensor& work_seq, const Tensor& work_qblk,
                      const Tensor& gate, const Tensor& out, double scale, int64_t window,
                      double lam, double eps, double out_mult, int64_t short_rows, bool mfma) {
  const bool f32 = act_f32(k_cache, "attn_diff_window k_cache");
  TORCH_CHECK(q.dim() == 3 && q.size(2) % 2 == 0, "attn_diff_window: q [T, H, 2 dim]");
  const int T = (int)q.size(0), H = (int)q.size(1), dim = (int)q.size(2) / 2;
  TORCH_CHECK(k_cache.dim() == 4 && v_cache.dim() == 4 && k_cache.is_contiguous() &&
              v_cache.is_contiguous() && v_cache.is_cuda() &&
              v_cache.scalar_type() == k_cache.scalar_type() && k_cache.size(3) == 2 * dim &&
              v_cache.size(1) == k_cache.size(1) && v_cache.size(0) == k_cache.size(0) &&
              v_cache.size(2) == k_cache.size(2),
              "attn_diff_window: k_cache [blocks, G, BS, 2 dim], v_cache [blocks, G, BS, vdim]");
  const int G = (int)k_cache.size(1), BS = (int)k_cache.size(2), vdim = (int)v_cache.size(3);
  TORCH_CHECK(G >= 1 && H % G == 0 && H <= 65535, "attn_diff_window: H a multiple of G");
  const int NB = (int)q_len.numel(), W = (int)work_seq.numel();
  TORCH_CHECK(bt.dim() == 2 && bt.size(0) == NB, "attn_diff_window: block_tables [NB, maxb]");
  TORCH_CHECK(work_qblk.numel() >= W, "attn_diff_window: work lists");
  TORCH_CHECK(gate.is_cuda() && gate.scalar_type() == k_cache.scalar_type() && rows2d(gate, T, H),
              "attn_diff_window: gate [T, H] in the cache's type");
  TORCH_CHECK(out.is_cuda() && out.scalar_type() == k_cache.scalar_type() &&
              rows2d(out, T, (int64_t)H * vdim), "attn_diff_window: out [T, H vdim]");
  TORCH_CHECK(window >= 0, "attn_diff_window: window");
  if (short_rows > 0) {
    // sequences of at most short_rows rows each (decode section): one workgroup per
    // (sequence, row, key/value head); falls through to the work items if the LDS is too small
    TORCH_CHECK(short_rows <= 65535 && G <= 65535, "attn_diff_window: short_rows");
    const int kt = rfqmix::launch_attn_diff_decode(
        f32, f32p(q, "q"), k_cache.data_ptr(), v_cache.data_ptr(), i32p(bt, "block_tables", 0),
        (int)bt.size(1), i32p(q_start, "q_start", NB), i32p(q_len, "q_len", NB),
        i32p(kv_len, "kv_len", NB), NB, (int)short_rows, gate.data_ptr(), gate.stride(0),
        out.data_ptr(), out.stride(0), (float)scale, (int)window, (float)lam, (float)eps,
        (float)out_mult, H, G, dim, vdim, BS, stream());
    if (kt > 0) return;
  }
  if (mfma && !f32 && rfqmix::diff_mfma_ok(dim, vdim, BS)) {
    // bf16 pages with sizes of the MFMA tiles; 16-byte rows of q and of the pages
    TORCH_CHECK(reinterpret_cast<uintptr_t>(q.data_ptr()) % 16 == 0 &&
                reinterpret_cast<uintptr_t>(k_cache.data_ptr()) % 16 == 0 &&
                reinterpret_cast<uintptr_t>(v_cache.data_ptr()) % 16 == 0,
                "attn_diff_window: alignment of q and the pages");
    rfqmix::launch_attn_diff_mfma(
        f32p(q, "q"), k_cache.data_ptr(), v_cache.data_ptr(), i32p(bt, "block_tables", 0),
        (int)bt.size(1), i32p(q_start, "q_start", NB), i32p(q_len, "q_len", NB),
        i32p(kv_len, "kv_len", NB), i32p(work_seq, "work_seq", W), i32p(work_qblk, "work_qblk", W),
        W, gate.data_ptr(), gate.stride(0), out.data_ptr(), out.stride(0), (float)scale,
        (int)window, (float)lam, (float)eps, (float)out_mult, H, G, dim, vdim, BS, stream());
    return;
  }
  const bool ok = rfqmix::launch_attn_diff_window(
      f32, f32p(q, "q"), k_cache.data_ptr(), v_cache.data_ptr(), i32p(bt, "block_tables", 0),
      (int)bt.size(1), i32p(q_start, "q_start", NB), i32p(q_len, "q_len", NB),
      i32p(kv_len, "kv_len", NB), i32p(work_seq, "work_seq", W), i32p(work_qblk, "work_qblk", W), W,
      gate.data_ptr(), gate.stride(0), out.data_ptr(), out.stride(0), (float)scale, (int)window,
      (float)lam, (float)eps, (float)out_mult, H, G, dim, vdim, BS, stream());
  TORCH_CHECK(ok, "attn_diff_window: value size too large for the LDS");
}

bool diff_mfma_ok(int64_t dim, int64_t vdim, int64_t BS) {
  return rfqmix::diff_mfma_ok((int)dim, (int)vdim, (int)BS);
}

// ---- projection norms + half-split rotation, attention with kept first tokens, xIELU
void qk_norm_rotary_append(const Tensor& proj, const OptT& bias, const OptT& q_norm_w,
                           const OptT& k_norm_w, bool norm_all, int64_t k_norm_n, double eps,
                           const Tensor& pos, const Tensor& inv_freq, double rot_mult,
                           int64_t q_rot_off, int64_t k_rot_off, const Tensor& slots,
                           const OptT& k_cache, const OptT& v_cache, int64_t H, int64_t G,
                           int64_t qw, int64_t kw, int64_t vdim, int64_t v_mode,
                           const Tensor& q_out) {
  const bool f32 = act_f32(proj, "qk_norm_rotary_append proj");
  TORCH_CHECK(proj.dim() == 2 && proj.stride(1) == 1, "qk_norm_rotary_append: proj [T, N]");
  const int T = (int)proj.size(0);
  TORCH_CHECK(H >= 1 && G >= 0 && qw >= 1 && kw >= 1 && vdim >= 0 && v_mode >= 0 && v_mode <= 2,
              "qk_norm_rotary_append: sizes");
  const int64_t W = H * qw + G * kw + (v_mode == 0 ? G * vdim : 0);
  TORCH_CHECK(proj.size(1) >= W, "qk_norm_rotary_append: proj narrower than q | k | v");
  TORCH_CHECK(v_mode != 1 || vdim == kw, "qk_norm_rotary_append: values that are the keys have their width");
  const int nrot = (int)inv_freq.numel();
  TORCH_CHECK(q_rot_off >= 0 && k_rot_off >= 0 && q_rot_off + 2 * nrot <= qw &&
              (G == 0 || k_rot_off + 2 * nrot <= kw),
              "qk_norm_rotary_append: the rotated entries lie outside a head");
  TORCH_CHECK(k_norm_n >= 0 && k_norm_n <= kw && (!norm_all || k_norm_n == kw),
              "qk_norm_rotary_append: k_norm_n");
  const int64_t nqw = norm_all ? H * qw : qw, nkw = norm_all ? G * kw : k_norm_n;
  void *kp = nullptr, *vp = nullptr;
  int BS = 1;
  int64_t pool_slots = 0;
  if (G > 0) {
    TORCH_CHECK(k_cache.has_value(), "qk_norm_rotary_append: key heads need pages");
    const Tensor& kc = *k_cache;
    TORCH_CHECK(kc.is_cuda() && kc.scalar_type() == proj.scalar_type() && kc.is_contiguous() &&
                kc.dim() == 4 && kc.size(1) == G && kc.size(3) == kw,
                "qk_norm_rotary_append: k_cache [blocks, G, BS, kw]");
    kp = kc.data_ptr();
    BS = (int)kc.size(2);
    pool_slots = kc.size(0) * kc.size(2);
    if (v_mode != 2) {
      TORCH_CHECK(v_cache.has_value(), "qk_norm_rotary_append: values need pages");
      const Tensor& vc = *v_cache;
      TORCH_CHECK(vc.is_cuda() && vc.scalar_type() == proj.scalar_type() && vc.is_contiguous() &&
                  vc.dim() == 4 && vc.size(0) == kc.size(0) && vc.size(1) == G &&
                  vc.size(2) == kc.size(2) && vc.size(3) == vdim,
                  "qk_norm_rotary_append: v_cache [blocks, G, BS, vdim]");
      vp = vc.data_ptr();
    }
  }
  TORCH_CHECK(q_out.dim() == 3 && q_out.size(0) == T && q_out.size(1) == H && q_out.size(2) == qw,
              "qk_norm_rotary_append: q_out [T, H, qw]");
  const float* fr = nrot > 0 ? f32p(inv_freq, "inv_freq") : nullptr;
  const bool ok = rfqmix::launch_qk_norm_rotary_append(
      f32, proj.data_ptr(), proj.stride(0), optf(bias, "bias", W), optf(q_norm_w, "q_norm_w", nqw),
      (G > 0 && k_norm_w.has_value()) ? f32p(*k_norm_w, "k_norm_w", nkw) : nullptr, norm_all,
      (int)k_norm_n, (float)eps, i32p(pos, "positions", T), fr, nrot, (float)rot_mult,
      (int)q_rot_off, (int)k_rot_off, i32p(slots, "slots", T), kp, vp, T, (int)H, (int)G, (int)qw,
      (int)kw, (int)vdim, (int)v_mode, BS, pool_slots, const_cast<float*>(f32p(q_out, "q_out")),
      stream());
  TORCH_CHECK(ok, "qk_norm_rotary_append: a row does not fit the LDS");
}

void attn_keep_window(const Tensor& q, const Tensor& k_cache, const Tensor& v_cache, int64_t vdim,
                      const Tensor& bt, const Tensor& q_start, const Tensor& q_len,
                      const Tensor& kv_len, const Tensor& work_seq, const Tensor& work_qblk,
                      const OptT& head_bias, const OptT& gate, const Tensor& out, double scale,
                      int64_t window, int64_t keep_first, bool sigmoid, int64_t short_rows,
                      bool mfma) {
  const bool f32 = act_f32(k_cache, "attn_keep_window k_cache");
  TORCH_CHECK(q.dim() == 3, "attn_keep_window: q [T, H, E]");
  const int T = (int)q.size(0), H = (int)q.size(1), E = (int)q.size(2);
  TORCH_CHECK(k_cache.dim() == 4 && v_cache.dim() == 4 && k_cache.is_contiguous() &&
              v_cache.is_contiguous() && v_cache.is_cuda() &&
              v_cache.scalar_type() == k_cache.scalar_type() && k_cache.size(3) == E &&
              v_cache.size(1) == k_cache.size(1) && v_cache.size(0) == k_cache.size(0) &&
              v_cache.size(2) == k_cache.size(2) && vdim >= 1 && v_cache.size(3) >= vdim,
              "attn_keep_window: k_cache [blocks, G, BS, E], v_cache [blocks, G, BS, >= vdim]");
  const int G = (int)k_cache.size(1), BS = (int)k_cache.size(2);
  const int64_t vrs = v_cache.size(3);
  TORCH_CHECK(G >= 1 && H % G == 0 && H <= 65535, "attn_keep_window: H a multiple of G");
  const int NB = (int)q_len.numel(), W = (int)work_seq.numel();
  TORCH_CHECK(bt.dim() == 2 && bt.size(0) == NB, "attn_keep_window: block_tables [NB, maxb]");
  TORCH_CHECK(work_qblk.numel() >= W, "attn_keep_window: work lists");
  TORCH_CHECK(!sigmoid || head_bias.has_value(), "attn_keep_window: sigmoid weights need a bias");
  const void* gp = nullptr;
  int64_t gs = 0;
  if (gate.has_value()) {
    TORCH_CHECK(gate->is_cuda() && gate->scalar_type() == k_cache.scalar_type() &&
                rows2d(*gate, T, H), "attn_keep_window: gate [T, H] in the cache's type");
    gp = gate->data_ptr();
    gs = gate->stride(0);
  }
  TORCH_CHECK(out.is_cuda() && out.scalar_type() == k_cache.scalar_type() &&
              rows2d(out, T, (int64_t)H * vdim), "attn_keep_window: out [T, H vdim]");
  TORCH_CHECK(window >= 0 && keep_first >= 0, "attn_keep_window: window, keep_first");
  const float* hb = optf(head_bias, "head_bias", H);
  // the values are the leading entries of the key pages themselves
  const bool shared = v_cache.data_ptr() == k_cache.data_ptr() && vrs == E;
  const bool tiles = mfma && !f32 && rfqmix::keep_mfma_ok(E, (int)vdim, BS, shared) &&
                     vrs % 8 == 0 && out.stride(0) % 4 == 0 &&
                     reinterpret_cast<uintptr_t>(q.data_ptr()) % 16 == 0 &&
                     reinterpret_cast<uintptr_t>(k_cache.data_ptr()) % 16 == 0 &&
                     reinterpret_cast<uintptr_t>(v_cache.data_ptr()) % 16 == 0 &&
                     reinterpret_cast<uintptr_t>(out.data_ptr()) % 8 == 0;
  TORCH_CHECK(short_rows >= 0 && short_rows <= 65535 && G <= 65535, "attn_keep_window: short_rows");
  if (short_rows > 0 && !(tiles && H / G >= 16)) {
    // sequences of at most short_rows rows each (decode section): one workgroup per
    // (sequence, key/value head) on the FMA kernel; groups of 16 heads or more fill the MFMA
    // tiles' columns and run there; falls through if the LDS is too small
    const int kt = rfqmix::launch_attn_keep_decode(
        f32, f32p(q, "q"), k_cache.data_ptr(), v_cache.data_ptr(), vrs, i32p(bt, "block_tables", 0),
        (int)bt.size(1), i32p(q_start, "q_start", NB), i32p(q_len, "q_len", NB),
        i32p(kv_len, "kv_len", NB), NB, (int)short_rows, hb, gp, gs, out.data_ptr(), out.stride(0),
        (float)scale, (int)window, (int)keep_first, sigmoid, H, G, E, (int)vdim, BS, stream());
    if (kt > 0) return;
  }
  if (tiles) {
    rfqmix::launch_attn_keep_mfma(
        f32p(q, "q"), k_cache.data_ptr(), v_cache.data_ptr(), vrs, i32p(bt, "block_tables", 0),
        (int)bt.size(1), i32p(q_start, "q_start", NB), i32p(q_len, "q_len", NB),
        i32p(kv_len, "kv_len", NB), i32p(work_seq, "work_seq", W), i32p(work_qblk, "work_qblk", W),
        W, hb, gp, gs, out.data_ptr(), out.stride(0), (float)scale, (int)window, (int)keep_first,
        sigmoid, H, G, E, (int)vdim, BS, shared, NB, (int)short_rows, stream());
    return;
  }
  const bool ok = rfqmix::launch_attn_keep_window(
      f32, f32p(q, "q"), k_cache.data_ptr(), v_cache.data_ptr(), vrs, i32p(bt, "block_tables", 0),
      (int)bt.size(1), i32p(q_start, "q_start", NB), i32p(q_len, "q_len", NB),
      i32p(kv_len, "kv_len", NB), i32p(work_seq, "work_seq", W), i32p(work_qblk, "work_qblk", W), W,
      hb, gp, gs, out.data_ptr(), out.stride(0), (float)scale, (int)window, (int)keep_first,
      sigmoid, H, G, E, (int)vdim, BS, stream());
  TORCH_CHECK(ok, "attn_keep_window: value size too large for the LDS");
}

bool keep_mfma_ok(int64_t E, int64_t vdim, int64_t BS, bool shared) {
  return rfqmix::keep_mfma_ok((int)E, (int)vdim, (int)BS, shared);
}

void xielu_rows(const Tensor& x, double ap, double an, const Tensor& out) {
  const bool f32 = act_f32(x, "xielu_rows x");
  TORCH_CHECK(x.dim() == 2 && out.dim() == 2 && out.sizes() == x.sizes() && x.stride(1) == 1 &&
              out.stride(1) == 1 && out.is_cuda() && out.scalar_type() == x.scalar_type(),
              "xielu_rows: x, out [T, F] of one type");
  TORCH_CHECK((x.size(1) + 255) / 256 <= 65535, "xielu_rows: F too large");
  rfqmix::launch_xielu_rows(f32, x.data_ptr(), x.stride(0), out.data_ptr(), out.stride(0),
                            (int)x.size(0), (int)x.size(1), (float)ap, (float)an, stream());
}

void conv_act_heads(const Tensor& x, const Tensor& w, const Tensor& state, const Tensor& row_state,
                    const Tensor& row_back, const Tensor& row_fwd, const Tensor& pos,
                    int64_t n_unit, int64_t dim, double unit_eps, const Tensor& out) {
  const bool f32 = act_f32(x, "conv_act_heads x");
  TORCH_CHECK(x.dim() == 2 && x.stride(1) == 1 && w.dim() == 2 && state.dim() == 3,
              "conv_act_heads: x [T, C], w [C, taps], state [2S, taps-1, C]");
  const int T = (int)x.size(0), C = (int)x.size(1), taps = (int)w.size(1);
  TORCH_CHECK(w.size(0) == C && taps >= 1, "conv_act_heads: w [C, taps]");
  TORCH_CHECK(state.size(0) % 2 == 0 && state.size(1) == taps - 1 && state.size(2) == C,
              "conv_act_heads: state [2S, taps-1, C]");
  TORCH_CHECK(n_unit >= 0 && dim >= 1 && n_unit * dim <= C, "conv_act_heads: unit heads");
  TORCH_CHECK(dim <= 8192 && (C + 255) / 256 <= 65535, "conv_act_heads: sizes");
  TORCH_CHECK(out.dim() == 2 && out.size(0) == T && out.size(1) == C, "conv_act_heads: out [T, C]");
  rfqmix::launch_conv_act_heads(f32, x.data_ptr(), x.stride(0), f32p(w, "w"),
                                const_cast<float*>(f32p(state, "state")),
                                i32p(row_state, "row_state", T), i32p(row_back, "row_back", T),
                                i32p(row_fwd, "row_fwd", T), i32p(pos, "positions", T),
                                const_cast<float*>(f32p(out, "out")), T, C, taps,
                                (int)state.size(0) / 2, (int)n_unit, (int)dim, (float)unit_eps,
                                stream());
}

void gated_linear_recurrence(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& z,
                             const Tensor& rate, const Tensor& zbias, double zsign,
                             const OptT& beta, const Tensor& gate, bool gate_sigmoid,
                             const Tensor& norm_w, double eps, double q_scale, const Tensor& state,
                             const Tensor& row_state, const Tensor& row_back, const Tensor& row_fwd,
                             const Tensor& pos, const OptT& run_rows, const Tensor& out,
                             bool decay_ready, const OptT& raw) {
  const bool in_f32 = act_f32(q, "gated_linear_recurrence q");
  const bool a_f32 = act_f32(out, "gated_linear_recurrence out");
  TORCH_CHECK(state.dim() == 4 && state.size(0) % 2 == 0,
              "gated_linear_recurrence: state [2 slots, H, dim, vdim]");
  const int H = (int)state.size(1), dim = (int)state.size(2), vdim = (int)state.size(3);
  TORCH_CHECK(q.dim() == 3 && k.dim() == 3 && v.dim() == 3 && q.stride(2) == 1 &&
              k.stride(2) == 1 && v.stride(2) == 1 && k.scalar_type() == q.scalar_type() &&
              v.scalar_type() == q.scalar_type() && k.is_cuda() && v.is_cuda(),
              "gated_linear_recurrence: q, k [T, Hq, dim], v [T, H, vdim] of one type");
  const int T = (int)q.size(0), Hq = (int)q.size(1);
  TORCH_CHECK(Hq >= 1 && H % Hq == 0 && q.size(2) == dim && k.size(0) == T && k.size(1) == Hq &&
              k.size(2) == dim && v.size(0) == T && v.size(1) == H && v.size(2) == vdim &&
              q.stride(1) == dim && k.stride(1) == dim && v.stride(1) == vdim,
              "gated_linear_recurrence: head counts and sizes of q, k, v");
  TORCH_CHECK(z.is_cuda() && z.scalar_type() == at::kFloat && rows2d(z, T, (int64_t)H * dim),
              "gated_linear_recurrence: z [T, H dim] float32");
  TORCH_CHECK(gate.is_cuda() && gate.scalar_type() == out.scalar_type() &&
              rows2d(gate, T, (int64_t)H * vdim), "gated_linear_recurrence: gate [T, H vdim]");
  TORCH_CHECK(rows2d(out, T, (int64_t)H * vdim) && out.is_contiguous(),
              "gated_linear_recurrence: out [T, H vdim]");
  TORCH_CHECK(rfqmix::linrec_ok(dim, vdim) && H <= 65535,
              "gated_linear_recurrence: head sizes outside the kernel's range");
  rfqmix::LinrecArgs a;
  a.q = q.data_ptr(); a.k = k.data_ptr(); a.v = v.data_ptr();
  a.qs = q.stride(0); a.ks = k.stride(0); a.vs = v.stride(0);
  a.z = z.data_ptr<float>(); a.zs = z.stride(0);
  a.rate = f32p(rate, "rate", H); a.zbias = f32p(zbias, "zbias", (int64_t)H * dim);
  a.zsign = (float)zsign;
  a.beta = nullptr; a.bs = 0;
  if (beta.has_value()) {
    TORCH_CHECK(beta->is_cuda() && beta->scalar_type() == out.scalar_type() && rows2d(*beta, T, H),
                "gated_linear_recurrence: beta [T, H]");
    a.beta = beta->data_ptr(); a.bs = beta->stride(0);
  }
  a.gate = gate.data_ptr(); a.gs = gate.stride(0); a.gate_sigmoid = gate_sigmoid ? 1 : 0;
  a.norm_w = f32p(norm_w, "norm_w", vdim);
  a.eps = (float)eps; a.q_scale = (float)q_scale;
  a.decay_ready = decay_ready ? 1 : 0;
  a.raw = raw.has_value() ? const_cast<float*>(f32p(*raw, "raw", (int64_t)T * H * vdim)) : nullptr;
  a.state = const_cast<float*>(f32p(state, "state"));
  a.row_state = i32p(row_state, "row_state", T); a.row_back = i32p(row_back, "row_back", T);
  a.row_fwd = i32p(row_fwd, "row_fwd", T); a.pos = i32p(pos, "positions", T);
  a.run_rows = run_rows.has_value() ? i32p(*run_rows, "run_rows", 0) : nullptr;
  a.runs = run_rows.has_value() ? (int)run_rows->numel() : 0;
  a.out = out.data_ptr();
  a.T = T; a.H = H; a.rep = H / Hq; a.dim = dim; a.vdim = vdim; a.slots = (int)state.size(0) / 2;
  rfqmix::launch_gated_linrec(in_f32, a_f32, beta.has_value(), a, stream());
}

void decay_from_logits(const Tensor& z, const Tensor& rate, const Tensor& zbias, double zsign,
                       int64_t dim) {
  TORCH_CHECK(z.is_cuda() && z.scalar_type() == at::kFloat && z.dim() == 2 && z.stride(1) == 1 &&
              dim >= 1 && z.size(1) % dim == 0, "decay_from_logits: z [T, H dim] float32");
  const int H = (int)(z.size(1) / dim);
  TORCH_CHECK((z.size(1) + 1023) / 1024 <= 65535, "decay_from_logits: too wide");
  rfqmix::launch_decay_from_logits(z.data_ptr<float>(), z.stride(0), f32p(rate, "rate", H),
                                   f32p(zbias, "zbias", z.size(1)), (float)zsign, (int)z.size(0), H,
                                   (int)dim, stream());
}

void moe_route_topk(const Tensor& z, const OptT& bias, int64_t top, const Tensor& ids,
                    const Tensor& weights) {
  TORCH_CHECK(z.dim() == 2, "moe_route_topk: z [T, E]");
  const int T = (int)z.size(0), E = (int)z.size(1);
  TORCH_CHECK(top >= 1 && top <= E, "moe_route_topk: top");
  TORCH_CHECK(ids.is_cuda() && ids.scalar_type() == at::kInt && ids.is_contiguous() &&
              ids.numel() == (int64_t)T * top, "moe_route_topk: ids [T, top] int32");
  rfqmix::launch_moe_route_topk(f32p(z, "z"), optf(bias, "bias", E), T, E, (int)top,
                                ids.data_ptr<int32_t>(),
                                const_cast<float*>(f32p(weights, "weights", (int64_t)T * top)),
                                stream());
}

void gelu_rows(const Tensor& x, const Tensor& out) {
  const bool f32 = act_f32(x, "gelu_rows x");
  TORCH_CHECK(x.dim() == 2 && x.stride(1) == 1 && out.is_cuda() &&
              out.scalar_type() == x.scalar_type() && rows2d(out, x.size(0), x.size(1)),
              "gelu_rows: x, out [T, F] of one type");
  rfqmix::launch_gelu_rows(f32, x.data_ptr(), x.stride(0), out.data_ptr(), out.stride(0),
                           (int)x.size(0), (int)x.size(1), stream());
}

}  // namespace

TORCH_LIBRARY(rfq_mix, m) {
  m.def("embed_sinusoid(Tensor ids, Tensor pos, Tensor table, Tensor inv_freq, float scale, Tensor(a!) out) -> ()");
  m.def("sandwich_norm(Tensor? y, Tensor(a!) residual, Tensor? w_post, Tensor? gain, Tensor w_pre, float eps, Tensor(b!) out) -> ()");
  m.def("canon_conv(Tensor h, Tensor w, Tensor(a!) state, Tensor row_state, Tensor row_back, Tensor row_fwd, Tensor pos, Tensor(b!) out) -> ()");
  m.def("head_norm_append(Tensor qkv, Tensor q_w, Tensor k_w, float eps, Tensor slots, Tensor(a!) k_cache, Tensor(b!) v_cache, int H, int G, int dim, int vdim, Tensor(c!) qn, Tensor? ts, Tensor(d!)? qmix, int mix_from) -> ()");
  m.def("attn_talk_decode(Tensor qn, Tensor k_cache, Tensor v_cache, Tensor bt, Tensor q_start, Tensor q_len, Tensor kv_len, Tensor(a!) out, Tensor slopes, Tensor? talk, Tensor? sink, float scale, int chunk, int max_rows) -> ()");
  m.def("attn_mixq_prefill(Tensor qmix, Tensor k_cache, Tensor v_cache, Tensor bt, Tensor q_start, Tensor q_len, Tensor kv_len, Tensor work_seq, Tensor work_qblk, Tensor(a!) out, Tensor slopes, Tensor? sink, int chunk, int qblk) -> ()");
  m.def("attn_mix_mfma(Tensor qn, Tensor ts, Tensor k_cache, Tensor v_cache, Tensor bt, Tensor q_start, Tensor q_len, Tensor kv_len, Tensor work_seq, Tensor work_qblk, Tensor(a!) out, Tensor slopes, Tensor? sink, int chunk, bool grouped) -> ()");
  m.def("glu_clamped(Tensor gate_up, float limit, float alpha, Tensor(a!) out) -> ()");
  m.def("mixq_mfma_ok", &mixq_mfma_ok);
  m.def("latent_mfma_ok", &latent_mfma_ok);
  m.def("attn_latent_mfma(Tensor q, Tensor pool, Tensor bt, Tensor q_start, Tensor q_len, Tensor kv_len, Tensor work_seq, Tensor work_qblk, Tensor(a!) out, Tensor? sink, float scale) -> ()");
  m.def("embed_rows(Tensor ids, Tensor table, Tensor(a!) out, float scale) -> ()");
  m.def("post_norm_add(Tensor y, Tensor(a!) residual, Tensor w, float mult, float eps, Tensor(b!)? copy) -> ()");
  m.def("rms_norm_rows(Tensor x, Tensor w, float eps, float offset, Tensor(a!) out) -> ()");
  m.def("latent_norm_append(Tensor x, Tensor w, float eps, Tensor slots, Tensor(a!) pool) -> ()");
  m.def("silu_mul_any(Tensor gate_up, Tensor(a!) out) -> ()");
  m.def("softcap(Tensor(a!) x, float cap) -> ()");
  m.def("token_shift_mix(Tensor x, Tensor mu, Tensor(a!) prev, Tensor row_state, Tensor row_back, Tensor row_fwd, Tensor pos, Tensor(b!) out) -> ()");
  m.def("wkv_recurrence(Tensor r, Tensor k, Tensor v, Tensor zw, Tensor w0, Tensor u, Tensor gate, Tensor norm_w, float eps, Tensor(a!) state, Tensor row_state, Tensor row_back, Tensor row_fwd, Tensor pos, Tensor? run_rows, Tensor(b!) out) -> ()");
  m.def("moe_route_grouped(Tensor z, Tensor correction, int top, int groups, int keep, Tensor(a!) ids, Tensor(b!) weights) -> ()");
  m.def("moe_pair_up(Tensor h, Tensor ids, Tensor w13, Tensor(a!) act) -> ()");
  m.def("residual_add_norm(Tensor(a!) x, Tensor? y1, Tensor? y2, Tensor? shift, Tensor? w, float eps, float offset, Tensor(b!)? out, float mult) -> ()");
  m.def("rotary_append(Tensor qkv, Tensor pos, Tensor inv_freq, Tensor slots, Tensor(a!) k_cache, Tensor(b!) v_cache, int H, int G, int maps, int dim, int vdim, Tensor(c!) q_out) -> ()");
  m.def("attn_diff_window(Tensor q, Tensor k_cache, Tensor v_cache, Tensor bt, Tensor q_start, Tensor q_len, Tensor kv_len, Tensor work_seq, Tensor work_qblk, Tensor gate, Tensor(a!) out, float scale, int window, float lam, float eps, float out_mult, int short_rows, bool mfma) -> ()");
  m.def("diff_mfma_ok", &diff_mfma_ok);
  m.def("qk_norm_rotary_append(Tensor proj, Tensor? bias, Tensor? q_norm_w, Tensor? k_norm_w, bool norm_all, int k_norm_n, float eps, Tensor pos, Tensor inv_freq, float rot_mult, int q_rot_off, int k_rot_off, Tensor slots, Tensor(a!)? k_cache, Tensor(b!)? v_cache, int H, int G, int qw, int kw, int vdim, int v_mode, Tensor(c!) q_out) -> ()");
  m.def("attn_keep_window(Tensor q, Tensor k_cache, Tensor v_cache, int vdim, Tensor bt, Tensor q_start, Tensor q_len, Tensor kv_len, Tensor work_seq, Tensor work_qblk, Tensor? head_bias, Tensor? gate, Tensor(a!) out, float scale, int window, int keep_first, bool sigmoid, int short_rows, bool mfma) -> ()");
  m.def("keep_mfma_ok", &keep_mfma_ok);
  m.def("xielu_rows(Tensor x, float ap, float an, Tensor(a!) out) -> ()");
  m.def("conv_act_heads(Tensor x, Tensor w, Tensor(a!) state, Tensor row_state, Tensor row_back, Tensor row_fwd, Tensor pos, int n_unit, int dim, float unit_eps, Tensor(b!) out) -> ()");
  m.def("gated_linear_recurrence(Tensor q, Tensor k, Tensor v, Tensor z, Tensor rate, Tensor zbias, float zsign, Tensor? beta, Tensor gate, bool gate_sigmoid, Tensor norm_w, float eps, float q_scale, Tensor(a!) state, Tensor row_state, Tensor row_back, Tensor row_fwd, Tensor pos, Tensor? run_rows, Tensor(b!) out, bool decay_ready, Tensor(c!)? raw) -> ()");
  m.def("decay_from_logits(Tensor(a!) z, Tensor rate, Tensor zbias, float zsign, int dim) -> ()");
  m.def("moe_route_topk(Tensor z, Tensor? bias, int top, Tensor(a!) ids, Tensor(b!) weights) -> ()");
  m.def("gelu_rows(Tensor x, Tensor(a!) out) -> ()");
  m.def("moe_pair_down(Tensor act, Tensor ids, Tensor weights, Tensor w2, Tensor? base, Tensor(a!) out) -> ()");
}

TORCH_LIBRARY_IMPL(rfq_mix, CUDA, m) {
  m.impl("embed_sinusoid", &embed_sinusoid);
  m.impl("sandwich_norm", &sandwich_norm);
  m.impl("canon_conv", &canon_conv);
  m.impl("head_norm_append", &head_norm_append);
  m.impl("attn_talk_decode", &attn_talk_decode);
  m.impl("attn_mixq_prefill", &attn_mixq_prefill);
  m.impl("attn_mix_mfma", &attn_mix_mfma);
  m.impl("glu_clamped", &glu_clamped);
  m.impl("attn_latent_mfma", &attn_latent_mfma);
  m.impl("embed_rows", &embed_rows);
  m.impl("post_norm_add", &post_norm_add);
  m.impl("rms_norm_rows", &rms_norm_rows);
  m.impl("latent_norm_append", &latent_norm_append);
  m.impl("silu_mul_any", &silu_mul_any);
  m.impl("softcap", &softcap);
  m.impl("token_shift_mix", &token_shift_mix);
  m.impl("wkv_recurrence", &wkv_recurrence);
  m.impl("moe_route_grouped", &moe_route_grouped);
  m.impl("moe_pair_up", &moe_pair_up);
  m.impl("moe_pair_down", &moe_pair_down);
  m.impl("residual_add_norm", &residual_add_norm);
  m.impl("rotary_append", &rotary_append);
  m.impl("attn_diff_window", &attn_diff_window);
  m.impl("qk_norm_rotary_append", &qk_norm_rotary_append);
  m.impl("attn_keep_window", &attn_keep_window);
  m.impl("xielu_rows", &xielu_rows);
  m.impl("conv_act_heads", &conv_act_heads);
  m.impl("gated_linear_recurrence", &gated_linear_recurrence);
  m.impl("decay_from_logits", &decay_from_logits);
  m.impl("moe_route_topk", &moe_route_topk);
  m.impl("gelu_rows", &gelu_rows);
}
