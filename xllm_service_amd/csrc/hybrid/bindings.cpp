// PyTorch bindings for the hybrid-mixer kernels (latent attention, decayed
// linear attention, grouped norms, routed experts). Shape/dtype validation
// lives here; activations may be bf16 or fp32, everything the kernels
// accumulate or carry is fp32.
#include <hip/hip_runtime.h>
#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>

#include <algorithm>
#include <cstdint>
#include <cstdlib>

namespace xllm {
namespace hyb {
template <typename TI, typename TO>
void launch_group_rmsnorm(TO*, const TI*, const float*, float, int, int, int,
                          long, hipStream_t);
template <typename TY, typename TG>
void launch_gated_norm_residual(float*, const TY*, const TG*, const float*,
                                const float*, const float*, float, float, int,
                                int, int, long, hipStream_t);
template <typename T>
void launch_norm_sigmoid_gate(T*, const float*, const float*, const T*, float,
                              int, int, long, int, hipStream_t);
template <typename TY, typename T>
void launch_norm_residual_add(float*, T*, const TY*, const float*, float, int,
                              int, long, const float*, hipStream_t);
template <typename T>
void launch_rope_headnorm_store(T*, const T*, const T*, const T*, long, long,
                                long, const long*, const double*, int, int,
                                int, float, int, int, int, int, int, T*, T*,
                                const long*, int, hipStream_t);
template <typename T>
void launch_polynorm(T*, const T*, const float*, float, long, int, long,
                     hipStream_t);
template <typename T>
void launch_gelu_tanh_gate(T*, const T*, const T*, long, int, long, long,
                           hipStream_t);
template <typename T>
void launch_silu_mul(T*, const T*, long, int, hipStream_t);
template <typename T>
void launch_gelu_tanh_mul(T*, const T*, long, int, hipStream_t);
template <typename T>
void launch_rownorm_rope_store(T*, const T*, const T*, const T*, long, long,
                               long, const float*, const float*, float,
                               const long*, const double*, int, int, int, int,
                               int, int, T*, T*, const long*, int,
                               hipStream_t);
template <typename T>
void launch_delta_rule(float*, const T*, const T*, const T*, const T*,
                       const T*, long, long, long, long, long, const float*,
                       const float*, float*, const int*, const int*,
                       const int*, int, int, int, int, int, int, int, float*,
                       hipStream_t);
template <typename T>
void launch_rope_interleaved(T*, const long*, const double*, float, int, int,
                             int, long, long, int, hipStream_t);
template <typename T>
void launch_latent_kv_store(T*, const T*, const float*, float, const long*,
                            const double*, float, int, const long*, int, int,
                            int, long, hipStream_t);
template <typename T>
void launch_latent_attn(float*, const T*, const T*, const int*, const int*,
                        const int*, int, int, int, int, int, int, int, float,
                        long, hipStream_t);
int latent_attn_mfma_class(int W, int r);
void launch_latent_attn_mfma(float*, float*, float*, const unsigned short*,
                             const unsigned short*, const int*, const int*,
                             const int*, int, int, int, int, int, int, int,
                             float, int, hipStream_t);
template <typename T>
void launch_decay_attn(float*, const T*, const T*, const T*, const float*,
                       float*, const int*, const int*, const int*, int, int,
                       int, int, long, long, long, int, int, float*,
                       hipStream_t);
void launch_moe_route(int*, float*, const float*, int, int, int, int, int,
                      int, const float*, int, int, hipStream_t);
template <typename T>
void launch_moe_combine(float*, const T*, const int*, const float*, long, int,
                        int, const T*, long, const T*, long, hipStream_t);
template <typename TO>
void launch_streams_mix_norm(TO*, const float*, const float*, const float*,
                             const float*, float, int, int, int, hipStream_t);
template <typename T>
void launch_streams_update(float*, const float*, const float*, const T*, float,
                           const T*, float, long, int, int, hipStream_t);
template <typename T>
void launch_streams_update_mix_norm(T*, float*, const float*, const float*,
                                    const T*, float, const T*, float,
                                    const float*, const float*, const float*,
                                    float, int, int, int, hipStream_t);
template <typename T>
void launch_relu_sq(T*, long, hipStream_t);
template <typename T>
void launch_softcap(float*, const T*, float, long, hipStream_t);
template <typename T>
void launch_short_conv(T*, long, T*, const long*, int, const T*, long,
                       const T*, const T*, const T*, long, int, const int*,
                       const int*, const int*, int, int, int, int, int, int,
                       int, const long*, const double*, hipStream_t);
template <typename T>
void launch_short_conv_state(T*, long, const T*, long, const int*, const int*,
                             int, int, int, hipStream_t);
template <typename T>
void launch_gated_recurrence(int, float*, const T*, const T*, const T*,
                             const T*, long, long, long, long, const float*,
                             const float*, const float*, float, float, float*,
                             const int*, const int*, const int*, int, int, int,
                             int, int, int, int, float*, float*, hipStream_t);
template <typename T>
void launch_gated_group_norm(T*, const float*, const float*, int, const T*,
                             long, float, int, int, int, int, int,
                             hipStream_t);
int capped_attn_mfma_class(int D, int Dv);
void launch_capped_attn_mfma(float*, float*, float*, const unsigned short*,
                             const unsigned short*, const unsigned short*,
                             const int*, const int*, const int*, int, int, int,
                             int, int, int, int, int, float, float, long, int,
                             int, const float*, int, const float*,
                             hipStream_t);
template <typename T>
void launch_capped_attn(float*, const T*, const T*, const T*, const int*,
                        const int*, const int*, int, int, int, int, int, int,
                        int, int, float, float, long, int, const float*, int,
                        const float*, hipStream_t);
}  // namespace hyb
}  // namespace xllm

namespace {
using torch::Tensor;
using bf = unsigned short;
namespace hy = xllm::hyb;

inline hipStream_t cur() { return at::hip::getCurrentHIPStream().stream(); }
inline bool is_bf16(const Tensor& t) { return t.dtype() == torch::kBFloat16; }
inline bool is_f32(const Tensor& t) { return t.dtype() == torch::kFloat; }

#define CHK_ACT(t)                                                       \
  TORCH_CHECK((t).is_cuda() && (is_bf16(t) || is_f32(t)),                \
              #t " must be a bf16/fp32 GPU tensor");                     \
  TORCH_CHECK((t).stride(-1) == 1, #t " innermost dim must be contiguous")
#define CHK_F32C(t)                                                      \
  TORCH_CHECK((t).is_cuda() && is_f32(t) && (t).is_contiguous(),         \
              #t " must be a contiguous fp32 GPU tensor")
#define CHK_I32C(t)                                                      \
  TORCH_CHECK((t).is_cuda() && (t).dtype() == torch::kInt &&             \
              (t).is_contiguous(), #t " must be contiguous int32 on GPU")
#define CHK_I64C(t)                                                      \
  TORCH_CHECK((t).is_cuda() && (t).dtype() == torch::kLong &&            \
              (t).is_contiguous(), #t " must be contiguous int64 on GPU")

template <typename T> T* ptr(const Tensor& t) {
  return reinterpret_cast<T*>(t.data_ptr());
}

// out [rows, width] contiguous (bf16|fp32), x 2-D with unit inner stride
void group_rmsnorm(Tensor out, Tensor x, Tensor w, double eps, long groups) {
  CHK_ACT(out); CHK_ACT(x); CHK_F32C(w);
  TORCH_CHECK(x.dim() == 2 && out.dim() == 2 && out.is_contiguous());
  const int rows = x.size(0), width = x.size(1);
  TORCH_CHECK(out.size(0) == rows && out.size(1) == width &&
              w.numel() == width && groups >= 1 && width % groups == 0);
  const long xs = x.stride(0);
  auto st = cur();
  if (is_f32(x) && is_f32(out))
    hy::launch_group_rmsnorm<float, float>(ptr<float>(out), ptr<float>(x), ptr<float>(w), eps, rows, width, groups, xs, st);
  else if (is_f32(x))
    hy::launch_group_rmsnorm<float, bf>(ptr<bf>(out), ptr<float>(x), ptr<float>(w), eps, rows, width, groups, xs, st);
  else if (is_f32(out))
    hy::launch_group_rmsnorm<bf, float>(ptr<float>(out), ptr<bf>(x), ptr<float>(w), eps, rows, width, groups, xs, st);
  else
    hy::launch_group_rmsnorm<bf, bf>(ptr<bf>(out), ptr<bf>(x), ptr<float>(w), eps, rows, width, groups, xs, st);
}

void gated_norm_residual(Tensor res, Tensor y, Tensor gate,
                         c10::optional<Tensor> bias, Tensor w, Tensor ls,
                         double mult, double eps, long groups) {
  CHK_F32C(res); CHK_ACT(y); CHK_ACT(gate); CHK_F32C(w); CHK_F32C(ls);
  TORCH_CHECK(res.dim() == 2 && y.dim() == 2 && gate.dim() == 2 &&
              y.is_contiguous());
  const int rows = res.size(0), width = res.size(1);
  TORCH_CHECK(y.size(0) == rows && y.size(1) == width &&
              gate.size(0) == rows && gate.size(1) == width &&
              w.numel() == width && ls.numel() == width &&
              groups >= 1 && width % groups == 0);
  const float* b = nullptr;
  if (bias.has_value()) {
    CHK_F32C(*bias);
    TORCH_CHECK(bias->numel() == width);
    b = ptr<float>(*bias);
  }
  const long gs = gate.stride(0);
  auto st = cur();
  if (is_f32(y) && is_f32(gate))
    hy::launch_gated_norm_residual<float, float>(ptr<float>(res), ptr<float>(y), ptr<float>(gate), b, ptr<float>(w), ptr<float>(ls), mult, eps, rows, width, groups, gs, st);
  else if (is_f32(y))
    hy::launch_gated_norm_residual<float, bf>(ptr<float>(res), ptr<float>(y), ptr<bf>(gate), b, ptr<float>(w), ptr<float>(ls), mult, eps, rows, width, groups, gs, st);
  else {
    TORCH_CHECK(is_bf16(gate), "bf16 y needs a bf16 gate");
    hy::launch_gated_norm_residual<bf, bf>(ptr<float>(res), ptr<bf>(y), ptr<bf>(gate), b, ptr<float>(w), ptr<float>(ls), mult, eps, rows, width, groups, gs, st);
  }
}

void norm_sigmoid_gate(Tensor out, Tensor o, c10::optional<Tensor> w,
                       Tensor gate, double eps, long gate_cols) {
  CHK_ACT(out); CHK_F32C(o); CHK_ACT(gate);
  TORCH_CHECK(out.is_contiguous() && out.dim() == 2 && gate.dim() == 2);
  const int rows = out.size(0), n = out.size(1);
  TORCH_CHECK(gate_cols >= 1 && n % gate_cols == 0);
  TORCH_CHECK(o.numel() == (long)rows * n && gate.size(0) == rows &&
              gate.size(1) == n / gate_cols && gate.dtype() == out.dtype());
  const float* wp = nullptr;
  if (w.has_value()) {
    CHK_F32C(*w);
    TORCH_CHECK(w->numel() == n);
    wp = ptr<float>(*w);
  }
  if (is_f32(out))
    hy::launch_norm_sigmoid_gate<float>(ptr<float>(out), ptr<float>(o), wp, ptr<float>(gate), eps, rows, n, gate.stride(0), gate_cols, cur());
  else
    hy::launch_norm_sigmoid_gate<bf>(ptr<bf>(out), ptr<float>(o), wp, ptr<bf>(gate), eps, rows, n, gate.stride(0), gate_cols, cur());
}

// res fp32 [rows, width] += y / rms(y) * w1 (y fp32 or h's type); h = the new
// res, or with w_next res / rms(res) * w_next
void norm_residual_add(Tensor res, Tensor h, Tensor y, Tensor w1, double eps,
                       c10::optional<Tensor> w_next) {
  CHK_F32C(res); CHK_ACT(h); CHK_ACT(y); CHK_F32C(w1);
  TORCH_CHECK(res.dim() == 2 && y.dim() == 2 && h.is_contiguous() &&
              (h.dtype() == y.dtype() || is_f32(y)));
  const int rows = res.size(0), width = res.size(1);
  TORCH_CHECK(y.size(0) == rows && y.size(1) == width &&
              h.numel() == res.numel() && w1.numel() == width);
  const float* wn = nullptr;
  if (w_next.has_value()) {
    CHK_F32C(*w_next);
    TORCH_CHECK(w_next->numel() == width);
    wn = ptr<float>(*w_next);
  }
  if (is_f32(y) && is_f32(h))
    hy::launch_norm_residual_add<float, float>(ptr<float>(res), ptr<float>(h), ptr<float>(y), ptr<float>(w1), eps, rows, width, y.stride(0), wn, cur());
  else if (is_f32(y))
    hy::launch_norm_residual_add<float, bf>(ptr<float>(res), ptr<bf>(h), ptr<float>(y), ptr<float>(w1), eps, rows, width, y.stride(0), wn, cur());
  else
    hy::launch_norm_residual_add<bf, bf>(ptr<float>(res), ptr<bf>(h), ptr<bf>(y), ptr<float>(w1), eps, rows, width, y.stride(0), wn, cur());
}

// out [rows, F] contiguous; z row view of the same type; coef fp32 [4]
void polynorm(Tensor out, Tensor z, Tensor coef, double eps) {
  CHK_ACT(out); CHK_ACT(z); CHK_F32C(coef);
  TORCH_CHECK(out.dim() == 2 && z.dim() == 2 && out.is_contiguous() &&
              out.dtype() == z.dtype() && out.size(0) == z.size(0) &&
              out.size(1) == z.size(1) && coef.numel() == 4);
  const long rows = z.size(0);
  const int F = z.size(1);
  if (is_f32(z)) hy::launch_polynorm<float>(ptr<float>(out), ptr<float>(z), ptr<float>(coef), eps, rows, F, z.stride(0), cur());
  else hy::launch_polynorm<bf>(ptr<bf>(out), ptr<bf>(z), ptr<float>(coef), eps, rows, F, z.stride(0), cur());
}

// out [rows, F] contiguous = gelu_tanh(g) * u; g, u row views
void gelu_tanh_gate(Tensor out, Tensor g, Tensor u) {
  CHK_ACT(out); CHK_ACT(g); CHK_ACT(u);
  TORCH_CHECK(out.dim() == 2 && g.dim() == 2 && u.dim() == 2 &&
              out.is_contiguous() && out.dtype() == g.dtype() &&
              out.dtype() == u.dtype() && g.sizes() == out.sizes() &&
              u.sizes() == out.sizes());
  const long rows = out.size(0);
  const int F = out.size(1);
  if (is_f32(g)) hy::launch_gelu_tanh_gate<float>(ptr<float>(out), ptr<float>(g), ptr<float>(u), rows, F, g.stride(0), u.stride(0), cur());
  else hy::launch_gelu_tanh_gate<bf>(ptr<bf>(out), ptr<bf>(g), ptr<bf>(u), rows, F, g.stride(0), u.stride(0), cur());
}

// q_out [T, H*D] contiguous; q/k/v row views of a projection (v absent: the
// values are the keys); caches [blocks, n_kv, block, D | Dv]
void rope_headnorm_store(Tensor q_out, Tensor q, Tensor k,
                         c10::optional<Tensor> v, Tensor pos, Tensor inv_freq,
                         long rot, bool pairs, bool unit, double eps,
                         long heads, long n_kv, Tensor k_cache,
                         Tensor v_cache, Tensor slot_mapping) {
  CHK_ACT(q_out); CHK_ACT(q); CHK_ACT(k); CHK_I64C(pos);
  CHK_I64C(slot_mapping); CHK_ACT(k_cache); CHK_ACT(v_cache);
  TORCH_CHECK(q.dim() == 2 && k.dim() == 2 && q_out.is_contiguous() &&
              k_cache.dim() == 4 && v_cache.dim() == 4 &&
              k_cache.is_contiguous() && v_cache.is_contiguous());
  TORCH_CHECK(q.dtype() == k.dtype() && q.dtype() == q_out.dtype() &&
              q.dtype() == k_cache.dtype() && q.dtype() == v_cache.dtype());
  const int T = q.size(0), D = k_cache.size(3), Dv = v_cache.size(3);
  const int bs = k_cache.size(2);
  TORCH_CHECK(heads >= 1 && n_kv >= 1 && D <= 64 * 8 &&
              q.size(1) == heads * D && k.size(1) == n_kv * D &&
              k.size(0) == T && q_out.numel() == q.numel() &&
              k_cache.size(1) == n_kv && v_cache.size(1) == n_kv &&
              v_cache.size(2) == bs && v_cache.size(0) == k_cache.size(0) &&
              pos.numel() == T && slot_mapping.numel() == T,
              "rope_headnorm_store: bad shapes");
  TORCH_CHECK(rot >= 0 && rot % 2 == 0 && rot <= D &&
              inv_freq.is_cuda() && inv_freq.dtype() == torch::kDouble &&
              inv_freq.is_contiguous() && inv_freq.numel() == rot / 2);
  const void* vp = nullptr;
  long vs = 0;
  if (v.has_value()) {
    CHK_ACT(*v);
    TORCH_CHECK(v->dim() == 2 && v->dtype() == q.dtype() &&
                v->size(0) == T && v->size(1) == n_kv * Dv,
                "rope_headnorm_store: bad value rows");
    vp = v->data_ptr();
    vs = v->stride(0);
  }
  if (is_f32(q))
    hy::launch_rope_headnorm_store<float>(ptr<float>(q_out), ptr<float>(q), ptr<float>(k), (const float*)vp, q.stride(0), k.stride(0), vs, ptr<long>(pos), ptr<double>(inv_freq), rot, pairs, unit, eps, T, heads, n_kv, D, Dv, ptr<float>(k_cache), ptr<float>(v_cache), ptr<long>(slot_mapping), bs, cur());
  else
    hy::launch_rope_headnorm_store<bf>(ptr<bf>(q_out), ptr<bf>(q), ptr<bf>(k), (const bf*)vp, q.stride(0), k.stride(0), vs, ptr<long>(pos), ptr<double>(inv_freq), rot, pairs, unit, eps, T, heads, n_kv, D, Dv, ptr<bf>(k_cache), ptr<bf>(v_cache), ptr<long>(slot_mapping), bs, cur());
}

void gelu_tanh_mul(Tensor out, Tensor x) {
  CHK_ACT(out); CHK_ACT(x);
  TORCH_CHECK(out.is_contiguous() && x.is_contiguous() &&
              out.dtype() == x.dtype());
  const int F = out.size(-1);
  TORCH_CHECK(x.size(-1) == 2 * F && x.numel() == 2 * out.numel());
  const long rows = out.numel() / F;
  if (is_f32(x)) hy::launch_gelu_tanh_mul<float>(ptr<float>(out), ptr<float>(x), rows, F, cur());
  else hy::launch_gelu_tanh_mul<bf>(ptr<bf>(out), ptr<bf>(x), rows, F, cur());
}

// q_out [T, H*D] contiguous; q/k/v row views of a projection; caches
// [blocks, n_kv, block, D | Dv]
void rownorm_rope_store(Tensor q_out, Tensor q, Tensor k, Tensor v, Tensor wq,
                        Tensor wk, double eps, Tensor pos, Tensor inv_freq,
                        long rot, long heads, long n_kv, Tensor k_cache,
                        Tensor v_cache, Tensor slot_mapping) {
  CHK_ACT(q_out); CHK_ACT(q); CHK_ACT(k); CHK_ACT(v); CHK_F32C(wq);
  CHK_F32C(wk); CHK_I64C(pos); CHK_I64C(slot_mapping); CHK_ACT(k_cache);
  CHK_ACT(v_cache);
  TORCH_CHECK(q.dim() == 2 && k.dim() == 2 && v.dim() == 2 &&
              q_out.is_contiguous() && k_cache.dim() == 4 &&
              v_cache.dim() == 4 && k_cache.is_contiguous() &&
              v_cache.is_contiguous());
  TORCH_CHECK(q.dtype() == k.dtype() && q.dtype() == v.dtype() &&
              q.dtype() == q_out.dtype() && q.dtype() == k_cache.dtype() &&
              q.dtype() == v_cache.dtype());
  const int T = q.size(0), D = k_cache.size(3), Dv = v_cache.size(3);
  const int bs = k_cache.size(2);
  TORCH_CHECK(heads >= 1 && n_kv >= 1 && q.size(1) == heads * D &&
              k.size(1) == n_kv * D && v.size(1) == n_kv * Dv &&
              k.size(0) == T && v.size(0) == T && q_out.numel() == q.numel() &&
              k_cache.size(1) == n_kv && v_cache.size(1) == n_kv &&
              v_cache.size(2) == bs && v_cache.size(0) == k_cache.size(0) &&
              wq.numel() == heads * D && wk.numel() == n_kv * D &&
              pos.numel() == T && slot_mapping.numel() == T,
              "rownorm_rope_store: bad shapes");
  TORCH_CHECK(rot >= 0 && rot % 2 == 0 && rot <= D && rot <= 8192 &&
              inv_freq.is_cuda() && inv_freq.dtype() == torch::kDouble &&
              inv_freq.is_contiguous() && inv_freq.numel() == rot / 2);
  if (is_f32(q))
    hy::launch_rownorm_rope_store<float>(ptr<float>(q_out), ptr<float>(q), ptr<float>(k), ptr<float>(v), q.stride(0), k.stride(0), v.stride(0), ptr<float>(wq), ptr<float>(wk), eps, ptr<long>(pos), ptr<double>(inv_freq), rot, T, heads, n_kv, D, Dv, ptr<float>(k_cache), ptr<float>(v_cache), ptr<long>(slot_mapping), bs, cur());
  else
    hy::launch_rownorm_rope_store<bf>(ptr<bf>(q_out), ptr<bf>(q), ptr<bf>(k), ptr<bf>(v), q.stride(0), k.stride(0), v.stride(0), ptr<float>(wq), ptr<float>(wk), eps, ptr<long>(pos), ptr<double>(inv_freq), rot, T, heads, n_kv, D, Dv, ptr<bf>(k_cache), ptr<bf>(v_cache), ptr<long>(slot_mapping), bs, cur());
}

// out fp32 [T, H, Dv]; state fp32 [slots, H, D, Dv]; q/k [T, groups*D],
// v [T, H*Dv], b/a [T, H] row views (after convolution: q, k, v)
void delta_rule(Tensor out, Tensor q, Tensor k, Tensor v, Tensor b, Tensor a,
                Tensor dt_bias, Tensor A_log, Tensor state, Tensor slots,
                c10::optional<Tensor> cu_q, Tensor ctx_lens, long groups,
                long max_q_len) {
  CHK_F32C(out); CHK_ACT(q); CHK_ACT(k); CHK_ACT(v); CHK_ACT(b); CHK_ACT(a);
  CHK_F32C(dt_bias); CHK_F32C(A_log); CHK_F32C(state); CHK_I32C(slots);
  CHK_I32C(ctx_lens);
  TORCH_CHECK(state.dim() == 4 && q.dim() == 2 && k.dim() == 2 &&
              v.dim() == 2 && b.dim() == 2 && a.dim() == 2 &&
              q.dtype() == k.dtype() && q.dtype() == v.dtype() &&
              q.dtype() == b.dtype() && q.dtype() == a.dtype());
  const int H = state.size(1), D = state.size(2), Dv = state.size(3);
  const int T = q.size(0);
  TORCH_CHECK(groups >= 1 && H % groups == 0 && q.size(1) == groups * D &&
              k.size(1) == groups * D && v.size(1) == H * Dv &&
              b.size(1) == H && a.size(1) == H && k.size(0) == T &&
              v.size(0) == T && b.size(0) == T && a.size(0) == T &&
              dt_bias.numel() == H && A_log.numel() == H,
              "delta_rule: bad shapes");
  TORCH_CHECK(D <= 256, "key dim > 256 unsupported");
  TORCH_CHECK(out.numel() == (long)T * H * Dv);
  const int n_seqs = slots.numel();
  TORCH_CHECK(ctx_lens.numel() == n_seqs);
  const int* cu = nullptr;
  if (cu_q.has_value()) {
    CHK_I32C(*cu_q);
    TORCH_CHECK(cu_q->numel() == n_seqs + 1);
    cu = ptr<int>(*cu_q);
  } else {
    TORCH_CHECK(n_seqs == T, "decode: one sequence per token");
  }
  // long chunks on a chip that the (sequence, head) pairs alone leave mostly
  // empty: piece-parallel passes (three times the arithmetic, many times the
  // workgroups). XLLM_DELTA_CHUNK: piece length, 0 switches the passes off.
  int chunk = 128, max_chunks = 1;
  Tensor ws;
  if (cu != nullptr) {
    const long bound = max_q_len > 0 ? std::min<long>(max_q_len, T) : T;
    if (const char* e = std::getenv("XLLM_DELTA_CHUNK"))
      chunk = std::min(1024, std::max(0, std::atoi(e)));
    const long rec = (long)H * D * (Dv + D) * 4;
    // shorter pieces while the first pass would not fill the chip
    while (chunk > 32 && (bound + chunk - 1) / chunk * n_seqs * H *
                             ((Dv + D + 63) / 64) < 1024)
      chunk /= 2;
    while (chunk > 0 && (bound + chunk - 1) / chunk * n_seqs * rec > (1L << 31))
      chunk *= 2;                             // keep the scratch under 2 GiB
    const long wgs = (long)n_seqs * H * ((Dv + 63) / 64);
    if (chunk > 0 && bound >= 4L * chunk && wgs < 512) {
      max_chunks = (int)((bound + chunk - 1) / chunk);
      ws = torch::empty({(long)n_seqs * max_chunks, (long)H, (long)D,
                         (long)(Dv + D)}, state.options());
    }
  }
  float* wsp = max_chunks > 1 ? ptr<float>(ws) : nullptr;
  if (is_f32(q))
    hy::launch_delta_rule<float>(ptr<float>(out), ptr<float>(q), ptr<float>(k), ptr<float>(v), ptr<float>(b), ptr<float>(a), q.stride(0), k.stride(0), v.stride(0), b.stride(0), a.stride(0), ptr<float>(dt_bias), ptr<float>(A_log), ptr<float>(state), ptr<int>(slots), cu, ptr<int>(ctx_lens), n_seqs, H, groups, D, Dv, chunk, max_chunks, wsp, cur());
  else
    hy::launch_delta_rule<bf>(ptr<float>(out), ptr<bf>(q), ptr<bf>(k), ptr<bf>(v), ptr<bf>(b), ptr<bf>(a), q.stride(0), k.stride(0), v.stride(0), b.stride(0), a.stride(0), ptr<float>(dt_bias), ptr<float>(A_log), ptr<float>(state), ptr<int>(slots), cu, ptr<int>(ctx_lens), n_seqs, H, groups, D, Dv, chunk, max_chunks, wsp, cur());
}

void silu_mul(Tensor out, Tensor x) {
  CHK_ACT(out); CHK_ACT(x);
  TORCH_CHECK(out.is_contiguous() && x.is_contiguous() &&
              out.dtype() == x.dtype());
  const int F = out.size(-1);
  TORCH_CHECK(x.size(-1) == 2 * F && x.numel() == 2 * out.numel());
  const long rows = out.numel() / F;
  if (is_f32(x)) hy::launch_silu_mul<float>(ptr<float>(out), ptr<float>(x), rows, F, cur());
  else hy::launch_silu_mul<bf>(ptr<bf>(out), ptr<bf>(x), rows, F, cur());
}

// x [T, H, D] view (unit inner stride); rotates x[..., off:off+rot_dims]
void rope_interleaved(Tensor x, Tensor pos, Tensor inv_freq, double mscale,
                      long off, long rot_dims) {
  CHK_ACT(x); CHK_I64C(pos);
  TORCH_CHECK(inv_freq.is_cuda() && inv_freq.dtype() == torch::kDouble &&
              inv_freq.is_contiguous());
  TORCH_CHECK(x.dim() == 3 && pos.numel() == x.size(0));
  TORCH_CHECK(rot_dims % 2 == 0 && off >= 0 && off + rot_dims <= x.size(2) &&
              inv_freq.numel() == rot_dims / 2);
  const int T = x.size(0), H = x.size(1);
  if (is_f32(x))
    hy::launch_rope_interleaved<float>(ptr<float>(x), ptr<long>(pos), ptr<double>(inv_freq), mscale, T, H, rot_dims / 2, x.stride(0), x.stride(1), off, cur());
  else
    hy::launch_rope_interleaved<bf>(ptr<bf>(x), ptr<long>(pos), ptr<double>(inv_freq), mscale, T, H, rot_dims / 2, x.stride(0), x.stride(1), off, cur());
}

// cache [blocks, bs, r+rd]; dkv [T, r+rd] row view
void latent_kv_store(Tensor cache, Tensor dkv, Tensor norm_w, double eps,
                     Tensor pos, Tensor inv_freq, double mscale,
                     long rot_dims, Tensor slots, long kv_rank) {
  CHK_ACT(cache); CHK_ACT(dkv); CHK_F32C(norm_w); CHK_I64C(pos);
  CHK_I64C(slots);
  TORCH_CHECK(cache.is_contiguous() && cache.dim() == 3 && dkv.dim() == 2 &&
              cache.dtype() == dkv.dtype());
  TORCH_CHECK(inv_freq.is_cuda() && inv_freq.dtype() == torch::kDouble &&
              inv_freq.is_contiguous());
  const int T = dkv.size(0), W = dkv.size(1);
  const int r = kv_rank, rd = W - r;
  TORCH_CHECK(cache.size(2) == W && r > 0 && rd >= 0 && rot_dims <= rd &&
              rot_dims % 2 == 0 && norm_w.numel() == r &&
              inv_freq.numel() == rot_dims / 2 && pos.numel() == T &&
              slots.numel() == T);
  if (is_f32(dkv))
    hy::launch_latent_kv_store<float>(ptr<float>(cache), ptr<float>(dkv), ptr<float>(norm_w), eps, ptr<long>(pos), ptr<double>(inv_freq), mscale, rot_dims, ptr<long>(slots), T, r, rd, dkv.stride(0), cur());
  else
    hy::launch_latent_kv_store<bf>(ptr<bf>(cache), ptr<bf>(dkv), ptr<float>(norm_w), eps, ptr<long>(pos), ptr<double>(inv_freq), mscale, rot_dims, ptr<long>(slots), T, r, rd, dkv.stride(0), cur());
}

// out fp32 [T, H, r]; q [T, H, r+rd] contiguous; cu_q None => decode
void latent_attn(Tensor out, Tensor q, Tensor cache, Tensor block_tables,
                 c10::optional<Tensor> cu_q, Tensor seq_lens, double scale,
                 long kv_rank) {
  CHK_F32C(out); CHK_ACT(q); CHK_ACT(cache); CHK_I32C(block_tables);
  CHK_I32C(seq_lens);
  TORCH_CHECK(q.dim() == 3 && q.is_contiguous() && cache.is_contiguous() &&
              cache.dim() == 3 && q.dtype() == cache.dtype() &&
              block_tables.dim() == 2);
  const int T = q.size(0), H = q.size(1), W = q.size(2);
  const int r = kv_rank;
  TORCH_CHECK(cache.size(2) == W && r > 0 && r <= W && r <= 64 * 16,
              "latent width mismatch or kv_rank > 1024");
  TORCH_CHECK(out.numel() == (long)T * H * r);
  const int n_seqs = seq_lens.numel();
  TORCH_CHECK(block_tables.size(0) == n_seqs);
  const int* cu = nullptr;
  if (cu_q.has_value()) {
    CHK_I32C(*cu_q);
    TORCH_CHECK(cu_q->numel() == n_seqs + 1);
    cu = ptr<int>(*cu_q);
  } else {
    TORCH_CHECK(n_seqs == T, "decode: one sequence per token");
  }
  // bf16: MFMA kernel when the sizes fit one of its instantiations
  if (is_bf16(q) && hy::latent_attn_mfma_class(W, r) != 0) {
    int n_part = 1;
    Tensor ws_acc, ws_ml;
    if (cu == nullptr) {
      // decode: split the context over workgroups when tokens alone do not
      // fill the chip (sizes known on the host only: no sync)
      // about one workgroup per CU measured best (batch 8/32/128 at 1k-4k
      // context): more parts only add fp32 partials to write and merge
      const int tps = (H + 63) / 64;
      const long max_tiles = ((long)block_tables.size(1) * cache.size(1) + 31) / 32;
      n_part = (int)std::min<long>(std::min<long>(32, (max_tiles + 1) / 2),
                                   std::max<long>(1, 256 / ((long)T * tps)));
      n_part = std::max(n_part, 1);
      // tuning knob: fixed partition count (1..32)
      if (const char* e = std::getenv("XLLM_LATENT_PARTS"))
        n_part = std::min(32, std::max(1, std::atoi(e)));
    }
    if (n_part > 1) {
      ws_acc = torch::empty({(long)T * H * n_part, (long)r}, out.options());
      ws_ml = torch::empty({(long)T * H * n_part, 2}, out.options());
    }
    hy::launch_latent_attn_mfma(
        ptr<float>(out), n_part > 1 ? ptr<float>(ws_acc) : nullptr,
        n_part > 1 ? ptr<float>(ws_ml) : nullptr, ptr<bf>(q), ptr<bf>(cache),
        ptr<int>(block_tables), cu, ptr<int>(seq_lens), T, n_seqs, H, r,
        W - r, cache.size(1), block_tables.size(1), scale, n_part, cur());
    return;
  }
  const int nw = H < 4 ? H : 4;
  TORCH_CHECK((size_t)nw * W * 4 <= 64 * 1024, "query row too wide for LDS");
  if (is_f32(q))
    hy::launch_latent_attn<float>(ptr<float>(out), ptr<float>(q), ptr<float>(cache), ptr<int>(block_tables), cu, ptr<int>(seq_lens), T, n_seqs, H, r, W - r, cache.size(1), block_tables.size(1), scale, q.stride(0), cur());
  else
    hy::launch_latent_attn<bf>(ptr<float>(out), ptr<bf>(q), ptr<bf>(cache), ptr<int>(block_tables), cu, ptr<int>(seq_lens), T, n_seqs, H, r, W - r, cache.size(1), block_tables.size(1), scale, q.stride(0), cur());
}

// out fp32 [T, H, Dv]; q,k [T, H*D] / v [T, H*Dv] row views (pre-activation)
// state fp32 [slots, H, D, Dv]; cu_q None => one token per sequence
// max_q_len: host-side bound on the longest sequence chunk (0 = unknown);
// long chunks take the chunk-parallel path
void decay_attn(Tensor out, Tensor q, Tensor k, Tensor v, Tensor decay,
                Tensor state, Tensor slots, c10::optional<Tensor> cu_q,
                Tensor ctx_lens, long max_q_len) {
  CHK_F32C(out); CHK_ACT(q); CHK_ACT(k); CHK_ACT(v); CHK_F32C(decay);
  CHK_F32C(state); CHK_I32C(slots); CHK_I32C(ctx_lens);
  TORCH_CHECK(state.dim() == 4 && q.dim() == 2 && k.dim() == 2 &&
              v.dim() == 2 && q.dtype() == k.dtype() && q.dtype() == v.dtype());
  const int H = state.size(1), D = state.size(2), Dv = state.size(3);
  const int T = q.size(0);
  TORCH_CHECK(q.size(1) == H * D && k.size(1) == H * D && v.size(1) == H * Dv &&
              k.size(0) == T && v.size(0) == T && decay.numel() == H);
  TORCH_CHECK(D <= 256, "key dim > 256 unsupported");
  TORCH_CHECK(out.numel() == (long)T * H * Dv);
  const int n_seqs = slots.numel();
  TORCH_CHECK(ctx_lens.numel() == n_seqs);
  const int* cu = nullptr;
  if (cu_q.has_value()) {
    CHK_I32C(*cu_q);
    TORCH_CHECK(cu_q->numel() == n_seqs + 1);
    cu = ptr<int>(*cu_q);
  } else {
    TORCH_CHECK(n_seqs == T, "decode: one sequence per token");
  }
  int chunk = 128, max_chunks = 1;
  Tensor ws;
  if (cu != nullptr) {
    const long bound = max_q_len > 0 ? std::min<long>(max_q_len, T) : T;
    const long per_seq = (long)H * D * Dv * 4;
    while ((bound + chunk - 1) / chunk * n_seqs * per_seq > (1L << 31))
      chunk *= 2;                             // keep the scratch under 2 GiB
    if (bound >= 2L * chunk) {
      max_chunks = (int)((bound + chunk - 1) / chunk);
      ws = torch::empty({(long)n_seqs * max_chunks, (long)H, (long)D, (long)Dv},
                        state.options());
    }
  }
  float* wsp = max_chunks > 1 ? ptr<float>(ws) : nullptr;
  if (is_f32(q))
    hy::launch_decay_attn<float>(ptr<float>(out), ptr<float>(q), ptr<float>(k), ptr<float>(v), ptr<float>(decay), ptr<float>(state), ptr<int>(slots), cu, ptr<int>(ctx_lens), n_seqs, H, D, Dv, q.stride(0), k.stride(0), v.stride(0), chunk, max_chunks, wsp, cur());
  else
    hy::launch_decay_attn<bf>(ptr<float>(out), ptr<bf>(q), ptr<bf>(k), ptr<bf>(v), ptr<float>(decay), ptr<float>(state), ptr<int>(slots), cu, ptr<int>(ctx_lens), n_seqs, H, D, Dv, q.stride(0), k.stride(0), v.stride(0), chunk, max_chunks, wsp, cur());
}

// z fp32 [T, E] router logits -> ids int32 [T, top], wts fp32 [T, top]
void moe_route(Tensor ids, Tensor wts, Tensor z, long top, long n_groups,
               long keep, bool softmax, c10::optional<Tensor> correction,
               bool group_max, bool normalize) {
  CHK_I32C(ids); CHK_F32C(wts); CHK_F32C(z);
  TORCH_CHECK(z.dim() == 2);
  const int T = z.size(0), E = z.size(1);
  TORCH_CHECK(ids.numel() == (long)T * top && wts.numel() == (long)T * top);
  TORCH_CHECK(top >= 1 && top <= E && n_groups >= 1 && E % n_groups == 0 &&
              keep >= 1 && keep <= n_groups &&
              keep * (E / n_groups) >= top, "bad routing constants");
  TORCH_CHECK((2 * E + n_groups) * 4 <= 64 * 1024, "too many experts");
  const float* corr = nullptr;
  if (correction.has_value()) {
    CHK_F32C(*correction);
    TORCH_CHECK(correction->numel() == E);
    corr = ptr<float>(*correction);
  }
  hy::launch_moe_route(ptr<int>(ids), ptr<float>(wts), ptr<float>(z), T, E,
                       top, n_groups, keep, softmax, corr, group_max,
                       normalize, cur());
}

// out fp32 [T, width]; y [R, width] contiguous; rows int32 [T, top] < R, a
// negative row reads ident [T, width] (0 without one); extra [T, width] is
// added
void moe_combine(Tensor out, Tensor y, Tensor rows, Tensor wts,
                 c10::optional<Tensor> ident, c10::optional<Tensor> extra) {
  CHK_F32C(out); CHK_ACT(y); CHK_I32C(rows); CHK_F32C(wts);
  TORCH_CHECK(y.is_contiguous() && out.dim() == 2 && rows.dim() == 2);
  const long T = out.size(0);
  const int width = out.size(1), top = rows.size(1);
  TORCH_CHECK(rows.size(0) == T && wts.numel() == T * top &&
              y.size(-1) == width);
  const void *ip = nullptr, *ep = nullptr;
  long is = 0, es = 0;
  if (ident.has_value()) {
    CHK_ACT(*ident);
    TORCH_CHECK(ident->dim() == 2 && ident->size(0) == T &&
                ident->size(1) == width && ident->dtype() == y.dtype());
    ip = ident->data_ptr(); is = ident->stride(0);
  }
  if (extra.has_value()) {
    CHK_ACT(*extra);
    TORCH_CHECK(extra->dim() == 2 && extra->size(0) == T &&
                extra->size(1) == width && extra->dtype() == y.dtype());
    ep = extra->data_ptr(); es = extra->stride(0);
  }
  if (is_f32(y))
    hy::launch_moe_combine<float>(ptr<float>(out), ptr<float>(y), ptr<int>(rows), ptr<float>(wts), T, width, top, (const float*)ip, is, (const float*)ep, es, cur());
  else
    hy::launch_moe_combine<bf>(ptr<float>(out), ptr<bf>(y), ptr<int>(rows), ptr<float>(wts), T, width, top, (const bf*)ip, is, (const bf*)ep, es, cur());
}

// x fp32 [T, S, W]; out [T, W] = layernorm(sum_s w_in[s] x[:, s]) * g + b
void streams_mix_norm(Tensor out, Tensor x, c10::optional<Tensor> w_in,
                      Tensor g, Tensor b, double eps) {
  CHK_ACT(out); CHK_F32C(x); CHK_F32C(g); CHK_F32C(b);
  TORCH_CHECK(x.dim() == 3 && out.dim() == 2 && out.is_contiguous());
  const int T = x.size(0), S = x.size(1), W = x.size(2);
  TORCH_CHECK(out.size(0) == T && out.size(1) == W && g.numel() == W &&
              b.numel() == W && S >= 1 && S <= 8, "streams: bad shapes");
  TORCH_CHECK((size_t)W * 4 <= 60 * 1024, "width too large for LDS");
  const float* wi = nullptr;
  if (w_in.has_value()) {
    CHK_F32C(*w_in);
    TORCH_CHECK(w_in->numel() == S);
    wi = ptr<float>(*w_in);
  }
  if (is_f32(out))
    hy::launch_streams_mix_norm<float>(ptr<float>(out), ptr<float>(x), wi, ptr<float>(g), ptr<float>(b), eps, T, S, W, cur());
  else
    hy::launch_streams_mix_norm<bf>(ptr<bf>(out), ptr<float>(x), wi, ptr<float>(g), ptr<float>(b), eps, T, S, W, cur());
}

// x[:, j] <- sum_s mix[s, j] x[:, s] + w_out[j] (a1 y1 + a2 y2), in place
void streams_update(Tensor x, c10::optional<Tensor> mix,
                    c10::optional<Tensor> w_out, Tensor y1, double a1,
                    c10::optional<Tensor> y2, double a2) {
  CHK_F32C(x); CHK_ACT(y1);
  TORCH_CHECK(x.dim() == 3 && y1.is_contiguous());
  const long T = x.size(0);
  const int S = x.size(1), W = x.size(2);
  TORCH_CHECK(S >= 1 && S <= 8 && y1.numel() == T * W);
  const float *mp = nullptr, *op = nullptr;
  if (mix.has_value()) {
    CHK_F32C(*mix);
    TORCH_CHECK(mix->numel() == S * S);
    mp = ptr<float>(*mix);
  }
  if (w_out.has_value()) {
    CHK_F32C(*w_out);
    TORCH_CHECK(w_out->numel() == S);
    op = ptr<float>(*w_out);
  }
  const void* y2p = nullptr;
  if (y2.has_value()) {
    CHK_ACT(*y2);
    TORCH_CHECK(y2->is_contiguous() && y2->numel() == T * W &&
                y2->dtype() == y1.dtype());
    y2p = y2->data_ptr();
  }
  if (is_f32(y1))
    hy::launch_streams_update<float>(ptr<float>(x), mp, op, ptr<float>(y1), a1, (const float*)y2p, a2, T, S, W, cur());
  else
    hy::launch_streams_update<bf>(ptr<float>(x), mp, op, ptr<bf>(y1), a1, (const bf*)y2p, a2, T, S, W, cur());
}

// streams_update followed by streams_mix_norm of the new values, one pass
void streams_update_mix_norm(Tensor out, Tensor x, c10::optional<Tensor> mix,
                             c10::optional<Tensor> w_out, Tensor y1, double a1,
                             c10::optional<Tensor> y2, double a2,
                             c10::optional<Tensor> w_in, Tensor g, Tensor b,
                             double eps) {
  CHK_ACT(out); CHK_F32C(x); CHK_ACT(y1); CHK_F32C(g); CHK_F32C(b);
  TORCH_CHECK(x.dim() == 3 && y1.is_contiguous() && out.is_contiguous() &&
              out.dim() == 2 && out.dtype() == y1.dtype());
  const int T = x.size(0), S = x.size(1), W = x.size(2);
  TORCH_CHECK(S >= 1 && S <= 8 && y1.numel() == (long)T * W &&
              out.size(0) == T && out.size(1) == W && g.numel() == W &&
              b.numel() == W);
  TORCH_CHECK((size_t)W * 4 <= 60 * 1024, "width too large for LDS");
  auto opt = [&](const c10::optional<Tensor>& t, long n) -> const float* {
    if (!t.has_value()) return nullptr;
    CHK_F32C(*t);
    TORCH_CHECK(t->numel() == n);
    return ptr<float>(*t);
  };
  const float* mp = opt(mix, (long)S * S);
  const float* op = opt(w_out, S);
  const float* ip = opt(w_in, S);
  const void* y2p = nullptr;
  if (y2.has_value()) {
    CHK_ACT(*y2);
    TORCH_CHECK(y2->is_contiguous() && y2->numel() == (long)T * W &&
                y2->dtype() == y1.dtype());
    y2p = y2->data_ptr();
  }
  if (is_f32(y1))
    hy::launch_streams_update_mix_norm<float>(ptr<float>(out), ptr<float>(x), mp, op, ptr<float>(y1), a1, (const float*)y2p, a2, ip, ptr<float>(g), ptr<float>(b), eps, T, S, W, cur());
  else
    hy::launch_streams_update_mix_norm<bf>(ptr<bf>(out), ptr<float>(x), mp, op, ptr<bf>(y1), a1, (const bf*)y2p, a2, ip, ptr<float>(g), ptr<float>(b), eps, T, S, W, cur());
}

void relu_sq(Tensor x) {
  CHK_ACT(x);
  TORCH_CHECK(x.is_contiguous());
  if (is_f32(x)) hy::launch_relu_sq<float>(ptr<float>(x), x.numel(), cur());
  else hy::launch_relu_sq<bf>(ptr<bf>(x), x.numel(), cur());
}

void softcap(Tensor out, Tensor x, double cap) {
  CHK_F32C(out); CHK_ACT(x);
  TORCH_CHECK(x.is_contiguous() && out.numel() == x.numel() && cap > 0);
  if (is_f32(x)) hy::launch_softcap<float>(ptr<float>(out), ptr<float>(x), cap, x.numel(), cur());
  else hy::launch_softcap<bf>(ptr<float>(out), ptr<bf>(x), cap, x.numel(), cur());
}

// Short causal convolution of x [T, heads*hd] (row view) with per-channel
// filters w [heads*hd, taps]; the sequence's earlier inputs come from
// state[slot, :, state_off : state_off + heads*hd]. Result to `out` (row
// view) or into the paged `cache` [blocks, heads, block, hd] at slot_mapping.
void short_conv(c10::optional<Tensor> out, c10::optional<Tensor> cache,
                c10::optional<Tensor> slot_mapping, Tensor x, Tensor w,
                c10::optional<Tensor> bias, Tensor state, long state_off,
                Tensor slots, c10::optional<Tensor> cu_q, Tensor ctx_lens,
                long heads, long hd, bool act_silu, long rot_dims,
                c10::optional<Tensor> pos, c10::optional<Tensor> inv_freq) {
  CHK_ACT(x); CHK_ACT(w); CHK_ACT(state); CHK_I32C(slots); CHK_I32C(ctx_lens);
  TORCH_CHECK(x.dim() == 2 && w.dim() == 2 && w.is_contiguous() &&
              state.dim() == 3 && state.is_contiguous() &&
              w.dtype() == x.dtype() && state.dtype() == x.dtype());
  const int T = x.size(0), C = heads * hd, taps = w.size(1);
  TORCH_CHECK(x.size(1) == C && w.size(0) == C && taps >= 1 && taps <= 16 &&
              state.size(1) == taps - 1 && state_off >= 0 &&
              state_off + C <= state.size(2), "short_conv: bad shapes");
  const int n_seqs = slots.numel();
  TORCH_CHECK(ctx_lens.numel() == n_seqs);
  const int* cu = nullptr;
  if (cu_q.has_value()) {
    CHK_I32C(*cu_q);
    TORCH_CHECK(cu_q->numel() == n_seqs + 1);
    cu = ptr<int>(*cu_q);
  } else {
    TORCH_CHECK(n_seqs == T, "decode: one sequence per token");
  }
  const void* bp = nullptr;
  if (bias.has_value()) {
    CHK_ACT(*bias);
    TORCH_CHECK(bias->numel() == C && bias->is_contiguous() &&
                bias->dtype() == x.dtype());
    bp = bias->data_ptr();
  }
  const long* posp = nullptr;
  const double* fp = nullptr;
  if (rot_dims > 0) {
    TORCH_CHECK(pos.has_value() && inv_freq.has_value() && rot_dims % 2 == 0 &&
                rot_dims <= hd);
    CHK_I64C(*pos);
    TORCH_CHECK(pos->numel() == T && inv_freq->is_cuda() &&
                inv_freq->dtype() == torch::kDouble &&
                inv_freq->is_contiguous() &&
                inv_freq->numel() == rot_dims / 2);
    posp = ptr<long>(*pos);
    fp = ptr<double>(*inv_freq);
  }
  void* outp = nullptr;
  long out_stride = 0;
  void* cachep = nullptr;
  const long* smp = nullptr;
  int bs = 1;
  if (cache.has_value()) {
    CHK_ACT(*cache);
    TORCH_CHECK(slot_mapping.has_value());
    CHK_I64C(*slot_mapping);
    TORCH_CHECK(cache->dim() == 4 && cache->is_contiguous() &&
                cache->size(1) == heads && cache->size(3) == hd &&
                cache->dtype() == x.dtype() && slot_mapping->numel() == T);
    cachep = cache->data_ptr();
    smp = ptr<long>(*slot_mapping);
    bs = cache->size(2);
  } else {
    TORCH_CHECK(out.has_value());
    CHK_ACT(*out);
    TORCH_CHECK(out->dim() == 2 && out->size(0) == T && out->size(1) == C &&
                out->dtype() == x.dtype());
    outp = out->data_ptr();
    out_stride = out->stride(0);
  }
  if (is_f32(x))
    hy::launch_short_conv<float>((float*)outp, out_stride, (float*)cachep, smp, bs, ptr<float>(x), x.stride(0), ptr<float>(w), (const float*)bp, ptr<float>(state), state.size(2), state_off, ptr<int>(slots), cu, ptr<int>(ctx_lens), T, n_seqs, heads, hd, taps, act_silu, rot_dims, posp, fp, cur());
  else
    hy::launch_short_conv<bf>((bf*)outp, out_stride, (bf*)cachep, smp, bs, ptr<bf>(x), x.stride(0), ptr<bf>(w), (const bf*)bp, ptr<bf>(state), state.size(2), state_off, ptr<int>(slots), cu, ptr<int>(ctx_lens), T, n_seqs, heads, hd, taps, act_silu, rot_dims, posp, fp, cur());
}

// state [slots, taps-1, C] <- the last taps-1 inputs after this step's rows
void short_conv_state(Tensor state, Tensor x, Tensor slots,
                      c10::optional<Tensor> cu_q) {
  CHK_ACT(state); CHK_ACT(x); CHK_I32C(slots);
  TORCH_CHECK(state.dim() == 3 && state.is_contiguous() && x.dim() == 2 &&
              x.size(1) == state.size(2) && x.dtype() == state.dtype());
  const int n_seqs = slots.numel(), taps = state.size(1) + 1;
  const int* cu = nullptr;
  if (cu_q.has_value()) {
    CHK_I32C(*cu_q);
    TORCH_CHECK(cu_q->numel() == n_seqs + 1);
    cu = ptr<int>(*cu_q);
  } else {
    TORCH_CHECK(n_seqs == x.size(0), "decode: one sequence per token");
  }
  if (is_f32(x))
    hy::launch_short_conv_state<float>(ptr<float>(state), state.size(2), ptr<float>(x), x.stride(0), ptr<int>(slots), cu, n_seqs, x.size(1), taps, cur());
  else
    hy::launch_short_conv_state<bf>(ptr<bf>(state), state.size(2), ptr<bf>(x), x.stride(0), ptr<int>(slots), cu, n_seqs, x.size(1), taps, cur());
}

// kind 0: selective state space (q = C, k = B shared per group, v = x,
//   g = dt_raw [T, H]; p0 = dt_bias, p1 = A_log, p2 = D skip)
// kind 1: gated linear attention (g = z [T, H*D]; p0 = z bias [H*D];
//   c0 = 1/tau, c1 = query scale)
// out fp32 [T, H, Dv]; state fp32 [slots, H, D, Dv]; q/k [T, groups*D] views
void gated_recurrence(long kind, Tensor out, Tensor q, Tensor k, Tensor v,
                      Tensor g, Tensor p0, c10::optional<Tensor> p1,
                      c10::optional<Tensor> p2, double c0, double c1,
                      Tensor state, Tensor slots, c10::optional<Tensor> cu_q,
                      Tensor ctx_lens, long groups, long max_q_len) {
  CHK_F32C(out); CHK_ACT(q); CHK_ACT(k); CHK_ACT(v); CHK_ACT(g); CHK_F32C(p0);
  CHK_F32C(state); CHK_I32C(slots); CHK_I32C(ctx_lens);
  TORCH_CHECK(state.dim() == 4 && q.dim() == 2 && k.dim() == 2 &&
              v.dim() == 2 && g.dim() == 2 && q.dtype() == k.dtype() &&
              q.dtype() == v.dtype() && q.dtype() == g.dtype());
  const int H = state.size(1), D = state.size(2), Dv = state.size(3);
  const int T = q.size(0);
  TORCH_CHECK(kind == 0 || kind == 1);
  TORCH_CHECK(groups >= 1 && H % groups == 0 && q.size(1) == groups * D &&
              k.size(1) == groups * D && v.size(1) == H * Dv &&
              k.size(0) == T && v.size(0) == T && g.size(0) == T,
              "gated_recurrence: bad shapes");
  TORCH_CHECK(D <= 256, "key dim > 256 unsupported");
  TORCH_CHECK(out.numel() == (long)T * H * Dv);
  const float *p1p = nullptr, *p2p = nullptr;
  if (kind == 0) {
    TORCH_CHECK(g.size(1) == H && p0.numel() == H && p1.has_value());
    CHK_F32C(*p1);
    TORCH_CHECK(p1->numel() == H);
    p1p = ptr<float>(*p1);
    if (p2.has_value()) {
      CHK_F32C(*p2);
      TORCH_CHECK(p2->numel() == H);
      p2p = ptr<float>(*p2);
    }
  } else {
    TORCH_CHECK(groups == H && g.size(1) == H * D && p0.numel() == H * D);
  }
  const int n_seqs = slots.numel();
  TORCH_CHECK(ctx_lens.numel() == n_seqs);
  const int* cu = nullptr;
  if (cu_q.has_value()) {
    CHK_I32C(*cu_q);
    TORCH_CHECK(cu_q->numel() == n_seqs + 1);
    cu = ptr<int>(*cu_q);
  } else {
    TORCH_CHECK(n_seqs == T, "decode: one sequence per token");
  }
  int chunk = 128, max_chunks = 1;
  Tensor ws, wa;
  if (cu != nullptr) {
    const long bound = max_q_len > 0 ? std::min<long>(max_q_len, T) : T;
    const long per_seq = (long)H * D * Dv * 4;
    // tuning knob: piece length of the piece-parallel passes
    if (const char* e = std::getenv("XLLM_RECURRENCE_CHUNK"))
      chunk = std::min(1024, std::max(16, std::atoi(e)));
    // few heads: shorter pieces, so that the piece-parallel passes still
    // fill the chip
    while (chunk > 32 &&
           (bound + chunk - 1) / chunk * n_seqs * H * ((Dv + 63) / 64) < 1024)
      chunk /= 2;
    while ((bound + chunk - 1) / chunk * n_seqs * per_seq > (1L << 31))
      chunk *= 2;                             // keep the scratch under 2 GiB
    if (bound >= 2L * chunk) {
      max_chunks = (int)((bound + chunk - 1) / chunk);
      ws = torch::empty({(long)n_seqs * max_chunks, (long)H, (long)D, (long)Dv},
                        state.options());
      wa = torch::empty({(long)n_seqs * max_chunks, (long)H,
                         (long)(kind == 0 ? 1 : D)}, state.options());
    }
  }
  float* wsp = max_chunks > 1 ? ptr<float>(ws) : nullptr;
  float* wap = max_chunks > 1 ? ptr<float>(wa) : nullptr;
  if (is_f32(q))
    hy::launch_gated_recurrence<float>(kind, ptr<float>(out), ptr<float>(q), ptr<float>(k), ptr<float>(v), ptr<float>(g), q.stride(0), k.stride(0), v.stride(0), g.stride(0), ptr<float>(p0), p1p, p2p, c0, c1, ptr<float>(state), ptr<int>(slots), cu, ptr<int>(ctx_lens), n_seqs, H, groups, D, Dv, chunk, max_chunks, wsp, wap, cur());
  else
    hy::launch_gated_recurrence<bf>(kind, ptr<float>(out), ptr<bf>(q), ptr<bf>(k), ptr<bf>(v), ptr<bf>(g), q.stride(0), k.stride(0), v.stride(0), g.stride(0), ptr<float>(p0), p1p, p2p, c0, c1, ptr<float>(state), ptr<int>(slots), cu, ptr<int>(ctx_lens), n_seqs, H, groups, D, Dv, chunk, max_chunks, wsp, wap, cur());
}

// out [rows, n] from o fp32 [rows, n], gate [rows, n] (row view), w fp32 with
// n or n/groups entries
void gated_group_norm(Tensor out, Tensor o, Tensor w, Tensor gate, double eps,
                      long groups, bool act_silu, bool gate_first) {
  CHK_ACT(out); CHK_F32C(o); CHK_F32C(w); CHK_ACT(gate);
  TORCH_CHECK(out.is_contiguous() && out.dim() == 2 && gate.dim() == 2);
  const int rows = out.size(0), n = out.size(1);
  TORCH_CHECK(o.numel() == (long)rows * n && gate.size(0) == rows &&
              gate.size(1) == n && gate.dtype() == out.dtype() &&
              groups >= 1 && n % groups == 0 &&
              (w.numel() == n || w.numel() == n / groups));
  if (is_f32(out))
    hy::launch_gated_group_norm<float>(ptr<float>(out), ptr<float>(o), ptr<float>(w), w.numel(), ptr<float>(gate), gate.stride(0), eps, rows, n, groups, act_silu, gate_first, cur());
  else
    hy::launch_gated_group_norm<bf>(ptr<bf>(out), ptr<float>(o), ptr<float>(w), w.numel(), ptr<bf>(gate), gate.stride(0), eps, rows, n, groups, act_silu, gate_first, cur());
}

// out fp32 [T, H, Dv]; q [T, H*D] row view; caches [blocks, n_kv, bs, D|Dv]
void capped_attn(Tensor out, Tensor q, Tensor k_cache, Tensor v_cache,
                 Tensor block_tables, c10::optional<Tensor> cu_q,
                 Tensor seq_lens, long heads, double scale, double cap,
                 long window, c10::optional<Tensor> sink, long keep_first,
                 c10::optional<Tensor> head_scale) {
  CHK_F32C(out); CHK_ACT(q); CHK_ACT(k_cache); CHK_ACT(v_cache);
  CHK_I32C(block_tables); CHK_I32C(seq_lens);
  TORCH_CHECK(q.dim() == 2 && k_cache.dim() == 4 && v_cache.dim() == 4 &&
              k_cache.is_contiguous() && v_cache.is_contiguous() &&
              q.dtype() == k_cache.dtype() && q.dtype() == v_cache.dtype() &&
              block_tables.dim() == 2);
  const int T = q.size(0), n_kv = k_cache.size(1), bs = k_cache.size(2);
  const int D = k_cache.size(3), Dv = v_cache.size(3);
  TORCH_CHECK(q.size(1) == heads * D && heads % n_kv == 0 &&
              v_cache.size(1) == n_kv && v_cache.size(2) == bs &&
              v_cache.size(0) == k_cache.size(0) && Dv <= 64 * 8,
              "capped_attn: bad shapes");
  TORCH_CHECK(out.numel() == (long)T * heads * Dv);
  const int n_seqs = seq_lens.numel();
  TORCH_CHECK(block_tables.size(0) == n_seqs);
  const int* cu = nullptr;
  if (cu_q.has_value()) {
    CHK_I32C(*cu_q);
    TORCH_CHECK(cu_q->numel() == n_seqs + 1);
    cu = ptr<int>(*cu_q);
  } else {
    TORCH_CHECK(n_seqs == T, "decode: one sequence per token");
  }
  TORCH_CHECK(window >= 0 && window < (1L << 30), "bad window");
  const float* sinkp = nullptr;
  if (sink.has_value()) {
    CHK_F32C(*sink);
    TORCH_CHECK(sink->numel() == heads);
    sinkp = ptr<float>(*sink);
  }
  TORCH_CHECK(keep_first >= 0 && keep_first < (1L << 30) &&
              (keep_first == 0 || window > 0), "bad keep_first");
  const float* hsp = nullptr;
  if (head_scale.has_value()) {
    CHK_F32C(*head_scale);
    TORCH_CHECK(head_scale->numel() == heads);
    hsp = ptr<float>(*head_scale);
  }
  // bf16: MFMA kernel when the sizes fit one of its instantiations
  if (is_bf16(q) && hy::capped_attn_mfma_class(D, Dv) != 0 &&
      q.stride(0) % 8 == 0 &&
      reinterpret_cast<uintptr_t>(q.data_ptr()) % 16 == 0) {
    int n_part = 1;
    Tensor ws_acc, ws_ml;
    if (cu == nullptr) {
      // decode: split the context over workgroups when (token, key/value
      // head) pairs alone do not fill the chip; sizes known on the host only.
      // About four workgroups per CU measured best (batch 8..128, 1k-4k
      // context, 4-8 key/value heads).
      const int per = heads / n_kv;
      const int rows_wg = per <= 16 ? 16 : per <= 32 ? 32 : 64;
      const long wgs = (long)T * n_kv * ((per + rows_wg - 1) / rows_wg);
      long max_tiles = ((long)block_tables.size(1) * bs + 31) / 32;
      if (window > 0)
        max_tiles = std::min<long>(
            max_tiles, (window + 31) / 32 + 1 + (keep_first + 31) / 32);
      n_part = (int)std::min<long>(std::min<long>(32, (max_tiles + 1) / 2),
                                   std::max<long>(1, 1024 / wgs));
      n_part = std::max(n_part, 1);
      // tuning knob: fixed partition count (1..32)
      if (const char* e = std::getenv("XLLM_CAPPED_PARTS"))
        n_part = std::min(32, std::max(1, std::atoi(e)));
    }
    if (n_part > 1) {
      ws_acc = torch::empty({(long)T * heads * n_part, (long)Dv}, out.options());
      ws_ml = torch::empty({(long)T * heads * n_part, 2}, out.options());
    }
    hy::launch_capped_attn_mfma(
        ptr<float>(out), n_part > 1 ? ptr<float>(ws_acc) : nullptr,
        n_part > 1 ? ptr<float>(ws_ml) : nullptr, ptr<bf>(q), ptr<bf>(k_cache),
        ptr<bf>(v_cache), ptr<int>(block_tables), cu, ptr<int>(seq_lens), T,
        n_seqs, heads, n_kv, D, Dv, bs, block_tables.size(1), scale, cap,
        q.stride(0), n_part, window, sinkp, keep_first, hsp, cur());
    return;
  }
  TORCH_CHECK((size_t)4 * D * 4 <= 64 * 1024, "query row too wide for LDS");
  if (is_f32(q))
    hy::launch_capped_attn<float>(ptr<float>(out), ptr<float>(q), ptr<float>(k_cache), ptr<float>(v_cache), ptr<int>(block_tables), cu, ptr<int>(seq_lens), T, n_seqs, heads, n_kv, D, Dv, bs, block_tables.size(1), scale, cap, q.stride(0), window, sinkp, keep_first, hsp, cur());
  else
    hy::launch_capped_attn<bf>(ptr<float>(out), ptr<bf>(q), ptr<bf>(k_cache), ptr<bf>(v_cache), ptr<int>(block_tables), cu, ptr<int>(seq_lens), T, n_seqs, heads, n_kv, D, Dv, bs, block_tables.size(1), scale, cap, q.stride(0), window, sinkp, keep_first, hsp, cur());
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("group_rmsnorm", &group_rmsnorm);
  m.def("gated_norm_residual", &gated_norm_residual);
  m.def("norm_sigmoid_gate", &norm_sigmoid_gate);
  m.def("silu_mul", &silu_mul);
  m.def("rope_interleaved", &rope_interleaved);
  m.def("latent_kv_store", &latent_kv_store);
  m.def("latent_attn", &latent_attn);
  m.def("decay_attn", &decay_attn);
  m.def("moe_route", &moe_route);
  m.def("moe_combine", &moe_combine);
  m.def("streams_mix_norm", &streams_mix_norm);
  m.def("streams_update", &streams_update);
  m.def("streams_update_mix_norm", &streams_update_mix_norm);
  m.def("relu_sq", &relu_sq);
  m.def("softcap", &softcap);
  m.def("short_conv", &short_conv);
  m.def("short_conv_state", &short_conv_state);
  m.def("gated_recurrence", &gated_recurrence);
  m.def("gated_group_norm", &gated_group_norm);
  m.def("capped_attn", &capped_attn);
  m.def("norm_residual_add", &norm_residual_add);
  m.def("gelu_tanh_mul", &gelu_tanh_mul);
  m.def("rownorm_rope_store", &rownorm_rope_store);
  m.def("delta_rule", &delta_rule);
  m.def("rope_headnorm_store", &rope_headnorm_store);
  m.def("polynorm", &polynorm);
  m.def("gelu_tanh_gate", &gelu_tanh_gate);
}
