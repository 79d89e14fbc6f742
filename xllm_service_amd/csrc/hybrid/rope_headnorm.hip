// Query/key preparation for attention with a norm per HEAD after the turn,
// and two row-wise activations of feed-forwards.
//
// rope_headnorm_store: rotary turn on the first `rot` entries of every head,
//   (u, v) -> (u cos a - v sin a, v cos a + u sin a),  a = pos * f_i,
// with the pair (u, v) = entries (2i, 2i+1) of the head (`pairs`) or entries
// (i, i + rot/2); then, with `unit`, the head is divided by its root mean
// square sqrt(mean(x^2) + eps). Angle and sincos in fp64, the turn and the
// norm in fp32. q' goes to a contiguous row tensor, k' and the untouched v
// (when there is one) into the paged caches [blocks, n_kv, block, D | Dv] at
// the token's slot (slot < 0: not stored). One workgroup per token; cos/sin
// of the token are made once in LDS; a wave owns a head at a time and keeps
// the head's entries in registers between the sum of squares and the store.
//
// polynorm: out = c0 N(z) + c1 N(z^2) + c2 N(z^3) + c3 per row, N(u) = u /
// sqrt(mean(u^2) + eps); powers element by element; fp32 inside.
//
// gelu_tanh_gate: out = gelu_tanh(g) * u for two row views.
#include "hybrid_common.h"

namespace xllm {
namespace hyb {

constexpr int RH_MAX = 8;      // head size <= 64 * 8

template <typename T>
__global__ void __launch_bounds__(256) rope_headnorm_store_kernel(
    T* __restrict__ q_out, const T* __restrict__ q, const T* __restrict__ k,
    const T* __restrict__ v, long q_stride, long k_stride, long v_stride,
    const long* __restrict__ pos, const double* __restrict__ inv_freq, int rot,
    int pairs, int unit, float eps, int heads, int n_kv, int D, int Dv,
    T* __restrict__ k_cache, T* __restrict__ v_cache,
    const long* __restrict__ slot_mapping, int block_size) {
  extern __shared__ float cs[];           // [rot/2] cos, [rot/2] sin
  const int t = blockIdx.x, tid = threadIdx.x;
  const int lane = tid & 63, wv = tid >> 6;
  const int half = rot >> 1;
  for (int i = tid; i < half; i += 256) {
    double s, c;
    sincos((double)pos[t] * inv_freq[i], &s, &c);
    cs[i] = (float)c;
    cs[half + i] = (float)s;
  }
  __syncthreads();
  const long slot = slot_mapping[t];
  const long blk = slot >= 0 ? slot / block_size : 0;
  const long off = slot >= 0 ? slot % block_size : 0;
  for (int u = wv; u < heads + n_kv; u += 4) {       // uniform per wave
    const bool is_q = u < heads;
    const int g = u - heads;
    if (!is_q && slot < 0) continue;
    const T* src = is_q ? q + (long)t * q_stride + (long)u * D
                        : k + (long)t * k_stride + (long)g * D;
    T* dst = is_q ? q_out + ((long)t * heads + u) * D
                  : k_cache + ((blk * n_kv + g) * block_size + off) * (long)D;
    float val[RH_MAX];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < RH_MAX; ++j) {
      const int d = lane + 64 * j;
      float x = 0.f;
      if (d < D) {
        x = IO<T>::ld(src + d);
        if (d < rot) {
          bool first; int i, pd;
          if (pairs) { first = !(d & 1); i = d >> 1; pd = d ^ 1; }
          else { first = d < half; i = first ? d : d - half;
                 pd = first ? d + half : d - half; }
          const float y = IO<T>::ld(src + pd);
          const float c = cs[i], s = cs[half + i];
          x = first ? x * c - y * s : x * c + y * s;
        }
      }
      val[j] = x;
      ss += x * x;
    }
    float rs = 1.f;
    if (unit) rs = 1.0f / sqrtf(wave_reduce_sum(ss) / (float)D + eps);
#pragma unroll
    for (int j = 0; j < RH_MAX; ++j) {
      const int d = lane + 64 * j;
      if (d < D) IO<T>::st(dst + d, val[j] * rs);
    }
  }
  if (v == nullptr || slot < 0) return;
  const T* vr = v + (long)t * v_stride;
  for (int i = tid; i < n_kv * Dv; i += 256) {
    const int g = i / Dv, d = i - g * Dv;
    v_cache[((blk * n_kv + g) * block_size + off) * (long)Dv + d] = vr[i];
  }
}

template <typename T>
__global__ void __launch_bounds__(256) polynorm_kernel(
    T* __restrict__ out, const T* __restrict__ z,
    const float* __restrict__ coef, float eps, int F, long z_stride) {
  __shared__ float tmp[16];
  const long row = blockIdx.x;
  const T* zr = z + row * z_stride;
  T* orow = out + row * (long)F;
  float s2 = 0.f, s4 = 0.f, s6 = 0.f;
  for (int i = threadIdx.x; i < F; i += 256) {
    const float x = IO<T>::ld(zr + i);
    const float x2 = x * x;
    s2 += x2; s4 += x2 * x2; s6 += x2 * x2 * x2;
  }
  s2 = block_reduce_sum(s2, tmp);
  __syncthreads();
  s4 = block_reduce_sum(s4, tmp);
  __syncthreads();
  s6 = block_reduce_sum(s6, tmp);
  const float inv = 1.0f / (float)F;
  const float a = coef[0] / sqrtf(s2 * inv + eps);
  const float b = coef[1] / sqrtf(s4 * inv + eps);
  const float c = coef[2] / sqrtf(s6 * inv + eps);
  const float e = coef[3];
  for (int i = threadIdx.x; i < F; i += 256) {
    const float x = IO<T>::ld(zr + i);
    const float x2 = x * x;
    IO<T>::st(orow + i, a * x + b * x2 + c * (x2 * x) + e);
  }
}

template <typename T>
__global__ void gelu_tanh_gate_kernel(T* __restrict__ out,
                                      const T* __restrict__ g,
                                      const T* __restrict__ u, long rows,
                                      int F, long g_stride, long u_stride) {
  const long n = rows * (long)F;
  for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < n;
       idx += (long)gridDim.x * blockDim.x) {
    const long r = idx / F;
    const int i = (int)(idx - r * F);
    const float x = IO<T>::ld(g + r * g_stride + i);
    const float y = IO<T>::ld(u + r * u_stride + i);
    const float gl =
        0.5f * x *
        (1.0f + tanhf(0.7978845608028654f * (x + 0.044715f * x * x * x)));
    IO<T>::st(out + idx, gl * y);
  }
}

template <typename T>
void launch_rope_headnorm_store(T* q_out, const T* q, const T* k, const T* v,
                                long q_stride, long k_stride, long v_stride,
                                const long* pos, const double* inv_freq,
                                int rot, int pairs, int unit, float eps,
                                int tokens, int heads, int n_kv, int D, int Dv,
                                T* k_cache, T* v_cache,
                                const long* slot_mapping, int block_size,
                                hipStream_t st) {
  if (tokens == 0) return;
  hipLaunchKernelGGL((rope_headnorm_store_kernel<T>), dim3(tokens), dim3(256),
                     (size_t)(rot > 0 ? rot : 1) * sizeof(float), st, q_out, q,
                     k, v, q_stride, k_stride, v_stride, pos, inv_freq, rot,
                     pairs, unit, eps, heads, n_kv, D, Dv, k_cache, v_cache,
                     slot_mapping, block_size);
}

template <typename T>
void launch_polynorm(T* out, const T* z, const float* coef, float eps,
                     long rows, int F, long z_stride, hipStream_t st) {
  if (rows == 0) return;
  hipLaunchKernelGGL((polynorm_kernel<T>), dim3((unsigned)rows), dim3(256), 0,
                     st, out, z, coef, eps, F, z_stride);
}

template <typename T>
void launch_gelu_tanh_gate(T* out, const T* g, const T* u, long rows, int F,
                           long g_stride, long u_stride, hipStream_t st) {
  const long n = rows * (long)F;
  if (n == 0) return;
  const int blocks = (int)((n + 255) / 256 < 65535 ? (n + 255) / 256 : 65535);
  hipLaunchKernelGGL((gelu_tanh_gate_kernel<T>), dim3(blocks), dim3(256), 0,
                     st, out, g, u, rows, F, g_stride, u_stride);
}

#define INST_RH(T)                                                            \
  template void launch_rope_headnorm_store<T>(                                \
      T*, const T*, const T*, const T*, long, long, long, const long*,        \
      const double*, int, int, int, float, int, int, int, int, int, T*, T*,   \
      const long*, int, hipStream_t);                                         \
  template void launch_polynorm<T>(T*, const T*, const float*, float, long,   \
                                   int, long, hipStream_t);                   \
  template void launch_gelu_tanh_gate<T>(T*, const T*, const T*, long, int,   \
                                         long, long, hipStream_t);
INST_RH(float)
INST_RH(unsigned short)

}  // namespace hyb
}  // namespace xllm
