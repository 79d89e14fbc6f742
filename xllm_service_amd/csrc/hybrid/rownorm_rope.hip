// Query/key preparation for attention with a norm over the WHOLE projection:
//
//   q' = q / rms(q[0 : H*D]) * wq        (one rms for all heads of a token)
//   k' = k / rms(k[0 : G*D]) * wk
//
// followed by a rotary turn in the rotate-half layout on the first `rot`
// entries of every head: entry i pairs with entry i + rot/2,
//   (u, v) -> (u cos a - v sin a, v cos a + u sin a),  a = pos * f_i
// (angle and sincos in fp64, the turn in fp32). q' goes to a contiguous row
// tensor, k' and the untouched v into the paged caches
// [blocks, n_kv, block, D | Dv] at the token's slot (slot < 0: not stored).
// One workgroup per token; cos/sin of the token are made once in LDS.
#include "hybrid_common.h"

namespace xllm {
namespace hyb {

template <typename T>
__global__ void __launch_bounds__(256) rownorm_rope_store_kernel(
    T* __restrict__ q_out, const T* __restrict__ q, const T* __restrict__ k,
    const T* __restrict__ v, long q_stride, long k_stride, long v_stride,
    const float* __restrict__ wq, const float* __restrict__ wk, float eps,
    const long* __restrict__ pos, const double* __restrict__ inv_freq,
    int rot, int heads, int n_kv, int D, int Dv, T* __restrict__ k_cache,
    T* __restrict__ v_cache, const long* __restrict__ slot_mapping,
    int block_size) {
  extern __shared__ float cs[];           // [rot/2] cos, [rot/2] sin
  __shared__ float tmp[16];
  const int t = blockIdx.x, tid = threadIdx.x;
  const int half = rot >> 1;
  const T* qr = q + (long)t * q_stride;
  const T* kr = k + (long)t * k_stride;
  const int nq = heads * D, nk = n_kv * D;
  for (int i = tid; i < half; i += 256) {
    double s, c;
    sincos((double)pos[t] * inv_freq[i], &s, &c);
    cs[i] = (float)c;
    cs[half + i] = (float)s;
  }
  float sq = 0.f, sk = 0.f;
  for (int i = tid; i < nq; i += 256) {
    const float x = IO<T>::ld(qr + i);
    sq += x * x;
  }
  for (int i = tid; i < nk; i += 256) {
    const float x = IO<T>::ld(kr + i);
    sk += x * x;
  }
  sq = block_reduce_sum(sq, tmp);
  __syncthreads();
  sk = block_reduce_sum(sk, tmp);
  __syncthreads();
  const float rq = 1.0f / sqrtf(sq / (float)nq + eps);
  const float rk = 1.0f / sqrtf(sk / (float)nk + eps);

  // entry d of a head: the partner of a rotated entry and its role
  auto turned = [&](const T* row, const float* w, float rs, int base, int d) {
    const float x = IO<T>::ld(row + base + d) * rs * w[base + d];
    if (d >= rot) return x;
    const bool first = d < half;
    const int i = first ? d : d - half;
    const int pd = first ? d + half : d - half;
    const float y = IO<T>::ld(row + base + pd) * rs * w[base + pd];
    const float c = cs[i], s = cs[half + i];
    return first ? x * c - y * s : x * c + y * s;
  };
  T* qo = q_out + (long)t * nq;
  for (int i = tid; i < nq; i += 256) {
    const int hh = i / D, d = i - hh * D;
    IO<T>::st(qo + i, turned(qr, wq, rq, hh * D, d));
  }
  const long slot = slot_mapping[t];
  if (slot < 0) return;
  const long blk = slot / block_size, off = slot % block_size;
  for (int i = tid; i < nk; i += 256) {
    const int g = i / D, d = i - g * D;
    IO<T>::st(k_cache + ((blk * n_kv + g) * block_size + off) * (long)D + d,
              turned(kr, wk, rk, g * D, d));
  }
  const T* vr = v + (long)t * v_stride;
  for (int i = tid; i < n_kv * Dv; i += 256) {
    const int g = i / Dv, d = i - g * Dv;
    v_cache[((blk * n_kv + g) * block_size + off) * (long)Dv + d] = vr[i];
  }
}

template <typename T>
void launch_rownorm_rope_store(T* q_out, const T* q, const T* k, const T* v,
                               long q_stride, long k_stride, long v_stride,
                               const float* wq, const float* wk, float eps,
                               const long* pos, const double* inv_freq,
                               int rot, int tokens, int heads, int n_kv, int D,
                               int Dv, T* k_cache, T* v_cache,
                               const long* slot_mapping, int block_size,
                               hipStream_t st) {
  if (tokens == 0) return;
  hipLaunchKernelGGL((rownorm_rope_store_kernel<T>), dim3(tokens), dim3(256),
                     (size_t)(rot > 0 ? rot : 1) * sizeof(float), st, q_out, q,
                     k, v, q_stride, k_stride, v_stride, wq, wk, eps, pos,
                     inv_freq, rot, heads, n_kv, D, Dv, k_cache, v_cache,
                     slot_mapping, block_size);
}

#define INST_RR(T)                                                            \
  template void launch_rownorm_rope_store<T>(                                 \
      T*, const T*, const T*, const T*, long, long, long, const float*,       \
      const float*, float, const long*, const double*, int, int, int, int,    \
      int, int, T*, T*, const long*, int, hipStream_t);
INST_RR(float)
INST_RR(unsigned short)

}  // namespace hyb
}  // namespace xllm
