// Causal softmax attention over a paged key/value cache with grouped
// key/value heads, separate key and value widths, a free score scale and an
// optional tanh soft cap on the scores:
//
//   s_ij = scale * (q_i . k_j);  s_ij <- cap * tanh(s_ij / cap);
//   o_i  = sum_j softmax_j(s_ij) v_j        over keys j <= i
//
// Optional: a sliding window (only the keys with i - j < window are seen; with
// keep_first the keys j < keep_first stay visible beside it), a per-head sink,
// a score without key or value whose exponential joins the softmax
// denominator, and one more score multiplier per head.
//
// Caches: keys [blocks, n_kv, block, D], values [blocks, n_kv, block, Dv].
// Scores, softmax weights and the weighted sum are fp32 for both storage
// types. One wavefront per (query token, head): 64 keys are scored per step,
// one per lane, then the lanes switch to owning output columns.
#include "hybrid_common.h"

namespace xllm {
namespace hyb {

constexpr int CA_MAX_ACC = 8;   // Dv <= 64 * 8

// q [T, H, D] (row stride given), out fp32 [T, H, Dv].
// cu_q == nullptr: decode (token t is sequence t, sees seq_lens[t] keys);
// else token t of sequence s sees seq_lens[s] - (cu_q[s+1] - 1 - t) keys.
template <typename T>
__global__ void capped_attn_kernel(
    float* __restrict__ out, const T* __restrict__ q,
    const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ block_tables, const int* __restrict__ cu_q,
    const int* __restrict__ seq_lens, int n_seqs, int heads, int n_kv, int D,
    int Dv, int block_size, int table_width, float scale, float cap,
    long q_row_stride, int window, const float* __restrict__ sink,
    int keep_first, const float* __restrict__ head_scale) {
  extern __shared__ float smem[];
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  const int nw = blockDim.x >> 6;
  const int h = blockIdx.y * nw + wid;

  int s, n_keys;
  if (cu_q == nullptr) {
    s = t;
    n_keys = seq_lens[t];
  } else {
    int lo = 0, hi = n_seqs - 1;          // last s with cu_q[s] <= t
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (cu_q[mid] <= t) lo = mid; else hi = mid - 1;
    }
    s = lo;
    n_keys = seq_lens[s] - (cu_q[s + 1] - 1 - t);
  }
  const bool active = h < heads;           // uniform per wave
  float* qs = smem + wid * D;
  if (active) {
    const T* qrow = q + (long)t * q_row_stride + (long)h * D;
    for (int i = lane; i < D; i += 64) qs[i] = IO<T>::ld(qrow + i);
  }
  __syncthreads();
  if (!active) return;

  const int kvh = h / (heads / n_kv);
  const int* table = block_tables + (long)s * table_width;
  const float inv_cap = cap > 0.f ? 1.0f / cap : 0.f;
  const float hs = head_scale != nullptr ? head_scale[h] : 1.0f;
  float m = -INFINITY, l = 0.f;
  float acc[CA_MAX_ACC];
#pragma unroll
  for (int i = 0; i < CA_MAX_ACC; ++i) acc[i] = 0.f;
  const int n_acc = (Dv + 63) >> 6;

  // two key ranges: the kept first keys that lie before the window, then
  // the window itself (all keys without one)
  const int k_first = window > 0 ? max(0, n_keys - window) : 0;
  const int kept = window > 0 ? min(keep_first, k_first) : 0;
  for (int seg = 0; seg < 2; ++seg) {
  const int seg_lo = seg == 0 ? 0 : k_first;
  const int seg_hi = seg == 0 ? kept : n_keys;
  for (int k0 = seg_lo; k0 < seg_hi; k0 += 64) {
    const int key = k0 + lane;
    float sc = -INFINITY;
    if (key < seg_hi) {
      const long blk = table[key / block_size];
      const T* krow = k_cache +
          ((blk * n_kv + kvh) * block_size + key % block_size) * (long)D;
      float d = 0.f;
      for (int i = 0; i < D; ++i) d += qs[i] * IO<T>::ld(krow + i);
      sc = d * scale * hs;
      if (cap > 0.f) sc = cap * tanhf(sc * inv_cap);
    }
    const float m_new = fmaxf(m, wave_reduce_max(sc));
    const float alpha = expf(m - m_new);         // m=-inf first: exp(-inf)=0
    const float p = (key < seg_hi) ? expf(sc - m_new) : 0.f;
    l = l * alpha + wave_reduce_sum(p);
    m = m_new;
#pragma unroll
    for (int i = 0; i < CA_MAX_ACC; ++i) acc[i] *= alpha;
    const int nk = min(64, seg_hi - k0);
    for (int j = 0; j < nk; ++j) {
      const float pj = __shfl(p, j, 64);
      const int kj = k0 + j;
      const long blk = table[kj / block_size];
      const T* vrow = v_cache +
          ((blk * n_kv + kvh) * block_size + kj % block_size) * (long)Dv;
#pragma unroll
      for (int i = 0; i < CA_MAX_ACC; ++i) {
        const int c = lane + 64 * i;
        if (i < n_acc && c < Dv) acc[i] += pj * IO<T>::ld(vrow + c);
      }
    }
  }
  }
  if (sink != nullptr) {                  // a key without a value
    const float sk = sink[h];
    const float m_new = fmaxf(m, sk);
    const float alpha = expf(m - m_new);
    l = l * alpha + expf(sk - m_new);
#pragma unroll
    for (int i = 0; i < CA_MAX_ACC; ++i) acc[i] *= alpha;
  }
  const float inv = (l > 0.f) ? 1.0f / l : 0.f;
  float* orow = out + ((long)t * heads + h) * Dv;
#pragma unroll
  for (int i = 0; i < CA_MAX_ACC; ++i) {
    const int c = lane + 64 * i;
    if (i < n_acc && c < Dv) orow[c] = acc[i] * inv;
  }
}

template <typename T>
void launch_capped_attn(float* out, const T* q, const T* k_cache,
                        const T* v_cache, const int* block_tables,
                        const int* cu_q, const int* seq_lens, int tokens,
                        int n_seqs, int heads, int n_kv, int D, int Dv,
                        int block_size, int table_width, float scale,
                        float cap, long q_row_stride, int window,
                        const float* sink, int keep_first,
                        const float* head_scale, hipStream_t st) {
  if (tokens == 0) return;
  const int nw = heads < 4 ? heads : 4;
  dim3 grid(tokens, (heads + nw - 1) / nw);
  hipLaunchKernelGGL((capped_attn_kernel<T>), grid, dim3(64 * nw),
                     (size_t)nw * D * sizeof(float), st, out, q, k_cache,
                     v_cache, block_tables, cu_q, seq_lens, n_seqs, heads,
                     n_kv, D, Dv, block_size, table_width, scale, cap,
                     q_row_stride, window, sink, keep_first, head_scale);
}

#define INST_CA(T)                                                          \
  template void launch_capped_attn<T>(                                      \
      float*, const T*, const T*, const T*, const int*, const int*,         \
      const int*, int, int, int, int, int, int, int, int, float, float,     \
      long, int, const float*, int, const float*, hipStream_t);
INST_CA(float)
INST_CA(unsigned short)

}  // namespace hyb
}  // namespace xllm
