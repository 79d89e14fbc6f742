// Routed-expert support kernels: the router's selection (sigmoid or softmax
// scores, group-limited top-k over fp32 logits) and the weighted combine of
// expert outputs. The expert matrix products themselves are library GEMMs.
#include "hybrid_common.h"

namespace xllm {
namespace hyb {

// One wavefront per token; z [T, E] are the fp32 router logits (an fp32 GEMM
// upstream). Scores: sigmoid(z), or with `softmax` the softmax of z over all
// experts. The choice runs on score + corr (corr nullable); the weights are
// the plain scores, divided by their sum + 1e-20 with `normalize`.
// Experts form n_groups equal neighbouring groups; a group's score is the
// sum of its two largest choice scores (the largest one with `group_max`);
// only the `keep` best groups are eligible. ids/weights [T, top]: the
// eligible experts with the largest choice scores. Ties go to the lower
// index. Masked or taken entries hold -inf (choice scores may be negative).
__global__ void moe_route_kernel(int* __restrict__ ids,
                                 float* __restrict__ wts,
                                 const float* __restrict__ z, int E, int top,
                                 int n_groups, int keep, int softmax,
                                 const float* __restrict__ corr, int group_max,
                                 int normalize) {
  extern __shared__ float smem[];
  float* sc = smem;                 // [E] scores
  float* el = sc + E;               // [E] eligible choice score or -inf
  float* gsc = el + E;              // [n_groups]
  const int t = blockIdx.x;
  const int lane = threadIdx.x;
  if (softmax) {
    float mx = -INFINITY;
    for (int e = lane; e < E; e += 64) mx = fmaxf(mx, z[(long)t * E + e]);
    mx = wave_reduce_max(mx);
    float sum = 0.f;
    for (int e = lane; e < E; e += 64) {
      const float p = expf(z[(long)t * E + e] - mx);
      sc[e] = p;
      sum += p;
    }
    sum = wave_reduce_sum(sum);
    for (int e = lane; e < E; e += 64) sc[e] = sc[e] / sum;
  } else {
    for (int e = lane; e < E; e += 64) sc[e] = sigmoidf_(z[(long)t * E + e]);
  }
  __syncthreads();
  auto choice = [&](int e) { return corr ? sc[e] + corr[e] : sc[e]; };
  const int gsz = E / n_groups;
  if (n_groups > 1) {
    for (int g = lane; g < n_groups; g += 64) {
      float a = -INFINITY, b = -INFINITY;      // two largest
      for (int i = 0; i < gsz; ++i) {
        const float x = choice(g * gsz + i);
        if (x > a) { b = a; a = x; } else if (x > b) { b = x; }
      }
      gsc[g] = (group_max || gsz < 2) ? a : a + b;
    }
    __syncthreads();
    for (int e = lane; e < E; e += 64) el[e] = -INFINITY;
    __syncthreads();
    if (lane == 0) {
      for (int kk = 0; kk < keep; ++kk) {
        int best = -1; float bv = -INFINITY;
        for (int g = 0; g < n_groups; ++g)
          if (gsc[g] > bv) { bv = gsc[g]; best = g; }
        if (best < 0) break;
        gsc[best] = -INFINITY;
        for (int i = 0; i < gsz; ++i)
          el[best * gsz + i] = choice(best * gsz + i);
      }
    }
    __syncthreads();
  } else {
    for (int e = lane; e < E; e += 64) el[e] = choice(e);
    __syncthreads();
  }
  for (int kk = 0; kk < top; ++kk) {
    float bv = -INFINITY; int bi = 0x7fffffff;
    for (int e = lane; e < E; e += 64)
      if (el[e] > bv) { bv = el[e]; bi = e; }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float ov = __shfl_xor(bv, off, 64);
      const int oi = __shfl_xor(bi, off, 64);
      if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
    }
    if (bi == 0x7fffffff) bi = 0;   // fewer eligible experts than top
    if (lane == 0) {
      ids[(long)t * top + kk] = bi;
      wts[(long)t * top + kk] = sc[bi];
      el[bi] = -INFINITY;
    }
    __syncthreads();
  }
  if (normalize && lane == 0) {
    float sum = 0.f;
    for (int kk = 0; kk < top; ++kk) sum += wts[(long)t * top + kk];
    sum += 1e-20f;
    for (int kk = 0; kk < top; ++kk)
      wts[(long)t * top + kk] = wts[(long)t * top + kk] / sum;
  }
}

// out[t, c] = sum_k wts[t, k] * y[rows[t, k], c] (+ extra[t, c]); a negative
// row reads ident[t, c] (an expert whose output is its input). fp32 sums.
template <typename T>
__global__ void moe_combine_kernel(float* __restrict__ out,
                                   const T* __restrict__ y,
                                   const int* __restrict__ rows,
                                   const float* __restrict__ wts, long tokens,
                                   int width, int top,
                                   const T* __restrict__ ident,
                                   long ident_stride,
                                   const T* __restrict__ extra,
                                   long extra_stride) {
  const long n = tokens * (long)width;
  for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < n;
       idx += (long)gridDim.x * blockDim.x) {
    const long t = idx / width;
    const int c = (int)(idx - t * width);
    float a = 0.f;
    for (int kk = 0; kk < top; ++kk) {
      const int r = rows[t * top + kk];
      float v = 0.f;
      if (r >= 0) v = IO<T>::ld(y + (long)r * width + c);
      else if (ident != nullptr) v = IO<T>::ld(ident + t * ident_stride + c);
      a += wts[t * top + kk] * v;
    }
    if (extra != nullptr) a += IO<T>::ld(extra + t * extra_stride + c);
    out[idx] = a;
  }
}

void launch_moe_route(int* ids, float* wts, const float* z, int tokens, int E,
                      int top, int n_groups, int keep, int softmax,
                      const float* corr, int group_max, int normalize,
                      hipStream_t st) {
  if (tokens == 0) return;
  const size_t lds = (size_t)(2 * E + n_groups) * sizeof(float);
  hipLaunchKernelGGL(moe_route_kernel, dim3(tokens), dim3(64), lds, st, ids,
                     wts, z, E, top, n_groups, keep, softmax, corr, group_max,
                     normalize);
}

template <typename T>
void launch_moe_combine(float* out, const T* y, const int* rows,
                        const float* wts, long tokens, int width, int top,
                        const T* ident, long ident_stride, const T* extra,
                        long extra_stride, hipStream_t st) {
  const long n = tokens * (long)width;
  if (n == 0) return;
  const int blocks = (int)((n + 255) / 256 < 65535 ? (n + 255) / 256 : 65535);
  hipLaunchKernelGGL((moe_combine_kernel<T>), dim3(blocks), dim3(256), 0, st,
                     out, y, rows, wts, tokens, width, top, ident,
                     ident_stride, extra, extra_stride);
}

#define INST_MOE(T)                                                          \
  template void launch_moe_combine<T>(float*, const T*, const int*,          \
                                      const float*, long, int, int,          \
                                      const T*, long, const T*, long,        \
                                      hipStream_t);
INST_MOE(float)
INST_MOE(unsigned short)

}  // namespace hyb
}  // namespace xllm
