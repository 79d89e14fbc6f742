// Grouped RMS norm, gated+scaled residual update, gated output norm,
// SiLU-multiply, interleaved-pair rotary rotation. One workgroup per row;
// reductions per group run in a single wavefront (64 lanes).
#include "hybrid_common.h"

namespace xllm {
namespace hyb {

// out[row] = x[row] / rms_group(x[row]) * w       (groups equal parts)
template <typename TI, typename TO>
__global__ void group_rmsnorm_kernel(TO* __restrict__ out,
                                     const TI* __restrict__ x,
                                     const float* __restrict__ w, float eps,
                                     int width, int groups, long x_stride) {
  const int row = blockIdx.x;
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  const int nw = blockDim.x >> 6;
  const int gs = width / groups;
  const TI* xr = x + (long)row * x_stride;
  TO* orow = out + (long)row * width;
  for (int g = wid; g < groups; g += nw) {
    float ss = 0.f;
    for (int i = lane; i < gs; i += 64) {
      float v = IO<TI>::ld(xr + g * gs + i);
      ss += v * v;
    }
    ss = wave_reduce_sum(ss);
    const float rs = 1.0f / sqrtf(ss / (float)gs + eps);
    for (int i = lane; i < gs; i += 64) {
      const int c = g * gs + i;
      IO<TO>::st(orow + c, IO<TI>::ld(xr + c) * rs * w[c]);
    }
  }
}

// res[row] += mult * ls * group_rmsnorm(y * sigmoid(gate + bias)) * w
template <typename TY, typename TG>
__global__ void gated_norm_residual_kernel(
    float* __restrict__ res, const TY* __restrict__ y,
    const TG* __restrict__ gate, const float* __restrict__ bias,
    const float* __restrict__ w, const float* __restrict__ ls, float mult,
    float eps, int width, int groups, long gate_stride) {
  const int row = blockIdx.x;
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  const int nw = blockDim.x >> 6;
  const int gs = width / groups;
  const TY* yr = y + (long)row * width;
  const TG* gr = gate + (long)row * gate_stride;
  float* rr = res + (long)row * width;
  for (int g = wid; g < groups; g += nw) {
    float ss = 0.f;
    for (int i = lane; i < gs; i += 64) {
      const int c = g * gs + i;
      float z = IO<TY>::ld(yr + c) *
                sigmoidf_(IO<TG>::ld(gr + c) + (bias ? bias[c] : 0.f));
      ss += z * z;
    }
    ss = wave_reduce_sum(ss);
    const float rs = 1.0f / sqrtf(ss / (float)gs + eps);
    for (int i = lane; i < gs; i += 64) {
      const int c = g * gs + i;
      float z = IO<TY>::ld(yr + c) *
                sigmoidf_(IO<TG>::ld(gr + c) + (bias ? bias[c] : 0.f));
      rr[c] += mult * ls[c] * (z * rs * w[c]);
    }
  }
}

// out = (w ? o / rms(o) * w : o) * sigmoid(gate);  o fp32 [rows, n]; gate
// entry i / gate_cols serves column i (gate_cols = head width: one gate
// number per head)
template <typename T>
__global__ void norm_sigmoid_gate_kernel(T* __restrict__ out,
                                         const float* __restrict__ o,
                                         const float* __restrict__ w,
                                         const T* __restrict__ gate,
                                         float eps, int n, long gate_stride,
                                         int gate_cols) {
  __shared__ float tmp[16];
  const int row = blockIdx.x;
  const float* orow = o + (long)row * n;
  const T* gr = gate + (long)row * gate_stride;
  float rs = 1.0f;
  if (w) {
    float ss = 0.f;
    for (int i = threadIdx.x; i < n; i += blockDim.x) ss += orow[i] * orow[i];
    ss = block_reduce_sum(ss, tmp);
    rs = 1.0f / sqrtf(ss / (float)n + eps);
  }
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    float v = orow[i] * rs * (w ? w[i] : 1.0f);
    IO<T>::st(out + (long)row * n + i,
              v * sigmoidf_(IO<T>::ld(gr + i / gate_cols)));
  }
}

// Gate and grouped RMS norm of an fp32 row, in either order:
//   gate_first: z = o * act(gate);  out = z / rms_g(z) * w
//   else:       out = o / rms_g(o) * w * act(gate)
// act = silu or sigmoid; rms over `groups` equal consecutive parts; w has
// w_period entries and repeats (w_period = n: one weight per column;
// w_period = n / groups: the same weights for every group).
template <typename T>
__global__ void gated_group_norm_kernel(
    T* __restrict__ out, const float* __restrict__ o,
    const float* __restrict__ w, int w_period, const T* __restrict__ gate,
    long gate_stride, float eps, int n, int groups, int act_silu,
    int gate_first) {
  const int row = blockIdx.x;
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  const int nw = blockDim.x >> 6;
  const int gs = n / groups;
  const float* orow = o + (long)row * n;
  const T* gr = gate + (long)row * gate_stride;
  T* dst = out + (long)row * n;
  for (int g = wid; g < groups; g += nw) {
    float ss = 0.f;
    for (int i = lane; i < gs; i += 64) {
      const int c = g * gs + i;
      float z = orow[c];
      if (gate_first) {
        const float gv = IO<T>::ld(gr + c);
        z *= act_silu ? siluf_(gv) : sigmoidf_(gv);
      }
      ss += z * z;
    }
    ss = wave_reduce_sum(ss);
    const float rs = 1.0f / sqrtf(ss / (float)gs + eps);
    for (int i = lane; i < gs; i += 64) {
      const int c = g * gs + i;
      const float gv = IO<T>::ld(gr + c);
      const float a = act_silu ? siluf_(gv) : sigmoidf_(gv);
      IO<T>::st(dst + c, orow[c] * a * rs * w[c % w_period]);
    }
  }
}

// res[row] += y[row] / rms(y[row]) * w1, and the new residual row once more
// in the activation type (the operand of the next sublayer's GEMM): as it
// is, or with w_next normed for that sublayer, res / rms(res) * w_next. y may
// be fp32 (a sum formed in fp32) or the activation type.
template <typename TY, typename T>
__global__ void norm_residual_add_kernel(float* __restrict__ res,
                                         T* __restrict__ h,
                                         const TY* __restrict__ y,
                                         const float* __restrict__ w1,
                                         float eps, int width, long y_stride,
                                         const float* __restrict__ w_next) {
  __shared__ float tmp[16];
  const int row = blockIdx.x;
  const TY* yr = y + (long)row * y_stride;
  float* rr = res + (long)row * width;
  T* hr = h + (long)row * width;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float v = IO<TY>::ld(yr + i);
    ss += v * v;
  }
  ss = block_reduce_sum(ss, tmp);
  const float rs = 1.0f / sqrtf(ss / (float)width + eps);
  float s2 = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float v = rr[i] + IO<TY>::ld(yr + i) * rs * w1[i];
    rr[i] = v;
    s2 += v * v;
    if (w_next == nullptr) IO<T>::st(hr + i, v);
  }
  if (w_next == nullptr) return;
  __syncthreads();
  s2 = block_reduce_sum(s2, tmp);
  const float r2 = 1.0f / sqrtf(s2 / (float)width + eps);
  // a thread reads back the entries it wrote itself
  for (int i = threadIdx.x; i < width; i += blockDim.x)
    IO<T>::st(hr + i, rr[i] * r2 * w_next[i]);
}

XLLM_DEV float gelu_tanhf_(float z) {
  return 0.5f * z *
         (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

// out[r, i] = act(x[r, i]) * x[r, F + i]; GELU false: SiLU, true: tanh-GELU
template <typename T, bool GELU>
__global__ void act_mul_kernel(T* __restrict__ out, const T* __restrict__ x,
                               long rows, int F) {
  const long n = rows * (long)F;
  for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < n;
       idx += (long)gridDim.x * blockDim.x) {
    const long r = idx / F;
    const int i = (int)(idx - r * F);
    const float g = IO<T>::ld(x + r * 2 * F + i);
    const float u = IO<T>::ld(x + r * 2 * F + F + i);
    IO<T>::st(out + idx, (GELU ? gelu_tanhf_(g) : siluf_(g)) * u);
  }
}

// Rotate pairs (2i, 2i+1), i < rot_dims/2, of x[t, h, off : off+rot_dims] by
// pos[t] * inv_freq[i] (angle in fp64), cos/sin scaled by mscale. In place.
template <typename T>
__global__ void rope_interleaved_kernel(T* __restrict__ x,
                                        const long* __restrict__ pos,
                                        const double* __restrict__ inv_freq,
                                        float mscale, int tokens, int heads,
                                        int half, long row_stride,
                                        long head_stride, int off) {
  const long n = (long)tokens * heads * half;
  for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < n;
       idx += (long)gridDim.x * blockDim.x) {
    const int i = (int)(idx % half);
    const long th = idx / half;
    const int h = (int)(th % heads);
    const long t = th / heads;
    double s, c;
    sincos((double)pos[t] * inv_freq[i], &s, &c);
    const float cf = (float)c * mscale, sf = (float)s * mscale;
    T* p = x + t * row_stride + h * head_stride + off + 2 * i;
    const float u = IO<T>::ld(p), v = IO<T>::ld(p + 1);
    IO<T>::st(p, u * cf - v * sf);
    IO<T>::st(p + 1, v * cf + u * sf);
  }
}

// ---- launchers --------------------------------------------------------------
template <typename TI, typename TO>
void launch_group_rmsnorm(TO* out, const TI* x, const float* w, float eps,
                          int rows, int width, int groups, long x_stride,
                          hipStream_t st) {
  if (rows == 0) return;
  hipLaunchKernelGGL((group_rmsnorm_kernel<TI, TO>), dim3(rows), dim3(256), 0,
                     st, out, x, w, eps, width, groups, x_stride);
}
template <typename TY, typename TG>
void launch_gated_norm_residual(float* res, const TY* y, const TG* gate,
                                const float* bias, const float* w,
                                const float* ls, float mult, float eps,
                                int rows, int width, int groups,
                                long gate_stride, hipStream_t st) {
  if (rows == 0) return;
  hipLaunchKernelGGL((gated_norm_residual_kernel<TY, TG>), dim3(rows),
                     dim3(256), 0, st, res, y, gate, bias, w, ls, mult, eps,
                     width, groups, gate_stride);
}
template <typename T>
void launch_norm_sigmoid_gate(T* out, const float* o, const float* w,
                              const T* gate, float eps, int rows, int n,
                              long gate_stride, int gate_cols,
                              hipStream_t st) {
  if (rows == 0) return;
  hipLaunchKernelGGL((norm_sigmoid_gate_kernel<T>), dim3(rows), dim3(256), 0,
                     st, out, o, w, gate, eps, n, gate_stride, gate_cols);
}
template <typename TY, typename T>
void launch_norm_residual_add(float* res, T* h, const TY* y, const float* w1,
                              float eps, int rows, int width, long y_stride,
                              const float* w_next, hipStream_t st) {
  if (rows == 0) return;
  hipLaunchKernelGGL((norm_residual_add_kernel<TY, T>), dim3(rows), dim3(256),
                     0, st, res, h, y, w1, eps, width, y_stride, w_next);
}
template <typename T>
void launch_gated_group_norm(T* out, const float* o, const float* w,
                             int w_period, const T* gate, long gate_stride,
                             float eps, int rows, int n, int groups,
                             int act_silu, int gate_first, hipStream_t st) {
  if (rows == 0) return;
  hipLaunchKernelGGL((gated_group_norm_kernel<T>), dim3(rows), dim3(256), 0,
                     st, out, o, w, w_period, gate, gate_stride, eps, n,
                     groups, act_silu, gate_first);
}
template <typename T>
void launch_silu_mul(T* out, const T* x, long rows, int F, hipStream_t st) {
  const long n = rows * (long)F;
  if (n == 0) return;
  const int blocks = (int)((n + 255) / 256 < 65535 ? (n + 255) / 256 : 65535);
  hipLaunchKernelGGL((act_mul_kernel<T, false>), dim3(blocks), dim3(256), 0,
                     st, out, x, rows, F);
}
template <typename T>
void launch_gelu_tanh_mul(T* out, const T* x, long rows, int F,
                          hipStream_t st) {
  const long n = rows * (long)F;
  if (n == 0) return;
  const int blocks = (int)((n + 255) / 256 < 65535 ? (n + 255) / 256 : 65535);
  hipLaunchKernelGGL((act_mul_kernel<T, true>), dim3(blocks), dim3(256), 0,
                     st, out, x, rows, F);
}
template <typename T>
void launch_rope_interleaved(T* x, const long* pos, const double* inv_freq,
                             float mscale, int tokens, int heads, int half,
                             long row_stride, long head_stride, int off,
                             hipStream_t st) {
  const long n = (long)tokens * heads * half;
  if (n == 0) return;
  const int blocks = (int)((n + 255) / 256 < 65535 ? (n + 255) / 256 : 65535);
  hipLaunchKernelGGL((rope_interleaved_kernel<T>), dim3(blocks), dim3(256), 0,
                     st, x, pos, inv_freq, mscale, tokens, heads, half,
                     row_stride, head_stride, off);
}

#define INST_NORMS(T)                                                         \
  template void launch_norm_sigmoid_gate<T>(T*, const float*, const float*,   \
                                            const T*, float, int, int, long,  \
                                            int, hipStream_t);                \
  template void launch_silu_mul<T>(T*, const T*, long, int, hipStream_t);     \
  template void launch_gelu_tanh_mul<T>(T*, const T*, long, int,              \
                                        hipStream_t);                         \
  template void launch_gated_group_norm<T>(T*, const float*, const float*,    \
                                           int, const T*, long, float, int,   \
                                           int, int, int, int, hipStream_t);  \
  template void launch_rope_interleaved<T>(T*, const long*, const double*,    \
                                           float, int, int, int, long, long,  \
                                           int, hipStream_t);
INST_NORMS(float)
INST_NORMS(unsigned short)

#define INST_NRA(TY, T)                                                      \
  template void launch_norm_residual_add<TY, T>(                             \
      float*, T*, const TY*, const float*, float, int, int, long,            \
      const float*, hipStream_t);
INST_NRA(float, float)
INST_NRA(float, unsigned short)
INST_NRA(unsigned short, unsigned short)

#define INST_GRN(TI, TO)                                                     \
  template void launch_group_rmsnorm<TI, TO>(TO*, const TI*, const float*,   \
                                             float, int, int, int, long,     \
                                             hipStream_t);
INST_GRN(float, float)
INST_GRN(float, unsigned short)
INST_GRN(unsigned short, unsigned short)
INST_GRN(unsigned short, float)

#define INST_GNR(TY, TG)                                                      \
  template void launch_gated_norm_residual<TY, TG>(                           \
      float*, const TY*, const TG*, const float*, const float*, const float*, \
      float, float, int, int, int, long, hipStream_t);
INST_GNR(float, float)
INST_GNR(float, unsigned short)
INST_GNR(unsigned short, unsigned short)

}  // namespace hyb
}  // namespace xllm
