// Gated delta rule with a carried fp32 state:
//
//   S <- g_t S;  u_t = beta_t (v_t - S^T k_t);  S <- S + k_t u_t^T;
//   o_t = S^T q_t                                  (S is [D, Dv] per head)
//
// with k_t, q_t made unit vectors per head (x / sqrt(sum x^2 + 1e-6)), q_t
// also times D^-1/2, beta_t = sigmoid(b_t), g_t = exp(-exp(A_log_h)
// softplus(a_t + dt_bias_h)). q and k are shared by the heads of a group.
// Everything below is fp32; only the loads convert.
//
// With a = S_old^T k and c = S_old^T q the step is one pass of reductions
// and one pass of updates over the state a thread holds in registers:
//   u = beta (v - g a);  o = g c + (k . q) u;  S = g S_old + k u^T
// The unit scales are folded into the reduced sums (a, c) and into u, so the
// staged rows stay as loaded.
//
// The state lives in a slot pool [slots, H, D, Dv]; a sequence with
// ctx_len == 0 starts from zero whatever its slot held before; slot < 0 runs
// from zero and stores nothing.
//
// Prompt chunks: one workgroup per (sequence, head, 16*CPT columns of Dv);
// thread (j, r) owns rows r, r+16, ... of CPT neighbouring columns; the 16
// lanes of a column group sum their partial a and c by DPP. Decode: one
// workgroup per (sequence, head) holds the whole state in registers as
// float4 row pieces and sums the row groups' partials through LDS.
#include "hybrid_common.h"

namespace xllm {
namespace hyb {

constexpr int DR_CG = 16;      // column groups per workgroup
constexpr int DR_R = 16;       // row groups (threads per column group)
constexpr int DR_TC = 16;      // tokens staged per LDS fill
constexpr int DR_MAXM = 16;    // D <= DR_R * DR_MAXM = 256
constexpr int DR_NS = 5;       // per-token scalars: kscale qscale kq g beta

XLLM_DEV float dr_row16_sum(float v) {
  v += __int_as_float(__builtin_amdgcn_update_dpp(
      0, __float_as_int(v), 0xB1, 0xF, 0xF, true));    // quad_perm [1,0,3,2]
  v += __int_as_float(__builtin_amdgcn_update_dpp(
      0, __float_as_int(v), 0x4E, 0xF, 0xF, true));    // quad_perm [2,3,0,1]
  v += __int_as_float(__builtin_amdgcn_update_dpp(
      0, __float_as_int(v), 0x141, 0xF, 0xF, true));   // row_half_mirror
  v += __int_as_float(__builtin_amdgcn_update_dpp(
      0, __float_as_int(v), 0x140, 0xF, 0xF, true));   // row_mirror
  return v;
}

XLLM_DEV float dr_softplus(float x) {
  return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x)));
}

template <typename T>
struct DRArgs {
  const T* q; const T* k; const T* v; const T* b; const T* a;
  long q_stride, k_stride, v_stride, b_stride, a_stride;
  const float* dt_bias; const float* A_log;
  int heads, groups, D, Dv;
};

// decay and write strength of token `row`, head h
template <typename T>
XLLM_DEV void dr_gates(const DRArgs<T>& A, long row, int h, float* g,
                       float* beta) {
  const float dt = dr_softplus(IO<T>::ld(A.a + row * A.a_stride + h) +
                               A.dt_bias[h]);
  *g = expf(-expf(A.A_log[h]) * dt);
  *beta = 1.0f / (1.0f + expf(-IO<T>::ld(A.b + row * A.b_stride + h)));
}

template <typename T, int CPT>
__global__ void __launch_bounds__(256) delta_rule_kernel(
    float* __restrict__ out, DRArgs<T> A, float* __restrict__ state,
    const int* __restrict__ slots, const int* __restrict__ cu_q,
    const int* __restrict__ ctx_lens) {
  extern __shared__ float smem[];
  constexpr int VS = DR_CG * CPT;         // value columns per workgroup
  const int D = A.D, Dv = A.Dv, heads = A.heads;
  float* qs = smem;                       // [TC][D]
  float* ks = qs + DR_TC * D;             // [TC][D]
  float* vs = ks + DR_TC * D;             // [TC][VS]
  float* sc = vs + DR_TC * VS;            // [TC][NS]

  const int s = blockIdx.x, h = blockIdx.y, v0 = blockIdx.z * VS;
  const int kg = h / (heads / A.groups);
  const int tid = threadIdx.x;
  const int j = tid / DR_R, r = tid % DR_R;
  const int col = v0 + j * CPT;           // first of this thread's columns
  const int t0 = cu_q ? cu_q[s] : s;
  const int t1 = cu_q ? cu_q[s + 1] : s + 1;
  const int slot = slots[s];
  const int M = (D + DR_R - 1) / DR_R;
  const float qmul = 1.0f / sqrtf((float)D);

  float S[DR_MAXM][CPT];
#pragma unroll
  for (int m = 0; m < DR_MAXM; ++m)
#pragma unroll
    for (int c = 0; c < CPT; ++c) S[m][c] = 0.f;
  float* sp = (slot >= 0)
      ? state + (((long)slot * heads + h) * D) * (long)Dv : nullptr;
  const bool load = sp && ctx_lens[s] > 0;
  const bool vec = CPT == 4 && (Dv & 3) == 0 && col + 3 < Dv;
  if (load) {
#pragma unroll
    for (int m = 0; m < DR_MAXM; ++m) {
      const int i = r + DR_R * m;
      if (m < M && i < D) {
        if (vec) {
          const float4 x = *reinterpret_cast<const float4*>(
              sp + (long)i * Dv + col);
          S[m][0] = x.x; S[m][CPT > 1 ? 1 : 0] = x.y;
          S[m][CPT > 2 ? 2 : 0] = x.z; S[m][CPT > 3 ? 3 : 0] = x.w;
        } else {
#pragma unroll
          for (int c = 0; c < CPT; ++c)
            if (col + c < Dv) S[m][c] = sp[(long)i * Dv + col + c];
        }
      }
    }
  }

  for (int tb = t0; tb < t1; tb += DR_TC) {
    const int nt = min(DR_TC, t1 - tb);
    __syncthreads();                      // previous tile fully consumed
    for (int idx = tid; idx < nt * D; idx += 256) {
      const int tt = idx / D, i = idx - tt * D;
      const long row = tb + tt;
      qs[idx] = IO<T>::ld(A.q + row * A.q_stride + kg * D + i);
      ks[idx] = IO<T>::ld(A.k + row * A.k_stride + kg * D + i);
    }
    for (int idx = tid; idx < nt * VS; idx += 256) {
      const int tt = idx / VS, jj = idx - tt * VS;
      const long row = tb + tt;
      vs[idx] = (v0 + jj < Dv)
          ? IO<T>::ld(A.v + row * A.v_stride + h * Dv + v0 + jj) : 0.f;
    }
    if (tid < nt)
      dr_gates<T>(A, tb + tid, h, sc + tid * DR_NS + 3, sc + tid * DR_NS + 4);
    __syncthreads();
    {                                     // unit scales: 16 lanes per token
      const int tt = tid / DR_R;          // DR_TC * DR_R == 256 threads
      float sq = 0.f, sk = 0.f, skq = 0.f;
      if (tt < nt)
        for (int i = r; i < D; i += DR_R) {
          const float qv = qs[tt * D + i], kv = ks[tt * D + i];
          sq += qv * qv; sk += kv * kv; skq += qv * kv;
        }
      sq = dr_row16_sum(sq); sk = dr_row16_sum(sk); skq = dr_row16_sum(skq);
      if (tt < nt && r == 0) {
        const float kscale = 1.0f / sqrtf(sk + 1e-6f);
        const float qscale = qmul / sqrtf(sq + 1e-6f);
        sc[tt * DR_NS] = kscale;
        sc[tt * DR_NS + 1] = qscale;
        sc[tt * DR_NS + 2] = skq * kscale * qscale;
      }
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const float kscale = sc[tt * DR_NS], qscale = sc[tt * DR_NS + 1];
      const float kq = sc[tt * DR_NS + 2], g = sc[tt * DR_NS + 3];
      const float beta = sc[tt * DR_NS + 4];
      float ak[CPT], aq[CPT];
#pragma unroll
      for (int c = 0; c < CPT; ++c) { ak[c] = 0.f; aq[c] = 0.f; }
#pragma unroll
      for (int m = 0; m < DR_MAXM; ++m) {
        const int i = r + DR_R * m;
        if (m < M && i < D) {
          const float kk = ks[tt * D + i], qq = qs[tt * D + i];
#pragma unroll
          for (int c = 0; c < CPT; ++c) {
            ak[c] += S[m][c] * kk;
            aq[c] += S[m][c] * qq;
          }
        }
      }
      float uk[CPT];
#pragma unroll
      for (int c = 0; c < CPT; ++c) {
        const float a = dr_row16_sum(ak[c]) * kscale;
        const float cq = dr_row16_sum(aq[c]) * qscale;
        const float u = beta * (vs[tt * VS + j * CPT + c] - g * a);
        uk[c] = u * kscale;
        ak[c] = g * cq + kq * u;          // the token's output column
      }
#pragma unroll
      for (int m = 0; m < DR_MAXM; ++m) {
        const int i = r + DR_R * m;
        if (m < M && i < D) {
          const float kk = ks[tt * D + i];
#pragma unroll
          for (int c = 0; c < CPT; ++c) S[m][c] = g * S[m][c] + kk * uk[c];
        }
      }
      if (r == 0) {
        float* op = out + ((long)(tb + tt) * heads + h) * Dv + col;
#pragma unroll
        for (int c = 0; c < CPT; ++c)
          if (col + c < Dv) op[c] = ak[c];
      }
    }
  }
  if (sp) {
#pragma unroll
    for (int m = 0; m < DR_MAXM; ++m) {
      const int i = r + DR_R * m;
      if (m < M && i < D) {
        if (vec) {
          *reinterpret_cast<float4*>(sp + (long)i * Dv + col) = make_float4(
              S[m][0], S[m][CPT > 1 ? 1 : 0], S[m][CPT > 2 ? 2 : 0],
              S[m][CPT > 3 ? 3 : 0]);
        } else {
#pragma unroll
          for (int c = 0; c < CPT; ++c)
            if (col + c < Dv) sp[(long)i * Dv + col + c] = S[m][c];
        }
      }
    }
  }
}

// Decode (one token per sequence): thread (rg, tc) owns columns 4tc..4tc+3 of
// rows rg, rg+RG, ... (NR of them, float4 each, kept in registers between the
// reduction pass and the update pass); the RG row groups' partial sums meet
// in LDS.
template <typename T, int NR>
__global__ void __launch_bounds__(256) delta_rule_decode_kernel(
    float* __restrict__ out, DRArgs<T> A, float* __restrict__ state,
    const int* __restrict__ slots, const int* __restrict__ ctx_lens) {
  extern __shared__ float smem[];
  __shared__ float red[6 * 4];
  const int D = A.D, Dv = A.Dv, heads = A.heads;
  const int Dp = (D + 3) & ~3;
  float* qs = smem;                 // [Dp]
  float* ks = qs + Dp;              // [Dp]
  float* vs = ks + Dp;              // [Dv]
  float* pa = vs + Dv;              // [RG][Dv] partial S^T k
  const int s = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int kg = h / (heads / A.groups);
  const int TCn = Dv >> 2, RG = 256 / TCn;
  float* pq = pa + RG * Dv;         // [RG][Dv] partial S^T q
  const int rg = tid / TCn, tc = tid - rg * TCn;
  float sq = 0.f, sk = 0.f, skq = 0.f;
  for (int i = tid; i < D; i += 256) {
    const float qv = IO<T>::ld(A.q + s * A.q_stride + kg * D + i);
    const float kv = IO<T>::ld(A.k + s * A.k_stride + kg * D + i);
    qs[i] = qv; ks[i] = kv;
    sq += qv * qv; sk += kv * kv; skq += qv * kv;
  }
  for (int i = tid; i < Dv; i += 256)
    vs[i] = IO<T>::ld(A.v + s * A.v_stride + h * Dv + i);
  sq = wave_reduce_sum(sq); sk = wave_reduce_sum(sk);
  skq = wave_reduce_sum(skq);
  if ((tid & 63) == 0) {
    red[(tid >> 6) * 3] = sq; red[(tid >> 6) * 3 + 1] = sk;
    red[(tid >> 6) * 3 + 2] = skq;
  }
  __syncthreads();
  sq = red[0] + red[3] + red[6] + red[9];
  sk = red[1] + red[4] + red[7] + red[10];
  skq = red[2] + red[5] + red[8] + red[11];
  const float kscale = 1.0f / sqrtf(sk + 1e-6f);
  const float qscale = 1.0f / sqrtf((float)D) / sqrtf(sq + 1e-6f);
  const float kq = skq * kscale * qscale;
  float g, beta;
  dr_gates<T>(A, s, h, &g, &beta);
  const int slot = slots[s];
  const bool load = slot >= 0 && ctx_lens[s] > 0;
  float* sp = state + (((long)max(slot, 0) * heads + h) * D) * (long)Dv + 4 * tc;
  float4 S[NR];
  float4 ak = make_float4(0.f, 0.f, 0.f, 0.f), aq = ak;
  if (rg < RG) {
#pragma unroll
    for (int n = 0; n < NR; ++n) {
      const int i = rg + n * RG;
      S[n] = make_float4(0.f, 0.f, 0.f, 0.f);
      if (i < D) {
        if (load) S[n] = *reinterpret_cast<const float4*>(sp + (long)i * Dv);
        const float ki = ks[i], qi = qs[i];
        ak.x += S[n].x * ki; ak.y += S[n].y * ki;
        ak.z += S[n].z * ki; ak.w += S[n].w * ki;
        aq.x += S[n].x * qi; aq.y += S[n].y * qi;
        aq.z += S[n].z * qi; aq.w += S[n].w * qi;
      }
    }
    *reinterpret_cast<float4*>(pa + rg * Dv + 4 * tc) = ak;
    *reinterpret_cast<float4*>(pq + rg * Dv + 4 * tc) = aq;
  }
  __syncthreads();
  if (rg < RG) {
    float uk[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      float a = 0.f, cq = 0.f;
      for (int g2 = 0; g2 < RG; ++g2) {
        a += pa[g2 * Dv + 4 * tc + c];
        cq += pq[g2 * Dv + 4 * tc + c];
      }
      const float u = beta * (vs[4 * tc + c] - g * a * kscale);
      uk[c] = u * kscale;
      if (rg == 0)
        out[((long)s * heads + h) * Dv + 4 * tc + c] = g * cq * qscale + kq * u;
    }
    if (slot >= 0) {
#pragma unroll
      for (int n = 0; n < NR; ++n) {
        const int i = rg + n * RG;
        if (i < D) {
          const float ki = ks[i];
          S[n].x = g * S[n].x + ki * uk[0]; S[n].y = g * S[n].y + ki * uk[1];
          S[n].z = g * S[n].z + ki * uk[2]; S[n].w = g * S[n].w + ki * uk[3];
          *reinterpret_cast<float4*>(sp + (long)i * Dv) = S[n];
        }
      }
    }
  }
}

template <typename T, int CPT>
void launch_delta_rule_cpt(float* out, const DRArgs<T>& A, float* state,
                           const int* slots, const int* cu_q,
                           const int* ctx_lens, int n_seqs, hipStream_t st) {
  constexpr int VS = DR_CG * CPT;
  const size_t lds = (size_t)(2 * DR_TC * A.D + DR_TC * VS + DR_TC * DR_NS) *
                     sizeof(float);
  const int vz = (A.Dv + VS - 1) / VS;
  hipLaunchKernelGGL((delta_rule_kernel<T, CPT>), dim3(n_seqs, A.heads, vz),
                     dim3(256), lds, st, out, A, state, slots, cu_q, ctx_lens);
}

template <typename T>
void launch_delta_rule(float* out, const T* q, const T* k, const T* v,
                       const T* b, const T* a, long q_stride, long k_stride,
                       long v_stride, long b_stride, long a_stride,
                       const float* dt_bias, const float* A_log, float* state,
                       const int* slots, const int* cu_q, const int* ctx_lens,
                       int n_seqs, int heads, int groups, int D, int Dv,
                       hipStream_t st) {
  if (n_seqs == 0) return;
  DRArgs<T> A{q, k, v, b, a, q_stride, k_stride, v_stride, b_stride, a_stride,
              dt_bias, A_log, heads, groups, D, Dv};
  if (cu_q == nullptr && Dv % 4 == 0 && Dv <= 1024) {
    const int RG = 256 / (Dv / 4);
    const int nr = RG >= 1 ? (D + RG - 1) / RG : 0;
    const size_t l2 =
        (size_t)(2 * ((D + 3) & ~3) + Dv + 2 * RG * Dv) * sizeof(float);
    if (RG >= 1 && nr <= 32 && l2 <= 64 * 1024) {
#define DR_DEC(NR)                                                            \
  hipLaunchKernelGGL((delta_rule_decode_kernel<T, NR>), dim3(n_seqs, heads),  \
                     dim3(256), l2, st, out, A, state, slots, ctx_lens)
      if (nr <= 4) DR_DEC(4);
      else if (nr <= 8) DR_DEC(8);
      else if (nr <= 16) DR_DEC(16);
      else DR_DEC(32);
#undef DR_DEC
      return;
    }
  }
  // wide values and enough workgroups: four columns per thread
  const bool wide = Dv >= 48 && (long)n_seqs * heads * ((Dv + 63) / 64) >= 256;
  if (wide)
    launch_delta_rule_cpt<T, 4>(out, A, state, slots, cu_q, ctx_lens, n_seqs,
                                st);
  else
    launch_delta_rule_cpt<T, 1>(out, A, state, slots, cu_q, ctx_lens, n_seqs,
                                st);
}

#define INST_DR(T)                                                            \
  template void launch_delta_rule<T>(                                         \
      float*, const T*, const T*, const T*, const T*, const T*, long, long,   \
      long, long, long, const float*, const float*, float*, const int*,       \
      const int*, const int*, int, int, int, int, int, hipStream_t);
INST_DR(float)
INST_DR(unsigned short)

}  // namespace hyb
}  // namespace xllm
