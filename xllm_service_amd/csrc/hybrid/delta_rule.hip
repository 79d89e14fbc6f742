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
//
// Long chunks run piece-parallel. A token maps the state linearly,
//   S <- g (I - beta k k^T) S + beta k v^T,
// so a piece of tokens maps S to M S + N with M [D, D] the product of its
// token matrices and N [D, Dv] what the piece builds from a zero state. M is
// what the same recurrence makes of an identity state with zero values:
// pass 1 runs every piece over Dv + D columns ([zero | identity] in,
// [N | M] out), a scan applies S <- M S + N piece after piece on the fp32
// matrix pipe (v_mfma_f32_16x16x4_f32, true 32-bit products) and leaves the
// state BEFORE each piece in N's place, pass 2 reruns the pieces from these
// states and writes the outputs.
#include <cstdlib>

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

// mode 0: the whole chunk of a sequence in one workgroup (slot in and out)
// mode 1: tokens [c*chunk, (c+1)*chunk) over Dv + D columns from [0 | I], no
//         outputs; [N | M] goes to the piece's record in ws
//         ([s*max_chunks + c][h][D][Dv + D])
// mode 2: the same tokens from the state the scan left in the record's first
//         Dv columns; outputs written, nothing stored
// NOOUT: a launch of mode 1 only; the read-out sums are not formed at all.
template <typename T, int CPT, bool NOOUT>
__global__ void __launch_bounds__(256) delta_rule_kernel(
    float* __restrict__ out, DRArgs<T> A, float* __restrict__ state,
    const int* __restrict__ slots, const int* __restrict__ cu_q,
    const int* __restrict__ ctx_lens, int mode, int chunk, int max_chunks,
    float* __restrict__ ws) {
  extern __shared__ float smem[];
  constexpr int VS = DR_CG * CPT;         // value columns per workgroup
  const int D = A.D, Dv = A.Dv, heads = A.heads;
  float* qs = smem;                       // [TC][D]
  float* ks = qs + DR_TC * D;             // [TC][D]
  float* vs = ks + DR_TC * D;             // [TC][VS]
  float* sc = vs + DR_TC * VS;            // [TC][NS]

  const int s = blockIdx.x / max_chunks, cidx = blockIdx.x % max_chunks;
  const int h = blockIdx.y, v0 = blockIdx.z * VS;
  const int kg = h / (heads / A.groups);
  const int tid = threadIdx.x;
  const int j = tid / DR_R, r = tid % DR_R;
  const int col = v0 + j * CPT;           // first of this thread's columns
  int t0 = cu_q ? cu_q[s] : s;
  int t1 = cu_q ? cu_q[s + 1] : s + 1;
  if (mode != 0) {
    t0 += cidx * chunk;
    if (t0 >= t1) return;                 // uniform for the workgroup
    t1 = min(t1, t0 + chunk);
  }
  const int E = Dv + D;                   // columns of a piece record
  const int ncols = mode == 1 ? E : Dv;   // columns this launch covers
  const int rs = mode == 0 ? Dv : E;      // row stride of what sp points at
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
  bool load = sp && ctx_lens[s] > 0;
  if (mode != 0) {
    sp = ws + ((((long)s * max_chunks + cidx) * heads + h) * D) * (long)E;
    load = mode == 2;
  }
  const bool vec = CPT == 4 && (Dv & 3) == 0 && (rs & 3) == 0 &&
                   col + 3 < ncols;
  if (load) {
#pragma unroll
    for (int m = 0; m < DR_MAXM; ++m) {
      const int i = r + DR_R * m;
      if (m < M && i < D) {
        if (vec) {
          const float4 x = *reinterpret_cast<const float4*>(
              sp + (long)i * rs + col);
          S[m][0] = x.x; S[m][CPT > 1 ? 1 : 0] = x.y;
          S[m][CPT > 2 ? 2 : 0] = x.z; S[m][CPT > 3 ? 3 : 0] = x.w;
        } else {
#pragma unroll
          for (int c = 0; c < CPT; ++c)
            if (col + c < ncols) S[m][c] = sp[(long)i * rs + col + c];
        }
      }
    }
  }
  if (mode == 1) {                        // identity under the M columns
#pragma unroll
    for (int m = 0; m < DR_MAXM; ++m)
#pragma unroll
      for (int c = 0; c < CPT; ++c)
        if (col + c - Dv == r + DR_R * m) S[m][c] = 1.f;
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
            if (!NOOUT) aq[c] += S[m][c] * qq;
          }
        }
      }
      float uk[CPT];
#pragma unroll
      for (int c = 0; c < CPT; ++c) {
        const float a = dr_row16_sum(ak[c]) * kscale;
        const float cq = NOOUT ? 0.f : dr_row16_sum(aq[c]) * qscale;
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
      if (!NOOUT && mode != 1 && r == 0) {
        float* op = out + ((long)(tb + tt) * heads + h) * Dv + col;
#pragma unroll
        for (int c = 0; c < CPT; ++c)
          if (col + c < Dv) op[c] = ak[c];
      }
    }
  }
  if (sp && mode != 2) {
#pragma unroll
    for (int m = 0; m < DR_MAXM; ++m) {
      const int i = r + DR_R * m;
      if (m < M && i < D) {
        if (vec) {
          *reinterpret_cast<float4*>(sp + (long)i * rs + col) = make_float4(
              S[m][0], S[m][CPT > 1 ? 1 : 0], S[m][CPT > 2 ? 2 : 0],
              S[m][CPT > 3 ? 3 : 0]);
        } else {
#pragma unroll
          for (int c = 0; c < CPT; ++c)
            if (col + c < ncols) sp[(long)i * rs + col + c] = S[m][c];
        }
      }
    }
  }
}

typedef __attribute__((__vector_size__(4 * sizeof(float)))) float dr_f32x4;

// S <- M_c S + N_c over the pieces of a sequence, for 16 columns of one head.
// S sits in LDS as [rows][16]; wave w owns the 16-row tile w of the result
// (the workgroup has one wave per tile). v_mfma_f32_16x16x4_f32: lane l gives
// A[l & 15][l >> 4] and B[l >> 4][l & 15] and holds C[(l >> 4) * 4 + r]
// [l & 15]. Within a block of 16 inner indices lane group g takes the indices
// 4g..4g+3 (one 16 B load of its M row), the same permutation on both
// operands. A wave's M rows and N tile of the NEXT piece are loaded into
// registers while the current piece multiplies (KB <= 8). The record's first
// Dv columns (N) are overwritten with the state before the piece.
template <int KB>                         // D <= 16 * KB
__global__ void __launch_bounds__(64 * KB) delta_rule_scan_kernel(
    float* __restrict__ ws, float* __restrict__ state,
    const int* __restrict__ slots, const int* __restrict__ cu_q,
    const int* __restrict__ ctx_lens, int heads, int D, int Dv, int chunk,
    int max_chunks) {
  extern __shared__ float Sl[];           // [Dp][16]
  constexpr bool PF = KB <= 8;
  const int s = blockIdx.x, h = blockIdx.y, col0 = blockIdx.z * 16;
  const int tid = threadIdx.x, lane = tid & 63, it = tid >> 6;
  const int nthr = blockDim.x;
  const int n = lane & 15, g = lane >> 4;
  const int E = Dv + D;
  const int qlen = cu_q[s + 1] - cu_q[s];
  const int n_chunks = min((qlen + chunk - 1) / chunk, max_chunks);
  const int slot = slots[s];
  const int n_tiles = (D + 15) >> 4, Dp = n_tiles << 4;
  const bool col_ok = col0 + n < Dv;
  const bool from_slot = slot >= 0 && ctx_lens[s] > 0;
  float* sst = state + (((long)max(slot, 0) * heads + h) * D) * (long)Dv;
  for (int idx = tid; idx < Dp * 16; idx += nthr) {
    const int i = idx >> 4, jj = idx & 15;
    Sl[idx] = (from_slot && i < D && col0 + jj < Dv)
        ? sst[(long)i * Dv + col0 + jj] : 0.f;
  }
  __syncthreads();
  const bool fast = (D & 15) == 0 && (E & 3) == 0 && (Dv & 3) == 0;
  const int ia = it * 16 + n;             // this lane's M row
  auto rec_of = [&](int c) {
    return ws + ((((long)s * max_chunks + c) * heads + h) * D) * (long)E;
  };
  auto load = [&](const float* rec, float4 (&m4)[KB], float (&n4)[4]) {
    const float* mrow = rec + (long)min(ia, D - 1) * E + Dv;
#pragma unroll
    for (int kbi = 0; kbi < KB; ++kbi) {
      const int k0 = kbi * 16 + 4 * g;
      m4[kbi] = make_float4(0.f, 0.f, 0.f, 0.f);
      if (kbi * 16 < D && it < n_tiles) {
        if (fast) {
          m4[kbi] = *reinterpret_cast<const float4*>(mrow + k0);
        } else if (ia < D) {
          if (k0 < D) m4[kbi].x = mrow[k0];
          if (k0 + 1 < D) m4[kbi].y = mrow[k0 + 1];
          if (k0 + 2 < D) m4[kbi].z = mrow[k0 + 2];
          if (k0 + 3 < D) m4[kbi].w = mrow[k0 + 3];
        }
      }
    }
#pragma unroll
    for (int rr = 0; rr < 4; ++rr) {
      const int i = it * 16 + 4 * g + rr;
      n4[rr] = (i < D && col_ok) ? rec[(long)i * E + col0 + n] : 0.f;
    }
  };
  float4 mc[KB], mn[KB];               // mn unused without prefetch
  float nc[4], nn[4];
  if constexpr (PF) {
    if (n_chunks > 0) load(rec_of(0), mc, nc);
  }
  for (int c = 0; c < n_chunks; ++c) {
    float* rec = rec_of(c);
    if constexpr (PF) {
      if (c + 1 < n_chunks) load(rec_of(c + 1), mn, nn);
    } else {
      load(rec, mc, nc);
    }
    dr_f32x4 acc = {nc[0], nc[1], nc[2], nc[3]};
    if (it < n_tiles) {                   // uniform per wave
#pragma unroll
      for (int kbi = 0; kbi < KB; ++kbi) {
        if (kbi * 16 < D) {
          const int kk = kbi * 16 + 4 * g;            // kk + 3 < Dp
          acc = __builtin_amdgcn_mfma_f32_16x16x4f32(
              mc[kbi].x, Sl[kk * 16 + n], acc, 0, 0, 0);
          acc = __builtin_amdgcn_mfma_f32_16x16x4f32(
              mc[kbi].y, Sl[(kk + 1) * 16 + n], acc, 0, 0, 0);
          acc = __builtin_amdgcn_mfma_f32_16x16x4f32(
              mc[kbi].z, Sl[(kk + 2) * 16 + n], acc, 0, 0, 0);
          acc = __builtin_amdgcn_mfma_f32_16x16x4f32(
              mc[kbi].w, Sl[(kk + 3) * 16 + n], acc, 0, 0, 0);
        }
      }
      // the state before this piece takes N's place (this thread has read
      // exactly these elements already)
#pragma unroll
      for (int rr = 0; rr < 4; ++rr) {
        const int i = it * 16 + 4 * g + rr;
        if (i < D && col_ok) rec[(long)i * E + col0 + n] = Sl[i * 16 + n];
      }
    }
    __syncthreads();                      // every wave is done reading Sl
    if (it < n_tiles) {
#pragma unroll
      for (int rr = 0; rr < 4; ++rr) {
        const int i = it * 16 + 4 * g + rr;
        Sl[i * 16 + n] = (i < D && col_ok) ? acc[rr] : 0.f;
      }
    }
    __syncthreads();
    if constexpr (PF) {
#pragma unroll
      for (int kbi = 0; kbi < KB; ++kbi) mc[kbi] = mn[kbi];
#pragma unroll
      for (int rr = 0; rr < 4; ++rr) nc[rr] = nn[rr];
    }
  }
  if (slot >= 0)
    for (int idx = tid; idx < Dp * 16; idx += nthr) {
      const int i = idx >> 4, jj = idx & 15;
      if (i < D && col0 + jj < Dv) sst[(long)i * Dv + col0 + jj] = Sl[idx];
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
                           const int* ctx_lens, int n_seqs, int chunk,
                           int max_chunks, float* ws, hipStream_t st) {
  constexpr int VS = DR_CG * CPT;
  const int D = A.D, Dv = A.Dv;
  const size_t lds = (size_t)(2 * DR_TC * D + DR_TC * VS + DR_TC * DR_NS) *
                     sizeof(float);
  const int vz = (Dv + VS - 1) / VS;
  if (ws == nullptr || max_chunks <= 1) {
    hipLaunchKernelGGL((delta_rule_kernel<T, CPT, false>),
                       dim3(n_seqs, A.heads, vz), dim3(256), lds, st, out, A,
                       state, slots, cu_q, ctx_lens, 0, 0, 1, nullptr);
    return;
  }
  const int vz1 = (Dv + D + VS - 1) / VS;
  hipLaunchKernelGGL((delta_rule_kernel<T, CPT, true>),
                     dim3(n_seqs * max_chunks, A.heads, vz1), dim3(256), lds,
                     st, out, A, state, slots, cu_q, ctx_lens, 1, chunk,
                     max_chunks, ws);
  const int n_tiles = (D + 15) >> 4, Dp = n_tiles << 4;
  const dim3 sgrid(n_seqs, A.heads, (Dv + 15) / 16);
#define DR_SCAN(KB)                                                           \
  hipLaunchKernelGGL(delta_rule_scan_kernel<KB>, sgrid, dim3(64 * KB),        \
                     (size_t)Dp * 16 * sizeof(float), st, ws, state, slots,   \
                     cu_q, ctx_lens, A.heads, D, Dv, chunk, max_chunks)
  if (n_tiles <= 4) DR_SCAN(4);
  else if (n_tiles <= 8) DR_SCAN(8);
  else DR_SCAN(16);
#undef DR_SCAN
  hipLaunchKernelGGL((delta_rule_kernel<T, CPT, false>),
                     dim3(n_seqs * max_chunks, A.heads, vz), dim3(256), lds,
                     st, out, A, state, slots, cu_q, ctx_lens, 2, chunk,
                     max_chunks, ws);
}

template <typename T>
void launch_delta_rule(float* out, const T* q, const T* k, const T* v,
                       const T* b, const T* a, long q_stride, long k_stride,
                       long v_stride, long b_stride, long a_stride,
                       const float* dt_bias, const float* A_log, float* state,
                       const int* slots, const int* cu_q, const int* ctx_lens,
                       int n_seqs, int heads, int groups, int D, int Dv,
                       int chunk, int max_chunks, float* ws, hipStream_t st) {
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
  // wide values and enough workgroups: four columns per thread.
  // XLLM_DELTA_COLS=1|4 fixes the choice (tuning knob).
  bool wide = Dv >= 48 &&
      (long)n_seqs * max_chunks * heads * ((Dv + 63) / 64) >= 256;
  if (const char* e = std::getenv("XLLM_DELTA_COLS")) wide = e[0] == '4';
  if (wide)
    launch_delta_rule_cpt<T, 4>(out, A, state, slots, cu_q, ctx_lens, n_seqs,
                                chunk, max_chunks, ws, st);
  else
    launch_delta_rule_cpt<T, 1>(out, A, state, slots, cu_q, ctx_lens, n_seqs,
                                chunk, max_chunks, ws, st);
}

#define INST_DR(T)                                                            \
  template void launch_delta_rule<T>(                                         \
      float*, const T*, const T*, const T*, const T*, const T*, long, long,   \
      long, long, long, const float*, const float*, float*, const int*,       \
      const int*, const int*, int, int, int, int, int, int, int, float*,      \
      hipStream_t);
INST_DR(float)
INST_DR(unsigned short)

}  // namespace hyb
}  // namespace xllm
