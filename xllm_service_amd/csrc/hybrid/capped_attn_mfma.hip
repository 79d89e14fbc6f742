// MFMA soft-capped attention over a paged key/value cache (bf16) for gfx950.
//
// Grouped heads: the `per` query heads that share one key/value head attend
// to the SAME cached rows, so within a sequence chunk and a key/value head
// the (query, head) pairs are rows of one query matrix: row
// rho = query * per + head_in_group. A workgroup (4 waves) owns 64 such rows
// of one key/value head, a wave 16.
//
// Per 32-key tile:
//   S^T[key][row] = K[key][:] . Q[row][:]      A = K rows, 16 B per lane from the
//                                              key tile staged in LDS; B = Q, held
//                                              in registers for the whole kernel
//   s <- scale * s, then cap * tanh(s / cap) when a cap is given
//   online softmax per row in fp32 (a lane holds 8 keys of ONE row)
//   O^T[col][row] += V^T[col][key] P^T[key][row]
//                                              A = V^T by hardware transpose
//                                              reads (ds_read_b64_tr_b16) of the
//                                              value tile staged in LDS with
//                                              plain 16 B writes; B = the lane's
//                                              own 8 weights: no exchange needed
// The C layout of S^T hands a lane rows g*4+r of both 16-row halves; feeding
// key k0 + (m>>2)*8 + half*4 + (m&3) as A row m makes those the keys
// g*8 .. g*8+7 in natural order, which is what the transposed V fragment
// holds. Softmax weights stay 32-bit: p is split exactly into three bf16
// terms (8+8+8 mantissa bits) and each term gets its own MFMA into the fp32
// accumulator.
//
// LDS image of a 32-key tile (keys and values each have one), per 16-column
// tile `nt` (512 bf16): element (k, d) at nt*512 + ((k>>2)&1)*256 +
// (k>>3)*64 + (k&3)*16 + (d&15); a lane reads 8 B at g*128 + n*8 (bytes) of
// each 512-byte half.
//
// Keys read as values (v_cache is the very tensor k_cache): the key image of
// a tile is also its value image (both have one layout), so the tile is
// fetched and staged once.
//
// Decode splits the context over `n_part` workgroups per (token, key/value
// head); partial (acc, max, sum) triples are merged by a second small kernel.
//
// Sliding window: a row sees the keys [limit - window, limit) and, with
// keep_first, the keys [0, keep_first) as well; the tile loop runs over the
// leading tiles that hold kept keys and then from the first tile any row of
// the workgroup needs (one list of tiles, split evenly over the context
// partitions). Sink: exp(sink_h) joins the denominator once, at the end (or
// in the merge kernel). head_scale: one more score multiplier per head.
//
// Fragment layouts of __builtin_amdgcn_mfma_f32_16x16x32_bf16 (lane l):
//   A[l&15][(l>>4)*8 + j], B[(l>>4)*8 + j][l&15], C[(l>>4)*4 + r][l&15].
#include "hybrid_common.h"

namespace xllm {
namespace hyb {

typedef __attribute__((__vector_size__(8 * sizeof(short)))) short bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

constexpr int CM_KT = 32;       // keys per tile

struct alignas(16) cm_u16x8 { unsigned short x[8]; };

XLLM_DEV bf16x8 cm_ld8(const unsigned short* p) {
  return *reinterpret_cast<const bf16x8*>(p);
}

XLLM_DEV float cm_tanh(float x) {          // 1 - 2 / (e^(2x) + 1)
  const float e = __expf(2.0f * fminf(x, 15.0f));
  return 1.0f - 2.0f / (e + 1.0f);
}

// KQ = 32-column chunks of a key row (D padded), NO = 16-column tiles of a
// value row (Dv padded to 64). CS = column split: the 4 waves of a workgroup
// form 4/CS row tiles, and CS waves share one row tile, each owning every
// CS-th 64-column batch of the output (decode: few rows per token).
// The decode instantiation for 128-wide heads sits at the edge of four waves
// per SIMD (128 registers); the second launch bound asks the compiler to stay
// inside it (0 = no request).
template <int KQ, int NO, int CS>
__global__ void
__launch_bounds__(256, (KQ == 4 && NO == 8 && CS == 4) ? 4 : 0)
capped_attn_mfma_kernel(
    float* __restrict__ out, float* __restrict__ ws_acc,
    float* __restrict__ ws_ml, const unsigned short* __restrict__ q,
    const unsigned short* __restrict__ k_cache,
    const unsigned short* __restrict__ v_cache,
    const int* __restrict__ block_tables, const int* __restrict__ cu_q,
    const int* __restrict__ seq_lens, int n_seqs, int heads, int n_kv, int D,
    int Dv, int block_size, int table_width, float scale, float cap,
    long q_stride, int n_part, int window, const float* __restrict__ sink,
    int keep_first, const float* __restrict__ head_scale) {
  extern __shared__ unsigned short cm_lds[];      // [key image | value image]
  __shared__ int tbl[512];                        // block ids of this key range
  constexpr int RT = 4 / CS;                      // row tiles per workgroup
  constexpr int ROWS_WG = 16 * RT;
  constexpr int NB = NO / 4;                      // 64-column batches
  constexpr int NBL = (NB + CS - 1) / CS;         // ... owned by one wave
  constexpr int NPK = (KQ + 1) / 2;               // 16 B key chunks per thread
  constexpr int NPV = NB;                         // 16 B value chunks per thread
  constexpr bool PF = CS > 1;
  constexpr int Dp = KQ * 32, Dvp = NO * 16;
  // keys read as values: one image (the instantiations with D == Dv have
  // Dp == Dvp)
  const bool same = (k_cache == v_cache) && Dp == Dvp;
  unsigned short* kt = cm_lds;                    // key image: Dp/16 tiles
  unsigned short* vt = same ? kt : cm_lds + (Dp / 16) * 512;  // NO tiles
  const int per = heads / n_kv;
  const int kvh = blockIdx.z;
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int g = lane >> 4, n = lane & 15;

  // ---- which sequence / row tile is this workgroup ----------------------
  int s, lt, qlen, q0;
  const int bid = blockIdx.x;
  if (cu_q == nullptr) {
    const int tps = (per + ROWS_WG - 1) / ROWS_WG;
    s = bid / tps; lt = bid - s * tps; qlen = 1; q0 = s;
    if (s >= n_seqs) return;
  } else {
    int acc = 0; s = -1; lt = 0;
    for (int i = 0; i < n_seqs; ++i) {
      const int nt = ((cu_q[i + 1] - cu_q[i]) * per + ROWS_WG - 1) / ROWS_WG;
      if (bid < acc + nt) { s = i; lt = bid - acc; break; }
      acc += nt;
    }
    if (s < 0) return;
    q0 = cu_q[s]; qlen = cu_q[s + 1] - q0;
  }
  const int rows_in_seq = qlen * per;
  const int ctx = seq_lens[s] - qlen;
  const int row0 = lt * ROWS_WG;
  const int last_row = min(row0 + ROWS_WG, rows_in_seq) - 1;
  const int kmax = ctx + last_row / per + 1;         // keys any row here sees
  const int n_tiles = (kmax + CM_KT - 1) / CM_KT;
  // first key the earliest row of this workgroup sees
  const int kmin = window > 0 ? max(0, ctx + row0 / per + 1 - window) : 0;
  const int t_first = kmin / CM_KT;
  // tile list: [0, t_keep) then [t_first, n_tiles)
  const int t_keep = (window > 0 && keep_first > 0)
      ? min((min(keep_first, kmax) + CM_KT - 1) / CM_KT, t_first) : 0;
  const int n_list = t_keep + n_tiles - t_first;
  const int tpp = (n_list + n_part - 1) / n_part;
  const int i_begin = blockIdx.y * tpp;
  const int i_end = min(n_list, i_begin + tpp);
  auto tile_at = [&](int i) { return i < t_keep ? i : t_first + (i - t_keep); };
  const int t_begin = tile_at(i_begin);
  const int t_end = i_end > i_begin ? tile_at(i_end - 1) + 1 : t_begin;
  const int* table = block_tables + (long)s * table_width;

  // ---- this lane's row -----------------------------------------------------
  const int rt = wv % RT, cpart = wv / RT;
  const int rho = row0 + rt * 16 + n;
  const bool wave_on = row0 + rt * 16 < rows_in_seq;
  const bool row_ok = rho < rows_in_seq;
  const int limit = row_ok ? ctx + rho / per + 1 : 0;
  const int lo = window > 0 ? max(0, limit - window) : 0;
  const int head = kvh * per + (row_ok ? rho % per : 0);
  const long tok = q0 + (row_ok ? rho / per : 0);
  const long grow = tok * heads + head;              // row in [T*H]

  bf16x8 qf[KQ];
#pragma unroll
  for (int kc = 0; kc < KQ; ++kc) {
    const int col = kc * 32 + g * 8;
    bf16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
    qf[kc] = (row_ok && col < D)
        ? cm_ld8(q + tok * q_stride + (long)head * D + col) : z;
  }
  f32x4 acc[NBL * 4];
#pragma unroll
  for (int i = 0; i < NBL * 4; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;
  const float inv_cap = cap > 0.f ? 1.0f / cap : 0.f;
  const float hs = head_scale != nullptr ? head_scale[head] : 1.0f;

  constexpr int CHK = Dp >> 3, CHV = Dvp >> 3;       // 16 B chunks per row
  // block ids of the keys [t_begin*32, t_end*32) into LDS (when they fit;
  // the range spans the gap between kept and window tiles, if there is one)
  const int blk0 = t_begin * CM_KT / block_size;
  const int nblk = (min(t_end * CM_KT, kmax) + block_size - 1) / block_size - blk0;
  const bool tbl_ok = nblk <= 512 && nblk > 0;
  if (tbl_ok)
    for (int i = tid; i < nblk; i += 256) tbl[i] = table[blk0 + i];
  __syncthreads();

  // chunk c of a tile: key c / CH, columns (c % CH)*8 .. +8
  auto fetch = [&](const unsigned short* cache, int width, int CH, int t,
                   int i) -> cm_u16x8 {
    const int c = tid + i * 256;
    cm_u16x8 v8 = {{0, 0, 0, 0, 0, 0, 0, 0}};
    if (c < CM_KT * CH) {
      const int kl = c / CH, col = (c - kl * CH) * 8;
      const int key = t * CM_KT + kl;
      if (key < kmax && col < width) {
        const int b = key / block_size;
        const long blk = tbl_ok ? tbl[b - blk0] : table[b];
        v8 = *reinterpret_cast<const cm_u16x8*>(
            cache + ((blk * n_kv + kvh) * block_size + key % block_size) *
                        (long)width + col);
      }
    }
    return v8;
  };
  auto put = [&](unsigned short* img, int CH, int i, const cm_u16x8& v8) {
    const int c = tid + i * 256;
    if (c < CM_KT * CH) {
      const int kl = c / CH, col = (c - kl * CH) * 8;
      *reinterpret_cast<cm_u16x8*>(
          img + (col >> 4) * 512 + ((kl >> 2) & 1) * 256 + (kl >> 3) * 64 +
          (kl & 3) * 16 + (col & 15)) = v8;
    }
  };
  cm_u16x8 prek[PF ? NPK : 1], prev[PF ? NPV : 1];
  if (PF && i_begin < i_end) {
#pragma unroll
    for (int i = 0; i < NPK; ++i) prek[i] = fetch(k_cache, D, CHK, t_begin, i);
    if (!same) {
#pragma unroll
      for (int i = 0; i < NPV; ++i) prev[i] = fetch(v_cache, Dv, CHV, t_begin, i);
    }
  }

  for (int it = i_begin; it < i_end; ++it) {
    const int t = tile_at(it);
    const int k0 = t * CM_KT;
    __syncthreads();
    if (PF) {
#pragma unroll
      for (int i = 0; i < NPK; ++i) put(kt, CHK, i, prek[i]);
      if (!same) {
#pragma unroll
        for (int i = 0; i < NPV; ++i) put(vt, CHV, i, prev[i]);
      }
    } else {
#pragma unroll
      for (int i = 0; i < NPK; ++i) put(kt, CHK, i, fetch(k_cache, D, CHK, t, i));
      if (!same) {
#pragma unroll
        for (int i = 0; i < NPV; ++i) put(vt, CHV, i, fetch(v_cache, Dv, CHV, t, i));
      }
    }
    __syncthreads();
    if (PF && it + 1 < i_end) {         // next tile flies during the compute
      const int tn = tile_at(it + 1);
#pragma unroll
      for (int i = 0; i < NPK; ++i) prek[i] = fetch(k_cache, D, CHK, tn, i);
      if (!same) {
#pragma unroll
        for (int i = 0; i < NPV; ++i) prev[i] = fetch(v_cache, Dv, CHV, tn, i);
      }
    }
    if (!wave_on) continue;
    // ---- scores ------------------------------------------------------------
    float sc[8];
#pragma unroll
    for (int h2 = 0; h2 < 2; ++h2) {
      // A row n is key k0 + (n>>2)*8 + h2*4 + (n&3); its image offset:
      const unsigned short* krow = kt + h2 * 256 + (n >> 2) * 64 + (n & 3) * 16;
      f32x4 sacc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kc = 0; kc < KQ; ++kc) {
        const int col = kc * 32 + g * 8;
        const bf16x8 a = cm_ld8(krow + (col >> 4) * 512 + (col & 15));
        sacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, qf[kc], sacc, 0, 0,
                                                       0);
      }
#pragma unroll
      for (int rr = 0; rr < 4; ++rr) {
        const int kk = k0 + g * 8 + h2 * 4 + rr;     // key of C row g*4+rr
        float sv = sacc[rr] * scale * hs;
        if (cap > 0.f) sv = cap * cm_tanh(sv * inv_cap);
        sc[h2 * 4 + rr] =
            (kk < limit && (kk >= lo || kk < keep_first)) ? sv : -INFINITY;
      }
    }
    float mloc = sc[0];
#pragma unroll
    for (int i = 1; i < 8; ++i) mloc = fmaxf(mloc, sc[i]);
    mloc = fmaxf(mloc, __shfl_xor(mloc, 16, 64));
    mloc = fmaxf(mloc, __shfl_xor(mloc, 32, 64));
    const float m_new = fmaxf(m, mloc);
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = __expf(m - m_use);
    float p[8], psum = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) { p[i] = __expf(sc[i] - m_use); psum += p[i]; }
    psum += __shfl_xor(psum, 16, 64);
    psum += __shfl_xor(psum, 32, 64);
    l = l * alpha + psum;
    m = m_new;
    // exact 3-way bf16 split of the fp32 weights
    bf16x8 b1, b2, b3;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const unsigned short h1 = f32_to_bf16(p[i]);
      const float r1 = p[i] - bf16_to_f32(h1);
      const unsigned short h2 = f32_to_bf16(r1);
      const float r2 = r1 - bf16_to_f32(h2);
      b1[i] = (short)h1; b2[i] = (short)h2; b3[i] = (short)f32_to_bf16(r2);
    }
    // four 16-column tiles per batch: 8 transpose reads, then 12 MFMAs
    const unsigned vbase = (unsigned)(unsigned long long)(vt) +
                           (unsigned)(g * 128 + n * 8);
#pragma unroll
    for (int lb = 0; lb < NBL; ++lb) {
      const int nb = lb * CS + cpart;
      if (nb * 64 < Dvp) {
        typedef __attribute__((__vector_size__(2 * sizeof(unsigned)))) unsigned u32x2;
        u32x2 tr[8];
        const unsigned va = vbase + (unsigned)(nb * 4096);
        asm volatile(
            "ds_read_b64_tr_b16 %[t0], %[a] offset:0\n\t"
            "ds_read_b64_tr_b16 %[t1], %[a] offset:512\n\t"
            "ds_read_b64_tr_b16 %[t2], %[a] offset:1024\n\t"
            "ds_read_b64_tr_b16 %[t3], %[a] offset:1536\n\t"
            "ds_read_b64_tr_b16 %[t4], %[a] offset:2048\n\t"
            "ds_read_b64_tr_b16 %[t5], %[a] offset:2560\n\t"
            "ds_read_b64_tr_b16 %[t6], %[a] offset:3072\n\t"
            "ds_read_b64_tr_b16 %[t7], %[a] offset:3584\n\t"
            "s_waitcnt lgkmcnt(0)"
            : [t0] "=&v"(tr[0]), [t1] "=&v"(tr[1]), [t2] "=&v"(tr[2]),
              [t3] "=&v"(tr[3]), [t4] "=&v"(tr[4]), [t5] "=&v"(tr[5]),
              [t6] "=&v"(tr[6]), [t7] "=&v"(tr[7])
            : [a] "v"(va)
            : "memory");
#pragma unroll
        for (int nn = 0; nn < 4; ++nn) {
          const int no = lb * 4 + nn;
          bf16x8 a;
          unsigned* aw = reinterpret_cast<unsigned*>(&a);
          aw[0] = tr[2 * nn][0];
          aw[1] = tr[2 * nn][1];
          aw[2] = tr[2 * nn + 1][0];
          aw[3] = tr[2 * nn + 1][1];
          acc[no] *= alpha;
          acc[no] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b1, acc[no], 0, 0, 0);
          acc[no] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b2, acc[no], 0, 0, 0);
          acc[no] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b3, acc[no], 0, 0, 0);
        }
      }
    }
  }
  if (!wave_on || !row_ok) return;
  // acc[lb*4+nn][rr] = O^T[col = ((lb*CS+cpart)*4+nn)*16 + g*4 + rr][row n]
  if (n_part == 1 && sink != nullptr) l += __expf(sink[head] - m);
  const float inv = l > 0.f ? 1.0f / l : 0.f;
  const long base = grow * n_part + blockIdx.y;
  float* orow = (n_part == 1) ? out + grow * Dv : ws_acc + base * Dv;
  const float mul = (n_part == 1) ? inv : 1.0f;
#pragma unroll
  for (int lb = 0; lb < NBL; ++lb)
#pragma unroll
    for (int nn = 0; nn < 4; ++nn)
#pragma unroll
      for (int rr = 0; rr < 4; ++rr) {
        const int col = ((lb * CS + cpart) * 4 + nn) * 16 + g * 4 + rr;
        if (col < Dv) orow[col] = acc[lb * 4 + nn][rr] * mul;
      }
  if (n_part > 1 && g == 0 && cpart == 0) {
    ws_ml[base * 2] = m; ws_ml[base * 2 + 1] = l;
  }
}

// out[row] = sum_p acc[row][p] e^(m_p - M) / sum_p l_p e^(m_p - M)
__global__ void __launch_bounds__(256) capped_attn_merge_kernel(
    float* __restrict__ out, const float* __restrict__ ws_acc,
    const float* __restrict__ ws_ml, int r, int n_part, int heads,
    const float* __restrict__ sink) {
  __shared__ float wgt[64];
  const long row = blockIdx.x;                 // token * heads + head
  const int tid = threadIdx.x;
  if (tid < 64) {
    const bool on = tid < n_part;
    const float mp = on ? ws_ml[(row * n_part + tid) * 2] : -INFINITY;
    const float lp = on ? ws_ml[(row * n_part + tid) * 2 + 1] : 0.f;
    float M = wave_reduce_max(mp);
    const float sk = sink ? sink[row % heads] : -INFINITY;
    M = fmaxf(M, sk);
    if (M == -INFINITY) M = 0.f;
    const float e = on ? __expf(mp - M) : 0.f;
    const float L = wave_reduce_sum(lp * e) + (sink ? __expf(sk - M) : 0.f);
    wgt[tid] = (L > 0.f) ? e / L : 0.f;
  }
  __syncthreads();
  const float* base = ws_acc + row * n_part * (long)r;
  for (int c = tid; c < r; c += 256) {
    float a = 0.f;
#pragma unroll 8
    for (int p = 0; p < n_part; ++p) a += base[(long)p * r + c] * wgt[p];
    out[row * r + c] = a;
  }
}

// Which instantiation covers (D, Dv); 0 = none (caller uses the scalar path).
int capped_attn_mfma_class(int D, int Dv) {
  if (D % 8 != 0 || Dv % 8 != 0) return 0;
  if (D <= 64 && Dv <= 64) return 1;
  if (D <= 128 && Dv <= 128) return 2;
  if (D <= 128 && Dv <= 256) return 3;
  if (D <= 256 && Dv <= 256) return 4;
  return 0;
}

void launch_capped_attn_mfma(float* out, float* ws_acc, float* ws_ml,
                             const unsigned short* q,
                             const unsigned short* k_cache,
                             const unsigned short* v_cache,
                             const int* block_tables, const int* cu_q,
                             const int* seq_lens, int tokens, int n_seqs,
                             int heads, int n_kv, int D, int Dv,
                             int block_size, int table_width, float scale,
                             float cap, long q_stride, int n_part, int window,
                             const float* sink, int keep_first,
                             const float* head_scale, hipStream_t st) {
  if (tokens == 0) return;
  const int cls = capped_attn_mfma_class(D, Dv);
  const int per = heads / n_kv;
  // decode with few heads per group: split the output columns over the waves
  const int cs = (cu_q == nullptr) ? (per <= 16 ? 4 : per <= 32 ? 2 : 1) : 1;
  const int rows_wg = 64 / cs;
  int blocks;
  if (cu_q == nullptr)
    blocks = n_seqs * ((per + rows_wg - 1) / rows_wg);
  else
    blocks = (int)(((long)tokens * per + rows_wg - 1) / rows_wg) + n_seqs;
  dim3 grid(blocks, n_part, n_kv);
#define CM_LAUNCH(KQ, NO, CS)                                                \
  hipLaunchKernelGGL((capped_attn_mfma_kernel<KQ, NO, CS>), grid, dim3(256), \
                     (size_t)(KQ * 2 + NO) * 1024, st, out, ws_acc, ws_ml,   \
                     q, k_cache, v_cache, block_tables, cu_q, seq_lens,      \
                     n_seqs, heads, n_kv, D, Dv, block_size, table_width,    \
                     scale, cap, q_stride, n_part, window, sink, keep_first, \
                     head_scale)
#define CM_BY_CS(KQ, NO)                                                     \
  do {                                                                       \
    if (cs == 4) CM_LAUNCH(KQ, NO, 4);                                       \
    else if (cs == 2) CM_LAUNCH(KQ, NO, 2);                                  \
    else CM_LAUNCH(KQ, NO, 1);                                               \
  } while (0)
  if (cls == 1) CM_BY_CS(2, 4);
  else if (cls == 2) CM_BY_CS(4, 8);
  else if (cls == 3) CM_BY_CS(4, 16);
  else CM_BY_CS(8, 16);
#undef CM_BY_CS
#undef CM_LAUNCH
  if (n_part > 1)
    hipLaunchKernelGGL(capped_attn_merge_kernel,
                       dim3((unsigned)tokens * heads), dim3(256), 0, st, out,
                       ws_acc, ws_ml, Dv, n_part, heads, sink);
}

}  // namespace hyb
}  // namespace xllm
