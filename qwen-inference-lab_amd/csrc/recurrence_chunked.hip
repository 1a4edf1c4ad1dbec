// The linear recurrences of recurrence.hip (S_t = a_t S_(t-1) + b_t k_t v_t^T, o_t = S_t^T q_t; the same gating modes,
// the same state slot) for long runs of tokens, in blocks of SCAN_BLOCK tokens that are worked on side by side.
//
// With the log gates f_u (keep) and i_s (input) of a block, F_t = f_0 + ... + f_t, e_s = i_s - F_s and the running
// maximum carried into the block m_in (over the state S_in, normaliser n_in that it scales):
//     M_t = max(m_in, e_0 .. e_t)                       m_t = F_t + M_t
//     S_t = exp(m_in - M_t) S_in + sum_(s <= t) exp(e_s - M_t) k_s v_s^T            (every exponent <= 0)
//     o_t = exp(m_in - M_t) S_in^T q_t + sum_(s <= t) exp(e_s - M_t) (q_t . k_s) v_s
// and n_t . q_t the same with 1 for v_s.  With a fixed decay d: exp(e_s - M_t) is d^(t - s) and exp(m_in - M_t) is
// d^(t + 1).  Four kernels, all float32 (sums of gates and their differences in float64, so that the exponent of a
// weight near 1 is not the rounded difference of two large numbers):
//   rotate   queries and keys rotated by position and scaled, once, into float32 rows;
//   sums     per block: U = sum_s w_s k_s v_s^T (and the normaliser's sum_s w_s k_s) with w_s = exp(e_s - max e), what
//            the block adds to the state at its end: a [dim, 64 tokens] x [64 tokens, vdim] product, tiled 64 x 64;
//   carry    block after block, S_out = exp(m_in - M_end) S_in + exp(max e - M_end) U, element by element; every block's
//            S_in replaces its U, the last S_out goes to the state slot;
//   outputs  per block: [q scaled by its carry weight | masked weighted q k^T] x [S_in ; v], tiled 64 tokens x 64 columns.
// The tiled products run on the vector units in float32 (4 x 4 outputs a thread, operands staged in LDS).
//
// QIL_SCAN_CHANNEL (every row i of S decays by a factor of its own, a_t[i] = exp(logsigmoid(z_t[i]) / tau)): with
// G_t[i] the sum of the block's log2 decays of row i up to token t (one more kernel, `decays`, walks them),
//     S_t = diag(2^G_t) S_in + sum_(s <= t) diag(2^(G_t - G_s)) k_s v_s^T
//     o_t = S_in^T (q_t * 2^G_t) + sum_(s <= t) (sum_i q_t[i] k_s[i] 2^(G_t[i] - G_s[i])) v_s
// so `sums` weighs row i of k_s by 2^(G_end[i] - G_s[i]), `carry` keeps row i by 2^G_end[i], and `outputs` makes the
// scores inside the block with the weight inside the sum over i (every exponent <= 0: nothing is divided by a decay).
#include "common.h"

enum { QIL_SCAN_DECAY = 0, QIL_SCAN_MLSTM = 1, QIL_SCAN_CHANNEL = 2 };
#define SCAN_BLOCK 64
#define SCAN_TOP_TILE 16                                         // recurrence.hip keeps one maximum per 16 state columns

__device__ __forceinline__ float log_sigmoid_c(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

// Lane t of a wave: F_t and e_t of token t of the block (e = -inf past the block's end).
struct GateLane { double sum, lead; };
__device__ __forceinline__ GateLane gate_lane(const float* __restrict__ gates, const float* __restrict__ gate_bias,
                                              float cap, int row, int h, int heads, bool live, int lane) {
  float in = 0.f, keep = 0.f;
  if (live) {
    in = cap * tanhf((gates[(size_t)row * 2 * heads + h] + gate_bias[h]) / cap);
    keep = log_sigmoid_c(cap * tanhf((gates[(size_t)row * 2 * heads + heads + h] + gate_bias[heads + h]) / cap));
  }
  double sum = keep;
#pragma unroll
  for (int d = 1; d < QIL_WAVE; d <<= 1) {
    const double up = __shfl_up(sum, d, QIL_WAVE);
    if (lane >= d) sum += up;
  }
  GateLane g;
  g.sum = sum;
  g.lead = live ? (double)in - sum : -INFINITY;
  return g;
}

// Where block c of sequence seq keeps its sums: sequences before it took at most row0 / SCAN_BLOCK + seq places.
__device__ __forceinline__ int block_place(int row0, int seq, int c) { return row0 / SCAN_BLOCK + seq + c; }

// CHANNEL: gsum[row, e] = sum over the block's tokens up to this row of log2(a[e]), e over heads * dim; the sum runs
// in float64 and is rounded once.  grid (blocks of the longest sequence, sequences, heads * dim / 256)
__global__ void __launch_bounds__(256)
scan_decays_kernel(const float* __restrict__ z, float tau, const int* __restrict__ cu_seqlens, float* __restrict__ gsum,
                   int hd) {
  const int c = blockIdx.x, seq = blockIdx.y, e = blockIdx.z * blockDim.x + threadIdx.x;
  const int row0 = cu_seqlens[seq], len = cu_seqlens[seq + 1] - row0;
  if (c * SCAN_BLOCK >= len || e >= hd) return;
  const int r0 = row0 + c * SCAN_BLOCK, lc = min(SCAN_BLOCK, len - c * SCAN_BLOCK);
  double sum = 0.0;
  for (int t0 = 0; t0 < lc; t0 += 8) {
    float in[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) in[u] = z[(size_t)(r0 + min(t0 + u, lc - 1)) * hd + e];
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (t0 + u < lc) {
        sum += (double)(log_sigmoid_c(in[u]) / tau) * 1.4426950408889634;
        gsum[(size_t)(r0 + t0 + u) * hd + e] = (float)sum;
      }
  }
}

template <typename T>
__global__ void scan_rotate_kernel(const T* __restrict__ proj, int proj_row, int q_off, int k_off,
                                   const float* __restrict__ freq, int rot, float q_scale, float k_scale,
                                   const int* __restrict__ cu_seqlens, const int* __restrict__ seq_starts, int n_seqs,
                                   float* __restrict__ qk, int heads, int dim) {
  const int row = blockIdx.x;
  int seq = 0;
  while (seq + 1 < n_seqs && cu_seqlens[seq + 1] <= row) ++seq;
  const float position = (float)(seq_starts[seq] + row - cu_seqlens[seq]);
  const int half = rot / 2, hd = heads * dim;
  for (int idx = threadIdx.x; idx < 2 * hd; idx += blockDim.x) {
    const int which = idx / hd, e = idx - which * hd, i = e % dim;
    const T* x = proj + (size_t)row * proj_row + (which ? k_off : q_off) + e;
    float value = ld(x);
    if (i < rot) {
      float sn, cs;
      sincosf(position * freq[i < half ? i : i - half], &sn, &cs);
      value = i < half ? value * cs - ld(x + half) * sn : value * cs + ld(x - half) * sn;
    }
    qk[(size_t)row * 2 * hd + idx] = value * (which ? k_scale : q_scale);
  }
}

// grid (blocks of the longest sequence, sequences x heads, dim tiles x vdim tiles)
template <typename T, int MODE>
__global__ void __launch_bounds__(256)
scan_sums_kernel(const T* __restrict__ proj, int proj_row, int v_off, const float* __restrict__ qk,
                 const float* __restrict__ gates, const float* __restrict__ gate_bias, float cap,
                 const float* __restrict__ decay, const float* __restrict__ state, size_t slot_stride,
                 const int* __restrict__ cu_seqlens, const int* __restrict__ seq_starts, const int* __restrict__ seq_slots,
                 float* __restrict__ sums, float* __restrict__ norm_sums, double* __restrict__ info,
                 float* __restrict__ carried, int heads, int dim, int vdim, int dim_tiles,
                 const float* __restrict__ gsum) {
  __shared__ __align__(16) float kw[SCAN_BLOCK][64];
  __shared__ __align__(16) float vs[SCAN_BLOCK][64];
  __shared__ float w[SCAN_BLOCK];
  const int c = blockIdx.x, seq = blockIdx.y / heads, h = blockIdx.y % heads;
  const int it = blockIdx.z % dim_tiles, jt = blockIdx.z / dim_tiles, tid = threadIdx.x;
  const int row0 = cu_seqlens[seq], len = cu_seqlens[seq + 1] - row0;
  if (c * SCAN_BLOCK >= len) return;
  const int r0 = row0 + c * SCAN_BLOCK, lc = min(SCAN_BLOCK, len - c * SCAN_BLOCK);
  const size_t at = (size_t)block_place(row0, seq, c) * heads + h;
  if (tid < QIL_WAVE) {
    const bool live = tid < lc;
    float weight;
    if (MODE == QIL_SCAN_MLSTM) {
      const GateLane g = gate_lane(gates, gate_bias, cap, r0 + (live ? tid : 0), h, heads, live, tid);
      double top = g.lead;
#pragma unroll
      for (int d = QIL_WAVE / 2; d > 0; d >>= 1) top = fmax(top, __shfl_xor(top, d, QIL_WAVE));
      weight = live ? expf((float)(g.lead - top)) : 0.f;
      const double total = __shfl(g.sum, lc - 1, QIL_WAVE);
      if (blockIdx.z == 0 && tid == 0) {
        info[at * 2] = top;
        info[at * 2 + 1] = total;
        if (c == 0) {                                            // the maximum the sequence brings: read before carry writes
          const int tiles = (vdim + SCAN_TOP_TILE - 1) / SCAN_TOP_TILE;
          const float* s_top = state + (size_t)seq_slots[seq] * slot_stride + (size_t)heads * dim * vdim +
                               (size_t)heads * dim + (size_t)h * (tiles + 1);
          carried[at] = seq_starts[seq] == 0 ? 0.f : *s_top;
        }
      }
    } else if (MODE == QIL_SCAN_CHANNEL) {
      weight = live ? 1.f : 0.f;                                 // (the rows' own weights follow below)
    } else {
      weight = live ? (float)pow((double)decay[h], (double)(lc - 1 - tid)) : 0.f;
    }
    w[tid] = weight;
  }
  __syncthreads();
  const size_t hd = (size_t)heads * dim;
  for (int idx = tid; idx < SCAN_BLOCK * 64; idx += 256) {
    const int s = idx / 64, x = idx % 64, i = it * 64 + x, j = jt * 64 + x;
    float weight = w[s];
    if (MODE == QIL_SCAN_CHANNEL && s < lc && i < dim)
      weight = __builtin_amdgcn_exp2f(gsum[(size_t)(r0 + lc - 1) * hd + (size_t)h * dim + i] -
                                      gsum[(size_t)(r0 + s) * hd + (size_t)h * dim + i]);
    kw[s][x] = (s < lc && i < dim) ? weight * qk[(size_t)(r0 + s) * 2 * hd + hd + (size_t)h * dim + i] : 0.f;
    vs[s][x] = (s < lc && j < vdim) ? ld(proj + (size_t)(r0 + s) * proj_row + v_off + h * vdim + j) : 0.f;
  }
  __syncthreads();
  const int ti = tid / 16, tj = tid % 16;
  float acc[4][4] = {};
  for (int s = 0; s < lc; ++s) {
    const float4 a4 = *reinterpret_cast<const float4*>(&kw[s][ti * 4]);
    const float4 b4 = *reinterpret_cast<const float4*>(&vs[s][tj * 4]);
    const float a[4] = {a4.x, a4.y, a4.z, a4.w}, b[4] = {b4.x, b4.y, b4.z, b4.w};
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
      for (int q = 0; q < 4; ++q) acc[r][q] += a[r] * b[q];
  }
  float* u = sums + at * dim * vdim;
#pragma unroll
  for (int r = 0; r < 4; ++r)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int i = it * 64 + ti * 4 + r, j = jt * 64 + tj * 4 + q;
      if (i < dim && j < vdim) u[(size_t)i * vdim + j] = acc[r][q];
    }
  if (MODE == QIL_SCAN_MLSTM && jt == 0 && tid < 64 && it * 64 + tid < dim) {
    float total = 0.f;
    for (int s = 0; s < lc; ++s) total += kw[s][tid];
    norm_sums[at * dim + it * 64 + tid] = total;
  }
}

// grid (sequences, heads, elements of a head's state / 256): one thread an element of S (or of n), block after block.
template <int MODE>
__global__ void __launch_bounds__(256)
scan_carry_kernel(float* __restrict__ sums, float* __restrict__ norm_sums, const double* __restrict__ info,
                  float* __restrict__ carried, const float* __restrict__ decay, float* __restrict__ state,
                  size_t slot_stride, const int* __restrict__ cu_seqlens, const int* __restrict__ seq_starts,
                  const int* __restrict__ seq_slots, int heads, int dim, int vdim, const float* __restrict__ gsum) {
  const int seq = blockIdx.x, h = blockIdx.y, e = blockIdx.z * blockDim.x + threadIdx.x;
  const int mat = dim * vdim, total = mat + (MODE == QIL_SCAN_MLSTM ? dim : 0);
  const int row0 = cu_seqlens[seq], len = cu_seqlens[seq + 1] - row0;
  if (len <= 0 || e >= total) return;
  const bool fresh = seq_starts[seq] == 0;
  const int tiles = (vdim + SCAN_TOP_TILE - 1) / SCAN_TOP_TILE;
  float* slot = state + (size_t)seq_slots[seq] * slot_stride;
  float* mine = e < mat ? slot + (size_t)h * mat + e : slot + (size_t)heads * mat + (size_t)h * dim + (e - mat);
  float* s_top = slot + (size_t)heads * mat + (size_t)heads * dim + (size_t)h * (tiles + 1);
  float value = fresh ? 0.f : *mine;
  const int blocks = (len + SCAN_BLOCK - 1) / SCAN_BLOCK;
  const size_t first = (size_t)block_place(row0, seq, 0) * heads + h;
  float top = MODE == QIL_SCAN_MLSTM ? carried[first] : 0.f;
  const double rate = MODE == QIL_SCAN_DECAY ? (double)decay[h] : 0.0;
  const float keep_whole = MODE == QIL_SCAN_DECAY ? (float)pow(rate, (double)SCAN_BLOCK) : 0.f;   // a whole block's decay
  for (int c = 0; c < blocks; ++c) {
    const size_t at = first + (size_t)c * heads;
    float* u = e < mat ? sums + at * mat + e : norm_sums + at * dim + (e - mat);
    float keep, take = 1.f;
    if (MODE == QIL_SCAN_MLSTM) {
      const double local = info[at * 2], end = fmax((double)top, local);
      keep = expf((float)((double)top - end));
      take = expf((float)(local - end));
      if (e == 0) carried[at] = top;
      top = (float)(info[at * 2 + 1] + end);
    } else if (MODE == QIL_SCAN_CHANNEL) {
      const int last = row0 + min((c + 1) * SCAN_BLOCK, len) - 1;       // the block's last token
      keep = __builtin_amdgcn_exp2f(gsum[(size_t)last * heads * dim + (size_t)h * dim + e / vdim]);
    } else {
      const int lc = min(SCAN_BLOCK, len - c * SCAN_BLOCK);
      keep = lc == SCAN_BLOCK ? keep_whole : (float)pow(rate, (double)lc);
    }
    const float add = *u;
    *u = value;
    value = keep * value + take * add;
  }
  *mine = value;
  if (MODE == QIL_SCAN_MLSTM && e <= tiles) s_top[e] = top;
}

// grid (blocks of the longest sequence, sequences x heads, vdim tiles)
#define OUT_SLAB 32                                               // elements of a head's dim staged at a time
#define OUT_PAD 68                                                // row of a transposed tile: 64 tokens and 4 to spread banks
template <typename T, int MODE>
__global__ void __launch_bounds__(256)
scan_outputs_kernel(const T* __restrict__ proj, int proj_row, int v_off, const float* __restrict__ qk,
                    const float* __restrict__ gates, const float* __restrict__ gate_bias, float cap,
                    const float* __restrict__ decay, const float* __restrict__ before, const float* __restrict__ norm_before,
                    const float* __restrict__ carried, const int* __restrict__ cu_seqlens, float* __restrict__ out,
                    float* __restrict__ below, int heads, int dim, int vdim, const float* __restrict__ gsum) {
  // first the slabs [q^T | k^T | S_in rows] (CHANNEL: and [G^T | (q 2^G)^T]), then [weighted scores^T | v]
  constexpr bool CHANNEL = MODE == QIL_SCAN_CHANNEL;
  __shared__ __align__(16) float stage[SCAN_BLOCK * OUT_PAD + SCAN_BLOCK * 64 + (CHANNEL ? 2 * OUT_SLAB * OUT_PAD : 0)];
  float* gT = stage + 2 * OUT_SLAB * OUT_PAD + OUT_SLAB * 64;
  float* eT = gT + OUT_SLAB * OUT_PAD;
  __shared__ float nin[OUT_SLAB], cw[SCAN_BLOCK], em[SCAN_BLOCK], pw[SCAN_BLOCK + 1];
  __shared__ double lead[SCAN_BLOCK], tops[SCAN_BLOCK];
  float* qT = stage;
  float* kT = stage + OUT_SLAB * OUT_PAD;
  float* sin = stage + 2 * OUT_SLAB * OUT_PAD;
  float* pT = stage;
  float* vs = stage + SCAN_BLOCK * OUT_PAD;
  const int c = blockIdx.x, seq = blockIdx.y / heads, h = blockIdx.y % heads, jt = blockIdx.z, tid = threadIdx.x;
  const int row0 = cu_seqlens[seq], len = cu_seqlens[seq + 1] - row0;
  if (c * SCAN_BLOCK >= len) return;
  const int r0 = row0 + c * SCAN_BLOCK, lc = min(SCAN_BLOCK, len - c * SCAN_BLOCK);
  const size_t at = (size_t)block_place(row0, seq, c) * heads + h;
  if (tid < QIL_WAVE) {
    if (MODE == QIL_SCAN_MLSTM) {
      const bool live = tid < lc;
      const GateLane g = gate_lane(gates, gate_bias, cap, r0 + (live ? tid : 0), h, heads, live, tid);
      const double brought = (double)carried[at];
      double top = g.lead;
#pragma unroll
      for (int d = 1; d < QIL_WAVE; d <<= 1) {
        const double up = __shfl_up(top, d, QIL_WAVE);
        if (tid >= d) top = fmax(top, up);
      }
      top = fmax(top, brought);
      lead[tid] = g.lead;
      tops[tid] = top;
      cw[tid] = expf((float)(brought - top));
      em[tid] = expf(-(float)(g.sum + top));
    } else if (!CHANNEL) {
      pw[tid] = (float)pow((double)decay[h], (double)tid);
      if (tid == 0) pw[SCAN_BLOCK] = (float)pow((double)decay[h], (double)SCAN_BLOCK);
    }
  }
  const int ti = tid / 16, tj = tid % 16;
  const size_t hd = (size_t)heads * dim;
  const float* s_in = before + at * dim * vdim;
  float p[4][4] = {}, o[4][4] = {}, nq[4] = {};
  for (int i0 = 0; i0 < dim; i0 += OUT_SLAB) {
    __syncthreads();
    for (int idx = tid; idx < SCAN_BLOCK * OUT_SLAB; idx += 256) {
      const int t = idx / OUT_SLAB, x = idx % OUT_SLAB, i = i0 + x;
      const bool ok = t < lc && i < dim;
      const float* src = qk + (size_t)(r0 + (ok ? t : 0)) * 2 * hd + (size_t)h * dim + (ok ? i : 0);
      qT[x * OUT_PAD + t] = ok ? src[0] : 0.f;
      kT[x * OUT_PAD + t] = ok ? src[hd] : 0.f;
      if (CHANNEL) {
        const float g = ok ? gsum[(size_t)(r0 + t) * hd + (size_t)h * dim + i] : 0.f;
        gT[x * OUT_PAD + t] = g;
        eT[x * OUT_PAD + t] = ok ? src[0] * __builtin_amdgcn_exp2f(g) : 0.f;
      }
    }
    for (int idx = tid; idx < OUT_SLAB * 64; idx += 256) {
      const int x = idx / 64, y = idx % 64, i = i0 + x, j = jt * 64 + y;
      sin[x * 64 + y] = (i < dim && j < vdim) ? s_in[(size_t)i * vdim + j] : 0.f;
    }
    if (MODE == QIL_SCAN_MLSTM && tid < OUT_SLAB) nin[tid] = i0 + tid < dim ? norm_before[at * dim + i0 + tid] : 0.f;
    __syncthreads();
#pragma unroll 4
    for (int x = 0; x < OUT_SLAB; ++x) {
      const float4 q4 = *reinterpret_cast<const float4*>(&qT[x * OUT_PAD + ti * 4]);
      const float4 k4 = *reinterpret_cast<const float4*>(&kT[x * OUT_PAD + tj * 4]);
      const float4 s4 = *reinterpret_cast<const float4*>(&sin[x * 64 + tj * 4]);
      const float q[4] = {q4.x, q4.y, q4.z, q4.w}, k[4] = {k4.x, k4.y, k4.z, k4.w}, s[4] = {s4.x, s4.y, s4.z, s4.w};
      const float nx = MODE == QIL_SCAN_MLSTM ? nin[x] : 0.f;
      if (CHANNEL) {
        // the weight 2^(G_t - G_s) of every (query, key, row of S) inside the sum; what came in is taken by q 2^G_t
        const float4 e4 = *reinterpret_cast<const float4*>(&eT[x * OUT_PAD + ti * 4]);
        const float qe[4] = {e4.x, e4.y, e4.z, e4.w};
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
          for (int u = 0; u < 4; ++u) o[r][u] += qe[r] * s[u];
        if (tj <= ti) {                                          // (tiles above the diagonal hold no visible key)
          const float4 a4 = *reinterpret_cast<const float4*>(&gT[x * OUT_PAD + ti * 4]);
          const float4 b4 = *reinterpret_cast<const float4*>(&gT[x * OUT_PAD + tj * 4]);
          const float gt[4] = {a4.x, a4.y, a4.z, a4.w}, gs[4] = {b4.x, b4.y, b4.z, b4.w};
#pragma unroll
          for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int u = 0; u < 4; ++u) p[r][u] += q[r] * k[u] * __builtin_amdgcn_exp2f(fminf(gt[r] - gs[u], 0.f));
        }
        continue;
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          p[r][u] += q[r] * k[u];
          o[r][u] += q[r] * s[u];
        }
        if (MODE == QIL_SCAN_MLSTM) nq[r] += q[r] * nx;
      }
    }
  }
  // the weights: scores of keys at or before the token by exp(e_s - M_t), what came in by exp(m_in - M_t)
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int t = ti * 4 + r;
    const float brought = MODE == QIL_SCAN_MLSTM ? cw[t] : CHANNEL ? 1.f : pw[t + 1];
    float row_sum = 0.f;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int s = tj * 4 + u;
      float weight = 0.f;
      if (s <= t && t < lc) weight = MODE == QIL_SCAN_MLSTM ? expf((float)(lead[s] - tops[t])) : CHANNEL ? 1.f : pw[t - s];
      p[r][u] *= weight;
      row_sum += p[r][u];
      o[r][u] *= brought;
    }
    if (MODE == QIL_SCAN_MLSTM) {
      row_sum += __shfl_xor(row_sum, 1, QIL_WAVE);
      row_sum += __shfl_xor(row_sum, 2, QIL_WAVE);
      row_sum += __shfl_xor(row_sum, 4, QIL_WAVE);
      row_sum += __shfl_xor(row_sum, 8, QIL_WAVE);
      nq[r] = nq[r] * brought + row_sum;
    }
  }
  __syncthreads();
#pragma unroll
  for (int u = 0; u < 4; ++u)
    *reinterpret_cast<float4*>(&pT[(tj * 4 + u) * OUT_PAD + ti * 4]) = make_float4(p[0][u], p[1][u], p[2][u], p[3][u]);
  for (int idx = tid; idx < SCAN_BLOCK * 64; idx += 256) {
    const int s = idx / 64, y = idx % 64, j = jt * 64 + y;
    vs[s * 64 + y] = (s < lc && j < vdim) ? ld(proj + (size_t)(r0 + s) * proj_row + v_off + h * vdim + j) : 0.f;
  }
  __syncthreads();
  for (int s = 0; s < lc; ++s) {
    const float4 p4 = *reinterpret_cast<const float4*>(&pT[s * OUT_PAD + ti * 4]);
    const float4 v4 = *reinterpret_cast<const float4*>(&vs[s * 64 + tj * 4]);
    const float a[4] = {p4.x, p4.y, p4.z, p4.w}, b[4] = {v4.x, v4.y, v4.z, v4.w};
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
      for (int u = 0; u < 4; ++u) o[r][u] += a[r] * b[u];
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int t = ti * 4 + r;
    if (t >= lc) continue;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int j = jt * 64 + tj * 4 + u;
      if (j < vdim) out[(size_t)(r0 + t) * heads * vdim + (size_t)h * vdim + j] = o[r][u];
    }
    if (MODE == QIL_SCAN_MLSTM && jt == 0 && tj == 0) below[(size_t)(r0 + t) * heads + h] = fmaxf(fabsf(nq[r]), em[t]) + 1e-6f;
  }
}

static size_t chunked_places(int n, int n_seqs) { return (size_t)n / SCAN_BLOCK + n_seqs; }

extern "C" {

// Floats of the scratch memory of a step of n rows in n_seqs sequences.
size_t qil_state_scan_chunked_workspace(int n, int n_seqs, int heads, int dim, int vdim, int mode) {
  const size_t places = chunked_places(n, n_seqs);
  size_t floats = places * heads * 4 + (places * heads + 3) / 4 * 4 + (size_t)n * 2 * heads * dim + places * heads * dim * vdim;
  if (mode == QIL_SCAN_MLSTM) floats += places * heads * dim;
  if (mode == QIL_SCAN_CHANNEL) floats += (size_t)n * heads * dim;
  return floats;
}

// As qil_state_scan, for steps in which a sequence has many rows (max_query: the most rows of one sequence).
int qil_state_scan_chunked(const void* proj, int dtype, int proj_row, int q_off, int k_off, int v_off, const float* gates,
                           const float* gate_bias, float cap, const float* decay, const float* freq, int rot, float q_scale,
                           float k_scale, float* state, size_t slot_stride, const int* cu_seqlens, const int* seq_starts,
                           const int* seq_slots, float* out, float* below, float* workspace, int n, int n_seqs,
                           int max_query, int heads, int dim, int vdim, int mode, hipStream_t s) {
  if (n_seqs == 0 || n == 0) return 0;
  if (dim < 1 || vdim < 1 || rot < 0 || rot % 2 || rot > dim || max_query < 1 ||
      mode < QIL_SCAN_DECAY || mode > QIL_SCAN_CHANNEL || !workspace || (size_t)n_seqs * heads > 65535)
    return -1;
  if ((mode == QIL_SCAN_MLSTM && (!gates || !gate_bias || !below)) || (mode == QIL_SCAN_DECAY && !decay) ||
      (mode == QIL_SCAN_CHANNEL && (!gates || !(cap > 0.f) || n_seqs > 65535)) || (rot && !freq)) return -1;
  const size_t places = chunked_places(n, n_seqs);
  double* info = reinterpret_cast<double*>(workspace);
  float* carried = workspace + places * heads * 4;
  float* qk = carried + (places * heads + 3) / 4 * 4;
  float* sums = qk + (size_t)n * 2 * heads * dim;
  float* norm_sums = sums + places * heads * dim * vdim;
  float* gsum = norm_sums;                                       // CHANNEL has no normaliser: its place holds the decays' sums
  const int blocks = (max_query + SCAN_BLOCK - 1) / SCAN_BLOCK;
  const int dim_tiles = (dim + 63) / 64, v_tiles = (vdim + 63) / 64;
  const int per_head = dim * vdim + (mode == QIL_SCAN_MLSTM ? dim : 0);
  const dim3 g_sums(blocks, n_seqs * heads, dim_tiles * v_tiles), g_carry(n_seqs, heads, (per_head + 255) / 256);
  const dim3 g_out(blocks, n_seqs * heads, v_tiles);
#define QIL_CHUNKED(T, MODE)                                                                                          \
  do {                                                                                                                \
    if (MODE == QIL_SCAN_CHANNEL)                                                                                     \
      hipLaunchKernelGGL(scan_decays_kernel, dim3(blocks, n_seqs, (heads * dim + 255) / 256), dim3(256), 0, s, gates,  \
                         cap, cu_seqlens, gsum, heads * dim);                                                          \
    hipLaunchKernelGGL(scan_rotate_kernel<T>, dim3(n), dim3(256), 0, s, (const T*)proj, proj_row, q_off, k_off, freq,  \
                       rot, q_scale, k_scale, cu_seqlens, seq_starts, n_seqs, qk, heads, dim);                         \
    hipLaunchKernelGGL((scan_sums_kernel<T, MODE>), g_sums, dim3(256), 0, s, (const T*)proj, proj_row, v_off, qk,      \
                       gates, gate_bias, cap, decay, state, slot_stride, cu_seqlens, seq_starts, seq_slots, sums,      \
                       norm_sums, info, carried, heads, dim, vdim, dim_tiles, gsum);                                   \
    hipLaunchKernelGGL(scan_carry_kernel<MODE>, g_carry, dim3(256), 0, s, sums, norm_sums, info, carried, decay,       \
                       state, slot_stride, cu_seqlens, seq_starts, seq_slots, heads, dim, vdim, gsum);                 \
    hipLaunchKernelGGL((scan_outputs_kernel<T, MODE>), g_out, dim3(256), 0, s, (const T*)proj, proj_row, v_off, qk,    \
                       gates, gate_bias, cap, decay, sums, norm_sums, carried, cu_seqlens, out, below, heads, dim,     \
                       vdim, gsum);                                                                                    \
  } while (0)
  if (dtype == QIL_F32) {
    if (mode == QIL_SCAN_MLSTM) QIL_CHUNKED(float, QIL_SCAN_MLSTM);
    else if (mode == QIL_SCAN_CHANNEL) QIL_CHUNKED(float, QIL_SCAN_CHANNEL);
    else QIL_CHUNKED(float, QIL_SCAN_DECAY);
  } else {
    if (mode == QIL_SCAN_MLSTM) QIL_CHUNKED(bf16_t, QIL_SCAN_MLSTM);
    else if (mode == QIL_SCAN_CHANNEL) QIL_CHUNKED(bf16_t, QIL_SCAN_CHANNEL);
    else QIL_CHUNKED(bf16_t, QIL_SCAN_DECAY);
  }
#undef QIL_CHUNKED
  QIL_RETURN_LAUNCH_STATUS();
}

}  // extern "C"
