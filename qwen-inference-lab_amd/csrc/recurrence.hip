// Linear recurrences with a matrix state per head, carried from token to token in float32:
//     S_t = a_t S_(t-1) + b_t k_t v_t^T          S [dim, vdim]
//     o_t = S_t^T q_t
// by gating mode:
//   QIL_SCAN_DECAY  a_t = decay_h (fixed per head), b_t = 1; o_t as above.
//   QIL_SCAN_MLSTM  log gates i_t = cap tanh((x_i + bias_i) / cap), f_t = logsigmoid(cap tanh((x_f + bias_f) / cap)),
//                   running maximum m_t = max(f_t + m_(t-1), i_t) with m = 0 before the first token,
//                   a_t = exp(f_t + m_(t-1) - m_t), b_t = exp(i_t - m_t); a normaliser n_t = a_t n_(t-1) + b_t k_t;
//                   o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6).
//   QIL_SCAN_CHANNEL a decay of its own for every row of S (key channel i of head h) and token:
//                   a_t[i] = sigmoid(z_t[h, i])^(1 / tau) = exp(logsigmoid(z_t[h, i]) / tau), b_t = 1, with z float32
//                   [n, heads * dim] in the place of the gates and tau in the place of the cap; o_t as above.
// Queries and keys may be rotated by position first (the leading rot elements of a head, element i with i + rot / 2,
// angle position * freq[i]) and are then scaled (q_scale, k_scale).  Gates, rotation, state and sums are float32.
//
// A block is one wave: one (sequence, head, 16 columns of the state).  The lanes are 16 columns by 4 groups of rows
// (group g owns the rows 4 m + r with m % 4 == g: the four groups read 64 consecutive bytes of a token's key); a lane
// keeps its quarter of a column of S in registers, two shuffles join the groups' parts of o_t, and the wave walks the
// sequence's tokens of this step in order.  (A wave's vector instruction takes four cycles: a lane with a whole column
// of 128 rows spent 1,500 cycles a token on 32 of the chip's 1,024 SIMDs.)  The tokens come in chunks of SCAN_CHUNK: a chunk's queries, keys,
// values and gate inputs are fetched into registers in one batch of requests while the chunk before is walked, then
// put into LDS, rotated and scaled there by the whole wave; the gates' factors a_t, b_t are made for the chunk (the
// running maximum by a short serial pass, the exponentials in parallel); the walk itself reads LDS 16 bytes at a time.
// MLSTM: the normaliser n_t is a column of its own kind; the last block along z keeps it (its lanes share the rows of
// n) and writes every token's denominator max(|n_t . q_t|, exp(-m_t)) + 1e-6; the blocks of S write S_t^T q_t
// undivided, and the head-norm kernel divides.  The state slot of a sequence is read unless the sequence starts at
// position 0, and written back at the end.
#include "common.h"

enum { QIL_SCAN_DECAY = 0, QIL_SCAN_MLSTM = 1, QIL_SCAN_CHANNEL = 2 };
#define SCAN_CHUNK 16
#define SCAN_COLUMNS 16                                          // state columns a block (one wave) owns

__device__ __forceinline__ float log_sigmoid(float z) {         // -softplus(-z), stable on both sides
  return fminf(z, 0.f) - log1pf(expf(-fabsf(z)));
}

// State of one slot: [heads][dim * vdim] matrices, then (MLSTM) [heads][dim] normalisers and [heads][tiles + 1] maxima,
// tiles = ceil(vdim / 16): every block along z reads and writes only its own copy of the maximum, so no block sees
// another's update.
template <typename T, int DMAX, int MODE>
__global__ void __launch_bounds__(64)
state_scan_kernel(const T* __restrict__ proj, int proj_row, int q_off, int k_off, int v_off,
                  const float* __restrict__ gates, const float* __restrict__ gate_bias, float cap,
                  const float* __restrict__ decay, const float* __restrict__ freq, int rot, float q_scale, float k_scale,
                  float* __restrict__ state, size_t slot_stride, const int* __restrict__ cu_seqlens,
                  const int* __restrict__ seq_starts, const int* __restrict__ seq_slots, float* __restrict__ out,
                  float* __restrict__ below, int heads, int dim, int vdim) {
  constexpr int CH = DMAX > 128 ? SCAN_CHUNK / 2 : SCAN_CHUNK;  // tokens a chunk
  constexpr int PER = CH * DMAX / 64;                           // elements of q (and of k) a lane fetches a chunk
  __shared__ __align__(16) float qs[CH][DMAX];
  __shared__ __align__(16) float ks[CH][DMAX];
  __shared__ float vs[CH][SCAN_COLUMNS];
  __shared__ __align__(16) float as[MODE == QIL_SCAN_CHANNEL ? CH : 1][DMAX];    // CHANNEL: every row's decay, token by token
  __shared__ float fa[CH], fb[CH], fe[CH], gi[CH], gk[CH], gm[CH + 1];
  const int seq = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int tiles = (vdim + SCAN_COLUMNS - 1) / SCAN_COLUMNS;
  const bool keeper = MODE == QIL_SCAN_MLSTM && (int)blockIdx.z == tiles;     // the block of the normaliser
  const int jj = lane & (SCAN_COLUMNS - 1), rg = lane / SCAN_COLUMNS;          // column of the tile, group of rows
  const int j = blockIdx.z * SCAN_COLUMNS + jj;
  const bool column = !keeper && j < vdim;
  const int row0 = cu_seqlens[seq], row1 = cu_seqlens[seq + 1], start = seq_starts[seq];
  float* slot = state + (size_t)seq_slots[seq] * slot_stride;
  float* s_mat = slot + (size_t)h * dim * vdim;
  float* s_norm = slot + (size_t)heads * dim * vdim + (size_t)h * dim;
  float* s_top = slot + (size_t)heads * dim * vdim + (size_t)heads * dim + (size_t)h * (tiles + 1) + blockIdx.z;
  const bool fresh = start == 0;

  // col[4 m + r]: row 16 m + 4 rg + r of the lane's column.  (keeper: rows lane, lane + 64, ... of n in col[0 .. DMAX / 64])
  float col[DMAX / 4];
#pragma unroll
  for (int e = 0; e < DMAX / 4; ++e) {
    const int i = 16 * (e / 4) + 4 * rg + (e & 3);
    col[e] = (!fresh && column && i < dim) ? s_mat[(size_t)i * vdim + j] : 0.f;
  }
  if (keeper) {
#pragma unroll
    for (int u = 0; u < (DMAX + 63) / 64; ++u) col[u] = (!fresh && lane + 64 * u < dim) ? s_norm[lane + 64 * u] : 0.f;
  }
  float top = 0.f;
  if (MODE == QIL_SCAN_MLSTM && !fresh) top = *s_top;
  const int half = rot / 2;
  const float fixed = MODE == QIL_SCAN_DECAY ? decay[h] : 0.f;

  // What a lane fetches of a chunk, all requests sent before any is used: elements lane + 64 u of the chunk's
  // [CH][DMAX] queries and keys, its own column of every token's values, and one token's gate inputs.
  float rq[PER], rk[PER], rz[MODE == QIL_SCAN_CHANNEL ? PER : 1], rv[CH], rgi = 0.f, rgk = 0.f;
  auto fetch = [&](int c0) {
    const int cn = min(CH, row1 - c0);
#pragma unroll
    for (int u = 0; u < PER; ++u) {
      const int idx = lane + 64 * u, t = idx / DMAX, i = idx % DMAX;
      const bool live = t < cn && i < dim;
      const T* x = proj + (size_t)(c0 + (live ? t : 0)) * proj_row + h * dim + (live ? i : 0);
      rq[u] = live ? ld(x + q_off) : 0.f;
      rk[u] = live ? ld(x + k_off) : 0.f;
      if (MODE == QIL_SCAN_CHANNEL) rz[u] = live ? gates[(size_t)(c0 + t) * heads * dim + h * dim + i] : 0.f;
    }
#pragma unroll
    for (int t = 0; t < CH; ++t)
      rv[t] = (column && t < cn) ? ld(proj + (size_t)(c0 + t) * proj_row + v_off + h * vdim + j) : 0.f;   // (each group fetches it)
    if (MODE == QIL_SCAN_MLSTM && lane < cn) {
      rgi = gates[(size_t)(c0 + lane) * 2 * heads + h];
      rgk = gates[(size_t)(c0 + lane) * 2 * heads + heads + h];
    }
  };
  fetch(row0);

  for (int c0 = row0; c0 < row1; c0 += CH) {
    const int cn = min(CH, row1 - c0);
    __syncthreads();                                             // the last chunk's reads are done
#pragma unroll
    for (int u = 0; u < PER; ++u) {                              // rows past dim: zeros, so that groups of four are whole
      const int idx = lane + 64 * u, t = idx / DMAX, i = idx % DMAX;
      qs[t][i] = i >= rot ? rq[u] * q_scale : rq[u];             // what is rotated is scaled behind the rotation
      ks[t][i] = i >= rot ? rk[u] * k_scale : rk[u];
      if (MODE == QIL_SCAN_CHANNEL) as[t][i] = expf(log_sigmoid(rz[u]) / cap);
    }
    if (rg == 0) {
#pragma unroll
      for (int t = 0; t < CH; ++t) vs[t][jj] = rv[t];
    }
    if (MODE == QIL_SCAN_MLSTM && lane < cn) {
      gi[lane] = cap * tanhf((rgi + gate_bias[h]) / cap);
      gk[lane] = log_sigmoid(cap * tanhf((rgk + gate_bias[heads + h]) / cap));
    }
    __syncthreads();
    if (c0 + CH < row1) fetch(c0 + CH);                          // on its way while this chunk is walked
    for (int idx = lane; idx < cn * half; idx += 64) {           // a lane turns both elements of a pair, for q and k
      const int t = idx / half, i = idx - t * half;
      float sn, cs;
      sincosf((float)(start + c0 - row0 + t) * freq[i], &sn, &cs);
      const float qu = qs[t][i], qv = qs[t][i + half], ku = ks[t][i], kv = ks[t][i + half];
      qs[t][i] = (qu * cs - qv * sn) * q_scale;
      qs[t][i + half] = (qv * cs + qu * sn) * q_scale;
      ks[t][i] = (ku * cs - kv * sn) * k_scale;
      ks[t][i + half] = (kv * cs + ku * sn) * k_scale;
    }
    if (MODE == QIL_SCAN_MLSTM) {
      if (lane == 0) {                                           // the running maximum: m_t = max(f_t + m_(t-1), i_t)
        float running = top;
        gm[0] = running;
        for (int t = 0; t < cn; ++t) {
          running = fmaxf(gk[t] + running, gi[t]);
          gm[t + 1] = running;
        }
      }
      __syncthreads();
      if (lane < cn) {
        fa[lane] = expf(gk[lane] + gm[lane] - gm[lane + 1]);
        fb[lane] = expf(gi[lane] - gm[lane + 1]);
        fe[lane] = expf(-gm[lane + 1]);
      }
      top = gm[cn];
    }
    __syncthreads();
    if (!keeper) {
      for (int t = 0; t < cn; ++t) {
        const float a = MODE == QIL_SCAN_MLSTM ? fa[t] : fixed, b = MODE == QIL_SCAN_MLSTM ? fb[t] : 1.f;
        const float bv = b * vs[t][jj];
        float o = 0.f;
#pragma unroll
        for (int e = 0; e < DMAX / 4; e += 4) {
          const int i = 4 * e + 4 * rg;                          // rows i .. i + 3 (zeros past dim)
          if (4 * e < dim) {
            const float4 k4 = *reinterpret_cast<const float4*>(&ks[t][i]);
            const float4 q4 = *reinterpret_cast<const float4*>(&qs[t][i]);
            float4 a4 = make_float4(a, a, a, a);
            if (MODE == QIL_SCAN_CHANNEL) a4 = *reinterpret_cast<const float4*>(&as[t][i]);
            col[e] = a4.x * col[e] + k4.x * bv;         o += col[e] * q4.x;
            col[e + 1] = a4.y * col[e + 1] + k4.y * bv; o += col[e + 1] * q4.y;
            col[e + 2] = a4.z * col[e + 2] + k4.z * bv; o += col[e + 2] * q4.z;
            col[e + 3] = a4.w * col[e + 3] + k4.w * bv; o += col[e + 3] * q4.w;
          }
        }
        o += __shfl_xor(o, 16, QIL_WAVE);
        o += __shfl_xor(o, 32, QIL_WAVE);
        if (column && rg == 0) out[(size_t)(c0 + t) * heads * vdim + (size_t)h * vdim + j] = o;
      }
    } else {
      for (int t = 0; t < cn; ++t) {
        float dot = 0.f;
#pragma unroll
        for (int u = 0; u < (DMAX + 63) / 64; ++u) {
          const int i = lane + 64 * u;
          if (i < dim) {
            col[u] = fa[t] * col[u] + fb[t] * ks[t][i];
            dot += col[u] * qs[t][i];
          }
        }
        dot = wave_sum(dot);
        if (lane == 0) below[(size_t)(c0 + t) * heads + h] = fmaxf(fabsf(dot), fe[t]) + 1e-6f;
      }
    }
  }

  if (column) {
#pragma unroll
    for (int e = 0; e < DMAX / 4; ++e) {
      const int i = 16 * (e / 4) + 4 * rg + (e & 3);
      if (i < dim) s_mat[(size_t)i * vdim + j] = col[e];
    }
  }
  if (keeper) {
#pragma unroll
    for (int u = 0; u < (DMAX + 63) / 64; ++u)
      if (lane + 64 * u < dim) s_norm[lane + 64 * u] = col[u];
  }
  if (MODE == QIL_SCAN_MLSTM && lane == 0) *s_top = top;
}

// o' = o[n, h, :] / below[n, h] (below optional);  y[n, h, j] = o'[j] / sqrt(mean_j(o'^2) + eps) * weight[h, j] * act(g[n, h, j]),
// weight optional; act: 0 sigmoid(g), 1 g * sigmoid(g).  One block per (row, head).
template <typename T>
__global__ void head_norm_gate_kernel(const float* __restrict__ o, const float* __restrict__ below, const T* __restrict__ g, int g_row, int g_off,
                                      const float* __restrict__ weight, T* __restrict__ y, int heads, int vdim, float eps,
                                      int act) {
  __shared__ float scratch[16];
  const int n = blockIdx.x, h = blockIdx.y;
  const float* src = o + ((size_t)n * heads + h) * vdim;
  const float divide = below ? below[(size_t)n * heads + h] : 1.f;
  float squares = 0.f;
  for (int j = threadIdx.x; j < vdim; j += blockDim.x) {
    const float v = src[j] / divide;
    squares += v * v;
  }
  squares = block_sum(squares, scratch);
  const float unit = 1.f / sqrtf(squares / (float)vdim + eps);
  for (int j = threadIdx.x; j < vdim; j += blockDim.x) {
    const float gate = ld(g + (size_t)n * g_row + g_off + h * vdim + j);
    const float sig = 1.f / (1.f + expf(-gate));
    float value = src[j] / divide * unit;
    if (weight) value *= weight[h * vdim + j];
    st(y + ((size_t)n * heads + h) * vdim + j, value * (act ? gate * sig : sig));
  }
}

extern "C" {

// Floats of one state slot.
size_t qil_state_scan_slot(int heads, int dim, int vdim, int mode) {
  const size_t tiles = (size_t)(vdim + SCAN_COLUMNS - 1) / SCAN_COLUMNS;
  return (size_t)heads * dim * vdim + (mode == QIL_SCAN_MLSTM ? (size_t)heads * dim + heads * (tiles + 1) : 0);
}

int qil_state_scan_takes(int dim, int vdim, int rot) {
  return dim >= 1 && dim <= 256 && vdim >= 1 && rot >= 0 && rot % 2 == 0 && rot <= dim;
}

// proj [n, proj_row] (dtype): a row holds the heads' queries from q_off, keys from k_off (heads x dim each) and
// values from v_off (heads x vdim).  gates [n, 2 heads] float32 (inputs first, then keeps), gate_bias [2 heads]: MLSTM.
// CHANNEL: gates [n, heads * dim] float32 (z, one per row of every head's state) and cap = tau.
// decay [heads]: DECAY.  freq [rot / 2] or rot == 0.  out [n, heads * vdim] float32; MLSTM: undivided, with every
// token's denominator in below [n, heads].
int qil_state_scan(const void* proj, int dtype, int proj_row, int q_off, int k_off, int v_off, const float* gates,
                   const float* gate_bias, float cap, const float* decay, const float* freq, int rot, float q_scale,
                   float k_scale, float* state, const int* cu_seqlens, const int* seq_starts, const int* seq_slots,
                   float* out, float* below, int n_seqs, int heads, int dim, int vdim, int mode, hipStream_t s) {
  if (n_seqs == 0) return 0;
  if (!qil_state_scan_takes(dim, vdim, rot) || mode < QIL_SCAN_DECAY || mode > QIL_SCAN_CHANNEL) return -1;
  if ((mode == QIL_SCAN_MLSTM && (!gates || !gate_bias || !below)) || (mode == QIL_SCAN_DECAY && !decay) ||
      (mode == QIL_SCAN_CHANNEL && (!gates || !(cap > 0.f))) || (rot && !freq)) return -1;
  const size_t slot_stride = qil_state_scan_slot(heads, dim, vdim, mode);
  dim3 grid(n_seqs, heads, (vdim + SCAN_COLUMNS - 1) / SCAN_COLUMNS + (mode == QIL_SCAN_MLSTM ? 1 : 0));
#define QIL_SCAN(T, DMAX, MODE)                                                                                      \
  hipLaunchKernelGGL((state_scan_kernel<T, DMAX, MODE>), grid, dim3(64), 0, s, (const T*)proj, proj_row, q_off, k_off, \
                     v_off, gates, gate_bias, cap, decay, freq, rot, q_scale, k_scale, state, slot_stride, cu_seqlens, \
                     seq_starts, seq_slots, out, below, heads, dim, vdim)
#define QIL_SCAN_DIM(T, MODE)                                                                                        \
  do {                                                                                                               \
    if (dim <= 32) QIL_SCAN(T, 32, MODE);                                                                            \
    else if (dim <= 64) QIL_SCAN(T, 64, MODE);                                                                       \
    else if (dim <= 128) QIL_SCAN(T, 128, MODE);                                                                     \
    else QIL_SCAN(T, 256, MODE);                                                                                     \
  } while (0)
  if (dtype == QIL_F32) {
    if (mode == QIL_SCAN_MLSTM) QIL_SCAN_DIM(float, QIL_SCAN_MLSTM);
    else if (mode == QIL_SCAN_CHANNEL) QIL_SCAN_DIM(float, QIL_SCAN_CHANNEL);
    else QIL_SCAN_DIM(float, QIL_SCAN_DECAY);
  } else {
    if (mode == QIL_SCAN_MLSTM) QIL_SCAN_DIM(bf16_t, QIL_SCAN_MLSTM);
    else if (mode == QIL_SCAN_CHANNEL) QIL_SCAN_DIM(bf16_t, QIL_SCAN_CHANNEL);
    else QIL_SCAN_DIM(bf16_t, QIL_SCAN_DECAY);
  }
#undef QIL_SCAN_DIM
#undef QIL_SCAN
  QIL_RETURN_LAUNCH_STATUS();
}

int qil_head_norm_gate(const float* o, const float* below, const void* g, int g_row, int g_off, const float* weight, void* y, int n, int heads,
                       int vdim, float eps, int act, int dtype, hipStream_t s) {
  if (n == 0 || heads == 0) return 0;
  if (vdim < 1) return -1;
  const int threads = vdim >= 256 ? 256 : (vdim + 63) / 64 * 64;
  if (dtype == QIL_F32)
    hipLaunchKernelGGL(head_norm_gate_kernel<float>, dim3(n, heads), dim3(threads), 0, s, o, below, (const float*)g, g_row, g_off,
                       weight, (float*)y, heads, vdim, eps, act);
  else
    hipLaunchKernelGGL(head_norm_gate_kernel<bf16_t>, dim3(n, heads), dim3(threads), 0, s, o, below, (const bf16_t*)g, g_row, g_off,
                       weight, (bf16_t*)y, heads, vdim, eps, act);
  QIL_RETURN_LAUNCH_STATUS();
}

}  // extern "C"
