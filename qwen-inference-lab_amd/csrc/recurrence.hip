// Linear recurrences with a matrix state per head, carried from token to token in float32:
//     S_t = a_t S_(t-1) + b_t k_t v_t^T          S [dim, vdim]
//     o_t = S_t^T q_t
// by gating mode:
//   QIL_SCAN_DECAY  a_t = decay_h (fixed per head), b_t = 1; o_t as above.
//   QIL_SCAN_MLSTM  log gates i_t = cap tanh((x_i + bias_i) / cap), f_t = logsigmoid(cap tanh((x_f + bias_f) / cap)),
//                   running maximum m_t = max(f_t + m_(t-1), i_t) with m = 0 before the first token,
//                   a_t = exp(f_t + m_(t-1) - m_t), b_t = exp(i_t - m_t); a normaliser n_t = a_t n_(t-1) + b_t k_t;
//                   o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6).
// Queries and keys may be rotated by position first (the leading rot elements of a head, element i with i + rot / 2,
// angle position * freq[i]) and are then scaled (q_scale, k_scale).  Gates, rotation, state and sums are float32.
//
// A block is one wave: one (sequence, head, 64 columns of the state).  A lane keeps its column of S in registers and
// walks the sequence's tokens of this step in order; q and k of a token pass through LDS.  The state slot of a sequence
// is read unless the sequence starts at position 0, and written back at the end.
#include "common.h"

enum { QIL_SCAN_DECAY = 0, QIL_SCAN_MLSTM = 1 };

__device__ __forceinline__ float log_sigmoid(float z) {         // -softplus(-z), stable on both sides
  return fminf(z, 0.f) - log1pf(expf(-fabsf(z)));
}

// State of one slot: [heads][dim * vdim] matrices, then (MLSTM) [heads][tiles][dim] normalisers and [heads][tiles]
// maxima, tiles = ceil(vdim / 64): a block reads and writes only its own copy, so no block sees another's update.
template <typename T, int DMAX, int MODE>
__global__ void __launch_bounds__(64)
state_scan_kernel(const T* __restrict__ proj, int proj_row, int q_off, int k_off, int v_off,
                  const float* __restrict__ gates, const float* __restrict__ gate_bias, float cap,
                  const float* __restrict__ decay, const float* __restrict__ freq, int rot, float q_scale, float k_scale,
                  float* __restrict__ state, size_t slot_stride, const int* __restrict__ cu_seqlens,
                  const int* __restrict__ seq_starts, const int* __restrict__ seq_slots, float* __restrict__ out,
                  int heads, int dim, int vdim) {
  __shared__ float qs[DMAX], ks[DMAX], ns[DMAX];
  const int seq = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int j = blockIdx.z * 64 + lane;
  const bool column = j < vdim;
  const int row0 = cu_seqlens[seq], row1 = cu_seqlens[seq + 1], start = seq_starts[seq];
  float* slot = state + (size_t)seq_slots[seq] * slot_stride;
  float* s_mat = slot + (size_t)h * dim * vdim;
  const int tiles = gridDim.z;                                  // every tile of columns keeps a copy of its own
  float* s_norm = slot + (size_t)heads * dim * vdim + ((size_t)h * tiles + blockIdx.z) * dim;
  float* s_top = slot + (size_t)heads * dim * vdim + (size_t)heads * tiles * dim + (size_t)h * tiles + blockIdx.z;
  const bool fresh = start == 0;

  float col[DMAX];
#pragma unroll
  for (int i = 0; i < DMAX; ++i) col[i] = (!fresh && column && i < dim) ? s_mat[(size_t)i * vdim + j] : 0.f;
  float top = 0.f;
  if (MODE == QIL_SCAN_MLSTM) {
    for (int i = lane; i < dim; i += 64) ns[i] = fresh ? 0.f : s_norm[i];
    if (!fresh) top = *s_top;
  }
  const int half = rot / 2;
  const float fixed = MODE == QIL_SCAN_DECAY ? decay[h] : 0.f;

  for (int row = row0; row < row1; ++row) {
    const T* x = proj + (size_t)row * proj_row;
    const float p = (float)(start + row - row0);
    __syncthreads();                                             // the last token's reads of qs / ks are done
    for (int i = lane; i < dim; i += 64) {
      float qv, kv;
      if (i < half || i >= rot) {
        qv = ld(x + q_off + h * dim + i);
        kv = ld(x + k_off + h * dim + i);
        if (i < half) {                                          // this lane makes both elements of the pair
          const float q2 = ld(x + q_off + h * dim + i + half), k2 = ld(x + k_off + h * dim + i + half);
          float sn, cs;
          sincosf(p * freq[i], &sn, &cs);
          qs[i + half] = (q2 * cs + qv * sn) * q_scale;
          ks[i + half] = (k2 * cs + kv * sn) * k_scale;
          qv = qv * cs - q2 * sn;
          kv = kv * cs - k2 * sn;
        }
        qs[i] = qv * q_scale;
        ks[i] = kv * k_scale;
      }
    }
    float a = fixed, b = 1.f;
    if (MODE == QIL_SCAN_MLSTM) {
      const float xi = gates[(size_t)row * 2 * heads + h] + gate_bias[h];
      const float xf = gates[(size_t)row * 2 * heads + heads + h] + gate_bias[heads + h];
      const float log_in = cap * tanhf(xi / cap);
      const float log_keep = log_sigmoid(cap * tanhf(xf / cap));
      const float now = fmaxf(log_keep + top, log_in);
      a = expf(log_keep + top - now);
      b = expf(log_in - now);
      top = now;
    }
    __syncthreads();
    const float v = column ? ld(x + v_off + h * vdim + j) : 0.f;
    float o = 0.f;
#pragma unroll
    for (int i = 0; i < DMAX; ++i) {
      if (i < dim) {
        col[i] = a * col[i] + (b * ks[i]) * v;
        o += col[i] * qs[i];
      }
    }
    if (MODE == QIL_SCAN_MLSTM) {
      float dot = 0.f;
      for (int i = lane; i < dim; i += 64) {
        const float nv = a * ns[i] + b * ks[i];
        ns[i] = nv;
        dot += nv * qs[i];
      }
      dot = wave_sum(dot);
      o = o / (fmaxf(fabsf(dot), expf(-top)) + 1e-6f);
    }
    if (column) out[(size_t)row * heads * vdim + (size_t)h * vdim + j] = o;
  }

  if (column) {
#pragma unroll
    for (int i = 0; i < DMAX; ++i)
      if (i < dim) s_mat[(size_t)i * vdim + j] = col[i];
  }
  if (MODE == QIL_SCAN_MLSTM) {
    __syncthreads();
    for (int i = lane; i < dim; i += 64) s_norm[i] = ns[i];
    if (lane == 0) *s_top = top;
  }
}

// y[n, h, j] = o[n, h, j] / sqrt(mean_j(o[n, h, :]^2) + eps) * weight[h, j] * act(g[n, h, j]),
// weight optional; act: 0 sigmoid(g), 1 g * sigmoid(g).  One block per (row, head).
template <typename T>
__global__ void head_norm_gate_kernel(const float* __restrict__ o, const T* __restrict__ g, int g_row, int g_off,
                                      const float* __restrict__ weight, T* __restrict__ y, int heads, int vdim, float eps,
                                      int act) {
  __shared__ float scratch[16];
  const int n = blockIdx.x, h = blockIdx.y;
  const float* src = o + ((size_t)n * heads + h) * vdim;
  float squares = 0.f;
  for (int j = threadIdx.x; j < vdim; j += blockDim.x) squares += src[j] * src[j];
  squares = block_sum(squares, scratch);
  const float unit = 1.f / sqrtf(squares / (float)vdim + eps);
  for (int j = threadIdx.x; j < vdim; j += blockDim.x) {
    const float gate = ld(g + (size_t)n * g_row + g_off + h * vdim + j);
    const float sig = 1.f / (1.f + expf(-gate));
    float value = src[j] * unit;
    if (weight) value *= weight[h * vdim + j];
    st(y + ((size_t)n * heads + h) * vdim + j, value * (act ? gate * sig : sig));
  }
}

extern "C" {

// Floats of one state slot.
size_t qil_state_scan_slot(int heads, int dim, int vdim, int mode) {
  const size_t tiles = (size_t)(vdim + 63) / 64;
  return (size_t)heads * dim * vdim + (mode == QIL_SCAN_MLSTM ? heads * tiles * dim + heads * tiles : 0);
}

int qil_state_scan_takes(int dim, int vdim, int rot) {
  return dim >= 1 && dim <= 256 && vdim >= 1 && rot >= 0 && rot % 2 == 0 && rot <= dim;
}

// proj [n, proj_row] (dtype): a row holds the heads' queries from q_off, keys from k_off (heads x dim each) and
// values from v_off (heads x vdim).  gates [n, 2 heads] float32 (inputs first, then keeps), gate_bias [2 heads]: MLSTM.
// decay [heads]: DECAY.  freq [rot / 2] or rot == 0.  out [n, heads * vdim] float32.
int qil_state_scan(const void* proj, int dtype, int proj_row, int q_off, int k_off, int v_off, const float* gates,
                   const float* gate_bias, float cap, const float* decay, const float* freq, int rot, float q_scale,
                   float k_scale, float* state, const int* cu_seqlens, const int* seq_starts, const int* seq_slots,
                   float* out, int n_seqs, int heads, int dim, int vdim, int mode, hipStream_t s) {
  if (n_seqs == 0) return 0;
  if (!qil_state_scan_takes(dim, vdim, rot) || (mode != QIL_SCAN_DECAY && mode != QIL_SCAN_MLSTM)) return -1;
  if ((mode == QIL_SCAN_MLSTM && (!gates || !gate_bias)) || (mode == QIL_SCAN_DECAY && !decay) || (rot && !freq)) return -1;
  const size_t slot_stride = qil_state_scan_slot(heads, dim, vdim, mode);
  dim3 grid(n_seqs, heads, (vdim + 63) / 64);
#define QIL_SCAN(T, DMAX, MODE)                                                                                      \
  hipLaunchKernelGGL((state_scan_kernel<T, DMAX, MODE>), grid, dim3(64), 0, s, (const T*)proj, proj_row, q_off, k_off, \
                     v_off, gates, gate_bias, cap, decay, freq, rot, q_scale, k_scale, state, slot_stride, cu_seqlens, \
                     seq_starts, seq_slots, out, heads, dim, vdim)
#define QIL_SCAN_DIM(T, MODE)                                                                                        \
  do {                                                                                                               \
    if (dim <= 32) QIL_SCAN(T, 32, MODE);                                                                            \
    else if (dim <= 64) QIL_SCAN(T, 64, MODE);                                                                       \
    else if (dim <= 128) QIL_SCAN(T, 128, MODE);                                                                     \
    else QIL_SCAN(T, 256, MODE);                                                                                     \
  } while (0)
  if (dtype == QIL_F32) {
    if (mode == QIL_SCAN_MLSTM) QIL_SCAN_DIM(float, QIL_SCAN_MLSTM); else QIL_SCAN_DIM(float, QIL_SCAN_DECAY);
  } else {
    if (mode == QIL_SCAN_MLSTM) QIL_SCAN_DIM(bf16_t, QIL_SCAN_MLSTM); else QIL_SCAN_DIM(bf16_t, QIL_SCAN_DECAY);
  }
#undef QIL_SCAN_DIM
#undef QIL_SCAN
  QIL_RETURN_LAUNCH_STATUS();
}

int qil_head_norm_gate(const float* o, const void* g, int g_row, int g_off, const float* weight, void* y, int n, int heads,
                       int vdim, float eps, int act, int dtype, hipStream_t s) {
  if (n == 0 || heads == 0) return 0;
  if (vdim < 1) return -1;
  const int threads = vdim >= 256 ? 256 : (vdim + 63) / 64 * 64;
  if (dtype == QIL_F32)
    hipLaunchKernelGGL(head_norm_gate_kernel<float>, dim3(n, heads), dim3(threads), 0, s, o, (const float*)g, g_row, g_off,
                       weight, (float*)y, heads, vdim, eps, act);
  else
    hipLaunchKernelGGL(head_norm_gate_kernel<bf16_t>, dim3(n, heads), dim3(threads), 0, s, o, (const bf16_t*)g, g_row, g_off,
                       weight, (bf16_t*)y, heads, vdim, eps, act);
  QIL_RETURN_LAUNCH_STATUS();
}

}  // extern "C"
