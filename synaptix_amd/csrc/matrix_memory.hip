// A matrix memory with exponential gates and a running maximum (the mLSTM cell), one state for each sequence and head:
//
//   i_t = cap tanh((i~ + b_i) / cap)                      log input gate   (cap <= 0: no cap)
//   f_t = logsigmoid(cap tanh((f~ + b_f) / cap))          log forget gate
//   m_t = max(f_t + m_(t-1), i_t)                         m_0 = 0
//   S_t = exp(f_t + m_(t-1) - m_t) S_(t-1) + exp(i_t - m_t) k_t v_t^T         S [dim][vdim], S_0 = 0
//   n_t = exp(f_t + m_(t-1) - m_t) n_(t-1) + exp(i_t - m_t) k_t               n [dim],       n_0 = 0
//   o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6),                   q_t = q~_t * q_scale
//
// All of it in 32-bit.  The state of a (slot, head) is dim * vdim + dim + 1 floats: S by rows, n, m.
// proj [N][width] float is the fused projection [q: H x dim | k: H x dim | v: H x vdim | gate: H x vdim | i~: H | f~: H].
#include "common.h"

#define MM_TC 16        // tokens whose q, k and gates are staged in LDS together
#define MM_VT 64        // columns of S a workgroup keeps (one a lane)
#define MM_DG 4         // waves of a workgroup; wave w keeps the rows d = w, w + 4, ... of its columns
#define MM_MAX_DIM 256

__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

// One workgroup for each (sequence of the step, head, tile of 64 columns); it walks the sequence's new tokens in order
// with its part of S in registers.  Tile 0 also keeps n and m for the state (every tile computes them).
template <int DPT>   // rows of S a thread keeps: dim <= 4 * DPT
__global__ void __launch_bounds__(MM_DG * SYN_WAVE)
matrix_memory_scan_kernel(const float* __restrict__ proj, int width, const float* __restrict__ i_bias,
                          const float* __restrict__ f_bias, float cap, float q_scale, float* __restrict__ state,
                          int spare_row, const int* __restrict__ seq_start, const int* __restrict__ seq_slot,
                          float* __restrict__ out, int H, int dim, int vdim) {
  __shared__ float qs[MM_TC][MM_MAX_DIM];
  __shared__ float ks[MM_TC][MM_MAX_DIM];
  __shared__ float gs[MM_TC][2];
  __shared__ float red[2][MM_DG][MM_VT];
  __shared__ float red_n[2][MM_DG];
  const int b = blockIdx.x, h = blockIdx.y, vt = blockIdx.z;
  const int wave = threadIdx.x / SYN_WAVE, lane = threadIdx.x % SYN_WAVE;
  const int v = vt * MM_VT + lane;
  const bool v_ok = v < vdim;
  const int t0 = seq_start[b], t1 = seq_start[b + 1];
  if (t0 >= t1) return;     // a sequence without tokens in this step (the spare ones of a padded step): nothing moves
  const int slot = seq_slot[b];
  const size_t per_head = (size_t)dim * vdim + dim + 1;
  float* st = state + ((size_t)(slot < 0 ? spare_row : slot) * H + h) * per_head;
  const int q_col = h * dim, k_col = H * dim + h * dim, v_col = 2 * H * dim + h * vdim;
  const int i_col = 2 * H * dim + 2 * H * vdim + h, f_col = i_col + H;
  const float bi = i_bias ? i_bias[h] : 0.f, bf = f_bias ? f_bias[h] : 0.f;

  float S[DPT];
#pragma unroll
  for (int j = 0; j < DPT; ++j) {
    const int d = wave + MM_DG * j;
    S[j] = (d < dim && v_ok) ? st[(size_t)d * vdim + v] : 0.f;
  }
  const int dn = wave + MM_DG * lane;          // the entry of n this thread keeps
  float n = dn < dim ? st[(size_t)dim * vdim + dn] : 0.f;
  float m = st[(size_t)dim * vdim + dim];

  for (int c0 = t0; c0 < t1; c0 += MM_TC) {
    const int nc = min(MM_TC, t1 - c0);
    __syncthreads();
    for (int idx = threadIdx.x; idx < nc * dim; idx += blockDim.x) {
      const int t = idx / dim, d = idx % dim;
      const float* row = proj + (size_t)(c0 + t) * width;
      qs[t][d] = row[q_col + d] * q_scale;
      ks[t][d] = row[k_col + d];
    }
    if (threadIdx.x < nc * 2) {
      const int t = threadIdx.x / 2, which = threadIdx.x % 2;
      const float raw = proj[(size_t)(c0 + t) * width + (which ? f_col : i_col)] + (which ? bf : bi);
      const float capped = cap > 0.f ? cap * tanhf(raw / cap) : raw;
      gs[t][which] = which ? log_sigmoid(capped) : capped;
    }
    float vv[MM_TC];
#pragma unroll
    for (int t = 0; t < MM_TC; ++t) vv[t] = (t < nc && v_ok) ? proj[(size_t)(c0 + t) * width + v_col + v] : 0.f;
    __syncthreads();
#pragma unroll
    for (int t = 0; t < MM_TC; ++t) {
      if (t < nc) {
        const float ig = gs[t][0], fg = gs[t][1];
        const float m_new = fmaxf(fg + m, ig);
        const float a = expf(fg + m - m_new), bb = expf(ig - m_new);
        m = m_new;
        float num = 0.f;
#pragma unroll
        for (int j = 0; j < DPT; ++j) {
          const int d = wave + MM_DG * j;
          if (d < dim) {
            S[j] = a * S[j] + (bb * ks[t][d]) * vv[t];
            num = fmaf(S[j], qs[t][d], num);
          }
        }
        float nq = 0.f;
        if (dn < dim) {
          n = a * n + bb * ks[t][dn];
          nq = n * qs[t][dn];
        }
        nq = wave_sum(nq);
        const int buf = t & 1;
        red[buf][wave][lane] = num;
        if (lane == 0) red_n[buf][wave] = nq;
        __syncthreads();
        if (wave == 0 && v_ok) {
          float total = 0.f, nqt = 0.f;
#pragma unroll
          for (int w = 0; w < MM_DG; ++w) total += red[buf][w][lane], nqt += red_n[buf][w];
          const float den = fmaxf(fabsf(nqt), expf(-m)) + 1e-6f;
          out[(size_t)(c0 + t) * H * vdim + (size_t)h * vdim + v] = total / den;
        }
      }
    }
  }
#pragma unroll
  for (int j = 0; j < DPT; ++j) {
    const int d = wave + MM_DG * j;
    if (d < dim && v_ok) st[(size_t)d * vdim + v] = S[j];
  }
  if (vt == 0) {
    if (dn < dim) st[(size_t)dim * vdim + dn] = n;
    if (threadIdx.x == 0) st[(size_t)dim * vdim + dim] = m;
  }
}

// out [N][H * vdim] float: o_t of every token, before the heads' norm
SYN_EXPORT int syn_matrix_memory_scan(const float* proj, int width, const float* i_bias, const float* f_bias, float cap,
                                      float q_scale, float* state, int state_rows, const int* seq_start,
                                      const int* seq_slot, int n_seqs, float* out, int H, int dim, int vdim,
                                      hipStream_t stream) {
  SYN_CHECK(n_seqs > 0 && H > 0, "matrix_memory_scan: empty input");
  SYN_CHECK(dim > 0 && dim <= MM_MAX_DIM && vdim > 0, "matrix_memory_scan: sizes %d x %d (keys up to %d)", dim, vdim,
            MM_MAX_DIM);
  SYN_CHECK(width >= 2 * H * dim + 2 * H * vdim + 2 * H, "matrix_memory_scan: rows of %d values do not hold q, k, v, "
            "the gate and the two gates of the cell", width);
  SYN_CHECK(state_rows >= 1, "matrix_memory_scan: no state rows");
  const dim3 grid(n_seqs, H, (vdim + MM_VT - 1) / MM_VT);
  const int dpt = (dim + MM_DG - 1) / MM_DG;
#define SYN_MM(D)                                                                                                   \
  matrix_memory_scan_kernel<D><<<grid, MM_DG * SYN_WAVE, 0, stream>>>(proj, width, i_bias, f_bias, cap, q_scale, state, \
                                                                      state_rows - 1, seq_start, seq_slot, out, H, dim, vdim)
  if (dpt <= 8) SYN_MM(8);
  else if (dpt <= 16) SYN_MM(16);
  else if (dpt <= 32) SYN_MM(32);
  else SYN_MM(64);
#undef SYN_MM
  SYN_LAUNCH_CHECK("matrix_memory_scan");
  return 0;
}

// Each head's o divided by its root mean square, times a gain over all heads' values, times sigmoid(gate):
// one wave for each (token, head).  gate: float rows of gate_stride values (the fused projection from its gate on).
template <typename TOut>
__global__ void head_norm_gate_kernel(const float* __restrict__ o, const float* __restrict__ gain, float eps,
                                      const float* __restrict__ gate, int gate_stride, TOut* __restrict__ out,
                                      int n_items, int H, int vdim) {
  const int item = blockIdx.x * (blockDim.x / SYN_WAVE) + threadIdx.x / SYN_WAVE;
  if (item >= n_items) return;
  const int lane = threadIdx.x % SYN_WAVE;
  const int tok = item / H, h = item % H;
  const float* x = o + ((size_t)tok * H + h) * vdim;
  float ss = 0.f;
  for (int d = lane; d < vdim; d += SYN_WAVE) ss += x[d] * x[d];
  const float inv = 1.f / sqrtf(wave_sum(ss) / (float)vdim + eps);
  const float* g = gate ? gate + (size_t)tok * gate_stride + (size_t)h * vdim : nullptr;
  for (int d = lane; d < vdim; d += SYN_WAVE) {
    float v = x[d] * inv;
    if (gain) v *= gain[h * vdim + d];
    if (g) v *= 1.f / (1.f + expf(-g[d]));
    out[((size_t)tok * H + h) * vdim + d] = from_f32<TOut>(v);
  }
}

SYN_EXPORT int syn_head_norm_gate(const float* o, const float* gain, float eps, const float* gate, int gate_stride,
                                  void* out, int out_is_f32, int n_tokens, int H, int vdim, hipStream_t stream) {
  SYN_CHECK(n_tokens > 0 && H > 0 && vdim > 0, "head_norm_gate: empty input");
  SYN_CHECK(gate == nullptr || gate_stride >= H * vdim, "head_norm_gate: gate rows of %d values", gate_stride);
  const int wpb = 4, items = n_tokens * H;
  const int grid = (items + wpb - 1) / wpb;
  if (out_is_f32)
    head_norm_gate_kernel<float><<<grid, wpb * SYN_WAVE, 0, stream>>>(o, gain, eps, gate, gate_stride, (float*)out, items,
                                                                      H, vdim);
  else
    head_norm_gate_kernel<bf16><<<grid, wpb * SYN_WAVE, 0, stream>>>(o, gain, eps, gate, gate_stride, (bf16*)out, items,
                                                                     H, vdim);
  SYN_LAUNCH_CHECK("head_norm_gate");
  return 0;
}
