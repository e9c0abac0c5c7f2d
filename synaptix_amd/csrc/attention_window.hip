// Attention over the paged cache for mixers whose scores, mask and softmax differ from the plain causal ones:
//
//   score(i, j) = scale (q_i . k_j) [soft cap] - slope_h (i - j) - r1_h ln(1 + r2_h (i - j))
//   key j is visible to the query at i iff  j <= i  and  (window <= 0 or i - j < window or j < keep_first):
//       a sliding window that never loses the first keep_first keys, which keep their true positions;
//   p_j = exp(score_j) / (sink + sum_j exp(score_j)),  sink = 1 with `sink_one` (a further key of score 0 that has
//       no value), else 0;
//   head h reads kv head h / (heads / kv heads); keys have `dim` values, values `vdim`;
//   the heads' results may be multiplied by sigmoid(gate) before they are stored.
// Scores, weights and sums are 32-bit whatever the cache's type; the weights are not rounded before they meet V.
//
// Cache pages hold 64 tokens: k_pages[page, kv_head, token, dim], v_pages[page, kv_head, vdim, token] (plain rows in
// both types).  One wave for each (token, head), plain FMA, online softmax over blocks of 64 keys: prompts and single
// tokens alike.
#include "common.h"

#define AW_MAX_DIM 256

struct WindowTerms {
  const float* slopes;   // [heads] or nullptr
  const float* r1;       // [heads] or nullptr (with r2)
  const float* r2;
  float softcap;         // 0: none
  int window;            // 0: every key
  int keep_first;
  int sink_one;
};

// ---------------------------------------------------------------- intake: bias, q/k norm, cache write
// proj [N][width] float holds the fused projection  [q heads x dim | k heads x dim | v heads x vdim | ...]; what lies
// behind v (a gate) is left where it is.  One wave for each (token, q head | k head | v head).
template <typename T>
__global__ void window_intake_kernel(const float* __restrict__ proj, int width, const float* __restrict__ bias,
                                     T* __restrict__ q_out, T* __restrict__ k_pages, T* __restrict__ v_pages,
                                     const int* __restrict__ page_table, int table_stride,
                                     const int* __restrict__ tok_seq, const int* __restrict__ tok_pos,
                                     const float* __restrict__ q_gain, const float* __restrict__ k_gain, float eps,
                                     int nh, int nkv, int dim, int vdim, int write_kv) {
  const int wave = threadIdx.x / SYN_WAVE, lane = threadIdx.x % SYN_WAVE;
  const int tok = blockIdx.x;
  const int item = blockIdx.y * (blockDim.x / SYN_WAVE) + wave;
  if (item >= (write_kv ? nh + 2 * nkv : nh)) return;
  const bool is_q = item < nh, is_k = !is_q && item < nh + nkv;
  const int len = (is_q || is_k) ? dim : vdim;
  const int col = is_q ? item * dim : (is_k ? nh * dim + (item - nh) * dim : (nh + nkv) * dim + (item - nh - nkv) * vdim);
  const float* src = proj + (size_t)tok * width + col;
  const float* b = bias ? bias + col : nullptr;
  const float* gain = is_q ? q_gain : (is_k ? k_gain : nullptr);
  float inv = 1.f;
  if (gain) {
    float ss = 0.f;
    for (int d = lane; d < len; d += SYN_WAVE) {
      const float v = src[d] + (b ? b[d] : 0.f);
      ss += v * v;
    }
    inv = 1.f / sqrtf(wave_sum(ss) / (float)len + eps);
  }
  const int pos = tok_pos[tok];
  T* dst;
  size_t stride = 1;
  if (is_q) {
    dst = q_out + ((size_t)tok * nh + item) * dim;
  } else {
    const int page = page_table[(size_t)tok_seq[tok] * table_stride + pos / SYN_PAGE];
    if (is_k) {
      dst = k_pages + (((size_t)page * nkv + (item - nh)) * SYN_PAGE + pos % SYN_PAGE) * dim;
    } else {
      dst = v_pages + ((size_t)page * nkv + (item - nh - nkv)) * vdim * SYN_PAGE + pos % SYN_PAGE;
      stride = SYN_PAGE;
    }
  }
  for (int d = lane; d < len; d += SYN_WAVE) {
    float v = src[d] + (b ? b[d] : 0.f);
    if (gain) v = v * inv * gain[d];
    dst[(size_t)d * stride] = from_f32<T>(v);
  }
}

SYN_EXPORT int syn_window_intake(const float* proj, int width, const float* bias, void* q_out, void* k_pages,
                                 void* v_pages, int is_f32, const int* page_table, int table_stride, const int* tok_seq,
                                 const int* tok_pos, const float* q_gain, const float* k_gain, float eps, int n_tokens,
                                 int nh, int nkv, int dim, int vdim, int write_kv, hipStream_t stream) {
  SYN_CHECK(n_tokens > 0 && nh > 0 && nkv > 0 && dim > 0 && vdim > 0, "window_intake: empty input");
  SYN_CHECK(width >= (nh + nkv) * dim + nkv * vdim, "window_intake: rows of %d values do not hold q, k and v", width);
  SYN_CHECK((q_gain == nullptr) == (k_gain == nullptr), "window_intake: q and k gains come together");
  const int wpb = 4, items = write_kv ? nh + 2 * nkv : nh;
  const dim3 grid(n_tokens, (items + wpb - 1) / wpb);
  if (is_f32)
    window_intake_kernel<float><<<grid, wpb * SYN_WAVE, 0, stream>>>(proj, width, bias, (float*)q_out, (float*)k_pages,
                                                                     (float*)v_pages, page_table, table_stride, tok_seq,
                                                                     tok_pos, q_gain, k_gain, eps, nh, nkv, dim, vdim,
                                                                     write_kv);
  else
    window_intake_kernel<bf16><<<grid, wpb * SYN_WAVE, 0, stream>>>(proj, width, bias, (bf16*)q_out, (bf16*)k_pages,
                                                                    (bf16*)v_pages, page_table, table_stride, tok_seq,
                                                                    tok_pos, q_gain, k_gain, eps, nh, nkv, dim, vdim,
                                                                    write_kv);
  SYN_LAUNCH_CHECK("window_intake");
  return 0;
}

// ---------------------------------------------------------------- attention, one wave a (token, head)
__device__ __forceinline__ float window_score(float dot, float scale, const WindowTerms& t, float slope, float r1,
                                              float r2, int pos, int key) {
  float s = dot * scale;
  if (t.softcap > 0.f) s = t.softcap * tanhf(s / t.softcap);
  const float dist = (float)(pos - key);
  s -= slope * dist;
  if (t.r1) s -= r1 * logf(1.f + r2 * dist);
  return s;
}

template <typename T>
__global__ void __launch_bounds__(SYN_WAVE)
window_attention_kernel(const T* __restrict__ q, const T* __restrict__ k_pages, const T* __restrict__ v_pages,
                        const int* __restrict__ page_table, int table_stride, const int* __restrict__ tok_seq,
                        const int* __restrict__ tok_pos, const float* __restrict__ gate, int gate_stride,
                        const float* __restrict__ gate_bias, T* __restrict__ out, float scale, int nh, int nkv, int dim,
                        int vdim, WindowTerms terms) {
  __shared__ float qs[AW_MAX_DIM];
  __shared__ float ps[SYN_PAGE];
  const int tok = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  const int seq = tok_seq[tok], pos = tok_pos[tok];
  const int kvh = head / (nh / nkv);
  const T* qr = q + ((size_t)tok * nh + head) * dim;
  for (int d = lane; d < dim; d += SYN_WAVE) qs[d] = to_f32<T>(qr[d]);
  __syncthreads();

  const int lo = terms.window > 0 ? max(0, pos - terms.window + 1) : 0;
  const int kept = min(terms.keep_first, lo);        // keys below `kept` are seen although the window has passed them
  const int last_kept_block = kept > 0 ? (kept - 1) / SYN_PAGE : -1;
  const int first_window_block = max(lo / SYN_PAGE, last_kept_block + 1);
  const int last_block = pos / SYN_PAGE;
  const float slope = terms.slopes ? terms.slopes[head] : 0.f;
  const float r1 = terms.r1 ? terms.r1[head] : 0.f, r2 = terms.r1 ? terms.r2[head] : 0.f;
  // the sink is a key of score 0 without a value: the running maximum and sum start from it
  float m = terms.sink_one ? 0.f : -INFINITY, l = terms.sink_one ? 1.f : 0.f;
  float o[AW_MAX_DIM / SYN_WAVE] = {0.f, 0.f, 0.f, 0.f};
  for (int kb = last_kept_block >= 0 ? 0 : first_window_block; kb <= last_block; ++kb) {
    if (kb == last_kept_block + 1 && kb < first_window_block) kb = first_window_block;
    const int page = page_table[(size_t)seq * table_stride + kb];
    const size_t kbase = ((size_t)page * nkv + kvh) * SYN_PAGE * dim;
    const size_t vbase = ((size_t)page * nkv + kvh) * SYN_PAGE * vdim;
    const int key = kb * SYN_PAGE + lane;
    const bool valid = key <= pos && (key >= lo || key < kept);
    float s = -INFINITY;
    if (valid) {
      const T* kr = k_pages + kbase + (size_t)lane * dim;
      float dot = 0.f;
      for (int d = 0; d < dim; ++d) dot = fmaf(qs[d], to_f32<T>(kr[d]), dot);
      s = window_score(dot, scale, terms, slope, r1, r2, pos, key);
    }
    const float m_new = fmaxf(m, wave_max(s));   // every block that is visited holds a visible key
    const float alpha = expf(m - m_new);
    const float p = valid ? expf(s - m_new) : 0.f;
    l = l * alpha + wave_sum(p);
    m = m_new;
    ps[lane] = p;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < AW_MAX_DIM / SYN_WAVE; ++i) {
      const int d = lane + i * SYN_WAVE;
      if (d < vdim) {
        const T* vr = v_pages + vbase + (size_t)d * SYN_PAGE;
        float acc = o[i] * alpha;
        for (int j = 0; j < SYN_PAGE; ++j) {
          const float pj = ps[j];
          if (pj != 0.f) acc = fmaf(pj, to_f32<T>(vr[j]), acc);   // slots past the sequence's end may hold anything
        }
        o[i] = acc;
      }
    }
    __syncthreads();
  }
  T* orow = out + ((size_t)tok * nh + head) * vdim;
  const float* g = gate ? gate + (size_t)tok * gate_stride + (size_t)head * vdim : nullptr;
#pragma unroll
  for (int i = 0; i < AW_MAX_DIM / SYN_WAVE; ++i) {
    const int d = lane + i * SYN_WAVE;
    if (d < vdim) {
      float v = o[i] / l;
      if (g) {
        const float z = g[d] + (gate_bias ? gate_bias[head * vdim + d] : 0.f);
        v *= 1.f / (1.f + expf(-z));
      }
      orow[d] = from_f32<T>(v);
    }
  }
}

// gate: float rows of gate_stride values whose first nh * vdim are the gate of each value (or null)
SYN_EXPORT int syn_window_attention(const void* q, const void* k_pages, const void* v_pages, int is_f32,
                                    const int* page_table, int table_stride, const int* tok_seq, const int* tok_pos,
                                    const float* gate, int gate_stride, const float* gate_bias, void* out, float scale,
                                    int n_tokens, int nh, int nkv, int dim, int vdim, const float* slopes,
                                    const float* r1, const float* r2, float softcap, int window, int keep_first,
                                    int sink_one, hipStream_t stream) {
  SYN_CHECK(n_tokens > 0 && nh > 0 && nkv > 0, "window_attention: empty input");
  SYN_CHECK(nh % nkv == 0, "window_attention: %d heads do not divide into %d kv heads", nh, nkv);
  SYN_CHECK(dim > 0 && dim <= AW_MAX_DIM && vdim > 0 && vdim <= AW_MAX_DIM,
            "window_attention: head sizes %d and %d are outside 1..%d", dim, vdim, AW_MAX_DIM);
  SYN_CHECK(softcap >= 0.f && window >= 0 && keep_first >= 0, "window_attention: soft cap %g, window %d, kept %d",
            (double)softcap, window, keep_first);
  SYN_CHECK((r1 == nullptr) == (r2 == nullptr), "window_attention: r1 and r2 come together");
  SYN_CHECK(gate == nullptr || gate_stride >= nh * vdim, "window_attention: gate rows of %d values", gate_stride);
  const WindowTerms terms = {slopes, r1, r2, softcap, window, keep_first, sink_one};
  const dim3 grid(n_tokens, nh);
  if (is_f32)
    window_attention_kernel<float><<<grid, SYN_WAVE, 0, stream>>>(
        (const float*)q, (const float*)k_pages, (const float*)v_pages, page_table, table_stride, tok_seq, tok_pos, gate,
        gate_stride, gate_bias, (float*)out, scale, nh, nkv, dim, vdim, terms);
  else
    window_attention_kernel<bf16><<<grid, SYN_WAVE, 0, stream>>>(
        (const bf16*)q, (const bf16*)k_pages, (const bf16*)v_pages, page_table, table_stride, tok_seq, tok_pos, gate,
        gate_stride, gate_bias, (bf16*)out, scale, nh, nkv, dim, vdim, terms);
  SYN_LAUNCH_CHECK("window_attention");
  return 0;
}
