// Intake of latent attention: what a token's fused projection becomes before its attention runs.
//
// proj [N][width] float holds  [ q: heads x (dim | rot_dim) | down: rank + rot_dim | ... ]  (what lies behind, a gate,
// stays where it is).  For each token at position p:
//   c      = RMSNorm(down[0 .. rank)) * gain                      the latent that keys and values are made from
//   k_rot  = rotate(down[rank .. rank + rot_dim), p)               one rotated key part for all heads
//   q_nope[h] = q[h][0 .. dim)                                     -> q_nope [N][heads][dim]
//   q_rot[h]  = rotate(q[h][dim .. dim + rot_dim), p)              -> q_full [N][heads][rank + rot_dim], behind the
//                                                                    rank places that the absorbed query fills later
// The cache row of the token is [c | k_rot] (k_pages[page][0][token][rank + rot_dim]); c is also written transposed
// as the row's value (v_pages[page][0][rank][token]; with v_fragments in the order of the bf16 attention kernel's
// fragments instead).  The rotation turns the pairs (2i, 2i + 1), i < n_pairs, by
// the angle of table row p (cos, sin [capacity][n_pairs]); what lies behind 2 n_pairs passes unchanged.
// Arithmetic in 32-bit; one rounding at each store.
#include "common.h"

// Where value d of the token in slot `slot` lies in a value page kept in the order of the bf16 attention kernel's
// fragments (csrc/latent_attention.hip, la_v_offset: the same rule).
__device__ __forceinline__ int latent_v_offset(int d, int slot) {
  const int half = slot >> 5, s = slot & 31, second = s >> 4, g = (s & 15) >> 2, e = (s & 3) + 4 * second;
  return ((((d >> 4) * 2 + half) * 64 + g * 16 + (d & 15)) << 3) + e;
}

template <typename T>
__global__ void __launch_bounds__(256)
latent_intake_kernel(const float* __restrict__ proj, int width, const void* __restrict__ gain, int gain_is_f32, float eps,
                     const float* __restrict__ cos_t, const float* __restrict__ sin_t, int n_pairs,
                     T* __restrict__ q_nope, T* __restrict__ q_full, T* __restrict__ k_pages, T* __restrict__ v_pages,
                     const int* __restrict__ page_table, int table_stride, const int* __restrict__ tok_seq,
                     const int* __restrict__ tok_pos, int heads, int dim, int rot, int rank, int write_kv, int v_fragments) {
  __shared__ float red[16];
  const int tok = blockIdx.x, pos = tok_pos[tok];
  const float* row = proj + (size_t)tok * width;
  const float* cs = cos_t + (size_t)pos * n_pairs;
  const float* sn = sin_t + (size_t)pos * n_pairs;
  const int R = rank + rot, qd = dim + rot;
  // queries: the unrotated part as it is, the rotated part turned
  for (int i = threadIdx.x; i < heads * dim; i += blockDim.x) {
    const int h = i / dim, d = i % dim;
    q_nope[(size_t)tok * heads * dim + i] = from_f32<T>(row[h * qd + d]);
  }
  for (int i = threadIdx.x; i < heads * rot; i += blockDim.x) {
    const int h = i / rot, e = i % rot;
    const float* src = row + h * qd + dim;
    float v = src[e];
    if (e < 2 * n_pairs) {
      const float c = cs[e / 2], s = sn[e / 2];
      v = (e & 1) ? src[e] * c + src[e - 1] * s : src[e] * c - src[e + 1] * s;
    }
    q_full[((size_t)tok * heads + h) * R + rank + e] = from_f32<T>(v);
  }
  if (!write_kv) return;            // (uniform: no barrier has been reached)
  const float* down = row + heads * qd;
  float ss = 0.f;
  for (int d = threadIdx.x; d < rank; d += blockDim.x) ss += down[d] * down[d];
  ss = block_sum(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)rank + eps);
  const int page = page_table[(size_t)tok_seq[tok] * table_stride + pos / SYN_PAGE], slot = pos % SYN_PAGE;
  T* krow = k_pages + ((size_t)page * SYN_PAGE + slot) * R;
  T* vpage = v_pages + (size_t)page * rank * SYN_PAGE;
  for (int d = threadIdx.x; d < rank; d += blockDim.x) {
    const T c = from_f32<T>(down[d] * inv * load_gain(gain, gain_is_f32, d));
    krow[d] = c;
    vpage[v_fragments ? latent_v_offset(d, slot) : d * SYN_PAGE + slot] = c;
  }
  for (int e = threadIdx.x; e < rot; e += blockDim.x) {
    const float* src = down + rank;
    float v = src[e];
    if (e < 2 * n_pairs) {
      const float c = cs[e / 2], s = sn[e / 2];
      v = (e & 1) ? src[e] * c + src[e - 1] * s : src[e] * c - src[e + 1] * s;
    }
    krow[rank + e] = from_f32<T>(v);
  }
}

SYN_EXPORT int syn_latent_intake(const float* proj, int width, const void* gain, int gain_is_f32, float eps,
                                 const float* cos_t, const float* sin_t, int n_pairs, int capacity, int max_position,
                                 void* q_nope, void* q_full, void* k_pages, void* v_pages, int is_f32,
                                 const int* page_table, int table_stride, const int* tok_seq, const int* tok_pos,
                                 int n_tokens, int heads, int dim, int rot, int rank, int write_kv, int v_fragments,
                                 hipStream_t stream) {
  SYN_CHECK(n_tokens > 0 && heads > 0 && dim > 0 && rot >= 0 && rank > 0, "latent_intake: empty input");
  SYN_CHECK(width >= heads * (dim + rot) + rank + rot, "latent_intake: rows of %d values do not hold the queries and the latent", width);
  SYN_CHECK(n_pairs >= 0 && 2 * n_pairs <= rot, "latent_intake: %d rotated pairs in %d values", n_pairs, rot);
  SYN_CHECK(!v_fragments || rank % 16 == 0, "latent_intake: value pages in fragment order need a latent that is a multiple of 16, not %d", rank);
  SYN_CHECK(n_pairs == 0 || (cos_t && sin_t && max_position < capacity),
            "latent_intake: position %d is beyond the rotation's table of %d", max_position, capacity);
  if (is_f32)
    latent_intake_kernel<float><<<n_tokens, 256, 0, stream>>>(proj, width, gain, gain_is_f32, eps, cos_t, sin_t, n_pairs,
                                                              (float*)q_nope, (float*)q_full, (float*)k_pages,
                                                              (float*)v_pages, page_table, table_stride, tok_seq, tok_pos,
                                                              heads, dim, rot, rank, write_kv, v_fragments);
  else
    latent_intake_kernel<bf16><<<n_tokens, 256, 0, stream>>>(proj, width, gain, gain_is_f32, eps, cos_t, sin_t, n_pairs,
                                                             (bf16*)q_nope, (bf16*)q_full, (bf16*)k_pages, (bf16*)v_pages,
                                                             page_table, table_stride, tok_seq, tok_pos, heads, dim, rot,
                                                             rank, write_kv, v_fragments);
  SYN_LAUNCH_CHECK("latent_intake");
  return 0;
}
