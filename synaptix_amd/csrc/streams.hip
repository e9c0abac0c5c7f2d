// A residual that runs in several streams (hyper-connections), and the norm without statistics.
//
// The residual of a token is S rows of W floats, X[token][s][:].  A sublayer reads one row that is a weighted sum of
// the streams,  u = sum_s in[s] X[s],  and its result y goes back into all of them at once,
//     X'[t] = sum_s mix[s][t] X[s] + out[t] y          (mix is indexed [from][to]),
// which takes the place of x + y.  S = 1 with in = out = mix = 1 is the plain residual.
//
// Dynamic tanh in place of a norm:  tanh(alpha u) w + b  with a scalar alpha; no mean, no variance, so the kernel
// that gathers u can apply it on the way.  Everything here is 32-bit; one rounding at the store of the normed row.
#include "common.h"

#define STREAMS_MAX 16

#define SYN_ROWNORM_NONE 0
#define SYN_ROWNORM_DYT 1

// out[i] = norm(sum_s in[s] X[row][s] (+ delta[row])) for row = rows ? rows[i] : i.  in == nullptr: every weight is 1
// (the sum of the streams).  delta: n_parts partial sums [n_parts][n_rows][W], only with S == 1, where without `rows`
// the sum is also written back into X (the plain residual sum in front of a norm).
template <typename TOut, int VEC>
__global__ void streams_read_norm_kernel(float* __restrict__ X, const float* __restrict__ delta, int n_parts,
                                         size_t part_stride, const int* __restrict__ rows,
                                         const float* __restrict__ in_w, int S, int W, int kind,
                                         const float* __restrict__ alpha, const float* __restrict__ gain,
                                         const float* __restrict__ shift, TOut* __restrict__ out) {
  typedef float vec_t __attribute__((ext_vector_type(VEC)));
  const int r = rows ? rows[blockIdx.x] : blockIdx.x;
  float* x = X + (size_t)r * S * W;
  const float* d = delta ? delta + (size_t)r * W : nullptr;
  TOut* o = out + (size_t)blockIdx.x * W;
  const bool write_back = rows == nullptr && d != nullptr;
  const float a = kind == SYN_ROWNORM_DYT ? alpha[0] : 0.f;
  float w_in[STREAMS_MAX];
#pragma unroll
  for (int s = 0; s < STREAMS_MAX; ++s) w_in[s] = (in_w && s < S) ? in_w[s] : 1.f;
  for (int i = threadIdx.x * VEC; i < W; i += blockDim.x * VEC) {
    vec_t u = 0.f;
#pragma unroll
    for (int s = 0; s < STREAMS_MAX; ++s)
      if (s < S) u += w_in[s] * *(const vec_t*)(x + (size_t)s * W + i);
    if (d) {
      for (int p = 0; p < n_parts; ++p) u += *(const vec_t*)(d + p * part_stride + i);
      if (write_back) *(vec_t*)(x + i) = u;
    }
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      float v = u[e];
      if (kind == SYN_ROWNORM_DYT) v = tanhf(a * v) * gain[i + e] + shift[i + e];
      o[i + e] = from_f32<TOut>(v);
    }
  }
}

SYN_EXPORT int syn_streams_read_norm(float* X, const float* delta, int n_parts, int n_rows, const int* rows, int n_out,
                                     const float* in_w, int S, int W, int kind, const float* alpha, const float* gain,
                                     const float* shift, void* out, int out_is_f32, hipStream_t stream) {
  SYN_CHECK(n_out > 0 && n_rows > 0 && W > 0, "streams_read_norm: empty input (%d rows, width %d)", n_out, W);
  SYN_CHECK(S >= 1 && S <= STREAMS_MAX, "streams_read_norm: %d streams (1 to %d)", S, STREAMS_MAX);
  SYN_CHECK(kind == SYN_ROWNORM_NONE || (kind == SYN_ROWNORM_DYT && alpha && gain && shift),
            "streams_read_norm: norm kind %d or its tensors", kind);
  SYN_CHECK(delta == nullptr || (S == 1 && n_parts >= 1 && n_parts <= 64),
            "streams_read_norm: a delta comes with one stream and 1 to 64 partial sums");
  const size_t stride = (size_t)n_rows * W;
  const bool vec = W % 4 == 0 && (uintptr_t)X % 16 == 0 && (uintptr_t)delta % 16 == 0;
  const int block = vec ? (W >= 4096 ? 512 : 256) : (W >= 2048 ? 512 : 256);
#define SYN_SR(T, V)                                                                                                   \
  streams_read_norm_kernel<T, V><<<n_out, block, 0, stream>>>(X, delta, n_parts, stride, rows, in_w, S, W, kind, alpha, \
                                                              gain, shift, (T*)out)
  if (out_is_f32) {
    if (vec) SYN_SR(float, 4); else SYN_SR(float, 1);
  } else {
    if (vec) SYN_SR(bf16, 4); else SYN_SR(bf16, 1);
  }
#undef SYN_SR
  SYN_LAUNCH_CHECK("streams_read_norm");
  return 0;
}

// X'[t] = sum_s mix[s][t] X[s] + out_w[t] y,   y = ca (sum_p a[p] + bias_a) + cb (sum_p b[p] + bias_b):
// a sublayer's result may come as two scaled terms (two mixers side by side), each as partial sums of a product cut
// along K and with the bias of its last product still to be added.
struct DeltaTerm {
  const float* y;      // [n_parts][n_rows][W] or nullptr
  int n_parts;
  float scale;
  const float* bias;   // [W] or nullptr
};

// What the next sublayer reads can leave in the same pass, while the new streams are still in registers:
// next.out[row] = norm(sum_t next.in_w[t] X'[t]) (in_w == nullptr: nothing leaves).
struct NextRead {
  const float* in_w;   // [S] or nullptr: no read
  int kind;            // SYN_ROWNORM_*
  const float* alpha;
  const float* gain;
  const float* shift;
  void* out;           // [n_rows][W]
};

template <typename TOut, int VEC>     // VEC columns a thread at a time (4: 16-byte loads and stores, W a multiple of 4)
__global__ void streams_update_kernel(float* __restrict__ X, int S, int W, size_t part_stride,
                                      const float* __restrict__ mix, const float* __restrict__ out_w, DeltaTerm ta,
                                      DeltaTerm tb, NextRead next) {
  __shared__ float m[STREAMS_MAX * STREAMS_MAX];
  __shared__ float ow[STREAMS_MAX];
  __shared__ float nw[STREAMS_MAX];
  for (int i = threadIdx.x; i < S * S; i += blockDim.x) m[i] = mix[i];
  for (int i = threadIdx.x; i < S; i += blockDim.x) ow[i] = out_w[i], nw[i] = next.in_w ? next.in_w[i] : 0.f;
  __syncthreads();
  typedef float vec_t __attribute__((ext_vector_type(VEC)));
  const size_t row = blockIdx.x;
  float* x = X + row * S * W;
  const float a = (next.in_w && next.kind == SYN_ROWNORM_DYT) ? next.alpha[0] : 0.f;
  auto term = [&](const DeltaTerm& t, int i) {
    vec_t sum = 0.f;
    for (int p = 0; p < t.n_parts; ++p) sum += *(const vec_t*)(t.y + p * part_stride + row * W + i);
    if (t.bias) sum += *(const vec_t*)(t.bias + i);
    return sum * t.scale;
  };
  for (int i = threadIdx.x * VEC; i < W; i += blockDim.x * VEC) {
    vec_t y = term(ta, i);
    if (tb.y) y += term(tb, i);
    vec_t xs[STREAMS_MAX];
#pragma unroll
    for (int s = 0; s < STREAMS_MAX; ++s)
      if (s < S) xs[s] = *(const vec_t*)(x + (size_t)s * W + i);
    vec_t u = 0.f;
#pragma unroll
    for (int t = 0; t < STREAMS_MAX; ++t) {
      if (t < S) {
        vec_t v = 0.f;
#pragma unroll
        for (int s = 0; s < STREAMS_MAX; ++s)
          if (s < S) v += m[s * S + t] * xs[s];
        v += ow[t] * y;
        *(vec_t*)(x + (size_t)t * W + i) = v;
        u += nw[t] * v;
      }
    }
    if (next.in_w) {
      TOut* o = (TOut*)next.out + row * W + i;
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        float r = u[e];
        if (next.kind == SYN_ROWNORM_DYT) r = tanhf(a * r) * next.gain[i + e] + next.shift[i + e];
        o[e] = from_f32<TOut>(r);
      }
    }
  }
}

// next_in .. next_out: see NextRead (next_in null: the streams are updated and nothing else)
SYN_EXPORT int syn_streams_update(float* X, int n_rows, int S, int W, const float* mix, const float* out_w,
                                  const float* ya, int na, float ca, const float* bias_a, const float* yb, int nb,
                                  float cb, const float* bias_b, const float* next_in, int next_kind,
                                  const float* next_alpha, const float* next_gain, const float* next_shift, void* next_out,
                                  int next_out_is_f32, hipStream_t stream) {
  SYN_CHECK(n_rows > 0 && W > 0, "streams_update: empty input (%d rows, width %d)", n_rows, W);
  SYN_CHECK(S >= 1 && S <= STREAMS_MAX, "streams_update: %d streams (1 to %d)", S, STREAMS_MAX);
  SYN_CHECK(ya != nullptr && na >= 1 && na <= 64 && (yb == nullptr || (nb >= 1 && nb <= 64)),
            "streams_update: the result comes as one or two terms of 1 to 64 partial sums");
  SYN_CHECK(next_in == nullptr || (next_out != nullptr && (next_kind == SYN_ROWNORM_NONE ||
                                   (next_kind == SYN_ROWNORM_DYT && next_alpha && next_gain && next_shift))),
            "streams_update: the read behind the update lacks its output or its norm's tensors");
  const DeltaTerm ta = {ya, na, ca, bias_a}, tb = {yb, nb, cb, bias_b};
  const NextRead next = {next_in, next_kind, next_alpha, next_gain, next_shift, next_out};
  const size_t stride = (size_t)n_rows * W;
  auto aligned = [](const void* p) { return (uintptr_t)p % 16 == 0; };
  const bool vec = W % 4 == 0 && aligned(X) && aligned(ya) && aligned(yb) && aligned(bias_a) && aligned(bias_b) &&
                   aligned(next_out);
  const int block = vec ? (W >= 4096 ? 512 : 256) : (W >= 2048 ? 512 : 256);
#define SYN_SU(T, V) streams_update_kernel<T, V><<<n_rows, block, 0, stream>>>(X, S, W, stride, mix, out_w, ta, tb, next)
  if (next_in != nullptr && !next_out_is_f32) {
    if (vec) SYN_SU(bf16, 4); else SYN_SU(bf16, 1);
  } else {
    if (vec) SYN_SU(float, 4); else SYN_SU(float, 1);
  }
#undef SYN_SU
  SYN_LAUNCH_CHECK("streams_update");
  return 0;
}

// X[token][s] = x[token] for every stream s: the streams all start as the embedding.
__global__ void streams_start_kernel(const float* __restrict__ x, float* __restrict__ X, int S, int W) {
  const size_t row = blockIdx.x;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    const float v = x[row * W + i];
    for (int s = 0; s < S; ++s) X[(row * S + s) * W + i] = v;
  }
}

SYN_EXPORT int syn_streams_start(const float* x, float* X, int n_rows, int S, int W, hipStream_t stream) {
  SYN_CHECK(n_rows > 0 && W > 0 && S >= 1, "streams_start: empty input (%d rows, %d streams, width %d)", n_rows, S, W);
  streams_start_kernel<<<n_rows, 256, 0, stream>>>(x, X, S, W);
  SYN_LAUNCH_CHECK("streams_start");
  return 0;
}
