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
template <typename TOut>
__global__ void streams_read_norm_kernel(float* __restrict__ X, const float* __restrict__ delta, int n_parts,
                                         size_t part_stride, const int* __restrict__ rows,
                                         const float* __restrict__ in_w, int S, int W, int kind,
                                         const float* __restrict__ alpha, const float* __restrict__ gain,
                                         const float* __restrict__ shift, TOut* __restrict__ out) {
  const int r = rows ? rows[blockIdx.x] : blockIdx.x;
  float* x = X + (size_t)r * S * W;
  const float* d = delta ? delta + (size_t)r * W : nullptr;
  TOut* o = out + (size_t)blockIdx.x * W;
  const bool write_back = rows == nullptr && d != nullptr;
  const float a = kind == SYN_ROWNORM_DYT ? alpha[0] : 0.f;
  float w_in[STREAMS_MAX];
#pragma unroll
  for (int s = 0; s < STREAMS_MAX; ++s) w_in[s] = (in_w && s < S) ? in_w[s] : 1.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    float u = 0.f;
#pragma unroll
    for (int s = 0; s < STREAMS_MAX; ++s)
      if (s < S) u += w_in[s] * x[(size_t)s * W + i];
    if (d) {
      for (int p = 0; p < n_parts; ++p) u += d[p * part_stride + i];
      if (write_back) x[i] = u;
    }
    if (kind == SYN_ROWNORM_DYT) u = tanhf(a * u) * gain[i] + shift[i];
    o[i] = from_f32<TOut>(u);
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
  const int block = W >= 2048 ? 512 : 256;
  const size_t stride = (size_t)n_rows * W;
  if (out_is_f32)
    streams_read_norm_kernel<float><<<n_out, block, 0, stream>>>(X, delta, n_parts, stride, rows, in_w, S, W, kind, alpha,
                                                                 gain, shift, (float*)out);
  else
    streams_read_norm_kernel<bf16><<<n_out, block, 0, stream>>>(X, delta, n_parts, stride, rows, in_w, S, W, kind, alpha,
                                                                gain, shift, (bf16*)out);
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

__global__ void streams_update_kernel(float* __restrict__ X, int S, int W, size_t part_stride,
                                      const float* __restrict__ mix, const float* __restrict__ out_w, DeltaTerm ta,
                                      DeltaTerm tb) {
  __shared__ float m[STREAMS_MAX * STREAMS_MAX];
  __shared__ float ow[STREAMS_MAX];
  for (int i = threadIdx.x; i < S * S; i += blockDim.x) m[i] = mix[i];
  for (int i = threadIdx.x; i < S; i += blockDim.x) ow[i] = out_w[i];
  __syncthreads();
  const size_t row = blockIdx.x;
  float* x = X + row * S * W;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    float y = 0.f;
    if (ta.y) {
      float t = 0.f;
      for (int p = 0; p < ta.n_parts; ++p) t += ta.y[p * part_stride + row * W + i];
      if (ta.bias) t += ta.bias[i];
      y = ta.scale * t;
    }
    if (tb.y) {
      float t = 0.f;
      for (int p = 0; p < tb.n_parts; ++p) t += tb.y[p * part_stride + row * W + i];
      if (tb.bias) t += tb.bias[i];
      y += tb.scale * t;
    }
    float xs[STREAMS_MAX];
#pragma unroll
    for (int s = 0; s < STREAMS_MAX; ++s) xs[s] = s < S ? x[(size_t)s * W + i] : 0.f;
#pragma unroll
    for (int t = 0; t < STREAMS_MAX; ++t) {
      if (t < S) {
        float v = 0.f;
#pragma unroll
        for (int s = 0; s < STREAMS_MAX; ++s)
          if (s < S) v += m[s * S + t] * xs[s];
        x[(size_t)t * W + i] = v + ow[t] * y;
      }
    }
  }
}

SYN_EXPORT int syn_streams_update(float* X, int n_rows, int S, int W, const float* mix, const float* out_w,
                                  const float* ya, int na, float ca, const float* bias_a, const float* yb, int nb,
                                  float cb, const float* bias_b, hipStream_t stream) {
  SYN_CHECK(n_rows > 0 && W > 0, "streams_update: empty input (%d rows, width %d)", n_rows, W);
  SYN_CHECK(S >= 1 && S <= STREAMS_MAX, "streams_update: %d streams (1 to %d)", S, STREAMS_MAX);
  SYN_CHECK(ya != nullptr && na >= 1 && na <= 64 && (yb == nullptr || (nb >= 1 && nb <= 64)),
            "streams_update: the result comes as one or two terms of 1 to 64 partial sums");
  const int block = W >= 2048 ? 512 : 256;
  streams_update_kernel<<<n_rows, block, 0, stream>>>(X, S, W, (size_t)n_rows * W, mix, out_w,
                                                      DeltaTerm{ya, na, ca, bias_a}, DeltaTerm{yb, nb, cb, bias_b});
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
