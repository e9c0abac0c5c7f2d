// Latent attention in bf16 on the matrix cores: every head's query against ONE key row a cached token.
//
//   q       [N][heads][R]        R = rank + rot: the query in the latent's space, then its rotated part
//   k_pages [pages][64][R]       a token's row [latent | rotated key part]
//   v_pages [pages][rank x 64]   the latent once more, in the order of this kernel's fragments (la_v_offset): the
//                                8 values that a lane feeds into one matrix instruction lie together, a wave's 64
//                                lanes one after another: a fragment is 1 KB of consecutive bytes
//   out     [N][heads][rank]     sum_j softmax_j(scale q . k_j) k_j[:rank]  over the keys j that the query sees:
//                                j <= position, and position - j < window if there is a window
//
// Since all heads share the keys, the 16 rows of a tile are 16 consecutive (token, head) pairs of one sequence: for
// a single token its heads (decoding is a small matrix product, not a matrix-vector one), for a prompt a few tokens
// with all their heads.  One wave a tile, no LDS:
//   S^T (keys x rows)  = K (16 keys x k) . Q^T (k x 16 rows)        a lane holds four keys of ONE row
//   O^T (rank x rows) += V^T (16 values x 32 keys) . P^T (32 keys x 16 rows)
// and what a lane holds of S^T is exactly its share of the operand P^T (the 32 keys of a k-step are taken in the
// order in which two score tiles leave them, and V^T's 8-byte pieces are fetched in that order too).  The scores
// and weights are 32-bit; a weight meets V as two bf16 numbers (the weight rounded, and what the rounding left), so
// it counts with 16 bits of mantissa although the product runs in bf16; sums are 32-bit.
// A tile's pages may be cut into splits (grid y) whose partial results a second kernel merges, and (SHARE) the four
// waves of a workgroup may work on one tile together: single tokens over long sequences then fill the chip, and no
// wave walks a page alone.
#include "common.h"

#define LA_ROWS 16

template <bool X32> struct LaFrag;
template <> struct LaFrag<false> { typedef bf16x4 type; };
template <> struct LaFrag<true> { typedef bf16x8 type; };

__device__ __forceinline__ f32x4 la_mfma(bf16x4 a, bf16x4 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(short4_t, a), __builtin_bit_cast(short4_t, b), c, 0, 0, 0);
}
__device__ __forceinline__ f32x4 la_mfma(bf16x8 a, bf16x8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

// Where value d of the token in slot `slot` of a page lies in a bf16 value page of latent attention: fragment (d / 16,
// slot / 32), lane 16 g + d % 16, element e, with the 32 slots of a half in the order in which two tiles of scores
// leave them in a lane: e < 4: slot 4 g + e; e >= 4: slot 16 + 4 g + (e - 4).
__host__ __device__ __forceinline__ int la_v_offset(int d, int slot) {
  const int half = slot >> 5, s = slot & 31, second = s >> 4, g = (s & 15) >> 2, e = (s & 3) + 4 * second;
  return ((((d >> 4) * 2 + half) * 64 + g * 16 + (d & 15)) << 3) + e;
}

// the sequence and the unit inside it of global unit t, a unit being `unit_rows` consecutive (token, head) rows.
// Every wave searches for itself, 64 sequences at a time: a lane a sequence, a prefix sum of their units across the
// lanes, the first lane whose sum passes t (one trip to memory for 64 sequences, not one for each).  t is the same in
// all lanes of the wave.
__device__ __forceinline__ bool la_find_unit(int t, int unit_rows, const int* seq_start, int n_seqs, int nh, int& seq,
                                             int& unit, int& start, int& rows) {
  const int lane = threadIdx.x % SYN_WAVE;
  for (int b0 = 0; b0 < n_seqs; b0 += SYN_WAVE) {
    const int b = b0 + lane;
    const int s0 = b < n_seqs ? seq_start[b] : 0;
    const int n = b < n_seqs ? (seq_start[b + 1] - s0) * nh : 0;
    const int units = (n + unit_rows - 1) / unit_rows;
    int upto = units;                                    // units of the sequences b0 .. b
#pragma unroll
    for (int off = 1; off < SYN_WAVE; off <<= 1) {
      const int other = __shfl_up(upto, off, SYN_WAVE);
      if (lane >= off) upto += other;
    }
    const unsigned long long found = __ballot(t < upto);
    if (found) {
      const int at = __ffsll((long long)found) - 1;
      seq = b0 + at;
      unit = t - (__shfl(upto, at, SYN_WAVE) - __shfl(units, at, SYN_WAVE));
      start = __shfl(s0, at, SYN_WAVE);
      rows = __shfl(n, at, SYN_WAVE);
      return true;
    }
    t -= __shfl(upto, SYN_WAVE - 1, SYN_WAVE);
  }
  return false;
}

// DT: tiles of 16 values that the accumulators hold (rank <= 16 DT); QS: k-steps that the query's registers hold
// (R <= QS * (X32 ? 32 : 16)); X32: k-steps of 32 (R a multiple of 32) or of 16.
// SHARE false (prompts): a workgroup takes four consecutive tiles of one sequence, a wave each, and walks the pages
// that any of them sees: a page's keys and values go through LDS once for the four (rows of keys padded by 16 bytes
// against bank conflicts; dynamic LDS: 64 (R + 8) + 64 rank bf16 values).  SHARE true (single tokens): a workgroup
// takes one tile; on every page its four waves split the keys for the scores and the values for the second product.
template <int DT, int QS, bool X32, bool SHARE>
__global__ void __launch_bounds__(256)
latent_attention_bf16_kernel(const bf16* __restrict__ q, const bf16* __restrict__ k_pages, const bf16* __restrict__ v_pages,
                             const int* __restrict__ page_table, int table_stride, const int* __restrict__ seq_start,
                             const int* __restrict__ seq_past, int n_seqs, bf16* __restrict__ out,
                             float* __restrict__ part_o, float* __restrict__ part_ml, float scale, int nh, int rank, int R,
                             int window, int n_splits) {
  typedef typename LaFrag<X32>::type frag;
  constexpr int KS = X32 ? 32 : 16, PIECE = KS / 4;
  extern __shared__ __attribute__((aligned(16))) bf16 la_stage[];      // (SHARE false) a page's keys, then its values
  const int wave = threadIdx.x / SYN_WAVE, lane = threadIdx.x % SYN_WAVE, i = lane % 16, g = lane / 16;
  const int split = blockIdx.y;
  int seq, unit, start, rows;
  if (!la_find_unit(blockIdx.x, SHARE ? LA_ROWS : 4 * LA_ROWS, seq_start, n_seqs, nh, seq, unit, start, rows)) return;
  const int tile = SHARE ? unit : unit * 4 + wave;
  const bool tile_ok = tile * LA_ROWS < rows;                            // (SHARE: always)
  const int past = seq_past[seq];
  const int flat0 = tile_ok ? tile * LA_ROWS : rows - 1, flat_last = min(flat0 + LA_ROWS, rows) - 1;
  const bool row_ok = tile_ok && flat0 + i < rows;
  const int flat = row_ok ? flat0 + i : flat_last;       // a row beyond the tile's end repeats the last one, unstored
  const int tok = flat / nh, head = flat % nh, pos = past + tok;
  const int kv_len = past + rows / nh;
  // the pages that some row of the tile sees
  const int pos_lo = past + flat0 / nh, pos_hi = past + flat_last / nh;
  const int my_lo = (window > 0 ? max(0, pos_lo - window + 1) : 0) / SYN_PAGE, my_hi = pos_hi / SYN_PAGE;
  const int n_qs = R / KS, n_dt = rank / 16;

  frag qf[QS];
  const bf16* qrow = q + ((size_t)(start + tok) * nh + head) * R + g * PIECE;
#pragma unroll
  for (int ks = 0; ks < QS; ++ks)
    if (ks < n_qs) qf[ks] = *(const frag*)(qrow + ks * KS);

  // SHARE: a wave holds a quarter of the value tiles (DTW of them, from dt0 on); else all of them
  constexpr int DTW = SHARE ? DT / 4 : DT;
  const int dt0 = SHARE ? wave * ((n_dt + 3) / 4) : 0;
  const int dt_end = SHARE ? min(dt0 + (n_dt + 3) / 4, n_dt) : n_dt;
  f32x4 acc[DTW];
#pragma unroll
  for (int dt = 0; dt < DTW; ++dt) acc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;
  const int* pages = page_table + (size_t)seq * table_stride;

  // one page of 64 keys against the tile: kb = the lane's place in the page's first key row (rows of k_ld values),
  // vb = the lane's place in the page's first value fragment
  auto one_page = [&](const bf16* kb, int k_ld, const bf16* vb, int p) {
    f32x4 s[4];
#pragma unroll
    for (int kt = 0; kt < 4; ++kt) s[kt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < QS; ++ks)
      if (ks < n_qs) {
#pragma unroll
        for (int kt = 0; kt < 4; ++kt) {
          const frag a = *(const frag*)(kb + kt * 16 * k_ld + ks * KS);
          s[kt] = la_mfma(a, qf[ks], s[kt]);
        }
      }
    // s[kt][e]: key p * 64 + kt * 16 + 4 g + e against this lane's row
    const int key0 = p * SYN_PAGE + 4 * g;
    float top = -INFINITY;
#pragma unroll
    for (int kt = 0; kt < 4; ++kt)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int key = key0 + kt * 16 + e;
        const bool seen = key <= pos && (window <= 0 || pos - key < window);
        s[kt][e] = seen ? s[kt][e] * scale : -INFINITY;
        top = fmaxf(top, s[kt][e]);
      }
    top = fmaxf(top, __shfl_xor(top, 16, SYN_WAVE));
    top = fmaxf(top, __shfl_xor(top, 32, SYN_WAVE));
    const float m_new = fmaxf(m, top);
    const float base = m_new == -INFINITY ? 0.f : m_new;          // (a row that sees nothing of this page)
    const float alpha = expf(m - base);
    float sum = 0.f;
    bf16x4 hi[4], lo[4];
#pragma unroll
    for (int kt = 0; kt < 4; ++kt)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float w = expf(s[kt][e] - base);
        sum += w;
        hi[kt][e] = (bf16)w;
        lo[kt][e] = (bf16)(w - (float)hi[kt][e]);
      }
    sum += __shfl_xor(sum, 16, SYN_WAVE);
    sum += __shfl_xor(sum, 32, SYN_WAVE);
    l = l * alpha + sum;
    m = m_new;
#pragma unroll
    for (int dt = 0; dt < DTW; ++dt)
      if (dt < n_dt) acc[dt] *= alpha;
    // slots behind the sequence's end may hold anything: their weights are 0, their values are made 0 as well
    const int left = kv_len - p * SYN_PAGE;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      bf16x8 ph, pl;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        ph[e] = hi[2 * half][e], ph[4 + e] = hi[2 * half + 1][e];
        pl[e] = lo[2 * half][e], pl[4 + e] = lo[2 * half + 1][e];
      }
#pragma unroll
      for (int dt = 0; dt < DTW; ++dt)
        if (dt < n_dt) {
          bf16x8 a = *(const bf16x8*)(vb + (dt * 2 + half) * 512);
          if (left < SYN_PAGE) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              if (32 * half + 4 * g + e >= left) a[e] = (bf16)0.f;
              if (32 * half + 16 + 4 * g + e >= left) a[4 + e] = (bf16)0.f;
            }
          }
          acc[dt] = la_mfma(a, ph, acc[dt]);
          acc[dt] = la_mfma(a, pl, acc[dt]);
        }
    }
  };

  if constexpr (SHARE) {
    // This split's share of the tile's pages, one after another, the four waves on the same page: wave w multiplies
    // the 16 keys w * 16 .. of the page with the queries, the waves exchange maxima, sums and weights through LDS (the
    // weights already in the order of the second product's operand), and wave w then multiplies its quarter of the
    // value tiles with all 64 weights.  Every load of a phase is asked for before the first result is needed, the
    // values before the scores are exchanged.  What goes through LDS is kept twice, for pages in turns: two barriers
    // a page are enough.
    __shared__ float sh_max[2][4][LA_ROWS], sh_sum[2][4][LA_ROWS];
    __shared__ __attribute__((aligned(16))) bf16 sh_hi[2][2][SYN_WAVE][8], sh_lo[2][2][SYN_WAVE][8];
    const int chunk = (my_hi - my_lo + n_splits) / n_splits;
    const int p0 = my_lo + split * chunk, p1 = min(p0 + chunk, my_hi + 1);
    int par = 0;
    for (int p = p0; p < p1; ++p, par ^= 1) {
      const int page = pages[p];
      const bf16* kb = k_pages + (size_t)page * SYN_PAGE * R + (size_t)(wave * 16 + i) * R + g * PIECE;
      const bf16* vb = v_pages + (size_t)page * rank * SYN_PAGE + lane * 8;
      f32x4 s = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < QS; ++ks)
        if (ks < n_qs) s = la_mfma(*(const frag*)(kb + ks * KS), qf[ks], s);
      bf16x8 va[DTW][2];
#pragma unroll
      for (int j = 0; j < DTW; ++j)
        if (dt0 + j < dt_end) {
          va[j][0] = *(const bf16x8*)(vb + ((dt0 + j) * 2) * 512);
          va[j][1] = *(const bf16x8*)(vb + ((dt0 + j) * 2 + 1) * 512);
        }
      // s[e]: key p * 64 + wave * 16 + 4 g + e against this lane's row
      const int key0 = p * SYN_PAGE + wave * 16 + 4 * g;
      float top = -INFINITY;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int key = key0 + e;
        const bool seen = key <= pos && (window <= 0 || pos - key < window);
        s[e] = seen ? s[e] * scale : -INFINITY;
        top = fmaxf(top, s[e]);
      }
      top = fmaxf(top, __shfl_xor(top, 16, SYN_WAVE));
      top = fmaxf(top, __shfl_xor(top, 32, SYN_WAVE));
      if (g == 0) sh_max[par][wave][i] = top;
      __syncthreads();
      float m_new = m;
#pragma unroll
      for (int w = 0; w < 4; ++w) m_new = fmaxf(m_new, sh_max[par][w][i]);
      const float base = m_new == -INFINITY ? 0.f : m_new;
      const float alpha = expf(m - base);
      float sum = 0.f;
      bf16x4 hi, lo;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float w = expf(s[e] - base);
        sum += w;
        hi[e] = (bf16)w;
        lo[e] = (bf16)(w - (float)hi[e]);
      }
      sum += __shfl_xor(sum, 16, SYN_WAVE);
      sum += __shfl_xor(sum, 32, SYN_WAVE);
      if (g == 0) sh_sum[par][wave][i] = sum;
      // key tile `wave` is elements 4 (wave % 2) .. of the operand of half wave / 2
      *(bf16x4*)&sh_hi[par][wave >> 1][lane][4 * (wave & 1)] = hi;
      *(bf16x4*)&sh_lo[par][wave >> 1][lane][4 * (wave & 1)] = lo;
      __syncthreads();
      float total = 0.f;
#pragma unroll
      for (int w = 0; w < 4; ++w) total += sh_sum[par][w][i];
      l = l * alpha + total;
      m = m_new;
      const int left = kv_len - p * SYN_PAGE;
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        const bf16x8 ph = *(const bf16x8*)&sh_hi[par][half][lane][0], pl = *(const bf16x8*)&sh_lo[par][half][lane][0];
#pragma unroll
        for (int j = 0; j < DTW; ++j)
          if (dt0 + j < dt_end) {
            if (half == 0) acc[j] *= alpha;
            bf16x8 a = va[j][half];
            if (left < SYN_PAGE) {
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                if (32 * half + 4 * g + e >= left) a[e] = (bf16)0.f;
                if (32 * half + 16 + 4 * g + e >= left) a[4 + e] = (bf16)0.f;
              }
            }
            acc[j] = la_mfma(a, ph, acc[j]);
            acc[j] = la_mfma(a, pl, acc[j]);
          }
      }
    }
  } else {
    // the pages that any of the workgroup's four tiles sees, each through LDS once
    const int k_ld = R + 8;
    bf16* ks_ = la_stage;
    bf16* vs_ = la_stage + SYN_PAGE * k_ld;
    const int g_first = unit * 4 * LA_ROWS, g_last = min(g_first + 4 * LA_ROWS, rows) - 1;
    const int g_lo = (window > 0 ? max(0, past + g_first / nh - window + 1) : 0) / SYN_PAGE;
    const int g_hi = (past + g_last / nh) / SYN_PAGE;
    const int cpr = R / 8;                                   // 16-byte chunks of a key row
    const int row_step = 256 / cpr, col_step = 256 % cpr;
    for (int p = g_lo; p <= g_hi; ++p) {
      const int page = pages[p];
      const bf16* ksrc = k_pages + (size_t)page * SYN_PAGE * R;
      const bf16* vsrc = v_pages + (size_t)page * rank * SYN_PAGE;
      __syncthreads();                                       // everybody has done with the page before
      int row = threadIdx.x / cpr, col = threadIdx.x % cpr;
      for (int c = threadIdx.x; c < SYN_PAGE * cpr; c += 256) {
        *(bf16x8*)(ks_ + row * k_ld + col * 8) = *(const bf16x8*)(ksrc + (size_t)c * 8);
        row += row_step, col += col_step;
        if (col >= cpr) col -= cpr, ++row;
      }
      for (int c = threadIdx.x; c < rank * 8; c += 256) *(bf16x8*)(vs_ + c * 8) = *(const bf16x8*)(vsrc + (size_t)c * 8);
      __syncthreads();
      if (tile_ok && p >= my_lo && p <= my_hi) one_page(ks_ + i * k_ld + g * PIECE, k_ld, vs_ + lane * 8, p);
    }
    if (!tile_ok) return;
  }
  // acc[j][e]: value (dt0 + j) * 16 + 4 g + e of this lane's row
  if (n_splits == 1) {
    if (!row_ok) return;
    const float inv = 1.f / l;
    bf16* orow = out + ((size_t)(start + tok) * nh + head) * rank + 4 * g;
#pragma unroll
    for (int j = 0; j < DTW; ++j)
      if (dt0 + j < dt_end) {
        bf16x4 r;
#pragma unroll
        for (int e = 0; e < 4; ++e) r[e] = (bf16)(acc[j][e] * inv);
        *(bf16x4*)(orow + (dt0 + j) * 16) = r;
      }
  } else {
    // (SHARE only: blockIdx.x is the tile's number among all tiles)
    const size_t at = ((size_t)blockIdx.x * n_splits + split) * LA_ROWS + i;
    if (g == 0 && wave == 0) part_ml[2 * at] = m, part_ml[2 * at + 1] = l;
    float* prow = part_o + at * rank + 4 * g;
#pragma unroll
    for (int j = 0; j < DTW; ++j)
      if (dt0 + j < dt_end) *(f32x4*)(prow + (dt0 + j) * 16) = acc[j];
  }
}

// the splits of a tile merged in their order: the largest maximum, every split's sum and values scaled to it.
// One workgroup a (tile, row): the splits' maxima and sums fetched side by side, their factors in LDS, then a thread a
// value.
#define LA_MAX_SPLITS 1024
__global__ void __launch_bounds__(256)
latent_attention_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                              const int* __restrict__ seq_start, int n_seqs, bf16* __restrict__ out, int nh, int rank,
                              int n_splits) {
  __shared__ float factor[LA_MAX_SPLITS];
  __shared__ float red[16];
  const int gt = blockIdx.x, r = blockIdx.y;
  int seq, tile, start, rows;
  if (!la_find_unit(gt, LA_ROWS, seq_start, n_seqs, nh, seq, tile, start, rows)) return;
  const int flat = tile * LA_ROWS + r;
  if (flat >= rows) return;                 // (the whole workgroup)
  const size_t at0 = (size_t)gt * n_splits * LA_ROWS + r;
  float top = -INFINITY;
  for (int s = threadIdx.x; s < n_splits; s += blockDim.x) {
    const float ms = part_ml[2 * (at0 + (size_t)s * LA_ROWS)];
    factor[s] = ms;
    top = fmaxf(top, ms);
  }
  // the largest maximum of all splits: through LDS (block_sum's barriers also publish `factor`)
  top = wave_max(top);
  if (threadIdx.x % SYN_WAVE == 0) red[threadIdx.x / SYN_WAVE] = top;
  __syncthreads();
  float mm = -INFINITY;
  for (int w = 0; w < 4; ++w) mm = fmaxf(mm, red[w]);
  __syncthreads();
  float part = 0.f;
  for (int s = threadIdx.x; s < n_splits; s += blockDim.x) {
    const float ms = factor[s];
    const float f = ms == -INFINITY ? 0.f : expf(ms - mm);
    factor[s] = f;
    part += f * part_ml[2 * (at0 + (size_t)s * LA_ROWS) + 1];
  }
  const float l = block_sum(part, red);
  bf16* orow = out + ((size_t)(start + flat / nh) * nh + flat % nh) * rank;
  for (int d = threadIdx.x; d < rank; d += blockDim.x) {
    float o = 0.f;
    for (int s = 0; s < n_splits; ++s) {
      const float f = factor[s];
      if (f != 0.f) o += f * part_o[(at0 + (size_t)s * LA_ROWS) * rank + d];
    }
    orow[d] = (bf16)(o / l);
  }
}

template <int DT, int QS, bool X32, bool SHARE>
static int la_launch(const void* q, const void* k_pages, const void* v_pages, const int* page_table, int table_stride,
                     const int* seq_start, const int* seq_past, int n_seqs, void* out, float* part_o, float* part_ml,
                     float scale, int n_tiles, int nh, int rank, int R, int window, int n_splits, hipStream_t stream) {
  // SHARE: a workgroup a tile; else a workgroup for every four tiles of a sequence (n_tiles bounds both counts)
  const dim3 grid(n_tiles, n_splits);
  const size_t lds = SHARE ? 0 : ((size_t)SYN_PAGE * (R + 8) + (size_t)SYN_PAGE * rank) * sizeof(bf16);
  static OncePerDevice raised;
  if (lds > 49152) {
    const hipError_t e = once_per_device(raised, [&] {
      return hipFuncSetAttribute((const void*)latent_attention_bf16_kernel<DT, QS, X32, SHARE>,
                                 hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 4096);
    });
    SYN_CHECK(e == hipSuccess, "latent_attention: %zu bytes of LDS refused: %s", lds, hipGetErrorString(e));
  }
  latent_attention_bf16_kernel<DT, QS, X32, SHARE><<<grid, 256, lds, stream>>>(
      (const bf16*)q, (const bf16*)k_pages, (const bf16*)v_pages, page_table, table_stride, seq_start, seq_past, n_seqs,
      (bf16*)out, part_o, part_ml, scale, nh, rank, R, window, n_splits);
  return 0;
}

// share: the four waves of a workgroup take one tile's pages in turns (few tiles: single tokens), else a tile each
// and no splits.  n_tiles: the workgroups, at least the number of all sequences' tiles (share) or groups of four tiles;
// with share at least the number of tiles of all sequences, sum_b ceil(new tokens_b * heads / 16) (the host may not know
// the counts: (n_tokens * heads + 15) / 16 + n_seqs bounds it).  workspace: floats for n_tiles * n_splits * 16 *
// (rank + 2), used when n_splits > 1.
SYN_EXPORT int syn_latent_attention_bf16(const void* q, const void* k_pages, const void* v_pages, const int* page_table,
                                         int table_stride, const int* seq_start, const int* seq_past, int n_seqs,
                                         void* out, float* workspace, long workspace_floats, float scale, int n_tiles,
                                         int nh, int rank, int rot, int window, int n_splits, int share,
                                         hipStream_t stream) {
  const int R = rank + rot;
  SYN_CHECK(n_seqs > 0 && n_tiles > 0 && nh > 0, "latent_attention: empty input");
  SYN_CHECK(rank > 0 && rank % 16 == 0 && rank <= 512 && R % 16 == 0 && R <= 640,
            "latent_attention: rows of %d + %d values (multiples of 16 up to 512 and 640 together)", rank, rot);
  SYN_CHECK(window >= 0 && n_splits >= 1 && n_splits <= LA_MAX_SPLITS, "latent_attention: window %d, %d splits", window, n_splits);
  SYN_CHECK(n_splits == 1 || (workspace != nullptr && workspace_floats >= (long)n_tiles * n_splits * LA_ROWS * (rank + 2)),
            "latent_attention: a workspace of %ld floats for %d tiles in %d splits", workspace_floats, n_tiles, n_splits);
  SYN_CHECK(share || n_splits == 1, "latent_attention: pages are cut into splits only where a workgroup shares a tile");
  float* part_o = workspace;
  float* part_ml = workspace ? workspace + (size_t)n_tiles * n_splits * LA_ROWS * rank : nullptr;
  const bool x32 = R % 32 == 0;
  int rc = 0;
#define SYN_LA(DT, QS, X)                                                                                          \
  rc = share ? la_launch<DT, QS, X, true>(q, k_pages, v_pages, page_table, table_stride, seq_start, seq_past, n_seqs, \
                                          out, part_o, part_ml, scale, n_tiles, nh, rank, R, window, n_splits, stream) \
             : la_launch<DT, QS, X, false>(q, k_pages, v_pages, page_table, table_stride, seq_start, seq_past, n_seqs, \
                                           out, part_o, part_ml, scale, n_tiles, nh, rank, R, window, n_splits, stream)
  if (rank <= 128 && R <= 160) {
    if (x32) SYN_LA(8, 5, true); else SYN_LA(8, 10, false);
  } else if (rank <= 256 && R <= 320) {
    if (x32) SYN_LA(16, 10, true); else SYN_LA(16, 20, false);
  } else {
    if (x32) SYN_LA(32, 20, true); else SYN_LA(32, 40, false);
  }
#undef SYN_LA
  if (rc) return rc;
  SYN_LAUNCH_CHECK("latent_attention");
  if (n_splits > 1) {
    latent_attention_merge_kernel<<<dim3((n_tiles + 3) / 4 * 4, LA_ROWS), 256, 0, stream>>>(part_o, part_ml, seq_start, n_seqs,
                                                                                            (bf16*)out, nh, rank, n_splits);
    SYN_LAUNCH_CHECK("latent_attention_merge");
  }
  return 0;
}
