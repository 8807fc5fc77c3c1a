// Attention over a cached latent: per position the cache holds one row [c | kr], the normed
// latent c (R numbers) from which every head's keys and values are linear maps, and an
// optional rotated key part kr (r numbers) that all heads share.
//
// The maps are taken to the query side, so that the cache is read as it lies and once for all
// heads: with k_h = U_h c the score q_h . k_h is (U_h^T q_h) . c, and with v_h = V_h c the
// output sum_j p_j v_hj is V_h (sum_j p_j c_j).  A step therefore runs
//   head_linear (q_h -> U_h^T q_h), latent_write (norm, rotation, cache write),
//   latent_attention (scores and weighted sums of cached rows), head_linear (V_h).
// Scores, softmax and sums are float32.  A query at position p sees keys at positions <= p and,
// under a window w, > p - w.  With a sink the softmax's denominator also holds exp(sink[h]):
// a key with that score (not scaled) and no value.
#include "common.h"
#include "tile_mma.h"

#include <math.h>

// ------------------------------------------------------------ one product per head
// y[t][h][n] = sum_k w[h][n][k] * x[t][h][k]; x rows ldx apart with heads x_head apart, y the
// same with ldy / y_head; w is (H, N, K) contiguous.  A wave takes 16 tokens x 64 columns.
template <typename T, typename TO, bool ALIGNED>
__global__ __launch_bounds__(256) void head_linear_kernel(
    const T* __restrict__ x, long long ldx, int x_head, const T* __restrict__ w,
    TO* __restrict__ y, long long ldy, int y_head, int rows, int N, int K) {
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int h = blockIdx.z;
  const int t0 = (blockIdx.x * 4 + wave) * 16;
  if (t0 >= rows) return;
  const int n0 = blockIdx.y * 64;
  const int ta = min(t0 + lane % 16, rows - 1);
  const T* a_row = x + (long long)ta * ldx + (long long)h * x_head;
  const T* b_row[4];
#pragma unroll
  for (int b = 0; b < 4; ++b) {
    const int n = min(n0 + b * 16 + lane % 16, N - 1);
    b_row[b] = w + ((long long)h * N + n) * K;
  }
  mma_f32x4 acc[4];
  wave_tile_product<T, 4, ALIGNED>(a_row, b_row, K, acc);
#pragma unroll
  for (int b = 0; b < 4; ++b) {
    const int n = n0 + b * 16 + lane % 16;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int t = t0 + (lane / 16) * 4 + i;
      if (t < rows && n < N) st(y + (long long)t * ldy + (long long)h * y_head + n, acc[b][i]);
    }
  }
}

RLIS_API int rlis_head_linear(const void* x, int dtype, long long ldx, int x_head, const void* w,
                              void* y, int y_dtype, long long ldy, int y_head, int rows, int H,
                              int N, int K, hipStream_t stream) {
  RLIS_REQUIRE(rows >= 0 && H > 0 && N > 0 && K > 0, "head_linear: bad sizes");
  RLIS_REQUIRE(x_head >= K && y_head >= N && ldx >= (long long)(H - 1) * x_head + K &&
                   ldy >= (long long)(H - 1) * y_head + N,
               "head_linear: strides shorter than the heads they hold");
  RLIS_REQUIRE(H <= 65535 && ceil_div(N, 64) <= 65535, "head_linear: too many heads or columns");
  if (rows == 0) return 0;
  dim3 grid(ceil_div(rows, 64), ceil_div(N, 64), H);
#define LAUNCH(T, TO, AL)                                                                  \
  head_linear_kernel<T, TO, AL><<<grid, 256, 0, stream>>>((const T*)x, ldx, x_head,        \
                                                         (const T*)w, (TO*)y, ldy, y_head, \
                                                         rows, N, K)
  if (dtype == RLIS_BF16) {
    const bool al = mma_rows_aligned<bf16_t>(x, ldx, x_head, K) &&
                    mma_rows_aligned<bf16_t>(w, K, 0, K);
    if (y_dtype == RLIS_BF16) { if (al) LAUNCH(bf16_t, bf16_t, true); else LAUNCH(bf16_t, bf16_t, false); }
    else { if (al) LAUNCH(bf16_t, float, true); else LAUNCH(bf16_t, float, false); }
  } else if (dtype == RLIS_F32) {
    RLIS_REQUIRE(y_dtype == RLIS_F32, "head_linear: a float32 product has a float32 result");
    const bool al = mma_rows_aligned<float>(x, ldx, x_head, K) && mma_rows_aligned<float>(w, K, 0, K);
    if (al) LAUNCH(float, float, true); else LAUNCH(float, float, false);
  } else {
    RLIS_REQUIRE(false, "head_linear: unknown dtype %d", dtype);
  }
#undef LAUNCH
  RLIS_LAUNCH_CHECK("head_linear");
  return 0;
}

// ------------------------------------------------- norm, rotation and cache write
// Per token: c = x[:R] / sqrt(mean(x[:R]^2) + eps) * weight goes to the token's cache row, the
// r numbers behind it are rotated by the token's position (the first rot of them: entry i with
// entry i + rot/2; the rest pass) and follow c in the row; the last r numbers of every query
// head are rotated the same way into the head's row of q_out behind its first R columns.
// x is float32; angles come from float32 tables (positions, rot/2).  With pages_t the latent is
// stored a second time with the positions of a page innermost ([page][j][offset]), which is how
// the matrix-core kernel reads it as values.
template <typename TX>
__global__ __launch_bounds__(256) void latent_write_kernel(
    const float* __restrict__ x, long long ldx, const float* __restrict__ weight, float eps,
    int R, int r, int rot, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    const int* __restrict__ positions, const int* __restrict__ slots, TX* __restrict__ pages,
    TX* __restrict__ pages_t, int page_size, int write, const TX* __restrict__ q, long long ldq, int q_head, int q_off,
    TX* __restrict__ q_out, long long ldo, int o_head, int H) {
  __shared__ float red[4];
  const int t = blockIdx.x;
  const int pos = positions[t];
  const int half = rot / 2;
  const float* xr = x + (long long)t * ldx;
  if (write) {
    TX* row = pages + (long long)slots[t] * (R + r);
    float ss = 0.f;
    for (int j = threadIdx.x; j < R; j += 256) ss += xr[j] * xr[j];
    ss = block_sum<256>(ss, red);
    const float mult = 1.0f / sqrtf(ss / (float)R + eps);
    for (int j = threadIdx.x; j < R; j += 256) st(row + j, xr[j] * mult * weight[j]);
    if (pages_t) {         // the same latent once more, positions innermost: [page][j][offset]
      TX* col = pages_t + (long long)(slots[t] / page_size) * R * page_size + slots[t] % page_size;
      for (int j = threadIdx.x; j < R; j += 256)
        st(col + (long long)j * page_size, xr[j] * mult * weight[j]);
    }
    for (int j = threadIdx.x; j < r; j += 256) {
      float v = xr[R + j];
      if (j < rot) {
        const int i = j < half ? j : j - half;
        const float c = cos_t[(long long)pos * half + i], s = sin_t[(long long)pos * half + i];
        const float u = xr[R + i], w = xr[R + i + half];
        v = j < half ? u * c - w * s : w * c + u * s;
      }
      st(row + R + j, v);
    }
  }
  for (int e = threadIdx.x; e < H * r; e += 256) {
    const int h = e / r, j = e % r;
    const TX* qh = q + (long long)t * ldq + (long long)h * q_head + q_off;
    float v = ld(qh + j);
    if (j < rot) {
      const int i = j < half ? j : j - half;
      const float c = cos_t[(long long)pos * half + i], s = sin_t[(long long)pos * half + i];
      const float u = ld(qh + i), w = ld(qh + i + half);
      v = j < half ? u * c - w * s : w * c + u * s;
    }
    st(q_out + (long long)t * ldo + (long long)h * o_head + R + j, v);
  }
}

RLIS_API int rlis_latent_write(const float* x, long long ldx, const float* weight, float eps,
                               int R, int r, int rot, const float* cos_t, const float* sin_t,
                               const int* positions, const int* slots, void* pages,
                               void* pages_t, int page_size, int dtype, int write, const void* q, long long ldq, int q_head, int q_off,
                               void* q_out, long long ldo, int o_head, int H, int T,
                               hipStream_t stream) {
  RLIS_REQUIRE(T >= 0 && R > 0 && r >= 0 && rot >= 0 && rot <= r && rot % 2 == 0 && H > 0,
               "latent_write: bad sizes R=%d r=%d rot=%d", R, r, rot);
  RLIS_REQUIRE(rot == 0 || (cos_t && sin_t), "latent_write: a rotation needs its tables");
  RLIS_REQUIRE(!write || (ldx >= R + r && pages && slots && weight),
               "latent_write: the cache write needs rows, pages and slots");
  RLIS_REQUIRE(!pages_t || page_size > 0, "latent_write: the transposed copy needs the page size");
  RLIS_REQUIRE(r == 0 || (q && q_out && q_head >= q_off + r && o_head >= R + r),
               "latent_write: the rotated query part needs its rows");
  if (T == 0 || (!write && r == 0)) return 0;
#define LAUNCH(TX)                                                                            \
  latent_write_kernel<TX><<<T, 256, 0, stream>>>(x, ldx, weight, eps, R, r, rot, cos_t, sin_t, \
                                                 positions, slots, (TX*)pages, (TX*)pages_t,   \
                                                 page_size, write,                             \
                                                 (const TX*)q, ldq, q_head, q_off, (TX*)q_out, \
                                                 ldo, o_head, H)
  if (dtype == RLIS_F32) LAUNCH(float);
  else if (dtype == RLIS_BF16) LAUNCH(bf16_t);
  else RLIS_REQUIRE(false, "latent_write: unknown dtype %d", dtype);
#undef LAUNCH
  RLIS_LAUNCH_CHECK("latent_write");
  return 0;
}

// --------------------------------------------------------------- attention, vector units
// One wave per (token, head).  q rows hold per head the D = R + r numbers that meet a cached
// row; the output per head is sum_j p_j c_j over the first R numbers of the rows.  A lane takes
// one key of a round of 64 (its whole dot product), then the lanes share the columns of the
// weighted sum.
template <typename TX, int CPL>
__global__ __launch_bounds__(64) void latent_attention_kernel(
    const TX* __restrict__ q, long long ldq, TX* __restrict__ out, long long ldo,
    const TX* __restrict__ pages, const int* __restrict__ block_tables, int max_pages,
    const int* __restrict__ seq_of_token, const int* __restrict__ positions, int H, int R,
    int D, int page_size, float scale, int window, const float* __restrict__ sink) {
  extern __shared__ float smem[];
  float* q_s = smem;                                // D
  float* p_s = smem + D;                            // 64
  long long* row_s = (long long*)(p_s + 64);        // 64
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int seq = seq_of_token[t];
  const int pos = positions[t];
  const int* table = block_tables + (long long)seq * max_pages;
  for (int j = lane; j < D; j += 64) q_s[j] = ld(q + (long long)t * ldq + (long long)h * D + j) * scale;
  __syncthreads();
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  // the sink is a key that every query sees: it opens the running maximum and denominator
  float m = sink ? sink[h] : -INFINITY;
  float l = sink ? 1.f : 0.f;
  float acc[CPL];
#pragma unroll
  for (int i = 0; i < CPL; ++i) acc[i] = 0.f;
  for (int k0 = lo; k0 <= pos; k0 += 64) {
    const int kpos = k0 + lane;
    const bool valid = kpos <= pos;
    const int kp = valid ? kpos : pos;
    const long long row = ((long long)table[kp / page_size] * page_size + kp % page_size) * D;
    const TX* c = pages + row;
    float dot = 0.f;
    for (int j = 0; j < D; ++j) dot = fmaf(q_s[j], ld(c + j), dot);
    const float s = valid ? dot : -INFINITY;
    const float m_new = fmaxf(m, wave_max(s));
    const float p = valid ? expf(s - m_new) : 0.f;
    const float corr = (m == -INFINITY) ? 0.f : expf(m - m_new);
    l = l * corr + wave_sum(p);
    p_s[lane] = p;
    row_s[lane] = row;
    __syncthreads();
    const int n = min(64, pos - k0 + 1);
#pragma unroll
    for (int i = 0; i < CPL; ++i) {
      const int j = lane + 64 * i;
      if (j < R) {
        float a = acc[i] * corr;
        for (int kk = 0; kk < n; ++kk) a = fmaf(p_s[kk], ld(pages + row_s[kk] + j), a);
        acc[i] = a;
      }
    }
    __syncthreads();
    m = m_new;
  }
  const float inv_l = 1.0f / l;
#pragma unroll
  for (int i = 0; i < CPL; ++i) {
    const int j = lane + 64 * i;
    if (j < R) st(out + (long long)t * ldo + (long long)h * R + j, acc[i] * inv_l);
  }
}

RLIS_API int rlis_latent_attention(const void* q, int dtype, long long ldq, void* out,
                                   long long ldo, const void* pages, const int* block_tables,
                                   int max_pages, const int* seq_of_token, const int* positions,
                                   int T, int H, int R, int D, int page_size, float scale,
                                   int window, const float* sink, hipStream_t stream) {
  RLIS_REQUIRE(T >= 0 && H > 0 && R > 0 && D >= R && page_size > 0 && max_pages > 0,
               "latent_attention: bad sizes");
  RLIS_REQUIRE(R <= 1024 && D <= 2048, "latent_attention: latent of %d (row of %d) is too wide",
               R, D);
  RLIS_REQUIRE(H <= 65535 && ldq >= (long long)H * D && ldo >= (long long)H * R,
               "latent_attention: rows shorter than their heads");
  if (T == 0) return 0;
  dim3 grid(T, H);
  const size_t smem = (size_t)D * 4 + 64 * 4 + 64 * 8 + 8;
  const int cpl = ceil_div(R, 64);
#define LAUNCH(TX, CPL)                                                                       \
  latent_attention_kernel<TX, CPL><<<grid, 64, smem, stream>>>(                               \
      (const TX*)q, ldq, (TX*)out, ldo, (const TX*)pages, block_tables, max_pages,            \
      seq_of_token, positions, H, R, D, page_size, scale, window, sink)
#define BY_CPL(TX)                         \
  do {                                     \
    if (cpl <= 1) LAUNCH(TX, 1);           \
    else if (cpl <= 2) LAUNCH(TX, 2);      \
    else if (cpl <= 4) LAUNCH(TX, 4);      \
    else if (cpl <= 8) LAUNCH(TX, 8);      \
    else LAUNCH(TX, 16);                   \
  } while (0)
  if (dtype == RLIS_F32) BY_CPL(float);
  else if (dtype == RLIS_BF16) BY_CPL(bf16_t);
  else RLIS_REQUIRE(false, "latent_attention: unknown dtype %d", dtype);
#undef BY_CPL
#undef LAUNCH
  RLIS_LAUNCH_CHECK("latent_attention");
  return 0;
}

// --------------------------------------------------------------- attention, matrix cores
// bfloat16.  A wave takes 16 (token, head) columns of one sequence: 16 heads of a token, or
// with fewer heads 16 / HP tokens x HP heads (HP the power of two that holds the heads), and
// walks the keys its columns see in chunks of 32.  Transposed products, so that a column's
// softmax statistics stay in its lanes and the probabilities never leave registers:
// S^T = C Q^T (rows: keys; the cached rows [c | kr] are loaded straight into operand layout)
// and O^T += C^T P^T (rows: latent channels; C^T comes from the copy that lies with positions
// innermost, 8 keys in one 16-byte load).  Row i of S^T's block u is key 8 (i / 4) + 4 u + i % 4
// of the chunk, which puts a lane's 8 probabilities on 8 consecutive keys.  The queries wait in
// LDS (a wave's own 16 rows); scale, mask, sink and sums are float32; P is rounded to
// bfloat16 as the second product's operand only.  How a sequence's keys are cut follows from
// its own positions, so a row does not depend on its neighbours.  A wave holds the sums of
// 16 NT latent channels; wider latents are shared out over gridDim.z workgroups, each of which
// forms the scores again (the walk is bound by the round trips of its loads, not by the matrix
// cores, and fewer sums per wave leave registers for loads in flight).
template <int NT, bool SPLIT>
__global__ __launch_bounds__(256) void latent_attention_mfma_kernel(
    const bf16_t* __restrict__ q, long long ldq, bf16_t* __restrict__ out, long long ldo,
    const bf16_t* __restrict__ pages, const bf16_t* __restrict__ pages_t,
    const int* __restrict__ block_tables, int max_pages, const int* __restrict__ cu,
    const int* __restrict__ positions, int num_seqs, int H, int R, int D, int page_size,
    float scale, int window, const float* __restrict__ sink, int HP) {
  extern __shared__ __align__(16) unsigned char lds_raw[];
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int c = lane % 16, g = lane / 16;
  const int TB = 16 / HP;
  const int stride = D + 8;
  // SPLIT: the four waves share one block of columns and take every fourth chunk of keys each
  // (steps of few tokens: the grid is small and a context is a long walk for one wave)
  bf16_t* q_s = reinterpret_cast<bf16_t*>(lds_raw) + (SPLIT ? 0 : (size_t)wave * 16 * stride);
  int blk = SPLIT ? blockIdx.x : blockIdx.x * 4 + wave;
  int seq = -1, t_first = 0, t_end = 0;
  for (int s = 0; s < num_seqs; ++s) {
    const int a = cu[s], b = cu[s + 1];
    const int tiles = (b - a + TB - 1) / TB;
    if (blk < tiles) {
      seq = s;
      t_first = a + blk * TB;
      t_end = b;
      break;
    }
    blk -= tiles;
  }
  if (seq < 0) return;       // (the whole wave, and with SPLIT the whole workgroup)
  const int tok = t_first + c / HP;
  const int head = blockIdx.y * HP + c % HP;
  const bool col_ok = tok < t_end && head < H;
  const int tok_c = min(tok, t_end - 1), head_c = min(head, H - 1);
  const int pos = positions[tok_c];
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int hi_blk = positions[min(t_first + TB, t_end) - 1];
  const int p_first = positions[t_first];
  const int lo_blk = (window > 0 && p_first - window + 1 > 0) ? p_first - window + 1 : 0;
  const bf16_t* q_row = q + (long long)tok_c * ldq + (long long)head_c * D;
  if (!SPLIT || wave == 0)
    for (int j = g * 8; j < D; j += 32)
      *reinterpret_cast<mma_u32x4*>(q_s + c * stride + j) =
          *reinterpret_cast<const mma_u32x4*>(q_row + j);
  if (SPLIT) __syncthreads();
  const int* table = block_tables + (long long)seq * max_pages;
  const int dim0 = blockIdx.z * NT * 16;         // this workgroup's share of the latent channels
  const bool opens = !SPLIT || wave == 0;        // whose sums the sink opens
  float m = (sink && opens) ? sink[head_c] : -INFINITY;
  float l = (sink && opens && g == 0) ? 1.f : 0.f;
  mma_f32x4 acc[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) acc[t] = mma_f32x4{0.f, 0.f, 0.f, 0.f};
  const int steps = (D + 31) / 32;
  const mma_u32x4 zero = {0u, 0u, 0u, 0u};
  constexpr int GS = NT == 4 ? 4 : 6;                    // key loads asked for together
  for (int k0 = (lo_blk & ~31) + (SPLIT ? 32 * wave : 0); k0 <= hi_blk;
       k0 += SPLIT ? 128 : 32) {
    const int kk0 = min(k0 + 8 * (c / 4) + c % 4, hi_blk), kk1 = min(kk0 + 4, hi_blk);
    const bf16_t* kr0 =
        pages + ((long long)table[kk0 / page_size] * page_size + kk0 % page_size) * D;
    const bf16_t* kr1 =
        pages + ((long long)table[kk1 / page_size] * page_size + kk1 % page_size) * D;
    mma_f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
    for (int sb = 0; sb < steps; sb += GS) {
      mma_u32x4 a0[GS], a1[GS];
#pragma unroll
      for (int u = 0; u < GS; ++u) {      // (past the row's end: a clamped address and zeros)
        a0[u] = mma_load<bf16_t, true>(kr0, 32 * (sb + u) + 8 * g, D);
        a1[u] = mma_load<bf16_t, true>(kr1, 32 * (sb + u) + 8 * g, D);
      }
#pragma unroll
      for (int u = 0; u < GS; ++u) {
        const int dch = 32 * (sb + u) + 8 * g;
        const mma_u32x4 qr =
            *reinterpret_cast<const mma_u32x4*>(q_s + c * stride + (dch < D ? dch : 0));
        const mma_bf16x8 qv = __builtin_bit_cast(mma_bf16x8, dch < D ? qr : zero);
        s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(mma_bf16x8, a0[u]), qv,
                                                     s0, 0, 0, 0);
        s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(mma_bf16x8, a1[u]), qv,
                                                     s1, 0, 0, 0);
      }
    }
    float sv[8];
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int key0 = k0 + 8 * g + i, key1 = key0 + 4;
      sv[i] = (col_ok && key0 >= lo && key0 <= pos) ? s0[i] * scale : -INFINITY;
      sv[4 + i] = (col_ok && key1 >= lo && key1 <= pos) ? s1[i] * scale : -INFINITY;
      mx = fmaxf(mx, fmaxf(sv[i], sv[4 + i]));
    }
    mx = xor32_max(xor16_max(mx));
    const float m_new = fmaxf(m, mx);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float corr = m == -INFINITY ? 0.f : __expf(m - m_use);
    float psum = 0.f;
    bf16_t pk[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float p = __expf(sv[j] - m_use);
      psum += p;
      pk[j] = f32_to_bf16(p);
    }
    l = l * corr + psum;
    m = m_new;
    const mma_bf16x8 pv = __builtin_bit_cast(mma_bf16x8, pk);
    const int kv = k0 + 8 * g;
    const long long vpage = table[min(kv / page_size, max_pages - 1)];
    const bf16_t* vt = pages_t + vpage * R * page_size + kv % page_size;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const int dim = min(dim0 + 16 * t + c, R - 1);
      const mma_u32x4 a = *reinterpret_cast<const mma_u32x4*>(vt + (long long)dim * page_size);
      acc[t] *= corr;
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(mma_bf16x8, a), pv,
                                                       acc[t], 0, 0, 0);
    }
  }
  if (SPLIT) {
    // waves 2, 3 hand their sums to waves 0, 1, then wave 1 hands the pair's to wave 0:
    // per lane m, l and the 4 NT sums, laid out [value][lane]
    float* hand = reinterpret_cast<float*>(lds_raw + 16 * stride * 2) ;
    constexpr int kVals = 4 * NT + 2;
#pragma unroll
    for (int round = 0; round < 2; ++round) {
      const bool gives = round == 0 ? wave >= 2 : wave == 1;
      const bool takes = round == 0 ? wave < 2 : wave == 0;
      float* mine = hand + (size_t)(round == 0 ? wave & 1 : 0) * kVals * kWave + lane;
      __syncthreads();
      if (gives) {
        mine[0] = m;
        mine[kWave] = l;
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
          for (int i = 0; i < 4; ++i) mine[(size_t)(2 + 4 * t + i) * kWave] = acc[t][i];
      }
      __syncthreads();
      if (takes) {
        const float m_b = mine[0], l_b = mine[kWave];
        const float m_ab = fmaxf(m, m_b);
        const float fa = m == -INFINITY ? 0.f : __expf(m - m_ab);
        const float fb = m_b == -INFINITY ? 0.f : __expf(m_b - m_ab);
        l = l * fa + l_b * fb;
        m = m_ab;
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
          for (int i = 0; i < 4; ++i)
            acc[t][i] = acc[t][i] * fa + mine[(size_t)(2 + 4 * t + i) * kWave] * fb;
      }
    }
    if (wave != 0) return;
  }
  const float total = xor32_sum(xor16_sum(l));
  if (!col_ok) return;
  const float inv = 1.0f / total;
  bf16_t* o = out + (long long)tok * ldo + (long long)head * R;
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int dim = dim0 + 16 * t + 4 * g + i;
      if (dim < R) o[dim] = f32_to_bf16(acc[t][i] * inv);
    }
}

// The same walk for steps of many tokens, with a chunk's keys and values staged once per
// workgroup: 4 DH waves, wave (cb, dh) taking column block cb (of four neighbouring ones: 4 x 16
// / HP tokens of one sequence) and the share dh of the latent channels (16 NT each).  All
// threads ask for the next chunk's rows together (one round trip, in flight during the
// products of the chunk at hand), park them in registers and move them to LDS behind a barrier;
// every fragment of a key or a value that was loaded once then serves the four column blocks.
// The arithmetic of a column is that of the kernel above (the two shares of a column block form
// the same scores and statistics).
template <int NT, int DH>
__global__ __launch_bounds__(256 * DH) void latent_attention_staged_kernel(
    const bf16_t* __restrict__ q, long long ldq, bf16_t* __restrict__ out, long long ldo,
    const bf16_t* __restrict__ pages, const bf16_t* __restrict__ pages_t,
    const int* __restrict__ block_tables, int max_pages, const int* __restrict__ cu,
    const int* __restrict__ positions, int num_seqs, int H, int R, int D, int page_size,
    float scale, int window, const float* __restrict__ sink, int HP) {
  extern __shared__ __align__(16) unsigned char lds_raw[];
  constexpr int THREADS = 256 * DH, VD = NT * 16 * DH, VSTRIDE = 40;
  constexpr int KL = DH == 2 ? 5 : 6, VL = NT / 4;
  const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
  const int c = lane % 16, g = lane / 16;
  const int cb = wave % 4, dh = wave / 4;
  const int TB = 16 / HP;
  const int stride = D + 8;
  bf16_t* q_s = reinterpret_cast<bf16_t*>(lds_raw) + (size_t)cb * 16 * stride;
  bf16_t* k_s = reinterpret_cast<bf16_t*>(lds_raw) + (size_t)64 * stride;
  bf16_t* v_s = k_s + (size_t)32 * stride;
  int blk = blockIdx.x;
  int seq = -1, t_first = 0, t_end = 0;
  for (int s = 0; s < num_seqs; ++s) {
    const int a = cu[s], b = cu[s + 1];
    const int tiles = (b - a + 4 * TB - 1) / (4 * TB);
    if (blk < tiles) {
      seq = s;
      t_first = a + blk * 4 * TB;
      t_end = b;
      break;
    }
    blk -= tiles;
  }
  if (seq < 0) return;                               // (the whole workgroup)
  const int tok = t_first + cb * TB + c / HP;
  const int head = blockIdx.y * HP + c % HP;
  const bool col_ok = tok < t_end && head < H;
  const int tok_c = min(tok, t_end - 1), head_c = min(head, H - 1);
  const int pos = positions[tok_c];
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int hi_wg = positions[min(t_first + 4 * TB, t_end) - 1];
  const int p_first = positions[t_first];
  const int lo_wg = (window > 0 && p_first - window + 1 > 0) ? p_first - window + 1 : 0;
  if (dh == 0) {
    const bf16_t* q_row = q + (long long)tok_c * ldq + (long long)head_c * D;
    for (int j = g * 8; j < D; j += 32)
      *reinterpret_cast<mma_u32x4*>(q_s + c * stride + j) =
          *reinterpret_cast<const mma_u32x4*>(q_row + j);
  }
  const int* table = block_tables + (long long)seq * max_pages;
  const int dim0 = blockIdx.z * VD + dh * NT * 16;   // this wave's latent channels
  float m = sink ? sink[head_c] : -INFINITY;
  float l = (sink && g == 0) ? 1.f : 0.f;
  mma_f32x4 acc[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) acc[t] = mma_f32x4{0.f, 0.f, 0.f, 0.f};
  const int steps = (D + 31) / 32;
  const int segs = D / 8, k_total = 32 * segs;
  const mma_u32x4 zero = {0u, 0u, 0u, 0u};
  mma_u32x4 pk[KL], pv[VL];
  // every thread's share of a chunk: KL 16-byte pieces of key rows, VL of value rows
  auto ask = [&](int k0) {
#pragma unroll
    for (int i = 0; i < KL; ++i) {
      const int idx = min(tid + i * THREADS, k_total - 1);
      const int key = min(k0 + idx / segs, hi_wg);
      pk[i] = *reinterpret_cast<const mma_u32x4*>(
          pages + ((long long)table[key / page_size] * page_size + key % page_size) * D +
          (idx % segs) * 8);
    }
#pragma unroll
    for (int i = 0; i < VL; ++i) {
      const int idx = tid + i * THREADS;             // < VD * 4
      const int key0 = k0 + 8 * (idx % 4);
      const long long page = table[min(key0 / page_size, max_pages - 1)];
      const int dim = min(blockIdx.z * VD + idx / 4, R - 1);
      pv[i] = *reinterpret_cast<const mma_u32x4*>(pages_t + (page * R + dim) * page_size +
                                                  key0 % page_size);
    }
  };
  auto park = [&]() {
#pragma unroll
    for (int i = 0; i < KL; ++i) {
      const int idx = tid + i * THREADS;
      if (idx < k_total)
        *reinterpret_cast<mma_u32x4*>(k_s + (idx / segs) * stride + (idx % segs) * 8) = pk[i];
    }
#pragma unroll
    for (int i = 0; i < VL; ++i) {
      const int idx = tid + i * THREADS;
      *reinterpret_cast<mma_u32x4*>(v_s + (idx / 4) * VSTRIDE + (idx % 4) * 8) = pv[i];
    }
  };
  const int k_first = lo_wg & ~31;
  ask(k_first);
  for (int k0 = k_first; k0 <= hi_wg; k0 += 32) {
    __syncthreads();                                 // the chunk before has been read
    park();
    __syncthreads();
    if (k0 + 32 <= hi_wg) ask(k0 + 32);
    const bf16_t* kr0 = k_s + (8 * (c / 4) + c % 4) * stride;
    const bf16_t* kr1 = kr0 + 4 * stride;
    mma_f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
    for (int s = 0; s < steps; ++s) {
      const int dch = 32 * s + 8 * g;
      const int at = dch < D ? dch : 0;
      const mma_u32x4 qr = *reinterpret_cast<const mma_u32x4*>(q_s + c * stride + at);
      const mma_u32x4 r0 = *reinterpret_cast<const mma_u32x4*>(kr0 + at);
      const mma_u32x4 r1 = *reinterpret_cast<const mma_u32x4*>(kr1 + at);
      const mma_bf16x8 qv = __builtin_bit_cast(mma_bf16x8, dch < D ? qr : zero);
      s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
          __builtin_bit_cast(mma_bf16x8, dch < D ? r0 : zero), qv, s0, 0, 0, 0);
      s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
          __builtin_bit_cast(mma_bf16x8, dch < D ? r1 : zero), qv, s1, 0, 0, 0);
    }
    float sv[8];
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int key0 = k0 + 8 * g + i, key1 = key0 + 4;
      sv[i] = (col_ok && key0 >= lo && key0 <= pos) ? s0[i] * scale : -INFINITY;
      sv[4 + i] = (col_ok && key1 >= lo && key1 <= pos) ? s1[i] * scale : -INFINITY;
      mx = fmaxf(mx, fmaxf(sv[i], sv[4 + i]));
    }
    mx = xor32_max(xor16_max(mx));
    const float m_new = fmaxf(m, mx);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float corr = m == -INFINITY ? 0.f : __expf(m - m_use);
    float psum = 0.f;
    bf16_t pb[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float p = __expf(sv[j] - m_use);
      psum += p;
      pb[j] = f32_to_bf16(p);
    }
    l = l * corr + psum;
    m = m_new;
    const mma_bf16x8 pr = __builtin_bit_cast(mma_bf16x8, pb);
    const bf16_t* vt = v_s + (size_t)(dh * NT * 16 + c) * VSTRIDE + 8 * g;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const mma_u32x4 a = *reinterpret_cast<const mma_u32x4*>(vt + (size_t)16 * t * VSTRIDE);
      acc[t] *= corr;
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(mma_bf16x8, a), pr,
                                                       acc[t], 0, 0, 0);
    }
  }
  const float total = xor32_sum(xor16_sum(l));
  if (!col_ok) return;
  const float inv = 1.0f / total;
  bf16_t* o = out + (long long)tok * ldo + (long long)head * R;
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int dim = dim0 + 16 * t + 4 * g + i;
      if (dim < R) o[dim] = f32_to_bf16(acc[t][i] * inv);
    }
}

static LdsGrant g_latent_lds[8];
static LdsGrant g_latent_staged_lds[3];

// Whether the matrix-core kernel takes a latent of R numbers in rows of D.
RLIS_API int rlis_latent_attention_mfma_ok(int R, int D, int page_size) {
  // (a workgroup's four waves keep 16 query rows of D numbers each in LDS)
  return (R > 0 && R <= 1024 && D >= R && D <= 1024 && D % 8 == 0 && page_size % 8 == 0) ? 1 : 0;
}

RLIS_API int rlis_latent_attention_mfma(const void* q, long long ldq, void* out, long long ldo,
                                        const void* pages, const void* pages_t,
                                        const int* block_tables, int max_pages, const int* cu,
                                        const int* positions, int T, int num_seqs, int H, int R,
                                        int D, int page_size, float scale, int window,
                                        const float* sink, int split_max_blocks, int staged,
                                        hipStream_t stream) {
  RLIS_REQUIRE(T >= 0 && num_seqs > 0 && H > 0 && D >= R && max_pages > 0,
               "latent_attention_mfma: bad sizes");
  RLIS_REQUIRE(rlis_latent_attention_mfma_ok(R, D, page_size),
               "latent_attention_mfma: a latent of %d in rows of %d with pages of %d is not taken",
               R, D, page_size);
  RLIS_REQUIRE(ldq % 8 == 0 && (uintptr_t)q % 16 == 0 && (uintptr_t)pages % 16 == 0 &&
                   (uintptr_t)pages_t % 16 == 0,
               "latent_attention_mfma: operands must lie on 16-byte boundaries");
  RLIS_REQUIRE(ldq >= (long long)H * D && ldo >= (long long)H * R,
               "latent_attention_mfma: rows shorter than their heads");
  if (T == 0) return 0;
  int hp = 1;
  while (hp < H && hp < 16) hp *= 2;
  const int tb = 16 / hp;
  const int blocks = ceil_div(T, tb) + num_seqs;
  const int heads_y = ceil_div(H, hp);
  RLIS_REQUIRE(heads_y <= 65535, "latent_attention_mfma: too many heads");
  // few blocks of columns (steps of few tokens): a workgroup's waves share one and split its keys
  const bool split = (long long)blocks * heads_y <= split_max_blocks;
  if (!split && staged && D <= 640) {
    // large steps: a chunk's keys and values staged once per workgroup of four column blocks
    const int tiles16 = ceil_div(R, 16);
    const int wgs = ceil_div(T, 4 * tb) + num_seqs;
#define STAGED(NT, DH, slot)                                                                     \
  do {                                                                                           \
    const int vd = NT * 16 * DH;                                                                 \
    const int lds = (64 + 32) * (D + 8) * 2 + vd * 40 * 2;                                       \
    if (lds > 48 * 1024) {                                                                       \
      hipError_t e = grant_lds(g_latent_staged_lds[slot],                                        \
                               (const void*)latent_attention_staged_kernel<NT, DH>, lds);        \
      RLIS_REQUIRE(e == hipSuccess, "latent_attention_mfma: LDS of %d bytes refused", lds);       \
    }                                                                                            \
    latent_attention_staged_kernel<NT, DH>                                                       \
        <<<dim3(wgs, heads_y, ceil_div(R, vd)), 256 * DH, lds, stream>>>(                        \
            (const bf16_t*)q, ldq, (bf16_t*)out, ldo, (const bf16_t*)pages,                      \
            (const bf16_t*)pages_t, block_tables, max_pages, cu, positions, num_seqs, H, R, D,   \
            page_size, scale, window, sink, hp);                                                 \
  } while (0)
    bool took = true;
    if (tiles16 > 16) STAGED(16, 2, 0);
    else if (tiles16 > 8 && D <= 384) STAGED(16, 1, 1);
    else if (tiles16 <= 8 && D <= 384) STAGED(8, 1, 2);
    else took = false;
#undef STAGED
    if (took) {
      RLIS_LAUNCH_CHECK("latent_attention_mfma");
      return 0;
    }
  }
  // sums per wave: up to 128 latent channels in small steps (more workgroups, more loads in
  // flight), up to 256 in large ones (the scores are formed once more per share)
  const int tiles = ceil_div(R, 16);
  const int nt = tiles <= 4 ? 4 : (tiles <= 8 || (split && (long long)blocks * heads_y <= 64)) ? 8 : 16;
  dim3 grid(split ? blocks : ceil_div(blocks, 4), heads_y, ceil_div(tiles, nt));
#define LAUNCH_AS(NT, SP, slot)                                                                \
  do {                                                                                         \
    const int lds = SP ? 16 * (D + 8) * 2 + 2 * (4 * NT + 2) * kWave * 4                       \
                       : 4 * 16 * (D + 8) * 2;                                                 \
    if (lds > 48 * 1024) {                                                                     \
      hipError_t e = grant_lds(g_latent_lds[slot],                                             \
                               (const void*)latent_attention_mfma_kernel<NT, SP>, lds);        \
      RLIS_REQUIRE(e == hipSuccess, "latent_attention_mfma: LDS of %d bytes refused", lds);     \
    }                                                                                          \
    latent_attention_mfma_kernel<NT, SP><<<grid, 256, lds, stream>>>(                          \
        (const bf16_t*)q, ldq, (bf16_t*)out, ldo, (const bf16_t*)pages, (const bf16_t*)pages_t, \
        block_tables, max_pages, cu, positions, num_seqs, H, R, D, page_size, scale, window,   \
        sink, hp);                                                                             \
  } while (0)
#define LAUNCH(NT, slot)                              \
  do {                                                \
    if (split) LAUNCH_AS(NT, true, 4 + slot);         \
    else LAUNCH_AS(NT, false, slot);                  \
  } while (0)
  if (nt == 4) LAUNCH(4, 0);
  else if (nt == 8) LAUNCH(8, 1);
  else LAUNCH(16, 2);
#undef LAUNCH
#undef LAUNCH_AS
  RLIS_LAUNCH_CHECK("latent_attention_mfma");
  return 0;
}

// ----------------------------------------------------------------- sigmoid gate
// o[t][j] *= sigmoid(g[t][j]) in place for rows ldo / ldg apart, the product in float32 with
// one rounding.
template <typename TX>
__global__ void sigmoid_gate_kernel(TX* __restrict__ o, long long ldo, const TX* __restrict__ g,
                                    long long ldg, int N, long long total) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const long long t = i / N;
  const int j = (int)(i % N);
  TX* p = o + t * ldo + j;
  st(p, ld(p) / (1.0f + expf(-ld(g + t * ldg + j))));
}

RLIS_API int rlis_sigmoid_gate(void* o, long long ldo, const void* g, long long ldg, int dtype,
                               int T, int N, hipStream_t stream) {
  RLIS_REQUIRE(T >= 0 && N > 0 && ldo >= N && ldg >= N, "sigmoid_gate: bad sizes");
  const long long total = (long long)T * N;
  if (total == 0) return 0;
  const unsigned blocks = (unsigned)ceil_div_ll(total, 256);
  if (dtype == RLIS_F32)
    sigmoid_gate_kernel<float><<<blocks, 256, 0, stream>>>((float*)o, ldo, (const float*)g, ldg, N, total);
  else if (dtype == RLIS_BF16)
    sigmoid_gate_kernel<bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)o, ldo, (const bf16_t*)g, ldg, N, total);
  else
    RLIS_REQUIRE(false, "sigmoid_gate: unknown dtype %d", dtype);
  RLIS_LAUNCH_CHECK("sigmoid_gate");
  return 0;
}
