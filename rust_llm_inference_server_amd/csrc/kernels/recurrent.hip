// Kernels of mixers that keep a state of fixed size per request instead of a cache that grows:
// the inputs of the last few tokens (token shift, short causal convolution) and, per head, a
// matrix S of key channels x value channels that every token decays, writes to and reads from.
//
// A request's state lives in its slot of the runner's state buffer: `state` points at this
// mixer's area inside slot 0 and `state_stride` floats lead from one slot to the next.  All of
// it is float32, and everything that enters a recurrence is float32 arithmetic.  Every kernel
// walks a sequence's tokens of the step in order (cu[s] .. cu[s + 1]) from the state that the
// step before left, whatever else is in the batch; a sequence at position 0 finds zeros (the
// runner clears the slot), which are the zeros in front of a sequence's first token.
//
// The matrix state is walked by one wave per (sequence, head, value channel j): lane i holds
// S[i][j] (and i + 64, ... for more than 64 key channels), a token's read-out is one sum over
// the wave, and nothing is shared between waves, so the columns of a head spread over the chip.
// State layout per head: [value channel][key channel], so a wave's column is contiguous.
#include "common.h"

namespace {

constexpr int kMaxTaps = 16;

__device__ __forceinline__ float sigmoidf_(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float siluf_(float x) { return x / (1.0f + expf(-x)); }
__device__ __forceinline__ float softplusf_(float x) { return x > 20.0f ? x : log1pf(expf(x)); }

// ------------------------------------------------------------------ token shift
// out[m][t][c] = x[t][c] + (prev[t][c] - x[t][c]) * mu[m][c], prev = the row of the token
// before (the tail row of the state for a sequence's first token of the step).
template <typename TX>
__global__ void shift_mix_kernel(TX* __restrict__ out, const TX* __restrict__ x,
                                 const float* __restrict__ mu, const float* __restrict__ state,
                                 long long state_stride, const int* __restrict__ seq_of_token,
                                 const int* __restrict__ cu, const int* __restrict__ slots, int T,
                                 int W, int mixes) {
  const int t = blockIdx.x;
  const int s = seq_of_token[t];
  const bool first = t == cu[s];
  const float* tail = state + (long long)slots[s] * state_stride;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float cur = ld(x + (long long)t * W + c);
    const float prev = first ? tail[c] : ld(x + (long long)(t - 1) * W + c);
    const float d = prev - cur;
    for (int m = 0; m < mixes; ++m)
      st(out + ((long long)m * T + t) * W + c, cur + d * mu[(long long)m * W + c]);
  }
}

// ------------------------------------------------------------------ input tails
// A sequence's tail holds the rows of its last R inputs, oldest first.  After a step of n rows
// it is the last R of (old tail ++ the step's rows).  A thread owns a channel, reads what it
// needs of the old tail and then writes, so a step shorter than the tail shifts it in place.
template <typename TX>
__global__ void tail_update_kernel(float* __restrict__ state, long long state_stride,
                                   const TX* __restrict__ x, long long ldx, int C, int R,
                                   const int* __restrict__ cu, const int* __restrict__ slots) {
  const int s = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int t0 = cu[s], n = cu[s + 1] - t0;
  float* tail = state + (long long)slots[s] * state_stride;
  float keep[kMaxTaps];
#pragma unroll
  for (int r = 0; r < kMaxTaps; ++r) {
    if (r < R) {
      const int src = n + r;          // index into (old tail ++ new rows) of the row kept at r
      keep[r] = src < R ? tail[(long long)src * C + c]
                        : ld(x + (long long)(t0 + src - R) * ldx + c);
    }
  }
#pragma unroll
  for (int r = 0; r < kMaxTaps; ++r)
    if (r < R) tail[(long long)r * C + c] = keep[r];
}

// ------------------------------------------- short causal convolution + SiLU (+ unit norm)
// y[t][c] = silu(sum_j taps[c][j] * x[t - (K - 1) + j][c]); rows in front of the step come from
// the tail, rows in front of the sequence are the tail's zeros.  Channels [0, unit_channels)
// are then made unit vectors in groups of unit_group (x / sqrt(sum x^2 + unit_eps)) and those
// below scaled_channels multiplied by `scale`; the other channels are cut into groups of
// rest_group for the grid only.  One block per (token, group), up to 4 channels per thread.
__global__ __launch_bounds__(256) void causal_conv_kernel(
    float* __restrict__ out, const float* __restrict__ x, long long ldx,
    const float* __restrict__ taps, int C, int K, const float* __restrict__ state,
    long long state_stride, const int* __restrict__ seq_of_token, const int* __restrict__ cu,
    const int* __restrict__ slots, int unit_channels, int unit_group, int scaled_channels,
    float scale, float unit_eps, int rest_group) {
  __shared__ float red[256 / kWave];
  const int t = blockIdx.x;
  const int groups_unit = unit_group > 0 ? unit_channels / unit_group : 0;
  const int g = blockIdx.y;
  int c0, width;
  const bool unit = g < groups_unit;
  if (unit) {
    c0 = g * unit_group;
    width = unit_group;
  } else {
    c0 = unit_channels + (g - groups_unit) * rest_group;
    width = min(rest_group, C - c0);
  }
  const int s = seq_of_token[t];
  const int rel = t - cu[s];                 // rows of the step in front of this one
  const int R = K - 1;
  const float* tail = state + (long long)slots[s] * state_stride;
  float y[4];
  float ss = 0.f;
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    const int c = c0 + threadIdx.x + v * 256;
    y[v] = 0.f;
    if (threadIdx.x + v * 256 < width) {
      float acc = 0.f;
      for (int j = 0; j < K; ++j) {
        const int back = R - j;              // how many rows before t
        const float in = back <= rel ? x[(long long)(t - back) * ldx + c]
                                     : tail[(long long)(R - (back - rel)) * C + c];
        acc += taps[(long long)c * K + j] * in;
      }
      y[v] = siluf_(acc);
      ss += y[v] * y[v];
    }
  }
  float mult = 1.0f;
  if (unit) {
    ss = block_sum<256>(ss, red);
    mult = 1.0f / sqrtf(ss + unit_eps);
    if (c0 < scaled_channels) mult *= scale;
  }
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    const int c = c0 + threadIdx.x + v * 256;
    if (threadIdx.x + v * 256 < width) out[(long long)t * C + c] = y[v] * mult;
  }
}

// ------------------------------------------------------------- gated delta rule
// Per token and head, with one decay g and one step size beta per head:
//   S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q.
// g = exp(-exp(A_log) * softplus(a + dt_bias)), beta = sigmoid(b), from the raw projections.
// Each column j of S is independent: u_j = beta (v_j - sum_i S_ij k_i), and so on.
template <int KR>
__global__ __launch_bounds__(256) void delta_scan_kernel(
    float* __restrict__ out, long long ldo, const float* __restrict__ q, const float* __restrict__ k,
    const float* __restrict__ v, long long ldqkv, const float* __restrict__ b_raw,
    const float* __restrict__ a_raw, long long ldba, const float* __restrict__ a_log,
    const float* __restrict__ dt_bias, float* __restrict__ state, long long state_stride,
    const int* __restrict__ cu, const int* __restrict__ slots, int heads, int kv_heads, int dk,
    int dv) {
  const int lane = threadIdx.x % kWave;
  const int wave = threadIdx.x / kWave;
  const int cols_per_block = blockDim.x / kWave;
  const int j = blockIdx.x * cols_per_block + wave;
  const int head = blockIdx.y;
  const int s = blockIdx.z;
  if (j >= dv) return;
  const int kh = head / (heads / kv_heads);
  const int t0 = cu[s], t1 = cu[s + 1];
  float* col = state + (long long)slots[s] * state_stride + ((long long)head * dv + j) * dk;
  float S[KR];
#pragma unroll
  for (int r = 0; r < KR; ++r) {
    const int i = lane + r * kWave;
    S[r] = i < dk ? col[i] : 0.f;
  }
  const float neg_a = -expf(a_log[head]);
  const float bias = dt_bias[head];
  float kn[KR], qn[KR], vn = 0.f, bn = 0.f, an = 0.f;
  auto fetch = [&](int t) {
    const float* kt = k + (long long)t * ldqkv + kh * dk;
    const float* qt = q + (long long)t * ldqkv + kh * dk;
#pragma unroll
    for (int r = 0; r < KR; ++r) {
      const int i = lane + r * kWave;
      kn[r] = i < dk ? kt[i] : 0.f;
      qn[r] = i < dk ? qt[i] : 0.f;
    }
    vn = v[(long long)t * ldqkv + head * dv + j];
    bn = b_raw[(long long)t * ldba + head];
    an = a_raw[(long long)t * ldba + head];
  };
  if (t0 < t1) fetch(t0);
  for (int t = t0; t < t1; ++t) {
    float kc[KR], qc[KR];
#pragma unroll
    for (int r = 0; r < KR; ++r) {
      kc[r] = kn[r];
      qc[r] = qn[r];
    }
    const float vc = vn, bc = bn, ac = an;
    if (t + 1 < t1) fetch(t + 1);
    const float g = expf(neg_a * softplusf_(ac + bias));
    const float beta = sigmoidf_(bc);
    float dot = 0.f;
#pragma unroll
    for (int r = 0; r < KR; ++r) {
      S[r] *= g;
      dot += S[r] * kc[r];
    }
    dot = wave_sum(dot);
    const float u = beta * (vc - dot);
    float o = 0.f;
#pragma unroll
    for (int r = 0; r < KR; ++r) {
      S[r] += kc[r] * u;
      o += S[r] * qc[r];
    }
    o = wave_sum(o);
    if (lane == 0) out[(long long)t * ldo + head * dv + j] = o;
  }
#pragma unroll
  for (int r = 0; r < KR; ++r) {
    const int i = lane + r * kWave;
    if (i < dk) col[i] = S[r];
  }
}

// ------------------------------------------------- decayed state with a bonus for the present
// Per token and head, with a decay per key channel w_i = exp(-exp(z_i + w0_i)):
//   o = (S + diag(u) k v^T)^T r;  S <- diag(w) S + k v^T.
// Keys, values and receptances have one size `d` here; z is the raw low-rank projection.
template <int KR>
__global__ __launch_bounds__(256) void decay_scan_kernel(
    float* __restrict__ out, const float* __restrict__ r_in, const float* __restrict__ k_in,
    const float* __restrict__ v_in, const float* __restrict__ z_in, long long ld,
    const float* __restrict__ w0, const float* __restrict__ bonus, float* __restrict__ state,
    long long state_stride, const int* __restrict__ cu, const int* __restrict__ slots, int heads,
    int d) {
  const int lane = threadIdx.x % kWave;
  const int wave = threadIdx.x / kWave;
  const int cols_per_block = blockDim.x / kWave;
  const int j = blockIdx.x * cols_per_block + wave;
  const int head = blockIdx.y;
  const int s = blockIdx.z;
  if (j >= d) return;
  const int t0 = cu[s], t1 = cu[s + 1];
  float* col = state + (long long)slots[s] * state_stride + ((long long)head * d + j) * d;
  float S[KR], u[KR], base[KR];
#pragma unroll
  for (int r = 0; r < KR; ++r) {
    const int i = lane + r * kWave;
    S[r] = i < d ? col[i] : 0.f;
    u[r] = i < d ? bonus[head * d + i] : 0.f;
    base[r] = i < d ? w0[head * d + i] : 0.f;
  }
  float rn[KR], kn[KR], zn[KR], vn = 0.f;
  auto fetch = [&](int t) {
    const long long row = (long long)t * ld + head * d;
#pragma unroll
    for (int r = 0; r < KR; ++r) {
      const int i = lane + r * kWave;
      rn[r] = i < d ? r_in[row + i] : 0.f;
      kn[r] = i < d ? k_in[row + i] : 0.f;
      zn[r] = i < d ? z_in[row + i] : 0.f;
    }
    vn = v_in[row + j];
  };
  if (t0 < t1) fetch(t0);
  for (int t = t0; t < t1; ++t) {
    float rc[KR], kc[KR], zc[KR];
#pragma unroll
    for (int r = 0; r < KR; ++r) {
      rc[r] = rn[r];
      kc[r] = kn[r];
      zc[r] = zn[r];
    }
    const float vc = vn;
    if (t + 1 < t1) fetch(t + 1);
    float o = 0.f;
#pragma unroll
    for (int r = 0; r < KR; ++r) {
      const float kv = kc[r] * vc;
      const float w = expf(-expf(zc[r] + base[r]));
      o += rc[r] * (S[r] + u[r] * kv);
      S[r] = w * S[r] + kv;
    }
    o = wave_sum(o);
    if (lane == 0) out[(long long)t * ld + head * d + j] = o;
  }
#pragma unroll
  for (int r = 0; r < KR; ++r) {
    const int i = lane + r * kWave;
    if (i < d) col[i] = S[r];
  }
}

// --------------------------------------------------- per-head RMS norm, weight and gate
// y[t][h][j] = o / sqrt(mean_j o^2 + eps) * weight[h * weight_stride + j] * silu(gate[t][h][j]).
// One wave per (token, head).
template <typename TG, typename TO>
__global__ __launch_bounds__(kWave) void head_norm_gate_kernel(
    TO* __restrict__ out, const float* __restrict__ o, const float* __restrict__ weight,
    int weight_stride, const TG* __restrict__ gate, long long ldg, int heads, int dv, float eps) {
  const int t = blockIdx.x, h = blockIdx.y;
  const float* row = o + ((long long)t * heads + h) * dv;
  float ss = 0.f;
  for (int j = threadIdx.x; j < dv; j += kWave) ss += row[j] * row[j];
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)dv + eps);
  for (int j = threadIdx.x; j < dv; j += kWave) {
    const float g = ld(gate + (long long)t * ldg + h * dv + j);
    st(out + ((long long)t * heads + h) * dv + j,
       row[j] * inv * weight[h * weight_stride + j] * siluf_(g));
  }
}

}  // namespace

// ============================================================================ entry points
RLIS_API int rlis_shift_mix(void* out, const void* x, int dtype, const float* mu,
                            const float* state, long long state_stride, const int* seq_of_token,
                            const int* cu, const int* slots, int T, int W, int mixes,
                            hipStream_t stream) {
  RLIS_REQUIRE(T >= 0 && W > 0 && mixes > 0, "shift_mix: bad sizes T=%d W=%d mixes=%d", T, W, mixes);
  RLIS_REQUIRE(state_stride >= W, "shift_mix: the state is shorter than a row");
  if (T == 0) return 0;
  if (dtype == RLIS_F32)
    shift_mix_kernel<float><<<T, 256, 0, stream>>>((float*)out, (const float*)x, mu, state,
                                                   state_stride, seq_of_token, cu, slots, T, W,
                                                   mixes);
  else if (dtype == RLIS_BF16)
    shift_mix_kernel<bf16_t><<<T, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)x, mu, state,
                                                    state_stride, seq_of_token, cu, slots, T, W,
                                                    mixes);
  else
    RLIS_REQUIRE(false, "shift_mix: unknown dtype %d", dtype);
  RLIS_LAUNCH_CHECK("shift_mix");
  return 0;
}

RLIS_API int rlis_tail_update(float* state, long long state_stride, const void* x, int dtype,
                              long long ldx, int C, int R, const int* cu, const int* slots,
                              int num_seqs, hipStream_t stream) {
  RLIS_REQUIRE(C > 0 && R >= 0 && R <= 16, "tail_update: bad sizes C=%d rows=%d (at most 16)", C, R);
  RLIS_REQUIRE(state_stride >= (long long)C * R && ldx >= C, "tail_update: strides too short");
  RLIS_REQUIRE(num_seqs <= 65535, "tail_update: %d sequences, at most 65535", num_seqs);
  if (num_seqs <= 0 || R == 0) return 0;
  const dim3 grid(ceil_div(C, 256), num_seqs);
  if (dtype == RLIS_F32)
    tail_update_kernel<float><<<grid, 256, 0, stream>>>(state, state_stride, (const float*)x, ldx,
                                                        C, R, cu, slots);
  else if (dtype == RLIS_BF16)
    tail_update_kernel<bf16_t><<<grid, 256, 0, stream>>>(state, state_stride, (const bf16_t*)x,
                                                         ldx, C, R, cu, slots);
  else
    RLIS_REQUIRE(false, "tail_update: unknown dtype %d", dtype);
  RLIS_LAUNCH_CHECK("tail_update");
  return 0;
}

RLIS_API int rlis_causal_conv(float* out, const float* x, long long ldx, const float* taps, int C,
                              int K, const float* state, long long state_stride,
                              const int* seq_of_token, const int* cu, const int* slots, int T,
                              int unit_channels, int unit_group, int scaled_channels, float scale,
                              float unit_eps, int rest_group, hipStream_t stream) {
  RLIS_REQUIRE(T >= 0 && C > 0 && K >= 1 && K <= 16, "causal_conv: bad sizes T=%d C=%d taps=%d", T, C, K);
  RLIS_REQUIRE(ldx >= C && state_stride >= (long long)C * (K - 1), "causal_conv: strides too short");
  RLIS_REQUIRE(unit_channels >= 0 && unit_channels <= C && scaled_channels <= unit_channels,
               "causal_conv: bad channel ranges");
  RLIS_REQUIRE(unit_channels == 0 || (unit_group > 0 && unit_group <= 1024 &&
                                      unit_channels % unit_group == 0 &&
                                      scaled_channels % unit_group == 0),
               "causal_conv: unit groups of %d do not tile %d channels", unit_group, unit_channels);
  RLIS_REQUIRE(unit_channels == C || (rest_group > 0 && rest_group <= 1024),
               "causal_conv: bad group size %d for the other channels", rest_group);
  if (T == 0) return 0;
  const int groups = (unit_channels ? unit_channels / unit_group : 0) +
                     (unit_channels < C ? ceil_div(C - unit_channels, rest_group) : 0);
  RLIS_REQUIRE(groups <= 65535, "causal_conv: too many groups");
  causal_conv_kernel<<<dim3(T, groups), 256, 0, stream>>>(
      out, x, ldx, taps, C, K, state, state_stride, seq_of_token, cu, slots, unit_channels,
      unit_group, scaled_channels, scale, unit_eps, rest_group > 0 ? rest_group : 1);
  RLIS_LAUNCH_CHECK("causal_conv");
  return 0;
}

RLIS_API int rlis_delta_scan(float* out, long long ldo, const float* q, const float* k,
                             const float* v, long long ldqkv, const float* b_raw,
                             const float* a_raw, long long ldba, const float* a_log,
                             const float* dt_bias, float* state, long long state_stride,
                             const int* cu, const int* slots, int num_seqs, int heads,
                             int kv_heads, int dk, int dv, hipStream_t stream) {
  RLIS_REQUIRE(heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && dk > 0 && dv > 0,
               "delta_scan: bad sizes heads=%d kv_heads=%d dk=%d dv=%d", heads, kv_heads, dk, dv);
  RLIS_REQUIRE(dk <= 256, "delta_scan: %d key channels, at most 256", dk);
  RLIS_REQUIRE(state_stride >= (long long)heads * dk * dv, "delta_scan: the state is too short");
  RLIS_REQUIRE(heads <= 65535 && num_seqs <= 65535, "delta_scan: grid too large");
  if (num_seqs <= 0) return 0;
  const dim3 grid(ceil_div(dv, 4), heads, num_seqs);
#define LAUNCH(KR)                                                                            \
  delta_scan_kernel<KR><<<grid, 256, 0, stream>>>(out, ldo, q, k, v, ldqkv, b_raw, a_raw, ldba, \
                                                  a_log, dt_bias, state, state_stride, cu,    \
                                                  slots, heads, kv_heads, dk, dv)
  if (dk <= 64) LAUNCH(1);
  else if (dk <= 128) LAUNCH(2);
  else LAUNCH(4);
#undef LAUNCH
  RLIS_LAUNCH_CHECK("delta_scan");
  return 0;
}

RLIS_API int rlis_decay_scan(float* out, const float* r, const float* k, const float* v,
                             const float* z, long long ld, const float* w0, const float* bonus,
                             float* state, long long state_stride, const int* cu,
                             const int* slots, int num_seqs, int heads, int d,
                             hipStream_t stream) {
  RLIS_REQUIRE(heads > 0 && d > 0 && d <= 256, "decay_scan: bad sizes heads=%d d=%d (at most 256)",
               heads, d);
  RLIS_REQUIRE(ld >= (long long)heads * d, "decay_scan: rows shorter than heads x d");
  RLIS_REQUIRE(state_stride >= (long long)heads * d * d, "decay_scan: the state is too short");
  RLIS_REQUIRE(heads <= 65535 && num_seqs <= 65535, "decay_scan: grid too large");
  if (num_seqs <= 0) return 0;
  const dim3 grid(ceil_div(d, 4), heads, num_seqs);
#define LAUNCH(KR)                                                                           \
  decay_scan_kernel<KR><<<grid, 256, 0, stream>>>(out, r, k, v, z, ld, w0, bonus, state,     \
                                                  state_stride, cu, slots, heads, d)
  if (d <= 64) LAUNCH(1);
  else if (d <= 128) LAUNCH(2);
  else LAUNCH(4);
#undef LAUNCH
  RLIS_LAUNCH_CHECK("decay_scan");
  return 0;
}

RLIS_API int rlis_head_norm_gate(void* out, int out_dtype, const float* o, const float* weight,
                                 int weight_stride, const void* gate, int gate_dtype,
                                 long long ldg, int T, int heads, int dv, float eps,
                                 hipStream_t stream) {
  RLIS_REQUIRE(T >= 0 && heads > 0 && dv > 0 && heads <= 65535,
               "head_norm_gate: bad sizes T=%d heads=%d dv=%d", T, heads, dv);
  RLIS_REQUIRE(weight_stride == 0 || weight_stride == dv, "head_norm_gate: bad weight stride");
  if (T == 0) return 0;
  const dim3 grid(T, heads);
  const int key = gate_dtype * 2 + out_dtype;
#define CASE(k_, TG, TO)                                                                     \
  case k_:                                                                                   \
    head_norm_gate_kernel<TG, TO><<<grid, kWave, 0, stream>>>(                               \
        (TO*)out, o, weight, weight_stride, (const TG*)gate, ldg, heads, dv, eps);           \
    break;
  switch (key) {
    CASE(0, float, float)
    CASE(1, float, bf16_t)
    CASE(2, bf16_t, float)
    CASE(3, bf16_t, bf16_t)
    default:
      RLIS_REQUIRE(false, "head_norm_gate: unknown dtypes %d %d", gate_dtype, out_dtype);
  }
#undef CASE
  RLIS_LAUNCH_CHECK("head_norm_gate");
  return 0;
}
