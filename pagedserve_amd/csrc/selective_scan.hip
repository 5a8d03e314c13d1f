// A selective state-space mixer (Mamba): a short causal convolution per channel, then a
// recurrence whose state is a vector of `states` numbers per channel with a step size that
// depends on the token:
//
//   x_t   = silu(sum_j conv[c, j] u_(t - taps + 1 + j) + conv_bias[c])      (u: the raw inputs)
//   dt_t  = softplus(dt_bias[c] + sum_r low_t[r] w_dt[c, r])
//   S_t[c, n] = exp(dt_t A[c, n]) S_(t-1)[c, n] + dt_t x_t B_t[n],   A = -exp(A_log)
//   y_t[c] = (sum_n S_t[c, n] C_t[n] + D[c] x_t) * silu(z_t[c])
//
// Per request the slot keeps, for every channel, the `states` numbers of S and behind them the
// last taps - 1 raw inputs (oldest first): [slots, channels, states + taps - 1] float.  The
// step sizes, the decays, the state and the sums are 32-bit in both engine dtypes.
#include <math.h>

#include "common.h"
#include "pagedserve_hip.h"

__device__ inline float silu_f(float v) { return v / (1.0f + expf(-v)); }

// softplus(v) = max(v, 0) + log1p(exp(-|v|))
__device__ inline float softplus_f(float v) { return fmaxf(v, 0.f) + log1pf(expf(-fabsf(v))); }

// x[t, c] = silu(conv(u)[t, c]): a thread per (token, channel).  Inputs before the step's first
// token of the item come from the slot (zeros for a new request: the slot was cleared).
template <typename T>
__global__ __launch_bounds__(256) void conv_silu_kernel(
    const float* __restrict__ proj, int64_t ld, int u_col, const float* __restrict__ w,
    const float* __restrict__ bias, const float* __restrict__ state, int row, int tail,
    T* __restrict__ x, const int* __restrict__ tok_item, const int* __restrict__ cu_tokens,
    const int* __restrict__ slots, int channels, int taps) {
  const int t = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= channels) return;
  const int item = tok_item[t];
  const int first = cu_tokens[item];
  const float* kept = state + ((int64_t)slots[item] * channels + c) * row + tail;
  float sum = bias ? bias[c] : 0.f;
  for (int j = 0; j < taps; ++j) {
    const int back = taps - 1 - j;           // the input `back` tokens before this one
    const int local = (t - first) - back;    // its place among the item's tokens of this step
    const float u = local >= 0 ? proj[(int64_t)(t - back) * ld + u_col + c]
                               : kept[taps - 1 + local];
    sum = fmaf(w[(int64_t)c * taps + j], u, sum);
  }
  x[(int64_t)t * channels + c] = from_float<T>(silu_f(sum));
}

// dt[t, c] = softplus(bias[c] + sum_r low[t, r] w[c, r]).
template <typename T>
__global__ __launch_bounds__(256) void step_size_kernel(
    const float* __restrict__ low, int64_t ld, int rank, const T* __restrict__ w,
    const float* __restrict__ bias, float* __restrict__ dt, int channels) {
  extern __shared__ float s_low[];
  const int t = blockIdx.x;
  for (int r = threadIdx.x; r < rank; r += blockDim.x) s_low[r] = low[(int64_t)t * ld + r];
  __syncthreads();
  for (int c = threadIdx.x; c < channels; c += blockDim.x) {
    float z = bias ? bias[c] : 0.f;
    const T* w_row = w + (int64_t)c * rank;
    for (int r = 0; r < rank; ++r) z = fmaf(s_low[r], to_float<T>(w_row[r]), z);
    dt[(int64_t)t * channels + c] = softplus_f(z);
  }
}

// The recurrence.  A block of one wave owns 64 / LPC channels of one item and walks the item's
// tokens in order; a channel's states are dealt to LPC neighbouring lanes (state n to lane
// n % LPC), SPL to a lane, in registers.  B and C of SS_CHUNK tokens wait in LDS.  At the end
// the states and the last taps - 1 raw inputs go back to the slot.
#define SS_CHUNK 16
template <typename T, int LPC, int SPL>
__global__ __launch_bounds__(64) void selective_scan_kernel(
    const T* __restrict__ x, const float* __restrict__ dt, const float* __restrict__ bc, int64_t bc_ld,
    int b_col, int c_col, const float* __restrict__ proj, int64_t ld, int u_col, int z_col,
    const float* __restrict__ a_log, const float* __restrict__ skip, float* __restrict__ state,
    T* __restrict__ y, const int* __restrict__ cu_tokens, const int* __restrict__ slots,
    int channels, int states, int taps) {
  constexpr int CPB = 64 / LPC;
  extern __shared__ float s_bc[];            // [SS_CHUNK][2 * states]
  const int item = blockIdx.x;
  const int lane = threadIdx.x;
  const int part = lane % LPC;
  const int c = blockIdx.y * CPB + lane / LPC;
  const bool live = c < channels;
  const int cc = live ? c : channels - 1;
  const int t0 = cu_tokens[item], t1 = cu_tokens[item + 1];
  const int row = states + taps - 1;
  float* mine = state + ((int64_t)slots[item] * channels + cc) * row;
  float S[SPL], A[SPL];
#pragma unroll
  for (int i = 0; i < SPL; ++i) {
    const int n = part + i * LPC;
    S[i] = n < states ? mine[n] : 0.f;
    A[i] = n < states ? -expf(a_log[(int64_t)cc * states + n]) : 0.f;
  }
  const float d_skip = skip[cc];
  for (int base = t0; base < t1; base += SS_CHUNK) {
    const int count = (t1 - base) < SS_CHUNK ? (t1 - base) : SS_CHUNK;
    __syncthreads();
    for (int idx = lane; idx < count * 2 * states; idx += 64) {
      const int tt = idx / (2 * states);
      const int n = idx - tt * 2 * states;
      s_bc[idx] = bc[(int64_t)(base + tt) * bc_ld + (n < states ? b_col + n : c_col + n - states)];
    }
    __syncthreads();
    for (int tt = 0; tt < count; ++tt) {
      const int64_t t = base + tt;
      const float step = dt[t * channels + cc];
      const float xv = to_float<T>(x[t * channels + cc]);
      const float* b_row = s_bc + tt * 2 * states;
      const float* c_row = b_row + states;
      const float sx = step * xv;
      float sum = 0.f;
#pragma unroll
      for (int i = 0; i < SPL; ++i) {
        const int n = part + i * LPC;
        if (n < states) {
          S[i] = fmaf(expf(step * A[i]), S[i], sx * b_row[n]);
          sum = fmaf(S[i], c_row[n], sum);
        }
      }
      sum = lanes_sum<LPC>(sum);
      if (part == 0 && live) {
        const float z = proj[t * ld + z_col + c];
        y[t * channels + c] = from_float<T>(fmaf(d_skip, xv, sum) * silu_f(z));
      }
    }
  }
  if (!live) return;
#pragma unroll
  for (int i = 0; i < SPL; ++i) {
    const int n = part + i * LPC;
    if (n < states) mine[n] = S[i];
  }
  if (part == 0 && t1 > t0) {
    // the last taps - 1 raw inputs of (what the slot kept, then this step's), oldest first
    const int count = t1 - t0;
    float* kept = mine + states;
    for (int j = 0; j < taps - 1; ++j) {
      const int local = count - (taps - 1) + j;      // place among this step's tokens
      // (ascending j reads kept[j + count] with count >= 1: never a place already written)
      kept[j] = local >= 0 ? proj[(int64_t)(t0 + local) * ld + u_col + c] : kept[j + count];
    }
  }
}

extern "C" int ps_conv_silu(const float* proj, int64_t ld, int u_col, const float* w,
                            const float* bias, const float* state, int states, void* x,
                            const int* tok_item, const int* cu_tokens, const int* slots, int tokens,
                            int channels, int taps, int dtype, void* stream) {
  PS_REQUIRE(tokens >= 0 && channels > 0 && taps >= 1 && taps <= 64 && states >= 0,
             "ps_conv_silu: bad sizes");
  PS_REQUIRE(dtype == PS_F32 || dtype == PS_BF16, "ps_conv_silu: unknown dtype %d", dtype);
  if (tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid(tokens, (channels + 255) / 256);
  const int row = states + taps - 1;
  if (dtype == PS_F32)
    hipLaunchKernelGGL(conv_silu_kernel<float>, grid, dim3(256), 0, s, proj, ld, u_col, w, bias, state,
                       row, states, (float*)x, tok_item, cu_tokens, slots, channels, taps);
  else
    hipLaunchKernelGGL(conv_silu_kernel<bf16_t>, grid, dim3(256), 0, s, proj, ld, u_col, w, bias, state,
                       row, states, (bf16_t*)x, tok_item, cu_tokens, slots, channels, taps);
  PS_CHECK_LAUNCH("ps_conv_silu");
  return 0;
}

extern "C" int ps_step_size(const float* low, int64_t ld, int rank, const void* w, const float* bias,
                            float* dt, int tokens, int channels, int dtype, void* stream) {
  PS_REQUIRE(tokens >= 0 && rank > 0 && rank <= 8192 && channels > 0, "ps_step_size: bad sizes");
  PS_REQUIRE(dtype == PS_F32 || dtype == PS_BF16, "ps_step_size: unknown dtype %d", dtype);
  if (tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const size_t lds = (size_t)rank * sizeof(float);
  if (dtype == PS_F32)
    hipLaunchKernelGGL(step_size_kernel<float>, dim3(tokens), dim3(256), lds, s, low, ld, rank,
                       (const float*)w, bias, dt, channels);
  else
    hipLaunchKernelGGL(step_size_kernel<bf16_t>, dim3(tokens), dim3(256), lds, s, low, ld, rank,
                       (const bf16_t*)w, bias, dt, channels);
  PS_CHECK_LAUNCH("ps_step_size");
  return 0;
}

extern "C" int ps_selective_scan(const void* x, const float* dt, const float* bc, int64_t bc_ld,
                                 int b_col, int c_col, const float* proj, int64_t ld, int u_col,
                                 int z_col, const float* a_log, const float* skip, float* state,
                                 void* y, const int* cu_tokens, const int* slots, int items,
                                 int channels, int states, int taps, int dtype, void* stream) {
  PS_REQUIRE(items >= 0 && channels > 0 && states > 0 && taps >= 1, "ps_selective_scan: bad sizes");
  PS_REQUIRE(states <= 256, "ps_selective_scan: %d states per channel, at most 256", states);
  PS_REQUIRE(dtype == PS_F32 || dtype == PS_BF16, "ps_selective_scan: unknown dtype %d", dtype);
  if (items == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const size_t lds = (size_t)SS_CHUNK * 2 * states * sizeof(float);
#define PS_LAUNCH_SS_T(T, LPC, SPL)                                                               \
  hipLaunchKernelGGL((selective_scan_kernel<T, LPC, SPL>),                                        \
                     dim3(items, (channels + 64 / LPC - 1) / (64 / LPC)), dim3(64), lds, s,       \
                     (const T*)x, dt, bc, bc_ld, b_col, c_col, proj, ld, u_col, z_col, a_log, skip, \
                     state, (T*)y, cu_tokens, slots, channels, states, taps)
#define PS_LAUNCH_SS(LPC, SPL)                  \
  do {                                          \
    if (dtype == PS_F32) {                      \
      PS_LAUNCH_SS_T(float, LPC, SPL);          \
    } else {                                    \
      PS_LAUNCH_SS_T(bf16_t, LPC, SPL);         \
    }                                           \
  } while (0)
  // a lane keeps at most 16 states; few states are dealt to few lanes
  if (states <= 4) PS_LAUNCH_SS(1, 4);
  else if (states <= 8) PS_LAUNCH_SS(2, 4);
  else if (states <= 16) PS_LAUNCH_SS(4, 4);
  else if (states <= 32) PS_LAUNCH_SS(4, 8);
  else if (states <= 64) PS_LAUNCH_SS(8, 8);
  else if (states <= 128) PS_LAUNCH_SS(16, 8);
  else PS_LAUNCH_SS(16, 16);
#undef PS_LAUNCH_SS
#undef PS_LAUNCH_SS_T
  PS_CHECK_LAUNCH("ps_selective_scan");
  return 0;
}
