// Mixture of experts: the router, and the experts' products for rows that are dealt to them
// token by token.
//
//   z = W_r x (32-bit),  s = softmax(z) over all experts
//   the experts form `groups` equal groups of neighbours; a group's score is its largest s; only
//   experts of the `keep` best groups may be chosen; the `top` largest s among them are, with
//   the weights s * scale (not renormalised)
//   out = sum over the chosen e of weight_e * W_down,e (silu(W_gate,e x) * (W_up,e x))
#include <math.h>

#include "common.h"
#include "pagedserve_hip.h"

#define MOE_MAX_EXPERTS 1024

// A block of one wave per token.  The logits are sums over the width dealt to the lanes; the
// choice itself is a few dozen comparisons and is left to lane 0.
template <typename T>
__global__ __launch_bounds__(64) void moe_route_kernel(
    const T* __restrict__ x, int64_t x_ld, const float* __restrict__ w, int width, int experts,
    int groups, int keep, int top, float scale, int* __restrict__ ids, float* __restrict__ weights) {
  __shared__ float s_score[MOE_MAX_EXPERTS];
  __shared__ unsigned char s_open[MOE_MAX_EXPERTS];
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x;
  const T* row = x + t * x_ld;
  for (int e = 0; e < experts; ++e) {
    const float* w_row = w + (int64_t)e * width;
    float sum = 0.f;
    for (int d = lane; d < width; d += 64) sum = fmaf(to_float<T>(row[d]), w_row[d], sum);
    sum = wave_sum(sum);
    if (lane == 0) s_score[e] = sum;
  }
  __syncthreads();
  if (lane != 0) return;
  float top_z = -INFINITY;
  for (int e = 0; e < experts; ++e) top_z = fmaxf(top_z, s_score[e]);
  float total = 0.f;
  for (int e = 0; e < experts; ++e) {
    s_score[e] = expf(s_score[e] - top_z);
    total += s_score[e];
  }
  const float inv = 1.0f / total;
  for (int e = 0; e < experts; ++e) {
    s_score[e] *= inv;
    s_open[e] = groups <= 1 || keep >= groups;
  }
  if (groups > 1 && keep < groups) {
    // the best groups one after the other; a group that was taken has its experts open
    const int size = experts / groups;
    for (int round = 0; round < keep; ++round) {
      int best = -1;
      float best_score = -INFINITY;
      for (int g = 0; g < groups; ++g) {
        if (s_open[g * size]) continue;
        float score = -INFINITY;
        for (int e = g * size; e < (g + 1) * size; ++e) score = fmaxf(score, s_score[e]);
        if (score > best_score) {
          best_score = score;
          best = g;
        }
      }
      if (best < 0) best = 0;      // (scores that are no numbers: any choice, but a valid one)
      for (int e = best * size; e < (best + 1) * size; ++e) s_open[e] = 1;
    }
  }
  for (int j = 0; j < top; ++j) {
    int best = -1;
    float best_score = -INFINITY;
    for (int e = 0; e < experts; ++e) {
      if (s_open[e] == 1 && s_score[e] > best_score) {
        best_score = s_score[e];
        best = e;
      }
    }
    if (best < 0) {       // (scores that are no numbers: any choice, but a valid one)
      best = 0;
      best_score = 0.f;
    }
    s_open[best] = 2;     // chosen: not again
    ids[t * top + j] = best;
    weights[t * top + j] = best_score * scale;
  }
}

// hidden[(t, j), c] = silu(W_gate,e[c] . x_t) * (W_up,e[c] . x_t) for e = ids[t, j].  The
// experts' first matrices lie one behind the other, [experts][gate rows | up rows][width].
// A block of four waves per (token, choice) and 4 * ROWS hidden columns; the lanes share a dot
// product's width.
template <typename T, int ROWS>
__global__ __launch_bounds__(256) void moe_hidden_kernel(
    const T* __restrict__ x, int64_t x_ld, const T* __restrict__ w1, const int* __restrict__ ids,
    T* __restrict__ hidden, int width, int inner) {
  extern __shared__ float s_x[];
  // (blockIdx.x: the token, blockIdx.z: which of its choices)
  const int64_t row_index = (int64_t)blockIdx.x * gridDim.z + blockIdx.z;
  const int e = ids[row_index];
  const T* x_row = x + (int64_t)blockIdx.x * x_ld;
  for (int d = threadIdx.x; d < width; d += 256) s_x[d] = to_float<T>(x_row[d]);
  __syncthreads();
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const T* base = w1 + (int64_t)e * 2 * inner * width;
  const int first = (blockIdx.y * 4 + wave) * ROWS;
  for (int r = 0; r < ROWS; ++r) {
    const int c = first + r;
    if (c >= inner) break;
    const T* g_row = base + (int64_t)c * width;
    const T* u_row = base + (int64_t)(inner + c) * width;
    float g = 0.f, u = 0.f;
    for (int d = lane; d < width; d += 64) {
      g = fmaf(to_float<T>(g_row[d]), s_x[d], g);
      u = fmaf(to_float<T>(u_row[d]), s_x[d], u);
    }
    g = wave_sum(g);
    u = wave_sum(u);
    if (lane == 0) hidden[row_index * inner + c] = from_float<T>(g / (1.0f + expf(-g)) * u);
  }
}

// y[t, d] += sum_j weights[t, j] * (W_down,e_j[d] . hidden[(t, j)]).  A block of four waves per
// token and 4 * ROWS output columns.
template <typename T, int ROWS>
__global__ __launch_bounds__(256) void moe_down_kernel(
    const T* __restrict__ hidden, const T* __restrict__ w2, const int* __restrict__ ids,
    const float* __restrict__ weights, float* __restrict__ y, int width, int inner, int top) {
  extern __shared__ float s_h[];        // [top][inner]
  const int64_t t = blockIdx.x;
  for (int i = threadIdx.x; i < top * inner; i += 256)
    s_h[i] = to_float<T>(hidden[t * top * inner + i]);
  __syncthreads();
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int first = (blockIdx.y * 4 + wave) * ROWS;
  for (int r = 0; r < ROWS; ++r) {
    const int d = first + r;
    if (d >= width) break;
    float total = 0.f;
    for (int j = 0; j < top; ++j) {
      const int e = ids[t * top + j];
      const T* w_row = w2 + ((int64_t)e * width + d) * inner;
      float sum = 0.f;
      for (int c = lane; c < inner; c += 64) sum = fmaf(to_float<T>(w_row[c]), s_h[j * inner + c], sum);
      total = fmaf(weights[t * top + j], wave_sum(sum), total);
    }
    if (lane == 0) y[t * width + d] += total;
  }
}

extern "C" int ps_moe_route(const void* x, int64_t x_ld, const float* w, int tokens, int width,
                            int experts, int groups, int keep, int top, float scale, int* ids,
                            float* weights, int dtype, void* stream) {
  PS_REQUIRE(tokens >= 0 && width > 0 && experts > 0 && experts <= MOE_MAX_EXPERTS,
             "ps_moe_route: %d experts, at most %d", experts, MOE_MAX_EXPERTS);
  PS_REQUIRE(groups >= 1 && experts % groups == 0 && keep >= 1 && keep <= groups,
             "ps_moe_route: %d groups (keep %d) do not divide %d experts", groups, keep, experts);
  PS_REQUIRE(top >= 1 && top <= (experts / groups) * keep,
             "ps_moe_route: %d experts per token, %d may be chosen", top, (experts / groups) * keep);
  PS_REQUIRE(dtype == PS_F32 || dtype == PS_BF16, "ps_moe_route: unknown dtype %d", dtype);
  if (tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == PS_F32)
    hipLaunchKernelGGL(moe_route_kernel<float>, dim3(tokens), dim3(64), 0, s, (const float*)x, x_ld, w,
                       width, experts, groups, keep, top, scale, ids, weights);
  else
    hipLaunchKernelGGL(moe_route_kernel<bf16_t>, dim3(tokens), dim3(64), 0, s, (const bf16_t*)x, x_ld,
                       w, width, experts, groups, keep, top, scale, ids, weights);
  PS_CHECK_LAUNCH("ps_moe_route");
  return 0;
}

extern "C" int ps_moe_experts(const void* x, int64_t x_ld, const void* w1, const void* w2,
                              const int* ids, const float* weights, void* hidden, float* y,
                              int tokens, int width, int inner, int top, int dtype, void* stream) {
  PS_REQUIRE(tokens >= 0 && width > 0 && inner > 0 && top > 0 && top <= 65535,
             "ps_moe_experts: bad sizes");
  PS_REQUIRE((size_t)width * 4 <= 64 * 1024 && (size_t)top * inner * 4 <= 64 * 1024,
             "ps_moe_experts: width %d or %d x %d hidden columns do not fit LDS", width, top, inner);
  PS_REQUIRE(dtype == PS_F32 || dtype == PS_BF16, "ps_moe_experts: unknown dtype %d", dtype);
  if (tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  constexpr int ROWS = 4;
  const dim3 grid1(tokens, (inner + 4 * ROWS - 1) / (4 * ROWS), top);
  const dim3 grid2(tokens, (width + 4 * ROWS - 1) / (4 * ROWS));
  if (dtype == PS_F32) {
    hipLaunchKernelGGL((moe_hidden_kernel<float, ROWS>), grid1, dim3(256), (size_t)width * 4, s,
                       (const float*)x, x_ld, (const float*)w1, ids, (float*)hidden, width, inner);
    hipLaunchKernelGGL((moe_down_kernel<float, ROWS>), grid2, dim3(256), (size_t)top * inner * 4, s,
                       (const float*)hidden, (const float*)w2, ids, weights, y, width, inner, top);
  } else {
    hipLaunchKernelGGL((moe_hidden_kernel<bf16_t, ROWS>), grid1, dim3(256), (size_t)width * 4, s,
                       (const bf16_t*)x, x_ld, (const bf16_t*)w1, ids, (bf16_t*)hidden, width, inner);
    hipLaunchKernelGGL((moe_down_kernel<bf16_t, ROWS>), grid2, dim3(256), (size_t)top * inner * 4, s,
                       (const bf16_t*)hidden, (const bf16_t*)w2, ids, weights, y, width, inner, top);
  }
  PS_CHECK_LAUNCH("ps_moe_experts");
  return 0;
}
