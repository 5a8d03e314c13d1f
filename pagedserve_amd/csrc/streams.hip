// Several copies of the residual stream ("hyper-connections"): X is [tokens, streams, width]
// in float.  A sublayer reads a weighted sum of the copies and writes its result y back into
// every copy while the copies are mixed with each other:
//
//   read:   u = sum_s in[s] X_s,  normed = u / sqrt(mean(u^2) + eps) * gamma
//   write:  X'_t = sum_s mix[s, t] X_s + out[t] y          (all t from the old copies)
//
// One kernel does a write, a read, or a write followed by the read of the next sublayer
// (the copies then make one trip through memory for both), and clears the buffer that the
// next sublayer's products add their result into.  Everything is 32-bit.
#include <math.h>

#include "common.h"
#include "pagedserve_hip.h"

#define HS_MAX_STREAMS 8
#define HS_THREADS 1024   // at most; a launch takes as many as the row has columns, so that a
                          // row of up to 1,024 columns is one round of loads

// STREAMS is a template argument so that every loop over the copies is unrolled and a
// thread's loads of one column (the copies and y) leave together, without a branch between
// them.  u waits in LDS (width floats) for the row's sum of squares.
template <typename TOut, int STREAMS>
__global__ __launch_bounds__(HS_THREADS) void hyper_step_kernel(
    float* __restrict__ X, const float* __restrict__ y, const float* __restrict__ mix,
    const float* __restrict__ out_w, const float* __restrict__ in_w,
    const float* __restrict__ gamma, float eps, TOut* __restrict__ normed,
    float* __restrict__ zero, int width) {
  extern __shared__ float s_u[];
  __shared__ float red[16];
  const int t = blockIdx.x;
  const bool writes = y != nullptr;
  const bool reads = normed != nullptr;
  // the few weights: every thread reads them itself (the same addresses in all lanes: scalar loads)
  float w_mix[STREAMS][STREAMS], w_out[STREAMS], w_in[STREAMS];
#pragma unroll
  for (int a = 0; a < STREAMS; ++a) {
    w_out[a] = writes ? out_w[a] : 0.f;
    w_in[a] = reads ? in_w[a] : 0.f;
#pragma unroll
    for (int b = 0; b < STREAMS; ++b) w_mix[a][b] = writes ? mix[a * STREAMS + b] : (a == b ? 1.f : 0.f);
  }
  float sumsq = 0.f;
  float* row = X + (int64_t)t * STREAMS * width;
  // what one column needs; returns its u
  auto column = [&](const int col) -> float {
    float x[STREAMS];
#pragma unroll
    for (int s = 0; s < STREAMS; ++s) x[s] = row[(int64_t)s * width + col];
    if (writes) {
      const float yv = y[(int64_t)t * width + col];
      float nx[STREAMS];
#pragma unroll
      for (int to = 0; to < STREAMS; ++to) {
        float acc = 0.f;
#pragma unroll
        for (int from = 0; from < STREAMS; ++from) acc = fmaf(w_mix[from][to], x[from], acc);
        nx[to] = fmaf(w_out[to], yv, acc);
        row[(int64_t)to * width + col] = nx[to];
      }
#pragma unroll
      for (int s = 0; s < STREAMS; ++s) x[s] = nx[s];
    }
    float uu = 0.f;
#pragma unroll
    for (int s = 0; s < STREAMS; ++s) uu = fmaf(w_in[s], x[s], uu);
    if (zero != nullptr) zero[(int64_t)t * width + col] = 0.f;
    return uu;
  };
  if (width <= (int)blockDim.x) {
    // a thread per column: u and the norm's scale stay in registers, and the scale's load
    // leaves with the others instead of behind the sum of squares
    const int col = threadIdx.x;
    const bool active = col < width;
    const float g = (reads && active) ? gamma[col] : 0.f;
    const float uu = active ? column(col) : 0.f;
    if (!reads) return;
    const float total = block_sum(uu * uu, red);
    const float inv = 1.0f / sqrtf(total / (float)width + eps);
    if (active) normed[(int64_t)t * width + col] = from_float<TOut>(uu * inv * g);
    return;
  }
  for (int col = threadIdx.x; col < width; col += blockDim.x) {
    const float uu = column(col);
    if (reads) {
      s_u[col] = uu;
      sumsq = fmaf(uu, uu, sumsq);
    }
  }
  if (!reads) return;
  const float total = block_sum(sumsq, red);
  const float inv = 1.0f / sqrtf(total / (float)width + eps);
  // (a thread reads back the columns that it wrote itself)
  for (int col = threadIdx.x; col < width; col += blockDim.x)
    normed[(int64_t)t * width + col] = from_float<TOut>(s_u[col] * inv * gamma[col]);
}

extern "C" int ps_hyper_step(float* x, const float* y, const float* mix, const float* out_w,
                             const float* in_w, const float* gamma, float eps, void* normed,
                             float* zero, int tokens, int width, int streams, int out_dtype,
                             void* stream) {
  PS_REQUIRE(tokens >= 0 && width > 0, "ps_hyper_step: bad sizes");
  PS_REQUIRE(streams >= 1 && streams <= HS_MAX_STREAMS, "ps_hyper_step: %d streams, the kernel takes 1..%d",
             streams, HS_MAX_STREAMS);
  PS_REQUIRE(width <= 15360, "ps_hyper_step: width %d above 15360 (a row's sums wait in LDS)", width);
  PS_REQUIRE(y == nullptr || (mix != nullptr && out_w != nullptr), "ps_hyper_step: a write needs mix and out weights");
  PS_REQUIRE(normed == nullptr || (in_w != nullptr && gamma != nullptr && eps > 0.f),
             "ps_hyper_step: a read needs in weights, gamma and a positive eps");
  PS_REQUIRE(out_dtype == PS_F32 || out_dtype == PS_BF16, "ps_hyper_step: unknown dtype %d", out_dtype);
  if (tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const size_t lds = normed != nullptr ? (size_t)width * sizeof(float) : 0;
  // few rows wait for their trips to memory: a thread per column; many rows fill the chip
  // anyway and run faster as blocks of four waves that walk their row
  int threads = width >= HS_THREADS ? HS_THREADS : (width + 63) / 64 * 64;
  if (tokens > 256 && threads > 256) threads = 256;
#define PS_LAUNCH_HS(TOut, S)                                                                     \
  hipLaunchKernelGGL((hyper_step_kernel<TOut, S>), dim3(tokens), dim3(threads), lds, s, x, y,     \
                     mix, out_w, in_w, gamma, eps, (TOut*)normed, zero, width)
#define PS_LAUNCH_HS_T(TOut)                         \
  switch (streams) {                                 \
    case 1: PS_LAUNCH_HS(TOut, 1); break;            \
    case 2: PS_LAUNCH_HS(TOut, 2); break;            \
    case 3: PS_LAUNCH_HS(TOut, 3); break;            \
    case 4: PS_LAUNCH_HS(TOut, 4); break;            \
    case 5: PS_LAUNCH_HS(TOut, 5); break;            \
    case 6: PS_LAUNCH_HS(TOut, 6); break;            \
    case 7: PS_LAUNCH_HS(TOut, 7); break;            \
    default: PS_LAUNCH_HS(TOut, 8); break;           \
  }
  if (out_dtype == PS_F32) {
    PS_LAUNCH_HS_T(float)
  } else {
    PS_LAUNCH_HS_T(bf16_t)
  }
#undef PS_LAUNCH_HS_T
#undef PS_LAUNCH_HS
  PS_CHECK_LAUNCH("ps_hyper_step");
  return 0;
}

// X[t, s, :] = e[t, :] for every copy s.
__global__ void streams_expand_kernel(const float* __restrict__ e, float* __restrict__ X,
                                      int width, int streams) {
  const int t = blockIdx.x;
  for (int col = threadIdx.x; col < width; col += blockDim.x) {
    const float v = e[(int64_t)t * width + col];
    for (int s = 0; s < streams; ++s) X[((int64_t)t * streams + s) * width + col] = v;
  }
}

extern "C" int ps_streams_expand(const float* e, float* x, int tokens, int width, int streams,
                                 void* stream) {
  PS_REQUIRE(tokens >= 0 && width > 0 && streams > 0, "ps_streams_expand: bad sizes");
  if (tokens == 0) return 0;
  hipLaunchKernelGGL(streams_expand_kernel, dim3(tokens), dim3(width >= 256 ? 256 : 64), 0,
                     (hipStream_t)stream, e, x, width, streams);
  PS_CHECK_LAUNCH("ps_streams_expand");
  return 0;
}

// out[r, :] = sum_s X[rows ? rows[r] : r, s, :].
__global__ void streams_collapse_kernel(const float* __restrict__ X, const int* __restrict__ rows,
                                        float* __restrict__ out, int width, int streams) {
  const int r = blockIdx.x;
  const int t = rows ? rows[r] : r;
  for (int col = threadIdx.x; col < width; col += blockDim.x) {
    float v = 0.f;
    for (int s = 0; s < streams; ++s) v += X[((int64_t)t * streams + s) * width + col];
    out[(int64_t)r * width + col] = v;
  }
}

extern "C" int ps_streams_collapse(const float* x, const int* rows, float* out, int n_rows,
                                   int width, int streams, void* stream) {
  PS_REQUIRE(n_rows >= 0 && width > 0 && streams > 0, "ps_streams_collapse: bad sizes");
  if (n_rows == 0) return 0;
  hipLaunchKernelGGL(streams_collapse_kernel, dim3(n_rows), dim3(width >= 256 ? 256 : 64), 0,
                     (hipStream_t)stream, x, rows, out, width, streams);
  PS_CHECK_LAUNCH("ps_streams_collapse");
  return 0;
}
