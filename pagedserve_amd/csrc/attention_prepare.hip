// Between the projection of an attention layer and the attention itself, one launch, a block
// per token: the float columns [q | k | v] of the projection become
//
//   * queries and keys normed over the WHOLE projection (all heads at once) with a weight per
//     column:  x / sqrt(mean(x^2) + eps) * w          (optional),
//   * rotated by the token's position on the first `rot_dims` dimensions of every head,
//     dimension 2i paired with 2i+1:  (a, b) -> (a cos t - b sin t, b cos t + a sin t) with
//     t = position * freqs[i]                          (optional),
//   * values mixed with the values that an earlier layer left for the same token:
//     v <- (1 - lambda) v + lambda v_first             (v_mode 2; v_mode 1 leaves them there),
//
// and the keys and values go straight into their cache pages while the queries are written in
// the storage type.  Heads are stored `cache_dim` wide (>= the key and the value head size,
// zeros behind), the one head size that the attention kernels then see for all three.
// Norm statistics, angles and the mixing are 32-bit.
#include <math.h>

#include "common.h"
#include "pagedserve_hip.h"

template <typename T>
__global__ __launch_bounds__(1024) void attention_prepare_kernel(
    const float* __restrict__ proj, int64_t ld, int q_col, int k_col, int v_col,
    T* __restrict__ q_out, int64_t q_stride, T* __restrict__ k_pool, T* __restrict__ v_pool,
    const float* __restrict__ q_gamma, const float* __restrict__ k_gamma, float eps,
    const float* __restrict__ freqs, int rot_dims, T* __restrict__ v_first,
    const float* __restrict__ v_lambda, int v_mode, const int* __restrict__ tok_item,
    const int* __restrict__ tok_pos, const int* __restrict__ tables, int table_width, int heads,
    int kv_heads, int key_dim, int value_dim, int cache_dim, int page_size, int num_pages) {
  __shared__ float red[2][16];
  __shared__ float s_cos[128], s_sin[128];   // the token's angles, one per rotated pair of a head
  const int t = blockIdx.x;
  const float* row = proj + (int64_t)t * ld;
  const int pos = tok_pos[t];
  const int q_cols = heads * key_dim, k_cols = kv_heads * key_dim;
  const int logical = pos / page_size;
  int page = -1;
  if (logical < table_width) page = tables[(int64_t)tok_item[t] * table_width + logical];
  const bool stored = page >= 0 && page < num_pages;
  const int offset = pos - logical * page_size;
  const int half = cache_dim / 2;   // cache_dim is even
  // Queries and keys, a pair of neighbouring dimensions per thread and turn.  A pair's values
  // and weights do not wait for the norms: a thread loads its first pair
  // before the block meets for the sums of squares (which the same values feed), so that a
  // step of few tokens makes one trip to memory; further pairs of a thread are read again.
  const int q_pairs = heads * half, k_pairs = kv_heads * half;
  struct Pair {
    float a, b, wa, wb;
    int head, d0;
    bool is_q;
  };
  auto load_pair = [&](const int i) -> Pair {
    Pair p;
    p.is_q = i < q_pairs;
    const int j = p.is_q ? i : i - q_pairs;
    p.head = j / half;
    p.d0 = (j - p.head * half) * 2;
    const int src = (p.is_q ? q_col : k_col) + p.head * key_dim + p.d0;
    const float* gamma = p.is_q ? q_gamma : k_gamma;
    p.a = p.d0 < key_dim ? row[src] : 0.f;
    p.b = p.d0 + 1 < key_dim ? row[src + 1] : 0.f;
    p.wa = (gamma && p.d0 < key_dim) ? gamma[p.head * key_dim + p.d0] : 1.f;
    p.wb = (gamma && p.d0 + 1 < key_dim) ? gamma[p.head * key_dim + p.d0 + 1] : 1.f;
    return p;
  };
  const int pairs = q_pairs + k_pairs;
  // every head turns by the same angles: they are worked out once per token, not once per head
  for (int i = threadIdx.x; i < rot_dims / 2; i += blockDim.x) sincosf((float)pos * freqs[i], &s_sin[i], &s_cos[i]);
  const bool has_first = (int)threadIdx.x < pairs;
  Pair first = {};
  if (has_first) first = load_pair(threadIdx.x);
  float q_inv = 1.f, k_inv = 1.f;
  if (q_gamma != nullptr || k_gamma != nullptr) {
    float q_sum = 0.f, k_sum = 0.f;
    if (has_first) {
      const float sq = first.a * first.a + first.b * first.b;
      if (first.is_q) q_sum = sq; else k_sum = sq;
    }
    for (int i = threadIdx.x + blockDim.x; i < pairs; i += blockDim.x) {
      const Pair p = load_pair(i);
      const float sq = p.a * p.a + p.b * p.b;
      if (p.is_q) q_sum += sq; else k_sum += sq;
    }
    q_sum = wave_sum(q_sum);
    k_sum = wave_sum(k_sum);
    const int wave = threadIdx.x >> 6;
    const int waves = (blockDim.x + 63) >> 6;
    if ((threadIdx.x & 63) == 0) {
      red[0][wave] = q_sum;
      red[1][wave] = k_sum;
    }
    __syncthreads();
    q_sum = 0.f;
    k_sum = 0.f;
    for (int w = 0; w < waves; ++w) {
      q_sum += red[0][w];
      k_sum += red[1][w];
    }
    if (q_gamma != nullptr) q_inv = 1.0f / sqrtf(q_sum / (float)q_cols + eps);
    if (k_gamma != nullptr) k_inv = 1.0f / sqrtf(k_sum / (float)k_cols + eps);
  } else {
    __syncthreads();      // the angles
  }
  for (int i = threadIdx.x; i < pairs; i += blockDim.x) {
    const Pair p = i == (int)threadIdx.x ? first : load_pair(i);
    const float inv = p.is_q ? q_inv : k_inv;
    const float a = p.a * inv * p.wa, b = p.b * inv * p.wb;
    const bool turned = p.d0 + 1 < rot_dims;
    const float cs = turned ? s_cos[p.d0 >> 1] : 1.f, sn = turned ? s_sin[p.d0 >> 1] : 0.f;
    const float ra = a * cs - b * sn;
    const float rb = b * cs + a * sn;
    if (p.is_q) {
      T* dst = q_out + (int64_t)t * q_stride + (int64_t)p.head * cache_dim + p.d0;
      dst[0] = from_float<T>(ra);
      dst[1] = from_float<T>(rb);
    } else if (stored) {
      T* dst = k_pool + (((int64_t)page * kv_heads + p.head) * page_size + offset) * cache_dim + p.d0;
      dst[0] = from_float<T>(ra);
      dst[1] = from_float<T>(rb);
    }
  }
  const float lambda = v_mode == 2 ? v_lambda[0] : 0.f;
  for (int i = threadIdx.x; i < kv_heads * cache_dim; i += blockDim.x) {
    const int head = i / cache_dim;
    const int d = i - head * cache_dim;
    float v = 0.f;
    if (d < value_dim) {
      v = row[v_col + head * value_dim + d];
      const int64_t at = ((int64_t)t * kv_heads + head) * value_dim + d;
      if (v_mode == 1) v_first[at] = from_float<T>(v);
      if (v_mode == 2) v = (1.f - lambda) * v + lambda * to_float<T>(v_first[at]);
    }
    if (stored)
      v_pool[(((int64_t)page * kv_heads + head) * page_size + offset) * cache_dim + d] = from_float<T>(v);
  }
}

extern "C" int ps_attention_prepare(const float* proj, int64_t ld, int q_col, int k_col, int v_col,
                                    void* q_out, int64_t q_stride, void* k_pool, void* v_pool,
                                    const float* q_gamma, const float* k_gamma, float eps,
                                    const float* freqs, int rot_dims, void* v_first,
                                    const float* v_lambda, int v_mode, const int* tok_item,
                                    const int* tok_pos, const int* tables, int table_width,
                                    int tokens, int heads, int kv_heads, int key_dim,
                                    int value_dim, int cache_dim, int page_size, int num_pages,
                                    int dtype, void* stream) {
  PS_REQUIRE(tokens >= 0 && heads > 0 && kv_heads > 0 && key_dim > 0 && value_dim > 0 &&
                 page_size > 0 && num_pages > 0 && table_width > 0,
             "ps_attention_prepare: bad sizes");
  PS_REQUIRE(cache_dim >= key_dim && cache_dim >= value_dim && cache_dim % 2 == 0,
             "ps_attention_prepare: cached head size %d must be even and hold keys of %d and values of %d",
             cache_dim, key_dim, value_dim);
  PS_REQUIRE(rot_dims <= 256, "ps_attention_prepare: %d rotated dimensions, the kernel keeps angles for 256", rot_dims);
  PS_REQUIRE(rot_dims >= 0 && rot_dims <= key_dim && rot_dims % 2 == 0,
             "ps_attention_prepare: %d rotated dimensions do not fit heads of %d", rot_dims, key_dim);
  PS_REQUIRE(rot_dims == 0 || freqs != nullptr, "ps_attention_prepare: rotation without frequencies");
  PS_REQUIRE(v_mode >= 0 && v_mode <= 2 && (v_mode == 0 || v_first != nullptr) &&
                 (v_mode != 2 || v_lambda != nullptr),
             "ps_attention_prepare: value mixing needs its buffer and its weight");
  PS_REQUIRE(q_stride >= (int64_t)heads * cache_dim, "ps_attention_prepare: query rows too short");
  PS_REQUIRE((q_gamma == nullptr && k_gamma == nullptr) || eps > 0.f, "ps_attention_prepare: eps must be positive");
  PS_REQUIRE(dtype == PS_F32 || dtype == PS_BF16, "ps_attention_prepare: unknown dtype %d", dtype);
  if (tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  // as many threads as the widest of the three passes has elements (the queries' columns, the
  // pairs of queries and keys), so that a pass is one round of loads where the row allows
  int widest = heads * key_dim;
  if ((heads + kv_heads) * (cache_dim / 2) > widest) widest = (heads + kv_heads) * (cache_dim / 2);
  int threads = widest >= 1024 ? 1024 : (widest + 63) / 64 * 64;
  if (tokens > 256 && threads > 256) threads = 256;   // (many rows fill the chip anyway)
  if (dtype == PS_F32)
    hipLaunchKernelGGL(attention_prepare_kernel<float>, dim3(tokens), dim3(threads), 0, s, proj, ld, q_col,
                       k_col, v_col, (float*)q_out, q_stride, (float*)k_pool, (float*)v_pool, q_gamma,
                       k_gamma, eps, freqs, rot_dims, (float*)v_first, v_lambda, v_mode, tok_item,
                       tok_pos, tables, table_width, heads, kv_heads, key_dim, value_dim, cache_dim,
                       page_size, num_pages);
  else
    hipLaunchKernelGGL(attention_prepare_kernel<bf16_t>, dim3(tokens), dim3(threads), 0, s, proj, ld, q_col,
                       k_col, v_col, (bf16_t*)q_out, q_stride, (bf16_t*)k_pool, (bf16_t*)v_pool,
                       q_gamma, k_gamma, eps, freqs, rot_dims, (bf16_t*)v_first, v_lambda, v_mode,
                       tok_item, tok_pos, tables, table_width, heads, kv_heads, key_dim, value_dim,
                       cache_dim, page_size, num_pages);
  PS_CHECK_LAUNCH("ps_attention_prepare");
  return 0;
}

// ctx[t, h, :] *= sigmoid(gate[t, h]): a gate per token and head on the attention's output.
template <typename T>
__global__ void head_gate_kernel(T* __restrict__ ctx, int64_t stride, const float* __restrict__ gate,
                                 int64_t gate_ld, int heads, int head_dim) {
  const int t = blockIdx.x;
  const int row = heads * head_dim;
  for (int i = threadIdx.x; i < row; i += blockDim.x) {
    const int head = i / head_dim;
    const float g = gate[(int64_t)t * gate_ld + head];
    const float s = 1.0f / (1.0f + expf(-g));
    T* p = ctx + (int64_t)t * stride + i;
    *p = from_float<T>(to_float<T>(*p) * s);
  }
}

extern "C" int ps_head_gate(void* ctx, int64_t stride, const float* gate, int64_t gate_ld,
                            int tokens, int heads, int head_dim, int dtype, void* stream) {
  PS_REQUIRE(tokens >= 0 && heads > 0 && head_dim > 0 && stride >= (int64_t)heads * head_dim &&
                 gate_ld >= heads,
             "ps_head_gate: bad sizes");
  PS_REQUIRE(dtype == PS_F32 || dtype == PS_BF16, "ps_head_gate: unknown dtype %d", dtype);
  if (tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const int threads = heads * head_dim >= 256 ? 256 : 64;
  if (dtype == PS_F32)
    hipLaunchKernelGGL(head_gate_kernel<float>, dim3(tokens), dim3(threads), 0, s, (float*)ctx, stride,
                       gate, gate_ld, heads, head_dim);
  else
    hipLaunchKernelGGL(head_gate_kernel<bf16_t>, dim3(tokens), dim3(threads), 0, s, (bf16_t*)ctx,
                       stride, gate, gate_ld, heads, head_dim);
  PS_CHECK_LAUNCH("ps_head_gate");
  return 0;
}
