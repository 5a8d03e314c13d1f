// Gated linear attention: a recurrent mixer whose state is a matrix per head.
//
//   S_t = diag(alpha_t) S_(t-1) + k_t v_t^T        (S: [key_dim, value_dim], float, per request)
//   o_t = S_t^T q_t
//
// with a decay alpha in (0, 1) per key channel, alpha = sigmoid(z)^(1/tau), z a low-rank
// projection of the layer's input.  Three launches: the decays of the step's tokens, the
// recurrence, and the output's norm and gate.  The state, the decays and everything they are
// made from are 32-bit; q, k, v arrive as the float columns of the layer's projection.
#include <math.h>

#include "common.h"
#include "pagedserve_hip.h"

// alpha[t, c] = exp(log_sigmoid(z) / tau), z = bias[c] + sum_r low[t, r] w[c, r].
template <typename T>
__global__ __launch_bounds__(256) void gla_decay_kernel(
    const float* __restrict__ proj, int64_t ld, int low_col, int rank, const T* __restrict__ w,
    const float* __restrict__ bias, float inv_tau, float* __restrict__ alpha, int channels) {
  extern __shared__ float low[];
  const int t = blockIdx.x;
  for (int r = threadIdx.x; r < rank; r += blockDim.x) low[r] = proj[(int64_t)t * ld + low_col + r];
  __syncthreads();
  for (int c = threadIdx.x; c < channels; c += blockDim.x) {
    float z = bias ? bias[c] : 0.f;
    const T* w_row = w + (int64_t)c * rank;
    for (int r = 0; r < rank; ++r) z = fmaf(low[r], to_float<T>(w_row[r]), z);
    // log sigmoid(z) = min(z, 0) - log(1 + exp(-|z|))
    const float log_sigmoid = fminf(z, 0.f) - log1pf(expf(-fabsf(z)));
    alpha[(int64_t)t * channels + c] = expf(log_sigmoid * inv_tau);
  }
}


// A block (one wave) owns COLS columns of one head's state for one item of the step and walks
// the item's tokens in order: lane = row group * COLS + column.  The state's rows are dealt to
// the 64 / COLS row groups, RPL rows per lane, in registers; o needs the sum over the row groups,
// which is taken through LDS once per chunk.  The walk is one dependent chain per token, so a launch with few
// blocks takes narrow ones (4 columns, 16 row groups: a quarter of the work per lane and token,
// four times the blocks), one with many the wide ones (16 columns, 4 row groups).  The
// tokens' q, k and decays come GLA_CHUNK at a time (32 for key heads up to 64, fewer for larger
// ones: 32 values per lane and array): a chunk's loads leave together into registers while the
// chunk before is being worked on from LDS; the work on a chunk has to last as long as a trip
// to memory for the walk not to wait, hence chunks as long as the registers allow.
template <int RPL, int COLS, int GLA_CHUNK>
__global__ __launch_bounds__(64) void gla_scan_kernel(
    const float* __restrict__ proj, int64_t ld, int q_col, int k_col, int v_col,
    const float* __restrict__ alpha, float* __restrict__ state, float* __restrict__ out,
    const int* __restrict__ cu_tokens, const int* __restrict__ slots, int heads, int key_dim,
    int value_dim, float q_scale, const float* __restrict__ head_decay, int silu_inputs) {
  constexpr int GROUPS = 64 / COLS;                // row groups
  constexpr int ROWS = GROUPS * RPL;               // rows with padding up to the lanes' share
  constexpr int PAD = RPL + 4;                     // row groups start in different banks
  constexpr int PER = GLA_CHUNK * ROWS / 64;       // values of a chunk per lane and array
  constexpr int PER_V = (GLA_CHUNK * COLS + 63) / 64;
  static_assert(GLA_CHUNK * ROWS % 64 == 0 && PER >= 1, "a chunk's rows are dealt evenly to the lanes");
  __shared__ __attribute__((aligned(16))) float s_q[GLA_CHUNK][GROUPS * PAD];
  __shared__ __attribute__((aligned(16))) float s_k[GLA_CHUNK][GROUPS * PAD];
  __shared__ __attribute__((aligned(16))) float s_a[GLA_CHUNK][GROUPS * PAD];
  __shared__ float s_v[GLA_CHUNK][COLS];
  __shared__ float s_o[GLA_CHUNK][65];     // every lane's share of o_t (rows one bank apart)
  const int item = blockIdx.x, head = blockIdx.y;
  const int lane = threadIdx.x;
  const int col = blockIdx.z * COLS + (lane % COLS);
  const int group = lane / COLS;
  const bool has_col = col < value_dim;
  const int t0 = cu_tokens[item], t1 = cu_tokens[item + 1];
  const int slot = slots[item];
  float* s_ptr = state + (((int64_t)slot * heads + head) * key_dim) * value_dim;
  float S[RPL];
#pragma unroll
  for (int i = 0; i < RPL; ++i) {
    const int r = group * RPL + i;
    S[i] = (r < key_dim && has_col) ? s_ptr[(int64_t)r * value_dim + col] : 0.f;
  }
  const int channels = heads * key_dim;
  float rq[PER], rk[PER], ra[PER], rv[PER_V];
  // one decay per head for all key channels and tokens (then no array of decays is read)
  const float fixed_decay = head_decay ? head_decay[head] : 0.f;
  // every load is unconditional from a clamped address; what lies outside is masked when stored
  auto fetch = [&](const int base) {
    const int count = (t1 - base) < GLA_CHUNK ? (t1 - base) : GLA_CHUNK;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int idx = lane + j * 64;
      const int tt = idx / ROWS;
      const int r = idx - tt * ROWS;
      const int64_t t = base + (tt < count ? tt : 0);
      const int c = head * key_dim + (r < key_dim ? r : 0);
      rq[j] = proj[t * ld + q_col + c];
      rk[j] = proj[t * ld + k_col + c];
      ra[j] = head_decay ? fixed_decay : alpha[t * channels + c];
    }
#pragma unroll
    for (int j = 0; j < PER_V; ++j) {
      const int idx = (lane + j * 64) % (GLA_CHUNK * COLS);
      const int tt = idx / COLS;
      const int c = blockIdx.z * COLS + (idx - tt * COLS);
      const int64_t t = base + (tt < count ? tt : 0);
      rv[j] = proj[t * ld + v_col + head * value_dim + (c < value_dim ? c : 0)];
    }
  };
  auto stash = [&](const int base) {
    const int count = (t1 - base) < GLA_CHUNK ? (t1 - base) : GLA_CHUNK;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int idx = lane + j * 64;
      const int tt = idx / ROWS;
      const int r = idx - tt * ROWS;
      const bool valid = tt < count && r < key_dim;
      const int at = (r / RPL) * PAD + (r % RPL);
      if (silu_inputs) {
        rq[j] = rq[j] / (1.0f + expf(-rq[j]));
        rk[j] = rk[j] / (1.0f + expf(-rk[j]));
      }
      s_q[tt][at] = valid ? rq[j] * q_scale : 0.f;
      s_k[tt][at] = valid ? rk[j] : 0.f;
      s_a[tt][at] = valid ? ra[j] : 0.f;
    }
#pragma unroll
    for (int j = 0; j < PER_V; ++j) {
      const int idx = lane + j * 64;
      if (idx < GLA_CHUNK * COLS) {
        const int tt = idx / COLS;
        const int c = blockIdx.z * COLS + (idx - tt * COLS);
        if (silu_inputs) rv[j] = rv[j] / (1.0f + expf(-rv[j]));
        s_v[tt][idx - tt * COLS] = (tt < count && c < value_dim) ? rv[j] : 0.f;
      }
    }
  };
  if (t0 < t1) fetch(t0);
  for (int base = t0; base < t1; base += GLA_CHUNK) {
    const int count = (t1 - base) < GLA_CHUNK ? (t1 - base) : GLA_CHUNK;
    __syncthreads();      // the chunk before has been read
    stash(base);
    __syncthreads();
    if (base + GLA_CHUNK < t1) fetch(base + GLA_CHUNK);   // in flight during the work below
    // a lane's share of o_t
    auto token = [&](const int tt) -> float {
      const float v = s_v[tt][lane % COLS];
      float o = 0.f;
#pragma unroll
      for (int i = 0; i < RPL; ++i) {
        const int at = group * PAD + i;
        S[i] = fmaf(s_a[tt][at], S[i], s_k[tt][at] * v);
        o = fmaf(S[i], s_q[tt][at], o);
      }
      return o;
    };
    // The lanes' shares wait in LDS: the state's chain then holds no exchange between lanes,
    // and the sums over the row groups are taken for all tokens of the chunk at once.
    if (count == GLA_CHUNK) {
      // a whole chunk: unrolled, so that the reads of the next tokens run ahead of the chain
#pragma unroll
      for (int tt = 0; tt < GLA_CHUNK; ++tt) s_o[tt][lane] = token(tt);
    } else {
      for (int tt = 0; tt < count; ++tt) s_o[tt][lane] = token(tt);
    }
    __syncthreads();
    for (int idx = lane; idx < count * COLS; idx += 64) {
      const int tt = idx / COLS;
      const int c = idx - tt * COLS;
      float sum = 0.f;
#pragma unroll
      for (int g = 0; g < GROUPS; ++g) sum += s_o[tt][g * COLS + c];
      const int to = blockIdx.z * COLS + c;
      if (to < value_dim) out[(int64_t)(base + tt) * heads * value_dim + head * value_dim + to] = sum;
    }
  }
#pragma unroll
  for (int i = 0; i < RPL; ++i) {
    const int r = group * RPL + i;
    if (r < key_dim && has_col) s_ptr[(int64_t)r * value_dim + col] = S[i];
  }
}

// out[t, h, :] = o[t, h, :] / sqrt(mean(o[t, h, :]^2) + eps) * w * silu(gate[t, h, :]).
template <typename T>
__global__ __launch_bounds__(64) void gla_output_kernel(
    const float* __restrict__ o, const float* __restrict__ w, float eps,
    const float* __restrict__ gate, int64_t gate_ld, T* __restrict__ out, int64_t out_stride,
    int heads, int value_dim) {
  const int t = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  const float* row = o + ((int64_t)t * heads + head) * value_dim;
  float sum = 0.f;
  for (int d = lane; d < value_dim; d += 64) sum = fmaf(row[d], row[d], sum);
  const float inv = 1.0f / sqrtf(wave_sum(sum) / (float)value_dim + eps);
  for (int d = lane; d < value_dim; d += 64) {
    const float g = gate[(int64_t)t * gate_ld + head * value_dim + d];
    const float silu = g / (1.0f + expf(-g));
    out[(int64_t)t * out_stride + head * value_dim + d] = from_float<T>(row[d] * inv * w[d] * silu);
  }
}

// out[t, :] = o[t, :] / sqrt(mean(o[t, :]^2) + eps) * w * sigmoid(gate[t, :]): the norm over the
// whole row (all heads together), a block per token.
template <typename T>
__global__ __launch_bounds__(256) void row_norm_gate_kernel(
    const float* __restrict__ o, const float* __restrict__ w, float eps,
    const float* __restrict__ gate, int64_t gate_ld, T* __restrict__ out, int64_t out_stride,
    int columns) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const float* row = o + (int64_t)t * columns;
  float sum = 0.f;
  for (int d = threadIdx.x; d < columns; d += blockDim.x) sum = fmaf(row[d], row[d], sum);
  const float inv = 1.0f / sqrtf(block_sum(sum, scratch) / (float)columns + eps);
  for (int d = threadIdx.x; d < columns; d += blockDim.x) {
    const float g = gate[(int64_t)t * gate_ld + d];
    out[(int64_t)t * out_stride + d] = from_float<T>(row[d] * inv * w[d] / (1.0f + expf(-g)));
  }
}

extern "C" int ps_row_norm_gate(const float* o, const float* w, float eps, const float* gate,
                                int64_t gate_ld, void* out, int64_t out_stride, int tokens,
                                int columns, int dtype, void* stream) {
  PS_REQUIRE(tokens >= 0 && columns > 0 && eps > 0.f, "ps_row_norm_gate: bad sizes");
  PS_REQUIRE(dtype == PS_F32 || dtype == PS_BF16, "ps_row_norm_gate: unknown dtype %d", dtype);
  if (tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == PS_F32)
    hipLaunchKernelGGL(row_norm_gate_kernel<float>, dim3(tokens), dim3(256), 0, s, o, w, eps, gate,
                       gate_ld, (float*)out, out_stride, columns);
  else
    hipLaunchKernelGGL(row_norm_gate_kernel<bf16_t>, dim3(tokens), dim3(256), 0, s, o, w, eps, gate,
                       gate_ld, (bf16_t*)out, out_stride, columns);
  PS_CHECK_LAUNCH("ps_row_norm_gate");
  return 0;
}

// ---- long portions in pieces that run side by side (recurrences with one decay per head) ----
// The recurrence is linear in the state: a piece of n tokens takes S to d^n S + E, with E what
// it leaves from a zero state.  So the items of a step are cut into pieces, every piece runs
// the recurrence kernel as an item of its own with a state of its own (first from zero, which
// leaves E there; then, once ps_decay_join has put every piece's true start in E's place, again,
// now for the outputs).
//
// piece_cu[k] .. piece_cu[k + 1]: the tokens of piece k (empty behind the last piece);
// item_first[i]: the first piece of item i.  One thread: a step has a handful of items.
__global__ void scan_pieces_kernel(const int* __restrict__ cu_tokens, int items, int piece,
                                   int max_pieces, int* __restrict__ piece_cu,
                                   int* __restrict__ item_first) {
  if (blockIdx.x != 0 || threadIdx.x != 0) return;
  int at = 0;
  for (int i = 0; i < items; ++i) {
    item_first[i] = at;
    for (int t = cu_tokens[i]; t < cu_tokens[i + 1] && at < max_pieces; t += piece) piece_cu[at++] = t;
  }
  item_first[items] = at;
  for (int k = at; k <= max_pieces; ++k) piece_cu[k] = cu_tokens[items];
}

// A thread per number of an item's state: S <- the slot's; for the item's pieces in order:
// E <-> S's place (the piece's start), S <- d^n S + E; the last S goes to the slot.
__global__ __launch_bounds__(256) void decay_join_kernel(
    float* __restrict__ piece_states, float* __restrict__ state, const int* __restrict__ piece_cu,
    const int* __restrict__ item_first, const int* __restrict__ slots,
    const float* __restrict__ head_decay, int heads, int per_head) {
  const int item = blockIdx.x, head = blockIdx.y;
  const int e = blockIdx.z * 256 + threadIdx.x;
  if (e >= per_head) return;
  const int first = item_first[item], last = item_first[item + 1];
  if (first == last) return;
  const float d = head_decay[head];
  float* mine = state + ((int64_t)slots[item] * heads + head) * per_head + e;
  float s = *mine;
  for (int k = first; k < last; ++k) {
    float* record = piece_states + ((int64_t)k * heads + head) * per_head + e;
    const float left = *record;
    *record = s;
    s = fmaf(powf(d, (float)(piece_cu[k + 1] - piece_cu[k])), s, left);
  }
  *mine = s;
}

extern "C" int ps_scan_pieces(const int* cu_tokens, int items, int piece, int max_pieces,
                              int* piece_cu, int* item_first, void* stream) {
  PS_REQUIRE(items >= 0 && piece > 0 && max_pieces >= 0, "ps_scan_pieces: bad sizes");
  hipLaunchKernelGGL(scan_pieces_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, cu_tokens, items,
                     piece, max_pieces, piece_cu, item_first);
  PS_CHECK_LAUNCH("ps_scan_pieces");
  return 0;
}

extern "C" int ps_decay_join(float* piece_states, float* state, const int* piece_cu,
                             const int* item_first, const int* slots, const float* head_decay,
                             int items, int heads, int per_head, void* stream) {
  PS_REQUIRE(items >= 0 && heads > 0 && per_head > 0, "ps_decay_join: bad sizes");
  if (items == 0) return 0;
  hipLaunchKernelGGL(decay_join_kernel, dim3(items, heads, (per_head + 255) / 256), dim3(256), 0,
                     (hipStream_t)stream, piece_states, state, piece_cu, item_first, slots,
                     head_decay, heads, per_head);
  PS_CHECK_LAUNCH("ps_decay_join");
  return 0;
}

extern "C" int ps_gla_decay(const float* proj, int64_t ld, int low_col, int rank, const void* w,
                            const float* bias, float tau, float* alpha, int tokens, int channels,
                            int dtype, void* stream) {
  PS_REQUIRE(tokens >= 0 && rank > 0 && channels > 0 && tau > 0.f, "ps_gla_decay: bad sizes");
  PS_REQUIRE(rank <= 8192, "ps_gla_decay: rank %d above 8192", rank);
  PS_REQUIRE(dtype == PS_F32 || dtype == PS_BF16, "ps_gla_decay: unknown dtype %d", dtype);
  if (tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const size_t lds = (size_t)rank * sizeof(float);
  if (dtype == PS_F32)
    hipLaunchKernelGGL(gla_decay_kernel<float>, dim3(tokens), dim3(256), lds, s, proj, ld, low_col,
                       rank, (const float*)w, bias, 1.0f / tau, alpha, channels);
  else
    hipLaunchKernelGGL(gla_decay_kernel<bf16_t>, dim3(tokens), dim3(256), lds, s, proj, ld, low_col,
                       rank, (const bf16_t*)w, bias, 1.0f / tau, alpha, channels);
  PS_CHECK_LAUNCH("ps_gla_decay");
  return 0;
}

extern "C" int ps_gla_scan(const float* proj, int64_t ld, int q_col, int k_col, int v_col,
                           const float* alpha, float* state, float* out, const int* cu_tokens,
                           const int* slots, int items, int max_slots, int heads, int key_dim,
                           int value_dim, float q_scale, int longest, const float* head_decay,
                           int silu_inputs, void* stream) {
  PS_REQUIRE(alpha != nullptr || head_decay != nullptr, "ps_gla_scan: no decays given");
  PS_REQUIRE(items >= 0 && heads > 0 && key_dim > 0 && value_dim > 0 && max_slots > 0,
             "ps_gla_scan: bad sizes");
  PS_REQUIRE(key_dim <= 256, "ps_gla_scan: key head size %d above 256", key_dim);
  PS_REQUIRE(heads <= 65535 && (value_dim + 3) / 4 <= 65535, "ps_gla_scan: grid too large");
  if (items == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  // narrow blocks while wide ones would leave the chip's SIMDs (four to a compute unit) idle
  const int64_t wide_blocks = (int64_t)items * heads * ((value_dim + 15) / 16);
  const bool narrow = wide_blocks < 2 * (int64_t)ps_compute_units();
  // items of a few tokens at most (decode steps): chunks of 8, which cost less to stage
  const bool brief = longest > 0 && longest <= 8;
#define PS_LAUNCH_GLA_C(RPL, COLS, CHUNK)                                                         \
  hipLaunchKernelGGL((gla_scan_kernel<RPL, COLS, CHUNK>),                                         \
                     dim3(items, heads, (value_dim + COLS - 1) / COLS),                           \
                     dim3(64), 0, s, proj, ld, q_col, k_col, v_col, alpha, state, out, cu_tokens, \
                     slots, heads, key_dim, value_dim, q_scale, head_decay, silu_inputs)
#define PS_LAUNCH_GLA(RPL, COLS)                                                                  \
  do {                                                                                            \
    if (brief) {                                                                                  \
      PS_LAUNCH_GLA_C(RPL, COLS, 8);                                                              \
    } else {                                                                                      \
      PS_LAUNCH_GLA_C(RPL, COLS, (2048 / (64 / COLS * RPL) < 32 ? 2048 / (64 / COLS * RPL) : 32)); \
    }                                                                                             \
  } while (0)
  if (narrow) {
    if (key_dim <= 32) PS_LAUNCH_GLA(2, 4);
    else if (key_dim <= 64) PS_LAUNCH_GLA(4, 4);
    else if (key_dim <= 128) PS_LAUNCH_GLA(8, 4);
    else PS_LAUNCH_GLA(16, 4);
  } else {
    if (key_dim <= 32) PS_LAUNCH_GLA(8, 16);
    else if (key_dim <= 64) PS_LAUNCH_GLA(16, 16);
    else if (key_dim <= 128) PS_LAUNCH_GLA(32, 16);
    else PS_LAUNCH_GLA(64, 16);
  }
#undef PS_LAUNCH_GLA
#undef PS_LAUNCH_GLA_C
  PS_CHECK_LAUNCH("ps_gla_scan");
  return 0;
}

extern "C" int ps_gla_output(const float* o, const float* w, float eps, const float* gate,
                             int64_t gate_ld, void* out, int64_t out_stride, int tokens, int heads,
                             int value_dim, int dtype, void* stream) {
  PS_REQUIRE(tokens >= 0 && heads > 0 && value_dim > 0 && eps > 0.f && heads <= 65535,
             "ps_gla_output: bad sizes");
  PS_REQUIRE(dtype == PS_F32 || dtype == PS_BF16, "ps_gla_output: unknown dtype %d", dtype);
  if (tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == PS_F32)
    hipLaunchKernelGGL(gla_output_kernel<float>, dim3(tokens, heads), dim3(64), 0, s, o, w, eps, gate,
                       gate_ld, (float*)out, out_stride, heads, value_dim);
  else
    hipLaunchKernelGGL(gla_output_kernel<bf16_t>, dim3(tokens, heads), dim3(64), 0, s, o, w, eps, gate,
                       gate_ld, (bf16_t*)out, out_stride, heads, value_dim);
  PS_CHECK_LAUNCH("ps_gla_output");
  return 0;
}
