// The gated delta rule with a decay per key channel.  Per request and head, token after token, with S [dim, vdim]:
//     S <- g * S (row d times g_d);  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
// where q and k are unit vectors per head (q also times dim^(-1/2)), beta = sigmoid(.), g = exp(-rate_h softplus(. + bias)).
// Everything after the projections and the short convolutions is float32: the unit norms, sigmoid, softplus, the
// exponentials, the state and its sums, the norm of the outputs.
//
// Three kernels.  `delta_prepare` is token-wise: the unit vectors, decays, betas and k . q of every token, float32, into a
// workspace.  `delta_recur` walks a request's tokens: a column of S is spread over R neighbouring lanes (RP rows each), so
// S^T k and S^T q are sums over RP registers and a butterfly over R lanes, and columns need nothing of each other - a
// block takes 256 / R columns of one head, the device as many blocks as heads x columns allow.  Since
// (g S + k u^T)^T q = (g S)^T q + u (k . q), both sums are taken over the decayed state in one pass.  A tile of tokens'
// q, k and g passes through LDS for all columns of the block.  `delta_finish` is token-wise again: o / rms(o) times a
// weight per value channel and the sigmoid of a gate.  A request's state lies in its slot transposed, [heads, vdim, dim]:
// a lane's rows of a column are consecutive floats.

#include "common.h"
#include "api_parts.h"

using namespace akv;

namespace {

__device__ __forceinline__ float softplus_of(float z) { return z > 20.f ? z : log1pf(expf(z)); }
__device__ __forceinline__ float sigmoid_of(float z) { return 1.f / (1.f + expf(-z)); }

// Workspace of a token: [q (groups x dim) | k (groups x dim) | g (heads x dim) | beta (heads) | k . q (heads)].
__host__ __device__ inline long prepared_width(int heads, int groups, int dim) {
  return 2L * groups * dim + static_cast<long>(heads) * dim + 2L * heads;
}

// One block per token.  conv rows: [q (groups x dim) | k (groups x dim) | v ...] after convolution and activation;
// beta_logits at `beta_stride` per token; decay_logits [tokens, heads x dim] float32.
template <typename T>
__global__ __launch_bounds__(256) void delta_prepare_kernel(const T* __restrict__ conv, long conv_stride,
                                                            const T* __restrict__ beta_logits, long beta_stride,
                                                            const float* __restrict__ decay_logits,
                                                            const float* __restrict__ decay_bias,
                                                            const float* __restrict__ rate, float unit_eps, float q_scale,
                                                            float* __restrict__ prepared, int heads, int groups, int dim) {
  const long n = blockIdx.x;
  const int waves = blockDim.x / kWave, wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1);
  const long width = prepared_width(heads, groups, dim);
  float* row = prepared + n * width;
  const T* x = conv + n * conv_stride;
  // unit vectors: a wave a vector (queries first, then keys)
  for (int item = wave; item < 2 * groups; item += waves) {
    const T* src = x + static_cast<long>(item) * dim;
    float squares = 0.f;
    for (int i = lane; i < dim; i += kWave) {
      const float v = to_float(src[i]);
      squares += v * v;
    }
    const float scale = (item < groups ? q_scale : 1.f) / sqrtf(wave_sum(squares) + unit_eps);
    for (int i = lane; i < dim; i += kWave) row[static_cast<long>(item) * dim + i] = to_float(src[i]) * scale;
  }
  float* g = row + 2L * groups * dim;
  for (int i = threadIdx.x; i < heads * dim; i += blockDim.x)
    g[i] = expf(-rate[i / dim] * softplus_of(decay_logits[n * heads * dim + i] + decay_bias[i]));
  float* beta = g + static_cast<long>(heads) * dim;
  for (int h = threadIdx.x; h < heads; h += blockDim.x) beta[h] = sigmoid_of(to_float(beta_logits[n * beta_stride + h]));
  __syncthreads();       // the unit vectors of this token are in memory: k . q per head, a wave a head
  const int share = heads / groups;
  for (int h = wave; h < heads; h += waves) {
    const float* qs = row + static_cast<long>(h / share) * dim;
    const float* ks = row + static_cast<long>(groups + h / share) * dim;
    float dot = 0.f;
    for (int i = lane; i < dim; i += kWave) dot = fmaf(qs[i], ks[i], dot);
    dot = wave_sum(dot);
    if (lane == 0) beta[heads + h] = dot;
  }
}

// A block: one request, one head, 256 / R columns of S.  Thread (column, part): rows part * RP .. part * RP + RP - 1.
// LDS: per token of a tile three arrays (q, k, g) of R segments of RP + 4 floats (the padding keeps the segments of
// neighbouring lanes in different banks), then the tile's values [tile][columns] and betas and k . q [tile][2].
template <typename T, int RP>
__global__ __launch_bounds__(256) void delta_recur_kernel(const float* __restrict__ prepared, const T* __restrict__ conv,
                                                          long conv_stride, long v_at, float* __restrict__ state,
                                                          long state_stride, const int* __restrict__ q_start,
                                                          const int* __restrict__ seq_slots, float* __restrict__ raw_out,
                                                          int heads, int groups, int dim, int vdim, int R, int tile) {
  extern __shared__ float lds[];
  constexpr int SP = RP + 4;
  const int columns = 256 / R, column_blocks = (vdim + columns - 1) / columns;
  const int r = blockIdx.x / (heads * column_blocks);
  const int h = blockIdx.x / column_blocks % heads;
  const int part = threadIdx.x % R;
  const int col = blockIdx.x % column_blocks * columns + threadIdx.x / R;
  const bool works = col < vdim;
  const int first = q_start[r], last = q_start[r + 1];
  const long width = prepared_width(heads, groups, dim);
  const int share = heads / groups;
  const long q_off = static_cast<long>(h / share) * dim, k_off = static_cast<long>(groups + h / share) * dim;
  const long g_off = 2L * groups * dim + static_cast<long>(h) * dim, b_off = 2L * groups * dim + static_cast<long>(heads) * dim + h;
  const int array = R * SP, token_floats = 3 * array;
  float* values = lds + static_cast<long>(tile) * token_floats;       // [tile][columns]
  float* scalars = values + static_cast<long>(tile) * columns;        // [tile][2]: beta, k . q

  float S[RP];
  float* kept = state + static_cast<long>(seq_slots[r]) * state_stride + (static_cast<long>(h) * vdim + (works ? col : 0)) * dim;
#pragma unroll
  for (int i = 0; i < RP; ++i) {
    const int d = part * RP + i;
    S[i] = works && d < dim ? kept[d] : 0.f;
  }
  const int padded = R * RP;
  for (int t0 = first; t0 < last; t0 += tile) {
    const int count = min(tile, last - t0);
    __syncthreads();          // the tile before has been used by everybody
    for (int index = threadIdx.x; index < count * padded; index += blockDim.x) {
      const int tt = index / padded, d = index % padded;
      const float* row = prepared + static_cast<long>(t0 + tt) * width;
      float* at = lds + static_cast<long>(tt) * token_floats + (d / RP) * SP + d % RP;
      const bool real = d < dim;
      at[0] = real ? row[q_off + d] : 0.f;
      at[array] = real ? row[k_off + d] : 0.f;
      at[2 * array] = real ? row[g_off + d] : 1.f;
    }
    for (int index = threadIdx.x; index < count * columns; index += blockDim.x) {
      const int tt = index / columns, c = blockIdx.x % column_blocks * columns + index % columns;
      values[index] = c < vdim ? to_float(conv[static_cast<long>(t0 + tt) * conv_stride + v_at + static_cast<long>(h) * vdim + c]) : 0.f;
    }
    for (int index = threadIdx.x; index < count * 2; index += blockDim.x)
      scalars[index] = prepared[static_cast<long>(t0 + index / 2) * width + b_off + (index & 1) * heads];
    __syncthreads();
    for (int tt = 0; tt < count; ++tt) {
      const float* qs = lds + static_cast<long>(tt) * token_floats + part * SP;
      const float* ks = qs + array;
      const float* gs = ks + array;
      float k[RP];
      float sum_k[4] = {0.f, 0.f, 0.f, 0.f}, sum_q[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int i = 0; i < RP; i += 4) {
        const float4 g4 = *reinterpret_cast<const float4*>(gs + i);
        const float4 k4 = *reinterpret_cast<const float4*>(ks + i);
        const float4 q4 = *reinterpret_cast<const float4*>(qs + i);
        const float gv[4] = {g4.x, g4.y, g4.z, g4.w}, kv[4] = {k4.x, k4.y, k4.z, k4.w}, qv[4] = {q4.x, q4.y, q4.z, q4.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          S[i + e] *= gv[e];
          k[i + e] = kv[e];
          sum_k[e] = fmaf(S[i + e], kv[e], sum_k[e]);
          sum_q[e] = fmaf(S[i + e], qv[e], sum_q[e]);
        }
      }
      float from_k = (sum_k[0] + sum_k[1]) + (sum_k[2] + sum_k[3]);
      float from_q = (sum_q[0] + sum_q[1]) + (sum_q[2] + sum_q[3]);
      for (int offset = R >> 1; offset > 0; offset >>= 1) {
        from_k += __shfl_xor(from_k, offset, kWave);
        from_q += __shfl_xor(from_q, offset, kWave);
      }
      const float u = scalars[2 * tt] * (values[tt * columns + threadIdx.x / R] - from_k);
#pragma unroll
      for (int i = 0; i < RP; ++i) S[i] = fmaf(k[i], u, S[i]);
      if (part == 0 && works)
        raw_out[(static_cast<long>(t0 + tt) * heads + h) * vdim + col] = fmaf(u, scalars[2 * tt + 1], from_q);
    }
  }
  if (works) {
#pragma unroll
    for (int i = 0; i < RP; ++i) {
      const int d = part * RP + i;
      if (d < dim) kept[d] = S[i];
    }
  }
}

// One wave per (token, head): out = raw / rms(raw) * weight * sigmoid(gate).
template <typename T>
__global__ __launch_bounds__(256) void delta_finish_kernel(const float* __restrict__ raw, const float* __restrict__ weight,
                                                           const float* __restrict__ gates, float eps, T* __restrict__ out,
                                                           long items, int vdim) {
  const long item = static_cast<long>(blockIdx.x) * (blockDim.x / kWave) + threadIdx.x / kWave;
  const int lane = threadIdx.x & (kWave - 1);
  if (item >= items) return;
  const float* x = raw + item * vdim;
  float squares = 0.f;
  for (int i = lane; i < vdim; i += kWave) squares = fmaf(x[i], x[i], squares);
  const float scale = rsqrtf(wave_sum(squares) / static_cast<float>(vdim) + eps);
  for (int i = lane; i < vdim; i += kWave)
    out[item * vdim + i] = from_float<T>(x[i] * scale * weight[i] * sigmoid_of(gates[item * vdim + i]));
}

}  // namespace

extern "C" {

long akv_delta_rule_workspace(int tokens, int heads, int groups, int dim, int vdim) {
  return static_cast<long>(tokens) * (prepared_width(heads, groups, dim) + static_cast<long>(heads) * vdim);
}

int akv_delta_rule(const void* conv, long conv_stride, int dtype, const void* beta_logits, long beta_stride,
                   const float* decay_logits, const float* decay_bias, const float* rate, const float* gates,
                   const float* norm_weight, float unit_eps, float norm_eps, float q_scale, float* state, long state_stride,
                   const int* q_start, const int* seq_slots, float* workspace, void* out, int tokens, int seqs, int heads,
                   int groups, int dim, int vdim, hipStream_t stream) {
  if (tokens <= 0 || seqs <= 0) return 0;
  if (heads <= 0 || groups <= 0 || heads % groups != 0 || dim <= 0 || vdim <= 0 || dim > 2048) return -2;
  float* prepared = workspace;
  float* raw = workspace + static_cast<long>(tokens) * prepared_width(heads, groups, dim);
  const int rp = dim <= 64 ? 8 : dim <= 256 ? 16 : 32;
  int R = 1;
  while (R * rp < dim) R *= 2;
  const int columns = 256 / R, column_blocks = (vdim + columns - 1) / columns;
  const long per_token = 3L * R * (rp + 4) + columns + 2;
  const int tile = static_cast<int>(max(1L, min(16L, (48L * 1024 / 4) / per_token)));
  const size_t lds = static_cast<size_t>(tile) * per_token * 4;
  const long v_at = 2L * groups * dim;
  const unsigned grid = static_cast<unsigned>(static_cast<long>(seqs) * heads * column_blocks);
  const long items = static_cast<long>(tokens) * heads;
#define AKV_RECUR(RP)                                                                                                      \
  delta_recur_kernel<T, RP><<<grid, 256, lds, stream>>>(prepared, static_cast<const T*>(conv), conv_stride, v_at, state,   \
                                                        state_stride, q_start, seq_slots, raw, heads, groups, dim, vdim, R, tile)
  AKV_DISPATCH(dtype, T, {
    delta_prepare_kernel<T><<<tokens, 256, 0, stream>>>(static_cast<const T*>(conv), conv_stride,
                                                        static_cast<const T*>(beta_logits), beta_stride, decay_logits,
                                                        decay_bias, rate, unit_eps, q_scale, prepared, heads, groups, dim);
    if (rp == 8) AKV_RECUR(8);
    else if (rp == 16) AKV_RECUR(16);
    else AKV_RECUR(32);
    delta_finish_kernel<T><<<static_cast<unsigned>((items + 3) / 4), 256, 0, stream>>>(raw, norm_weight, gates, norm_eps,
                                                                                      static_cast<T*>(out), items, vdim);
  });
#undef AKV_RECUR
  return AKV_LAUNCH_STATUS();
}
}
