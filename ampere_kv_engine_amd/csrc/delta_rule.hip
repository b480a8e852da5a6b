// The gated delta rule with a decay per key channel.  Per request and head, token after token, with S [dim, vdim]:
//     S <- g * S (row d times g_d);  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
// where q and k are unit vectors per head (q also times dim^(-1/2)), beta = sigmoid(.), g = exp(-rate_h softplus(. + bias)).
// Everything after the projections and the short convolutions is float32: the unit norms, sigmoid, softplus, the
// exponentials, the state and its sums, the norm of the outputs.
//
// Three kernels.  `delta_prepare` is token-wise: the unit vectors, decays, betas and k . q of every token, float32, into a
// workspace.  `delta_recur` walks a request's tokens: a column of S is spread over R neighbouring lanes (RP rows each), so
// S^T k and S^T q are sums over RP registers and a butterfly over R lanes inside the vector unit, and columns need nothing
// of each other - a block takes 256 / R columns of one head.  The recurrence is a chain through the tokens whose length
// nothing shortens, so what counts is a wave's instructions per token: with four rows a lane, one request's heads of
// 128 x 128 are 1,024 waves - one on every vector unit of the device.  Since (g S + k u^T)^T q = (g S)^T q + u (k . q),
// both sums are taken over the decayed state in one pass.  A tile of tokens' q, k and g passes through LDS for all columns
// of the block; the next tile's values are asked for before this tile's tokens are walked; a whole tile is walked without a
// loop (constant LDS addresses, a token's reads issued one token ahead) and its outputs are stored after the next tile's
// barriers, which would otherwise wait for them.  `delta_finish` is token-wise
// again: o / rms(o) times a weight per value channel and the sigmoid of a gate.  A request's state lies in its slot
// transposed, [heads, vdim, dim]: a lane's rows of a column are consecutive floats.

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

// A wave is a token's unit of work: units 0 .. groups - 1 are a q / k pair (sums of squares and the product from one pass
// over the raw vectors: k . q of the unit vectors follows without reading them back; the betas of the pair's heads go
// along), every further unit 256 decays.  conv rows: [q (groups x dim) | k (groups x dim) | v ...] after convolution and
// activation; beta_logits at `beta_stride` per token; decay_logits [tokens, heads x dim] float32.
template <typename T>
__global__ __launch_bounds__(256) void delta_prepare_kernel(const T* __restrict__ conv, long conv_stride,
                                                            const T* __restrict__ beta_logits, long beta_stride,
                                                            const float* __restrict__ decay_logits,
                                                            const float* __restrict__ decay_bias,
                                                            const float* __restrict__ rate, float unit_eps, float q_scale,
                                                            float* __restrict__ prepared, int heads, int groups, int dim) {
  const long n = blockIdx.x;
  const int lane = threadIdx.x & (kWave - 1);
  const int unit = blockIdx.y * (blockDim.x / kWave) + threadIdx.x / kWave;
  const long width = prepared_width(heads, groups, dim);
  float* row = prepared + n * width;
  float* g = row + 2L * groups * dim;
  float* beta = g + static_cast<long>(heads) * dim;
  const int share = heads / groups;
  if (unit < groups) {
    const T* qs = conv + n * conv_stride + static_cast<long>(unit) * dim;
    const T* ks = qs + static_cast<long>(groups) * dim;
    float qq = 0.f, kk = 0.f, qk = 0.f;
    for (int i = lane; i < dim; i += kWave) {
      const float a = to_float(qs[i]), b = to_float(ks[i]);
      qq = fmaf(a, a, qq), kk = fmaf(b, b, kk), qk = fmaf(a, b, qk);
    }
    const float q_unit = q_scale / sqrtf(wave_sum(qq) + unit_eps), k_unit = 1.f / sqrtf(wave_sum(kk) + unit_eps);
    const float dot = wave_sum(qk) * q_unit * k_unit;
    for (int i = lane; i < dim; i += kWave) {
      row[static_cast<long>(unit) * dim + i] = to_float(qs[i]) * q_unit;
      row[static_cast<long>(groups + unit) * dim + i] = to_float(ks[i]) * k_unit;
    }
    for (int j = lane; j < share; j += kWave) {
      const int h = unit * share + j;
      beta[h] = sigmoid_of(to_float(beta_logits[n * beta_stride + h]));
      beta[heads + h] = dot;
    }
    return;
  }
  const int first = (unit - groups) * 256;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int i = first + e * kWave + lane;
    if (i < heads * dim) g[i] = expf(-rate[i / dim] * softplus_of(decay_logits[n * heads * dim + i] + decay_bias[i]));
  }
}

// Sums over the R neighbouring lanes of a column, in all of them, without a trip through LDS: exchanges inside quads, the
// two mirrors of a row of 16 lanes, then swaps of rows and of the wave's halves.
template <int CTRL> __device__ __forceinline__ float lane_exchange(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}
template <int R> __device__ __forceinline__ float column_sum(float v) {
  if (R >= 2) v += lane_exchange<0xB1>(v);       // quad_perm [1, 0, 3, 2]
  if (R >= 4) v += lane_exchange<0x4E>(v);       // quad_perm [2, 3, 0, 1]
  if (R >= 8) v += lane_exchange<0x141>(v);      // row_half_mirror
  if (R >= 16) v += lane_exchange<0x140>(v);     // row_mirror
  if (R >= 32) {
    const uint32_t bits = __float_as_uint(v);
    const auto swapped = __builtin_amdgcn_permlane16_swap(bits, bits, false, false);
    v = __uint_as_float(swapped[0]) + __uint_as_float(swapped[1]);
  }
  if (R >= 64) {
    const uint32_t bits = __float_as_uint(v);
    const auto swapped = __builtin_amdgcn_permlane32_swap(bits, bits, false, false);
    v = __uint_as_float(swapped[0]) + __uint_as_float(swapped[1]);
  }
  return v;
}

// Tokens of a tile: what 48 KB of LDS hold of their q, k and g, CAP at most.  Every tile costs two barriers, its loads'
// addresses and its stores: 32 tokens instead of 16 took an eighth off a long walk's time.  Steps of single tokens take
// tiles of 4: many blocks of little LDS fit a compute unit and hide each other's loads of the state.
template <int RP, int R, int CAP> struct DeltaTile {
  static constexpr int kSegment = RP == 4 ? 4 : RP + 4;     // (padding keeps the longer segments of neighbouring lanes in different banks)
  static constexpr int kArray = R * kSegment;
  static constexpr int kColumns = 256 / R;
  static constexpr int kRoom = 12288 / (3 * kArray);
  static constexpr int kTokens = kRoom >= CAP ? CAP : kRoom >= 16 ? 16 : kRoom >= 1 ? kRoom : 1;
  static constexpr int kFloats = kTokens * (3 * kArray + kColumns + 2);
};

// What a lane needs of one token: its RP rows of q, k and g, its column's value, the head's beta and k . q.
template <int RP> struct TokenOperands {
  float q[RP], k[RP], g[RP], value, beta, kq;
  __device__ __forceinline__ void read(const float* qs, int array, const float* value_at, const float* scalar_at) {
#pragma unroll
    for (int i = 0; i < RP; i += 4) {
      const float4 q4 = *reinterpret_cast<const float4*>(qs + i);
      const float4 k4 = *reinterpret_cast<const float4*>(qs + array + i);
      const float4 g4 = *reinterpret_cast<const float4*>(qs + 2 * array + i);
      q[i] = q4.x, q[i + 1] = q4.y, q[i + 2] = q4.z, q[i + 3] = q4.w;
      k[i] = k4.x, k[i + 1] = k4.y, k[i + 2] = k4.z, k[i + 3] = k4.w;
      g[i] = g4.x, g[i + 1] = g4.y, g[i + 2] = g4.z, g[i + 3] = g4.w;
    }
    value = *value_at, beta = scalar_at[0], kq = scalar_at[1];
  }
};

// A block: one request, one head, 256 / R columns of S.  Thread (column, part): rows part * RP .. part * RP + RP - 1.
// LDS: per token of a tile three arrays (q, k, g) of R segments, then the tile's values [tile][columns] and its betas and
// k . q [tile][2].
template <typename T, int RP, int R, int CAP>
__global__ __launch_bounds__(256) void delta_recur_kernel(const float* __restrict__ prepared, const T* __restrict__ conv,
                                                          long conv_stride, long v_at, float* __restrict__ state,
                                                          long state_stride, const int* __restrict__ q_start,
                                                          const int* __restrict__ seq_slots, float* __restrict__ raw_out,
                                                          int heads, int groups, int dim, int vdim) {
  using Tile = DeltaTile<RP, R, CAP>;
  constexpr int SP = Tile::kSegment, kArray = Tile::kArray, kColumns = Tile::kColumns, kTile = Tile::kTokens;
  constexpr int kPadded = R * RP;
  constexpr int kVectorLoads = (kTile * kPadded + 255) / 256, kValueLoads = (kTile * kColumns + 255) / 256;
  __shared__ __attribute__((aligned(16))) float lds[Tile::kFloats];
  float* values = lds + kTile * 3 * kArray;        // [tile][columns]
  float* scalars = values + kTile * kColumns;      // [tile][2]: beta, k . q
  const int column_blocks = (vdim + kColumns - 1) / kColumns;
  const int r = blockIdx.x / (heads * column_blocks);
  const int h = blockIdx.x / column_blocks % heads;
  const int part = threadIdx.x % R;
  const int col0 = blockIdx.x % column_blocks * kColumns;
  const int col = col0 + threadIdx.x / R;
  const bool works = col < vdim;
  const int first = q_start[r], last = q_start[r + 1];
  const long width = prepared_width(heads, groups, dim);
  const int share = heads / groups;
  const long q_off = static_cast<long>(h / share) * dim, k_off = static_cast<long>(groups + h / share) * dim;
  const long g_off = 2L * groups * dim + static_cast<long>(h) * dim, b_off = 2L * groups * dim + static_cast<long>(heads) * dim + h;

  float S[RP];
  float* kept = state + static_cast<long>(seq_slots[r]) * state_stride + (static_cast<long>(h) * vdim + (works ? col : 0)) * dim;
  const bool whole_fours = dim % 4 == 0 && state_stride % 4 == 0;      // (16-byte accesses need their alignment)
#pragma unroll
  for (int i = 0; i < RP; i += 4) {
    const int d = part * RP + i;
    if (works && whole_fours && d < dim) {
      const float4 four = *reinterpret_cast<const float4*>(kept + d);
      S[i] = four.x, S[i + 1] = four.y, S[i + 2] = four.z, S[i + 3] = four.w;
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) S[i + e] = works && d + e < dim ? kept[d + e] : 0.f;
    }
  }

  // a tile's operands on their way from memory: asked for one tile ahead, laid into LDS when the tile before is done
  // (with four rows a lane the segments lie in LDS without padding: where rows of the workspace allow 16-byte loads, four
  // neighbouring floats travel together)
  constexpr int kFourLoads = (kTile * kPadded / 4 + 255) / 256;
  constexpr int kFetched = RP == 4 && 4 * kFourLoads > kVectorLoads ? 4 * kFourLoads : kVectorLoads;
  const bool fours = RP == 4 && dim % 4 == 0 && width % 4 == 0 && (reinterpret_cast<uintptr_t>(prepared) & 15) == 0;
  float fetched_q[kFetched], fetched_k[kFetched], fetched_g[kFetched], fetched_v[kValueLoads], fetched_s = 0.f;
  // (loads are never skipped: a token or row that the tile does not have reads a neighbour's address, and what it read
  // is replaced by a value without effect when the tile is laid down - no branch stands between a load and the walk)
  int fetched_count = 0;
  auto fetch = [&](int t0) {
    const int count = min(kTile, last - t0);
    fetched_count = count;
    if (fours) {
#pragma unroll
      for (int j = 0; j < kFourLoads; ++j) {
        const int index = threadIdx.x + j * 256;
        const int tt = min(index / (kPadded / 4), count - 1), d = index % (kPadded / 4) * 4;
        const float* row = prepared + static_cast<long>(t0 + tt) * width + (d < dim ? d : 0);
        const float4 q4 = *reinterpret_cast<const float4*>(row + q_off);
        const float4 k4 = *reinterpret_cast<const float4*>(row + k_off);
        const float4 g4 = *reinterpret_cast<const float4*>(row + g_off);
        fetched_q[4 * j] = q4.x, fetched_q[4 * j + 1] = q4.y, fetched_q[4 * j + 2] = q4.z, fetched_q[4 * j + 3] = q4.w;
        fetched_k[4 * j] = k4.x, fetched_k[4 * j + 1] = k4.y, fetched_k[4 * j + 2] = k4.z, fetched_k[4 * j + 3] = k4.w;
        fetched_g[4 * j] = g4.x, fetched_g[4 * j + 1] = g4.y, fetched_g[4 * j + 2] = g4.z, fetched_g[4 * j + 3] = g4.w;
      }
    } else {
#pragma unroll
    for (int j = 0; j < kVectorLoads; ++j) {
      const int index = threadIdx.x + j * 256;
      const int tt = index / kPadded, d = index % kPadded;
      const bool real = tt < count && d < dim;
      const float* row = prepared + static_cast<long>(t0 + tt) * width;
      fetched_q[j] = real ? row[q_off + d] : 0.f;
      fetched_k[j] = real ? row[k_off + d] : 0.f;
      fetched_g[j] = real ? row[g_off + d] : 1.f;
    }
    }
#pragma unroll
    for (int j = 0; j < kValueLoads; ++j) {
      const int index = threadIdx.x + j * 256;
      const int tt = index / kColumns, c = col0 + index % kColumns;
      fetched_v[j] = to_float(conv[static_cast<long>(t0 + min(tt, count - 1)) * conv_stride + v_at + static_cast<long>(h) * vdim +
                                   (c < vdim ? c : 0)]);
    }
    const int which = min(static_cast<int>(threadIdx.x), 2 * count - 1);
    fetched_s = prepared[static_cast<long>(t0 + which / 2) * width + b_off + (which & 1) * heads];
  };
  auto lay_down = [&]() {
    if (fours) {
#pragma unroll
      for (int j = 0; j < kFourLoads; ++j) {
        const int index = threadIdx.x + j * 256;
        if (index >= kTile * kPadded / 4) continue;
        float* at = lds + index / (kPadded / 4) * 3 * kArray + index % (kPadded / 4) * 4;
        const bool real = index / (kPadded / 4) < fetched_count && index % (kPadded / 4) * 4 < dim;
        const float4 zeros = make_float4(0.f, 0.f, 0.f, 0.f), ones = make_float4(1.f, 1.f, 1.f, 1.f);
        *reinterpret_cast<float4*>(at) = real ? make_float4(fetched_q[4 * j], fetched_q[4 * j + 1], fetched_q[4 * j + 2], fetched_q[4 * j + 3]) : zeros;
        *reinterpret_cast<float4*>(at + kArray) = real ? make_float4(fetched_k[4 * j], fetched_k[4 * j + 1], fetched_k[4 * j + 2], fetched_k[4 * j + 3]) : zeros;
        *reinterpret_cast<float4*>(at + 2 * kArray) = real ? make_float4(fetched_g[4 * j], fetched_g[4 * j + 1], fetched_g[4 * j + 2], fetched_g[4 * j + 3]) : ones;
      }
    } else {
#pragma unroll
      for (int j = 0; j < kVectorLoads; ++j) {
        const int index = threadIdx.x + j * 256;
        if (index >= kTile * kPadded) continue;
        const int tt = index / kPadded, d = index % kPadded;
        float* at = lds + tt * 3 * kArray + (d / RP) * SP + d % RP;
        at[0] = fetched_q[j], at[kArray] = fetched_k[j], at[2 * kArray] = fetched_g[j];
      }
    }
#pragma unroll
    for (int j = 0; j < kValueLoads; ++j) {
      const int index = threadIdx.x + j * 256;
      if (index < kTile * kColumns)
        values[index] = index / kColumns < fetched_count && col0 + index % kColumns < vdim ? fetched_v[j] : 0.f;
    }
    if (threadIdx.x < 2 * kTile) scalars[threadIdx.x] = static_cast<int>(threadIdx.x) < 2 * fetched_count ? fetched_s : 0.f;
  };

  // one token: the state decays, takes the token's write and is read out; returns the column's output
  auto walk = [&](const TokenOperands<RP>& now) {
    float sum_k[4] = {0.f, 0.f, 0.f, 0.f}, sum_q[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < RP; i += 4) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        S[i + e] *= now.g[i + e];
        sum_k[e] = fmaf(S[i + e], now.k[i + e], sum_k[e]);
        sum_q[e] = fmaf(S[i + e], now.q[i + e], sum_q[e]);
      }
    }
    const float from_k = column_sum<R>((sum_k[0] + sum_k[1]) + (sum_k[2] + sum_k[3]));
    const float from_q = column_sum<R>((sum_q[0] + sum_q[1]) + (sum_q[2] + sum_q[3]));
    const float u = now.beta * (now.value - from_k);
#pragma unroll
    for (int i = 0; i < RP; ++i) S[i] = fmaf(now.k[i], u, S[i]);
    return fmaf(u, now.kq, from_q);
  };

  // A whole tile's outputs wait in registers and are stored after the next tile's barriers: a barrier waits for every
  // store before it, and stores issued right before one would have the wave wait out their whole way to memory.
  float outs[kTile];
  int stored_from = -1;
  auto store_tile = [&]() {
    if (stored_from >= 0 && part == 0 && works) {
      float* out_at = raw_out + (static_cast<long>(stored_from) * heads + h) * vdim + col;
#pragma unroll
      for (int tt = 0; tt < kTile; ++tt) out_at[static_cast<long>(tt) * heads * vdim] = outs[tt];
    }
    stored_from = -1;
  };

  if (first < last) fetch(first);
  for (int t0 = first; t0 < last; t0 += kTile) {
    const int count = min(kTile, last - t0);
    __syncthreads();          // the tile before has been used by everybody
    lay_down();
    __syncthreads();
    if (t0 + kTile < last) fetch(t0 + kTile);
    store_tile();
    if (count == kTile) {
      // a whole tile: its tokens one after the other without a loop around them - every LDS address is a constant and
      // the tile's outputs leave in one go
      TokenOperands<RP> ahead[2];
      ahead[0].read(lds + part * SP, kArray, values + threadIdx.x / R, scalars);
#pragma unroll
      for (int tt = 0; tt < kTile; ++tt) {
        // the next token's reads are issued before this token's sums and stay there: a wave alone on its vector unit has
        // nobody to hide their way behind
        if (tt + 1 < kTile)
          ahead[(tt + 1) & 1].read(lds + (tt + 1) * 3 * kArray + part * SP, kArray,
                                   values + (tt + 1) * kColumns + threadIdx.x / R, scalars + 2 * (tt + 1));
        __builtin_amdgcn_sched_barrier(0);
        outs[tt] = walk(ahead[tt & 1]);
        __builtin_amdgcn_sched_barrier(0);
      }
      stored_from = t0;
    } else {
      for (int tt = 0; tt < count; ++tt) {
        TokenOperands<RP> now;
        now.read(lds + tt * 3 * kArray + part * SP, kArray, values + tt * kColumns + threadIdx.x / R, scalars + 2 * tt);
        const float out = walk(now);
        if (part == 0 && works) raw_out[(static_cast<long>(t0 + tt) * heads + h) * vdim + col] = out;
      }
    }
  }
  store_tile();
  if (works) {
#pragma unroll
    for (int i = 0; i < RP; i += 4) {
      const int d = part * RP + i;
      if (whole_fours && d < dim) {
        *reinterpret_cast<float4*>(kept + d) = make_float4(S[i], S[i + 1], S[i + 2], S[i + 3]);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (d + e < dim) kept[d + e] = S[i + e];
      }
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
                   int groups, int dim, int vdim, int longest, hipStream_t stream) {
  if (tokens <= 0 || seqs <= 0) return 0;
  if (heads <= 0 || groups <= 0 || heads % groups != 0 || dim <= 0 || vdim <= 0 || dim > 2048) return -2;
  float* prepared = workspace;
  float* raw = workspace + static_cast<long>(tokens) * prepared_width(heads, groups, dim);
  const int rp = dim <= 256 ? 4 : dim <= 512 ? 8 : dim <= 1024 ? 16 : 32;
  int R = 1;
  while (R * rp < dim) R *= 2;
  const int columns = 256 / R, column_blocks = (vdim + columns - 1) / columns;
  const long v_at = 2L * groups * dim;
  const unsigned grid = static_cast<unsigned>(static_cast<long>(seqs) * heads * column_blocks);
  const long items = static_cast<long>(tokens) * heads;
  const dim3 prepare_grid(static_cast<unsigned>(tokens), static_cast<unsigned>((groups + (heads * dim + 255) / 256 + 3) / 4));
#define AKV_RECUR_ARGS                                                                                                  \
  prepared, static_cast<const T*>(conv), conv_stride, v_at, state, state_stride, q_start, seq_slots, raw, heads, groups, dim, \
      vdim
#define AKV_RECUR(RP, R_)                                                                                   \
  do {                                                                                                      \
    if (longest < 16) delta_recur_kernel<T, RP, R_, 4><<<grid, 256, 0, stream>>>(AKV_RECUR_ARGS);           \
    else delta_recur_kernel<T, RP, R_, 32><<<grid, 256, 0, stream>>>(AKV_RECUR_ARGS);                       \
  } while (0)
  AKV_DISPATCH(dtype, T, {
    delta_prepare_kernel<T><<<prepare_grid, 256, 0, stream>>>(static_cast<const T*>(conv), conv_stride,
                                                              static_cast<const T*>(beta_logits), beta_stride, decay_logits,
                                                              decay_bias, rate, unit_eps, q_scale, prepared, heads, groups, dim);
    if (rp == 32) AKV_RECUR(32, 64);
    else if (rp == 16) AKV_RECUR(16, 64);
    else if (rp == 8) AKV_RECUR(8, 64);
    else if (R == 64) AKV_RECUR(4, 64);
    else if (R == 32) AKV_RECUR(4, 32);
    else if (R == 16) AKV_RECUR(4, 16);
    else if (R == 8) AKV_RECUR(4, 8);
    else if (R == 4) AKV_RECUR(4, 4);
    else if (R == 2) AKV_RECUR(4, 2);
    else AKV_RECUR(4, 1);
    delta_finish_kernel<T><<<static_cast<unsigned>((items + 3) / 4), 256, 0, stream>>>(raw, norm_weight, gates, norm_eps,
                                                                                      static_cast<T*>(out), items, vdim);
  });
#undef AKV_RECUR
#undef AKV_RECUR_ARGS
  return AKV_LAUNCH_STATUS();
}
}
