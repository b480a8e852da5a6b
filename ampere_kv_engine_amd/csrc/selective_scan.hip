// A selective scan with its short causal convolution.  What a request carries from token to token lies in its slot, in
// float32: S [channels, n_state], then the convolution's last taps - 1 inputs [taps - 1, channels], oldest first.
//
//   x_t = silu(sum_k w[c, k] * in[t - (taps - 1 - k)] + b[c])                (inputs before the sequence's start are 0)
//   S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n;   y_c = sum_n S[c, n] C_n + D_c x_c;   out = y * silu(z)
// with dt = softplus(dt_raw).  Step sizes, decays, exponentials, the state and the sums are float32.

#include "common.h"
#include "api_parts.h"

using namespace akv;

namespace {

__device__ __forceinline__ float silu(float v) { return v / (1.f + expf(-v)); }
__device__ __forceinline__ float softplus(float v) { return v > 20.f ? v : log1pf(expf(v)); }

// ---- convolution over the portion and what the slot remembers of the tokens before it --------------------------------
template <typename T, typename TW, bool SILU>
__global__ __launch_bounds__(256) void conv_silu_kernel(const T* __restrict__ x, long x_stride, const TW* __restrict__ weight,
                                                        const TW* __restrict__ bias, const float* __restrict__ state,
                                                        long state_stride, long conv_at,
                                                        const int* __restrict__ seq_of_token,
                                                        const int* __restrict__ q_start, const int* __restrict__ seq_slots,
                                                        T* __restrict__ out, int channels, int taps) {
  const int n = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int r = seq_of_token[n];
  const int first = q_start[r];
  const float* kept = state + static_cast<long>(seq_slots[r]) * state_stride + conv_at;   // [taps - 1][channels]
  float acc = bias != nullptr ? to_float(bias[c]) : 0.f;
  for (int k = 0; k < taps; ++k) {
    const int row = n - (taps - 1 - k);
    float v;
    if (row >= first) {
      v = to_float(x[row * x_stride + c]);
    } else {
      const int back = first - row;                  // 1 .. taps - 1 tokens before the portion
      v = kept[static_cast<long>(taps - 1 - back) * channels + c];
    }
    acc = fmaf(to_float(weight[static_cast<long>(c) * taps + k]), v, acc);
  }
  out[static_cast<long>(n) * channels + c] = from_float<T>(SILU ? silu(acc) : acc);
}

// The same sums for eight neighbouring channels and TOK neighbouring tokens a thread, where the number of taps is one the
// kernel is compiled for, channels come in eights and rows are 16-byte aligned: a row's eight inputs are one load and
// serve every token of the thread that reaches back to them; the eight channels' weights are TAPS loads.  A token's
// taps that lie before its request's portion come from the slot, as above.
template <typename T> struct Eight {
  static constexpr int kChunks = sizeof(T) * 8 / 16;
  uint4 bits[kChunks];
  __device__ __forceinline__ void load(const T* at) {
#pragma unroll
    for (int i = 0; i < kChunks; ++i) bits[i] = reinterpret_cast<const uint4*>(at)[i];
  }
  __device__ __forceinline__ void store(T* at) const {
#pragma unroll
    for (int i = 0; i < kChunks; ++i) reinterpret_cast<uint4*>(at)[i] = bits[i];
  }
  __device__ __forceinline__ float get(int i) const { return to_float(reinterpret_cast<const T*>(bits)[i]); }
  __device__ __forceinline__ void set(int i, float v) { reinterpret_cast<T*>(bits)[i] = from_float<T>(v); }
};

template <typename T, typename TW, bool SILU, int TAPS, int TOK>
__global__ __launch_bounds__(256) void conv_eights_kernel(const T* __restrict__ x, long x_stride, const TW* __restrict__ weight,
                                                          const TW* __restrict__ bias, const float* __restrict__ state,
                                                          long state_stride, long conv_at,
                                                          const int* __restrict__ seq_of_token,
                                                          const int* __restrict__ q_start, const int* __restrict__ seq_slots,
                                                          T* __restrict__ out, int tokens, int channels) {
  const int n0 = blockIdx.x * TOK;
  const int c = (blockIdx.y * blockDim.x + threadIdx.x) * 8;
  if (c >= channels) return;
  float w[TAPS][8];              // w[k][i]: tap k of channel c + i
  {
    Eight<TW> chunk[TAPS];
#pragma unroll
    for (int j = 0; j < TAPS; ++j) chunk[j].load(weight + static_cast<long>(c) * TAPS + j * 8);
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int k = 0; k < TAPS; ++k) w[k][i] = chunk[(i * TAPS + k) / 8].get((i * TAPS + k) % 8);
  }
  float b[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) b[i] = bias != nullptr ? to_float(bias[c + i]) : 0.f;
  Eight<T> rows[TOK + TAPS - 1];       // rows[j]: token n0 - (TAPS - 1) + j
#pragma unroll
  for (int j = 0; j < TOK + TAPS - 1; ++j) {
    const int row = n0 - (TAPS - 1) + j;
    if (row >= 0 && row < tokens) rows[j].load(x + static_cast<long>(row) * x_stride + c);
  }
#pragma unroll
  for (int t = 0; t < TOK; ++t) {
    const int n = n0 + t;
    if (n >= tokens) break;
    const int r = seq_of_token[n];
    const int first = q_start[r];
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = b[i];
#pragma unroll
    for (int k = 0; k < TAPS; ++k) {
      const int row = n - (TAPS - 1 - k);
      if (row >= first) {
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = fmaf(w[k][i], rows[t + k].get(i), acc[i]);
      } else {
        const float* kept = state + static_cast<long>(seq_slots[r]) * state_stride + conv_at
                            + static_cast<long>(TAPS - 1 - (first - row)) * channels + c;
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = fmaf(w[k][i], kept[i], acc[i]);
      }
    }
    Eight<T> result;
#pragma unroll
    for (int i = 0; i < 8; ++i) result.set(i, SILU ? silu(acc[i]) : acc[i]);
    result.store(out + static_cast<long>(n) * channels + c);
  }
}

// After the convolution has read the old inputs: the slot keeps the last taps - 1 of (old inputs, the portion's).
template <typename T>
__global__ __launch_bounds__(256) void conv_state_update_kernel(const T* __restrict__ x, long x_stride,
                                                                float* __restrict__ state, long state_stride,
                                                                long conv_at, const int* __restrict__ q_start,
                                                                const int* __restrict__ seq_slots, int channels,
                                                                int taps) {
  const int r = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int first = q_start[r], count = q_start[r + 1] - first;
  float* kept = state + static_cast<long>(seq_slots[r]) * state_stride + conv_at;
  // entry k of the new state is input number count - (taps - 1) + k of the portion; negative numbers reach into the
  // old state at taps - 1 + that number, which is at least k: ascending k never reads what it has already replaced
  for (int k = 0; k < taps - 1; ++k) {
    const int index = count - (taps - 1) + k;
    const float v = index >= 0 ? to_float(x[(first + index) * x_stride + c])
                               : kept[static_cast<long>(taps - 1 + index) * channels + c];
    kept[static_cast<long>(k) * channels + c] = v;
  }
}

// ---- step sizes: dt <- softplus(dt), every element for itself (inside the scan each of a channel's lanes would repeat it) --
__global__ void softplus_kernel(float* __restrict__ values, long count) {
  const long i = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < count) values[i] = softplus(values[i]);
}

// ---- the scan ---------------------------------------------------------------------------------------------------------
// A channel's state is spread over LP lanes (LP: the state's size rounded up to a power of two, at most 64; a lane owns
// states lane, lane + LP, ... - NK of them): per token a lane forms one decay and one product per state it owns, and
// the channel's output is the sum over its lanes, which a butterfly of lane exchanges leaves in all of them.  The
// recurrence of a state is a chain through all tokens; everything else of a token hangs off that chain, so tokens are
// taken kScanAhead at a time: their inputs are asked for together, the block lays their B and C, which all channels
// share, into LDS once, and the eight sums' exchanges overlap.  exp(dt A) is formed as exp2(dt (A log2 e)).
constexpr int kScanAhead = 8;
constexpr float kLog2e = 1.4426950408889634f;

template <typename T, int LP, int NK>
__global__ __launch_bounds__(256) void selective_scan_kernel(const T* __restrict__ x, const float* __restrict__ dt,
                                                             const float* __restrict__ bc, const T* __restrict__ z,
                                                             long z_stride, const float* __restrict__ a,
                                                             const float* __restrict__ d, float* __restrict__ state,
                                                             long state_stride, const int* __restrict__ q_start,
                                                             const int* __restrict__ seq_slots, T* __restrict__ out,
                                                             int channels, int n_state) {
  extern __shared__ float shared_bc[];                // two of [kScanAhead][2 * n_state]
  const int r = blockIdx.x;
  const int part = threadIdx.x % LP;                  // which of the channel's lanes
  const int c = blockIdx.y * (256 / LP) + threadIdx.x / LP;
  const bool works = c < channels;
  const int cc = works ? c : channels - 1;            // (lanes beyond the channels keep the block's steps and store nothing)
  float* kept = state + static_cast<long>(seq_slots[r]) * state_stride + static_cast<long>(cc) * n_state;
  float S[NK], A[NK];
#pragma unroll
  for (int k = 0; k < NK; ++k) {
    const int n = part + k * LP;
    S[k] = n < n_state ? kept[n] : 0.f;
    A[k] = n < n_state ? a[static_cast<long>(cc) * n_state + n] * kLog2e : 0.f;
  }
  const float skip = d[cc];
  const int first = q_start[r], last = q_start[r + 1];
  const int row = 2 * n_state;
  // the tokens after these are asked for while these are worked on: their inputs into a second set of registers, their
  // B and C into the other half of the LDS buffer
  float xn[kScanAhead], stepn[kScanAhead], gaten[kScanAhead];
  auto fetch = [&](int t0, float* into) {
    for (int e = threadIdx.x; e < kScanAhead * row; e += blockDim.x) {
      const int t = min(t0 + e / row, last - 1);
      into[e] = bc[static_cast<long>(t) * row + e % row];
    }
#pragma unroll
    for (int u = 0; u < kScanAhead; ++u) {
      const long t = min(t0 + u, last - 1);
      xn[u] = to_float(x[t * channels + cc]);
      stepn[u] = dt[t * channels + cc];
      gaten[u] = to_float(z[t * z_stride + cc]);
    }
  };
  if (first < last) fetch(first, shared_bc);
  int turn = 0;
  for (int t0 = first; t0 < last; t0 += kScanAhead, turn ^= 1) {
    float xv[kScanAhead], step[kScanAhead], gate[kScanAhead], y[kScanAhead];
#pragma unroll
    for (int u = 0; u < kScanAhead; ++u) {
      xv[u] = xn[u];
      step[u] = stepn[u];
      gate[u] = gaten[u];
    }
    __syncthreads();                                  // this turn's B and C are in place; the other half has been read
    const float* mine_bc = shared_bc + turn * kScanAhead * row;
    if (t0 + kScanAhead < last) fetch(t0 + kScanAhead, shared_bc + (turn ^ 1) * kScanAhead * row);
#pragma unroll
    for (int u = 0; u < kScanAhead; ++u) {
      const float h = step[u];                        // (softplus has been taken)
      const float drive = h * xv[u];
      const float* B = mine_bc + u * row;
      const float* C = B + n_state;
      float sum = 0.f;
      if (t0 + u < last) {                            // (uniform over the block)
#pragma unroll
        for (int k = 0; k < NK; ++k) {
          const int n = part + k * LP;
          if (n < n_state) {
            S[k] = fmaf(__builtin_amdgcn_exp2f(h * A[k]), S[k], drive * B[n]);
            sum = fmaf(S[k], C[n], sum);
          }
        }
      }
      y[u] = sum;
    }
#pragma unroll
    for (int offset = LP / 2; offset > 0; offset >>= 1)
#pragma unroll
      for (int u = 0; u < kScanAhead; ++u) y[u] += __shfl_xor(y[u], offset, kWave);
    if (works && part < kScanAhead && t0 + part < last) {      // lane u of a channel stores token u
      float mine = 0.f, xm = 0.f, gm = 0.f;
#pragma unroll
      for (int u = 0; u < kScanAhead; ++u)
        if (u == part) {
          mine = y[u];
          xm = xv[u];
          gm = gate[u];
        }
      out[static_cast<long>(t0 + part) * channels + c] = from_float<T>(fmaf(skip, xm, mine) * silu(gm));
    }
    if constexpr (LP < kScanAhead) {                  // fewer lanes than tokens: lane 0 stores the rest
      if (works && part == 0) {
#pragma unroll
        for (int u = LP; u < kScanAhead; ++u)
          if (t0 + u < last) out[static_cast<long>(t0 + u) * channels + c] = from_float<T>(fmaf(skip, xv[u], y[u]) * silu(gate[u]));
      }
    }
  }
  if (!works) return;
#pragma unroll
  for (int k = 0; k < NK; ++k) {
    const int n = part + k * LP;
    if (n < n_state) kept[n] = S[k];
  }
}

}  // namespace

extern "C" {

int akv_conv_silu(const void* x, long x_stride, int dtype, const void* weight, const void* bias, int w_dtype,
                  const float* state, long state_stride, long conv_at, const int* seq_of_token, const int* q_start,
                  const int* seq_slots, void* out, int tokens, int channels, int taps, hipStream_t stream) {
  return akv_conv_taps(x, x_stride, dtype, weight, bias, w_dtype, state, state_stride, conv_at, seq_of_token, q_start,
                       seq_slots, out, tokens, channels, taps, 1, stream);
}

int akv_conv_taps(const void* x, long x_stride, int dtype, const void* weight, const void* bias, int w_dtype,
                  const float* state, long state_stride, long conv_at, const int* seq_of_token, const int* q_start,
                  const int* seq_slots, void* out, int tokens, int channels, int taps, int activation,
                  hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (taps < 1 || channels <= 0 || activation < 0 || activation > 1) return -2;
  const dim3 grid(tokens, (channels + 255) / 256);
  // eight channels a thread where rows, weights and outputs allow 16-byte accesses and the taps are among the compiled
  // ones (a few tokens fill the device better with a thread a channel; both kernels sum in the same order)
  const bool eights = tokens >= 32 && channels % 8 == 0 && x_stride % 8 == 0 && taps >= 2 && taps <= 5 &&
                      reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0 &&
                      reinterpret_cast<uintptr_t>(weight) % 16 == 0;
  const int per_thread = tokens >= 256 ? 4 : 1;
  const dim3 grid_eights((tokens + per_thread - 1) / per_thread, (channels / 8 + 255) / 256);
#define AKV_CONV_EIGHTS(T, TW, ACT, TAPS)                                                                                  \
  do {                                                                                                                     \
    if (per_thread == 4) conv_eights_kernel<T, TW, ACT, TAPS, 4><<<grid_eights, 256, 0, stream>>>(                         \
        static_cast<const T*>(x), x_stride, static_cast<const TW*>(weight), static_cast<const TW*>(bias), state,           \
        state_stride, conv_at, seq_of_token, q_start, seq_slots, static_cast<T*>(out), tokens, channels);                  \
    else conv_eights_kernel<T, TW, ACT, TAPS, 1><<<grid_eights, 256, 0, stream>>>(                                         \
        static_cast<const T*>(x), x_stride, static_cast<const TW*>(weight), static_cast<const TW*>(bias), state,           \
        state_stride, conv_at, seq_of_token, q_start, seq_slots, static_cast<T*>(out), tokens, channels);                  \
  } while (0)
#define AKV_CONV_EIGHTS_TAPS(T, TW, ACT)                 \
  do {                                                   \
    if (taps == 2) AKV_CONV_EIGHTS(T, TW, ACT, 2);       \
    else if (taps == 3) AKV_CONV_EIGHTS(T, TW, ACT, 3);  \
    else if (taps == 4) AKV_CONV_EIGHTS(T, TW, ACT, 4);  \
    else AKV_CONV_EIGHTS(T, TW, ACT, 5);                 \
  } while (0)
#define AKV_CONV_ARGS(T, TW)                                                                                         \
  static_cast<const T*>(x), x_stride, static_cast<const TW*>(weight), static_cast<const TW*>(bias), state, state_stride, \
      conv_at, seq_of_token, q_start, seq_slots, static_cast<T*>(out), channels, taps
#define AKV_CONV(T, TW)                                                                          \
  do {                                                                                           \
    if (eights && activation == 1) AKV_CONV_EIGHTS_TAPS(T, TW, true);                            \
    else if (eights) AKV_CONV_EIGHTS_TAPS(T, TW, false);                                         \
    else if (activation == 1) conv_silu_kernel<T, TW, true><<<grid, 256, 0, stream>>>(AKV_CONV_ARGS(T, TW)); \
    else conv_silu_kernel<T, TW, false><<<grid, 256, 0, stream>>>(AKV_CONV_ARGS(T, TW));           \
  } while (0)
  if (dtype == kF32 && w_dtype == kF32) AKV_CONV(float, float);
  else if (dtype == kBF16 && w_dtype == kBF16) AKV_CONV(bf16_t, bf16_t);
  else if (dtype == kBF16 && w_dtype == kF32) AKV_CONV(bf16_t, float);
  else return -1;
#undef AKV_CONV
#undef AKV_CONV_ARGS
#undef AKV_CONV_EIGHTS_TAPS
#undef AKV_CONV_EIGHTS
  return AKV_LAUNCH_STATUS();
}

int akv_conv_state_update(const void* x, long x_stride, int dtype, float* state, long state_stride, long conv_at,
                          const int* q_start, const int* seq_slots, int seqs, int channels, int taps,
                          hipStream_t stream) {
  if (seqs <= 0 || taps <= 1) return 0;
  const dim3 grid(seqs, (channels + 255) / 256);
  AKV_DISPATCH(dtype, T, conv_state_update_kernel<T><<<grid, 256, 0, stream>>>(
                             static_cast<const T*>(x), x_stride, state, state_stride, conv_at, q_start, seq_slots, channels,
                             taps));
  return AKV_LAUNCH_STATUS();
}

int akv_selective_scan(const void* x, int dtype, float* dt, const float* bc, const void* z, long z_stride,
                       const float* a, const float* d, float* state, long state_stride, const int* q_start,
                       const int* seq_slots, void* out, int tokens, int seqs, int channels, int n_state,
                       hipStream_t stream) {
  if (seqs <= 0) return 0;
  if (n_state <= 0 || n_state > 256) return -2;
  if (tokens > 0) {
    const long count = static_cast<long>(tokens) * channels;
    softplus_kernel<<<static_cast<unsigned>((count + 255) / 256), 256, 0, stream>>>(dt, count);
  }
  int lanes = 1;
  while (lanes < n_state && lanes < 64) lanes <<= 1;
  const dim3 grid(seqs, (channels + 256 / lanes - 1) / (256 / lanes));
#define AKV_SCAN(T, LP, NK)                                                                                         \
  selective_scan_kernel<T, LP, NK><<<grid, 256, 2 * kScanAhead * 2 * n_state * 4, stream>>>(                              \
      static_cast<const T*>(x), dt, bc, static_cast<const T*>(z), z_stride, a, d, state, state_stride, q_start,     \
      seq_slots, static_cast<T*>(out), channels, n_state)
  AKV_DISPATCH(dtype, T, {
    if (lanes == 1) AKV_SCAN(T, 1, 1);
    else if (lanes == 2) AKV_SCAN(T, 2, 1);
    else if (lanes == 4) AKV_SCAN(T, 4, 1);
    else if (lanes == 8) AKV_SCAN(T, 8, 1);
    else if (lanes == 16) AKV_SCAN(T, 16, 1);
    else if (lanes == 32) AKV_SCAN(T, 32, 1);
    else if (n_state <= 64) AKV_SCAN(T, 64, 1);
    else if (n_state <= 128) AKV_SCAN(T, 64, 2);
    else AKV_SCAN(T, 64, 4);
  });
#undef AKV_SCAN
  return AKV_LAUNCH_STATUS();
}
}
