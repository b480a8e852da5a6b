// A routed feed-forward's token-wise kernels: the choice of experts from the router's float32 logits (softmax over all
// experts, the choice restricted to the best groups of neighbouring experts) and the experts' activation times the router's weight.

#include "common.h"
#include "api_parts.h"

using namespace akv;

namespace {

// One wave per token, from the router's logits (a product of the engine's, float32 sums).  scores = softmax(logits);
// a group's score is its best expert's; only experts of the `keep` best groups can be chosen; the `top` best of those
// are, each weighted by its own score (the weights are not renormalised).  Equal scores go to the lower index.
// gates[t, e] = score of a chosen expert, 0 of any other.
__global__ __launch_bounds__(256) void route_kernel(const float* __restrict__ logits, float* __restrict__ gates,
                                                    int tokens, int experts, int top, int groups, int keep) {
  extern __shared__ float lds[];
  const int waves = blockDim.x / kWave, wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1);
  const int n = blockIdx.x * waves + wave;
  if (n >= tokens) return;
  float* score = lds + static_cast<size_t>(wave) * (2 * experts + groups);   // [experts]
  float* open = score + experts;        // [experts]: 1 while the expert may still be chosen, 2 once it is chosen, 0 shut
  float* best = open + experts;         // [groups]
  float highest = -INFINITY;
  for (int e = lane; e < experts; e += kWave) {
    const float z = logits[static_cast<size_t>(n) * experts + e];
    score[e] = z;
    highest = fmaxf(highest, z);
  }
  highest = wave_max(highest);
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  if (lane == 0) {       // a few dozen numbers: one lane does the choosing
    float total = 0.f;
    for (int e = 0; e < experts; ++e) {
      score[e] = expf(score[e] - highest);
      total += score[e];
    }
    const int size = experts / groups;
    for (int e = 0; e < experts; ++e) {
      score[e] = score[e] / total;
      open[e] = 0.f;
    }
    for (int g = 0; g < groups; ++g) {
      float top_of = -INFINITY;
      for (int e = g * size; e < (g + 1) * size; ++e) top_of = fmaxf(top_of, score[e]);
      best[g] = top_of;
    }
    for (int k = 0; k < keep; ++k) {
      int at = -1;
      for (int g = 0; g < groups; ++g)
        if (best[g] >= 0.f && (at < 0 || best[g] > best[at])) at = g;
      if (at < 0) break;
      best[at] = -1.f;              // (scores are never negative)
      for (int e = at * size; e < (at + 1) * size; ++e) open[e] = 1.f;
    }
    for (int k = 0; k < top; ++k) {
      int at = -1;
      for (int e = 0; e < experts; ++e)
        if (open[e] == 1.f && (at < 0 || score[e] > score[at])) at = e;
      if (at < 0) break;
      open[at] = 2.f;
    }
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  for (int e = lane; e < experts; e += kWave) gates[static_cast<size_t>(n) * experts + e] = open[e] == 2.f ? score[e] : 0.f;
}

// act[t, e * ff + j] = gates[t, e] * relu(up[t, e * ff + j])^2, formed in float32 and rounded once; an expert that was
// not chosen gives exact zeros whatever its product holds.
template <typename T>
__global__ void gate_relu_squared_kernel(const T* __restrict__ up, const float* __restrict__ gates, T* __restrict__ act,
                                         long tokens, int experts, int ff) {
  const long index = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x;
  const long width = static_cast<long>(experts) * ff;
  if (index >= tokens * width) return;
  const long n = index / width;
  const int e = static_cast<int>((index % width) / ff);
  const float g = gates[n * experts + e];
  float value = 0.f;
  if (g != 0.f) {
    const float u = fmaxf(to_float(up[index]), 0.f);
    value = g * (u * u);
  }
  act[index] = from_float<T>(value);
}

// The same, eight values a thread (16 bytes of bfloat16 in, 16 out) where an expert's width is a multiple of 8.
__global__ void gate_relu_squared_by8_kernel(const bf16_t* __restrict__ up, const float* __restrict__ gates,
                                             bf16_t* __restrict__ act, long tokens, int experts, int ff) {
  const long index = (static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x) * 8;
  const long width = static_cast<long>(experts) * ff;
  if (index >= tokens * width) return;
  const long n = index / width;
  const int e = static_cast<int>((index % width) / ff);
  const float g = gates[n * experts + e];
  uint4 packed = make_uint4(0u, 0u, 0u, 0u);
  if (g != 0.f) {
    const uint4 raw = *reinterpret_cast<const uint4*>(up + index);
    const uint32_t words[4] = {raw.x, raw.y, raw.z, raw.w};
    uint32_t outs[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float lo = fmaxf(__uint_as_float(words[k] << 16), 0.f), hi = fmaxf(__uint_as_float(words[k] & 0xffff0000u), 0.f);
      outs[k] = bf16_pair(g * (lo * lo), g * (hi * hi));
    }
    packed = make_uint4(outs[0], outs[1], outs[2], outs[3]);
  }
  *reinterpret_cast<uint4*>(act + index) = packed;
}

// One wave per token: the `top` experts with the largest logits (equal logits go to the lower index) are chosen and
// weighted by the softmax over their logits alone; every other expert's gate is an exact zero.  A row may hold further
// logits after the experts' (`scored` in all): each of those becomes its own sigmoid - the gate of an expert that every
// token uses.  `law` 1: a chosen expert's gate is the sigmoid of its own logit (nothing is renormalised), the logits' rows
// hold the experts alone (`scored_in` of them) and every further column of a gates' row becomes 1: an expert that every token
// uses with no gate at all.
__global__ __launch_bounds__(256) void route_chosen_kernel(const float* __restrict__ logits, float* __restrict__ gates,
                                                           int tokens, int experts, int scored, int top, int law,
                                                           int scored_in) {
  extern __shared__ float lds[];
  const int waves = blockDim.x / kWave, wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1);
  const int n = blockIdx.x * waves + wave;
  if (n >= tokens) return;
  float* score = lds + static_cast<size_t>(wave) * (experts + 2 * top);   // [experts], -inf once chosen
  float* chosen_value = score + experts;                                  // [top]
  float* chosen_index = chosen_value + top;                               // [top]
  const float* row = logits + static_cast<size_t>(n) * scored_in;
  float* gate_row = gates + static_cast<size_t>(n) * scored;
  for (int e = lane; e < scored; e += kWave) {
    if (e < experts) {
      score[e] = row[e];
      gate_row[e] = 0.f;
    } else {
      gate_row[e] = law == 1 ? 1.f : 1.f / (1.f + expf(-row[e]));
    }
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int at = 0x7fffffff;
    for (int e = lane; e < experts; e += kWave) {
      const float z = score[e];
      if (z > best) {          // (ascending e: the lower index keeps an equal score)
        best = z;
        at = e;
      }
    }
#pragma unroll
    for (int offset = kWave / 2; offset > 0; offset >>= 1) {
      const float other = __shfl_xor(best, offset, kWave);
      const int other_at = __shfl_xor(at, offset, kWave);
      if (other > best || (other == best && other_at < at)) {
        best = other;
        at = other_at;
      }
    }
    if (at == 0x7fffffff) at = 0;     // (nothing finite left: cannot happen while top <= experts and logits are finite)
    if (lane == 0) {
      chosen_value[k] = best;
      chosen_index[k] = static_cast<float>(at);
      score[at] = -INFINITY;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
  if (lane == 0 && law == 1) {
    for (int k = 0; k < top; ++k) gate_row[static_cast<int>(chosen_index[k])] = 1.f / (1.f + expf(-chosen_value[k]));
  } else if (lane == 0) {
    const float highest = chosen_value[0];     // the first chosen is the largest
    float total = 0.f;
    for (int k = 0; k < top; ++k) total += expf(chosen_value[k] - highest);
    for (int k = 0; k < top; ++k) gate_row[static_cast<int>(chosen_index[k])] = expf(chosen_value[k] - highest) / total;
  }
}

// act[t, c] = gates[t, e(c)] * silu(gate_up[t, c]) * gate_up[t, columns + c]: the experts' gate rows first, then their up
// rows; column c belongs to expert c / ff while c < experts * ff and to the expert every token uses beyond (gate number
// `experts`).  Float32 up to the one rounding; an expert that was not chosen gives exact zeros.
template <typename T>
__global__ void gate_silu_mul_kernel(const T* __restrict__ gate_up, const float* __restrict__ gates, T* __restrict__ act,
                                     long tokens, int experts, int ff, int columns, int scored) {
  const long index = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (index >= tokens * columns) return;
  const long n = index / columns;
  const int c = static_cast<int>(index % columns);
  const int e = c < experts * ff ? c / ff : experts;
  const float g = gates[n * scored + e];
  float value = 0.f;
  if (g != 0.f) {
    const float z = to_float(gate_up[n * 2 * columns + c]);
    value = g * (z / (1.f + expf(-z)) * to_float(gate_up[n * 2 * columns + columns + c]));
  }
  act[index] = from_float<T>(value);
}

// The same, eight values a thread (16 bytes of bfloat16 per load and store), where every expert's width and the shared
// one's are multiples of 8: a thread's eight columns then belong to one expert.
__global__ void gate_silu_mul_by8_kernel(const bf16_t* __restrict__ gate_up, const float* __restrict__ gates,
                                         bf16_t* __restrict__ act, long tokens, int experts, int ff, int columns,
                                         int scored) {
  const long index = (static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x) * 8;
  if (index >= tokens * columns) return;
  const long n = index / columns;
  const int c = static_cast<int>(index % columns);
  const int e = c < experts * ff ? c / ff : experts;
  const float g = gates[n * scored + e];
  uint4 packed = make_uint4(0u, 0u, 0u, 0u);
  if (g != 0.f) {
    const uint4 zs = *reinterpret_cast<const uint4*>(gate_up + n * 2 * columns + c);
    const uint4 us = *reinterpret_cast<const uint4*>(gate_up + n * 2 * columns + columns + c);
    const uint32_t zw[4] = {zs.x, zs.y, zs.z, zs.w}, uw[4] = {us.x, us.y, us.z, us.w};
    uint32_t outs[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float z0 = __uint_as_float(zw[k] << 16), z1 = __uint_as_float(zw[k] & 0xffff0000u);
      const float u0 = __uint_as_float(uw[k] << 16), u1 = __uint_as_float(uw[k] & 0xffff0000u);
      outs[k] = bf16_pair(g * (z0 / (1.f + expf(-z0)) * u0), g * (z1 / (1.f + expf(-z1)) * u1));
    }
    packed = make_uint4(outs[0], outs[1], outs[2], outs[3]);
  }
  *reinterpret_cast<uint4*>(act + index) = packed;
}

// act[t, c] = f(gates[t, e(c)] * up[t, c]) (`inside`: the router's weight multiplies what enters the activation, which for
// an expert without biases is the expert run on the weighted input) or gates[t, e(c)] * f(up[t, c]); f 0: the exact gelu
// (erf), 1: its tanh form, 2: silu, 3: relu squared.  Column c belongs to expert c / ff below experts * ff and to the expert
// every token uses beyond (gate number `experts`).  Float32 up to the one rounding; an expert that was not chosen gives
// exact zeros.
__device__ __forceinline__ float expert_activation(float z, int kind) {
  switch (kind) {
    case 0: return 0.5f * z * (1.f + erff(z * 0.7071067811865476f));
    case 1: return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
    case 2: return z / (1.f + expf(-z));
    default: return z > 0.f ? z * z : 0.f;
  }
}

template <typename T>
__global__ void gate_activation_kernel(const T* __restrict__ up, const float* __restrict__ gates, T* __restrict__ act,
                                       long tokens, int experts, int ff, int columns, int scored, int kind, int inside) {
  const long index = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (index >= tokens * columns) return;
  const long n = index / columns;
  const int c = static_cast<int>(index % columns);
  const float g = gates[n * scored + (c < experts * ff ? c / ff : experts)];
  float value = 0.f;
  if (g != 0.f) {
    const float z = to_float(up[index]);
    value = inside ? expert_activation(g * z, kind) : g * expert_activation(z, kind);
  }
  act[index] = from_float<T>(value);
}

// The same, eight values a thread, where every expert's width and the shared one's are multiples of 8.
__global__ void gate_activation_by8_kernel(const bf16_t* __restrict__ up, const float* __restrict__ gates,
                                           bf16_t* __restrict__ act, long tokens, int experts, int ff, int columns, int scored,
                                           int kind, int inside) {
  const long index = (static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x) * 8;
  if (index >= tokens * columns) return;
  const long n = index / columns;
  const int c = static_cast<int>(index % columns);
  const float g = gates[n * scored + (c < experts * ff ? c / ff : experts)];
  uint4 packed = make_uint4(0u, 0u, 0u, 0u);
  if (g != 0.f) {
    const uint4 zs = *reinterpret_cast<const uint4*>(up + index);
    const uint32_t zw[4] = {zs.x, zs.y, zs.z, zs.w};
    uint32_t outs[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float z0 = __uint_as_float(zw[k] << 16), z1 = __uint_as_float(zw[k] & 0xffff0000u);
      outs[k] = inside ? bf16_pair(expert_activation(g * z0, kind), expert_activation(g * z1, kind))
                       : bf16_pair(g * expert_activation(z0, kind), g * expert_activation(z1, kind));
    }
    packed = make_uint4(outs[0], outs[1], outs[2], outs[3]);
  }
  *reinterpret_cast<uint4*>(act + index) = packed;
}

}  // namespace

extern "C" {

int akv_gate_activation(const void* up, const float* gates, void* act, int dtype, long tokens, int experts, int ff,
                        int columns, int scored, int kind, int inside, hipStream_t stream) {
  const long count = tokens * columns;
  if (count <= 0) return 0;
  if (columns < experts * ff || scored < experts + (columns > experts * ff ? 1 : 0) || kind < 0 || kind > 3) return -2;
  if (dtype == kBF16 && ff % 8 == 0 && columns % 8 == 0 && reinterpret_cast<uintptr_t>(up) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(act) % 16 == 0) {
    gate_activation_by8_kernel<<<static_cast<unsigned>((count / 8 + 255) / 256), 256, 0, stream>>>(
        static_cast<const bf16_t*>(up), gates, static_cast<bf16_t*>(act), tokens, experts, ff, columns, scored, kind, inside);
    return AKV_LAUNCH_STATUS();
  }
  AKV_DISPATCH(dtype, T, gate_activation_kernel<T><<<static_cast<unsigned>((count + 255) / 256), 256, 0, stream>>>(
                             static_cast<const T*>(up), gates, static_cast<T*>(act), tokens, experts, ff, columns, scored,
                             kind, inside));
  return AKV_LAUNCH_STATUS();
}

int akv_route_chosen(const float* logits, float* gates, int tokens, int experts, int scored, int top, int law,
                     hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (experts <= 0 || top <= 0 || top > experts || scored < experts || law < 0 || law > 1) return -2;
  const int waves = 4;
  const size_t lds_bytes = static_cast<size_t>(waves) * (experts + 2 * top) * 4;
  if (lds_bytes > 64 * 1024) return -2;
  route_chosen_kernel<<<(tokens + waves - 1) / waves, waves * kWave, lds_bytes, stream>>>(
      logits, gates, tokens, experts, scored, top, law, law == 1 ? experts : scored);
  return AKV_LAUNCH_STATUS();
}

int akv_gate_silu_mul(const void* gate_up, const float* gates, void* act, int dtype, long tokens, int experts, int ff,
                      int columns, int scored, hipStream_t stream) {
  const long count = tokens * columns;
  if (count <= 0) return 0;
  if (columns < experts * ff || scored < experts + (columns > experts * ff ? 1 : 0)) return -2;
  if (dtype == kBF16 && ff % 8 == 0 && columns % 8 == 0 && reinterpret_cast<uintptr_t>(gate_up) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(act) % 16 == 0) {
    gate_silu_mul_by8_kernel<<<static_cast<unsigned>((count / 8 + 255) / 256), 256, 0, stream>>>(
        static_cast<const bf16_t*>(gate_up), gates, static_cast<bf16_t*>(act), tokens, experts, ff, columns, scored);
    return AKV_LAUNCH_STATUS();
  }
  AKV_DISPATCH(dtype, T, gate_silu_mul_kernel<T><<<static_cast<unsigned>((count + 255) / 256), 256, 0, stream>>>(
                             static_cast<const T*>(gate_up), gates, static_cast<T*>(act), tokens, experts, ff, columns,
                             scored));
  return AKV_LAUNCH_STATUS();
}

int akv_route(const float* logits, float* gates, int tokens, int experts, int top, int groups, int keep,
              hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (experts <= 0 || groups <= 0 || experts % groups || keep <= 0 || keep > groups || top <= 0 || top > experts) return -2;
  const int waves = 4;
  const size_t lds_bytes = static_cast<size_t>(waves) * (2 * experts + groups) * 4;
  if (lds_bytes > 64 * 1024) return -2;
  route_kernel<<<(tokens + waves - 1) / waves, waves * kWave, lds_bytes, stream>>>(logits, gates, tokens, experts, top,
                                                                                   groups, keep);
  return AKV_LAUNCH_STATUS();
}

int akv_gate_relu_squared(const void* up, const float* gates, void* act, int dtype, long tokens, int experts, int ff,
                          hipStream_t stream) {
  const long count = tokens * experts * ff;
  if (count <= 0) return 0;
  if (dtype == kBF16 && ff % 8 == 0) {
    gate_relu_squared_by8_kernel<<<static_cast<unsigned>((count / 8 + 255) / 256), 256, 0, stream>>>(
        static_cast<const bf16_t*>(up), gates, static_cast<bf16_t*>(act), tokens, experts, ff);
    return AKV_LAUNCH_STATUS();
  }
  AKV_DISPATCH(dtype, T, gate_relu_squared_kernel<T><<<static_cast<unsigned>((count + 255) / 256), 256, 0, stream>>>(
                             static_cast<const T*>(up), gates, static_cast<T*>(act), tokens, experts, ff));
  return AKV_LAUNCH_STATUS();
}
}
