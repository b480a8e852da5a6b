// Token-wise kernels of designs whose norms and residual sum are float32 from end to end: an embedding that adds a row
// of a hashed table of token pairs, and the norm kernel of blocks that norm every branch before AND after.  Nothing
// is rounded between a sum of squares and the one store of a result.

#include "common.h"
#include "api_parts.h"

using namespace akv;

namespace {

constexpr unsigned kPoison = 0x7fc00000u;

// ---- embedding plus a row of the pair table ---------------------------------------------------------------------------
// The pair of a portion's first token reaches back into the previous step: the request's slot keeps the id it was
// fed last (kSlotFedToken), written by note_fed_tokens_kernel after this kernel has read it.
template <typename T>
__global__ __launch_bounds__(256) void embed_pairs_kernel(
    const int* __restrict__ ids, const T* __restrict__ table, const T* __restrict__ pairs, float* __restrict__ out,
    int hidden, int vocab, long buckets, long mul_prev, long mul_cur, const int* __restrict__ seq_of_token,
    const int* __restrict__ q_start, const int* __restrict__ positions, const int* __restrict__ seq_slots,
    const int* __restrict__ slot_words) {
  const int n = blockIdx.x;
  const int r = seq_of_token[n];
  const long slot = seq_slots[r];
  int id = ids[n];
  if (id == -1) id = slot_words[slot * kSlotWords + kSlotLastToken];
  long pair_row = buckets;                   // a request's first token: the table's last row
  bool bad = id < 0 || id >= vocab;
  if (positions[n] > 0) {
    const int prev = n > q_start[r] ? ids[n - 1] : slot_words[slot * kSlotWords + kSlotFedToken];
    bad = bad || prev < 0 || prev >= vocab;
    const long mixed = (static_cast<long>(prev) * mul_prev + static_cast<long>(id) * mul_cur) % buckets;
    pair_row = mixed < 0 ? mixed + buckets : mixed;
  }
  float* dst = out + static_cast<size_t>(n) * hidden;
  if (bad) {     // never read outside a table; a poisoned row shows the fault downstream
    for (int d = threadIdx.x; d < hidden; d += blockDim.x) dst[d] = __uint_as_float(kPoison);
    return;
  }
  const T* token_row = table + static_cast<size_t>(id) * hidden;
  const T* pair = pairs + static_cast<size_t>(pair_row) * hidden;
  for (int d = threadIdx.x; d < hidden; d += blockDim.x) dst[d] = to_float(token_row[d]) + to_float(pair[d]);
}

__global__ void note_fed_tokens_kernel(const int* __restrict__ ids, const int* __restrict__ q_start,
                                       const int* __restrict__ seq_slots, int* __restrict__ slot_words, int seqs) {
  const int r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= seqs) return;
  const long slot = seq_slots[r];
  int id = ids[q_start[r + 1] - 1];
  if (id == -1) id = slot_words[slot * kSlotWords + kSlotLastToken];
  slot_words[slot * kSlotWords + kSlotFedToken] = id;
}

// ---- stream += norm_post(delta); out = norm_pre(stream) -----------------------------------------------------------------
// One block per row.  Rows of up to 256 * 4 * GROUPS elements (a multiple of 4) stay in registers from their one trip to
// memory to the store; others take three passes over a row that the caches hold: the branch's sum of squares; the
// update of the residual sum, which gathers the new sum of squares as it goes; the normed row.
template <typename T> __device__ __forceinline__ float4 read4(const T* p);
template <> __device__ __forceinline__ float4 read4<float>(const float* p) { return *reinterpret_cast<const float4*>(p); }
template <> __device__ __forceinline__ float4 read4<bf16_t>(const bf16_t* p) {
  const uint2 v = *reinterpret_cast<const uint2*>(p);
  return make_float4(__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u), __uint_as_float(v.y << 16),
                     __uint_as_float(v.y & 0xffff0000u));
}
template <typename T> __device__ __forceinline__ void write4(T* p, float4 v);
template <> __device__ __forceinline__ void write4<float>(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
template <> __device__ __forceinline__ void write4<bf16_t>(bf16_t* p, float4 v) {
  uint2 packed;
  packed.x = bf16_pair(v.x, v.y);
  packed.y = bf16_pair(v.z, v.w);
  *reinterpret_cast<uint2*>(p) = packed;
}

template <typename T, int GROUPS>
__global__ __launch_bounds__(256) void norm_add_norm_rows_kernel(float* __restrict__ stream, const T* __restrict__ delta,
                                                                 const float* __restrict__ post_weight, float post_eps,
                                                                 const float* __restrict__ pre_weight, float pre_eps,
                                                                 T* __restrict__ out, int hidden, float delta_scale,
                                                                 const float* __restrict__ offset,
                                                                 const T* __restrict__ delta2) {
  __shared__ float scratch[16];
  const size_t base = static_cast<size_t>(blockIdx.x) * hidden;
  float4 kept[GROUPS], added[GROUPS];
  // every load goes out before anything waits (a group beyond the row reads its last four values and counts for nothing)
#pragma unroll
  for (int j = 0; j < GROUPS; ++j) {
    const int i = min((j * 256 + static_cast<int>(threadIdx.x)) * 4, hidden - 4);
    kept[j] = read4<float>(stream + base + i);
    if (delta != nullptr) added[j] = read4<T>(delta + base + i);
    if (delta2 != nullptr) {      // a second branch beside the first: the two are added in float32 before they meet the sum
      const float4 b = read4<T>(delta2 + base + i);
      added[j] = make_float4(added[j].x + b.x, added[j].y + b.y, added[j].z + b.z, added[j].w + b.w);
    }
  }
  float squares = 0.f;
  if (delta != nullptr) {
    float post_scale = 1.f;
    if (post_weight != nullptr) {
      float acc = 0.f;
#pragma unroll
      for (int j = 0; j < GROUPS; ++j)
        if ((j * 256 + static_cast<int>(threadIdx.x)) * 4 < hidden)
          acc += added[j].x * added[j].x + added[j].y * added[j].y + added[j].z * added[j].z + added[j].w * added[j].w;
      post_scale = rsqrtf(block_sum(acc, scratch) / static_cast<float>(hidden) + post_eps);
    }
#pragma unroll
    for (int j = 0; j < GROUPS; ++j) {
      const int i = (j * 256 + static_cast<int>(threadIdx.x)) * 4;
      if (i >= hidden) continue;
      float4 d = added[j];
      if (post_weight != nullptr) {
        const float4 w = read4<float>(post_weight + i);
        d = make_float4(d.x * post_scale * w.x, d.y * post_scale * w.y, d.z * post_scale * w.z, d.w * post_scale * w.w);
      } else {
        d = make_float4(d.x * delta_scale, d.y * delta_scale, d.z * delta_scale, d.w * delta_scale);
      }
      kept[j] = make_float4(kept[j].x + d.x, kept[j].y + d.y, kept[j].z + d.z, kept[j].w + d.w);
      if (offset == nullptr) write4<float>(stream + base + i, kept[j]);
    }
  }
  if (offset != nullptr) {      // the same vector on every row, after the branch
#pragma unroll
    for (int j = 0; j < GROUPS; ++j) {
      const int i = (j * 256 + static_cast<int>(threadIdx.x)) * 4;
      if (i >= hidden) continue;
      const float4 b = read4<float>(offset + i);
      kept[j] = make_float4(kept[j].x + b.x, kept[j].y + b.y, kept[j].z + b.z, kept[j].w + b.w);
      write4<float>(stream + base + i, kept[j]);
    }
  }
  if (out == nullptr) return;
#pragma unroll
  for (int j = 0; j < GROUPS; ++j)
    if ((j * 256 + static_cast<int>(threadIdx.x)) * 4 < hidden)
      squares += kept[j].x * kept[j].x + kept[j].y * kept[j].y + kept[j].z * kept[j].z + kept[j].w * kept[j].w;
  const float scale = rsqrtf(block_sum(squares, scratch) / static_cast<float>(hidden) + pre_eps);
#pragma unroll
  for (int j = 0; j < GROUPS; ++j) {
    const int i = (j * 256 + static_cast<int>(threadIdx.x)) * 4;
    if (i >= hidden) continue;
    const float4 w = read4<float>(pre_weight + i), v = kept[j];
    write4<T>(out + base + i, make_float4(v.x * scale * w.x, v.y * scale * w.y, v.z * scale * w.z, v.w * scale * w.w));
  }
}

template <typename T>
__global__ __launch_bounds__(256) void norm_add_norm_kernel(float* __restrict__ stream, const T* __restrict__ delta,
                                                            const float* __restrict__ post_weight, float post_eps,
                                                            const float* __restrict__ pre_weight, float pre_eps,
                                                            T* __restrict__ out, int hidden, float delta_scale,
                                                            const float* __restrict__ offset,
                                                            const T* __restrict__ delta2) {
  __shared__ float scratch[16];
  const size_t base = static_cast<size_t>(blockIdx.x) * hidden;
  float* s = stream + base;
  float squares = 0.f;
  if (delta != nullptr || offset != nullptr) {
    // (a thread meets the same elements in every pass: it reads back what it wrote itself)
    if (delta != nullptr) {
      const T* d = delta + base;
      float post_scale = 1.f;
      if (post_weight != nullptr) {
        float acc = 0.f;
        for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
          const float v = to_float(d[i]);
          acc += v * v;
        }
        post_scale = rsqrtf(block_sum(acc, scratch) / static_cast<float>(hidden) + post_eps);
      }
      for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
        const float both = delta2 != nullptr ? to_float(d[i]) + to_float(delta2[base + i]) : to_float(d[i]);
        s[i] += post_weight != nullptr ? both * post_scale * post_weight[i] : both * delta_scale;
      }
    }
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
      const float v = offset != nullptr ? s[i] + offset[i] : s[i];
      if (offset != nullptr) s[i] = v;
      squares += v * v;
    }
  } else if (out != nullptr) {
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
      const float v = s[i];
      squares += v * v;
    }
  }
  if (out == nullptr) return;
  const float scale = rsqrtf(block_sum(squares, scratch) / static_cast<float>(hidden) + pre_eps);
  T* o = out + base;
  // (a thread reads back what it wrote itself: the same elements in every pass)
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) o[i] = from_float<T>(s[i] * scale * pre_weight[i]);
}

// ---- embedding followed by a norm: out = table[id] / rms(table[id]) * weight, float32 --------------------------------
template <typename T>
__global__ __launch_bounds__(256) void embed_normed_kernel(const int* __restrict__ ids, const T* __restrict__ table,
                                                           const float* __restrict__ weight, float eps,
                                                           float* __restrict__ out, int hidden, int vocab,
                                                           const int* __restrict__ seq_of_token,
                                                           const int* __restrict__ seq_slots,
                                                           const int* __restrict__ slot_words) {
  __shared__ float scratch[16];
  const int n = blockIdx.x;
  int id = ids[n];
  if (id == -1 && slot_words != nullptr)
    id = slot_words[static_cast<long>(seq_slots[seq_of_token[n]]) * kSlotWords + kSlotLastToken];
  float* dst = out + static_cast<size_t>(n) * hidden;
  if (id < 0 || id >= vocab) {     // never read outside the table; a poisoned row shows the fault downstream
    for (int d = threadIdx.x; d < hidden; d += blockDim.x) dst[d] = __uint_as_float(kPoison);
    return;
  }
  const T* row = table + static_cast<size_t>(id) * hidden;
  float squares = 0.f;
  for (int d = threadIdx.x; d < hidden; d += blockDim.x) {
    const float v = to_float(row[d]);
    squares += v * v;
  }
  const float scale = rsqrtf(block_sum(squares, scratch) / static_cast<float>(hidden) + eps);
  for (int d = threadIdx.x; d < hidden; d += blockDim.x) dst[d] = to_float(row[d]) * scale * weight[d];
}

// ---- rows of an embedding table into (or onto) the residual sum --------------------------------------------------------
// out[n] = table[id] (or out[n] += table[id] with `accumulate`), float32; an id of -1 is the token chosen last for the row's
// request, where the slot words are given.
template <typename T>
__global__ __launch_bounds__(256) void embed_rows_kernel(const int* __restrict__ ids, const T* __restrict__ table,
                                                         float* __restrict__ out, int hidden, int vocab, int accumulate,
                                                         const int* __restrict__ seq_of_token,
                                                         const int* __restrict__ seq_slots,
                                                         const int* __restrict__ slot_words) {
  const int n = blockIdx.x;
  int id = ids[n];
  if (id == -1 && slot_words != nullptr)
    id = slot_words[static_cast<long>(seq_slots[seq_of_token[n]]) * kSlotWords + kSlotLastToken];
  float* dst = out + static_cast<size_t>(n) * hidden;
  if (id < 0 || id >= vocab) {     // never read outside the table; a poisoned row shows the fault downstream
    for (int d = threadIdx.x; d < hidden; d += blockDim.x) dst[d] = __uint_as_float(kPoison);
    return;
  }
  const T* row = table + static_cast<size_t>(id) * hidden;
  for (int d = threadIdx.x; d < hidden; d += blockDim.x) dst[d] = accumulate ? dst[d] + to_float(row[d]) : to_float(row[d]);
}

// ---- a row's norm, weight and gate in one pass ------------------------------------------------------------------------------
// x [tokens, width] (TX: float32, or the activation dtype) at `x_stride` per token.  out = x / rms(x) * weight (`normed`; the
// root mean square over the whole row, `weight` may be null) times act(gate), the gate read from `gates` at `gate_stride`
// per token (gate_act 0: none, 1: sigmoid, 2: silu), times out_scale.  One block per token; float32 up to the store.
template <typename TX, typename T>
__global__ __launch_bounds__(256) void norm_gate_rows_kernel(const TX* __restrict__ x, long x_stride, int width, int normed,
                                                             const float* __restrict__ weight, float eps,
                                                             const T* __restrict__ gates, long gate_stride, int gate_act,
                                                             T* __restrict__ out, long out_stride, float out_scale) {
  __shared__ float scratch[16];
  const long n = blockIdx.x;
  const TX* row = x + n * x_stride;
  float scale = out_scale;
  if (normed) {
    float squares = 0.f;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
      const float v = to_float(row[i]);
      squares += v * v;
    }
    scale *= rsqrtf(block_sum(squares, scratch) / static_cast<float>(width) + eps);
  }
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float v = to_float(row[i]) * scale;
    if (weight != nullptr) v *= weight[i];
    if (gate_act != 0) {
      const float g = to_float(gates[n * gate_stride + i]);
      v *= gate_act == 1 ? 1.f / (1.f + expf(-g)) : g / (1.f + expf(-g));
    }
    out[n * out_stride + i] = from_float<T>(v);
  }
}

// The same for rows of up to 256 * 4 * GROUPS values whose width, strides and addresses are multiples of four values: a row
// stays in registers between its one trip to memory and its store, four values a load.
template <typename TX, typename T, int GROUPS>
__global__ __launch_bounds__(256) void norm_gate_rows4_kernel(const TX* __restrict__ x, long x_stride, int width, int normed,
                                                              const float* __restrict__ weight, float eps,
                                                              const T* __restrict__ gates, long gate_stride, int gate_act,
                                                              T* __restrict__ out, long out_stride, float out_scale) {
  __shared__ float scratch[16];
  const long n = blockIdx.x;
  float4 kept[GROUPS], gate[GROUPS];
#pragma unroll
  for (int j = 0; j < GROUPS; ++j) {      // (a group beyond the row reads the row's last four values and counts for nothing)
    const int i = min((j * 256 + static_cast<int>(threadIdx.x)) * 4, width - 4);
    kept[j] = read4<TX>(x + n * x_stride + i);
    if (gate_act != 0) gate[j] = read4<T>(gates + n * gate_stride + i);
  }
  float scale = out_scale;
  if (normed) {
    float squares = 0.f;
#pragma unroll
    for (int j = 0; j < GROUPS; ++j)
      if ((j * 256 + static_cast<int>(threadIdx.x)) * 4 < width)
        squares += kept[j].x * kept[j].x + kept[j].y * kept[j].y + kept[j].z * kept[j].z + kept[j].w * kept[j].w;
    scale *= rsqrtf(block_sum(squares, scratch) / static_cast<float>(width) + eps);
  }
  auto gated = [gate_act](float g) { return gate_act == 1 ? 1.f / (1.f + expf(-g)) : g / (1.f + expf(-g)); };
#pragma unroll
  for (int j = 0; j < GROUPS; ++j) {
    const int i = (j * 256 + static_cast<int>(threadIdx.x)) * 4;
    if (i >= width) continue;
    float4 v = make_float4(kept[j].x * scale, kept[j].y * scale, kept[j].z * scale, kept[j].w * scale);
    if (weight != nullptr) {
      const float4 w = read4<float>(weight + i);
      v = make_float4(v.x * w.x, v.y * w.y, v.z * w.z, v.w * w.w);
    }
    if (gate_act != 0) v = make_float4(v.x * gated(gate[j].x), v.y * gated(gate[j].y), v.z * gated(gate[j].z), v.w * gated(gate[j].w));
    write4<T>(out + n * out_stride + i, v);
  }
}

// ---- a gated feed-forward's activation after a stacked product: out = act(gate) * up --------------------------------------
__device__ __forceinline__ float gelu_tanh_of(float z) {
  return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

template <typename T>
__global__ void gated_activation_kernel(const T* __restrict__ gate_up, T* __restrict__ out, long tokens, int inter,
                                        int activation) {
  const long index = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (index >= tokens * inter) return;
  const long n = index / inter;
  const int i = static_cast<int>(index % inter);
  const float gate = to_float(gate_up[n * 2 * inter + i]), up = to_float(gate_up[n * 2 * inter + inter + i]);
  const float act = activation == 1 ? gelu_tanh_of(gate) : gate / (1.f + expf(-gate));
  out[index] = from_float<T>(act * up);
}

// ---- the difference of two attention maps, normed and gated ------------------------------------------------------------
// maps [tokens, heads, 2, vdim]: o = a1 - lambda a2; o / rms(o) * after; times sigmoid(gates[t, gate_at + h * vdim + i]).
// One wave per (token, head); lambda is read on the device.
template <typename T>
__global__ __launch_bounds__(256) void difference_norm_gate_kernel(const T* __restrict__ maps, const float* __restrict__ lambda,
                                                                   float eps, float after, const T* __restrict__ gates,
                                                                   long gate_stride, long gate_at, T* __restrict__ out,
                                                                   long items, int heads, int vdim) {
  const long item = static_cast<long>(blockIdx.x) * (blockDim.x / kWave) + threadIdx.x / kWave;
  const int lane = threadIdx.x & (kWave - 1);
  if (item >= items) return;
  const long n = item / heads;
  const int h = static_cast<int>(item % heads);
  const T* first = maps + item * 2 * vdim;
  const T* second = first + vdim;
  const float lam = lambda[0];
  float squares = 0.f;
  for (int i = lane; i < vdim; i += kWave) {
    const float o = to_float(first[i]) - lam * to_float(second[i]);
    squares = fmaf(o, o, squares);
  }
  const float scale = rsqrtf(wave_sum(squares) / static_cast<float>(vdim) + eps) * after;
  for (int i = lane; i < vdim; i += kWave) {
    const float o = to_float(first[i]) - lam * to_float(second[i]);
    const float gate = 1.f / (1.f + expf(-to_float(gates[n * gate_stride + gate_at + static_cast<long>(h) * vdim + i])));
    out[item * vdim + i] = from_float<T>(o * scale * gate);
  }
}

// out = a * scale_a + b * scale_b, formed in float32 and rounded once (out may be a or b).
template <typename T>
__global__ void scaled_sum_kernel(const T* a, float scale_a, const T* b, float scale_b, T* out, long count) {
  const long index = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (index < count) out[index] = from_float<T>(to_float(a[index]) * scale_a + to_float(b[index]) * scale_b);
}

}  // namespace

extern "C" {

int akv_scaled_sum(const void* a, float scale_a, const void* b, float scale_b, void* out, int dtype, long count,
                   hipStream_t stream) {
  if (count <= 0) return 0;
  AKV_DISPATCH(dtype, T, scaled_sum_kernel<T><<<static_cast<unsigned>((count + 255) / 256), 256, 0, stream>>>(
                             static_cast<const T*>(a), scale_a, static_cast<const T*>(b), scale_b, static_cast<T*>(out), count));
  return AKV_LAUNCH_STATUS();
}

int akv_embed_normed(const int* ids, const void* table, int dtype, const float* weight, float eps, float* out, int tokens,
                     int hidden, int vocab, const int* seq_of_token, const int* seq_slots, const int* slot_words,
                     hipStream_t stream) {
  if (tokens <= 0) return 0;
  AKV_DISPATCH(dtype, T, embed_normed_kernel<T><<<tokens, 256, 0, stream>>>(ids, static_cast<const T*>(table), weight, eps,
                                                                            out, hidden, vocab, seq_of_token, seq_slots,
                                                                            slot_words));
  return AKV_LAUNCH_STATUS();
}

int akv_gated_activation(const void* gate_up, void* out, int dtype, long tokens, int inter, int activation,
                         hipStream_t stream) {
  if (tokens <= 0 || inter <= 0) return 0;
  if (activation != 0 && activation != 1) return -2;
  const long count = tokens * inter;
  AKV_DISPATCH(dtype, T, gated_activation_kernel<T><<<static_cast<unsigned>((count + 255) / 256), 256, 0, stream>>>(
                             static_cast<const T*>(gate_up), static_cast<T*>(out), tokens, inter, activation));
  return AKV_LAUNCH_STATUS();
}

int akv_difference_norm_gate(const void* maps, const float* lambda, float eps, float after, const void* gates,
                             long gate_stride, long gate_at, void* out, int dtype, long tokens, int heads, int vdim,
                             hipStream_t stream) {
  if (tokens <= 0) return 0;
  const long items = tokens * heads;
  AKV_DISPATCH(dtype, T, difference_norm_gate_kernel<T><<<static_cast<unsigned>((items + 3) / 4), 256, 0, stream>>>(
                             static_cast<const T*>(maps), lambda, eps, after, static_cast<const T*>(gates), gate_stride,
                             gate_at, static_cast<T*>(out), items, heads, vdim));
  return AKV_LAUNCH_STATUS();
}

int akv_embed_rows(const int* ids, const void* table, int dtype, float* out, int tokens, int hidden, int vocab, int accumulate,
                   const int* seq_of_token, const int* seq_slots, const int* slot_words, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (hidden <= 0 || vocab <= 0) return -2;
  AKV_DISPATCH(dtype, T, embed_rows_kernel<T><<<tokens, 256, 0, stream>>>(ids, static_cast<const T*>(table), out, hidden, vocab,
                                                                         accumulate, seq_of_token, seq_slots, slot_words));
  return AKV_LAUNCH_STATUS();
}

int akv_norm_gate_rows(const void* x, int x_dtype, long x_stride, int width, int normed, const float* weight, float eps,
                       const void* gates, long gate_stride, int gate_act, void* out, int dtype, long out_stride,
                       float out_scale, long tokens, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (width <= 0 || gate_act < 0 || gate_act > 2 || (gate_act != 0 && gates == nullptr)) return -2;
  if (x_dtype != kF32 && x_dtype != dtype) return -2;
  const size_t x_size = x_dtype == kF32 ? 4 : 2, size = dtype == kF32 ? 4 : 2;
  const bool by_four = width % 4 == 0 && width >= 4 && width <= 256 * 4 * 8 && x_stride % 4 == 0 && out_stride % 4 == 0 &&
                       (gate_act == 0 || gate_stride % 4 == 0) && reinterpret_cast<uintptr_t>(x) % (4 * x_size) == 0 &&
                       reinterpret_cast<uintptr_t>(out) % (4 * size) == 0 && reinterpret_cast<uintptr_t>(gates) % (4 * size) == 0 &&
                       (weight == nullptr || reinterpret_cast<uintptr_t>(weight) % 16 == 0);
  const unsigned grid = static_cast<unsigned>(tokens);
#define AKV_ROW_ARGS(TX) static_cast<const TX*>(x), x_stride, width, normed, weight, eps, static_cast<const T*>(gates), gate_stride, gate_act, static_cast<T*>(out), out_stride, out_scale
  AKV_DISPATCH(dtype, T, {
    if (x_dtype == kF32 && dtype != kF32) {
      if (by_four && width <= 256 * 4 * 2) norm_gate_rows4_kernel<float, T, 2><<<grid, 256, 0, stream>>>(AKV_ROW_ARGS(float));
      else if (by_four) norm_gate_rows4_kernel<float, T, 8><<<grid, 256, 0, stream>>>(AKV_ROW_ARGS(float));
      else norm_gate_rows_kernel<float, T><<<grid, 256, 0, stream>>>(AKV_ROW_ARGS(float));
    } else {
      if (by_four && width <= 256 * 4 * 2) norm_gate_rows4_kernel<T, T, 2><<<grid, 256, 0, stream>>>(AKV_ROW_ARGS(T));
      else if (by_four) norm_gate_rows4_kernel<T, T, 8><<<grid, 256, 0, stream>>>(AKV_ROW_ARGS(T));
      else norm_gate_rows_kernel<T, T><<<grid, 256, 0, stream>>>(AKV_ROW_ARGS(T));
    }
  });
#undef AKV_ROW_ARGS
  return AKV_LAUNCH_STATUS();
}

int akv_parts_slot_layout(int* out) {
  out[0] = kSlotWords;
  out[1] = kSlotLastToken;
  out[2] = kSlotFedToken;
  return 0;
}

int akv_embed_pairs(const int* ids, const void* table, const void* pairs, int dtype, float* out, int tokens, int hidden,
                    int vocab, long buckets, long mul_prev, long mul_cur, const int* seq_of_token, const int* q_start,
                    const int* positions, const int* seq_slots, int* slot_words, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (buckets <= 0) return -2;
  AKV_DISPATCH(dtype, T, embed_pairs_kernel<T><<<tokens, 256, 0, stream>>>(
                             ids, static_cast<const T*>(table), static_cast<const T*>(pairs), out, hidden, vocab, buckets,
                             mul_prev, mul_cur, seq_of_token, q_start, positions, seq_slots, slot_words));
  return AKV_LAUNCH_STATUS();
}

int akv_note_fed_tokens(const int* ids, const int* q_start, const int* seq_slots, int* slot_words, int seqs,
                        hipStream_t stream) {
  if (seqs <= 0) return 0;
  note_fed_tokens_kernel<<<(seqs + 63) / 64, 64, 0, stream>>>(ids, q_start, seq_slots, slot_words, seqs);
  return AKV_LAUNCH_STATUS();
}

int akv_norm_add_norm(float* stream_buf, const void* delta, const float* post_weight, float post_eps,
                      const float* pre_weight, float pre_eps, void* out, int dtype, int tokens, int hidden,
                      float delta_scale, const float* offset, const void* delta2, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (out != nullptr && pre_weight == nullptr) return -2;
  if (delta2 != nullptr && (delta == nullptr || post_weight != nullptr)) return -2;
#define AKV_NORM_ARGS stream_buf, static_cast<const T*>(delta), post_weight, post_eps, pre_weight, pre_eps, static_cast<T*>(out), hidden, delta_scale, offset, static_cast<const T*>(delta2)
  AKV_DISPATCH(dtype, T, {
    if (hidden % 4 == 0 && hidden >= 4 && hidden <= 256 * 4 * 2) norm_add_norm_rows_kernel<T, 2><<<tokens, 256, 0, stream>>>(AKV_NORM_ARGS);
    else if (hidden % 4 == 0 && hidden <= 256 * 4 * 8) norm_add_norm_rows_kernel<T, 8><<<tokens, 256, 0, stream>>>(AKV_NORM_ARGS);
    else norm_add_norm_kernel<T><<<tokens, 256, 0, stream>>>(AKV_NORM_ARGS);
  });
#undef AKV_NORM_ARGS
  return AKV_LAUNCH_STATUS();
}
}
