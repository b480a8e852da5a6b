// Grouped-query attention for designs whose scores and weights are float32 and whose keys and values may differ in
// width: unit norm of queries and keys with the cache write, and the attention itself with an optional softcap on the
// scores, chunks of positions, a window, a sink in the softmax's denominator and a gate per head.
//
// Keys lie [pages, kv_heads, page, dim], values [pages, kv_heads, vdim, page].  `gated_attention_rows` is the plain path:
// one wave per (token, query head); keys are visited in tiles of 64 aligned to absolute key positions, so the order of
// every sum depends on the token's own position only - not on how the request was cut into steps or on what else is in
// the batch.  Scores, the softmax and the weighted sum are float32.

#include "common.h"
#include "api_parts.h"

using namespace akv;

namespace {

__device__ __forceinline__ void wave_sync_lds() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// One wave per (token, item): the token's query heads (normed into q_out), its key heads (normed into the token's slot
// of the key pages) and its value heads (copied into the value pages).  projected rows: [q | k | v | ...].
// With `maps` > 1 a head's queries and keys are `maps` vectors of `dim` side by side: the token has q_heads * maps query
// vectors and kv_heads * maps key vectors, each normed and rotated for itself, and a key head's record in the pages is
// its `maps` vectors one after the other.  With `table` [positions, rot_dims / 2, 2] (cos, sin) a vector's first rot_dims
// dimensions are rotated by the token's position, dimension i with i + rot_dims / 2 - or, with `interleaved`, dimension 2 i
// with 2 i + 1.  With `whole` the root mean square is taken over all of the token's query vectors at once (and over all of
// its key vectors): every wave sums its side's whole projection for itself.  `q_weight` [q vectors x dim] and `k_weight`
// [k vectors x dim] (float32, either may be null) multiply the normed values, before the rotation.
// One (token, item): `which` < q_vectors is a query vector, then the key vectors, then the value heads.  `given` > 0: the
// factor 1 / rms of the item's side, formed by the caller over the whole projection; else the vector norms itself.
template <typename T>
__device__ __forceinline__ void unit_norm_item(const T* __restrict__ row, long n, int which, int lane, int q_heads, int kv_heads,
                                               int dim, int vdim, float eps, int normed, float given,
                                               const int* __restrict__ slot_map, T* __restrict__ k_pages, T* __restrict__ v_pages,
                                               int page_size, long num_pages, T* __restrict__ q_out, int maps,
                                               const float* __restrict__ table, int table_positions, int rot_dims,
                                               const int* __restrict__ positions, const float* __restrict__ q_weight,
                                               const float* __restrict__ k_weight, int interleaved) {
  const int q_vectors = q_heads * maps, k_vectors = kv_heads * maps;
  if (which < q_vectors + k_vectors) {
    const bool is_q = which < q_vectors;
    const T* x = row + static_cast<long>(which) * dim;       // (key vectors follow the query vectors at the same width)
    T* y;
    if (is_q) {
      y = q_out + (n * q_vectors + which) * dim;
    } else {
      if (slot_map == nullptr) return;
      const long slot = slot_map[n];
      const long page = slot / page_size;
      if (slot < 0 || page >= num_pages) return;
      const int vector = which - q_vectors;
      y = k_pages + (((page * kv_heads + vector / maps) * page_size + slot % page_size) * maps + vector % maps) * dim;
    }
    float scale = 1.f;
    if (normed && given > 0.f) {
      scale = given;
    } else if (normed) {
      float squares = 0.f;
      for (int i = lane; i < dim; i += kWave) {
        const float v = to_float(x[i]);
        squares += v * v;
      }
      scale = rsqrtf(wave_sum(squares) / static_cast<float>(dim) + eps);
    }
    const float* gain = is_q ? q_weight : k_weight;
    if (gain != nullptr) gain += static_cast<long>(is_q ? which : which - q_vectors) * dim;
    if (table == nullptr || rot_dims <= 0) {
      for (int i = lane; i < dim; i += kWave) y[i] = from_float<T>(to_float(x[i]) * scale * (gain != nullptr ? gain[i] : 1.f));
    } else {
      const int half = rot_dims / 2;
      const int pos = positions[n];
      const bool known = pos >= 0 && pos < table_positions;      // (a position beyond the table poisons the vector)
      const float* angles = table + static_cast<long>(known ? pos : 0) * half * 2;
      for (int i = lane; i < dim; i += kWave) {
        float v = to_float(x[i]) * scale * (gain != nullptr ? gain[i] : 1.f);
        if (i < rot_dims) {
          const bool low = interleaved ? (i & 1) == 0 : i < half;
          const int pair = interleaved ? i >> 1 : (low ? i : i - half);
          const int mate = interleaved ? i ^ 1 : (low ? i + half : i - half);
          const float c = angles[2 * pair], s = angles[2 * pair + 1];
          const float other = to_float(x[mate]) * scale * (gain != nullptr ? gain[mate] : 1.f);
          v = low ? v * c - other * s : v * c + other * s;
          if (!known) v = __uint_as_float(0x7fc00000u);
        }
        y[i] = from_float<T>(v);
      }
    }
  } else {
    if (slot_map == nullptr) return;
    const int h = which - q_vectors - k_vectors;
    const long slot = slot_map[n];
    const long page = slot / page_size;
    if (slot < 0 || page >= num_pages) return;
    const T* x = row + static_cast<long>(q_vectors + k_vectors) * dim + static_cast<long>(h) * vdim;
    T* y = v_pages + (page * kv_heads + h) * vdim * page_size + slot % page_size;
    for (int i = lane; i < vdim; i += kWave) y[static_cast<long>(i) * page_size] = x[i];
  }
}

template <typename T>
__global__ __launch_bounds__(256) void unit_norm_write_kernel(const T* __restrict__ projected, long stride, long tokens,
                                                              int q_heads, int kv_heads, int dim, int vdim, float eps,
                                                              int normed, const int* __restrict__ slot_map,
                                                              T* __restrict__ k_pages, T* __restrict__ v_pages, int page_size,
                                                              long num_pages, T* __restrict__ q_out, int maps,
                                                              const float* __restrict__ table, int table_positions,
                                                              int rot_dims, const int* __restrict__ positions,
                                                              const float* __restrict__ q_weight,
                                                              const float* __restrict__ k_weight, int interleaved) {
  const int waves = blockDim.x / kWave, wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1);
  const int items = (q_heads + kv_heads) * maps + kv_heads;
  const long item = static_cast<long>(blockIdx.x) * waves + wave;
  if (item >= tokens * items) return;
  const long n = item / items;
  unit_norm_item<T>(projected + n * stride, n, static_cast<int>(item % items), lane, q_heads, kv_heads, dim, vdim, eps, normed,
                    0.f, slot_map, k_pages, v_pages, page_size, num_pages, q_out, maps, table, table_positions, rot_dims,
                    positions, q_weight, k_weight, interleaved);
}

// The same with the root mean square taken over all of a token's query vectors at once, and over all its key vectors: a
// block is a token, sums both sides' squares once, and its waves then take the token's items in turn.
template <typename T>
__global__ __launch_bounds__(1024) void unit_norm_write_whole_kernel(const T* __restrict__ projected, long stride, int q_heads,
                                                                    int kv_heads, int dim, int vdim, float eps,
                                                                    const int* __restrict__ slot_map, T* __restrict__ k_pages,
                                                                    T* __restrict__ v_pages, int page_size, long num_pages,
                                                                    T* __restrict__ q_out, int maps,
                                                                    const float* __restrict__ table, int table_positions,
                                                                    int rot_dims, const int* __restrict__ positions,
                                                                    const float* __restrict__ q_weight,
                                                                    const float* __restrict__ k_weight, int interleaved) {
  __shared__ float scratch[16];
  const int waves = blockDim.x / kWave, wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1);
  const long n = blockIdx.x;
  const T* row = projected + n * stride;
  const int q_count = q_heads * maps * dim, k_count = kv_heads * maps * dim;
  float q_squares = 0.f, k_squares = 0.f;
  for (int i = threadIdx.x; i < q_count + k_count; i += blockDim.x) {
    const float v = to_float(row[i]);
    if (i < q_count) q_squares += v * v;
    else k_squares += v * v;
  }
  const float q_scale = rsqrtf(block_sum(q_squares, scratch) / static_cast<float>(q_count) + eps);
  const float k_scale = rsqrtf(block_sum(k_squares, scratch) / static_cast<float>(k_count) + eps);
  const int q_vectors = q_heads * maps, items = (q_heads + kv_heads) * maps + kv_heads;
  for (int which = wave; which < items; which += waves)
    unit_norm_item<T>(row, n, which, lane, q_heads, kv_heads, dim, vdim, eps, 1, which < q_vectors ? q_scale : k_scale, slot_map,
                      k_pages, v_pages, page_size, num_pages, q_out, maps, table, table_positions, rot_dims, positions, q_weight,
                      k_weight, interleaved);
}

constexpr int kMaxValueRegs = 4;  // value widths up to 256: each lane owns dims lane, lane + 64, ...
constexpr int kMaxRowWaves = 16;  // the most waves that share a (token, head): wave w of W takes the key tiles w, w + W, ...

// Eight bfloat16 (or float32) values from 16-byte aligned memory, widened.
__device__ __forceinline__ void load8(const bf16_t* p, float (&v)[8]) {
  const uint4 raw = *reinterpret_cast<const uint4*>(p);
  const uint32_t words[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    v[2 * k] = __uint_as_float(words[k] << 16);
    v[2 * k + 1] = __uint_as_float(words[k] & 0xffff0000u);
  }
}
__device__ __forceinline__ void load8(const float* p, float (&v)[8]) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  v[0] = a.x, v[1] = a.y, v[2] = a.z, v[3] = a.w, v[4] = b.x, v[5] = b.y, v[6] = b.z, v[7] = b.w;
}

// A block is a token and G query heads that read the same key head (G = 1: a single head); its waves (1 to 16, the
// caller's choice) take the row's tiles of 64 keys in turn and their shares - maximum, sum of weights, weighted values,
// per head - meet in LDS in the order of the waves.  Inside a tile a lane scores one key for all G heads from one read of
// it (VEC: its dimensions eight at a time) and then owns value dimensions, for which it reads eight neighbouring keys'
// values at a time (the value pages lie [vdim, page]) - once for the G heads.  VEC needs key rows and groups of eight
// values that are 16-byte aligned.
template <typename T, bool VEC, int G>
__global__ __launch_bounds__(kMaxRowWaves * kWave) void gated_attention_rows_kernel(
    const T* __restrict__ q, const T* __restrict__ k_pages, const T* __restrict__ v_pages, const T* __restrict__ gates,
    long gate_stride, int gate_at, const int* __restrict__ seq_of_token, const int* __restrict__ positions,
    const int* __restrict__ block_table, const int* __restrict__ table_rows, int table_width, T* __restrict__ out,
    long tokens, int q_heads, int kv_heads, int dim, int vdim, int page_size, long num_pages, float scale, float softcap,
    int chunk, int window, int sink, long out_stride, float out_scale, const float* __restrict__ sink_logits, int maps,
    int keep_first) {
  // (`q_heads` counts query vectors: with `maps` > 1 a head has `maps` of them, which read the `maps` vectors of their key
  // head's record in turn and the same values; vector v's key head is still v / (q_heads / kv_heads))
  extern __shared__ unsigned char lds_raw[];
  const int wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1), kRowWaves = blockDim.x / kWave;
  // blocks go to the XCDs in turn: neighbouring rows - which read the same or neighbouring keys and values - are given to
  // blocks of one XCD
  const long row = static_cast<long>(blockIdx.x % kXcds) * (gridDim.x / kXcds) + blockIdx.x / kXcds;
  const int bundles = q_heads / G;           // rows of a token
  if (row >= tokens * bundles) return;
  // the block: G x dim floats of q; per wave G x 64 weights and 64 value-row offsets; then the waves' shares
  float* qs = reinterpret_cast<float*>(lds_raw);
  const size_t q_bytes = (static_cast<size_t>(G) * dim * 4 + 7) / 8 * 8;
  float* ps = reinterpret_cast<float*>(lds_raw + q_bytes) + wave * G * kWave;
  long* offs = reinterpret_cast<long*>(lds_raw + q_bytes + static_cast<size_t>(kRowWaves) * G * kWave * 4) + wave * kWave;
  float* shares = reinterpret_cast<float*>(lds_raw + q_bytes + static_cast<size_t>(kRowWaves) * kWave * (G * 4 + 8));

  const long n = row / bundles;
  const int h0 = static_cast<int>(row % bundles) * G;
  const int kvh = h0 / (q_heads / kv_heads);
  const int r = table_rows != nullptr ? table_rows[seq_of_token[n]] : seq_of_token[n];
  const int pos = positions[n];
  int lowest = window > 0 ? max(0, pos - window + 1) : 0;
  if (chunk > 0) lowest = max(lowest, pos / chunk * chunk);
  for (int i = threadIdx.x; i < G * dim; i += blockDim.x) qs[i] = to_float(q[(n * q_heads + h0) * dim + i]);
  __syncthreads();

  // with a sink the sums start as if a key of score 0 and no value had been seen (in the first wave's share)
  // (a learned sink: the term is exp(sink_logits[head]) instead of exp(0))
  float m[G], l[G], acc[G][kMaxValueRegs];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    m[g] = sink && wave == 0 ? (sink_logits != nullptr ? sink_logits[h0 + g] : 0.f) : -INFINITY;
    l[g] = sink && wave == 0 ? 1.f : 0.f;
#pragma unroll
    for (int c = 0; c < kMaxValueRegs; ++c) acc[g][c] = 0.f;
  }
  // the request's first `keep_first` keys stay visible behind the window: their tiles come first, then the window's
  const int first_tile = lowest / kWave, kept_tiles = min((keep_first + kWave - 1) / kWave, first_tile);
  const int all_tiles = kept_tiles + pos / kWave - first_tile + 1;
  for (int turn = wave; turn < all_tiles; turn += kRowWaves) {
    const int tile = turn < kept_tiles ? turn : first_tile + turn - kept_tiles;
    const int j = tile * kWave + lane;
    const bool valid = (j >= lowest || j < keep_first) && j <= pos;
    float s[G];
#pragma unroll
    for (int g = 0; g < G; ++g) s[g] = -INFINITY;
    long value_at = -1;
    if (valid) {
      const long page = block_table[static_cast<long>(r) * table_width + j / page_size];
      if (page < 0 || page >= num_pages) {
#pragma unroll
        for (int g = 0; g < G; ++g) s[g] = __uint_as_float(0x7fc00000u);  // a page that is not the request's: poison
      } else {
        const T* kp = k_pages + (((page * kv_heads + kvh) * page_size + j % page_size) * maps + h0 % maps) * dim;
        float dot[G];
#pragma unroll
        for (int g = 0; g < G; ++g) dot[g] = 0.f;
        int i = 0;
        if (VEC) {
          for (; i + 16 <= dim; i += 16) {       // two loads are asked for before the first is used
            float kv[2][8];
#pragma unroll
            for (int u = 0; u < 2; ++u) load8(kp + i + 8 * u, kv[u]);
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
              for (int e = 0; e < 8; ++e)
#pragma unroll
                for (int g = 0; g < G; ++g) dot[g] = fmaf(qs[g * dim + i + 8 * u + e], kv[u][e], dot[g]);
          }
          for (; i + 8 <= dim; i += 8) {
            float kv[8];
            load8(kp + i, kv);
#pragma unroll
            for (int e = 0; e < 8; ++e)
#pragma unroll
              for (int g = 0; g < G; ++g) dot[g] = fmaf(qs[g * dim + i + e], kv[e], dot[g]);
          }
        }
        for (; i < dim; ++i) {
          const float kv = to_float(kp[i]);
#pragma unroll
          for (int g = 0; g < G; ++g) dot[g] = fmaf(qs[g * dim + i], kv, dot[g]);
        }
#pragma unroll
        for (int g = 0; g < G; ++g) {
          s[g] = dot[g] * scale;
          if (softcap > 0.f) s[g] = softcap * tanhf(s[g] / softcap);
        }
        value_at = (page * kv_heads + kvh) * vdim * page_size + j % page_size;  // values are [vdim, page_size]
      }
    }
    float correction[G];
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const float m_new = fmaxf(m[g], wave_max(s[g]));
      const float p = valid ? expf(s[g] - m_new) : 0.f;
      correction[g] = m_new == m[g] ? 1.f : expf(m[g] - m_new);
      l[g] = l[g] * correction[g] + wave_sum(p);
      m[g] = m_new;
      ps[g * kWave + lane] = value_at >= 0 || !VEC ? p : 0.f;
    }
    offs[lane] = value_at;
    wave_sync_lds();
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int c = 0; c < kMaxValueRegs; ++c) acc[g][c] *= correction[g];
    if (VEC) {
      // a group of eight keys shares a page: its first key that counts tells where the group's values lie
#pragma unroll 2
      for (int k = 0; k < 8; ++k) {
        long at = -1;
#pragma unroll
        for (int e = 7; e >= 0; --e)
          if (offs[8 * k + e] >= 0) at = offs[8 * k + e] - e;
        if (at < 0) continue;  // uniform over the wave
        float weights[G][8];
#pragma unroll
        for (int g = 0; g < G; ++g)
#pragma unroll
          for (int e = 0; e < 8; ++e) weights[g][e] = ps[g * kWave + 8 * k + e];
#pragma unroll
        for (int c = 0; c < kMaxValueRegs; ++c) {
          const int i = lane + c * kWave;
          if (i < vdim) {
            float values[8];
            load8(v_pages + at + static_cast<long>(i) * page_size, values);
#pragma unroll
            for (int e = 0; e < 8; ++e)
#pragma unroll
              for (int g = 0; g < G; ++g) acc[g][c] += weights[g][e] != 0.f ? weights[g][e] * values[e] : 0.f;
          }
        }
      }
    } else {
      for (int jj = 0; jj < kWave; ++jj) {
        const long at = offs[jj];
        if (at < 0) continue;  // uniform over the wave
#pragma unroll
        for (int c = 0; c < kMaxValueRegs; ++c) {
          const int i = lane + c * kWave;
          if (i < vdim) {
            const float value = to_float(v_pages[at + static_cast<long>(i) * page_size]);
#pragma unroll
            for (int g = 0; g < G; ++g) acc[g][c] = fmaf(ps[g * kWave + jj], value, acc[g][c]);
          }
        }
      }
    }
    wave_sync_lds();
  }
  const int share = 2 + vdim;
#pragma unroll
  for (int g = 0; g < G; ++g) {
    float* mine = shares + static_cast<size_t>(wave * G + g) * share;
    if (lane == 0) mine[0] = m[g], mine[1] = l[g];
#pragma unroll
    for (int c = 0; c < kMaxValueRegs; ++c) {
      const int i = lane + c * kWave;
      if (i < vdim) mine[2 + i] = acc[g][c];
    }
  }
  __syncthreads();
  for (int g = 0; g < G; ++g) {
    float highest = -INFINITY;
    for (int w = 0; w < kRowWaves; ++w) highest = fmaxf(highest, shares[static_cast<size_t>(w * G + g) * share]);
    float total = 0.f, factors[kMaxRowWaves];
#pragma unroll
    for (int w = 0; w < kMaxRowWaves; ++w) {
      const float m_w = w < kRowWaves ? shares[static_cast<size_t>(w * G + g) * share] : -INFINITY;
      factors[w] = m_w == -INFINITY ? 0.f : expf(m_w - highest);
      total += w < kRowWaves ? shares[static_cast<size_t>(w * G + g) * share + 1] * factors[w] : 0.f;
    }
    const int h = h0 + g;
    float gate = out_scale;
    if (gates != nullptr) gate = out_scale / (1.f + expf(-to_float(gates[n * gate_stride + gate_at + h])));
    for (int i = threadIdx.x; i < vdim; i += blockDim.x) {
      float sum = 0.f;
#pragma unroll
      for (int w = 0; w < kMaxRowWaves; ++w)
        if (w < kRowWaves) sum += shares[static_cast<size_t>(w * G + g) * share + 2 + i] * factors[w];
      out[n * out_stride + static_cast<long>(h) * vdim + i] = from_float<T>(sum / total * gate);
    }
  }
}

}  // namespace

namespace {

// ---- prompt portions on the matrix cores ----------------------------------------------------------------------------
// bfloat16, keys 16 DT and values 16 VT wide, pages of a multiple of 16 tokens.  A wave is 16 neighbouring rows of the
// step and one query head.  S^T = K Q^T (16 keys x 16 queries a step, the keys as A operand straight from the page) leaves
// lane (c = l % 16, g = l / 16) with the scores of keys 4 g .. 4 g + 3 for query c - which is where the B operand of
// O^T = V^T P^T wants the weights, so they never leave the registers; the values, [vdim, page] in the page, are its A
// operand as they lie.  Scores, softcap, maxima, weights and sums are float32; a weight enters the second product as
// two bfloat16 (its rounding and what the rounding left).  Rows of one tile may belong to several requests (the end of
// one portion and the start of the next): the wave then takes the requests one after the other, each over its own keys,
// with the other requests' columns switched off.  Key tiles lie at absolute positions.
typedef __attribute__((ext_vector_type(4))) short short4_t;
typedef __attribute__((ext_vector_type(4))) float float4_t;

__device__ __forceinline__ short4_t load_bf16x4(const bf16_t* p) {
  return __builtin_bit_cast(short4_t, *reinterpret_cast<const uint2*>(p));
}

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;

__device__ __forceinline__ uint4 load_bf16x8(const bf16_t* p) { return *reinterpret_cast<const uint4*>(p); }

// DT: key width / 32 (the first product runs in steps of 32 dimensions), VT: value width / 16.
template <int DT, int VT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu((DT + VT <= 12 ? 3 : 2), 4))) void gated_attention_tiles_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_pages, const bf16_t* __restrict__ v_pages,
    const bf16_t* __restrict__ gates, long gate_stride, int gate_at, const int* __restrict__ seq_of_token,
    const int* __restrict__ q_start, const int* __restrict__ positions, const int* __restrict__ block_table,
    const int* __restrict__ table_rows, int table_width, bf16_t* __restrict__ out, int first_row, int tokens, int q_heads,
    int kv_heads, int page_size, long num_pages, float scale, float softcap, int chunk, int window, int sink,
    long out_stride, float out_scale, const float* __restrict__ sink_logits, int maps, int keep_first) {
  constexpr int DIM = 32 * DT, VDIM = 16 * VT;
  extern __shared__ float tile_shares[];      // [waves][2 + 4 VT][64]: what the block's waves found over their keys
  // a block is 16 rows and a head; its waves take the steps of 16 keys in turn
  const int wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1), waves = blockDim.x / kWave;
  // blocks go to the XCDs in turn: the heads of a tile, which share keys and values, are given to blocks of one XCD, the
  // tiles to the XCDs in turn, and the tiles with the most keys before them - the last of a portion - start first
  const int tiles = (tokens - first_row + 15) / 16;
  const int slot = blockIdx.x / kXcds;
  const int head = slot % q_heads, turned = slot / q_heads * kXcds + blockIdx.x % kXcds;
  if (turned >= tiles) return;
  const int tile = tiles - 1 - turned;
  const int kvh = head / (q_heads / kv_heads);
  const int col = lane & 15, grp = lane >> 4;
  const int row0 = first_row + tile * 16, row_end = min(row0 + 16, tokens);
  const int my_row = row0 + col;
  const bool have = my_row < row_end;
  int my_pos = -1, my_lowest = 0;
  uint4 qb[DT];
  if (have) {
    my_pos = positions[my_row];
    my_lowest = window > 0 ? max(0, my_pos - window + 1) : 0;
    if (chunk > 0) my_lowest = max(my_lowest, my_pos / chunk * chunk);
    const bf16_t* qp = q + (static_cast<long>(my_row) * q_heads + head) * DIM + grp * 8;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) qb[dt] = load_bf16x8(qp + dt * 32);
  } else {
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) qb[dt] = make_uint4(0u, 0u, 0u, 0u);
  }
  float m = sink && wave == 0 ? (sink_logits != nullptr ? sink_logits[head] : 0.f) : -INFINITY, l = sink && wave == 0 ? 1.f : 0.f;
  const float inverse_cap = softcap > 0.f ? 1.f / softcap : 0.f;
  float4_t o[VT];
#pragma unroll
  for (int vt = 0; vt < VT; ++vt) o[vt] = float4_t{0.f, 0.f, 0.f, 0.f};

  int row = row0;
  while (row < row_end) {
    const int r = seq_of_token[row];
    const int run_end = min(row_end, q_start[r + 1]);
    const int p_first = positions[row], p_last = p_first + (run_end - row - 1);
    int lo_run = window > 0 ? max(0, p_first - window + 1) : 0;
    if (chunk > 0) lo_run = max(lo_run, p_first / chunk * chunk);
    const long table_at = static_cast<long>(table_rows != nullptr ? table_rows[r] : r) * table_width;
    const bool in_run = have && my_row >= row && my_row < run_end;
    // a step's keys and values are asked for while the step before is worked on
    uint4 keys[DT], keys_next[DT];
    short4_t values[VT], values_next[VT];
    bool there = false, there_next = false;
    auto fetch = [&](int j0, uint4 (&ks)[DT], short4_t (&vs)[VT]) -> bool {
      const long page = block_table[table_at + j0 / page_size];
      if (page < 0 || page >= num_pages) return false;      // (uniform; a page that is not the request's is never read)
      const int o0 = j0 % page_size;
      const bf16_t* kp = k_pages + (((page * kv_heads + kvh) * page_size + o0 + col) * maps + head % maps) * DIM + grp * 8;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) ks[dt] = load_bf16x8(kp + dt * 32);
      const bf16_t* vp = v_pages + ((page * kv_heads + kvh) * VDIM + col) * page_size + o0 + grp * 4;
#pragma unroll
      for (int vt = 0; vt < VT; ++vt) vs[vt] = load_bf16x4(vp + static_cast<long>(vt) * 16 * page_size);
      return true;
    };
    // steps of 16 keys: those of the request's first `keep_first` keys that lie before the window, then the window's
    const int first_step = lo_run >> 4, kept_steps = min((keep_first + 15) >> 4, first_step);
    const int all_steps = kept_steps + (p_last >> 4) - first_step + 1;
    auto keys_of = [&](int turn) { return (turn < kept_steps ? turn : first_step + turn - kept_steps) << 4; };
    if (wave < all_steps) there = fetch(keys_of(wave), keys, values);
    for (int turn = wave; turn < all_steps; turn += waves) {
      const int j0 = keys_of(turn);
      there_next = turn + waves < all_steps ? fetch(keys_of(turn + waves), keys_next, values_next) : false;
      if (there) {
        float4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
          acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, keys[dt]),
                                                        __builtin_bit_cast(bf16x8_t, qb[dt]), acc, 0, 0, 0);
        float s[4];
        float highest = -INFINITY;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int j = j0 + grp * 4 + i;
          float v = acc[i] * scale;
          if (softcap > 0.f) {      // tanh(x) = 1 - 2 / (exp(2 x) + 1), with the hardware's exponential and reciprocal
            const float e = __expf(2.f * fabsf(v) * inverse_cap);
            v = copysignf(softcap * (1.f - 2.f * __frcp_rn(e + 1.f)), v);
          }
          s[i] = (in_run && (j >= my_lowest || j < keep_first) && j <= my_pos) ? v : -INFINITY;
          highest = fmaxf(highest, s[i]);
        }
        highest = fmaxf(highest, __shfl_xor(highest, 16, kWave));
        highest = fmaxf(highest, __shfl_xor(highest, 32, kWave));
        const float m_new = fmaxf(m, highest);
        const float correction = m_new == m ? 1.f : __expf(m - m_new);
        float p[4], added = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          p[i] = s[i] == -INFINITY ? 0.f : __expf(s[i] - m_new);
          added += p[i];
        }
        added += __shfl_xor(added, 16, kWave);
        added += __shfl_xor(added, 32, kWave);
        l = l * correction + added;
        m = m_new;
        short4_t p_high, p_low;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const uint16_t high = bf16_bits(p[i]);
          p_high[i] = static_cast<short>(high);
          p_low[i] = static_cast<short>(bf16_bits(p[i] - __uint_as_float(static_cast<uint32_t>(high) << 16)));
        }
        const int beyond = j0 + grp * 4 + 3 - p_last;      // this many of the lane's four keys are not written yet
#pragma unroll
        for (int vt = 0; vt < VT; ++vt) {
          short4_t operand = values[vt];
          if (beyond > 0) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
              if (i > 3 - beyond) operand[i] = 0;
          }
          float4_t sum = o[vt];
#pragma unroll
          for (int i = 0; i < 4; ++i) sum[i] *= correction;
          sum = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(operand, p_high, sum, 0, 0, 0);
          o[vt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(operand, p_low, sum, 0, 0, 0);
        }
      }
      there = there_next;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) keys[dt] = keys_next[dt];
#pragma unroll
      for (int vt = 0; vt < VT; ++vt) values[vt] = values_next[vt];
    }
    row = run_end;
  }
  if (waves > 1) {      // the waves' shares meet in LDS and the first wave adds them in the order of the waves
    float* mine = tile_shares + static_cast<size_t>(wave) * (2 + 4 * VT) * kWave + lane;
    mine[0] = m;
    mine[kWave] = l;
#pragma unroll
    for (int vt = 0; vt < VT; ++vt)
#pragma unroll
      for (int i = 0; i < 4; ++i) mine[(2 + 4 * vt + i) * kWave] = o[vt][i];
    __syncthreads();
    if (wave != 0) return;
    float highest = m;
    for (int w = 1; w < waves; ++w) highest = fmaxf(highest, tile_shares[static_cast<size_t>(w) * (2 + 4 * VT) * kWave + lane]);
    const float own = m == -INFINITY ? 0.f : expf(m - highest);
    l *= own;
#pragma unroll
    for (int vt = 0; vt < VT; ++vt)
#pragma unroll
      for (int i = 0; i < 4; ++i) o[vt][i] *= own;
    for (int w = 1; w < waves; ++w) {
      const float* other = tile_shares + static_cast<size_t>(w) * (2 + 4 * VT) * kWave + lane;
      const float factor = other[0] == -INFINITY ? 0.f : expf(other[0] - highest);
      l += other[kWave] * factor;
#pragma unroll
      for (int vt = 0; vt < VT; ++vt)
#pragma unroll
        for (int i = 0; i < 4; ++i) o[vt][i] += other[(2 + 4 * vt + i) * kWave] * factor;
    }
  }
  if (!have) return;
  float gate = out_scale;
  if (gates != nullptr) gate = out_scale / (1.f + expf(-to_float(gates[static_cast<long>(my_row) * gate_stride + gate_at + head])));
  const float factor = gate / l;
  bf16_t* dst = out + static_cast<long>(my_row) * out_stride + head * VDIM + grp * 4;
#pragma unroll
  for (int vt = 0; vt < VT; ++vt) {
    uint2 packed;
    packed.x = bf16_pair(o[vt][0] * factor, o[vt][1] * factor);
    packed.y = bf16_pair(o[vt][2] * factor, o[vt][3] * factor);
    *reinterpret_cast<uint2*>(dst + vt * 16) = packed;
  }
}

}  // namespace

extern "C" {

// The same for rows first_row .. tokens - 1 of a bfloat16 step on the matrix cores: keys and values of 32, 64, 128 or 256,
// pages of a multiple of 16 tokens (-2 otherwise).  Rows of a request follow each other in the order of their positions.
int akv_gated_attention_tiles(const void* q, const void* k_pages, const void* v_pages, const void* gates, long gate_stride,
                              int gate_at, const int* seq_of_token, const int* q_start, const int* positions,
                              const int* block_table, const int* table_rows, int table_width, void* out, int first_row,
                              int tokens, int q_heads, int kv_heads, int dim, int vdim, int page_size, long num_pages,
                              float scale, float softcap, int chunk, int window, int sink, long out_stride, float out_scale,
                              const float* sink_logits, int maps, int keep_first, hipStream_t stream) {
  if (tokens <= first_row) return 0;
  if (page_size % 16 != 0 || q_heads % kv_heads != 0 || maps < 1) return -2;
  const long items = static_cast<long>((tokens - first_row + 15) / 16) * q_heads;
  const unsigned grid = static_cast<unsigned>(((tokens - first_row + 15) / 16 + kXcds - 1) / kXcds * kXcds * q_heads);
  const int waves = vdim > 128 ? 2 : 4;       // (their shares must fit into 64 KB of LDS)
  const size_t lds = static_cast<size_t>(waves) * (2 + vdim / 4) * kWave * 4;
#define AKV_TILES(DT, VT)                                                                                              \
  gated_attention_tiles_kernel<DT, VT><<<grid, waves * kWave, lds, stream>>>(                                                    \
      static_cast<const bf16_t*>(q), static_cast<const bf16_t*>(k_pages), static_cast<const bf16_t*>(v_pages),         \
      static_cast<const bf16_t*>(gates), gate_stride, gate_at, seq_of_token, q_start, positions, block_table, table_rows, \
      table_width, static_cast<bf16_t*>(out), first_row, tokens, q_heads, kv_heads, page_size, num_pages, scale, softcap, \
      chunk, window, sink, out_stride, out_scale, sink_logits, maps, keep_first)
#define AKV_TILES_V(DT)                    \
  switch (vdim) {                          \
    case 32: AKV_TILES(DT, 2); break;      \
    case 64: AKV_TILES(DT, 4); break;      \
    case 128: AKV_TILES(DT, 8); break;     \
    case 256: AKV_TILES(DT, 16); break;    \
    default: return -2;                    \
  }
  switch (dim) {
    case 32: AKV_TILES_V(1); break;
    case 64: AKV_TILES_V(2); break;
    case 128: AKV_TILES_V(4); break;
    case 256: AKV_TILES_V(8); break;
    default: return -2;
  }
#undef AKV_TILES_V
#undef AKV_TILES
  return AKV_LAUNCH_STATUS();
}

int akv_unit_norm_write(const void* projected, long stride, int dtype, long tokens, int q_heads, int kv_heads, int dim,
                        int vdim, float eps, int normed, const int* slot_map, void* k_pages, void* v_pages, int page_size,
                        long num_pages, void* q_out, int maps, const float* table, int table_positions, int rot_dims,
                        const int* positions, const float* q_weight, const float* k_weight, int whole, int interleaved,
                        hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (q_heads <= 0 || kv_heads <= 0 || dim <= 0 || vdim <= 0 || page_size <= 0 || maps < 1) return -2;
  if (table != nullptr && (rot_dims < 0 || rot_dims % 2 != 0 || rot_dims > dim || positions == nullptr)) return -2;
  const long items = tokens * ((q_heads + kv_heads) * maps + kv_heads);
  if (whole && normed) {
    // (few tokens: sixteen waves a token share its items; many: four, and the tokens fill the device)
    const int threads = tokens <= 256 ? 1024 : 256;
    AKV_DISPATCH(dtype, T, unit_norm_write_whole_kernel<T><<<static_cast<unsigned>(tokens), threads, 0, stream>>>(
                               static_cast<const T*>(projected), stride, q_heads, kv_heads, dim, vdim, eps, slot_map,
                               static_cast<T*>(k_pages), static_cast<T*>(v_pages), page_size, num_pages, static_cast<T*>(q_out),
                               maps, table, table_positions, rot_dims, positions, q_weight, k_weight, interleaved));
    return AKV_LAUNCH_STATUS();
  }
  AKV_DISPATCH(dtype, T, unit_norm_write_kernel<T><<<static_cast<unsigned>((items + 3) / 4), 256, 0, stream>>>(
                             static_cast<const T*>(projected), stride, tokens, q_heads, kv_heads, dim, vdim, eps, normed,
                             slot_map, static_cast<T*>(k_pages), static_cast<T*>(v_pages), page_size, num_pages,
                             static_cast<T*>(q_out), maps, table, table_positions, rot_dims, positions, q_weight,
                             k_weight, interleaved));
  return AKV_LAUNCH_STATUS();
}

int akv_gated_attention_rows(const void* q, const void* k_pages, const void* v_pages, const void* gates, long gate_stride,
                             int gate_at, const int* seq_of_token, const int* positions, const int* block_table,
                             const int* table_rows, int table_width, void* out, int dtype, long tokens, int q_heads,
                             int kv_heads, int dim, int vdim, int page_size, long num_pages, float scale, float softcap,
                             int chunk, int window, int sink, long out_stride, float out_scale, int row_waves,
                             const float* sink_logits, int maps, int keep_first, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (maps < 1) return -2;
  const int kRowWaves = row_waves;
  if (row_waves < 1 || row_waves > kMaxRowWaves) return -2;
  if (vdim > kMaxValueRegs * kWave || dim <= 0 || q_heads % kv_heads != 0) return -2;
  // A block a head.  (The kernel can take 2 or 4 query heads of a key head in one block, reading keys and values once
  // for them; with a quarter of the blocks at its register count that was slower at 8 requests of 2,048 keys, 16 query
  // and 4 key heads - 66 us against 39 - and is not chosen.)
  int bundle = 1;
  int waves = kRowWaves;
  auto lds_of = [&](int g, int w) {
    return (static_cast<size_t>(g) * dim * 4 + 7) / 8 * 8 + static_cast<size_t>(w) * kWave * (g * 4 + 8) +
           static_cast<size_t>(w) * g * (2 + vdim) * 4;
  };
  while (lds_of(bundle, waves) > 64 * 1024 && waves > 1) waves /= 2;
  while (lds_of(bundle, waves) > 64 * 1024 && bundle > 1) bundle /= 2;
  const size_t lds = lds_of(bundle, waves);
  if (lds > 64 * 1024) return -2;
  const long rows = tokens * (q_heads / bundle);
  const size_t element = dtype == kBF16 ? 2 : 4;
  // 16-byte loads: key rows and groups of eight neighbouring keys' values must be aligned
  const bool vec = (dim * element) % 16 == 0 && page_size % 8 == 0 &&
                   (static_cast<size_t>(page_size) * element) % 16 == 0 && reinterpret_cast<uintptr_t>(k_pages) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(v_pages) % 16 == 0;
  const unsigned grid = static_cast<unsigned>((rows + kXcds - 1) / kXcds * kXcds);
#define AKV_ROWS(VEC, G)                                                                                                \
  AKV_DISPATCH(dtype, T,                                                                                                \
               gated_attention_rows_kernel<T, VEC, G><<<grid, waves * kWave, lds, stream>>>(                           \
                   static_cast<const T*>(q), static_cast<const T*>(k_pages), static_cast<const T*>(v_pages),            \
                   static_cast<const T*>(gates), gate_stride, gate_at, seq_of_token, positions, block_table, table_rows, \
                   table_width, static_cast<T*>(out), tokens, q_heads, kv_heads, dim, vdim, page_size, num_pages, scale, \
                   softcap, chunk, window, sink, out_stride, out_scale, sink_logits, maps, keep_first))
#define AKV_ROWS_G(VEC)          \
  switch (bundle) {              \
    case 4: AKV_ROWS(VEC, 4); break; \
    case 2: AKV_ROWS(VEC, 2); break; \
    default: AKV_ROWS(VEC, 1); break; \
  }
  if (vec) AKV_ROWS_G(true)
  else AKV_ROWS_G(false)
#undef AKV_ROWS_G
#undef AKV_ROWS
  return AKV_LAUNCH_STATUS();
}
}
