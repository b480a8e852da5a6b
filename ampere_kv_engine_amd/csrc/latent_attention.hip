// Attention over a compressed latent, with a sliding window.
//
// A token's cache record is [c | k_rot]: the normed latent (kv_rank) and one rotated key part (rot) that all heads
// share.  Keys and values of a head are linear in c (k_h = U_h c, v_h = V_h c), so the scores and the weighted sum can
// be taken over the records themselves:
//     q_h . k_h(j) = (U_h^T q_h) . c_j            sum_j p_j v_h(j) = V_h (sum_j p_j c_j)
// `heads_linear` forms U_h^T q_h before and V_h (...) after; in between every head attends the same records - one
// kv head whose keys are kv_rank + rot wide and whose values are the keys' first kv_rank dimensions.  Norms, angles,
// scores, softmax and the weighted sums are float32.

#include "common.h"
#include "mfma_tiles.h"
#include "api_parts.h"

using namespace akv;

namespace {

constexpr unsigned kPoison = 0x7fc00000u;

// ---- norms of the two latents, rotation of the shared key part, cache write -------------------------------------------
// One block per token.  down = [q latent | kv latent | key part]; the last two only where the layer keeps a cache.
template <typename T>
__global__ __launch_bounds__(256) void latent_encode_kernel(
    const T* __restrict__ down, int q_rank, int kv_rank, int rot, int rot_dims, const float* __restrict__ q_weight,
    const float* __restrict__ kv_weight, float eps, const float* __restrict__ table, int table_positions,
    const int* __restrict__ positions, const int* __restrict__ slot_map, T* __restrict__ cq, T* __restrict__ records,
    long record_slots, T* __restrict__ latents_t, int page_size, int interleaved, long down_stride) {
  __shared__ float scratch[16];
  const int n = blockIdx.x;
  const bool writes = records != nullptr;
  const T* src = down + static_cast<size_t>(n) * down_stride;
  float acc = 0.f;
  for (int i = threadIdx.x; i < q_rank; i += blockDim.x) {
    const float v = to_float(src[i]);
    acc += v * v;
  }
  const float q_scale = rsqrtf(block_sum(acc, scratch) / static_cast<float>(q_rank) + eps);
  for (int i = threadIdx.x; i < q_rank; i += blockDim.x)
    cq[static_cast<size_t>(n) * q_rank + i] = from_float<T>(to_float(src[i]) * q_scale * q_weight[i]);
  if (!writes) return;
  const long slot = slot_map[n];
  if (slot < 0 || slot >= record_slots) return;     // (never write outside the pages)
  T* record = records + slot * (kv_rank + rot);
  const T* latent = src + q_rank;
  acc = 0.f;
  for (int i = threadIdx.x; i < kv_rank; i += blockDim.x) {
    const float v = to_float(latent[i]);
    acc += v * v;
  }
  const float kv_scale = rsqrtf(block_sum(acc, scratch) / static_cast<float>(kv_rank) + eps);
  // (the second copy of the latent, keys contiguous: [page][dimension][place in the page])
  T* turned = latents_t != nullptr ? latents_t + (slot / page_size) * kv_rank * page_size + slot % page_size : nullptr;
  for (int i = threadIdx.x; i < kv_rank; i += blockDim.x) {
    const T value = from_float<T>(to_float(latent[i]) * kv_scale * kv_weight[i]);
    record[i] = value;
    if (turned != nullptr) turned[static_cast<long>(i) * page_size] = value;
  }
  const T* key = latent + kv_rank;
  const int half = rot_dims / 2;
  const int pos = positions[n];
  const bool known = pos >= 0 && pos < table_positions;
  for (int i = threadIdx.x; i < rot; i += blockDim.x) {
    float value;
    if (i >= rot_dims) {
      value = to_float(key[i]);
    } else if (!known) {
      value = __uint_as_float(kPoison);
    } else {
      // pair j is dimensions (j, j + half), or (2 j, 2 j + 1) where the pairs are interleaved
      const int j = interleaved ? i >> 1 : (i < half ? i : i - half);
      const bool low = interleaved ? (i & 1) == 0 : i < half;
      const float c = table[(static_cast<size_t>(pos) * half + j) * 2], s = table[(static_cast<size_t>(pos) * half + j) * 2 + 1];
      const float u = to_float(key[interleaved ? 2 * j : j]), v = to_float(key[interleaved ? 2 * j + 1 : j + half]);
      value = low ? u * c - v * s : v * c + u * s;
    }
    record[kv_rank + i] = from_float<T>(value);
  }
}

// ---- the rotated part of every query head, into its place behind the absorbed part --------------------------------------
template <typename T, typename TY>
__global__ void rotate_queries_kernel(const T* __restrict__ q, long tokens, int heads, int dim, int rot, int rot_dims,
                                      const float* __restrict__ table, int table_positions,
                                      const int* __restrict__ positions, TY* __restrict__ q_abs, int width, int at,
                                      int interleaved) {
  const long index = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (index >= tokens * heads * rot) return;
  const int i = static_cast<int>(index % rot);
  const long row = index / rot;                     // token * heads + head
  const long n = row / heads;
  const T* src = q + row * (dim + rot) + dim;
  const int half = rot_dims / 2;
  float value;
  if (i >= rot_dims) {
    value = to_float(src[i]);
  } else {
    const int pos = positions[n];
    if (pos < 0 || pos >= table_positions) {
      value = __uint_as_float(kPoison);
    } else {
      const int j = interleaved ? i >> 1 : (i < half ? i : i - half);
      const bool low = interleaved ? (i & 1) == 0 : i < half;
      const float c = table[(static_cast<size_t>(pos) * half + j) * 2], s = table[(static_cast<size_t>(pos) * half + j) * 2 + 1];
      const float u = to_float(src[interleaved ? 2 * j : j]), v = to_float(src[interleaved ? 2 * j + 1 : j + half]);
      value = low ? u * c - v * s : v * c + u * s;
    }
  }
  q_abs[row * width + at + i] = from_float<TY>(value);
}

// ---- y[t, h, j] = sum_i x[t, h, i] w[h, i, j] ------------------------------------------------------------------------------
// A block takes kTokens tokens of one head and up to 256 outputs: thread j streams column j of the head's matrix
// (neighbouring threads read neighbouring addresses) against the tokens' inputs, which lie in LDS as [i][token] so
// that a thread reads the eight of an i as two 16-byte broadcasts.  Sums are float32 in the order of i whatever the
// batch.
constexpr int kHeadTokens = 8;

// With few tokens (SPLIT) a head's matrix is the work: a block is 64 outputs, and its four waves take every fourth
// input each and add their sums through LDS in the waves' order.
template <typename TX, typename TW, typename TY, bool SPLIT>
__global__ __launch_bounds__(256) void heads_linear_kernel(const TX* __restrict__ x, long x_token_stride,
                                                           long x_head_stride, const TW* __restrict__ w,
                                                           TY* __restrict__ y, long y_token_stride, long y_head_stride,
                                                           int tokens, int ins, int outs) {
  extern __shared__ float xs[];      // [ins][kHeadTokens], then (SPLIT) [3][64][kHeadTokens]
  const int h = blockIdx.y;
  const int first = blockIdx.x * kHeadTokens;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1);
  const int j = SPLIT ? blockIdx.z * kWave + lane : blockIdx.z * blockDim.x + threadIdx.x;
  for (int e = threadIdx.x; e < ins * kHeadTokens; e += blockDim.x) {
    const int t = e / ins, i = e % ins;             // (consecutive threads read consecutive inputs of one token)
    const int n = first + t;
    xs[i * kHeadTokens + t] = n < tokens ? to_float(x[n * x_token_stride + h * x_head_stride + i]) : 0.f;
  }
  __syncthreads();
  const int jj = min(j, outs - 1);                  // (a thread beyond the outputs keeps the block's steps, stores nothing)
  const TW* column = w + static_cast<size_t>(h) * ins * outs + jj;
  float acc[kHeadTokens];
#pragma unroll
  for (int t = 0; t < kHeadTokens; ++t) acc[t] = 0.f;
  const int begin = SPLIT ? wave : 0, stride = SPLIT ? 4 : 1;
#pragma unroll 8
  for (int i = begin; i < ins; i += stride) {
    const float weight = to_float(column[static_cast<size_t>(i) * outs]);
    const float4 a = *reinterpret_cast<const float4*>(xs + i * kHeadTokens);
    const float4 b = *reinterpret_cast<const float4*>(xs + i * kHeadTokens + 4);
    acc[0] = fmaf(a.x, weight, acc[0]);
    acc[1] = fmaf(a.y, weight, acc[1]);
    acc[2] = fmaf(a.z, weight, acc[2]);
    acc[3] = fmaf(a.w, weight, acc[3]);
    acc[4] = fmaf(b.x, weight, acc[4]);
    acc[5] = fmaf(b.y, weight, acc[5]);
    acc[6] = fmaf(b.z, weight, acc[6]);
    acc[7] = fmaf(b.w, weight, acc[7]);
  }
  if constexpr (SPLIT) {
    float* shares = xs + ins * kHeadTokens;         // [3][64][kHeadTokens]
    if (wave > 0) {
#pragma unroll
      for (int t = 0; t < kHeadTokens; ++t) shares[((wave - 1) * kWave + lane) * kHeadTokens + t] = acc[t];
    }
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int other = 0; other < 3; ++other)
#pragma unroll
      for (int t = 0; t < kHeadTokens; ++t) acc[t] += shares[(other * kWave + lane) * kHeadTokens + t];
  }
  if (j >= outs) return;
#pragma unroll
  for (int t = 0; t < kHeadTokens; ++t) {
    const int n = first + t;
    if (n < tokens) y[n * y_token_stride + h * y_head_stride + j] = from_float<TY>(acc[t]);
  }
}

// ---- the attention itself ----------------------------------------------------------------------------------------------
// A block is one token and up to eight heads, a wave each.  The records of KT keys at a time are fetched once for all
// of the block's heads into LDS, as float32 rows an odd number of words apart.  Scores: a lane takes one key and one of
// 64 / KT interleaved shares of the dimensions; the shares are added across lanes.  Weighted sum: a lane owns the
// latent's dimensions lane, lane + 64, ...  Tiles are aligned to absolute key positions, so the order of every sum
// depends on the token's position alone - not on the portion it arrived in, nor on what else is in the batch.
constexpr int kMaxLatentRegs = 16;     // latents up to 1,024 wide

template <typename T, int KT>
__global__ __launch_bounds__(512) void latent_attend_kernel(
    const float* __restrict__ q_abs, const T* __restrict__ records, const int* __restrict__ seq_of_token,
    const int* __restrict__ positions, const int* __restrict__ block_table, const int* __restrict__ table_rows,
    int table_width, float* __restrict__ out, int heads, int kv_rank, int width, int page_size, long num_pages,
    float scale, int window) {
  extern __shared__ float lds[];
  constexpr int kShares = kWave / KT;
  const int waves = blockDim.x / kWave, wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1);
  const int padded = width | 1;
  float* tile = lds;                                      // [KT][padded]
  long* slot_of = reinterpret_cast<long*>(tile + KT * padded + (KT * padded & 1));   // [KT], -1: no such key
  float* qs = reinterpret_cast<float*>(slot_of + KT) + wave * (width + KT);           // [width] and the weights [KT]
  float* ps = qs + width;

  const int n = blockIdx.x;
  const int h = blockIdx.y * waves + wave;
  const bool works = h < heads;
  const int r = table_rows != nullptr ? table_rows[seq_of_token[n]] : seq_of_token[n];
  const int pos = positions[n];
  const int lowest = window > 0 ? max(0, pos - window + 1) : 0;
  if (works)
    for (int i = lane; i < width; i += kWave) qs[i] = q_abs[(static_cast<size_t>(n) * heads + h) * width + i];

  const int key = lane % KT, share = lane / KT;
  float m = -INFINITY, l = 0.f;
  float acc[kMaxLatentRegs];
#pragma unroll
  for (int c = 0; c < kMaxLatentRegs; ++c) acc[c] = 0.f;
  bool poisoned = false;

  for (int t0 = lowest / KT * KT; t0 <= pos; t0 += KT) {
    __syncthreads();                    // the tile of the turn before has been read by everybody
    if (threadIdx.x < KT) {
      const int j = t0 + threadIdx.x;
      long slot = -1;
      if (j >= lowest && j <= pos) {
        const long page = block_table[static_cast<long>(r) * table_width + j / page_size];
        slot = (page < 0 || page >= num_pages) ? -2 : page * page_size + j % page_size;   // -2: a page that is not the request's
      }
      slot_of[threadIdx.x] = slot;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < KT * width; e += blockDim.x) {
      const int k = e / width, i = e % width;
      const long slot = slot_of[k];
      tile[k * padded + i] = slot >= 0 ? to_float(records[slot * width + i]) : 0.f;
    }
    __syncthreads();
    if (!works) continue;
    const long slot = slot_of[key];
    poisoned = poisoned || slot == -2;
    float dot = 0.f;
    const float* row = tile + key * padded;
    for (int i = share; i < width; i += kShares) dot = fmaf(qs[i], row[i], dot);
#pragma unroll
    for (int offset = KT; offset < kWave; offset <<= 1) dot += __shfl_xor(dot, offset, kWave);
    const float s = slot >= 0 ? dot * scale : -INFINITY;
    const float m_new = fmaxf(m, wave_max(s));
    const float p = slot >= 0 ? expf(s - m_new) : 0.f;
    const float correction = expf(m - m_new);
    l = l * correction + wave_sum(p) * (1.f / kShares);
    m = m_new;
    if (share == 0) ps[key] = p;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int c = 0; c < kMaxLatentRegs; ++c) acc[c] *= correction;
    for (int k = 0; k < KT; ++k) {
      const float pk = ps[k];
      const float* value = tile + k * padded;
#pragma unroll
      for (int c = 0; c < kMaxLatentRegs; ++c) {
        const int i = lane + c * kWave;
        if (i < kv_rank) acc[c] = fmaf(pk, value[i], acc[c]);
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
  if (!works) return;
  // (any lane that met a foreign page poisons the head's output)
  const bool any_poison = __any(poisoned);
  float* dst = out + (static_cast<size_t>(n) * heads + h) * kv_rank;
#pragma unroll
  for (int c = 0; c < kMaxLatentRegs; ++c) {
    const int i = lane + c * kWave;
    if (i < kv_rank) dst[i] = any_poison ? __uint_as_float(kPoison) : acc[c] / l;
  }
}


// ---- the same on the matrix cores (bfloat16) --------------------------------------------------------------------------
// For layers whose heads are a multiple of 16: a wave is one token and 16 of its heads - the 16 columns of the matrix
// instruction, which all see the same keys.  S^T = K Q^T (keys are the A operand, 16 bytes a lane straight from the
// records) and O^T = C^T P^T, where C^T, the latents with the keys contiguous, is a second copy that the layer keeps
// beside the records as [kv_rank, page] per page: 8 keys of a dimension are then one 16-byte load, and the weights
// are the B operand as they stand in the registers.  Row rho of a score tile is key base + (rho / 4) * 8 + j * 4 +
// rho % 4 (j: which of a step's two tiles), so that a lane's 8 weights of a step are 8 consecutive keys.  Weights
// enter the second product as high + low bfloat16.  Steps of 32 keys lie at absolute positions.
typedef __attribute__((ext_vector_type(2))) float floatx2;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;

template <int VT>      // kv_rank / 16
__global__ __launch_bounds__(256) void latent_attend_mfma_kernel(
    const bf16_t* __restrict__ q_abs, const bf16_t* __restrict__ records, const bf16_t* __restrict__ latents_t,
    const int* __restrict__ seq_of_token, const int* __restrict__ positions, const int* __restrict__ block_table,
    const int* __restrict__ table_rows, int table_width, bf16_t* __restrict__ out, long tiles, int heads, int width,
    int page_size, long num_pages, float scale_log2, int window, int segment, int segments, float* __restrict__ parts) {
  extern __shared__ unsigned char lds_bytes[];
  constexpr int kv_rank = VT * 16;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1);
  const long tile = static_cast<long>(blockIdx.x) * (blockDim.x / kWave) + wave;
  if (tile >= tiles) return;
  const int part = blockIdx.y;            // which run of `segment` keys (aligned to absolute positions) this wave takes
  const int rho = lane & 15, g = lane >> 4;
  const long n = tile * 16 / heads;                         // the tile's token (heads are a multiple of 16)
  const int r = table_rows != nullptr ? table_rows[seq_of_token[n]] : seq_of_token[n];
  const int pos = positions[n];
  const int lowest = window > 0 ? max(0, pos - window + 1) : 0;
  const int* table = block_table + static_cast<long>(r) * table_width;
  // the tile's 16 query rows into LDS, rows 16 bytes further apart than they are wide
  const int chunks = width / 8, stride = (chunks + 1) * 16;
  unsigned char* qs = lds_bytes + static_cast<size_t>(wave) * 16 * stride;
  const uintx4* q_rows = reinterpret_cast<const uintx4*>(q_abs + tile * 16 * width);
  for (int e = lane; e < 16 * chunks; e += kWave)
    *reinterpret_cast<uintx4*>(qs + (e / chunks) * stride + (e % chunks) * 16) = q_rows[e];
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  const unsigned char* q_mine = qs + rho * stride + g * 16;

  // the token's own slot: always written, what a lane reads in place of a key it may not see
  const long own_page = table[pos / page_size];
  const bool lost = own_page < 0 || own_page >= num_pages;
  const long safe_page = lost ? 0 : own_page;
  const long safe_slot = safe_page * page_size + pos % page_size;

  floatx4 o[VT];
#pragma unroll
  for (int dt = 0; dt < VT; ++dt) o[dt] = floatx4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;
  bool poisoned = lost;
  const int steps32 = width / 32;

  // keys this wave looks at: all the token may see, or - where the launch cuts them - its run of them.  Runs are
  // counted from the window's first key rounded down to a run's size, so a token's cut depends on its position alone.
  int first_base = lowest & ~31, last_key = pos;
  if (segments > 1) {
    const int run0 = lowest / segment * segment + part * segment;
    first_base = max(first_base, run0);
    last_key = min(pos, run0 + segment - 1);
  }
  constexpr int kAhead = 6;               // operands asked for before the first of them is multiplied

  for (int base = first_base; base <= last_key; base += 32) {
    const bool edge = base < lowest || base + 31 > pos;
    // ---- this step's latents (needed after the softmax): asked for first ------------------------------------------------
    const int first_key = base + g * 8;
    long value_page = safe_page;
    int value_at = 0;
    uint32_t keep[4] = {0u, 0u, 0u, 0u};          // which of the 8 keys count (others may hold anything)
    if (first_key + 7 >= lowest && first_key <= pos) {
      const long page = table[first_key / page_size];
      if (page >= 0 && page < num_pages) {
        value_page = page;
        value_at = first_key % page_size;
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (first_key + e >= lowest && first_key + e <= pos) keep[e >> 1] |= (e & 1) ? 0xffff0000u : 0x0000ffffu;
      } else {
        poisoned = true;
      }
    }
    const bf16_t* values = latents_t + (value_page * kv_rank + rho) * page_size + value_at;
    uintx4 vreg[VT];
#pragma unroll
    for (int dt = 0; dt < VT; ++dt) vreg[dt] = *reinterpret_cast<const uintx4*>(values + static_cast<long>(dt) * 16 * page_size);
    // ---- scores: two tiles of 16 keys, their operands fetched kAhead at a time ------------------------------------------
    const uintx4* rows[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int key = base + (rho >> 2) * 8 + j * 4 + (rho & 3);
      long slot = safe_slot;
      if (key >= lowest && key <= pos) {
        const long page = table[key / page_size];
        if (page < 0 || page >= num_pages) poisoned = true;
        else slot = page * page_size + key % page_size;
      }
      rows[j] = reinterpret_cast<const uintx4*>(records + slot * width) + g;
    }
    floatx4 s[2] = {floatx4{0.f, 0.f, 0.f, 0.f}, floatx4{0.f, 0.f, 0.f, 0.f}};
    for (int t0 = 0; t0 < steps32; t0 += kAhead) {
      uintx4 k0[kAhead], k1[kAhead], qq[kAhead];
#pragma unroll
      for (int u = 0; u < kAhead; ++u) {
        const int t = min(t0 + u, steps32 - 1);     // (beyond the record: its last operand again, against zeros)
        k0[u] = rows[0][t * 4];
        k1[u] = rows[1][t * 4];
        qq[u] = *reinterpret_cast<const uintx4*>(q_mine + t * 64);
        if (t0 + u >= steps32) qq[u] = uintx4{0u, 0u, 0u, 0u};
      }
#pragma unroll
      for (int u = 0; u < kAhead; ++u) {
        s[0] = mfma16(k0[u], qq[u], s[0]);
        s[1] = mfma16(k1[u], qq[u], s[1]);
      }
    }
    if (edge) {
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int key = base + g * 8 + j * 4 + i;
          if (key < lowest || key > pos) s[j][i] = -INFINITY;
        }
    }
    float top = fmaxf(fmaxf(fmaxf(s[0][0], s[0][1]), fmaxf(s[0][2], s[0][3])),
                      fmaxf(fmaxf(s[1][0], s[1][1]), fmaxf(s[1][2], s[1][3])));
    top = fmaxf(top, __shfl_xor(top, 16, kWave));
    top = fmaxf(top, __shfl_xor(top, 32, kWave));
    const float m_new = fmaxf(m, top * scale_log2);
    const float m_safe = m_new == -INFINITY ? 0.f : m_new;
    const float correction = __builtin_amdgcn_exp2f(m - m_safe);
    floatx2 p[4];
    float sum = 0.f;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      p[e][0] = __builtin_amdgcn_exp2f(fmaf(s[e >> 1][(e & 1) * 2], scale_log2, -m_safe));
      p[e][1] = __builtin_amdgcn_exp2f(fmaf(s[e >> 1][(e & 1) * 2 + 1], scale_log2, -m_safe));
      sum += p[e][0] + p[e][1];
    }
    l = l * correction + sum;
    m = m_new;
    uint32_t high[4], low[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      high[e] = __builtin_bit_cast(uint32_t, __builtin_convertvector(p[e], bf16x2));
      const floatx2 rest = {p[e][0] - __uint_as_float(high[e] << 16), p[e][1] - __uint_as_float(high[e] & 0xffff0000u)};
      low[e] = __builtin_bit_cast(uint32_t, __builtin_convertvector(rest, bf16x2));
    }
    const uintx4 p_high = uintx4{high[0], high[1], high[2], high[3]}, p_low = uintx4{low[0], low[1], low[2], low[3]};
    if (__any(correction != 1.f)) {
#pragma unroll
      for (int dt = 0; dt < VT; ++dt) o[dt] *= correction;
    }
    // ---- O^T += C^T P^T: this lane's 8 keys base + g * 8 .. + 7 of dimension dt * 16 + rho ---------------------------
#pragma unroll
    for (int dt = 0; dt < VT; ++dt) {
      uintx4 v = vreg[dt];
      if (edge) v = uintx4{v[0] & keep[0], v[1] & keep[1], v[2] & keep[2], v[3] & keep[3]};
      o[dt] = mfma16(v, p_low, mfma16(v, p_high, o[dt]));
    }
  }
  if (segments > 1) {
    // this run's share: the sums as they are, with the maximum and the sum of weights they were formed against, for the
    // merge.  parts: [tile][part][16 columns][kv_rank + 2]
    float* mine = parts + ((tile * segments + part) * 16 + rho) * (kv_rank + 2);
    l += __shfl_xor(l, 16, kWave);
    l += __shfl_xor(l, 32, kWave);
    const bool bad = __any(poisoned);
#pragma unroll
    for (int dt = 0; dt < VT; ++dt) {
      floatx4 v = o[dt];
      if (bad) v = floatx4{__uint_as_float(kPoison), __uint_as_float(kPoison), __uint_as_float(kPoison), __uint_as_float(kPoison)};
      store4<float>(mine + dt * 16 + g * 4, v);
    }
    if (g == 0) {
      mine[kv_rank] = m;
      mine[kv_rank + 1] = l;
    }
    return;
  }
  l += __shfl_xor(l, 16, kWave);
  l += __shfl_xor(l, 32, kWave);
  const bool any_poison = __any(poisoned);
  const float inverse = 1.f / l;
  bf16_t* dst = out + (tile * 16 + rho) * kv_rank + g * 4;
#pragma unroll
  for (int dt = 0; dt < VT; ++dt) {
    floatx4 v = o[dt] * inverse;
    if (any_poison) v = floatx4{__uint_as_float(kPoison), __uint_as_float(kPoison), __uint_as_float(kPoison), __uint_as_float(kPoison)};
    store4<bf16_t>(dst + dt * 16, v);
  }
}


// ---- the same for one request's long portion: four waves share every step's records through LDS -------------------------
// The four waves of a block hold neighbouring tokens of ONE request (the launch has no other), whose windows differ by
// a few keys: a step's 32 records and the 32 keys' latents are fetched once per block - asked for one step ahead, into
// registers, while the step before is multiplied - and laid into LDS as the matrix cores read them: record rows in
// the order of the score tiles' rows (so the 16 rows a wave reads together are neighbours, 16 bytes further apart
// than they are wide: no two lanes in one bank), latents as [dimension][32 keys].  Each wave masks with its own
// token's window; a wave whose token does not see a step at all sits it out.
template <int VT>
__global__ __launch_bounds__(256) void latent_attend_shared_kernel(
    const bf16_t* __restrict__ q_abs, const bf16_t* __restrict__ records, const bf16_t* __restrict__ latents_t,
    const int* __restrict__ seq_of_token, const int* __restrict__ positions, const int* __restrict__ block_table,
    const int* __restrict__ table_rows, int table_width, bf16_t* __restrict__ out, long tiles, int heads, int width,
    int page_size, long num_pages, float scale_log2, int window) {
  extern __shared__ unsigned char lds_bytes[];
  constexpr int kv_rank = VT * 16;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1);
  const long tile = static_cast<long>(blockIdx.x) * 4 + wave;      // (tiles are a multiple of 4)
  const int rho = lane & 15, g = lane >> 4;
  const long n = tile * 16 / heads;
  const int r = table_rows != nullptr ? table_rows[seq_of_token[n]] : seq_of_token[n];
  const int pos = positions[n];
  const int lowest = window > 0 ? max(0, pos - window + 1) : 0;
  const int* table = block_table + static_cast<long>(r) * table_width;
  // the block's tokens: the first wave's to the last wave's (positions rise with the rows of one request)
  const long n_first = static_cast<long>(blockIdx.x) * 4 * 16 / heads, n_last = (static_cast<long>(blockIdx.x) * 4 + 3) * 16 / heads;
  const int pos_first = positions[n_first], pos_last = positions[n_last];
  const int low_block = window > 0 ? max(0, pos_first - window + 1) : 0;

  const int chunks = width / 8, stride = (chunks + 1) * 16;
  unsigned char* qs = lds_bytes + static_cast<size_t>(wave) * 16 * stride;
  unsigned char* k_tile = lds_bytes + static_cast<size_t>(4) * 16 * stride;       // [32 rows][stride]
  unsigned char* v_tile = k_tile + 32 * stride;                                   // [kv_rank][64 bytes]
  const uintx4* q_rows = reinterpret_cast<const uintx4*>(q_abs + tile * 16 * width);
  for (int e = lane; e < 16 * chunks; e += kWave)
    *reinterpret_cast<uintx4*>(qs + (e / chunks) * stride + (e % chunks) * 16) = q_rows[e];
  const unsigned char* q_mine = qs + rho * stride + g * 16;

  // who fetches what of a step: thread (kk = t / 8, c0 = t % 8) the pieces c0, c0 + 8, ... of key kk's record; thread
  // (group = t % 4, d0 = t / 4) the 8 keys of `group` for the dimensions d0, d0 + 64, ...  One look into the block table
  // for each of the two, then loads that depend on nothing else.
  constexpr int kRecordTurns = 10, kLatentTurns = VT / 4;     // (host: chunks <= 8 * kRecordTurns)
  const int kk = threadIdx.x >> 3, c0 = threadIdx.x & 7;
  const int group = threadIdx.x & 3, d0 = threadIdx.x >> 2;
  const int row = ((kk >> 2) & 1) * 16 + (kk >> 3) * 4 + (kk & 3);     // the place of key kk among the score tiles' rows
  uintx4 ahead_k[kRecordTurns], ahead_v[kLatentTurns];
  bool poisoned = false;
  auto fetch = [&](int base) {
    const int key = base + kk, first = base + group * 8;
    const bool wanted_k = key >= low_block && key <= pos_last;
    const bool wanted_v = first + 7 >= low_block && first <= pos_last;
    const long page_k = wanted_k ? table[key / page_size] : 0;
    const long page_v = wanted_v ? table[first / page_size] : 0;
    const bool good_k = wanted_k && page_k >= 0 && page_k < num_pages, good_v = wanted_v && page_v >= 0 && page_v < num_pages;
    poisoned = poisoned || (wanted_k && !good_k) || (wanted_v && !good_v);
    const uintx4* from_k = reinterpret_cast<const uintx4*>(records + ((good_k ? page_k : 0) * page_size + key % page_size) * width);
    const bf16_t* from_v = latents_t + (good_v ? page_v : 0) * kv_rank * page_size + first % page_size;
#pragma unroll
    for (int i = 0; i < kRecordTurns; ++i) {
      const int c = c0 + 8 * i;
      ahead_k[i] = good_k && c < chunks ? from_k[c] : uintx4{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int i = 0; i < kLatentTurns; ++i)
      ahead_v[i] = good_v ? *reinterpret_cast<const uintx4*>(from_v + static_cast<long>(d0 + 64 * i) * page_size)
                          : uintx4{0u, 0u, 0u, 0u};
  };
  auto file = [&]() {
#pragma unroll
    for (int i = 0; i < kRecordTurns; ++i) {
      const int c = c0 + 8 * i;
      if (c < chunks) *reinterpret_cast<uintx4*>(k_tile + row * stride + c * 16) = ahead_k[i];
    }
#pragma unroll
    for (int i = 0; i < kLatentTurns; ++i)
      *reinterpret_cast<uintx4*>(v_tile + (d0 + 64 * i) * 64 + group * 16) = ahead_v[i];
  };

  floatx4 o[VT];
#pragma unroll
  for (int dt = 0; dt < VT; ++dt) o[dt] = floatx4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;
  const int steps32 = width / 32;
  const int first_base = low_block & ~31;
  fetch(first_base);
  for (int base = first_base; base <= pos_last; base += 32) {
    __syncthreads();                    // the step before has been read by everybody (and, the first time, q is in place)
    file();
    __syncthreads();
    if (base + 32 <= pos_last) fetch(base + 32);
    if (base + 31 < lowest || base > pos) continue;          // nothing of this step is this wave's token's to see
    const bool edge = base < lowest || base + 31 > pos;
    floatx4 s[2] = {floatx4{0.f, 0.f, 0.f, 0.f}, floatx4{0.f, 0.f, 0.f, 0.f}};
    const unsigned char* k0 = k_tile + rho * stride + g * 16;
    const unsigned char* k1 = k0 + 16 * stride;
    for (int t = 0; t < steps32; ++t) {
      const uintx4 qq = *reinterpret_cast<const uintx4*>(q_mine + t * 64);
      s[0] = mfma16(*reinterpret_cast<const uintx4*>(k0 + t * 64), qq, s[0]);
      s[1] = mfma16(*reinterpret_cast<const uintx4*>(k1 + t * 64), qq, s[1]);
    }
    uint32_t keep[4] = {0xffffffffu, 0xffffffffu, 0xffffffffu, 0xffffffffu};
    if (edge) {
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int key = base + g * 8 + j * 4 + i;
          if (key < lowest || key > pos) s[j][i] = -INFINITY;
        }
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int key = base + g * 8 + e;
        if (key < lowest || key > pos) keep[e >> 1] &= (e & 1) ? 0x0000ffffu : 0xffff0000u;
      }
    }
    float top = fmaxf(fmaxf(fmaxf(s[0][0], s[0][1]), fmaxf(s[0][2], s[0][3])),
                      fmaxf(fmaxf(s[1][0], s[1][1]), fmaxf(s[1][2], s[1][3])));
    top = fmaxf(top, __shfl_xor(top, 16, kWave));
    top = fmaxf(top, __shfl_xor(top, 32, kWave));
    const float m_new = fmaxf(m, top * scale_log2);
    const float m_safe = m_new == -INFINITY ? 0.f : m_new;
    const float correction = __builtin_amdgcn_exp2f(m - m_safe);
    floatx2 p[4];
    float sum = 0.f;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      p[e][0] = __builtin_amdgcn_exp2f(fmaf(s[e >> 1][(e & 1) * 2], scale_log2, -m_safe));
      p[e][1] = __builtin_amdgcn_exp2f(fmaf(s[e >> 1][(e & 1) * 2 + 1], scale_log2, -m_safe));
      sum += p[e][0] + p[e][1];
    }
    l = l * correction + sum;
    m = m_new;
    uint32_t high[4], low[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      high[e] = __builtin_bit_cast(uint32_t, __builtin_convertvector(p[e], bf16x2));
      const floatx2 rest = {p[e][0] - __uint_as_float(high[e] << 16), p[e][1] - __uint_as_float(high[e] & 0xffff0000u)};
      low[e] = __builtin_bit_cast(uint32_t, __builtin_convertvector(rest, bf16x2));
    }
    const uintx4 p_high = uintx4{high[0], high[1], high[2], high[3]}, p_low = uintx4{low[0], low[1], low[2], low[3]};
    if (__any(correction != 1.f)) {
#pragma unroll
      for (int dt = 0; dt < VT; ++dt) o[dt] *= correction;
    }
    const unsigned char* v_mine = v_tile + rho * 64 + g * 16;
#pragma unroll
    for (int dt = 0; dt < VT; ++dt) {
      uintx4 v = *reinterpret_cast<const uintx4*>(v_mine + dt * 16 * 64);
      if (edge) v = uintx4{v[0] & keep[0], v[1] & keep[1], v[2] & keep[2], v[3] & keep[3]};
      o[dt] = mfma16(v, p_low, mfma16(v, p_high, o[dt]));
    }
  }
  l += __shfl_xor(l, 16, kWave);
  l += __shfl_xor(l, 32, kWave);
  const bool any_poison = __syncthreads_or(poisoned);       // (a foreign page met by any thread of the block)
  const float inverse = 1.f / l;
  bf16_t* dst = out + (tile * 16 + rho) * kv_rank + g * 4;
#pragma unroll
  for (int dt = 0; dt < VT; ++dt) {
    floatx4 v = o[dt] * inverse;
    if (any_poison) v = floatx4{__uint_as_float(kPoison), __uint_as_float(kPoison), __uint_as_float(kPoison), __uint_as_float(kPoison)};
    store4<bf16_t>(dst + dt * 16, v);
  }
}

// The runs' shares of a column added up: each was formed against its own maximum m; against the largest of them
// every share counts exp2(m - M) times.  One block per (tile, column): the runs' factors are formed once, into LDS; a
// thread then owns dimensions and adds the runs' values in the order of the runs - loads that wait for nothing but
// each other's sum.
constexpr int kMergeRuns = 64;
__global__ __launch_bounds__(256) void latent_merge_kernel(const float* __restrict__ parts, bf16_t* __restrict__ out,
                                                           int segments, int kv_rank) {
  __shared__ float factors[kMergeRuns];
  __shared__ float total_of;
  const long column = blockIdx.x;                   // tile * 16 + rho
  const long tile = column / 16, rho = column % 16;
  const float* first = parts + ((tile * segments) * 16 + rho) * (kv_rank + 2);
  const long step = 16L * (kv_rank + 2);            // from a run's share to the next run's
  if (threadIdx.x < kWave) {
    const int lane = threadIdx.x;
    const float m = lane < segments ? first[lane * step + kv_rank] : -INFINITY;
    const float top = wave_max(m);
    const float factor = m == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m - top);
    factors[lane] = factor;
    const float total = wave_sum(lane < segments && m != -INFINITY ? first[lane * step + kv_rank + 1] * factor : 0.f);
    if (lane == 0) total_of = total;
  }
  __syncthreads();
  const float inverse = 1.f / total_of;
  for (int d = threadIdx.x; d < kv_rank; d += blockDim.x) {
    float acc = 0.f;
#pragma unroll 8
    for (int p = 0; p < segments; ++p) {
      const float f = factors[p];
      acc += f != 0.f ? first[p * step + d] * f : 0.f;
    }
    out[column * kv_rank + d] = from_float<bf16_t>(acc * inverse);
  }
}

template <int VT>
int launch_attend_mfma(const void* q_abs, const void* records, const void* latents_t, const int* seq_of_token,
                       const int* positions, const int* block_table, const int* table_rows, int table_width, void* out,
                       long tiles, int heads, int width, int page_size, long num_pages, float scale, int window,
                       int segment, int segments, float* parts, int one_request, hipStream_t stream) {
  constexpr int waves = 4;
  const size_t row_bytes = static_cast<size_t>(width / 8 + 1) * 16;
  // one request's long portion: blocks of four neighbouring tokens share each step's records through LDS
  const size_t shared_lds = (waves * 16 + 32) * row_bytes + static_cast<size_t>(VT) * 16 * 64;
  if (one_request && segments == 1 && tiles % 4 == 0 && tiles >= 64 && shared_lds <= device_facts().lds_bytes &&
      width / 8 <= 80 && VT % 4 == 0) {
    auto shared_kernel = latent_attend_shared_kernel<VT>;
    if (shared_lds > 64 * 1024 &&
        hipFuncSetAttribute(reinterpret_cast<const void*>(shared_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            static_cast<int>(shared_lds)) != hipSuccess)
      return -2;
    shared_kernel<<<static_cast<unsigned>(tiles / 4), 256, shared_lds, stream>>>(
        static_cast<const bf16_t*>(q_abs), static_cast<const bf16_t*>(records), static_cast<const bf16_t*>(latents_t),
        seq_of_token, positions, block_table, table_rows, table_width, static_cast<bf16_t*>(out), tiles, heads, width,
        page_size, num_pages, scale * 1.4426950408889634f, window);
    return AKV_LAUNCH_STATUS();
  }
  const size_t lds = static_cast<size_t>(waves) * 16 * (width / 8 + 1) * 16;
  auto kernel = latent_attend_mfma_kernel<VT>;
  if (lds > device_facts().lds_bytes) return -2;
  if (lds > 64 * 1024 && hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                             static_cast<int>(lds)) != hipSuccess)
    return -2;
  kernel<<<dim3(static_cast<unsigned>((tiles + waves - 1) / waves), segments), waves * kWave, lds, stream>>>(
      static_cast<const bf16_t*>(q_abs), static_cast<const bf16_t*>(records), static_cast<const bf16_t*>(latents_t),
      seq_of_token, positions, block_table, table_rows, table_width, static_cast<bf16_t*>(out), tiles, heads, width,
      page_size, num_pages, scale * 1.4426950408889634f, window, segment, segments, parts);
  const int status = AKV_LAUNCH_STATUS();
  if (status != 0 || segments == 1) return status;
  if (segments > kMergeRuns) return -2;
  latent_merge_kernel<<<static_cast<unsigned>(tiles * 16), 256, 0, stream>>>(parts, static_cast<bf16_t*>(out), segments, VT * 16);
  return AKV_LAUNCH_STATUS();
}

template <typename T, int KT>
int launch_attend(const float* q_abs, const void* records, const int* seq_of_token, const int* positions,
                  const int* block_table, const int* table_rows, int table_width, float* out, int tokens, int heads,
                  int kv_rank, int width, int page_size, long num_pages, float scale, int window, int waves,
                  size_t lds_bytes, hipStream_t stream) {
  auto kernel = latent_attend_kernel<T, KT>;
  if (lds_bytes > 64 * 1024 &&
      hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                          static_cast<int>(lds_bytes)) != hipSuccess)
    return -2;
  kernel<<<dim3(tokens, (heads + waves - 1) / waves), waves * kWave, lds_bytes, stream>>>(
      q_abs, static_cast<const T*>(records), seq_of_token, positions, block_table, table_rows, table_width, out, heads,
      kv_rank, width, page_size, num_pages, scale, window);
  return AKV_LAUNCH_STATUS();
}

size_t attend_lds(int kt, int width, int waves) {
  const size_t padded = width | 1;
  size_t floats = kt * padded;
  floats += floats & 1;
  return floats * 4 + static_cast<size_t>(kt) * 8 + static_cast<size_t>(waves) * (width + kt) * 4;
}

}  // namespace

extern "C" {

int akv_latent_encode(const void* down, int dtype, int tokens, int q_rank, int kv_rank, int rot, int rot_dims,
                      const float* q_weight, const float* kv_weight, float eps, const float* table, int table_positions,
                      const int* positions, const int* slot_map, void* cq, void* records, long record_slots,
                      void* latents_t, int page_size, int interleaved, long down_stride, hipStream_t stream) {
  if (tokens <= 0) return 0;
  const long needed = q_rank + (records != nullptr ? kv_rank + rot : 0);
  if (down_stride == 0) down_stride = needed;
  if (down_stride < needed) return -2;
  if (rot_dims % 2 || rot_dims > rot || q_rank <= 0 || (latents_t != nullptr && page_size <= 0)) return -2;
  AKV_DISPATCH(dtype, T, latent_encode_kernel<T><<<tokens, 256, 0, stream>>>(
                             static_cast<const T*>(down), q_rank, kv_rank, rot, rot_dims, q_weight, kv_weight, eps, table,
                             table_positions, positions, slot_map, static_cast<T*>(cq), static_cast<T*>(records),
                             record_slots, static_cast<T*>(latents_t), page_size, interleaved, down_stride));
  return AKV_LAUNCH_STATUS();
}

int akv_rotate_queries(const void* q, int dtype, long tokens, int heads, int dim, int rot, int rot_dims,
                       const float* table, int table_positions, const int* positions, void* q_abs, int out_dtype,
                       int width, int at, int interleaved, hipStream_t stream) {
  const long count = tokens * heads * rot;
  if (count <= 0) return 0;
  if (rot_dims % 2 || rot_dims > rot || at + rot > width) return -2;
  const unsigned blocks = static_cast<unsigned>((count + 255) / 256);
  if (out_dtype == kF32) {
    AKV_DISPATCH(dtype, T, rotate_queries_kernel<T, float><<<blocks, 256, 0, stream>>>(
                               static_cast<const T*>(q), tokens, heads, dim, rot, rot_dims, table, table_positions, positions,
                               static_cast<float*>(q_abs), width, at, interleaved));
  } else if (out_dtype == kBF16 && dtype == kBF16) {
    rotate_queries_kernel<bf16_t, bf16_t><<<blocks, 256, 0, stream>>>(
        static_cast<const bf16_t*>(q), tokens, heads, dim, rot, rot_dims, table, table_positions, positions,
        static_cast<bf16_t*>(q_abs), width, at, interleaved);
  } else {
    return -1;
  }
  return AKV_LAUNCH_STATUS();
}

int akv_heads_linear(const void* x, int x_dtype, long x_token_stride, long x_head_stride, const void* w, int w_dtype,
                     void* y, int y_dtype, long y_token_stride, long y_head_stride, int tokens, int heads, int ins,
                     int outs, hipStream_t stream) {
  if (tokens <= 0 || heads <= 0) return 0;
  if (ins <= 0 || outs <= 0) return -2;
  // few tokens: blocks of 64 outputs whose waves share the inputs (not in float32, whose sums keep one order whatever
  // the batch)
  const bool split = tokens <= 2 * kHeadTokens && !(x_dtype == kF32 && w_dtype == kF32 && y_dtype == kF32);
  const size_t lds_bytes = static_cast<size_t>(ins) * kHeadTokens * 4 + (split ? 3 * kWave * kHeadTokens * 4 : 0);
  if (lds_bytes > 64 * 1024) return -2;
  const int threads = split ? 256 : outs >= 256 ? 256 : (outs + kWave - 1) / kWave * kWave;
  const int per_block = split ? kWave : threads;
  const dim3 grid((tokens + kHeadTokens - 1) / kHeadTokens, heads, (outs + per_block - 1) / per_block);
#define AKV_HEADS_AS(TX, TW, TY, SPLIT)                                                                             \
  heads_linear_kernel<TX, TW, TY, SPLIT><<<grid, threads, lds_bytes, stream>>>(                                     \
      static_cast<const TX*>(x), x_token_stride, x_head_stride, static_cast<const TW*>(w), static_cast<TY*>(y),    \
      y_token_stride, y_head_stride, tokens, ins, outs)
#define AKV_HEADS(TX, TW, TY)                 \
  do {                                        \
    if (split) AKV_HEADS_AS(TX, TW, TY, true); \
    else AKV_HEADS_AS(TX, TW, TY, false);     \
  } while (0)
  if (x_dtype == kF32 && w_dtype == kF32 && y_dtype == kF32) AKV_HEADS(float, float, float);
  else if (x_dtype == kBF16 && w_dtype == kBF16 && y_dtype == kF32) AKV_HEADS(bf16_t, bf16_t, float);
  else if (x_dtype == kF32 && w_dtype == kBF16 && y_dtype == kBF16) AKV_HEADS(float, bf16_t, bf16_t);
  else if (x_dtype == kF32 && w_dtype == kBF16 && y_dtype == kF32) AKV_HEADS(float, bf16_t, float);
  else if (x_dtype == kBF16 && w_dtype == kBF16 && y_dtype == kBF16) AKV_HEADS(bf16_t, bf16_t, bf16_t);
  else return -1;
#undef AKV_HEADS_AS
#undef AKV_HEADS
  return AKV_LAUNCH_STATUS();
}

int akv_latent_attend(const float* q_abs, const void* records, int dtype, const int* seq_of_token, const int* positions,
                      const int* block_table, const int* table_rows, int table_width, float* out, int tokens, int heads,
                      int kv_rank, int width, int page_size, long num_pages, float scale, int window,
                      hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (kv_rank <= 0 || kv_rank > width || kv_rank > kMaxLatentRegs * kWave || page_size <= 0) return -2;
  const int waves = heads < 8 ? heads : 8;
  // the most keys a turn whose records, beside the heads' queries, fit the 64 KB every block may ask for
  int kt = 64;
  while (kt > 8 && attend_lds(kt, width, waves) > 64 * 1024) kt >>= 1;
  const size_t lds_bytes = attend_lds(kt, width, waves);
  if (lds_bytes > device_facts().lds_bytes) return -2;
#define AKV_ATTEND(T, KT)                                                                                               \
  return launch_attend<T, KT>(q_abs, records, seq_of_token, positions, block_table, table_rows, table_width, out, tokens, \
                              heads, kv_rank, width, page_size, num_pages, scale, window, waves, lds_bytes, stream)
  AKV_DISPATCH(dtype, T, {
    if (kt == 64) AKV_ATTEND(T, 64);
    if (kt == 32) AKV_ATTEND(T, 32);
    if (kt == 16) AKV_ATTEND(T, 16);
    AKV_ATTEND(T, 8);
  });
#undef AKV_ATTEND
  return -2;
}

int akv_latent_attend_mfma(const void* q_abs, const void* records, const void* latents_t, const int* seq_of_token,
                           const int* positions, const int* block_table, const int* table_rows, int table_width,
                           void* out, int tokens, int heads, int kv_rank, int width, int page_size, long num_pages,
                           float scale, int window, int segment, int segments, float* parts, int one_request,
                           hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (heads % 16 || width % 32 || kv_rank % 16 || kv_rank > width || page_size % 8) return -2;
  if (segments < 1 || (segments > 1 && (segment < 32 || segment % 32 || parts == nullptr))) return -2;
  const long tiles = static_cast<long>(tokens) * heads / 16;
#define AKV_MFMA(VT)                                                                                                   \
  return launch_attend_mfma<VT>(q_abs, records, latents_t, seq_of_token, positions, block_table, table_rows, table_width, \
                                out, tiles, heads, width, page_size, num_pages, scale, window, segment, segments, parts, one_request, stream)
  if (kv_rank == 128) AKV_MFMA(8);
  if (kv_rank == 256) AKV_MFMA(16);
  if (kv_rank == 512) AKV_MFMA(32);
#undef AKV_MFMA
  return -2;
}
}
