// Mixers whose requests carry a float32 state of fixed size from token to token:
//   retention - S [dim, vdim] per head, S <- decay S + k v^T, o = S^T q, with rotary positions on q and k, the unit norm of o
//   per head and the gate silu(g) in the same kernel - or, for a mixer that norms and gates all heads together, the raw
//   outputs in float32 for a kernel of its own; q, k and v may pass silu as they are read (`input_act`);
//   a gated linear recurrence - S [channels], S <- a S + sqrt(1 - a^2) i u with a = exp(rate r), r and i sigmoids of
//   block-diagonal products, the output S * gelu_tanh(y).
// Everything but the loads of the projections is float32.  A request's tokens are taken in the order of their positions
// whatever the step's cutting, and a token's sums run in a fixed order, so cuttings agree to rounding.

#include "common.h"
#include "api_parts.h"

using namespace akv;

namespace {

__device__ __forceinline__ float silu(float v) { return v / (1.f + expf(-v)); }
__device__ __forceinline__ float sigmoid(float v) { return 1.f / (1.f + expf(-v)); }
__device__ __forceinline__ float gelu_tanh(float v) {
  return 0.5f * v * (1.f + tanhf(0.7978845608028654f * (v + 0.044715f * v * v * v)));
}

// ---- retention ------------------------------------------------------------------------------------------------------
// A block is a (request, head).  Thread (p, v) owns S[p R + r][v], r < R, in registers.  Tokens are taken TB at a time:
// their rotated queries and keys and their values go to LDS, every thread runs its share of the TB recurrence steps and
// leaves its shares of the outputs, which are then added over p, normed and gated, a wave a token.
template <typename T, int R>
__global__ __launch_bounds__(1024) void retention_kernel(
    const T* __restrict__ projected, long stride, int heads, int dim, int vdim, int rot_dims,
    const float* __restrict__ table, int table_positions, float key_scale, const float* __restrict__ decay, float eps,
    float* __restrict__ state, long state_stride, const int* __restrict__ q_start, const int* __restrict__ seq_slots,
    const int* __restrict__ positions, T* __restrict__ out, int parts, int batch, long out_stride, float out_scale,
    int input_act, float* __restrict__ raw) {
  extern __shared__ float lds[];
  const int seq = blockIdx.x, h = blockIdx.y;
  const int tid = threadIdx.x, threads = blockDim.x;
  const int first = q_start[seq], count = q_start[seq + 1] - first;
  const int p = tid / vdim, v = tid % vdim;
  const bool owner = p < parts;
  float* qs = lds;                          // [batch][dim]
  float* ks = qs + batch * dim;             // [batch][dim]
  float* vs = ks + batch * dim;             // [batch][vdim]
  float* shares = vs + batch * vdim;        // [batch][parts][vdim]
  float* os = shares + batch * parts * vdim;  // [batch][vdim]
  float* mine = state + static_cast<long>(seq_slots[seq]) * state_stride + static_cast<long>(h) * dim * vdim;
  const float keep = decay[h];
  float S[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int d = p * R + r;
    S[r] = owner && d < dim ? mine[static_cast<long>(d) * vdim + v] : 0.f;
  }
  const long q_at = static_cast<long>(h) * dim, k_at = static_cast<long>(heads) * dim + q_at;
  const long v_at = 2L * heads * dim + static_cast<long>(h) * vdim, g_at = v_at + static_cast<long>(heads) * vdim;
  const int half = rot_dims / 2;
  const int waves = threads / kWave, wave = tid / kWave, lane = tid & (kWave - 1);
  for (int base = 0; base < count; base += batch) {
    const int tb = min(batch, count - base);
    for (int index = tid; index < tb * dim; index += threads) {
      const int t = index / dim, d = index % dim;
      const T* row = projected + static_cast<long>(first + base + t) * stride;
      float qv = to_float(row[q_at + d]), kv = to_float(row[k_at + d]);
      if (input_act) qv = silu(qv), kv = silu(kv);
      if (d < rot_dims) {
        const int i = d < half ? d : d - half;
        const int pos = min(positions[first + base + t], table_positions - 1);
        const float c = table[(static_cast<long>(pos) * half + i) * 2], s = table[(static_cast<long>(pos) * half + i) * 2 + 1];
        const int other = d < half ? d + half : d - half;
        float qo = to_float(row[q_at + other]), ko = to_float(row[k_at + other]);
        if (input_act) qo = silu(qo), ko = silu(ko);
        qv = d < half ? qv * c - qo * s : qv * c + qo * s;
        kv = d < half ? kv * c - ko * s : kv * c + ko * s;
      }
      qs[t * dim + d] = qv;
      ks[t * dim + d] = kv * key_scale;
    }
    for (int index = tid; index < tb * vdim; index += threads) {
      const int t = index / vdim, c = index % vdim;
      const float value = to_float(projected[static_cast<long>(first + base + t) * stride + v_at + c]);
      vs[index] = input_act ? silu(value) : value;
    }
    __syncthreads();
    if (owner) {
      for (int t = 0; t < tb; ++t) {
        const float value = vs[t * vdim + v];
        float share = 0.f;
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const int d = p * R + r;
          if (d < dim) {
            S[r] = fmaf(keep, S[r], ks[t * dim + d] * value);
            share = fmaf(S[r], qs[t * dim + d], share);
          }
        }
        shares[(t * parts + p) * vdim + v] = share;
      }
    }
    __syncthreads();
    for (int index = tid; index < tb * vdim; index += threads) {
      const int t = index / vdim, c = index % vdim;
      float o = 0.f;
      for (int part = 0; part < parts; ++part) o += shares[(t * parts + part) * vdim + c];
      os[index] = o;
    }
    __syncthreads();
    for (int t = wave; t < tb; t += waves) {
      const long n = first + base + t;
      if (raw != nullptr) {      // the heads' outputs as they are: whoever called norms and gates them
        for (int c = lane; c < vdim; c += kWave) raw[(n * heads + h) * vdim + c] = os[t * vdim + c];
        continue;
      }
      float squares = 0.f;
      for (int c = lane; c < vdim; c += kWave) squares += os[t * vdim + c] * os[t * vdim + c];
      const float scale = rsqrtf(wave_sum(squares) / static_cast<float>(vdim) + eps);
      for (int c = lane; c < vdim; c += kWave) {
        const float g = to_float(projected[n * stride + g_at + c]);
        out[n * out_stride + static_cast<long>(h) * vdim + c] = from_float<T>(os[t * vdim + c] * scale * silu(g) * out_scale);
      }
    }
    __syncthreads();
  }
  if (owner) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int d = p * R + r;
      if (d < dim) mine[static_cast<long>(d) * vdim + v] = S[r];
    }
  }
}

// ---- retention over portions: chunks of L tokens side by side -----------------------------------------------------------
// With w = decay:  S after a chunk = w^n S before + U,  U = sum_j w^(n - 1 - j) k_j v_j^T  (n tokens in the chunk), and
// o_t = w^(t + 1) S_before^T q_t + sum_(j <= t) w^(t - j) (q_t . k_j) v_j.  Three launches: every chunk's U; per request and
// head the states before its chunks, one after the other (U is replaced by them), and the request's new state; every
// chunk's outputs, normed and gated.  All of float32.
__device__ __forceinline__ float power(float w, int n) { return n == 0 ? 1.f : powf(w, static_cast<float>(n)); }

// rotated q (if `with_q`) and scaled rotated k of a chunk's tokens into LDS rows of `pitch` floats, its values into vs
template <typename T>
__device__ __forceinline__ void load_chunk(const T* __restrict__ projected, long stride, int heads, int h, int dim, int vdim,
                                           int rot_dims, const float* __restrict__ table, int table_positions,
                                           float key_scale, const int* __restrict__ positions, int first, int n,
                                           float* qs, float* ks, float* vs, int pitch, bool with_q, int input_act) {
  const long q_at = static_cast<long>(h) * dim, k_at = static_cast<long>(heads) * dim + q_at;
  const long v_at = 2L * heads * dim + static_cast<long>(h) * vdim;
  const int half = rot_dims / 2;
  for (int index = threadIdx.x; index < n * dim; index += blockDim.x) {
    const int t = index / dim, d = index % dim;
    const T* row = projected + static_cast<long>(first + t) * stride;
    float qv = with_q ? to_float(row[q_at + d]) : 0.f, kv = to_float(row[k_at + d]);
    if (input_act) qv = silu(qv), kv = silu(kv);
    if (d < rot_dims) {
      const int i = d < half ? d : d - half;
      const int pos = min(positions[first + t], table_positions - 1);
      const float c = table[(static_cast<long>(pos) * half + i) * 2], sn = table[(static_cast<long>(pos) * half + i) * 2 + 1];
      const int other = d < half ? d + half : d - half;
      float ko = to_float(row[k_at + other]);
      if (input_act) ko = silu(ko);
      kv = d < half ? kv * c - ko * sn : kv * c + ko * sn;
      if (with_q) {
        float qo = to_float(row[q_at + other]);
        if (input_act) qo = silu(qo);
        qv = d < half ? qv * c - qo * sn : qv * c + qo * sn;
      }
    }
    if (with_q) qs[t * pitch + d] = qv;
    ks[t * pitch + d] = kv * key_scale;
  }
  for (int index = threadIdx.x; index < n * vdim; index += blockDim.x) {
    const float value = to_float(projected[static_cast<long>(first + index / vdim) * stride + v_at + index % vdim]);
    vs[index] = input_act ? silu(value) : value;
  }
}

template <typename T>
__global__ __launch_bounds__(256) void retention_chunk_sums_kernel(
    const T* __restrict__ projected, long stride, int heads, int dim, int vdim, int rot_dims,
    const float* __restrict__ table, int table_positions, float key_scale, const float* __restrict__ decay,
    const int* __restrict__ q_start, const int* __restrict__ positions, float* __restrict__ sums, int length, int chunks,
    int input_act) {
  extern __shared__ float lds[];
  const int seq = blockIdx.x, h = blockIdx.y, chunk = blockIdx.z;
  const int first = q_start[seq], count = q_start[seq + 1] - first;
  if (chunk * length >= count) return;
  const int n = min(length, count - chunk * length), pitch = dim + 1;
  float* ks = lds;                   // [length][pitch]
  float* vs = ks + length * pitch;   // [length][vdim]
  float* ws = vs + length * vdim;    // [length]
  load_chunk(projected, stride, heads, h, dim, vdim, rot_dims, table, table_positions, key_scale, positions,
             first + chunk * length, n, nullptr, ks, vs, pitch, false, input_act);
  const float w = decay[h];
  for (int j = threadIdx.x; j < n; j += blockDim.x) ws[j] = power(w, n - 1 - j);
  __syncthreads();
  float* mine = sums + ((static_cast<long>(seq) * heads + h) * chunks + chunk) * dim * vdim;
  // a thread owns patches of 8 x 8 of U: a token's 8 keys and 8 values from LDS feed 64 multiply-adds
  const int across = (vdim + 7) / 8, patches = ((dim + 7) / 8) * across;
  for (int patch = threadIdx.x; patch < patches; patch += blockDim.x) {
    const int d0 = patch / across * 8, v0 = patch % across * 8;
    float total[8][8];
#pragma unroll
    for (int a = 0; a < 8; ++a)
#pragma unroll
      for (int b = 0; b < 8; ++b) total[a][b] = 0.f;
    for (int j = 0; j < n; ++j) {
      float kd[8], vv[8];
#pragma unroll
      for (int a = 0; a < 8; ++a) kd[a] = d0 + a < dim ? ws[j] * ks[j * pitch + d0 + a] : 0.f;
#pragma unroll
      for (int b = 0; b < 8; ++b) vv[b] = v0 + b < vdim ? vs[j * vdim + v0 + b] : 0.f;
#pragma unroll
      for (int a = 0; a < 8; ++a)
#pragma unroll
        for (int b = 0; b < 8; ++b) total[a][b] = fmaf(kd[a], vv[b], total[a][b]);
    }
#pragma unroll
    for (int a = 0; a < 8; ++a)
#pragma unroll
      for (int b = 0; b < 8; ++b)
        if (d0 + a < dim && v0 + b < vdim) mine[static_cast<long>(d0 + a) * vdim + v0 + b] = total[a][b];
  }
}

// sums [seq][head][chunk][dim * vdim]: U of every chunk; before: the state before every chunk, laid out the same way
__global__ __launch_bounds__(256) void retention_chunk_states_kernel(const float* __restrict__ sums,
                                                                     float* __restrict__ before, float* __restrict__ state,
                                                                     long state_stride, const float* __restrict__ decay,
                                                                     const int* __restrict__ q_start,
                                                                     const int* __restrict__ seq_slots, int heads,
                                                                     int size, int length, int chunks) {
  const int seq = blockIdx.x, h = blockIdx.y;
  const int item = blockIdx.z * blockDim.x + threadIdx.x;
  if (item >= size) return;
  const int count = q_start[seq + 1] - q_start[seq];
  float* kept = state + static_cast<long>(seq_slots[seq]) * state_stride + static_cast<long>(h) * size + item;
  const long base = (static_cast<long>(seq) * heads + h) * chunks * size + item;
  const float w = decay[h], whole = power(w, length);
  float S = *kept;
#pragma unroll 8
  for (int chunk = 0; chunk * length < count; ++chunk) {
    const int n = min(length, count - chunk * length);
    const float added = sums[base + static_cast<long>(chunk) * size];
    before[base + static_cast<long>(chunk) * size] = S;
    S = fmaf(n == length ? whole : power(w, n), S, added);
  }
  *kept = S;
}

template <typename T, int GROUPS>
__global__ __launch_bounds__(256) void retention_chunk_outputs_kernel(
    const T* __restrict__ projected, long stride, int heads, int dim, int vdim, int rot_dims,
    const float* __restrict__ table, int table_positions, float key_scale, const float* __restrict__ decay, float eps,
    const int* __restrict__ q_start, const int* __restrict__ positions, const float* __restrict__ states, int length,
    int chunks, T* __restrict__ out, long out_stride, float out_scale, int input_act, float* __restrict__ raw) {
  extern __shared__ float lds[];
  const int seq = blockIdx.x, h = blockIdx.y, chunk = blockIdx.z;
  const int first = q_start[seq], count = q_start[seq + 1] - first;
  if (chunk * length >= count) return;
  const int n = min(length, count - chunk * length), pitch = dim + 1;
  float* qs = lds;                   // [length][pitch]
  float* ks = qs + length * pitch;   // [length][pitch]
  float* vs = ks + length * pitch;   // [length][vdim]
  float* os = vs + length * vdim;    // [length][vdim]
  float* as = os + length * vdim;    // [length][length + 1]: w^(t - j) (q_t . k_j), j <= t
  float* ws = as + length * (length + 1);   // [length + 1]: w^0 .. w^length
  const int row0 = first + chunk * length;
  load_chunk(projected, stride, heads, h, dim, vdim, rot_dims, table, table_positions, key_scale, positions, row0, n, qs, ks,
             vs, pitch, true, input_act);
  const float w = decay[h];
  for (int j = threadIdx.x; j <= n; j += blockDim.x) ws[j] = power(w, j);
  __syncthreads();
  for (int item = threadIdx.x; item < n * n; item += blockDim.x) {
    const int t = item / n, j = item % n;
    float dot = 0.f;
    if (j <= t) {
      for (int d = 0; d < dim; ++d) dot = fmaf(qs[t * pitch + d], ks[j * pitch + d], dot);
      dot *= ws[t - j];
    }
    as[t * (length + 1) + j] = dot;
  }
  __syncthreads();
  const float* before = states + ((static_cast<long>(seq) * heads + h) * chunks + chunk) * dim * vdim;
  // a thread keeps a column v of the values and the tokens group, group + GROUPS, ...: what it reads of the state before
  // the chunk and of the chunk's values it reads once for all its tokens
  constexpr int TP = 32 / GROUPS;
  const int lanes = 256 / GROUPS, group = threadIdx.x / lanes;
  for (int v = threadIdx.x % lanes; v < vdim; v += lanes) {
    float carried[TP], within[TP];
#pragma unroll
    for (int k = 0; k < TP; ++k) carried[k] = within[k] = 0.f;
    for (int d0 = 0; d0 < dim; d0 += 8) {       // eight rows of the state are asked for before the first is used
      float held[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) held[e] = d0 + e < dim ? before[static_cast<long>(d0 + e) * vdim + v] : 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int d = min(d0 + e, dim - 1);
#pragma unroll
        for (int k = 0; k < TP; ++k) {
          const int t = min(group + k * GROUPS, length - 1);      // (rows beyond the chunk's tokens count for nothing)
          carried[k] = fmaf(qs[t * pitch + d], held[e], carried[k]);
        }
      }
    }
    for (int j = 0; j < n; ++j) {
      const float value = vs[j * vdim + v];
#pragma unroll
      for (int k = 0; k < TP; ++k) {
        const int t = group + k * GROUPS;
        if (t < n && j <= t) within[k] = fmaf(as[t * (length + 1) + j], value, within[k]);
      }
    }
#pragma unroll
    for (int k = 0; k < TP; ++k) {
      const int t = group + k * GROUPS;
      if (t < n) os[t * vdim + v] = fmaf(ws[t + 1], carried[k], within[k]);
    }
  }
  __syncthreads();
  const int waves = blockDim.x / kWave, wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1);
  const long g_at = 2L * heads * dim + static_cast<long>(heads) * vdim + static_cast<long>(h) * vdim;
  for (int t = wave; t < n; t += waves) {
    const long row = row0 + t;
    if (raw != nullptr) {
      for (int c = lane; c < vdim; c += kWave) raw[(row * heads + h) * vdim + c] = os[t * vdim + c];
      continue;
    }
    float squares = 0.f;
    for (int c = lane; c < vdim; c += kWave) squares += os[t * vdim + c] * os[t * vdim + c];
    const float scale = rsqrtf(wave_sum(squares) / static_cast<float>(vdim) + eps);
    for (int c = lane; c < vdim; c += kWave) {
      const float g = to_float(projected[row * stride + g_at + c]);
      out[row * out_stride + static_cast<long>(h) * vdim + c] = from_float<T>(os[t * vdim + c] * scale * silu(g) * out_scale);
    }
  }
}

// ---- gated linear recurrence ------------------------------------------------------------------------------------------
// A block is a request and `ch` neighbouring channels (64, or 16 where runs are many); its threads cut the request's
// tokens of this step into blockDim.x / ch runs.
// Thread (run, channel) first takes its run from a state of zero - which gives the run's product of decays and what the
// run adds -, the runs' pairs meet in LDS, every thread folds the pairs of the runs before its own onto the request's
// state, and takes its run again from there, now writing S * gelu_tanh(y).  Tokens eight at a time: everything that
// does not depend on the state - gates, decays, the fed values - is formed for the eight first.
template <typename T>
__global__ __launch_bounds__(1024) void gated_linear_scan_kernel(
    const T* __restrict__ u, const float* __restrict__ gates, const float* __restrict__ gate_bias,
    const float* __restrict__ rate, const T* __restrict__ y, long y_stride, int channels, int block_width,
    float* __restrict__ state, long state_stride, const int* __restrict__ q_start, const int* __restrict__ seq_slots,
    T* __restrict__ out, int ch) {
  __shared__ float products[1024], sums[1024];
  const int seq = blockIdx.x;
  const int lane = threadIdx.x % ch, run = threadIdx.x / ch, runs = blockDim.x / ch;
  const int c = blockIdx.y * ch + lane;
  const bool live = c < channels;
  const int first = q_start[seq], count = q_start[seq + 1] - first;
  const int per_run = (count + runs - 1) / runs;
  const int lo = min(run * per_run, count), hi = min(lo + per_run, count);
  const int cc = live ? c : 0;
  const int b = cc / block_width, j = cc % block_width;
  const long gate_at = static_cast<long>(b) * 2 * block_width + j;      // (recurrence gate; the input gate block_width on)
  const float bias_r = gate_bias[gate_at], bias_i = gate_bias[gate_at + block_width], slope = rate[cc];
  float* mine = state + static_cast<long>(seq_slots[seq]) * state_stride + cc;
  constexpr int kStep = 8;
  float S = runs > 1 ? 0.f : *mine;
  for (int pass = (runs > 1 ? 0 : 1); pass < 2; ++pass) {
    float product = 1.f;
    for (int base = lo; base < hi; base += kStep) {
      float a[kStep], f[kStep];
#pragma unroll
      for (int t = 0; t < kStep; ++t) {
        const long n = first + min(base + t, hi - 1);
        const float r = sigmoid(gates[n * 2 * channels + gate_at] + bias_r);
        const float i = sigmoid(gates[n * 2 * channels + gate_at + block_width] + bias_i);
        a[t] = expf(slope * r);
        // 1 - a^2 = -expm1(2 log a): for decays close to 1 the difference of the squares would keep few of its bits
        f[t] = sqrtf(-expm1f(2.f * slope * r)) * i * to_float(u[n * channels + cc]);
      }
      if (pass == 0) {
#pragma unroll
        for (int t = 0; t < kStep; ++t) {
          if (base + t < hi) {
            S = fmaf(a[t], S, f[t]);
            product *= a[t];
          }
        }
      } else {
#pragma unroll
        for (int t = 0; t < kStep; ++t) {
          if (base + t < hi) {
            S = fmaf(a[t], S, f[t]);
            const long n = first + base + t;
            if (live) out[n * channels + c] = from_float<T>(S * gelu_tanh(to_float(y[n * y_stride + c])));
          }
        }
      }
    }
    if (pass == 0) {
      products[run * ch + lane] = product;
      sums[run * ch + lane] = S;
      __syncthreads();
      S = *mine;
      for (int before = 0; before < run; ++before) S = fmaf(products[before * ch + lane], S, sums[before * ch + lane]);
    }
  }
  if (run == runs - 1 && live) *mine = S;
}

template <typename T, int GROUPS>
int launch_retention_outputs(const dim3 grid, size_t lds, hipStream_t stream, const T* projected, long stride, int heads, int dim,
                             int vdim, int rot_dims, const float* table, int table_positions, float key_scale,
                             const float* decay, float eps, const int* q_start, const int* positions, const float* states,
                             int length, int chunks, T* out, long out_stride, float out_scale, int input_act, float* raw) {
  // (asked for once per kernel, for the most a launch may want: a step that is being recorded then changes no attribute)
  static bool allowed = false;
  if (lds > 64 * 1024 && !allowed) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&retention_chunk_outputs_kernel<T, GROUPS>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024) != hipSuccess)
      return -2;
    allowed = true;
  }
  retention_chunk_outputs_kernel<T, GROUPS><<<grid, 256, lds, stream>>>(projected, stride, heads, dim, vdim, rot_dims, table,
                                                                        table_positions, key_scale, decay, eps, q_start,
                                                                        positions, states, length, chunks, out, out_stride,
                                                                        out_scale, input_act, raw);
  return 0;
}

template <typename T>
int launch_retention_chunked(const T* projected, long stride, int seqs, int heads, int dim, int vdim, int rot_dims,
                             const float* table, int table_positions, float key_scale, const float* decay, float eps,
                             float* state, long state_stride, const int* q_start, const int* seq_slots, const int* positions,
                             T* out, long out_stride, float out_scale, float* sums, float* states, int length, int chunks,
                             size_t lds_sums, size_t lds_outputs, int input_act, float* raw, hipStream_t stream) {
  const dim3 grid(seqs, heads, chunks);
  const int size = dim * vdim;
  static bool allowed = false;
  if (lds_sums > 64 * 1024 && !allowed) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&retention_chunk_sums_kernel<T>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024) != hipSuccess)
      return -2;
    allowed = true;
  }
  retention_chunk_sums_kernel<T><<<grid, 256, lds_sums, stream>>>(projected, stride, heads, dim, vdim, rot_dims, table,
                                                                table_positions, key_scale, decay, q_start, positions, sums,
                                                                length, chunks, input_act);
  retention_chunk_states_kernel<<<dim3(seqs, heads, (size + 255) / 256), 256, 0, stream>>>(
      sums, states, state, state_stride, decay, q_start, seq_slots, heads, size, length, chunks);
#define AKV_OUTPUTS(GROUPS)                                                                                               \
  launch_retention_outputs<T, GROUPS>(grid, lds_outputs, stream, projected, stride, heads, dim, vdim, rot_dims, table,       \
                                      table_positions, key_scale, decay, eps, q_start, positions, states, length, chunks, out, \
                                      out_stride, out_scale, input_act, raw)
  if (vdim <= 32) return AKV_OUTPUTS(8);
  if (vdim <= 64) return AKV_OUTPUTS(4);
  if (vdim <= 128) return AKV_OUTPUTS(2);
  return AKV_OUTPUTS(1);
#undef AKV_OUTPUTS
}

}  // namespace

extern "C" {

int akv_retention(const void* projected, long stride, int dtype, int seqs, int heads, int dim, int vdim, int rot_dims,
                  const float* table, int table_positions, float key_scale, const float* decay, float eps, float* state,
                  long state_stride, const int* q_start, const int* seq_slots, const int* positions, void* out,
                  long out_stride, float out_scale, int input_act, float* raw, hipStream_t stream) {
  if (seqs <= 0) return 0;
  if (heads <= 0 || dim <= 0 || vdim <= 0 || vdim > 1024 || rot_dims < 0 || rot_dims % 2 || rot_dims > dim) return -2;
  if (rot_dims > 0 && (table == nullptr || table_positions <= 0)) return -2;
  int per_thread = 0;
  for (int r : {4, 8, 16, 32, 64}) {
    if (static_cast<long>(vdim) * ((dim + r - 1) / r) <= 1024) {
      per_thread = r;
      break;
    }
  }
  if (per_thread == 0) return -2;
  const int parts = (dim + per_thread - 1) / per_thread;
  const int threads = (vdim * parts + kWave - 1) / kWave * kWave;
  int batch = 16;
  auto lds_of = [&](int tb) { return static_cast<size_t>(tb) * (2 * dim + 2 * vdim + parts * vdim) * 4; };
  while (batch > 1 && lds_of(batch) > 64 * 1024) batch /= 2;
  if (lds_of(batch) > 64 * 1024) return -2;
  const dim3 grid(seqs, heads);
#define AKV_RETENTION(R)                                                                                                \
  AKV_DISPATCH(dtype, T, retention_kernel<T, R><<<grid, threads, lds_of(batch), stream>>>(                             \
                             static_cast<const T*>(projected), stride, heads, dim, vdim, rot_dims, table, table_positions, \
                             key_scale, decay, eps, state, state_stride, q_start, seq_slots, positions,                 \
                             static_cast<T*>(out), parts, batch, out_stride, out_scale, input_act, raw))
  switch (per_thread) {
    case 4: AKV_RETENTION(4); break;
    case 8: AKV_RETENTION(8); break;
    case 16: AKV_RETENTION(16); break;
    case 32: AKV_RETENTION(32); break;
    default: AKV_RETENTION(64); break;
  }
#undef AKV_RETENTION
  return AKV_LAUNCH_STATUS();
}

// The same over chunks of `length` tokens side by side (see above): `sums` holds 2 * seqs * heads * chunks * dim * vdim
// floats (the chunks' sums, then the states before them), chunks = the most chunks a request of the step has.
int akv_retention_chunked(const void* projected, long stride, int dtype, int seqs, int heads, int dim, int vdim, int rot_dims,
                          const float* table, int table_positions, float key_scale, const float* decay, float eps,
                          float* state, long state_stride, const int* q_start, const int* seq_slots, const int* positions,
                          void* out, long out_stride, float out_scale, float* sums, int length, int chunks, int input_act,
                          float* raw, hipStream_t stream) {
  if (seqs <= 0 || chunks <= 0) return 0;
  if (heads <= 0 || dim <= 0 || vdim <= 0 || rot_dims < 0 || rot_dims % 2 || rot_dims > dim || length < 1 || length > 32) return -2;
  if (rot_dims > 0 && (table == nullptr || table_positions <= 0)) return -2;
  const int pitch = dim + 1;
  const size_t lds_sums = static_cast<size_t>(length * pitch + length * vdim + length) * 4;
  const size_t lds_outputs = static_cast<size_t>(2 * length * pitch + 2 * length * vdim + length * (length + 1) + length + 1) * 4;
  if (lds_sums > 128 * 1024 || lds_outputs > 128 * 1024) return -2;
  float* states = sums + static_cast<long>(seqs) * heads * chunks * dim * vdim;
  int status = 0;
  AKV_DISPATCH(dtype, T, status = launch_retention_chunked<T>(
                             static_cast<const T*>(projected), stride, seqs, heads, dim, vdim, rot_dims, table, table_positions,
                             key_scale, decay, eps, state, state_stride, q_start, seq_slots, positions, static_cast<T*>(out),
                             out_stride, out_scale, sums, states, length, chunks, lds_sums, lds_outputs, input_act, raw,
                             stream));
  if (status != 0) return status;
  return AKV_LAUNCH_STATUS();
}

int akv_gated_linear_scan(const void* u, int dtype, const float* gates, const float* gate_bias, const float* rate,
                          const void* y, long y_stride, int seqs, int channels, int blocks, int runs, float* state,
                          long state_stride, const int* q_start, const int* seq_slots, void* out, hipStream_t stream) {
  if (seqs <= 0) return 0;
  if (channels <= 0 || blocks <= 0 || channels % blocks || runs < 1 || runs > 64) return -2;
  const int ch = runs > 16 ? 16 : kWave;
  const dim3 grid(seqs, (channels + ch - 1) / ch);
  AKV_DISPATCH(dtype, T, gated_linear_scan_kernel<T><<<grid, runs * ch, 0, stream>>>(
                             static_cast<const T*>(u), gates, gate_bias, rate, static_cast<const T*>(y), y_stride, channels,
                             channels / blocks, state, state_stride, q_start, seq_slots, static_cast<T*>(out), ch));
  return AKV_LAUNCH_STATUS();
}
}
