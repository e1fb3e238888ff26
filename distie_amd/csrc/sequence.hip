// Kernels of mixers and arrangements that carry something from token to token besides keys and values:
// several residual streams with learned read, mix and write weights; a short causal convolution over time
// whose last inputs are a request's state; attention projections with such a convolution, a partial rotation
// and the cache write behind it; a decayed outer-product state (linear attention) scanned over the tokens;
// gates. What such designs keep in 32-bit is float32 here in either precision: the
// streams, norm statistics, angles, the state and every sum that enters it.
//
// A step is a flattened batch: token t belongs to request token_request[t], whose new tokens are rows
// cu_q[b] .. cu_q[b+1]-1 and whose state is row state_slots[b] of a state tensor.
#include "common.h"

namespace {

constexpr int MAX_STREAMS = 8;
constexpr int MAX_TAPS = 16;

__device__ __forceinline__ float sigmoidf(float x) { return 1.f / (1.f + __expf(-x)); }
__device__ __forceinline__ float siluf(float x) { return x / (1.f + __expf(-x)); }
// kinds: 0 relu squared, 1 silu, 2 gelu (tanh form), 3 relu
__device__ __forceinline__ float activate(float z, int kind) {
  if (kind == 0) {
    const float p = fmaxf(z, 0.f);
    return p * p;
  }
  if (kind == 1) return z / (1.f + expf(-z));
  if (kind == 2) return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
  return fmaxf(z, 0.f);
}
// a query temperature by position: 1 + coef * ln(floor((p + 1) / every) + 1); every < 1: none
__device__ __forceinline__ float query_temperature(const int32_t* __restrict__ positions, int64_t t, float coef, int every) {
  if (every < 1) return 1.f;
  return 1.f + coef * logf(static_cast<float>((positions[t] + 1) / every) + 1.f);
}
// two values rounded to bfloat16 as one 32-bit word (the first in the low half)
__device__ __forceinline__ uint32_t bf16_word(float lo, float hi) {
  return static_cast<uint32_t>(__builtin_bit_cast(uint16_t, static_cast<bf16_t>(lo))) |
         (static_cast<uint32_t>(__builtin_bit_cast(uint16_t, static_cast<bf16_t>(hi))) << 16);
}

// ---------------------------------------------------------------------------------------------------
// Residual streams. streams float32 [T, S, C]. In this order, each step optional:
//   init:   x_s = init[t] for every s                                   (the embedding output)
//   write:  x_j <- sum_s mix[s, j] x_s + out_w[j] * y * sigmoid(gate)   (all streams at once from the old ones)
//   read:   u = sum_s in_w[s] x_s;  h = norm(u) * weight                (kind 0: u itself, 1: centred, 2: root mean square)
// One block a token; u of the whole row waits in LDS between the two passes of the statistics.
// MS: the most streams this instance takes (its loops are unrolled to that, so the streams stay in registers).
// V: channels a thread takes at a time, 4 (16-byte loads of float32, 8-byte loads of bfloat16; the width must be a
// multiple of 4) or 1. With V = 4 a row of up to 4 x the block's threads is loaded in one go, every load under way
// at once, which is what a step of few rows waits for.
template <int V, typename T>
__device__ __forceinline__ void loadv(const T* __restrict__ p, float out[V]) {
  if constexpr (V == 4 && sizeof(T) == 4) {
    const float4 v = *reinterpret_cast<const float4*>(p);
    out[0] = v.x, out[1] = v.y, out[2] = v.z, out[3] = v.w;
  } else if constexpr (V == 4) {
    const uint2 v = *reinterpret_cast<const uint2*>(p);
    out[0] = __uint_as_float(v.x << 16), out[1] = __uint_as_float(v.x & 0xffff0000u);
    out[2] = __uint_as_float(v.y << 16), out[3] = __uint_as_float(v.y & 0xffff0000u);
  } else {
#pragma unroll
    for (int k = 0; k < V; ++k) out[k] = to_float(p[k]);
  }
}

template <int V, typename T>
__device__ __forceinline__ void storev(T* __restrict__ p, const float v[V]) {
  if constexpr (V == 4 && sizeof(T) == 4) {
    *reinterpret_cast<float4*>(p) = float4{v[0], v[1], v[2], v[3]};
  } else if constexpr (V == 4) {
    *reinterpret_cast<uint2*>(p) = uint2{bf16_word(v[0], v[1]), bf16_word(v[2], v[3])};
  } else {
#pragma unroll
    for (int k = 0; k < V; ++k) p[k] = from_float<T>(v[k]);
  }
}

// the sum of `slices` vectors that lie `stride` elements apart, added in order
template <int V, typename T>
__device__ __forceinline__ void sumv(const T* __restrict__ p, int slices, int64_t stride, float out[V]) {
  loadv<V>(p, out);
  for (int s = 1; s < slices; s += 4) {
    float a[4][V];
#pragma unroll
    for (int u = 0; u < 4; ++u) loadv<V>(p + min(s + u, slices - 1) * stride, a[u]);
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (s + u < slices) {
#pragma unroll
        for (int k = 0; k < V; ++k) out[k] += a[u][k];
      }
  }
}

template <int MS, int V, typename Y, typename G, typename W, typename H>
__global__ void hyper_step_kernel(float* __restrict__ streams, int S, const float* __restrict__ init, const Y* __restrict__ y,
                                  int y_slices, int64_t y_slice_stride, const G* __restrict__ gate, int64_t gate_ld,
                                  int gate_slices, int64_t gate_slice_stride,
                                  const float* __restrict__ mix, const float* __restrict__ out_w,
                                  const float* __restrict__ in_w, const W* __restrict__ norm_w, int kind, float eps,
                                  H* __restrict__ h, int C) {
  extern __shared__ float row[];
  __shared__ float scratch[16];
  const int64_t t = blockIdx.x;
  float* x = streams + t * S * C;
  float m[MS][MS], ow[MS], iw[MS];
#pragma unroll
  for (int i = 0; i < MS; ++i) {
    ow[i] = (y != nullptr && i < S) ? out_w[i] : 0.f;
    iw[i] = (h != nullptr && i < S) ? in_w[i] : 0.f;
#pragma unroll
    for (int j = 0; j < MS; ++j) m[i][j] = (y != nullptr && i < S && j < S) ? mix[i * S + j] : 0.f;
  }
  float sum = 0.f;
  for (int c = V * threadIdx.x; c < C; c += V * blockDim.x) {
    float v[MS][V];
#pragma unroll
    for (int s = 0; s < MS; ++s) {
      if (s < S) {
        loadv<V>(init != nullptr ? init + t * C + c : x + s * C + c, v[s]);
      } else {
#pragma unroll
        for (int k = 0; k < V; ++k) v[s][k] = 0.f;
      }
    }
    if (y != nullptr) {
      float d[V];
      sumv<V>(y + t * C + c, y_slices, y_slice_stride, d);
      if (gate != nullptr) {
        float g[V];
        sumv<V>(gate + t * gate_ld + c, gate_slices, gate_slice_stride, g);
#pragma unroll
        for (int k = 0; k < V; ++k) d[k] *= sigmoidf(g[k]);
      }
      float n[MS][V];
#pragma unroll
      for (int j = 0; j < MS; ++j)
#pragma unroll
        for (int k = 0; k < V; ++k) {
          float a = 0.f;
#pragma unroll
          for (int s = 0; s < MS; ++s) a += m[s][j] * v[s][k];
          n[j][k] = a + ow[j] * d[k];
        }
#pragma unroll
      for (int j = 0; j < MS; ++j)
#pragma unroll
        for (int k = 0; k < V; ++k) v[j][k] = n[j][k];
    }
    if (init != nullptr || y != nullptr) {
#pragma unroll
      for (int s = 0; s < MS; ++s)
        if (s < S) storev<V>(x + s * C + c, v[s]);
    }
    if (h != nullptr) {
#pragma unroll
      for (int k = 0; k < V; ++k) {
        float u = 0.f;
#pragma unroll
        for (int s = 0; s < MS; ++s) u += iw[s] * v[s][k];
        row[c + k] = u;
        sum += kind == 2 ? u * u : u;
      }
    }
  }
  if (h == nullptr) return;
  H* out = h + t * C;
  if (kind == 0) {
    for (int c = V * threadIdx.x; c < C; c += V * blockDim.x) storev<V>(out + c, row + c);
    return;
  }
  sum = block_sum(sum, scratch);
  float mean = 0.f, scale;
  if (kind == 1) {
    mean = sum / C;
    float dev = 0.f;
    for (int c = V * threadIdx.x; c < C; c += V * blockDim.x) {
#pragma unroll
      for (int k = 0; k < V; ++k) {
        const float d = row[c + k] - mean;
        dev += d * d;
      }
    }
    dev = block_sum(dev, scratch);
    scale = 1.f / sqrtf(dev / C + eps);
  } else {
    scale = 1.f / sqrtf(sum / C + eps);
  }
  for (int c = V * threadIdx.x; c < C; c += V * blockDim.x) {
    float w[V], r[V];
    loadv<V>(norm_w + c, w);
#pragma unroll
    for (int k = 0; k < V; ++k) r[k] = (row[c + k] - mean) * scale * w[k];
    storev<V>(out + c, r);
  }
}

// ---------------------------------------------------------------------------------------------------
// Short causal convolution over time, one filter a channel:
//   out[t, c] = (residual ? x[t, c] : 0) + sum_j w[c, j] * x_(t - taps + 1 + j)[c],
// inputs before the start of the step's rows come from the request's state (float32 [slots, taps - 1, N], the
// last taps - 1 inputs, oldest first; zeros at the start of a sequence). A request that brings one token has
// its state moved on here as well (nobody else reads it); the others by `conv_state_kernel` behind this one.
template <typename X>
__device__ __forceinline__ float conv_at(const X* __restrict__ x, int64_t ldx, const float* __restrict__ state,
                                         const float* w, int taps, int64_t t, int i, int c, int N) {
  float acc = 0.f;
  for (int j = 0; j < taps; ++j) {
    const int back = taps - 1 - j;                       // how many tokens before t
    const float v = back <= i ? to_float(x[(t - back) * ldx + c]) : state[static_cast<int64_t>(taps - 1 - (back - i)) * N + c];
    acc += w[j] * v;
  }
  return acc;
}

template <typename X, typename W, typename O>
__global__ void causal_conv_kernel(const X* __restrict__ x, int64_t ldx, const W* __restrict__ weight, int taps,
                                   float* __restrict__ state, O* __restrict__ out, int64_t ldo, int residual,
                                   const float* __restrict__ bias, const int32_t* __restrict__ cu_q,
                                   const int32_t* __restrict__ token_request, const int32_t* __restrict__ state_slots, int N) {
  const int64_t t = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= N) return;
  const int b = token_request[t];
  const int first = cu_q[b];
  const int i = static_cast<int>(t) - first;
  const int n = cu_q[b + 1] - first;
  float* own = state + static_cast<int64_t>(state_slots[b]) * (taps - 1) * N;
  float w[MAX_TAPS];
  for (int j = 0; j < taps; ++j) w[j] = to_float(weight[static_cast<int64_t>(c) * taps + j]);
  float acc = conv_at(x, ldx, own, w, taps, t, i, c, N);
  const float self = to_float(x[t * ldx + c]);
  if (residual & 1) acc += self;
  if (bias != nullptr) acc += bias[c];
  if (residual >> 1) acc = activate(acc, (residual >> 1) - 1);       // an activation on the float32 sum
  out[t * ldo + c] = from_float<O>(acc);
  if (n == 1) {
    float keep[MAX_TAPS];
    for (int k = 1; k < taps - 1; ++k) keep[k] = own[static_cast<int64_t>(k) * N + c];
    for (int k = 1; k < taps - 1; ++k) own[static_cast<int64_t>(k - 1) * N + c] = keep[k];
    if (taps > 1) own[static_cast<int64_t>(taps - 2) * N + c] = self;
  }
}

// new state = the last taps - 1 of (old state, the step's rows), for requests that bring `skip_single ? > 1 : >= 1` rows
template <typename X>
__global__ void conv_state_kernel(const X* __restrict__ x, int64_t ldx, int taps, float* __restrict__ state,
                                  const int32_t* __restrict__ cu_q, const int32_t* __restrict__ state_slots, int N,
                                  int skip_single) {
  const int b = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= N) return;
  const int first = cu_q[b];
  const int n = cu_q[b + 1] - first;
  if (n < 1 || (n == 1 && skip_single)) return;
  float* own = state + static_cast<int64_t>(state_slots[b]) * (taps - 1) * N;
  float keep[MAX_TAPS];
  for (int k = 0; k < taps - 1; ++k) {
    const int s = n + k - (taps - 1);                    // row of the step, or behind its start
    keep[k] = s >= 0 ? to_float(x[static_cast<int64_t>(first + s) * ldx + c]) : own[static_cast<int64_t>(n + k) * N + c];
  }
  for (int k = 0; k < taps - 1; ++k) own[static_cast<int64_t>(k) * N + c] = keep[k];
}

// ---------------------------------------------------------------------------------------------------
// Behind the stacked projection of attention: product [T, ld] holds q (H heads of D), then k (G heads of D) and
// v (G heads of E) unless `has_kv` is 0. Each channel goes through its short convolution (taps 0: none); the
// first 2 * pairs dimensions of every q and k head are turned by the token's angle (pair (j, j + pairs); cosine
// and sine from `table` [T, pairs, 2], both times `magnitude`); q goes to q_out [T, H, DP] (zeros beyond D), k
// and v to the token's slot of the cache, k [pages, G, P, DP], v [pages, G, DP, P] (what lies beyond D and E there
// was zero when the cache was made and is never written).
// One block a (token, head): q heads, then k heads, then v heads. A thread owns its channels alone, so for a request
// that brings one row it also moves the convolution's state on (`conv_state_kernel` does it for the others).
template <typename X, typename W, typename Q, typename C>
__global__ void conv_rope_kv_write_kernel(const X* __restrict__ product, int64_t ld, const W* __restrict__ weight, int taps,
                                          float* __restrict__ state, const float2* __restrict__ table, int pairs,
                                          float magnitude, Q* __restrict__ q_out, C* __restrict__ k_cache,
                                          C* __restrict__ v_cache, const int32_t* __restrict__ slots,
                                          const int32_t* __restrict__ cu_q, const int32_t* __restrict__ token_request,
                                          const int32_t* __restrict__ state_slots, int H, int G, int D, int E, int DP,
                                          int block_size, int has_kv, int write, const int32_t* __restrict__ positions,
                                          float temp_coef, int temp_every, const float* __restrict__ q_norm,
                                          const float* __restrict__ k_norm, float norm_eps, int slices, int64_t stride) {
  // slices > 1 (taps 0 only): the product is partial sums that lie `stride` elements apart, added in order while read
  const int64_t t = blockIdx.x;
  const int head = blockIdx.y;
  const int N = H * D + (has_kv ? G * (D + E) : 0);
  const int b = token_request[t];
  const int first = cu_q[b];
  const int i = static_cast<int>(t) - first;
  const bool single = cu_q[b + 1] - first == 1;
  float* own = taps > 1 ? state + static_cast<int64_t>(state_slots[b]) * (taps - 1) * N : nullptr;
  const int64_t slot = (has_kv && write) ? slots[t] : 0;
  const int64_t page = slot / block_size;
  const int offset = static_cast<int>(slot % block_size);
  auto value = [&](int c) {
    float self = to_float(product[t * ld + c]);
    for (int s = 1; s < slices; ++s) self += to_float(product[s * stride + t * ld + c]);
    if (taps < 1) return self;
    float w[MAX_TAPS];
    for (int j = 0; j < taps; ++j) w[j] = to_float(weight[static_cast<int64_t>(c) * taps + j]);
    const float acc = conv_at(product, ld, own, w, taps, t, i, c, N);
    if (single && taps > 1) {
      float keep[MAX_TAPS];
      for (int k = 1; k < taps - 1; ++k) keep[k] = own[static_cast<int64_t>(k) * N + c];
      for (int k = 1; k < taps - 1; ++k) own[static_cast<int64_t>(k - 1) * N + c] = keep[k];
      own[static_cast<int64_t>(taps - 2) * N + c] = self;
    }
    return acc;
  };
  if (head >= H + G) {                                   // a v head
    if (!write) {
      if (single && taps > 1)
        for (int e = threadIdx.x; e < E; e += blockDim.x) (void)value((H + G) * D + (head - H - G) * E + e);
      return;
    }
    for (int e = threadIdx.x; e < E; e += blockDim.x) {
      const float v = value((H + G) * D + (head - H - G) * E + e);
      v_cache[((page * G + (head - H - G)) * DP + e) * block_size + offset] = from_float<C>(to_float(from_float<Q>(v)));
    }
    return;
  }
  // q and k: a thread owns a pair, or a single dimension beyond the turned ones (the launcher gives a block at least
  // DP - pairs threads, so a thread has one item and the whole head is in the block at once)
  const int base = head * D;                             // q heads, then k heads: both D wide, one after the other
  const int j = threadIdx.x;
  float x0 = 0.f, x1 = 0.f;
  int d0 = -1, d1 = -1;
  if (j < DP - pairs) {
    if (j < pairs) {
      d0 = j;
      d1 = j + pairs;
      x0 = value(base + d0);
      x1 = value(base + d1);
    } else {
      d0 = j + pairs;
      if (d0 < D) x0 = value(base + d0);
    }
  }
  const float* norm_weight = head < H ? q_norm : k_norm;
  if (norm_weight != nullptr) {
    // the norm over the head's D values, in float32, in front of the rotation
    __shared__ float scratch[16];
    const float r = 1.f / sqrtf(block_sum(x0 * x0 + x1 * x1, scratch) / D + norm_eps);
    if (d0 >= 0 && d0 < D) x0 = x0 * r * norm_weight[d0];
    if (d1 >= 0) x1 = x1 * r * norm_weight[d1];
  }
  if (d0 < 0) return;
  float a = x0, bq = 0.f;
  if (d1 >= 0) {
    const float2 e = table[t * pairs + j];
    const float cs = e.x * magnitude, sn = e.y * magnitude;
    a = x0 * cs - x1 * sn;
    bq = x1 * cs + x0 * sn;
  }
  if (head < H) {
    Q* q = q_out + (t * H + head) * DP;
    const float qt = query_temperature(positions, t, temp_coef, temp_every);
    q[d0] = from_float<Q>(a * qt);
    if (d1 >= 0) q[d1] = from_float<Q>(bq * qt);
  } else if (write && d0 < D) {
    C* k = k_cache + ((page * G + (head - H)) * block_size + offset) * DP;
    k[d0] = from_float<C>(to_float(from_float<Q>(a)));
    if (d1 >= 0) k[d1] = from_float<C>(to_float(from_float<Q>(bq)));
  }
}

// ---------------------------------------------------------------------------------------------------
// out[t, h * E + e] = x[t, h * ldh + e] * sigmoid(gates[t, ldg-row][h * E + e])
template <typename X, typename G, typename O>
__global__ void sigmoid_gate_kernel(const X* __restrict__ x, int ldh, int E, const G* __restrict__ gates, int64_t ldg,
                                    O* __restrict__ out, int width) {
  const int64_t t = blockIdx.x;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < width; c += gridDim.y * blockDim.x) {
    const int head = c / E, e = c % E;
    const float v = to_float(x[(t * (width / E) + head) * ldh + e]);
    out[t * width + c] = from_float<O>(gates != nullptr ? v * sigmoidf(to_float(gates[t * ldg + c])) : v);
  }
}

// out = x / sqrt(mean(x^2) + eps) * weight * sigmoid(gate): the norm over all heads together, then the gate.
// V channels a thread at a time (4: 16-byte loads of x, every load of a row under way before the sum).
// A row of x may be one group of a wider row (blockIdx.y: the group, `ld` columns a row, the weight shared by the
// groups); `silu`: the gate is g * sigmoid(g).
template <int V, typename W, typename G, typename O>
__global__ void rmsnorm_gate_kernel(const float* __restrict__ x, const W* __restrict__ weight, float eps,
                                    const G* __restrict__ gates, int64_t ldg, O* __restrict__ out, int N, int64_t ld,
                                    int silu) {
  __shared__ float scratch[16];
  const int64_t t = blockIdx.x;
  const float* row = x + t * ld + static_cast<int64_t>(blockIdx.y) * N;
  if (gates != nullptr) gates += static_cast<int64_t>(blockIdx.y) * N;
  out += t * (ld - N) + static_cast<int64_t>(blockIdx.y) * N;
  float sq = 0.f;
  for (int c = V * threadIdx.x; c < N; c += V * blockDim.x) {
    float v[V];
    loadv<V>(row + c, v);
#pragma unroll
    for (int k = 0; k < V; ++k) sq += v[k] * v[k];
  }
  sq = block_sum(sq, scratch);
  const float scale = 1.f / sqrtf(sq / N + eps);
  for (int c = V * threadIdx.x; c < N; c += V * blockDim.x) {
    float v[V], w[V];
    loadv<V>(row + c, v);
    loadv<V>(weight + c, w);
#pragma unroll
    for (int k = 0; k < V; ++k) v[k] *= scale * w[k];
    if (gates != nullptr) {
      float g[V];
      loadv<V>(gates + t * ldg + c, g);
#pragma unroll
      for (int k = 0; k < V; ++k) v[k] *= silu ? siluf(g[k]) : sigmoidf(g[k]);
    }
    storev<V>(out + t * N + c, v);
  }
}

// kinds: 0 relu squared, 1 silu, 2 gelu (tanh form), 3 relu
template <typename I, typename T>
__global__ void activation_kernel(const I* __restrict__ in, int slices, int64_t slice_stride, T* __restrict__ out,
                                  int64_t count, int kind) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= count) return;
  const float z = sum_strided(in + i, slices, slice_stride);
  float r;
  if (kind == 0) {
    const float p = fmaxf(z, 0.f);
    r = p * p;
  } else if (kind == 1) {
    r = siluf(z);
  } else if (kind == 2) {
    r = 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
  } else {
    r = fmaxf(z, 0.f);
  }
  out[i] = from_float<T>(r);
}

// ---------------------------------------------------------------------------------------------------
// Decayed outer-product state, token by token:  S <- decay_h S + k v^T,  o = S^T q  per head, with
// q = silu(product q), k = silu(product k), v = silu(product v); product [T, ld] holds q (H x D), k (H x D),
// v (H x E). state float32 [slots, H, D, E]. A block owns 64 columns e of one head of one request and walks the
// request's rows in order; thread (e, part) keeps rows d = part, part + PARTS, ... of its column in registers,
// the PARTS partial sums of a column meet in LDS.
template <typename X, int PARTS, int ROWS>
__global__ void __launch_bounds__(64 * PARTS)
decay_scan_kernel(const X* __restrict__ product, int64_t ld, float* __restrict__ state, const float* __restrict__ decay,
                  float* __restrict__ out, const int32_t* __restrict__ cu_q, const int32_t* __restrict__ state_slots,
                  int H, int D, int E) {
  __shared__ float q_s[PARTS * ROWS], k_s[PARTS * ROWS];
  __shared__ float partial[PARTS][64];
  const int b = blockIdx.x, head = blockIdx.y;
  const int lane = threadIdx.x % 64, part = threadIdx.x / 64;
  const int e = blockIdx.z * 64 + lane;
  const int first = cu_q[b], last = cu_q[b + 1];
  const float rate = decay[head];
  float* own = state + (static_cast<int64_t>(state_slots[b]) * H + head) * D * E;
  float s[ROWS];
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    const int d = part + r * PARTS;
    s[r] = (d < D && e < E) ? own[static_cast<int64_t>(d) * E + e] : 0.f;
  }
  for (int t = first; t < last; ++t) {
    const X* row = product + static_cast<int64_t>(t) * ld;
    __syncthreads();
    for (int d = threadIdx.x; d < D; d += blockDim.x) {
      q_s[d] = siluf(to_float(row[head * D + d]));
      k_s[d] = siluf(to_float(row[(H + head) * D + d]));
    }
    const float v = e < E ? siluf(to_float(row[2 * H * D + head * E + e])) : 0.f;
    __syncthreads();
    float o = 0.f;
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
      const int d = part + r * PARTS;
      if (d < D) {
        s[r] = rate * s[r] + k_s[d] * v;
        o += s[r] * q_s[d];
      }
    }
    partial[part][lane] = o;
    __syncthreads();
    if (part == 0 && e < E) {
      float total = 0.f;
#pragma unroll
      for (int p = 0; p < PARTS; ++p) total += partial[p][lane];
      out[(static_cast<int64_t>(t) * H + head) * E + e] = total;
    }
  }
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    const int d = part + r * PARTS;
    if (d < D && e < E) own[static_cast<int64_t>(d) * E + e] = s[r];
  }
}

// ---------------------------------------------------------------------------------------------------
// bfloat16 with 16-byte loads and stores: eight channels a thread. Values are put together as whole 32-bit words.
__device__ __forceinline__ void unpack_bf16x8(const uint4& raw, float v[8]) {
  const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    v[2 * e] = __uint_as_float(w[e] << 16);
    v[2 * e + 1] = __uint_as_float(w[e] & 0xffff0000u);
  }
}
__device__ __forceinline__ uint32_t bf16_bits(float x) {
  return static_cast<uint32_t>(__builtin_bit_cast(uint16_t, static_cast<bf16_t>(x)));
}
__device__ __forceinline__ uint4 pack_bf16x8(const float v[8]) {
  uint32_t w[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) w[e] = bf16_bits(v[2 * e]) | (bf16_bits(v[2 * e + 1]) << 16);
  return uint4{w[0], w[1], w[2], w[3]};
}
__device__ __forceinline__ uint4 load16(const bf16_t* p) { return *reinterpret_cast<const uint4*>(p); }

// the convolution at eight channels c0 .. c0 + 7 of row t (filters of `taps` taps, bfloat16, [N, taps])
__device__ __forceinline__ void conv8(const bf16_t* __restrict__ x, int64_t ldx, const float* __restrict__ state,
                                      const bf16_t* __restrict__ weight, int taps, int64_t t, int i, int c0, int N,
                                      float acc[8], float self[8]) {
  unpack_bf16x8(load16(x + t * ldx + c0), self);
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;
  if (taps < 1) {
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = self[e];
    return;
  }
  for (int j = 0; j < taps; ++j) {
    const int back = taps - 1 - j;
    float v[8];
    if (back == 0) {
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = self[e];
    } else if (back <= i) {
      unpack_bf16x8(load16(x + (t - back) * ldx + c0), v);
    } else {
      const float4* p = reinterpret_cast<const float4*>(state + static_cast<int64_t>(taps - 1 - (back - i)) * N + c0);
      const float4 lo = p[0], hi = p[1];
      v[0] = lo.x, v[1] = lo.y, v[2] = lo.z, v[3] = lo.w, v[4] = hi.x, v[5] = hi.y, v[6] = hi.z, v[7] = hi.w;
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] += to_float(weight[static_cast<int64_t>(c0 + e) * taps + j]) * v[e];
  }
}

// a request that brings one row: its state of eight channels moved on by that row
__device__ __forceinline__ void shift_state8(float* __restrict__ own, int taps, int c0, int N, const float self[8]) {
  float4 keep[MAX_TAPS][2];
  for (int k = 1; k < taps - 1; ++k) {
    const float4* p = reinterpret_cast<const float4*>(own + static_cast<int64_t>(k) * N + c0);
    keep[k][0] = p[0], keep[k][1] = p[1];
  }
  for (int k = 1; k < taps - 1; ++k) {
    float4* p = reinterpret_cast<float4*>(own + static_cast<int64_t>(k - 1) * N + c0);
    p[0] = keep[k][0], p[1] = keep[k][1];
  }
  float4* last = reinterpret_cast<float4*>(own + static_cast<int64_t>(taps - 2) * N + c0);
  last[0] = float4{self[0], self[1], self[2], self[3]};
  last[1] = float4{self[4], self[5], self[6], self[7]};
}

__global__ void causal_conv_bf16x8_kernel(const bf16_t* __restrict__ x, int64_t ldx, const bf16_t* __restrict__ weight,
                                          int taps, float* __restrict__ state, bf16_t* __restrict__ out, int64_t ldo,
                                          int residual, const float* __restrict__ bias,
                                          const int32_t* __restrict__ cu_q, const int32_t* __restrict__ token_request,
                                          const int32_t* __restrict__ state_slots, int N) {
  const int64_t t = blockIdx.x;
  const int c0 = 8 * (blockIdx.y * blockDim.x + threadIdx.x);
  if (c0 >= N) return;
  const int b = token_request[t];
  const int first = cu_q[b];
  const int i = static_cast<int>(t) - first;
  float* own = state + static_cast<int64_t>(state_slots[b]) * (taps - 1) * N;
  float acc[8], self[8];
  conv8(x, ldx, own, weight, taps, t, i, c0, N, acc, self);
  if (residual & 1) {
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] += self[e];
  }
  if (bias != nullptr) {
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] += bias[c0 + e];
  }
  if (residual >> 1) {
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = activate(acc[e], (residual >> 1) - 1);
  }
  *reinterpret_cast<uint4*>(out + t * ldo + c0) = pack_bf16x8(acc);
  if (cu_q[b + 1] - first == 1 && taps > 1) shift_state8(own, taps, c0, N, self);
}

__device__ __forceinline__ void load_f32x8(const float* __restrict__ p, float v[8]);

// The same for filters of TAPS = 2, 3 or 4 taps: the filters, the last TAPS - 1 inputs and the sums stay in registers
// (every index is known when the kernel is compiled), and a thread walks R rows of the step one after the other, so a
// row of x is read once and serves the TAPS rows that see it. Where a row is its request's first of the step, the
// inputs before it come from the request's state.
template <int TAPS, int R>
__global__ void causal_conv_bf16_taps_kernel(const bf16_t* __restrict__ x, int64_t ldx, const bf16_t* __restrict__ weight,
                                             float* __restrict__ state, bf16_t* __restrict__ out, int64_t ldo, int mode,
                                             const float* __restrict__ bias, const int32_t* __restrict__ cu_q,
                                             const int32_t* __restrict__ token_request,
                                             const int32_t* __restrict__ state_slots, int N, int T) {
  const int c0 = 8 * (blockIdx.y * blockDim.x + threadIdx.x);
  if (c0 >= N) return;
  const int t0 = blockIdx.x * R;
  float w[TAPS][8];                     // w[j][e]: tap j of channel c0 + e
  {
    float flat[8 * TAPS];
#pragma unroll
    for (int q = 0; q < TAPS; ++q) unpack_bf16x8(load16(weight + static_cast<int64_t>(c0) * TAPS + 8 * q), flat + 8 * q);
#pragma unroll
    for (int e = 0; e < 8; ++e)
#pragma unroll
      for (int j = 0; j < TAPS; ++j) w[j][e] = flat[e * TAPS + j];
  }
  float add[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) add[e] = bias != nullptr ? bias[c0 + e] : 0.f;
  float win[TAPS - 1][8];               // the inputs of the TAPS - 1 rows before this one, oldest first
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int t = t0 + r;
    if (t >= T) break;
    const int b = token_request[t];
    const int first = cu_q[b];
    const int i = t - first;
    float* own = state + static_cast<int64_t>(state_slots[b]) * (TAPS - 1) * N;
    if (r == 0 || i == 0) {
#pragma unroll
      for (int k = 0; k < TAPS - 1; ++k) {
        const int back = TAPS - 1 - k;
        if (back <= i) unpack_bf16x8(load16(x + static_cast<int64_t>(t - back) * ldx + c0), win[k]);
        else load_f32x8(own + static_cast<int64_t>(TAPS - 1 - (back - i)) * N + c0, win[k]);
      }
    }
    float self[8], acc[8];
    unpack_bf16x8(load16(x + static_cast<int64_t>(t) * ldx + c0), self);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      float sum = 0.f;
#pragma unroll
      for (int k = 0; k < TAPS - 1; ++k) sum += w[k][e] * win[k][e];
      sum += w[TAPS - 1][e] * self[e];
      if (mode & 1) sum += self[e];
      sum += add[e];
      acc[e] = (mode >> 1) ? activate(sum, (mode >> 1) - 1) : sum;
    }
    *reinterpret_cast<uint4*>(out + static_cast<int64_t>(t) * ldo + c0) = pack_bf16x8(acc);
#pragma unroll
    for (int k = 0; k + 1 < TAPS - 1; ++k)
#pragma unroll
      for (int e = 0; e < 8; ++e) win[k][e] = win[k + 1][e];
#pragma unroll
    for (int e = 0; e < 8; ++e) win[TAPS - 2][e] = self[e];
    if (i == 0 && cu_q[b + 1] - first == 1) {
      // a request that brings one row: the window, moved on by that row, is its new state
#pragma unroll
      for (int k = 0; k < TAPS - 1; ++k) {
        float4* to = reinterpret_cast<float4*>(own + static_cast<int64_t>(k) * N + c0);
        to[0] = float4{win[k][0], win[k][1], win[k][2], win[k][3]};
        to[1] = float4{win[k][4], win[k][5], win[k][6], win[k][7]};
      }
    }
  }
}

// conv_rope_kv_write for steps of 32 rows and more, bfloat16 products and caches, D, E and the number of pairs multiples of 8, DP == D or the
// places beyond D zeroed by eight. Blocks 0 .. T-1: q and k of one token (a thread turns eight pairs, or copies eight
// single dimensions). The blocks behind them: v for 16 tokens each; a thread owns one channel of v and, where
// the 16 tokens lie side by side in one page, writes their values as one run of 32 bytes (the cache keeps v with
// the key index innermost).
// NORM: every q and k head first goes through x / sqrt(mean(x^2) + norm_eps) * weight over its D values (behind the
// convolution, in front of the rotation): a first walk over the items leaves each item's sum of squares in LDS, and
// an item of the second walk adds up those of its head, in their order.
constexpr int VGROUP = 16;

// eight float32 values from a 16-byte aligned place, two loads
__device__ __forceinline__ void load_f32x8(const float* __restrict__ p, float v[8]) {
  const float4 lo = reinterpret_cast<const float4*>(p)[0], hi = reinterpret_cast<const float4*>(p)[1];
  v[0] = lo.x, v[1] = lo.y, v[2] = lo.z, v[3] = lo.w, v[4] = hi.x, v[5] = hi.y, v[6] = hi.z, v[7] = hi.w;
}

template <bool NORM>
__global__ void conv_rope_kv_write_bf16_kernel(const bf16_t* __restrict__ product, int64_t ld, const bf16_t* __restrict__ weight,
                                               int taps, float* __restrict__ state, const float2* __restrict__ table,
                                               int pairs, float magnitude, bf16_t* __restrict__ q_out,
                                               bf16_t* __restrict__ k_cache, bf16_t* __restrict__ v_cache,
                                               const int32_t* __restrict__ slots, const int32_t* __restrict__ cu_q,
                                               const int32_t* __restrict__ token_request,
                                               const int32_t* __restrict__ state_slots, int T, int H, int G, int D, int E,
                                               int DP, int block_size, int has_kv, int write,
                                               const int32_t* __restrict__ positions, float temp_coef, int temp_every,
                                               const float* __restrict__ q_norm, const float* __restrict__ k_norm,
                                               float norm_eps) {
  extern __shared__ float squares[];                     // NORM: [heads of q and k, items of a head]
  const int N = H * D + (has_kv ? G * (D + E) : 0);
  if (static_cast<int>(blockIdx.x) >= T) {
    // ---- v: 16 tokens, one channel a thread
    const int t0 = (static_cast<int>(blockIdx.x) - T) / G * VGROUP;
    const int g = (static_cast<int>(blockIdx.x) - T) % G;
    const int n = min(VGROUP, T - t0);
    const int64_t slot0 = write ? slots[t0] : 0;
    bool together = write && n == VGROUP && block_size % 8 == 0 && slot0 % block_size % 8 == 0 &&
                    slot0 % block_size + VGROUP <= block_size;
    if (write) {
#pragma unroll
      for (int k = 1; k < VGROUP; ++k) together = together && slots[min(t0 + k, T - 1)] == slot0 + k;
    }
    uint16_t* cache = reinterpret_cast<uint16_t*>(v_cache);
    for (int e = threadIdx.x; e < E; e += blockDim.x) {
      const int c = (H + G) * D + g * E + e;
      float w[MAX_TAPS];
      for (int j = 0; j < taps; ++j) w[j] = to_float(weight[static_cast<int64_t>(c) * taps + j]);
      uint32_t bits[VGROUP];
#pragma unroll
      for (int k = 0; k < VGROUP; ++k) {
        bits[k] = 0;
        if (k >= n) continue;
        const int64_t t = t0 + k;
        const int b = token_request[t];
        const int first = cu_q[b];
        const int i = static_cast<int>(t) - first;
        float* own = taps > 1 ? state + static_cast<int64_t>(state_slots[b]) * (taps - 1) * N : nullptr;
        const float self = to_float(product[t * ld + c]);
        const float v = taps < 1 ? self : conv_at(product, ld, own, w, taps, t, i, c, N);
        bits[k] = bf16_bits(v);
        if (taps > 1 && cu_q[b + 1] - first == 1) {
          float keep[MAX_TAPS];
          for (int m = 1; m < taps - 1; ++m) keep[m] = own[static_cast<int64_t>(m) * N + c];
          for (int m = 1; m < taps - 1; ++m) own[static_cast<int64_t>(m - 1) * N + c] = keep[m];
          own[static_cast<int64_t>(taps - 2) * N + c] = self;
        }
      }
      if (!write) continue;
      if (together) {
        const int64_t page = slot0 / block_size;
        uint16_t* dst = cache + ((page * G + g) * DP + e) * block_size + slot0 % block_size;
        *reinterpret_cast<uint4*>(dst) = uint4{bits[0] | (bits[1] << 16), bits[2] | (bits[3] << 16),
                                               bits[4] | (bits[5] << 16), bits[6] | (bits[7] << 16)};
        *reinterpret_cast<uint4*>(dst + 8) = uint4{bits[8] | (bits[9] << 16), bits[10] | (bits[11] << 16),
                                                   bits[12] | (bits[13] << 16), bits[14] | (bits[15] << 16)};
      } else {
#pragma unroll
        for (int k = 0; k < VGROUP; ++k) {
          if (k >= n) break;
          const int64_t slot = slots[t0 + k];
          cache[((slot / block_size * G + g) * DP + e) * block_size + slot % block_size] = static_cast<uint16_t>(bits[k]);
        }
      }
    }
    return;
  }
  // ---- q and k of token t
  const int64_t t = blockIdx.x;
  const int b = token_request[t];
  const int first = cu_q[b];
  const int i = static_cast<int>(t) - first;
  const bool single = cu_q[b + 1] - first == 1 && taps > 1;
  float* own = taps > 1 ? state + static_cast<int64_t>(state_slots[b]) * (taps - 1) * N : nullptr;
  const int64_t slot = (has_kv && write) ? slots[t] : 0;
  const int64_t page = slot / block_size;
  const int offset = static_cast<int>(slot % block_size);
  const int turned = has_kv ? H + G : H;
  const float qt = query_temperature(positions, t, temp_coef, temp_every);
  const int pair8 = pairs / 8, rest8 = (DP - 2 * pairs) / 8;
  const int per_head = pair8 + rest8;
  if constexpr (NORM) {
    for (int item = threadIdx.x; item < turned * per_head; item += blockDim.x) {
      const int j8 = item % per_head;
      const int base = item / per_head * D;
      const int d0 = j8 < pair8 ? 8 * j8 : 2 * pairs + 8 * (j8 - pair8);
      float x[8] = {}, self[8], sq = 0.f;
      if (d0 < D) conv8(product, ld, own, weight, taps, t, i, base + d0, N, x, self);
#pragma unroll
      for (int e = 0; e < 8; ++e) sq += x[e] * x[e];
      if (j8 < pair8) {
        conv8(product, ld, own, weight, taps, t, i, base + d0 + pairs, N, x, self);
#pragma unroll
        for (int e = 0; e < 8; ++e) sq += x[e] * x[e];
      }
      squares[item] = sq;
    }
    __syncthreads();
  }
  for (int item = threadIdx.x; item < turned * per_head; item += blockDim.x) {
    const int head = item / per_head;
    const int j8 = item % per_head;
    const int base = head * D;
    bf16_t* dst = head < H ? q_out + (t * H + head) * DP
                           : k_cache + ((page * G + (head - H)) * block_size + offset) * DP;
    const bool store = head < H || write;
    const float* norm_weight = nullptr;
    float r = 1.f;
    if constexpr (NORM) {
      norm_weight = head < H ? q_norm : k_norm;
      if (norm_weight != nullptr) {
        float total = 0.f;
        for (int k = 0; k < per_head; ++k) total += squares[head * per_head + k];
        r = 1.f / sqrtf(total / D + norm_eps);
      }
    }
    if (j8 < pair8) {
      const int d0 = 8 * j8, d1 = d0 + pairs;
      float x0[8], x1[8], s0[8], s1[8], a[8], c[8];
      conv8(product, ld, own, weight, taps, t, i, base + d0, N, x0, s0);
      conv8(product, ld, own, weight, taps, t, i, base + d1, N, x1, s1);
      if (norm_weight != nullptr) {
        float w0[8], w1[8];
        load_f32x8(norm_weight + d0, w0);
        load_f32x8(norm_weight + d1, w1);
#pragma unroll
        for (int e = 0; e < 8; ++e) x0[e] *= r * w0[e], x1[e] *= r * w1[e];
      }
      const float4* angles = reinterpret_cast<const float4*>(table + t * pairs + d0);       // (cos, sin) x 8
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float4 cs = angles[e];
        a[2 * e] = x0[2 * e] * (cs.x * magnitude) - x1[2 * e] * (cs.y * magnitude);
        c[2 * e] = x1[2 * e] * (cs.x * magnitude) + x0[2 * e] * (cs.y * magnitude);
        a[2 * e + 1] = x0[2 * e + 1] * (cs.z * magnitude) - x1[2 * e + 1] * (cs.w * magnitude);
        c[2 * e + 1] = x1[2 * e + 1] * (cs.z * magnitude) + x0[2 * e + 1] * (cs.w * magnitude);
      }
      if (head < H) {
#pragma unroll
        for (int e = 0; e < 8; ++e) a[e] *= qt, c[e] *= qt;
      }
      if (store) {
        *reinterpret_cast<uint4*>(dst + d0) = pack_bf16x8(a);
        *reinterpret_cast<uint4*>(dst + d1) = pack_bf16x8(c);
      }
      if (single) {
        shift_state8(own, taps, base + d0, N, s0);
        shift_state8(own, taps, base + d1, N, s1);
      }
    } else {
      const int d0 = 2 * pairs + 8 * (j8 - pair8);
      float a[8] = {}, s0[8];
      if (d0 < D) {
        conv8(product, ld, own, weight, taps, t, i, base + d0, N, a, s0);
        if (single) shift_state8(own, taps, base + d0, N, s0);
        if (norm_weight != nullptr) {
          float w0[8];
          load_f32x8(norm_weight + d0, w0);
#pragma unroll
          for (int e = 0; e < 8; ++e) a[e] *= r * w0[e];
        }
      }
      if (head < H) {
#pragma unroll
        for (int e = 0; e < 8; ++e) a[e] *= qt;
      }
      if (head < H || (write && d0 < D)) *reinterpret_cast<uint4*>(dst + d0) = pack_bf16x8(a);
    }
  }
}

// The same work for steps with head norms and no filter, a run of lanes a (token, q or k head): a lane owns eight
// neighbouring dimensions (D a multiple of 8, DP at most 512), the head's sum of squares is a sum over its lanes, and a
// lane gets the other half of its pairs from the lane pairs / 8 away. One walk over the values, no barrier. The blocks from
// `qk_blocks` on write v: 16 tokens each, one channel a thread, as above.
__global__ void __launch_bounds__(256)
head_norm_rope_kv_write_bf16_kernel(const bf16_t* __restrict__ product, int64_t ld, const float2* __restrict__ table,
                                    int pairs, float magnitude, bf16_t* __restrict__ q_out, bf16_t* __restrict__ k_cache,
                                    bf16_t* __restrict__ v_cache, const int32_t* __restrict__ slots, int T, int H, int G,
                                    int D, int E, int DP, int block_size, int has_kv, int write,
                                    const int32_t* __restrict__ positions, float temp_coef, int temp_every,
                                    const float* __restrict__ q_norm, const float* __restrict__ k_norm, float norm_eps,
                                    int qk_blocks, int lanes) {
  if (static_cast<int>(blockIdx.x) >= qk_blocks) {
    const int t0 = (static_cast<int>(blockIdx.x) - qk_blocks) / G * VGROUP;
    const int g = (static_cast<int>(blockIdx.x) - qk_blocks) % G;
    const int n = min(VGROUP, T - t0);
    const int64_t slot0 = slots[t0];
    bool together = n == VGROUP && block_size % 8 == 0 && slot0 % block_size % 8 == 0 &&
                    slot0 % block_size + VGROUP <= block_size;
#pragma unroll
    for (int k = 1; k < VGROUP; ++k) together = together && slots[min(t0 + k, T - 1)] == slot0 + k;
    const uint16_t* rows = reinterpret_cast<const uint16_t*>(product);
    uint16_t* cache = reinterpret_cast<uint16_t*>(v_cache);
    for (int e = threadIdx.x; e < E; e += blockDim.x) {
      const int c = (H + G) * D + g * E + e;
      uint32_t bits[VGROUP];
#pragma unroll
      for (int k = 0; k < VGROUP; ++k) bits[k] = k < n ? rows[static_cast<int64_t>(t0 + k) * ld + c] : 0u;
      if (together) {
        uint16_t* dst = cache + ((slot0 / block_size * G + g) * DP + e) * block_size + slot0 % block_size;
        *reinterpret_cast<uint4*>(dst) = uint4{bits[0] | (bits[1] << 16), bits[2] | (bits[3] << 16),
                                               bits[4] | (bits[5] << 16), bits[6] | (bits[7] << 16)};
        *reinterpret_cast<uint4*>(dst + 8) = uint4{bits[8] | (bits[9] << 16), bits[10] | (bits[11] << 16),
                                                   bits[12] | (bits[13] << 16), bits[14] | (bits[15] << 16)};
      } else {
#pragma unroll
        for (int k = 0; k < VGROUP; ++k) {
          if (k >= n) break;
          const int64_t slot = slots[t0 + k];
          cache[((slot / block_size * G + g) * DP + e) * block_size + slot % block_size] = static_cast<uint16_t>(bits[k]);
        }
      }
    }
    return;
  }
  // `lanes` (a power of two, DP / 8 rounded up) lanes a head, 64 / lanes heads a wave
  const int turned = has_kv ? H + G : H;
  const int lane = threadIdx.x % 64 % lanes;
  const int64_t unit = (static_cast<int64_t>(blockIdx.x) * 4 + threadIdx.x / 64) * (64 / lanes) + threadIdx.x % 64 / lanes;
  const int64_t t = min(unit, static_cast<int64_t>(T) * turned - 1) / turned;
  const int head = static_cast<int>(min(unit, static_cast<int64_t>(T) * turned - 1) % turned);
  const bool valid = unit < static_cast<int64_t>(T) * turned && (head < H || write);      // the others only take part in the shuffles
  const int d0 = 8 * lane;
  float x[8] = {};
  if (valid && d0 < D) unpack_bf16x8(load16(product + t * ld + head * D + d0), x);
  const float* norm_weight = head < H ? q_norm : k_norm;
  float sq = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) sq += x[e] * x[e];
  for (int o = lanes / 2; o > 0; o >>= 1) sq += __shfl_xor(sq, o, 64);       // every lane of the wave, whatever its head
  if (norm_weight != nullptr) {
    const float r = 1.f / sqrtf(sq / D + norm_eps);
    if (d0 < D) {
      float w[8];
      load_f32x8(norm_weight + d0, w);
#pragma unroll
      for (int e = 0; e < 8; ++e) x[e] *= r * w[e];
    }
  }
  const int shift = pairs / 8;                           // lanes [0, shift) hold the first halves, [shift, 2 shift) the second
  const int partner = threadIdx.x % 64 - lane + (lane < shift ? lane + shift : (lane < 2 * shift ? lane - shift : lane));
  float other[8], out[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) other[e] = __shfl(x[e], partner, 64);
  if (!valid) return;
  if (lane < 2 * shift) {
    const bool first = lane < shift;
    const float4* angles = reinterpret_cast<const float4*>(table + t * pairs + 8 * (first ? lane : lane - shift));
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float4 cs = angles[e];
      const float c0 = cs.x * magnitude, s0 = cs.y * magnitude, c1 = cs.z * magnitude, s1 = cs.w * magnitude;
      // (u, v) -> (u cos - v sin, v cos + u sin): the first half holds u, the second v
      out[2 * e] = first ? x[2 * e] * c0 - other[2 * e] * s0 : x[2 * e] * c0 + other[2 * e] * s0;
      out[2 * e + 1] = first ? x[2 * e + 1] * c1 - other[2 * e + 1] * s1 : x[2 * e + 1] * c1 + other[2 * e + 1] * s1;
    }
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) out[e] = x[e];
  }
  if (head < H) {
    if (d0 >= DP) return;
    const float qt = query_temperature(positions, t, temp_coef, temp_every);
#pragma unroll
    for (int e = 0; e < 8; ++e) out[e] *= qt;
    *reinterpret_cast<uint4*>(q_out + (t * H + head) * DP + d0) = pack_bf16x8(out);
  } else if (d0 < D) {
    const int64_t slot = slots[t];
    bf16_t* dst = k_cache + ((slot / block_size * G + (head - H)) * block_size + slot % block_size) * DP;
    *reinterpret_cast<uint4*>(dst + d0) = pack_bf16x8(out);
  }
}

// out = x * sigmoid(gates), eight a thread
__global__ void sigmoid_gate_bf16x8_kernel(const bf16_t* __restrict__ x, int ldh, int E, const bf16_t* __restrict__ gates,
                                           int64_t ldg, bf16_t* __restrict__ out, int width, int64_t T) {
  const int width8 = width / 8;
  const int64_t total = T * width8;
  for (int64_t it = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; it < total;
       it += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int64_t t = it / width8;
    const int c = 8 * static_cast<int>(it % width8);
    const int head = c / E, e = c % E;
    float v[8], g[8];
    unpack_bf16x8(load16(x + (t * (width / E) + head) * ldh + e), v);
    unpack_bf16x8(load16(gates + t * ldg + c), g);
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] *= sigmoidf(g[k]);
    *reinterpret_cast<uint4*>(out + t * width + c) = pack_bf16x8(v);
  }
}

__global__ void activation_bf16x8_kernel(const uint4* __restrict__ in, uint4* __restrict__ out, int64_t count8, int kind) {
  for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < count8;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    float v[8];
    unpack_bf16x8(in[i], v);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const float z = v[k];
      if (kind == 0) {
        const float p = fmaxf(z, 0.f);
        v[k] = p * p;
      } else if (kind == 1) {
        v[k] = siluf(z);
      } else if (kind == 2) {
        v[k] = 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
      } else {
        v[k] = fmaxf(z, 0.f);
      }
    }
    out[i] = pack_bf16x8(v);
  }
}

// ---------------------------------------------------------------------------------------------------
// The same recurrence over portions of prompts, in chunks of 64 rows that run side by side. With L the rows of a
// chunk, S the state in front of it and w^m the decay's powers (a table made by repeated multiplication):
//   sums:     P[d][e]   = sum_j w^(L-1-j) k_j[d] v_j[e]                      (each chunk alone)
//   states:   S_next    = w^L S + P, chunk after chunk; S (the state in front) takes P's place in the scratch
//   outputs:  o_i[e]    = w^(i+1) sum_d q_i[d] S[d][e] + sum_{j<=i} w^(i-j) (q_i . k_j) v_j[e]
// Only non-negative powers occur, so nothing grows with the chunk's length. Float32 throughout, FMAs on tiles
// held in LDS; a chunk's table entry is {request, first row, rows, unused}.
constexpr int SCAN_L = 64;
constexpr int SCAN_PAD = 68;      // row stride of the transposed tiles: keeps 16-byte reads aligned
constexpr int SCAN_BATCH = 8;     // loads a thread has under way while it fills a tile

__device__ __forceinline__ void decay_powers(float* pw, float rate, int count) {
  if (threadIdx.x == 0) {
    float p = 1.f;
    for (int m = 0; m < count; ++m) {
      pw[m] = p;
      p *= rate;
    }
  }
}

template <typename X>
__global__ void __launch_bounds__(256)
scan_chunk_sums_kernel(const X* __restrict__ product, int64_t ld, const float* __restrict__ decay, float* __restrict__ scratch,
                       const int4* __restrict__ chunks, int H, int D, int E) {
  extern __shared__ float lds[];
  float* Ks = lds;                       // [64][D], each row times its power of the decay
  float* Vs = Ks + SCAN_L * D;           // [64][64]
  float* pw = Vs + SCAN_L * 64;          // [65]
  const int c = blockIdx.x, head = blockIdx.y, e0 = blockIdx.z * 64;
  const int4 chunk = chunks[c];
  const int64_t row0 = chunk.y;
  const int len = chunk.z;
  decay_powers(pw, decay[head], SCAN_L + 1);
  __syncthreads();
  // Tiles are filled row by row: lane = column, four rows a pass of the block, eight passes' loads under way at a
  // time (a load that waits for the one before it costs a trip to memory each; no division by D in the loop).
  const int col = threadIdx.x % 64, sub = threadIdx.x / 64;
  for (int j0 = sub; j0 < SCAN_L; j0 += 4 * SCAN_BATCH) {
    for (int d = col; d < D; d += 64) {
      float k[SCAN_BATCH];
#pragma unroll
      for (int u = 0; u < SCAN_BATCH; ++u) {
        const int j = j0 + 4 * u;
        k[u] = j < len ? to_float(product[(row0 + j) * ld + (H + head) * D + d]) : 0.f;
      }
#pragma unroll
      for (int u = 0; u < SCAN_BATCH; ++u) {
        const int j = j0 + 4 * u;
        Ks[j * D + d] = j < len ? pw[len - 1 - j] * siluf(k[u]) : 0.f;
      }
    }
    float v[SCAN_BATCH];
#pragma unroll
    for (int u = 0; u < SCAN_BATCH; ++u) {
      const int j = j0 + 4 * u;
      v[u] = (j < len && e0 + col < E) ? to_float(product[(row0 + j) * ld + 2 * H * D + head * E + e0 + col]) : 0.f;
    }
#pragma unroll
    for (int u = 0; u < SCAN_BATCH; ++u) Vs[(j0 + 4 * u) * 64 + col] = siluf(v[u]);
  }
  __syncthreads();
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
  float acc[2][4][4] = {};
#pragma unroll 4
  for (int j = 0; j < len; ++j) {
    const float4 v4 = *reinterpret_cast<const float4*>(Vs + j * 64 + 4 * tx);
    const float v[4] = {v4.x, v4.y, v4.z, v4.w};
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const int d0 = 4 * ty + 64 * s;
      if (d0 >= D) break;
      const float4 k4 = *reinterpret_cast<const float4*>(Ks + j * D + d0);
      const float k[4] = {k4.x, k4.y, k4.z, k4.w};
#pragma unroll
      for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < 4; ++b) acc[s][a][b] += k[a] * v[b];
    }
  }
  float* dst = scratch + (static_cast<int64_t>(c) * H + head) * D * E;
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      const int d = 4 * ty + 64 * s + a;
      if (d >= D) continue;
      const int e = e0 + 4 * tx;                          // E is a multiple of 4: four columns are there or none
      if (e < E)
        *reinterpret_cast<float4*>(dst + static_cast<int64_t>(d) * E + e) =
            float4{acc[s][a][0], acc[s][a][1], acc[s][a][2], acc[s][a][3]};
    }
}

__global__ void scan_chunk_states_kernel(float* __restrict__ scratch, float* __restrict__ state, const float* __restrict__ decay,
                                         const int4* __restrict__ chunks, const int32_t* __restrict__ request_chunks,
                                         const int32_t* __restrict__ state_slots, int H, int D, int E) {
  const int b = blockIdx.x, head = blockIdx.y;
  const int idx = blockIdx.z * blockDim.x + threadIdx.x;
  if (idx >= D * E) return;
  const int c0 = request_chunks[b], c1 = request_chunks[b + 1];
  if (c0 >= c1) return;
  const float rate = decay[head];
  float full = 1.f;
  for (int m = 0; m < SCAN_L; ++m) full *= rate;
  float* own = state + (static_cast<int64_t>(state_slots[b]) * H + head) * D * E + idx;
  const int64_t stride = static_cast<int64_t>(H) * D * E;
  float* p = scratch + (static_cast<int64_t>(c0) * H + head) * D * E + idx;
  float S = *own;
  for (int c = c0; c < c1; c += 4) {
    // the sums of four chunks are asked for together; each then gives way to the state in front of its chunk
    float add[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) add[u] = c + u < c1 ? p[u * stride] : 0.f;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (c + u >= c1) break;
      const int len = chunks[c + u].z;
      float f = full;
      if (len != SCAN_L) {
        f = 1.f;
        for (int m = 0; m < len; ++m) f *= rate;
      }
      p[u * stride] = S;
      S = f * S + add[u];
    }
    p += 4 * stride;
  }
  *own = S;
}

template <typename X>
__global__ void __launch_bounds__(256)
scan_chunk_outputs_kernel(const X* __restrict__ product, int64_t ld, const float* __restrict__ decay,
                          const float* __restrict__ scratch, float* __restrict__ out, const int4* __restrict__ chunks,
                          int H, int D, int E) {
  extern __shared__ float lds[];
  float* Qt = lds;                       // [D][68]: Qt[d][i]
  float* Kt = Qt + D * SCAN_PAD;         // [D][68]; once the scores are made, the state in front of the chunk [D][64]
  float* At = Kt + D * SCAN_PAD;         // [64][68]: At[j][i] = w^(i-j) q_i . k_j for j <= i
  float* Vs = At + SCAN_L * SCAN_PAD;    // [64][64]
  float* pw = Vs + SCAN_L * 64;          // [66]
  const int c = blockIdx.x, head = blockIdx.y, e0 = blockIdx.z * 64;
  const int4 chunk = chunks[c];
  const int64_t row0 = chunk.y;
  const int len = chunk.z;
  decay_powers(pw, decay[head], SCAN_L + 2);
  const int col = threadIdx.x % 64, sub = threadIdx.x / 64;
  for (int j0 = sub; j0 < SCAN_L; j0 += 4 * SCAN_BATCH) {
    for (int d = col; d < D; d += 64) {
      float q[SCAN_BATCH], k[SCAN_BATCH];
#pragma unroll
      for (int u = 0; u < SCAN_BATCH; ++u) {
        const int j = j0 + 4 * u;
        const X* row = product + (row0 + j) * ld;
        q[u] = j < len ? to_float(row[head * D + d]) : 0.f;
        k[u] = j < len ? to_float(row[(H + head) * D + d]) : 0.f;
      }
#pragma unroll
      for (int u = 0; u < SCAN_BATCH; ++u) {
        const int j = j0 + 4 * u;
        Qt[d * SCAN_PAD + j] = siluf(q[u]);
        Kt[d * SCAN_PAD + j] = siluf(k[u]);
      }
    }
    float v[SCAN_BATCH];
#pragma unroll
    for (int u = 0; u < SCAN_BATCH; ++u) {
      const int j = j0 + 4 * u;
      v[u] = (j < len && e0 + col < E) ? to_float(product[(row0 + j) * ld + 2 * H * D + head * E + e0 + col]) : 0.f;
    }
#pragma unroll
    for (int u = 0; u < SCAN_BATCH; ++u) Vs[(j0 + 4 * u) * 64 + col] = siluf(v[u]);
  }
  __syncthreads();
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
  float s4[4][4] = {};
  if (tx <= ty) {
#pragma unroll 8
    for (int d = 0; d < D; ++d) {
      const float4 q4 = *reinterpret_cast<const float4*>(Qt + d * SCAN_PAD + 4 * ty);
      const float4 k4 = *reinterpret_cast<const float4*>(Kt + d * SCAN_PAD + 4 * tx);
      const float q[4] = {q4.x, q4.y, q4.z, q4.w}, k[4] = {k4.x, k4.y, k4.z, k4.w};
#pragma unroll
      for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < 4; ++b) s4[a][b] += q[a] * k[b];
    }
  }
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const int i = 4 * ty + a, j = 4 * tx + b;
      At[j * SCAN_PAD + i] = j <= i ? pw[i - j] * s4[a][b] : 0.f;
    }
  __syncthreads();
  float* Ss = Kt;
  const float* src = scratch + (static_cast<int64_t>(c) * H + head) * D * E;
  for (int d0 = sub; d0 < D; d0 += 4 * SCAN_BATCH) {
    float t[SCAN_BATCH];
#pragma unroll
    for (int u = 0; u < SCAN_BATCH; ++u) {
      const int d = d0 + 4 * u;
      t[u] = (d < D && e0 + col < E) ? src[static_cast<int64_t>(d) * E + e0 + col] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < SCAN_BATCH; ++u)
      if (d0 + 4 * u < D) Ss[(d0 + 4 * u) * 64 + col] = t[u];
  }
  __syncthreads();
  float o[4][4] = {}, r[4][4] = {};
#pragma unroll 8
  for (int d = 0; d < D; ++d) {
    const float4 q4 = *reinterpret_cast<const float4*>(Qt + d * SCAN_PAD + 4 * ty);
    const float4 t4 = *reinterpret_cast<const float4*>(Ss + d * 64 + 4 * tx);
    const float q[4] = {q4.x, q4.y, q4.z, q4.w}, t[4] = {t4.x, t4.y, t4.z, t4.w};
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int b = 0; b < 4; ++b) r[a][b] += q[a] * t[b];
  }
  const int reach = min(len, 4 * ty + 4);
#pragma unroll 4
  for (int j = 0; j < reach; ++j) {
    const float4 a4 = *reinterpret_cast<const float4*>(At + j * SCAN_PAD + 4 * ty);
    const float4 v4 = *reinterpret_cast<const float4*>(Vs + j * 64 + 4 * tx);
    const float w[4] = {a4.x, a4.y, a4.z, a4.w}, v[4] = {v4.x, v4.y, v4.z, v4.w};
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int b = 0; b < 4; ++b) o[a][b] += w[a] * v[b];
  }
#pragma unroll
  for (int a = 0; a < 4; ++a) {
    const int i = 4 * ty + a;
    if (i >= len) continue;
    const int e = e0 + 4 * tx;
    const float w = pw[i + 1];
    if (e < E)
      *reinterpret_cast<float4*>(out + ((row0 + i) * H + head) * E + e) =
          float4{o[a][0] + w * r[a][0], o[a][1] + w * r[a][1], o[a][2] + w * r[a][2], o[a][3] + w * r[a][3]};
  }
}

}  // namespace

extern "C" int distie_hyper_step(float* streams, int S, const float* init, const void* y, int y_dtype, int y_slices,
                                 const void* gate, int gate_dtype, int64_t gate_ld, int gate_slices, const float* mix,
                                 const float* out_w,
                                 const float* in_w, const void* norm_w, int norm_dtype, int kind, float eps, void* h,
                                 int h_dtype, int T, int C, hipStream_t stream) {
  if (T <= 0) return 0;
  if (S < 1 || S > MAX_STREAMS || C < 1 || kind < 0 || kind > 2 || y_slices < 1 || gate_slices < 1) return DISTIE_BAD_ARGUMENT;
  if (y != nullptr && (mix == nullptr || out_w == nullptr)) return DISTIE_BAD_ARGUMENT;
  if (h != nullptr && (in_w == nullptr || (kind != 0 && norm_w == nullptr))) return DISTIE_BAD_ARGUMENT;
  // 16-byte pieces where every row of every operand starts at a multiple of 16 bytes
  const bool wide = C % 8 == 0 && gate_ld % 8 == 0 && reinterpret_cast<uintptr_t>(streams) % 16 == 0 &&
                    reinterpret_cast<uintptr_t>(init) % 16 == 0 && reinterpret_cast<uintptr_t>(y) % 16 == 0 &&
                    reinterpret_cast<uintptr_t>(gate) % 16 == 0 && reinterpret_cast<uintptr_t>(norm_w) % 16 == 0 &&
                    reinterpret_cast<uintptr_t>(h) % 16 == 0;
  const int per = wide ? C / 4 : C;
  const int threads = per >= 1024 ? 1024 : (per >= 512 ? 512 : (per >= 256 ? 256 : (per >= 128 ? 128 : 64)));
  const size_t lds = h != nullptr ? static_cast<size_t>(C) * sizeof(float) : 0;
  const int64_t y_stride = static_cast<int64_t>(T) * C;
  if (y == nullptr) y_dtype = DISTIE_F32;
  if (gate == nullptr) gate_dtype = y_dtype;
  if (norm_w == nullptr) norm_dtype = DISTIE_F32;
  if (h == nullptr) h_dtype = DISTIE_F32;
  if (lds > 48 * 1024) return DISTIE_BAD_ARGUMENT;      // a row of u waits in LDS: widths up to 12,288
#define DISTIE_HYPER_V(MS, V)                                                                                          \
  DISTIE_DISPATCH(y_dtype, Y, DISTIE_DISPATCH(gate_dtype, G, DISTIE_DISPATCH(norm_dtype, W, DISTIE_DISPATCH(h_dtype, HT,  \
      hyper_step_kernel<MS, V, Y, G, W, HT><<<T, threads, lds, stream>>>(                                             \
          streams, S, init, static_cast<const Y*>(y), y_slices, y_stride, static_cast<const G*>(gate), gate_ld,       \
          gate_slices, gate_ld * T, mix, out_w, in_w, static_cast<const W*>(norm_w), kind, eps, static_cast<HT*>(h), C)))))
#define DISTIE_HYPER(MS)   \
  if (wide) {              \
    DISTIE_HYPER_V(MS, 4); \
  } else {                 \
    DISTIE_HYPER_V(MS, 1); \
  }
  if (S == 1) {
    DISTIE_HYPER(1);
  } else if (S == 2) {
    DISTIE_HYPER(2);
  } else if (S <= 4) {
    DISTIE_HYPER(4);
  } else {
    DISTIE_HYPER(8);
  }
#undef DISTIE_HYPER_V
#undef DISTIE_HYPER
  return launch_status();
}

// `residual`: bit 0: the input itself is added; the bits above it: 1 + the kind of an activation on the sum (0: none)
extern "C" int distie_causal_conv(const void* x, int x_dtype, int64_t ldx, const void* weight, int w_dtype, int taps,
                                  float* state, void* out, int out_dtype, int64_t ldo, int residual, const float* bias,
                                  const int32_t* cu_q, const int32_t* token_request, const int32_t* state_slots, int T,
                                  int N, hipStream_t stream) {
  if (T <= 0) return 0;
  if (taps < 1 || taps > MAX_TAPS || N < 1 || ldx < N || ldo < N || (taps > 1 && state == nullptr) || residual < 0 ||
      (residual >> 1) > 4)
    return DISTIE_BAD_ARGUMENT;
  if (x_dtype == DISTIE_BF16 && w_dtype == DISTIE_BF16 && out_dtype == DISTIE_BF16 && N % 8 == 0 && ldx % 8 == 0 &&
      ldo % 8 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0 && reinterpret_cast<uintptr_t>(state) % 16 == 0) {
    const int items = N / 8;
    const int threads8 = items >= 256 ? 256 : (items >= 128 ? 128 : 64);
    if (taps >= 2 && taps <= 4 && reinterpret_cast<uintptr_t>(weight) % 16 == 0) {
      const bf16_t* xb = static_cast<const bf16_t*>(x);
      const bf16_t* wb = static_cast<const bf16_t*>(weight);
      bf16_t* ob = static_cast<bf16_t*>(out);
      // few rows: a thread a row, narrow blocks, so that the chip has something to do; many: four rows a thread
      const int rows = T >= 256 ? 4 : 1;
      const int threads = T >= 256 ? threads8 : 64;
      const dim3 grid((T + rows - 1) / rows, (items + threads - 1) / threads);
#define DISTIE_CONV_TAPS(TAPS)                                                                                          \
  if (rows == 4) causal_conv_bf16_taps_kernel<TAPS, 4><<<grid, threads, 0, stream>>>(                                   \
      xb, ldx, wb, state, ob, ldo, residual, bias, cu_q, token_request, state_slots, N, T);                             \
  else causal_conv_bf16_taps_kernel<TAPS, 1><<<grid, threads, 0, stream>>>(                                             \
      xb, ldx, wb, state, ob, ldo, residual, bias, cu_q, token_request, state_slots, N, T)
      if (taps == 2) { DISTIE_CONV_TAPS(2); } else if (taps == 3) { DISTIE_CONV_TAPS(3); } else { DISTIE_CONV_TAPS(4); }
#undef DISTIE_CONV_TAPS
      return launch_status();
    }
    causal_conv_bf16x8_kernel<<<dim3(T, (items + threads8 - 1) / threads8), threads8, 0, stream>>>(
        static_cast<const bf16_t*>(x), ldx, static_cast<const bf16_t*>(weight), taps, state, static_cast<bf16_t*>(out), ldo,
        residual, bias, cu_q, token_request, state_slots, N);
    return launch_status();
  }
  const int threads = N >= 256 ? 256 : (N >= 128 ? 128 : 64);
  const dim3 grid(T, (N + threads - 1) / threads);
  DISTIE_DISPATCH(x_dtype, X, DISTIE_DISPATCH(w_dtype, W, DISTIE_DISPATCH(out_dtype, O,
      causal_conv_kernel<X, W, O><<<grid, threads, 0, stream>>>(
          static_cast<const X*>(x), ldx, static_cast<const W*>(weight), taps, state, static_cast<O*>(out), ldo, residual,
          bias, cu_q, token_request, state_slots, N))));
  return launch_status();
}

extern "C" int distie_conv_state(const void* x, int x_dtype, int64_t ldx, int taps, float* state, const int32_t* cu_q,
                                 const int32_t* state_slots, int B, int N, int skip_single, hipStream_t stream) {
  if (B <= 0 || taps <= 1) return 0;
  if (taps > MAX_TAPS || N < 1 || ldx < N || state == nullptr) return DISTIE_BAD_ARGUMENT;
  const int threads = N >= 256 ? 256 : (N >= 128 ? 128 : 64);
  const dim3 grid(B, (N + threads - 1) / threads);
  DISTIE_DISPATCH(x_dtype, X, conv_state_kernel<X><<<grid, threads, 0, stream>>>(
      static_cast<const X*>(x), ldx, taps, state, cu_q, state_slots, N, skip_single));
  return launch_status();
}

extern "C" int distie_conv_rope_kv_write(const void* product, int dtype, int64_t ld, const void* weight, int w_dtype,
                                         int taps, float* state, const void* table, int pairs, float magnitude,
                                         void* q_out, void* k_cache, void* v_cache, int cache_dtype, const int32_t* slots,
                                         const int32_t* cu_q, const int32_t* token_request, const int32_t* state_slots,
                                         int T, int H, int G, int D, int E, int DP, int block_size, int has_kv, int write,
                                         const int32_t* positions, float temp_coef, int temp_every, const float* q_norm,
                                         const float* k_norm, float norm_eps, int slices, int q_dtype, hipStream_t stream) {
  // slices > 1: `product` is float32 partial sums [slices, T, ld] (no convolution then); q_out is of `q_dtype`
  // temp_every >= 1: q of the token at position p times 1 + temp_coef * ln(floor((p + 1) / temp_every) + 1)
  // q_norm / k_norm (float32 [D], null: none): every q / k head goes through x / sqrt(mean(x^2) + norm_eps) * weight
  // over its D values, behind the convolution and in front of the rotation
  if (T <= 0) return 0;
  if ((q_norm != nullptr || k_norm != nullptr) && !(norm_eps >= 0.f)) return DISTIE_BAD_ARGUMENT;
  if (temp_every >= 1 && positions == nullptr) return DISTIE_BAD_ARGUMENT;
  if (H < 1 || G < 1 || D < 1 || E < 1 || DP < D || DP < E || block_size < 1 || pairs < 0 || 2 * pairs > D ||
      taps < 0 || taps > MAX_TAPS)
    return DISTIE_BAD_ARGUMENT;
  if ((pairs > 0 && table == nullptr) || (taps > 1 && state == nullptr) || (taps >= 1 && weight == nullptr))
    return DISTIE_BAD_ARGUMENT;
  if (has_kv && write && (k_cache == nullptr || v_cache == nullptr || slots == nullptr)) return DISTIE_BAD_ARGUMENT;
  if (slices < 1 || (slices > 1 && (dtype != DISTIE_F32 || taps >= 1)) || (q_dtype != dtype && dtype != DISTIE_F32))
    return DISTIE_BAD_ARGUMENT;
  const int64_t stride = static_cast<int64_t>(T) * ld;
  const bool normed = q_norm != nullptr || k_norm != nullptr;
  const int norm_items = (has_kv ? H + G : H) * ((DP - pairs) / 8);
  if ((!normed || (static_cast<size_t>(norm_items) * sizeof(float) <= 48 * 1024 && D % 8 == 0 && pairs % 4 == 0 &&
                   reinterpret_cast<uintptr_t>(q_norm) % 16 == 0 && reinterpret_cast<uintptr_t>(k_norm) % 16 == 0)) &&
      dtype == DISTIE_BF16 && q_dtype == DISTIE_BF16 && (weight == nullptr || w_dtype == DISTIE_BF16) && (!write || cache_dtype == DISTIE_BF16) &&
      T >= 32 && D % 8 == 0 && E % 8 == 0 && DP % 8 == 0 && pairs % 8 == 0 && ld % 8 == 0 &&
      reinterpret_cast<uintptr_t>(product) % 16 == 0 && reinterpret_cast<uintptr_t>(q_out) % 16 == 0 && reinterpret_cast<uintptr_t>(k_cache) % 16 == 0 && reinterpret_cast<uintptr_t>(v_cache) % 16 == 0 && reinterpret_cast<uintptr_t>(state) % 16 == 0 && reinterpret_cast<uintptr_t>(table) % 16 == 0) {
    const int items = (has_kv ? H + G : H) * ((DP - pairs) / 8);
    // with head norms a thread walks its items twice: as many threads as items (up to 512), so that it has one
    const int threads8 = normed && items <= 512 ? (items + 63) / 64 * 64 : (items > 128 ? 256 : (items > 64 ? 128 : 64));
    const int v_blocks = has_kv && (write || taps > 1) ? (T + VGROUP - 1) / VGROUP * G : 0;
    if (normed && taps == 0 && DP <= 512) {
      const int64_t units = static_cast<int64_t>(T) * (has_kv ? H + G : H);
      int lanes = 1;
      while (8 * lanes < DP) lanes *= 2;
      const int per_block = 4 * (64 / lanes);
      const int qk_blocks = static_cast<int>((units + per_block - 1) / per_block);
      const int v_only = has_kv && write ? (T + VGROUP - 1) / VGROUP * G : 0;
      head_norm_rope_kv_write_bf16_kernel<<<qk_blocks + v_only, 256, 0, stream>>>(
          static_cast<const bf16_t*>(product), ld, static_cast<const float2*>(table), pairs, magnitude,
          static_cast<bf16_t*>(q_out), static_cast<bf16_t*>(k_cache), static_cast<bf16_t*>(v_cache), slots, T, H, G, D, E, DP,
          block_size, has_kv, write, positions, temp_coef, temp_every, q_norm, k_norm, norm_eps, qk_blocks, lanes);
      return launch_status();
    }
#define DISTIE_CONV_ROPE_BF16(NORM, LDS)                                                                                 \
    conv_rope_kv_write_bf16_kernel<NORM><<<T + v_blocks, threads8, LDS, stream>>>(                                        \
        static_cast<const bf16_t*>(product), ld, static_cast<const bf16_t*>(weight), taps, state,                         \
        static_cast<const float2*>(table), pairs, magnitude, static_cast<bf16_t*>(q_out), static_cast<bf16_t*>(k_cache),  \
        static_cast<bf16_t*>(v_cache), slots, cu_q, token_request, state_slots, T, H, G, D, E, DP, block_size, has_kv,    \
        write, positions, temp_coef, temp_every, q_norm, k_norm, norm_eps)
    if (normed) {
      DISTIE_CONV_ROPE_BF16(true, static_cast<size_t>(norm_items) * sizeof(float));
    } else {
      DISTIE_CONV_ROPE_BF16(false, 0);
    }
#undef DISTIE_CONV_ROPE_BF16
    return launch_status();
  }
  const int work = DP - pairs > E ? DP - pairs : E;
  const int threads = work > 128 ? 256 : (work > 64 ? 128 : 64);
  const dim3 grid(T, has_kv ? H + 2 * G : H);
  if (weight == nullptr) w_dtype = dtype;
  if (q_dtype != dtype) {
    // a float32 product (partial sums or not) behind a model that computes in bfloat16: no filter, q in `q_dtype`
    if (taps >= 1) return DISTIE_BAD_ARGUMENT;
    DISTIE_DISPATCH(q_dtype, Q, DISTIE_DISPATCH(cache_dtype, C,
        conv_rope_kv_write_kernel<float, float, Q, C><<<grid, threads, 0, stream>>>(
            static_cast<const float*>(product), ld, nullptr, taps, state, static_cast<const float2*>(table),
            pairs, magnitude, static_cast<Q*>(q_out), static_cast<C*>(k_cache), static_cast<C*>(v_cache), slots, cu_q,
            token_request, state_slots, H, G, D, E, DP, block_size, has_kv, write, positions, temp_coef, temp_every,
            q_norm, k_norm, norm_eps, slices, stride)));
    return launch_status();
  }
  DISTIE_DISPATCH(dtype, X, DISTIE_DISPATCH(w_dtype, W, DISTIE_DISPATCH(cache_dtype, C,
      conv_rope_kv_write_kernel<X, W, X, C><<<grid, threads, 0, stream>>>(
          static_cast<const X*>(product), ld, static_cast<const W*>(weight), taps, state, static_cast<const float2*>(table),
          pairs, magnitude, static_cast<X*>(q_out), static_cast<C*>(k_cache), static_cast<C*>(v_cache), slots, cu_q,
          token_request, state_slots, H, G, D, E, DP, block_size, has_kv, write, positions, temp_coef, temp_every,
          q_norm, k_norm, norm_eps, slices, stride))));
  return launch_status();
}

extern "C" int distie_sigmoid_gate(const void* x, int x_dtype, int ldh, int E, const void* gates, int g_dtype, int64_t ldg,
                                   void* out, int out_dtype, int T, int width, hipStream_t stream) {
  if (T <= 0) return 0;
  if (E < 1 || width < 1 || width % E || ldh < E || (gates != nullptr && ldg < width)) return DISTIE_BAD_ARGUMENT;
  if (gates == nullptr) g_dtype = x_dtype;
  if (gates != nullptr && x_dtype == DISTIE_BF16 && g_dtype == DISTIE_BF16 && out_dtype == DISTIE_BF16 && E % 8 == 0 && ldh % 8 == 0 &&
      ldg % 8 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(gates) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0) {
    const int64_t pieces = static_cast<int64_t>(T) * (width / 8);
    const int blocks8 = static_cast<int>(pieces / 256 + 1 < 16384 ? pieces / 256 + 1 : 16384);
    sigmoid_gate_bf16x8_kernel<<<blocks8, 256, 0, stream>>>(static_cast<const bf16_t*>(x), ldh, E,
                                                            static_cast<const bf16_t*>(gates), ldg,
                                                            static_cast<bf16_t*>(out), width, T);
    return launch_status();
  }
  const int threads = width >= 256 ? 256 : (width >= 128 ? 128 : 64);
  const dim3 grid(T, (width + threads - 1) / threads);
  DISTIE_DISPATCH(x_dtype, X, DISTIE_DISPATCH(g_dtype, G, DISTIE_DISPATCH(out_dtype, O,
      sigmoid_gate_kernel<X, G, O><<<grid, threads, 0, stream>>>(
          static_cast<const X*>(x), ldh, E, static_cast<const G*>(gates), ldg, static_cast<O*>(out), width))));
  return launch_status();
}

extern "C" int distie_rmsnorm_gate(const float* x, const void* weight, int w_dtype, float eps, const void* gates,
                                   int g_dtype, int64_t ldg, void* out, int out_dtype, int T, int N, int groups, int silu,
                                   hipStream_t stream) {
  // N: columns of one norm; a row of x, of the gates and of out holds `groups` of them side by side
  if (T <= 0) return 0;
  if (N < 1 || groups < 1 || (gates != nullptr && ldg < static_cast<int64_t>(N) * groups)) return DISTIE_BAD_ARGUMENT;
  if (gates == nullptr) g_dtype = DISTIE_F32;
  const bool wide = N % 8 == 0 && ldg % 8 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 &&
                    reinterpret_cast<uintptr_t>(weight) % 16 == 0 && reinterpret_cast<uintptr_t>(gates) % 16 == 0 &&
                    reinterpret_cast<uintptr_t>(out) % 16 == 0;
  const int per = wide ? N / 4 : N;
  const int threads = per >= 1024 ? 1024 : (per >= 512 ? 512 : (per >= 256 ? 256 : (per >= 128 ? 128 : 64)));
  const dim3 grid(T, groups);
  const int64_t ld = static_cast<int64_t>(N) * groups;
#define DISTIE_NORM_GATE(V)                                                                                  \
  DISTIE_DISPATCH(w_dtype, W, DISTIE_DISPATCH(g_dtype, G, DISTIE_DISPATCH(out_dtype, O,                      \
      rmsnorm_gate_kernel<V, W, G, O><<<grid, threads, 0, stream>>>(                                         \
          x, static_cast<const W*>(weight), eps, static_cast<const G*>(gates), ldg, static_cast<O*>(out), N, ld, silu))))
  if (wide) {
    DISTIE_NORM_GATE(4);
  } else {
    DISTIE_NORM_GATE(1);
  }
#undef DISTIE_NORM_GATE
  return launch_status();
}

extern "C" int distie_activation(const void* in, int in_dtype, int slices, void* out, int dtype, int64_t count, int kind,
                                 hipStream_t stream) {
  if (count <= 0) return 0;
  if (kind < 0 || kind > 3 || slices < 1) return DISTIE_BAD_ARGUMENT;
  if (in_dtype == DISTIE_BF16 && dtype == DISTIE_BF16 && slices == 1 && count % 8 == 0 && reinterpret_cast<uintptr_t>(in) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0) {
    const int64_t pieces = count / 8;
    const int blocks8 = static_cast<int>(pieces / 256 + 1 < 16384 ? pieces / 256 + 1 : 16384);
    activation_bf16x8_kernel<<<blocks8, 256, 0, stream>>>(static_cast<const uint4*>(in), static_cast<uint4*>(out), pieces, kind);
    return launch_status();
  }
  const int threads = 256;
  const int64_t blocks = (count + threads - 1) / threads;
  if (blocks > 0x7fffffff) return DISTIE_BAD_ARGUMENT;
  DISTIE_DISPATCH(in_dtype, I, DISTIE_DISPATCH(dtype, T,
      activation_kernel<I, T><<<static_cast<unsigned>(blocks), threads, 0, stream>>>(
          static_cast<const I*>(in), slices, count, static_cast<T*>(out), count, kind)));
  return launch_status();
}

// the largest per-head key size the scan takes (rows of the state a thread keeps: PARTS x ROWS)
extern "C" int distie_decay_scan_max_dim() { return 256; }

extern "C" int distie_decay_scan(const void* product, int dtype, int64_t ld, float* state, const float* decay, float* out,
                                 const int32_t* cu_q, const int32_t* state_slots, int B, int H, int D, int E,
                                 hipStream_t stream) {
  if (B <= 0) return 0;
  if (H < 1 || D < 1 || E < 1 || D > 256 || ld < static_cast<int64_t>(H) * (2 * D + E)) return DISTIE_BAD_ARGUMENT;
  const dim3 grid(B, H, (E + 63) / 64);
#define DISTIE_SCAN(PARTS, ROWS)                                                                                     \
  DISTIE_DISPATCH(dtype, X, decay_scan_kernel<X, PARTS, ROWS><<<grid, 64 * PARTS, 0, stream>>>(                      \
      static_cast<const X*>(product), ld, state, decay, out, cu_q, state_slots, H, D, E))
  if (D <= 32) {
    DISTIE_SCAN(4, 8);
  } else if (D <= 64) {
    DISTIE_SCAN(4, 16);
  } else if (D <= 128) {
    DISTIE_SCAN(4, 32);
  } else {
    DISTIE_SCAN(8, 32);
  }
#undef DISTIE_SCAN
  return launch_status();
}

// rows of a chunk, and the largest key size the chunked scan takes (its tiles must fit the LDS)
extern "C" int distie_decay_scan_chunk_rows() { return SCAN_L; }
extern "C" int distie_decay_scan_chunked_max_dim() { return 128; }

template <typename K>
static int more_lds(K kernel, size_t lds) {
  if (lds <= 48 * 1024) return 0;
  return static_cast<int>(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                              static_cast<int>(lds)));
}

// chunks: int32 [num_chunks][4] = {request, first row, rows (1..64), 0}, the chunks of a request one after the other;
// request_chunks: int32 [B + 1], the first chunk of every request; scratch: float32 [num_chunks, H, D, E]
extern "C" int distie_decay_scan_chunked(const void* product, int dtype, int64_t ld, float* state, const float* decay,
                                         float* out, float* scratch, const int32_t* chunks, const int32_t* request_chunks,
                                         const int32_t* state_slots, int num_chunks, int B, int H, int D, int E,
                                         hipStream_t stream) {
  if (B <= 0 || num_chunks <= 0) return 0;
  if (H < 1 || D < 4 || E < 4 || D % 4 || E % 4 || D > 128 || ld < static_cast<int64_t>(H) * (2 * D + E))
    return DISTIE_BAD_ARGUMENT;
  const dim3 grid(num_chunks, H, (E + 63) / 64);
  const int4* table = reinterpret_cast<const int4*>(chunks);
  const size_t lds_sums = (static_cast<size_t>(SCAN_L) * D + SCAN_L * 64 + SCAN_L + 1) * sizeof(float);
  const size_t lds_out = (2 * static_cast<size_t>(D) * SCAN_PAD + SCAN_L * SCAN_PAD + SCAN_L * 64 + SCAN_L + 2) * sizeof(float);
  int status = 0;
  DISTIE_DISPATCH(dtype, X, {
    if ((status = more_lds(scan_chunk_sums_kernel<X>, lds_sums)) != 0) return status;
    scan_chunk_sums_kernel<X><<<grid, 256, lds_sums, stream>>>(static_cast<const X*>(product), ld, decay, scratch, table, H, D, E);
  });
  if ((status = launch_status()) != 0) return status;
  scan_chunk_states_kernel<<<dim3(B, H, (D * E + 255) / 256), 256, 0, stream>>>(scratch, state, decay, table, request_chunks,
                                                                               state_slots, H, D, E);
  if ((status = launch_status()) != 0) return status;
  DISTIE_DISPATCH(dtype, X, {
    if ((status = more_lds(scan_chunk_outputs_kernel<X>, lds_out)) != 0) return status;
    scan_chunk_outputs_kernel<X><<<grid, 256, lds_out, stream>>>(static_cast<const X*>(product), ld, decay, scratch, out, table,
                                                                H, D, E);
  });
  return launch_status();
}
