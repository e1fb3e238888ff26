// Kernels of designs that put norms behind their sub-layers, run mixers side by side, keep a state whose decay is
// computed from the token (gated linear attention, a real-gated linear recurrent unit) and route tokens to experts.
// What such designs keep in 32-bit is float32 here in either precision: norm statistics, decays with their
// sigmoids, logarithms and exponentials, the gates of a recurrence, the states and every sum into them, router
// logits and weights.
//
// A step is a flattened batch: token t belongs to request token_request[t], whose new tokens are rows
// cu_q[b] .. cu_q[b+1]-1 and whose state is row state_slots[b] of a state tensor.
#include "common.h"

namespace {

__device__ __forceinline__ float sigmoid_exact(float x) { return 1.f / (1.f + expf(-x)); }
// ln(sigmoid(x)) and ln(1 + e^x) without overflow and without cancellation
__device__ __forceinline__ float log_sigmoid(float x) { return fminf(x, 0.f) - log1pf(expf(-fabsf(x))); }
__device__ __forceinline__ float softplus(float x) { return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x))); }

__device__ __forceinline__ float activate(float z, int kind) {   // the kinds of `distie_activation`; -1: z itself
  if (kind == 0) {
    const float p = fmaxf(z, 0.f);
    return p * p;
  }
  if (kind == 1) return z / (1.f + expf(-z));
  if (kind == 2) return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
  if (kind == 3) return fmaxf(z, 0.f);
  return z;
}

// ---------------------------------------------------------------------------------------------------
// A chain of norms around the residual sum, one block a row; every stage but the first is optional:
//   y   = scale * (rms(t0) * w0 + rms(t1) * w1)      (w0 null: y = t0 as it is; t1 null: one term)
//   y   = rms(y) * post_w                            (the norm behind a sub-layer)
//   x  += y                                          (residual, float32, in place; null: y goes to y_out)
//   out = rms(x) * pre_w                             (the norm in front of the next sub-layer)
// rms(v) = v / sqrt(mean(v^2) + eps). A term may be partial sums (slices that lie `stride` apart, added in order).
// The row waits in LDS between the passes; a thread meets the same columns in every pass. `held`: the terms and the
// residual are read once, up front and together, and wait in LDS too (rows of up to NORM_HELD_MAX columns); else
// they are read again where they are needed.
constexpr int NORM_HELD_MAX = 8192;

// V values at p as floats: V = 4 takes one 16-byte (float32) or 8-byte (bfloat16) load, V = 8 two or one of 16 bytes
template <int V, typename T>
__device__ __forceinline__ void load_values(const T* __restrict__ p, float out[V]) {
  if constexpr (V == 8 && sizeof(T) == 4) {
    load_values<4>(p, out);
    load_values<4>(p + 4, out + 4);
  } else if constexpr (V == 8) {
    const uint4 v = *reinterpret_cast<const uint4*>(p);
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int k = 0; k < 4; ++k) out[2 * k] = __uint_as_float(w[k] << 16), out[2 * k + 1] = __uint_as_float(w[k] & 0xffff0000u);
  } else if constexpr (V == 4 && sizeof(T) == 4) {
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
__device__ __forceinline__ void store_values(T* __restrict__ p, const float v[V]) {
  const auto word = [](float lo, float hi) {
    return static_cast<uint32_t>(__builtin_bit_cast(uint16_t, static_cast<bf16_t>(lo))) |
           (static_cast<uint32_t>(__builtin_bit_cast(uint16_t, static_cast<bf16_t>(hi))) << 16);
  };
  if constexpr (V == 8 && sizeof(T) == 4) {
    store_values<4>(p, v);
    store_values<4>(p + 4, v + 4);
  } else if constexpr (V == 8) {
    *reinterpret_cast<uint4*>(p) = uint4{word(v[0], v[1]), word(v[2], v[3]), word(v[4], v[5]), word(v[6], v[7])};
  } else if constexpr (V == 4 && sizeof(T) == 4) {
    *reinterpret_cast<float4*>(p) = float4{v[0], v[1], v[2], v[3]};
  } else if constexpr (V == 4) {
    *reinterpret_cast<uint2*>(p) = uint2{word(v[0], v[1]), word(v[2], v[3])};
  } else {
#pragma unroll
    for (int k = 0; k < V; ++k) p[k] = from_float<T>(v[k]);
  }
}

// the sum of `slices` vectors that lie `stride` elements apart, added in order; eight slices' loads under way together
template <int V, typename T>
__device__ __forceinline__ void sum_values(const T* __restrict__ p, int slices, int64_t stride, float out[V]) {
  load_values<V>(p, out);
  for (int s = 1; s < slices; s += 8) {
    float a[8][V];
#pragma unroll
    for (int u = 0; u < 8; ++u) load_values<V>(p + min(s + u, slices - 1) * stride, a[u]);
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (s + u < slices) {
#pragma unroll
        for (int k = 0; k < V; ++k) out[k] += a[u][k];
      }
  }
}

template <int V, typename A, typename B, typename O>
__global__ void norm_chain_kernel(const A* __restrict__ t0, int slices0, int64_t stride0, const float* __restrict__ w0,
                                  const B* __restrict__ t1, int slices1, int64_t stride1, const float* __restrict__ w1,
                                  float term_eps, float scale, const float* __restrict__ post_w, float post_eps,
                                  float* __restrict__ residual, const float* __restrict__ pre_w, float pre_eps,
                                  O* __restrict__ out, float* __restrict__ y_out, int C, int held) {
  extern __shared__ float row[];
  __shared__ float scratch[16];
  const int64_t base = static_cast<int64_t>(blockIdx.x) * C;
  float* held_a = row + C;
  float* held_b = row + 2 * C;
  float* held_x = row + 3 * C;
  const int step = V * blockDim.x;
  if (held) {
    for (int c = V * threadIdx.x; c < C; c += step) {
      float a[V], b[V] = {}, x[V] = {};
      sum_values<V>(t0 + base + c, slices0, stride0, a);
      if (t1 != nullptr) sum_values<V>(t1 + base + c, slices1, stride1, b);
      if (residual != nullptr) load_values<V>(residual + base + c, x);
      store_values<V>(held_a + c, a);
      store_values<V>(held_b + c, b);
      store_values<V>(held_x + c, x);
    }
  }
  float r0 = 1.f, r1 = 1.f;
  if (w0 != nullptr) {
    float q0 = 0.f, q1 = 0.f;
    for (int c = V * threadIdx.x; c < C; c += step) {
      float a[V], b[V] = {};
      if (held) {
        load_values<V>(held_a + c, a);
        load_values<V>(held_b + c, b);
      } else {
        sum_values<V>(t0 + base + c, slices0, stride0, a);
        if (t1 != nullptr) sum_values<V>(t1 + base + c, slices1, stride1, b);
      }
#pragma unroll
      for (int k = 0; k < V; ++k) q0 += a[k] * a[k], q1 += b[k] * b[k];
    }
    r0 = 1.f / sqrtf(block_sum(q0, scratch) / C + term_eps);
    if (t1 != nullptr) r1 = 1.f / sqrtf(block_sum(q1, scratch) / C + term_eps);
  }
  float q = 0.f;
  for (int c = V * threadIdx.x; c < C; c += step) {
    float y[V];
    if (held) {
      load_values<V>(held_a + c, y);
    } else {
      sum_values<V>(t0 + base + c, slices0, stride0, y);
    }
    if (w0 != nullptr) {
      float w[V];
      load_values<V>(w0 + c, w);
#pragma unroll
      for (int k = 0; k < V; ++k) y[k] = y[k] * r0 * w[k];
      if (t1 != nullptr) {
        float b[V];
        if (held) {
          load_values<V>(held_b + c, b);
        } else {
          sum_values<V>(t1 + base + c, slices1, stride1, b);
        }
        load_values<V>(w1 + c, w);
#pragma unroll
        for (int k = 0; k < V; ++k) y[k] += b[k] * r1 * w[k];
      }
#pragma unroll
      for (int k = 0; k < V; ++k) y[k] *= scale;
    }
    store_values<V>(row + c, y);
#pragma unroll
    for (int k = 0; k < V; ++k) q += y[k] * y[k];
  }
  float rp = 1.f;
  if (post_w != nullptr) rp = 1.f / sqrtf(block_sum(q, scratch) / C + post_eps);
  float q2 = 0.f;
  for (int c = V * threadIdx.x; c < C; c += step) {
    float y[V];
    load_values<V>(row + c, y);
    if (post_w != nullptr) {
      float w[V];
      load_values<V>(post_w + c, w);
#pragma unroll
      for (int k = 0; k < V; ++k) y[k] = y[k] * rp * w[k];
    }
    if (residual != nullptr) {
      float x[V];
      if (held) {
        load_values<V>(held_x + c, x);
      } else {
        load_values<V>(residual + base + c, x);
      }
#pragma unroll
      for (int k = 0; k < V; ++k) x[k] += y[k], q2 += x[k] * x[k];
      store_values<V>(residual + base + c, x);
      store_values<V>(row + c, x);
    } else {
      store_values<V>(y_out + base + c, y);
    }
  }
  if (residual == nullptr || out == nullptr) return;
  if (pre_w == nullptr) {
    // no norm in front of the next sub-layer: it reads the new residual itself, in its own precision
    for (int c = V * threadIdx.x; c < C; c += step) {
      float x[V];
      load_values<V>(row + c, x);
      store_values<V>(out + base + c, x);
    }
    return;
  }
  const float rn = 1.f / sqrtf(block_sum(q2, scratch) / C + pre_eps);
  for (int c = V * threadIdx.x; c < C; c += step) {
    float x[V], w[V];
    load_values<V>(row + c, x);
    load_values<V>(pre_w + c, w);
#pragma unroll
    for (int k = 0; k < V; ++k) x[k] = x[k] * rn * w[k];
    store_values<V>(out + base + c, x);
  }
}

// ---------------------------------------------------------------------------------------------------
// A state that decays by a factor of its own for every key channel and token, row after row:
//   alpha = sigmoid(z)^(1 / tau);   S <- diag(alpha) S + k v^T;   o = S^T (q * q_scale)     per head
// product [T, ld] holds q (H x D), k (H x D), v (H x E); z float32 [T, H * D]; state float32 [slots, H, D, E].
// A block owns 64 columns e of one head of one request and walks the request's rows in order; thread (e, part)
// keeps rows d = part, part + PARTS, ... of its column in registers, the PARTS partial sums of a column meet in LDS.
// The next row's values are asked for before this row's are used. LOW: z is not given; it is made here from `low`
// ([T, ld_low], `rank` columns: the decay's projection through few dimensions) as z = up[h * D + d] . low + up_bias
// (up float32 [H * D, rank], rank <= GS_RANK_MAX), which saves a step of few rows two small products.
constexpr int GS_RANK_MAX = 32;

template <typename X, int PARTS, int ROWS, bool LOW>
__global__ void __launch_bounds__(64 * PARTS)
gated_decay_scan_kernel(const X* __restrict__ product, int64_t ld, const float* __restrict__ logits,
                        const X* __restrict__ low, int64_t ld_low, const float* __restrict__ up,
                        const float* __restrict__ up_bias, int rank, float* __restrict__ state,
                        float* __restrict__ out, const int32_t* __restrict__ cu_q, const int32_t* __restrict__ state_slots,
                        int H, int D, int E, float q_scale, float tau) {
  __shared__ float q_s[PARTS * ROWS], k_s[PARTS * ROWS], a_s[PARTS * ROWS];
  __shared__ float partial[PARTS][64];
  const int b = blockIdx.x, head = blockIdx.y;
  const int lane = threadIdx.x % 64, part = threadIdx.x / 64;
  const int e = blockIdx.z * 64 + lane;
  const int first = cu_q[b], last = cu_q[b + 1];
  if (first >= last) return;
  float* own = state + (static_cast<int64_t>(state_slots[b]) * H + head) * D * E;
  float s[ROWS];
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    const int d = part + r * PARTS;
    s[r] = (d < D && e < E) ? own[static_cast<int64_t>(d) * E + e] : 0.f;
  }
  const int d_own = threadIdx.x;                      // the channel whose q, k and decay this thread fetches
  float nq = 0.f, nk = 0.f, nz = 0.f, nv = 0.f;
  float up_row[LOW ? GS_RANK_MAX : 1], nl[LOW ? GS_RANK_MAX : 1];
  float bias = 0.f;
  if constexpr (LOW) {
    if (d_own < D) {
      bias = up_bias[head * D + d_own];
#pragma unroll
      for (int r = 0; r < GS_RANK_MAX; ++r) up_row[r] = r < rank ? up[static_cast<int64_t>(head * D + d_own) * rank + r] : 0.f;
    }
  }
  auto fetch = [&](int t) {
    const X* row = product + static_cast<int64_t>(t) * ld;
    if (d_own < D) {
      nq = to_float(row[head * D + d_own]);
      nk = to_float(row[(H + head) * D + d_own]);
      if constexpr (LOW) {
#pragma unroll
        for (int r = 0; r < GS_RANK_MAX; ++r) nl[r] = r < rank ? to_float(low[static_cast<int64_t>(t) * ld_low + r]) : 0.f;
      } else {
        nz = logits[(static_cast<int64_t>(t) * H + head) * D + d_own];
      }
    }
    nv = e < E ? to_float(row[2 * H * D + head * E + e]) : 0.f;
  };
  fetch(first);
  for (int t = first; t < last; ++t) {
    __syncthreads();
    if (d_own < D) {
      if constexpr (LOW) {
        nz = 0.f;
#pragma unroll
        for (int r = 0; r < GS_RANK_MAX; ++r) nz += up_row[r] * nl[r];
        nz += bias;
      }
      q_s[d_own] = nq * q_scale;
      k_s[d_own] = nk;
      a_s[d_own] = expf(log_sigmoid(nz) / tau);
    }
    const float v = nv;
    if (t + 1 < last) fetch(t + 1);
    __syncthreads();
    float o = 0.f;
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
      const int d = part + r * PARTS;
      if (d < D) {
        s[r] = a_s[d] * s[r] + k_s[d] * v;
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
// The same recurrence over portions of prompts, in chunks of 64 rows that run side by side. With L the rows of a
// chunk, S the state in front of it and c_i[d] = sum_{m <= i} ln alpha_m[d] (the chunk's own running sum, <= 0):
//   sums:     P[d][e] = sum_j exp(c_L[d] - c_j[d]) k_j[d] v_j[e],   G[d] = exp(c_L[d])           (each chunk alone)
//   states:   S_next = diag(G) S + P, chunk after chunk; S (the state in front) takes P's place in the scratch
//   outputs:  o_i[e] = sum_d q_i[d] exp(c_i[d]) S[d][e] + sum_{j <= i} (sum_d q_i[d] k_j[d] exp(c_i[d] - c_j[d])) v_j[e]
// Every exponent is <= 0: nothing grows, however fast a channel forgets, and no quotient of decays is ever formed
// (the decay differs from channel to channel, so the scores of a pair of rows are summed channel by channel with the
// pair's own factor). Float32 throughout, FMAs on tiles held in LDS; a chunk's table entry is {request, first row,
// rows, unused}.
constexpr int GS_L = 64;
constexpr int GS_PAD = 68;        // row stride of the transposed tiles: keeps 16-byte reads aligned

// ln alpha of the chunk's rows into `c` (laid out [d][GS_PAD], rows beyond the chunk 0), then the running sums down
// the rows, one thread a channel
__device__ __forceinline__ void decay_prefix(float* __restrict__ c, const float* __restrict__ logits, int64_t row0, int len,
                                             int head, int H, int D, float tau) {
  for (int idx = threadIdx.x; idx < GS_L * D; idx += blockDim.x) {
    const int j = idx / D, d = idx % D;
    c[d * GS_PAD + j] = j < len ? log_sigmoid(logits[((row0 + j) * H + head) * D + d]) / tau : 0.f;
  }
  __syncthreads();
  for (int d = threadIdx.x; d < D; d += blockDim.x) {
    float run = 0.f;
    for (int j = 0; j < GS_L; ++j) {
      run += c[d * GS_PAD + j];
      c[d * GS_PAD + j] = run;
    }
  }
  __syncthreads();
}

template <typename X>
__global__ void __launch_bounds__(256)
gated_chunk_sums_kernel(const X* __restrict__ product, int64_t ld, const float* __restrict__ logits, float tau,
                        float* __restrict__ scratch, float* __restrict__ totals, const int4* __restrict__ chunks, int H,
                        int D, int E) {
  extern __shared__ float lds[];
  float* Ct = lds;                        // [D][68]
  float* Ks = Ct + D * GS_PAD;            // [64][D]: k_j[d] exp(c_L[d] - c_j[d])
  float* Vs = Ks + GS_L * D;              // [64][64]
  const int c = blockIdx.x, head = blockIdx.y, e0 = blockIdx.z * 64;
  const int4 chunk = chunks[c];
  const int64_t row0 = chunk.y;
  const int len = chunk.z;
  decay_prefix(Ct, logits, row0, len, head, H, D, tau);
  for (int idx = threadIdx.x; idx < GS_L * D; idx += blockDim.x) {
    const int j = idx / D, d = idx % D;
    const float k = j < len ? to_float(product[(row0 + j) * ld + (H + head) * D + d]) : 0.f;
    Ks[j * D + d] = k * expf(Ct[d * GS_PAD + GS_L - 1] - Ct[d * GS_PAD + j]);
  }
  for (int idx = threadIdx.x; idx < GS_L * 64; idx += blockDim.x) {
    const int j = idx / 64, col = idx % 64;
    Vs[idx] = (j < len && e0 + col < E) ? to_float(product[(row0 + j) * ld + 2 * H * D + head * E + e0 + col]) : 0.f;
  }
  if (blockIdx.z == 0)
    for (int d = threadIdx.x; d < D; d += blockDim.x)
      totals[(static_cast<int64_t>(c) * H + head) * D + d] = expf(Ct[d * GS_PAD + GS_L - 1]);
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

__global__ void gated_chunk_states_kernel(float* __restrict__ scratch, const float* __restrict__ totals,
                                          float* __restrict__ state, const int32_t* __restrict__ request_chunks,
                                          const int32_t* __restrict__ state_slots, int H, int D, int E) {
  const int b = blockIdx.x, head = blockIdx.y;
  const int idx = blockIdx.z * blockDim.x + threadIdx.x;
  if (idx >= D * E) return;
  const int c0 = request_chunks[b], c1 = request_chunks[b + 1];
  if (c0 >= c1) return;
  const int d = idx / E;
  float* own = state + (static_cast<int64_t>(state_slots[b]) * H + head) * D * E + idx;
  const int64_t stride = static_cast<int64_t>(H) * D * E;
  float* p = scratch + (static_cast<int64_t>(c0) * H + head) * D * E + idx;
  const float* g = totals + (static_cast<int64_t>(c0) * H + head) * D + d;
  float S = *own;
  for (int c = c0; c < c1; c += 4) {
    // the sums of four chunks are asked for together; each then gives way to the state in front of its chunk
    float add[4], keep[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      add[u] = c + u < c1 ? p[u * stride] : 0.f;
      keep[u] = c + u < c1 ? g[static_cast<int64_t>(u) * H * D] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (c + u >= c1) break;
      p[u * stride] = S;
      S = keep[u] * S + add[u];
    }
    p += 4 * stride;
    g += 4 * static_cast<int64_t>(H) * D;
  }
  *own = S;
}

template <typename X>
__global__ void __launch_bounds__(256)
gated_chunk_outputs_kernel(const X* __restrict__ product, int64_t ld, const float* __restrict__ logits, float tau,
                           float q_scale, const float* __restrict__ scratch, float* __restrict__ out,
                           const int4* __restrict__ chunks, int H, int D, int E) {
  extern __shared__ float lds[];
  float* Ct = lds;                        // [D][68]: Ct[d][i] = c_i[d]
  float* Qt = Ct + D * GS_PAD;            // [D][68]: q_i[d] * q_scale; behind the scores, times exp(c_i[d])
  float* Kt = Qt + D * GS_PAD;            // [D][68]; behind the scores, the state in front of the chunk [D][64]
  float* At = Kt + D * GS_PAD;            // [64][68]: At[j][i] = sum_d q_i[d] k_j[d] exp(c_i[d] - c_j[d]) for j <= i
  float* Vs = At + GS_L * GS_PAD;         // [64][64]
  const int c = blockIdx.x, head = blockIdx.y, e0 = blockIdx.z * 64;
  const int4 chunk = chunks[c];
  const int64_t row0 = chunk.y;
  const int len = chunk.z;
  decay_prefix(Ct, logits, row0, len, head, H, D, tau);
  for (int idx = threadIdx.x; idx < GS_L * D; idx += blockDim.x) {
    const int j = idx / D, d = idx % D;
    const X* row = product + (row0 + j) * ld;
    Qt[d * GS_PAD + j] = j < len ? to_float(row[head * D + d]) * q_scale : 0.f;
    Kt[d * GS_PAD + j] = j < len ? to_float(row[(H + head) * D + d]) : 0.f;
  }
  for (int idx = threadIdx.x; idx < GS_L * 64; idx += blockDim.x) {
    const int j = idx / 64, col = idx % 64;
    Vs[idx] = (j < len && e0 + col < E) ? to_float(product[(row0 + j) * ld + 2 * H * D + head * E + e0 + col]) : 0.f;
  }
  __syncthreads();
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
  float s4[4][4] = {};
  if (tx <= ty) {
#pragma unroll 2
    for (int d = 0; d < D; ++d) {
      const float4 q4 = *reinterpret_cast<const float4*>(Qt + d * GS_PAD + 4 * ty);
      const float4 k4 = *reinterpret_cast<const float4*>(Kt + d * GS_PAD + 4 * tx);
      const float4 i4 = *reinterpret_cast<const float4*>(Ct + d * GS_PAD + 4 * ty);
      const float4 j4 = *reinterpret_cast<const float4*>(Ct + d * GS_PAD + 4 * tx);
      const float q[4] = {q4.x, q4.y, q4.z, q4.w}, k[4] = {k4.x, k4.y, k4.z, k4.w};
      const float ci[4] = {i4.x, i4.y, i4.z, i4.w}, cj[4] = {j4.x, j4.y, j4.z, j4.w};
#pragma unroll
      for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          // (bfloat16 steps take the hardware's exponent: their q and k carry eight bits)
          const float x = fminf(ci[a] - cj[b], 0.f);
          s4[a][b] += q[a] * k[b] * (sizeof(X) == 2 ? __expf(x) : expf(x));
        }
    }
  }
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const int i = 4 * ty + a, j = 4 * tx + b;
      At[j * GS_PAD + i] = j <= i ? s4[a][b] : 0.f;
    }
  __syncthreads();
  float* Ss = Kt;
  const float* src = scratch + (static_cast<int64_t>(c) * H + head) * D * E;
  for (int idx = threadIdx.x; idx < D * 64; idx += blockDim.x) {
    const int d = idx / 64, col = idx % 64;
    Ss[idx] = e0 + col < E ? src[static_cast<int64_t>(d) * E + e0 + col] : 0.f;
  }
  for (int idx = threadIdx.x; idx < GS_L * D; idx += blockDim.x) {
    const int j = idx % GS_L, d = idx / GS_L;
    Qt[d * GS_PAD + j] *= expf(Ct[d * GS_PAD + j]);
  }
  __syncthreads();
  float o[4][4] = {};
#pragma unroll 8
  for (int d = 0; d < D; ++d) {
    const float4 q4 = *reinterpret_cast<const float4*>(Qt + d * GS_PAD + 4 * ty);
    const float4 t4 = *reinterpret_cast<const float4*>(Ss + d * 64 + 4 * tx);
    const float q[4] = {q4.x, q4.y, q4.z, q4.w}, t[4] = {t4.x, t4.y, t4.z, t4.w};
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int b = 0; b < 4; ++b) o[a][b] += q[a] * t[b];
  }
  const int reach = min(len, 4 * ty + 4);
#pragma unroll 4
  for (int j = 0; j < reach; ++j) {
    const float4 a4 = *reinterpret_cast<const float4*>(At + j * GS_PAD + 4 * ty);
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
    if (e < E)
      *reinterpret_cast<float4*>(out + ((row0 + i) * H + head) * E + e) = float4{o[a][0], o[a][1], o[a][2], o[a][3]};
  }
}

// ---------------------------------------------------------------------------------------------------
// The gates of a real-gated linear recurrent unit. u [T, ldu] holds R channels in B parts of n; in part b
//   r = sigmoid(ra[b] u_b + ra_b[b]),  i = sigmoid(ri[b] u_b + ri_b[b])          (ra[b], ri[b]: [n, n], [out, in])
//   a = exp(-rate * r * softplus(lam)),  x = sqrt(1 - a^2) * i * u     -> a_out, x_out float32 [T, R]
// A block owns 32 tokens x 64 output channels of one part, both gates at once; tiles of 32 inputs through LDS,
// float32 sums. 1 - a^2 is taken as -expm1(2 ln a), which keeps its digits where a is close to one.
constexpr int LG_TOKENS = 32, LG_OUT = 64, LG_K = 32;

template <typename X, typename W>
__global__ void __launch_bounds__(256)
lru_gates_kernel(const X* __restrict__ u, int64_t ldu, const W* __restrict__ ra, const float* __restrict__ ra_b,
                 const W* __restrict__ ri, const float* __restrict__ ri_b, const float* __restrict__ lam, float rate,
                 float* __restrict__ a_out, float* __restrict__ x_out, int T, int R, int n) {
  __shared__ float Us[LG_TOKENS][LG_K];
  __shared__ float Wa[LG_OUT][LG_K + 1], Wi[LG_OUT][LG_K + 1];
  const int t0 = blockIdx.x * LG_TOKENS, part = blockIdx.y, o0 = blockIdx.z * LG_OUT;
  const int tx = threadIdx.x % 64, ty = threadIdx.x / 64;
  const W* wa = ra + static_cast<int64_t>(part) * n * n;
  const W* wi = ri + static_cast<int64_t>(part) * n * n;
  float acc_a[8] = {}, acc_i[8] = {};
  for (int k0 = 0; k0 < n; k0 += LG_K) {
#pragma unroll
    for (int it = 0; it < LG_TOKENS * LG_K / 256; ++it) {
      const int idx = threadIdx.x + 256 * it;
      const int tok = idx / LG_K, kk = idx % LG_K;
      Us[tok][kk] = (t0 + tok < T && k0 + kk < n) ? to_float(u[static_cast<int64_t>(t0 + tok) * ldu + part * n + k0 + kk]) : 0.f;
    }
#pragma unroll
    for (int it = 0; it < LG_OUT * LG_K / 256; ++it) {
      const int idx = threadIdx.x + 256 * it;
      const int o = idx / LG_K, kk = idx % LG_K;
      const bool in = o0 + o < n && k0 + kk < n;
      Wa[o][kk] = in ? to_float(wa[static_cast<int64_t>(o0 + o) * n + k0 + kk]) : 0.f;
      Wi[o][kk] = in ? to_float(wi[static_cast<int64_t>(o0 + o) * n + k0 + kk]) : 0.f;
    }
    __syncthreads();
#pragma unroll 8
    for (int kk = 0; kk < LG_K; ++kk) {
      const float a = Wa[tx][kk], i = Wi[tx][kk];
#pragma unroll
      for (int m = 0; m < 8; ++m) {
        const float x = Us[ty * 8 + m][kk];
        acc_a[m] += a * x;
        acc_i[m] += i * x;
      }
    }
    __syncthreads();
  }
  if (o0 + tx >= n) return;
  const int c = part * n + o0 + tx;
  const float bias_a = ra_b[c], bias_i = ri_b[c];
  const float decay = -rate * softplus(lam[c]);
#pragma unroll
  for (int m = 0; m < 8; ++m) {
    const int t = t0 + ty * 8 + m;
    if (t >= T) break;
    const float r = sigmoid_exact(acc_a[m] + bias_a), i = sigmoid_exact(acc_i[m] + bias_i);
    const float log_a = decay * r;
    a_out[static_cast<int64_t>(t) * R + c] = expf(log_a);
    x_out[static_cast<int64_t>(t) * R + c] = sqrtf(-expm1f(2.f * log_a)) * i * to_float(u[static_cast<int64_t>(t) * ldu + c]);
  }
}

// The same for steps of up to LG_FEW rows: a wave owns one output channel, its lanes share the inputs of the part; both
// weight rows and every row's inputs are asked for before the first is used, so a step waits for one trip to memory.
constexpr int LG_FEW = 8;

template <typename X, typename W>
__global__ void __launch_bounds__(256)
lru_gates_few_kernel(const X* __restrict__ u, int64_t ldu, const W* __restrict__ ra, const float* __restrict__ ra_b,
                     const W* __restrict__ ri, const float* __restrict__ ri_b, const float* __restrict__ lam, float rate,
                     float* __restrict__ a_out, float* __restrict__ x_out, int T, int R, int n) {
  const int lane = threadIdx.x % 64;
  const int c = blockIdx.x * 4 + threadIdx.x / 64;
  if (c >= R) return;
  const int part = c / n;
  const W* wa = ra + static_cast<int64_t>(c) * n;          // [part][c - part * n][:] is row c of the stacked blocks
  const W* wi = ri + static_cast<int64_t>(c) * n;
  float acc_a[LG_FEW] = {}, acc_i[LG_FEW] = {};
  const float bias_a = ra_b[c], bias_i = ri_b[c], lam_c = lam[c];
  const float self = lane < T ? to_float(u[static_cast<int64_t>(lane) * ldu + c]) : 0.f;     // lane t: row t's own input
  for (int k0 = lane; k0 < n; k0 += 64 * 2) {
    float a[2], i[2], x[2][LG_FEW];
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const int k = k0 + 64 * s;
      a[s] = k < n ? to_float(wa[k]) : 0.f;
      i[s] = k < n ? to_float(wi[k]) : 0.f;
#pragma unroll
      for (int t = 0; t < LG_FEW; ++t) x[s][t] = (k < n && t < T) ? to_float(u[static_cast<int64_t>(t) * ldu + part * n + k]) : 0.f;
    }
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int t = 0; t < LG_FEW; ++t) acc_a[t] += a[s] * x[s][t], acc_i[t] += i[s] * x[s][t];
  }
  float sum_a = 0.f, sum_i = 0.f;                      // lane t: row t's sums
#pragma unroll
  for (int t = 0; t < LG_FEW; ++t) {
    if (t >= T) break;
    const float sa = wave_sum(acc_a[t]), si = wave_sum(acc_i[t]);
    if (lane == t) sum_a = sa, sum_i = si;
  }
  if (lane < T) {
    const float r = sigmoid_exact(sum_a + bias_a), i = sigmoid_exact(sum_i + bias_i);
    const float log_a = -rate * softplus(lam_c) * r;
    a_out[static_cast<int64_t>(lane) * R + c] = expf(log_a);
    x_out[static_cast<int64_t>(lane) * R + c] = sqrtf(-expm1f(2.f * log_a)) * i * self;
  }
}

// h_t = a_t h_(t-1) + x_t for every channel over a request's rows in order; out = h * act(mul). One thread a
// (request, channel); the loads of four rows are under way together (they do not hang on h).
template <typename M, typename O>
__global__ void lru_scan_kernel(const float* __restrict__ a, const float* __restrict__ x, float* __restrict__ state,
                                const M* __restrict__ mul, int64_t ldm, int kind, O* __restrict__ out,
                                const int32_t* __restrict__ cu_q, const int32_t* __restrict__ state_slots, int R) {
  const int b = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= R) return;
  const int first = cu_q[b], last = cu_q[b + 1];
  if (first >= last) return;
  float* own = state + static_cast<int64_t>(state_slots[b]) * R + c;
  float h = *own;
  for (int t = first; t < last; t += 4) {
    float av[4], xv[4], mv[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int64_t r = min(t + k, last - 1);
      av[k] = a[r * R + c];
      xv[k] = x[r * R + c];
      mv[k] = mul != nullptr ? to_float(mul[r * ldm + c]) : 1.f;
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      if (t + k >= last) break;
      h = av[k] * h + xv[k];
      out[static_cast<int64_t>(t + k) * R + c] = from_float<O>(mul != nullptr ? h * activate(mv[k], kind) : h);
    }
  }
  *own = h;
}

// The same scan over portions of prompts in chunks of rows that run side by side: every chunk first alone from
// h = 0 (its last value X and the product A of its factors), then again from the value in front of it, which a thread
// gets by walking the request's earlier chunks, h <- A h + X. The request's first chunk hands the state in front of
// the step to `init`, so that the last chunk may write the state behind it while others still read.
constexpr int LS_ROWS = 64;

__global__ void lru_chunk_sums_kernel(const float* __restrict__ a, const float* __restrict__ x, const float* __restrict__ state,
                                      float* __restrict__ factors, float* __restrict__ sums, float* __restrict__ init,
                                      const int4* __restrict__ chunks, const int32_t* __restrict__ request_chunks,
                                      const int32_t* __restrict__ state_slots, int R) {
  const int chunk = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= R) return;
  const int4 entry = chunks[chunk];
  const int64_t row0 = entry.y;
  const int len = entry.z;
  if (request_chunks[entry.x] == chunk) init[static_cast<int64_t>(entry.x) * R + c] = state[static_cast<int64_t>(state_slots[entry.x]) * R + c];
  float A = 1.f, X = 0.f;
  for (int j = 0; j < len; j += 4) {
    float av[4], xv[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int64_t r = row0 + min(j + k, len - 1);
      av[k] = a[r * R + c];
      xv[k] = x[r * R + c];
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      if (j + k >= len) break;
      X = av[k] * X + xv[k];
      A *= av[k];
    }
  }
  factors[static_cast<int64_t>(chunk) * R + c] = A;
  sums[static_cast<int64_t>(chunk) * R + c] = X;
}

template <typename M, typename O>
__global__ void lru_chunk_apply_kernel(const float* __restrict__ a, const float* __restrict__ x, float* __restrict__ state,
                                       const float* __restrict__ factors, const float* __restrict__ sums,
                                       const float* __restrict__ init, const M* __restrict__ mul, int64_t ldm, int kind,
                                       O* __restrict__ out, const int4* __restrict__ chunks,
                                       const int32_t* __restrict__ request_chunks, const int32_t* __restrict__ state_slots,
                                       int R) {
  const int chunk = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= R) return;
  const int4 entry = chunks[chunk];
  const int64_t row0 = entry.y;
  const int len = entry.z;
  float h = init[static_cast<int64_t>(entry.x) * R + c];
  for (int before = request_chunks[entry.x]; before < chunk; ++before)
    h = factors[static_cast<int64_t>(before) * R + c] * h + sums[static_cast<int64_t>(before) * R + c];
  for (int j = 0; j < len; j += 4) {
    float av[4], xv[4], mv[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int64_t r = row0 + min(j + k, len - 1);
      av[k] = a[r * R + c];
      xv[k] = x[r * R + c];
      mv[k] = mul != nullptr ? to_float(mul[r * ldm + c]) : 1.f;
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      if (j + k >= len) break;
      h = av[k] * h + xv[k];
      out[(row0 + j + k) * R + c] = from_float<O>(mul != nullptr ? h * activate(mv[k], kind) : h);
    }
  }
  if (chunk + 1 == request_chunks[entry.x + 1]) state[static_cast<int64_t>(state_slots[entry.x]) * R + c] = h;
}

// ---------------------------------------------------------------------------------------------------
// The router of a mixture of experts, one block a token: z = W x + b in float32 (a wave an expert at a time), then
// the `top` largest z by one wave (the lower index among equals), largest first, and the softmax over those alone.
constexpr int ROUTE_MAX_EXPERTS = 1024;
constexpr int ROUTE_MAX_TOP = 32;

// the weights of the chosen experts from their logits (largest first): softmax over those alone, or each one's own sigmoid
__device__ __forceinline__ void write_route_weights(const float* chosen, float* __restrict__ out, int top, int sigmoid) {
  if (sigmoid) {
    for (int k = 0; k < top; ++k) out[k] = 1.f / (1.f + expf(-chosen[k]));
    return;
  }
  const float peak = chosen[0];
  float total = 0.f;
  for (int k = 0; k < top; ++k) total += expf(chosen[k] - peak);
  for (int k = 0; k < top; ++k) out[k] = expf(chosen[k] - peak) / total;
}

template <typename X, typename W>
__global__ void __launch_bounds__(256)
route_topk_kernel(const X* __restrict__ x, const W* __restrict__ weight, const float* __restrict__ bias,
                  int32_t* __restrict__ experts, float* __restrict__ gates, int C, int E, int top, int sigmoid) {
  extern __shared__ float xs[];                       // the token's row as float32
  __shared__ float z[ROUTE_MAX_EXPERTS];
  __shared__ float chosen[ROUTE_MAX_TOP];
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  for (int c = threadIdx.x; c < C; c += blockDim.x) xs[c] = to_float(x[t * C + c]);
  __syncthreads();
  for (int e = wave; e < E; e += 4) {
    const W* w = weight + static_cast<int64_t>(e) * C;
    float acc = 0.f;
    for (int c0 = lane; c0 < C; c0 += 64 * 8) {
      float wv[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) wv[u] = c0 + 64 * u < C ? to_float(w[c0 + 64 * u]) : 0.f;
#pragma unroll
      for (int u = 0; u < 8; ++u)
        if (c0 + 64 * u < C) acc += wv[u] * xs[c0 + 64 * u];
    }
    acc = wave_sum(acc);
    if (lane == 0) z[e] = acc + (bias != nullptr ? bias[e] : 0.f);
  }
  __syncthreads();
  if (wave != 0) return;
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int at = 0x7fffffff;
    for (int e = lane; e < E; e += 64) {
      const float v = z[e];
      if (v > best || (v == best && e < at)) best = v, at = e;
    }
    // a NaN or a row of -inf never wins the comparison above: then the lowest index not yet taken does
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float other = __shfl_xor(best, o, 64);
      const int other_at = __shfl_xor(at, o, 64);
      if (other > best || (other == best && other_at < at)) best = other, at = other_at;
    }
    if (at == 0x7fffffff) at = k;                     // (unreachable for finite logits)
    if (lane == 0) {
      experts[t * top + k] = at;
      chosen[k] = best;
    }
    if (at % 64 == lane) z[at] = -INFINITY;           // the lane that reads this place takes it out itself
  }
  if (lane == 0) write_route_weights(chosen, gates + t * top, top, sigmoid);
}

// The same for bfloat16 rows and weights whose width is a multiple of 8: a thread takes 16-byte pieces of the token's
// row and of every expert's weight row, all asked for together (a step of few tokens waits for one trip to memory);
// experts in groups of 16.
constexpr int ROUTE_GROUP = 16;

__device__ __forceinline__ void unpack8(const uint4& raw, float v[8]) {
  const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    v[2 * e] = __uint_as_float(w[e] << 16);
    v[2 * e + 1] = __uint_as_float(w[e] & 0xffff0000u);
  }
}

// One row's router by one block of 256 threads: the chosen experts (largest logit first) and their weights end up in
// `ids` and `weights` (LDS), for every thread of the block to read.
struct RouteScratch {
  float z[ROUTE_MAX_EXPERTS];
  float part[4][ROUTE_GROUP];
  float chosen[ROUTE_MAX_TOP];
  int ids[ROUTE_MAX_TOP];
  float weights[ROUTE_MAX_TOP];
};

template <int GROUP>                                   // experts worked on side by side: 16, or 8 where there are no more
__device__ __forceinline__ void route_row_bf16(const bf16_t* __restrict__ x_row, const bf16_t* __restrict__ weight,
                                               const float* __restrict__ bias, int C, int E, int top, int sigmoid,
                                               RouteScratch& lds) {
  static_assert(GROUP <= ROUTE_GROUP, "the scratch holds ROUTE_GROUP sums a wave");
  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  const int pieces = C / 8;
  for (int e0 = 0; e0 < E; e0 += GROUP) {
    float acc[GROUP] = {};
    for (int p = threadIdx.x; p < pieces; p += 256) {
      uint4 raw[GROUP];
      const uint4 mine = *reinterpret_cast<const uint4*>(x_row + 8 * p);
#pragma unroll
      for (int g = 0; g < GROUP; ++g)
        raw[g] = *reinterpret_cast<const uint4*>(weight + static_cast<int64_t>(min(e0 + g, E - 1)) * C + 8 * p);
      float xv[8];
      unpack8(mine, xv);
#pragma unroll
      for (int g = 0; g < GROUP; ++g) {
        float wv[8];
        unpack8(raw[g], wv);
#pragma unroll
        for (int k = 0; k < 8; ++k) acc[g] += wv[k] * xv[k];
      }
    }
#pragma unroll
    for (int g = 0; g < GROUP; ++g) {
      const float total = wave_sum(acc[g]);
      if (lane == 0) lds.part[wave][g] = total;
    }
    __syncthreads();
    if (threadIdx.x < GROUP && e0 + threadIdx.x < E) {
      const int e = e0 + threadIdx.x;
      lds.z[e] = lds.part[0][threadIdx.x] + lds.part[1][threadIdx.x] + lds.part[2][threadIdx.x] + lds.part[3][threadIdx.x] +
                 (bias != nullptr ? bias[e] : 0.f);
    }
    __syncthreads();
  }
  if (wave == 0) {
    for (int k = 0; k < top; ++k) {
      float best = -INFINITY;
      int at = 0x7fffffff;
      for (int e = lane; e < E; e += 64) {
        const float v = lds.z[e];
        if (v > best || (v == best && e < at)) best = v, at = e;
      }
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) {
        const float other = __shfl_xor(best, o, 64);
        const int other_at = __shfl_xor(at, o, 64);
        if (other > best || (other == best && other_at < at)) best = other, at = other_at;
      }
      if (at == 0x7fffffff) at = k;
      if (lane == 0) {
        lds.ids[k] = at;
        lds.chosen[k] = best;
      }
      if (at % 64 == lane) lds.z[at] = -INFINITY;
    }
    if (lane == 0) write_route_weights(lds.chosen, lds.weights, top, sigmoid);
  }
  __syncthreads();
}

__global__ void __launch_bounds__(256)
route_topk_bf16_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ weight, const float* __restrict__ bias,
                       int32_t* __restrict__ experts, float* __restrict__ gates, int C, int E, int top, int sigmoid) {
  __shared__ RouteScratch lds;
  const int64_t t = blockIdx.x;
  if (E <= 8) {
    route_row_bf16<8>(x + t * C, weight, bias, C, E, top, sigmoid, lds);
  } else {
    route_row_bf16<ROUTE_GROUP>(x + t * C, weight, bias, C, E, top, sigmoid, lds);
  }
  if (threadIdx.x < top) {
    experts[t * top + threadIdx.x] = lds.ids[threadIdx.x];
    gates[t * top + threadIdx.x] = lds.weights[threadIdx.x];
  }
}

// hidden [T, ld]: the columns [e * F, (e + 1) * F) of expert e times the row's weight for e, zero if e was not chosen
template <typename X>
__global__ void route_scale_kernel(X* __restrict__ hidden, int64_t ld, const int32_t* __restrict__ experts,
                                   const float* __restrict__ gates, int top, int F, int width) {
  const int64_t t = blockIdx.x;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < width; c += gridDim.y * blockDim.x) {
    const int e = c / F;
    float g = 0.f;
    for (int k = 0; k < top; ++k)
      if (experts[t * top + k] == e) g = gates[t * top + k];
    X* p = hidden + t * ld + c;
    *p = from_float<X>(to_float(*p) * g);
  }
}

// the same on 16-byte pieces of bfloat16 rows (F, ld multiples of 8)
__global__ void route_scale_bf16x8_kernel(bf16_t* __restrict__ hidden, int64_t ld, const int32_t* __restrict__ experts,
                                          const float* __restrict__ gates, int top, int F, int width, int64_t T) {
  const int width8 = width / 8;
  const int64_t total = T * width8;
  for (int64_t it = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; it < total;
       it += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int64_t t = it / width8;
    const int c = 8 * static_cast<int>(it % width8);
    const int e = c / F;
    float g = 0.f;
    for (int k = 0; k < top; ++k)
      if (experts[t * top + k] == e) g = gates[t * top + k];
    uint4* p = reinterpret_cast<uint4*>(hidden + t * ld + c);
    float v[8];
    unpack8(*p, v);
    uint32_t w[4];
#pragma unroll
    for (int k = 0; k < 4; ++k)
      w[k] = static_cast<uint32_t>(__builtin_bit_cast(uint16_t, static_cast<bf16_t>(v[2 * k] * g))) |
             (static_cast<uint32_t>(__builtin_bit_cast(uint16_t, static_cast<bf16_t>(v[2 * k + 1] * g))) << 16);
    *p = uint4{w[0], w[1], w[2], w[3]};
  }
}

// The hidden values of routed gated experts from the stacked product: gate_up [T, ld] holds every expert's gate columns
// (E x F), then every expert's up columns; `slices` partial sums lie `stride` elements apart. For the expert e that owns
// column c, chosen by the row with weight w: g and u times w if `on_input`, clamped if limit > 0 (g from above, u on both
// sides), hidden = g * sigmoid(slope * g) * (u + up_shift), times w unless `on_input`; zero if the row did not choose e.
// V columns a thread (V > 1: F a multiple of V, rows aligned to V values). blockIdx.y walks the rows, so a row's choice is
// the same for the whole block and is read once; blockIdx.x and the thread give the columns.
constexpr int GLU_ROWS = 4;

template <int V, typename X, typename O>
__global__ void route_glu_kernel(const X* __restrict__ gate_up, int64_t ld, int slices, int64_t stride,
                                 const int32_t* __restrict__ experts, const float* __restrict__ gates, int top, int F,
                                 int width, float limit, float slope, float up_shift, int on_input, O* __restrict__ out,
                                 int64_t T) {
  // Blocks go to the chip's eight dies in turn by their number (blockIdx.x fastest): with the columns taken from
  // blockIdx.x alone, the blocks of one expert's columns would all land on the same die, and where most rows choose the
  // same experts two dies would do the reading for all. The block row shifts the columns, so every die gets its share.
  // A block's waves take runs of columns that lie a whole row of blocks apart, so a block meets several experts and has
  // its share of the chosen ones.
  const int column_block = (blockIdx.x + blockIdx.y) % gridDim.x;
  const int c = V * static_cast<int>((threadIdx.x / 64 * gridDim.x + column_block) * 64 + threadIdx.x % 64);
  if (c >= width) return;
  const int e = c / F;
  // GLU_ROWS rows a block row: their choices first, then every chosen row's loads together, then the arithmetic
  for (int64_t t0 = static_cast<int64_t>(blockIdx.y) * GLU_ROWS; t0 < T; t0 += static_cast<int64_t>(gridDim.y) * GLU_ROWS) {
    float w[GLU_ROWS], g[GLU_ROWS][V], u[GLU_ROWS][V];
    bool chosen[GLU_ROWS];
#pragma unroll
    for (int r = 0; r < GLU_ROWS; ++r) {
      w[r] = 0.f, chosen[r] = false;
      const int64_t t = t0 + r;
      if (t < T) {
        for (int k = 0; k < top; ++k)
          if (experts[t * top + k] == e) w[r] = gates[t * top + k], chosen[r] = true;
      }
    }
#pragma unroll
    for (int r = 0; r < GLU_ROWS; ++r) {
      if (!chosen[r]) continue;
      sum_values<V>(gate_up + (t0 + r) * ld + c, slices, stride, g[r]);
      sum_values<V>(gate_up + (t0 + r) * ld + width + c, slices, stride, u[r]);
    }
#pragma unroll
    for (int r = 0; r < GLU_ROWS; ++r) {
      if (t0 + r >= T) break;
      float h[V] = {};
      if (chosen[r]) {
#pragma unroll
        for (int k = 0; k < V; ++k) {
          float gk = g[r][k], uk = u[r][k];
          if (on_input) gk *= w[r], uk *= w[r];
          if (limit > 0.f) gk = fminf(gk, limit), uk = fminf(fmaxf(uk, -limit), limit);
          h[k] = gk / (1.f + expf(-slope * gk)) * (uk + up_shift);
          if (!on_input) h[k] *= w[r];
        }
      }
      store_values<V>(out + (t0 + r) * width + c, h);
    }
  }
}

// Router and hidden values in one launch, for steps of few rows (bfloat16 rows and router weights, C a multiple of 8):
// every block works out its row's choice again (the row and the router's weights come from the cache) and then does
// `route_glu_kernel`'s work on its 256 * V columns. blockIdx.y: the row.
template <int V, typename X, typename O>
__global__ void __launch_bounds__(256)
route_topk_glu_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ weight, const float* __restrict__ bias, int C,
                      int E, int top, int sigmoid, const X* __restrict__ gate_up, int64_t ld, int slices, int64_t stride,
                      int F, int width, float limit, float slope, float up_shift, int on_input, O* __restrict__ out) {
  __shared__ RouteScratch lds;
  const int64_t t = blockIdx.y;
  const int c = V * static_cast<int>(blockIdx.x * blockDim.x + threadIdx.x);
  // the thread's columns are asked for before the choice is known (few rows: reading what is not chosen costs nothing
  // beside the wait it saves)
  float g[V] = {}, u[V] = {};
  if (c < width) {
    sum_values<V>(gate_up + t * ld + c, slices, stride, g);
    sum_values<V>(gate_up + t * ld + width + c, slices, stride, u);
  }
  if (E <= 8) {
    route_row_bf16<8>(x + t * C, weight, bias, C, E, top, sigmoid, lds);
  } else {
    route_row_bf16<ROUTE_GROUP>(x + t * C, weight, bias, C, E, top, sigmoid, lds);
  }
  if (c >= width) return;
  const int e = c / F;
  float w = 0.f;
  bool chosen = false;
  for (int k = 0; k < top; ++k)
    if (lds.ids[k] == e) w = lds.weights[k], chosen = true;
  float h[V] = {};
  if (chosen) {
#pragma unroll
    for (int k = 0; k < V; ++k) {
      float gk = g[k], uk = u[k];
      if (on_input) gk *= w, uk *= w;
      if (limit > 0.f) gk = fminf(gk, limit), uk = fminf(fmaxf(uk, -limit), limit);
      h[k] = gk / (1.f + expf(-slope * gk)) * (uk + up_shift);
      if (!on_input) h[k] *= w;
    }
  }
  store_values<V>(out + t * width + c, h);
}

// x <- cap * tanh(x / cap)
__global__ void softcap_f32_kernel(float* __restrict__ x, int64_t count, float cap) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < count) x[i] = cap * tanhf(x[i] / cap);
}

__global__ void scale_f32_kernel(float* __restrict__ x, int64_t count, float scale) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < count) x[i] *= scale;
}

}  // namespace

extern "C" int distie_norm_chain(const void* t0, int t0_dtype, int slices0, const float* w0, const void* t1, int t1_dtype,
                                 int slices1, const float* w1, float term_eps, float scale, const float* post_w,
                                 float post_eps, float* residual, const float* pre_w, float pre_eps, void* out,
                                 int out_dtype, float* y_out, int T, int C, hipStream_t stream) {
  if (T <= 0) return 0;
  if (C < 1 || t0 == nullptr || slices0 < 1 || (t1 != nullptr && (slices1 < 1 || w0 == nullptr || w1 == nullptr)) ||
      (residual == nullptr && y_out == nullptr) || (residual != nullptr && pre_w != nullptr && out == nullptr) ||
      static_cast<size_t>(C) * sizeof(float) > 64 * 1024)
    return DISTIE_BAD_ARGUMENT;
  if (t1 == nullptr) t1_dtype = t0_dtype, slices1 = 1;
  if (out == nullptr) out_dtype = DISTIE_F32;
  const int64_t stride = static_cast<int64_t>(T) * C;
  const int held = C <= NORM_HELD_MAX ? 1 : 0;
  const size_t lds = static_cast<size_t>(C) * sizeof(float) * (held ? 4 : 1);
  const auto aligned = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  const bool wide = C % 4 == 0 && aligned(t0) && aligned(t1) && aligned(w0) && aligned(w1) && aligned(post_w) &&
                    aligned(residual) && aligned(pre_w) && aligned(out) && aligned(y_out);
  const int per = wide ? C / 4 : C;
  const int threads = per >= 1024 ? 1024 : (per >= 512 ? 512 : (per >= 256 ? 256 : (per >= 128 ? 128 : 64)));
#define DISTIE_NORM_CHAIN(V)                                                                                          \
  DISTIE_DISPATCH(t0_dtype, A, DISTIE_DISPATCH(t1_dtype, B, DISTIE_DISPATCH(out_dtype, O, {                           \
    if (lds > 48 * 1024 &&                                                                                            \
        hipFuncSetAttribute(reinterpret_cast<const void*>(norm_chain_kernel<V, A, B, O>),                             \
                            hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)) != hipSuccess)         \
      return DISTIE_BAD_ARGUMENT;                                                                                     \
    norm_chain_kernel<V, A, B, O><<<T, threads, lds, stream>>>(                                                       \
        static_cast<const A*>(t0), slices0, stride, w0, static_cast<const B*>(t1), slices1, stride, w1, term_eps,     \
        scale, post_w, post_eps, residual, pre_w, pre_eps, static_cast<O*>(out), y_out, C, held);                     \
  })))
  if (wide) {
    DISTIE_NORM_CHAIN(4);
  } else {
    DISTIE_NORM_CHAIN(1);
  }
#undef DISTIE_NORM_CHAIN
  return launch_status();
}

extern "C" int distie_gated_decay_scan_max_dim() { return 256; }

extern "C" int distie_gated_decay_scan_max_rank() { return GS_RANK_MAX; }

// logits null: z is made from low ([T, ld_low] of the product's dtype), up (float32 [H * D, rank]) and up_bias
extern "C" int distie_gated_decay_scan(const void* product, int dtype, int64_t ld, const float* logits, const void* low,
                                       int64_t ld_low, const float* up, const float* up_bias, int rank, float* state,
                                       float* out, const int32_t* cu_q, const int32_t* state_slots, int B, int H, int D,
                                       int E, float q_scale, float tau, hipStream_t stream) {
  if (B <= 0) return 0;
  if (H < 1 || D < 1 || E < 1 || D > 256 || !(tau > 0.f) || ld < static_cast<int64_t>(H) * (2 * D + E))
    return DISTIE_BAD_ARGUMENT;
  if (logits == nullptr && (low == nullptr || up == nullptr || up_bias == nullptr || rank < 1 || rank > GS_RANK_MAX ||
                            ld_low < rank))
    return DISTIE_BAD_ARGUMENT;
  const dim3 grid(B, H, (E + 63) / 64);
#define DISTIE_GSCAN(PARTS, ROWS)                                                                                     \
  DISTIE_DISPATCH(dtype, X, {                                                                                         \
    if (logits != nullptr)                                                                                            \
      gated_decay_scan_kernel<X, PARTS, ROWS, false><<<grid, 64 * PARTS, 0, stream>>>(                                \
          static_cast<const X*>(product), ld, logits, nullptr, 0, nullptr, nullptr, 0, state, out, cu_q, state_slots, \
          H, D, E, q_scale, tau);                                                                                     \
    else                                                                                                              \
      gated_decay_scan_kernel<X, PARTS, ROWS, true><<<grid, 64 * PARTS, 0, stream>>>(                                 \
          static_cast<const X*>(product), ld, nullptr, static_cast<const X*>(low), ld_low, up, up_bias, rank, state,  \
          out, cu_q, state_slots, H, D, E, q_scale, tau);                                                             \
  })
  if (D <= 32) {
    DISTIE_GSCAN(4, 8);
  } else if (D <= 64) {
    DISTIE_GSCAN(4, 16);
  } else if (D <= 128) {
    DISTIE_GSCAN(4, 32);
  } else {
    DISTIE_GSCAN(8, 32);
  }
#undef DISTIE_GSCAN
  return launch_status();
}

extern "C" int distie_gated_decay_scan_chunk_rows() { return GS_L; }
// the largest per-head key size the chunked scan takes (its tiles must fit the LDS of a compute unit)
extern "C" int distie_gated_decay_scan_chunked_max_dim() { return 128; }

template <typename K>
static int more_lds(K kernel, size_t lds) {
  if (lds <= 48 * 1024) return 0;
  return static_cast<int>(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                              static_cast<int>(lds)));
}

// chunks: int32 [num_chunks][4] = {request, first row, rows (1..64), 0}, the chunks of a request one after the other;
// request_chunks: int32 [B + 1], the first chunk of every request; scratch: float32 [num_chunks, H, D, E];
// totals: float32 [num_chunks, H, D]
extern "C" int distie_gated_decay_scan_chunked(const void* product, int dtype, int64_t ld, const float* logits,
                                               float* state, float* out, float* scratch, float* totals,
                                               const int32_t* chunks, const int32_t* request_chunks,
                                               const int32_t* state_slots, int num_chunks, int B, int H, int D, int E,
                                               float q_scale, float tau, hipStream_t stream) {
  if (B <= 0 || num_chunks <= 0) return 0;
  if (H < 1 || D < 4 || E < 4 || D % 4 || E % 4 || D > 128 || !(tau > 0.f) || ld < static_cast<int64_t>(H) * (2 * D + E))
    return DISTIE_BAD_ARGUMENT;
  const dim3 grid(num_chunks, H, (E + 63) / 64);
  const int4* table = reinterpret_cast<const int4*>(chunks);
  const size_t lds_sums = (static_cast<size_t>(D) * GS_PAD + GS_L * D + GS_L * 64) * sizeof(float);
  const size_t lds_out = (3 * static_cast<size_t>(D) * GS_PAD + GS_L * GS_PAD + GS_L * 64) * sizeof(float);
  int status = 0;
  DISTIE_DISPATCH(dtype, X, {
    if ((status = more_lds(gated_chunk_sums_kernel<X>, lds_sums)) != 0) return status;
    if ((status = more_lds(gated_chunk_outputs_kernel<X>, lds_out)) != 0) return status;
    gated_chunk_sums_kernel<X><<<grid, 256, lds_sums, stream>>>(static_cast<const X*>(product), ld, logits, tau, scratch,
                                                                totals, table, H, D, E);
    if ((status = launch_status()) != 0) return status;
    gated_chunk_states_kernel<<<dim3(B, H, (D * E + 255) / 256), 256, 0, stream>>>(scratch, totals, state, request_chunks,
                                                                                  state_slots, H, D, E);
    if ((status = launch_status()) != 0) return status;
    gated_chunk_outputs_kernel<X><<<grid, 256, lds_out, stream>>>(static_cast<const X*>(product), ld, logits, tau, q_scale,
                                                                  scratch, out, table, H, D, E);
  });
  return launch_status();
}

extern "C" int distie_lru_gates(const void* u, int u_dtype, int64_t ldu, const void* ra, const float* ra_b, const void* ri,
                                const float* ri_b, int w_dtype, const float* lam, float rate, float* a_out, float* x_out,
                                int T, int R, int blocks, hipStream_t stream) {
  if (T <= 0) return 0;
  if (R < 1 || blocks < 1 || R % blocks || ldu < R) return DISTIE_BAD_ARGUMENT;
  const int n = R / blocks;
  if (T <= LG_FEW) {
    DISTIE_DISPATCH(u_dtype, X, DISTIE_DISPATCH(w_dtype, W,
        lru_gates_few_kernel<X, W><<<(R + 3) / 4, 256, 0, stream>>>(
            static_cast<const X*>(u), ldu, static_cast<const W*>(ra), ra_b, static_cast<const W*>(ri), ri_b, lam, rate,
            a_out, x_out, T, R, n)));
    return launch_status();
  }
  const dim3 grid((T + LG_TOKENS - 1) / LG_TOKENS, blocks, (n + LG_OUT - 1) / LG_OUT);
  DISTIE_DISPATCH(u_dtype, X, DISTIE_DISPATCH(w_dtype, W,
      lru_gates_kernel<X, W><<<grid, 256, 0, stream>>>(
          static_cast<const X*>(u), ldu, static_cast<const W*>(ra), ra_b, static_cast<const W*>(ri), ri_b, lam, rate,
          a_out, x_out, T, R, n)));
  return launch_status();
}

extern "C" int distie_lru_scan(const float* a, const float* x, float* state, const void* mul, int mul_dtype, int64_t ldm,
                               int kind, void* out, int out_dtype, const int32_t* cu_q, const int32_t* state_slots, int B,
                               int R, hipStream_t stream) {
  if (B <= 0) return 0;
  if (R < 1 || kind < -1 || kind > 3 || (mul != nullptr && ldm < R)) return DISTIE_BAD_ARGUMENT;
  if (mul == nullptr) mul_dtype = DISTIE_F32;
  const int threads = R >= 256 ? 256 : (R >= 128 ? 128 : 64);
  const dim3 grid(B, (R + threads - 1) / threads);
  DISTIE_DISPATCH(mul_dtype, M, DISTIE_DISPATCH(out_dtype, O,
      lru_scan_kernel<M, O><<<grid, threads, 0, stream>>>(a, x, state, static_cast<const M*>(mul), ldm, kind,
                                                          static_cast<O*>(out), cu_q, state_slots, R)));
  return launch_status();
}

extern "C" int distie_lru_scan_chunk_rows() { return LS_ROWS; }

// chunks / request_chunks as for the chunked scans of states; factors, sums: float32 [num_chunks, R]; init: float32 [B, R]
extern "C" int distie_lru_scan_chunked(const float* a, const float* x, float* state, float* factors, float* sums, float* init,
                                       const void* mul, int mul_dtype, int64_t ldm, int kind, void* out, int out_dtype,
                                       const int32_t* chunks, const int32_t* request_chunks, const int32_t* state_slots,
                                       int num_chunks, int B, int R, hipStream_t stream) {
  if (B <= 0 || num_chunks <= 0) return 0;
  if (R < 1 || kind < -1 || kind > 3 || (mul != nullptr && ldm < R)) return DISTIE_BAD_ARGUMENT;
  if (mul == nullptr) mul_dtype = DISTIE_F32;
  const int threads = R >= 256 ? 256 : (R >= 128 ? 128 : 64);
  const dim3 grid(num_chunks, (R + threads - 1) / threads);
  const int4* table = reinterpret_cast<const int4*>(chunks);
  lru_chunk_sums_kernel<<<grid, threads, 0, stream>>>(a, x, state, factors, sums, init, table, request_chunks, state_slots, R);
  const int status = launch_status();
  if (status != 0) return status;
  DISTIE_DISPATCH(mul_dtype, M, DISTIE_DISPATCH(out_dtype, O,
      lru_chunk_apply_kernel<M, O><<<grid, threads, 0, stream>>>(a, x, state, factors, sums, init,
                                                                 static_cast<const M*>(mul), ldm, kind, static_cast<O*>(out),
                                                                 table, request_chunks, state_slots, R)));
  return launch_status();
}

extern "C" int distie_route_topk(const void* x, int x_dtype, const void* weight, int w_dtype, const float* bias,
                                 int32_t* experts, float* gates, int T, int C, int E, int top, int sigmoid,
                                 hipStream_t stream) {
  if (T <= 0) return 0;
  if (C < 1 || E < 1 || E > ROUTE_MAX_EXPERTS || top < 1 || top > E || top > ROUTE_MAX_TOP ||
      static_cast<size_t>(C) * sizeof(float) > 96 * 1024)
    return DISTIE_BAD_ARGUMENT;
  if (x_dtype == DISTIE_BF16 && w_dtype == DISTIE_BF16 && C % 8 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(weight) % 16 == 0) {
    route_topk_bf16_kernel<<<T, 256, 0, stream>>>(static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(weight), bias,
                                                  experts, gates, C, E, top, sigmoid);
    return launch_status();
  }
  const size_t lds = static_cast<size_t>(C) * sizeof(float);
  DISTIE_DISPATCH(x_dtype, X, DISTIE_DISPATCH(w_dtype, W, {
    if (lds > 48 * 1024 &&
        hipFuncSetAttribute(reinterpret_cast<const void*>(route_topk_kernel<X, W>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)) != hipSuccess)
      return DISTIE_BAD_ARGUMENT;
    route_topk_kernel<X, W><<<T, 256, lds, stream>>>(static_cast<const X*>(x), static_cast<const W*>(weight), bias,
                                                     experts, gates, C, E, top, sigmoid);
  }));
  return launch_status();
}

extern "C" int distie_route_scale(void* hidden, int dtype, int64_t ld, const int32_t* experts, const float* gates, int T,
                                  int top, int E, int F, hipStream_t stream) {
  if (T <= 0) return 0;
  if (top < 1 || E < 1 || F < 1 || ld < static_cast<int64_t>(E) * F) return DISTIE_BAD_ARGUMENT;
  const int width = E * F;
  if (dtype == DISTIE_BF16 && F % 8 == 0 && ld % 8 == 0 && reinterpret_cast<uintptr_t>(hidden) % 16 == 0) {
    const int64_t pieces = static_cast<int64_t>(T) * (width / 8);
    const int blocks8 = static_cast<int>(pieces / 256 + 1 < 16384 ? pieces / 256 + 1 : 16384);
    route_scale_bf16x8_kernel<<<blocks8, 256, 0, stream>>>(static_cast<bf16_t*>(hidden), ld, experts, gates, top, F, width, T);
    return launch_status();
  }
  const int per_row = (width + 255) / 256;
  const dim3 grid(T, per_row < 64 ? per_row : 64);
  DISTIE_DISPATCH(dtype, X, route_scale_kernel<X><<<grid, 256, 0, stream>>>(static_cast<X*>(hidden), ld, experts, gates,
                                                                            top, F, width));
  return launch_status();
}

// gate_up: [T, ld] of `dtype`, or `slices` float32 partial sums [slices, T, ld]; out: [T, E * F] of `out_dtype`.
// limit <= 0: no clamps.
extern "C" int distie_route_glu(const void* gate_up, int dtype, int64_t ld, int slices, const int32_t* experts,
                                const float* gates, int T, int top, int E, int F, float limit, float slope, float up_shift,
                                int on_input, void* out, int out_dtype, hipStream_t stream) {
  if (T <= 0) return 0;
  if (top < 1 || E < 1 || F < 1 || slices < 1 || (slices > 1 && dtype != DISTIE_F32) || ld < 2 * static_cast<int64_t>(E) * F)
    return DISTIE_BAD_ARGUMENT;
  const int width = E * F;
  const int64_t stride = static_cast<int64_t>(T) * ld;
  const bool aligned = reinterpret_cast<uintptr_t>(gate_up) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0;
  const int V = aligned && F % 8 == 0 && ld % 8 == 0 ? 8 : (aligned && F % 4 == 0 && ld % 4 == 0 ? 4 : 1);
  const int per_row = width / V;
  const int threads = per_row >= 256 ? 256 : (per_row > 64 ? 128 : 64);
  const int row_groups = (T + GLU_ROWS - 1) / GLU_ROWS;
  const dim3 grid((per_row + threads - 1) / threads, row_groups < 32768 ? row_groups : 32768);
#define DISTIE_ROUTE_GLU(V)                                                                                           \
  DISTIE_DISPATCH(dtype, X, DISTIE_DISPATCH(out_dtype, O, (route_glu_kernel<V, X, O><<<grid, threads, 0, stream>>>(   \
      static_cast<const X*>(gate_up), ld, slices, stride, experts, gates, top, F, width, limit, slope, up_shift,      \
      on_input, static_cast<O*>(out), T))))
  if (V == 8) {
    DISTIE_ROUTE_GLU(8);
  } else if (V == 4) {
    DISTIE_ROUTE_GLU(4);
  } else {
    DISTIE_ROUTE_GLU(1);
  }
#undef DISTIE_ROUTE_GLU
  return launch_status();
}

// `distie_route_topk` (bfloat16 rows and weights) and `distie_route_glu` in one launch; for steps of few rows.
extern "C" int distie_route_topk_glu(const void* x, const void* weight, const float* bias, int C, int sigmoid,
                                     const void* gate_up, int dtype, int64_t ld, int slices, int T, int top, int E, int F,
                                     float limit, float slope, float up_shift, int on_input, void* out, int out_dtype,
                                     hipStream_t stream) {
  if (T <= 0) return 0;
  if (C < 8 || C % 8 || E < 1 || E > ROUTE_MAX_EXPERTS || top < 1 || top > E || top > ROUTE_MAX_TOP || F < 1 || slices < 1 ||
      T > 65535 || (slices > 1 && dtype != DISTIE_F32) || ld < 2 * static_cast<int64_t>(E) * F ||
      reinterpret_cast<uintptr_t>(x) % 16 != 0 || reinterpret_cast<uintptr_t>(weight) % 16 != 0)
    return DISTIE_BAD_ARGUMENT;
  const int width = E * F;
  const int64_t stride = static_cast<int64_t>(T) * ld;
  const bool aligned = reinterpret_cast<uintptr_t>(gate_up) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0;
  const int V = aligned && F % 8 == 0 && ld % 8 == 0 ? 8 : (aligned && F % 4 == 0 && ld % 4 == 0 ? 4 : 1);
  const dim3 grid((width / V + 255) / 256, T);
#define DISTIE_ROUTE_TOPK_GLU(V)                                                                                          \
  DISTIE_DISPATCH(dtype, X, DISTIE_DISPATCH(out_dtype, O, (route_topk_glu_kernel<V, X, O><<<grid, 256, 0, stream>>>(       \
      static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(weight), bias, C, E, top, sigmoid,                        \
      static_cast<const X*>(gate_up), ld, slices, stride, F, width, limit, slope, up_shift, on_input, static_cast<O*>(out)))))
  if (V == 8) {
    DISTIE_ROUTE_TOPK_GLU(8);
  } else if (V == 4) {
    DISTIE_ROUTE_TOPK_GLU(4);
  } else {
    DISTIE_ROUTE_TOPK_GLU(1);
  }
#undef DISTIE_ROUTE_TOPK_GLU
  return launch_status();
}

extern "C" int distie_softcap_f32(float* x, int64_t count, float cap, hipStream_t stream) {
  if (count <= 0) return 0;
  if (!(cap > 0.f)) return DISTIE_BAD_ARGUMENT;
  const int64_t blocks = (count + 255) / 256;
  if (blocks > 0x7fffffff) return DISTIE_BAD_ARGUMENT;
  softcap_f32_kernel<<<static_cast<unsigned>(blocks), 256, 0, stream>>>(x, count, cap);
  return launch_status();
}

extern "C" int distie_scale_f32(float* x, int64_t count, float scale, hipStream_t stream) {
  if (count <= 0) return 0;
  const int64_t blocks = (count + 255) / 256;
  if (blocks > 0x7fffffff) return DISTIE_BAD_ARGUMENT;
  scale_f32_kernel<<<static_cast<unsigned>(blocks), 256, 0, stream>>>(x, count, scale);
  return launch_status();
}
