// Kernels of attention over a latent that all heads share, and of gates that are one number a head.
//
// Latent attention keeps, for every token, one normed latent vector c (kv_rank wide) and one rotated key part r
// (rot_dim wide). The attention kernels read them as one key/value head of size DP >= kv_rank + rot_dim: the key of a
// token is (c, r, zeros), its value (c, zeros). What is float32 in either precision: both norms' statistics, the
// angles' cosines and sines, the rotation, every sum of a product.
//
// A step is a flattened batch: token t writes its key and value at slot slots[t] = page * P + offset of the cache,
// k [pages, 1, P, DP], v [pages, 1, DP, P] (values transposed inside a page).
#include "common.h"

namespace {

__device__ __forceinline__ float sigmoidf(float x) { return 1.f / (1.f + __expf(-x)); }

// ---------------------------------------------------------------------------------------------------
// Behind the stacked down-projection: down float32 [T, ld] holds the queries' latent (q_rank), the keys' and values'
// latent (kv_rank) and the key part that is rotated (rot_dim). One block a token.
//   latent[t]   = down[:q_rank] / sqrt(mean(.^2) + eps) * q_weight                    (O, [T, q_rank])
//   c           = down[q_rank : q_rank + kv_rank] / sqrt(mean(.^2) + eps) * kv_weight  -> k[slot][:kv_rank], v[:kv_rank][slot]
//   r           = the last rot_dim values, turned by the token's angles                -> k[slot][kv_rank : kv_rank + rot_dim]
// table [T, pairs] holds (cos, sin) of every pair's angle; both are multiplied by `magnitude`. `neighbours`: the pair
// is (2 j, 2 j + 1), else (j, j + pairs). What lies beyond kv_rank + rot_dim in a key and beyond kv_rank in a value
// was zero when the cache was made and is never written.
template <typename O, typename C>
__global__ void latent_norm_rope_write_kernel(const float* __restrict__ down, int64_t ld, int q_rank,
                                              const float* __restrict__ q_weight, int kv_rank,
                                              const float* __restrict__ kv_weight, float eps, int rot_dim,
                                              const float2* __restrict__ table, float magnitude, int neighbours,
                                              O* __restrict__ latent, C* __restrict__ k_cache, C* __restrict__ v_cache,
                                              const int32_t* __restrict__ slots, int P, int DP, int write) {
  __shared__ float scratch[16];
  const int64_t t = blockIdx.x;
  const float* row = down + t * ld;
  if (q_rank > 0) {
    float sq = 0.f;
    for (int c = threadIdx.x; c < q_rank; c += blockDim.x) sq += row[c] * row[c];
    sq = block_sum(sq, scratch);
    const float scale = 1.f / sqrtf(sq / q_rank + eps);
    for (int c = threadIdx.x; c < q_rank; c += blockDim.x)
      latent[t * q_rank + c] = from_float<O>(row[c] * scale * q_weight[c]);
  }
  if (!write) return;
  const float* kv = row + q_rank;
  float sq = 0.f;
  for (int c = threadIdx.x; c < kv_rank; c += blockDim.x) sq += kv[c] * kv[c];
  sq = block_sum(sq, scratch);
  const float scale = 1.f / sqrtf(sq / kv_rank + eps);
  const int slot = slots[t];
  const int64_t page = slot / P;
  const int off = slot % P;
  C* key = k_cache + (page * P + off) * DP;
  C* value = v_cache + page * DP * P + off;
  for (int c = threadIdx.x; c < kv_rank; c += blockDim.x) {
    const C v = from_float<C>(kv[c] * scale * kv_weight[c]);
    key[c] = v;
    value[static_cast<int64_t>(c) * P] = v;
  }
  const float* r = kv + kv_rank;
  const int pairs = rot_dim / 2;
  for (int j = threadIdx.x; j < pairs; j += blockDim.x) {
    const int a = neighbours ? 2 * j : j, b = neighbours ? 2 * j + 1 : j + pairs;
    float cs = 1.f, sn = 0.f;
    if (table != nullptr) {
      const float2 w = table[t * pairs + j];
      cs = w.x * magnitude, sn = w.y * magnitude;
    }
    const float u = r[a], v = r[b];
    key[kv_rank + a] = from_float<C>(u * cs - v * sn);
    key[kv_rank + b] = from_float<C>(v * cs + u * sn);
  }
}

// ---------------------------------------------------------------------------------------------------
// out[t, h * lo + offset_out + (a, b)] = the pair (a, b) at x[t, h * lx + offset_in + .] turned by the token's angle.
// One block a token, a thread a (head, pair).
template <typename X>
__global__ void rope_heads_kernel(const X* __restrict__ x, int lx, int offset_in, X* __restrict__ out, int lo,
                                  int offset_out, int H, int pairs, const float2* __restrict__ table, float magnitude,
                                  int neighbours) {
  const int64_t t = blockIdx.x;
  for (int i = threadIdx.x; i < H * pairs; i += blockDim.x) {
    const int h = i / pairs, j = i % pairs;
    const int a = neighbours ? 2 * j : j, b = neighbours ? 2 * j + 1 : j + pairs;
    const float2 w = table[t * pairs + j];
    const float cs = w.x * magnitude, sn = w.y * magnitude;
    const X* in = x + (t * H + h) * lx + offset_in;
    X* to = out + (t * H + h) * lo + offset_out;
    const float u = to_float(in[a]), v = to_float(in[b]);
    to[a] = from_float<X>(u * cs - v * sn);
    to[b] = from_float<X>(v * cs + u * sn);
  }
}

// ---------------------------------------------------------------------------------------------------
// A product for every head: out[t, h * lo + n] = sum_k x[t, h * lx + k] * w[h][n][k], n < N, k < K. Tiles of 64 rows
// of x by 64 rows of a head's weight, 16 of k at a time through LDS, float32 sums (FMAs): the path of float32 steps
// and of sizes the matrix-core kernel does not take. blockIdx = (tile of n, tile of t, head).
constexpr int HL_TILE = 64, HL_K = 16;

template <typename X, typename W>
__global__ void __launch_bounds__(256)
heads_linear_kernel(const X* __restrict__ x, int lx, const W* __restrict__ w, X* __restrict__ out, int lo, int T, int H,
                    int N, int K) {
  __shared__ float xs[HL_K][HL_TILE + 1], ws[HL_K][HL_TILE + 1];
  const int h = blockIdx.z;
  const int t0 = blockIdx.y * HL_TILE, n0 = blockIdx.x * HL_TILE;
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;          // tx: columns n, ty: rows t
  const W* wh = w + static_cast<int64_t>(h) * N * K;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += HL_K) {
    __syncthreads();
    for (int i = threadIdx.x; i < HL_TILE * HL_K; i += 256) {
      const int r = i / HL_K, k = i % HL_K;
      const int t = t0 + r, n = n0 + r;
      xs[k][r] = (t < T && k0 + k < K) ? to_float(x[(static_cast<int64_t>(t) * H + h) * lx + k0 + k]) : 0.f;
      ws[k][r] = (n < N && k0 + k < K) ? to_float(wh[static_cast<int64_t>(n) * K + k0 + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < HL_K; ++k) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = xs[k][ty + 16 * i], b[i] = ws[k][tx + 16 * i];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] += a[i] * b[j];
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int t = t0 + ty + 16 * i;
    if (t >= T) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx + 16 * j;
      if (n < N) out[(static_cast<int64_t>(t) * H + h) * lo + n] = from_float<X>(acc[i][j]);
    }
  }
}

// The same product for few rows of x (a decode step): a wave a (head, row n of its weight), lanes along k, every row of
// x against the one weight row that the wave holds in registers. Up to HLR_ROWS rows of x a launch row (blockIdx.y).
constexpr int HLR_ROWS = 8;

template <typename X, typename W>
__global__ void __launch_bounds__(256)
heads_linear_rows_kernel(const X* __restrict__ x, int lx, const W* __restrict__ w, X* __restrict__ out, int lo, int T,
                         int H, int N, int K) {
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int64_t item = static_cast<int64_t>(blockIdx.x) * 4 + wave;          // (head, n)
  if (item >= static_cast<int64_t>(H) * N) return;
  const int h = static_cast<int>(item / N), n = static_cast<int>(item % N);
  const W* wr = w + item * K;
  const int t0 = blockIdx.y * HLR_ROWS;
  float acc[HLR_ROWS] = {};
  for (int k = lane; k < K; k += 64) {
    const float wv = to_float(wr[k]);
#pragma unroll
    for (int r = 0; r < HLR_ROWS; ++r) {
      const int t = t0 + r;
      if (t < T) acc[r] += wv * to_float(x[(static_cast<int64_t>(t) * H + h) * lx + k]);
    }
  }
#pragma unroll
  for (int r = 0; r < HLR_ROWS; ++r) {
    const float total = wave_sum(acc[r]);
    const int t = t0 + r;
    if (lane == 0 && t < T) out[(static_cast<int64_t>(t) * H + h) * lo + n] = from_float<X>(total);
  }
}

// The same product on the matrix cores, bfloat16 operands and float32 sums (v_mfma_f32_32x32x16_bf16): a wave owns 32
// rows of x by 32 * NB rows of a head's weight and walks k sixteen at a time; both operands are rows with k innermost,
// so a lane's eight values are one 16-byte load (row = lane % 32, k = 8 * (lane / 32) ..). The weights of a head are
// small (they stay in the caches), so nothing goes through LDS. A workgroup is WT x WN waves; blockIdx = (tile of n,
// tile of t, head). K and the row strides are multiples of 8.
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 hl_bf16x8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float hl_floatx16;

template <int WT, int WN, int NB>
__global__ void __launch_bounds__(64 * WT * WN)
heads_linear_mfma_kernel(const bf16_t* __restrict__ x, int lx, const bf16_t* __restrict__ w, bf16_t* __restrict__ out,
                         int lo, int T, int H, int N, int K) {
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int h = blockIdx.z;
  const int t0 = (blockIdx.y * WT + wave / WN) * 32;
  const int n0 = (blockIdx.x * WN + wave % WN) * 32 * NB;
  if (t0 >= T || n0 >= N) return;
  const int r = lane % 32, kk = 8 * (lane / 32);
  const bool t_in = t0 + r < T;
  const bf16_t* xr = x + (static_cast<int64_t>(t_in ? t0 + r : t0) * H + h) * lx + kk;
  const bf16_t* wr[NB];
  bool n_in[NB];
#pragma unroll
  for (int b = 0; b < NB; ++b) {
    n_in[b] = n0 + 32 * b + r < N;
    wr[b] = w + (static_cast<int64_t>(h) * N + (n_in[b] ? n0 + 32 * b + r : n0)) * K + kk;
  }
  hl_floatx16 acc[NB];
#pragma unroll
  for (int b = 0; b < NB; ++b)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[b][i] = 0.f;
  for (int k0 = 0; k0 < K; k0 += 32) {
    // two k-steps' loads under way together
    hl_bf16x8 a[2], bw[2][NB];
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const int k = k0 + 16 * s;
      const bool k_in = k + kk < K;
      a[s] = (t_in && k_in) ? *reinterpret_cast<const hl_bf16x8*>(xr + k) : hl_bf16x8{};
#pragma unroll
      for (int b = 0; b < NB; ++b)
        bw[s][b] = (n_in[b] && k_in) ? *reinterpret_cast<const hl_bf16x8*>(wr[b] + k) : hl_bf16x8{};
    }
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int b = 0; b < NB; ++b) acc[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[s], bw[s][b], acc[b], 0, 0, 0);
  }
  // acc[b][4 i + j]: row t0 + 8 i + 4 (lane / 32) + j of x, weight row n0 + 32 b + lane % 32
#pragma unroll
  for (int b = 0; b < NB; ++b) {
    const int n = n0 + 32 * b + r;
    if (n >= N) continue;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int t = t0 + 8 * i + 4 * (lane / 32) + j;
        if (t < T) out[(static_cast<int64_t>(t) * H + h) * lo + n] = static_cast<bf16_t>(acc[b][4 * i + j]);
      }
  }
}

// ---------------------------------------------------------------------------------------------------
// out[t, h * E + e] = x[t, h * ldh + e] * sigmoid(gates[t * ldg + h]): one gate a head
template <typename X, typename G, typename O>
__global__ void head_gate_kernel(const X* __restrict__ x, int ldh, int E, const G* __restrict__ gates, int64_t ldg,
                                 O* __restrict__ out, int width) {
  const int64_t t = blockIdx.x;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < width; c += gridDim.y * blockDim.x) {
    const int head = c / E, e = c % E;
    const float v = to_float(x[(t * (width / E) + head) * ldh + e]);
    out[t * width + c] = from_float<O>(v * sigmoidf(to_float(gates[t * ldg + head])));
  }
}

}  // namespace

extern "C" int distie_latent_norm_rope_write(const float* down, int64_t ld, int q_rank, const float* q_weight, int kv_rank,
                                             const float* kv_weight, float eps, int rot_dim, const void* table,
                                             float magnitude, int neighbours, void* latent, int out_dtype, void* k_cache,
                                             void* v_cache, int cache_dtype, const int32_t* slots, int T, int P, int DP,
                                             int write, hipStream_t stream) {
  if (T <= 0) return 0;
  if (q_rank < 0 || kv_rank < 1 || rot_dim < 0 || rot_dim % 2 || ld < static_cast<int64_t>(q_rank) + kv_rank + rot_dim ||
      (q_rank > 0 && (q_weight == nullptr || latent == nullptr)) || kv_weight == nullptr ||
      (write && (k_cache == nullptr || v_cache == nullptr || slots == nullptr || P < 1 || DP < kv_rank + rot_dim)))
    return DISTIE_BAD_ARGUMENT;
  const int widest = q_rank > kv_rank ? q_rank : kv_rank;
  const int threads = widest >= 256 ? 256 : (widest >= 128 ? 128 : 64);
  DISTIE_DISPATCH(out_dtype, O, DISTIE_DISPATCH(cache_dtype, C,
      latent_norm_rope_write_kernel<O, C><<<T, threads, 0, stream>>>(
          down, ld, q_rank, q_weight, kv_rank, kv_weight, eps, rot_dim, static_cast<const float2*>(table), magnitude,
          neighbours, static_cast<O*>(latent), static_cast<C*>(k_cache), static_cast<C*>(v_cache), slots, P, DP, write)));
  return launch_status();
}

extern "C" int distie_rope_heads(const void* x, int dtype, int lx, int offset_in, void* out, int lo, int offset_out, int T,
                                 int H, int pairs, const void* table, float magnitude, int neighbours, hipStream_t stream) {
  if (T <= 0 || pairs <= 0) return 0;
  if (H < 1 || table == nullptr || offset_in < 0 || offset_out < 0 || offset_in + 2 * pairs > lx || offset_out + 2 * pairs > lo)
    return DISTIE_BAD_ARGUMENT;
  const int items = H * pairs;
  const int threads = items >= 256 ? 256 : (items >= 128 ? 128 : 64);
  DISTIE_DISPATCH(dtype, X, rope_heads_kernel<X><<<T, threads, 0, stream>>>(
      static_cast<const X*>(x), lx, offset_in, static_cast<X*>(out), lo, offset_out, H, pairs,
      static_cast<const float2*>(table), magnitude, neighbours));
  return launch_status();
}

// the most rows of x that the kernel for few rows is chosen for
extern "C" int distie_heads_linear_few_rows() { return 2 * HLR_ROWS; }

extern "C" int distie_heads_linear(const void* x, int dtype, int lx, const void* w, int w_dtype, void* out, int lo, int T,
                                   int H, int N, int K, hipStream_t stream) {
  if (T <= 0) return 0;
  if (H < 1 || N < 1 || K < 1 || lx < K || lo < N || H > 65535) return DISTIE_BAD_ARGUMENT;
  if (dtype == DISTIE_BF16 && w_dtype == DISTIE_BF16 && K % 8 == 0 && lx % 8 == 0 &&
      reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0) {
    const bf16_t* xb = static_cast<const bf16_t*>(x);
    const bf16_t* wb = static_cast<const bf16_t*>(w);
    bf16_t* ob = static_cast<bf16_t*>(out);
    if (T <= 32) {
      heads_linear_mfma_kernel<1, 4, 1><<<dim3((N + 127) / 128, 1, H), 256, 0, stream>>>(xb, lx, wb, ob, lo, T, H, N, K);
    } else {
      const dim3 grid((N + 127) / 128, (T + 63) / 64, H);
      if (grid.y > 65535) return DISTIE_BAD_ARGUMENT;
      heads_linear_mfma_kernel<2, 2, 2><<<grid, 256, 0, stream>>>(xb, lx, wb, ob, lo, T, H, N, K);
    }
    return launch_status();
  }
  if (T <= 2 * HLR_ROWS) {
    const int64_t items = static_cast<int64_t>(H) * N;
    const dim3 grid(static_cast<unsigned>((items + 3) / 4), (T + HLR_ROWS - 1) / HLR_ROWS);
    DISTIE_DISPATCH(dtype, X, DISTIE_DISPATCH(w_dtype, W, heads_linear_rows_kernel<X, W><<<grid, 256, 0, stream>>>(
        static_cast<const X*>(x), lx, static_cast<const W*>(w), static_cast<X*>(out), lo, T, H, N, K)));
    return launch_status();
  }
  const dim3 grid((N + HL_TILE - 1) / HL_TILE, (T + HL_TILE - 1) / HL_TILE, H);
  if (grid.y > 65535) return DISTIE_BAD_ARGUMENT;
  DISTIE_DISPATCH(dtype, X, DISTIE_DISPATCH(w_dtype, W, heads_linear_kernel<X, W><<<grid, 256, 0, stream>>>(
      static_cast<const X*>(x), lx, static_cast<const W*>(w), static_cast<X*>(out), lo, T, H, N, K)));
  return launch_status();
}

extern "C" int distie_head_gate(const void* x, int x_dtype, int ldh, int E, const void* gates, int g_dtype, int64_t ldg,
                                void* out, int out_dtype, int T, int width, hipStream_t stream) {
  if (T <= 0) return 0;
  if (E < 1 || width < 1 || width % E || ldh < E || gates == nullptr || ldg < width / E) return DISTIE_BAD_ARGUMENT;
  const int threads = width >= 256 ? 256 : (width >= 128 ? 128 : 64);
  const dim3 grid(T, (width + threads - 1) / threads);
  DISTIE_DISPATCH(x_dtype, X, DISTIE_DISPATCH(g_dtype, G, DISTIE_DISPATCH(out_dtype, O,
      head_gate_kernel<X, G, O><<<grid, threads, 0, stream>>>(
          static_cast<const X*>(x), ldh, E, static_cast<const G*>(gates), ldg, static_cast<O*>(out), width))));
  return launch_status();
}
