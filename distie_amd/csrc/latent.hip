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
// `down` may be `slices` partial sums of the product, `slice_stride` elements apart (added in order while the row is
// read into LDS, where both norms and the rotation find it).
template <typename O, typename C>
__global__ void latent_norm_rope_write_kernel(const float* __restrict__ down, int slices, int64_t slice_stride, int64_t ld,
                                              int q_rank, const float* __restrict__ q_weight, int kv_rank,
                                              const float* __restrict__ kv_weight, float eps, int rot_dim,
                                              const float2* __restrict__ table, float magnitude, int neighbours,
                                              O* __restrict__ latent, C* __restrict__ k_cache, C* __restrict__ v_cache,
                                              const int32_t* __restrict__ slots, int P, int DP, int write) {
  extern __shared__ float row[];               // q_rank + kv_rank + rot_dim values
  __shared__ float scratch[16];
  const int64_t t = blockIdx.x;
  const int width = q_rank + kv_rank + rot_dim;
  for (int c = threadIdx.x; c < width; c += blockDim.x) row[c] = sum_strided(down + t * ld + c, slices, slice_stride);
  __syncthreads();
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

// What a fused call adds behind a head's product, for latent attention's queries: the 2 * pairs columns at `offset_in`
// of the head's input, turned by the token's angle, go to the columns behind the product's N results, and the rest of
// the head's `lo` output columns is zeroed. pairs 0: nothing of this.
struct QueryTail {
  const float2* table;        // [T, pairs] cosine and sine
  float magnitude;
  int pairs, offset_in, neighbours;
};

// SLICED: x is float32 [slices, T, H * lx], partial sums of the product that made it, added in order and rounded to
// bfloat16 once (what a kernel that adds them up in front of this one would hand over).
template <bool SLICED>
__device__ __forceinline__ float load_x(const void* x, int64_t at, int slices, int64_t slice_stride) {
  if constexpr (SLICED) return sum_strided(static_cast<const float*>(x) + at, slices, slice_stride);
  else return to_float(static_cast<const bf16_t*>(x)[at]);
}

template <int WT, int WN, int NB, bool SLICED>
__global__ void __launch_bounds__(64 * WT * WN)
heads_linear_mfma_kernel(const void* __restrict__ x, int slices, int64_t slice_stride, int lx, const bf16_t* __restrict__ w,
                         bf16_t* __restrict__ out, int lo, int T, int H, int N, int K, QueryTail tail) {
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int h = blockIdx.z;
  const int t0 = (blockIdx.y * WT + wave / WN) * 32;
  const int n0 = (blockIdx.x * WN + wave % WN) * 32 * NB;
  if (t0 < T && n0 < N) {
    const int r = lane % 32, kk = 8 * (lane / 32);
    const bool t_in = t0 + r < T;
    const int64_t x_at = (static_cast<int64_t>(t_in ? t0 + r : t0) * H + h) * lx + kk;
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
        a[s] = hl_bf16x8{};
        if (t_in && k_in) {
          if constexpr (SLICED) {
            const float* xf = static_cast<const float*>(x) + x_at + k;
            float4 lo4 = *reinterpret_cast<const float4*>(xf), hi4 = *reinterpret_cast<const float4*>(xf + 4);
            for (int q = 1; q < slices; ++q) {
              const float4 l2 = *reinterpret_cast<const float4*>(xf + q * slice_stride);
              const float4 h2 = *reinterpret_cast<const float4*>(xf + q * slice_stride + 4);
              lo4.x += l2.x, lo4.y += l2.y, lo4.z += l2.z, lo4.w += l2.w;
              hi4.x += h2.x, hi4.y += h2.y, hi4.z += h2.z, hi4.w += h2.w;
            }
            a[s][0] = static_cast<bf16_t>(lo4.x), a[s][1] = static_cast<bf16_t>(lo4.y);
            a[s][2] = static_cast<bf16_t>(lo4.z), a[s][3] = static_cast<bf16_t>(lo4.w);
            a[s][4] = static_cast<bf16_t>(hi4.x), a[s][5] = static_cast<bf16_t>(hi4.y);
            a[s][6] = static_cast<bf16_t>(hi4.z), a[s][7] = static_cast<bf16_t>(hi4.w);
          } else {
            a[s] = *reinterpret_cast<const hl_bf16x8*>(static_cast<const bf16_t*>(x) + x_at + k);
          }
        }
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
  if (tail.pairs == 0 || blockIdx.x != 0) return;
  // the workgroup's rows of x, this head: the turned part behind the product's columns, zeros behind that
  const int first = blockIdx.y * WT * 32;
  const int rows = min(WT * 32, T - first);
  for (int i = threadIdx.x; i < rows * tail.pairs; i += blockDim.x) {
    const int t = first + i / tail.pairs, j = i % tail.pairs;
    const int a = tail.neighbours ? 2 * j : j, b = tail.neighbours ? 2 * j + 1 : j + tail.pairs;
    const float2 cs = tail.table[static_cast<int64_t>(t) * tail.pairs + j];
    const int64_t in = (static_cast<int64_t>(t) * H + h) * lx + tail.offset_in;
    // (the unfused path rounds the summed product before it is turned)
    const float u = to_float(static_cast<bf16_t>(load_x<SLICED>(x, in + a, slices, slice_stride)));
    const float v = to_float(static_cast<bf16_t>(load_x<SLICED>(x, in + b, slices, slice_stride)));
    bf16_t* to = out + (static_cast<int64_t>(t) * H + h) * lo + N;
    to[a] = static_cast<bf16_t>(u * cs.x * tail.magnitude - v * cs.y * tail.magnitude);
    to[b] = static_cast<bf16_t>(v * cs.x * tail.magnitude + u * cs.y * tail.magnitude);
  }
  const int pad = lo - N - 2 * tail.pairs;
  for (int i = threadIdx.x; i < rows * pad; i += blockDim.x) {
    const int t = first + i / pad;
    out[(static_cast<int64_t>(t) * H + h) * lo + N + 2 * tail.pairs + i % pad] = static_cast<bf16_t>(0.f);
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

// bfloat16 with 16-byte loads and stores: eight of a head's columns a thread (E and ldh multiples of 8)
__global__ void head_gate_bf16x8_kernel(const bf16_t* __restrict__ x, int ldh, int E, const bf16_t* __restrict__ gates,
                                        int64_t ldg, bf16_t* __restrict__ out, int width, int T) {
  const int per_row = width / 8;
  const int64_t total = static_cast<int64_t>(T) * per_row;
  for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < total;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int64_t t = i / per_row;
    const int c = 8 * static_cast<int>(i % per_row);
    const int head = c / E, e = c % E;
    const uint4 raw = *reinterpret_cast<const uint4*>(x + (t * (width / E) + head) * ldh + e);
    const float g = sigmoidf(to_float(gates[t * ldg + head]));
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
    uint32_t o[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const bf16_t lo = static_cast<bf16_t>(__uint_as_float(w[k] << 16) * g);
      const bf16_t hi = static_cast<bf16_t>(__uint_as_float(w[k] & 0xffff0000u) * g);
      o[k] = static_cast<uint32_t>(__builtin_bit_cast(uint16_t, lo)) | (static_cast<uint32_t>(__builtin_bit_cast(uint16_t, hi)) << 16);
    }
    *reinterpret_cast<uint4*>(out + t * width + c) = uint4{o[0], o[1], o[2], o[3]};
  }
}

}  // namespace

// the widest row (q_rank + kv_rank + rot_dim) that the kernel stages
extern "C" int distie_latent_norm_max_width() { return 12288; }

extern "C" int distie_latent_norm_rope_write(const float* down, int slices, int64_t ld, int q_rank, const float* q_weight, int kv_rank,
                                             const float* kv_weight, float eps, int rot_dim, const void* table,
                                             float magnitude, int neighbours, void* latent, int out_dtype, void* k_cache,
                                             void* v_cache, int cache_dtype, const int32_t* slots, int T, int P, int DP,
                                             int write, hipStream_t stream) {
  if (T <= 0) return 0;
  if (q_rank < 0 || kv_rank < 1 || rot_dim < 0 || rot_dim % 2 || ld < static_cast<int64_t>(q_rank) + kv_rank + rot_dim ||
      slices < 1 || q_rank + kv_rank + rot_dim > 12288 ||
      (q_rank > 0 && (q_weight == nullptr || latent == nullptr)) || kv_weight == nullptr ||
      (write && (k_cache == nullptr || v_cache == nullptr || slots == nullptr || P < 1 || DP < kv_rank + rot_dim)))
    return DISTIE_BAD_ARGUMENT;
  const int widest = q_rank > kv_rank ? q_rank : kv_rank;
  const int threads = widest >= 256 ? 256 : (widest >= 128 ? 128 : 64);
  DISTIE_DISPATCH(out_dtype, O, DISTIE_DISPATCH(cache_dtype, C,
      latent_norm_rope_write_kernel<O, C><<<T, threads, sizeof(float) * (q_rank + kv_rank + rot_dim), stream>>>(
          down, slices, static_cast<int64_t>(T) * ld, ld, q_rank, q_weight, kv_rank, kv_weight, eps, rot_dim, static_cast<const float2*>(table), magnitude,
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

static bool heads_linear_mfma_fits(const void* x, int dtype, const void* w, int w_dtype, int lx, int K, int slices) {
  const bool x_ok = slices > 1 ? (dtype == DISTIE_F32 && lx % 4 == 0) : (dtype == DISTIE_BF16 && lx % 8 == 0);
  return x_ok && w_dtype == DISTIE_BF16 && K % 8 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 &&
         reinterpret_cast<uintptr_t>(w) % 16 == 0;
}

// x: bfloat16 [T, H * lx], or (slices > 1) float32 [slices, T, H * lx]
static int heads_linear_mfma(const void* x, int slices, int lx, const void* w, void* out, int lo, int T, int H, int N, int K,
                             QueryTail tail, hipStream_t stream) {
  const bf16_t* wb = static_cast<const bf16_t*>(w);
  bf16_t* ob = static_cast<bf16_t*>(out);
  const int64_t stride = static_cast<int64_t>(T) * H * lx;
  if (T <= 32) {
    const dim3 grid((N + 127) / 128, 1, H);
    if (slices > 1) heads_linear_mfma_kernel<1, 4, 1, true><<<grid, 256, 0, stream>>>(x, slices, stride, lx, wb, ob, lo, T, H, N, K, tail);
    else heads_linear_mfma_kernel<1, 4, 1, false><<<grid, 256, 0, stream>>>(x, 1, 0, lx, wb, ob, lo, T, H, N, K, tail);
  } else {
    const dim3 grid((N + 127) / 128, (T + 63) / 64, H);
    if (grid.y > 65535) return DISTIE_BAD_ARGUMENT;
    if (slices > 1) heads_linear_mfma_kernel<2, 2, 2, true><<<grid, 256, 0, stream>>>(x, slices, stride, lx, wb, ob, lo, T, H, N, K, tail);
    else heads_linear_mfma_kernel<2, 2, 2, false><<<grid, 256, 0, stream>>>(x, 1, 0, lx, wb, ob, lo, T, H, N, K, tail);
  }
  return launch_status();
}

// Latent attention's queries in one launch, bfloat16 on the matrix cores: head h's first K input columns times
// w[h] ([N, K]) into the first N of its `lo` output columns, the next 2 * pairs input columns turned by the token's
// angle into the columns behind them, zeros in the rest. x: bfloat16 [T, H * lx] or float32 [slices, T, H * lx].
// Returns DISTIE_BAD_ARGUMENT for what the kernel does not take (the caller then composes the unfused operations).
extern "C" int distie_latent_queries(const void* x, int dtype, int slices, int lx, const void* w, int w_dtype, void* out,
                                     int lo, int T, int H, int N, int K, int pairs, const void* table, float magnitude,
                                     int neighbours, hipStream_t stream) {
  if (T <= 0) return 0;
  if (H < 1 || N < 1 || K < 1 || pairs < 1 || slices < 1 || H > 65535 || lx < K + 2 * pairs || lo < N + 2 * pairs ||
      table == nullptr || !heads_linear_mfma_fits(x, dtype, w, w_dtype, lx, K, slices) || (slices == 1 && dtype != DISTIE_BF16))
    return DISTIE_BAD_ARGUMENT;
  return heads_linear_mfma(x, slices, lx, w, out, lo, T, H, N, K,
                           QueryTail{static_cast<const float2*>(table), magnitude, pairs, K, neighbours}, stream);
}

extern "C" int distie_heads_linear(const void* x, int dtype, int lx, const void* w, int w_dtype, void* out, int lo, int T,
                                   int H, int N, int K, hipStream_t stream) {
  if (T <= 0) return 0;
  if (H < 1 || N < 1 || K < 1 || lx < K || lo < N || H > 65535) return DISTIE_BAD_ARGUMENT;
  if (heads_linear_mfma_fits(x, dtype, w, w_dtype, lx, K, 1))
    return heads_linear_mfma(x, 1, lx, w, out, lo, T, H, N, K, QueryTail{nullptr, 1.f, 0, 0, 0}, stream);
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
  if (x_dtype == DISTIE_BF16 && g_dtype == DISTIE_BF16 && out_dtype == DISTIE_BF16 && E % 8 == 0 && ldh % 8 == 0 &&
      reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0) {
    const int64_t pieces = static_cast<int64_t>(T) * (width / 8);
    const int blocks8 = static_cast<int>(pieces / 256 + 1 < 16384 ? pieces / 256 + 1 : 16384);
    head_gate_bf16x8_kernel<<<blocks8, 256, 0, stream>>>(static_cast<const bf16_t*>(x), ldh, E,
                                                         static_cast<const bf16_t*>(gates), ldg, static_cast<bf16_t*>(out), width, T);
    return launch_status();
  }
  const int threads = width >= 256 ? 256 : (width >= 128 ? 128 : 64);
  const dim3 grid(T, (width + threads - 1) / threads);
  DISTIE_DISPATCH(x_dtype, X, DISTIE_DISPATCH(g_dtype, G, DISTIE_DISPATCH(out_dtype, O,
      head_gate_kernel<X, G, O><<<grid, threads, 0, stream>>>(
          static_cast<const X*>(x), ldh, E, static_cast<const G*>(gates), ldg, static_cast<O*>(out), width))));
  return launch_status();
}
