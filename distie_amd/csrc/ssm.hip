// Kernels of the selective state-space mixer in its scalar-decay form, of the gated norm behind it, and of gated
// activations other than silu.
//
// Per head h (group g = h / (H / G) of B and C), with d = softplus(dt + dt_bias[h]) and a = exp(-exp(a_log[h]) * d):
//     S <- a S + d * B x^T   (S is N x P, float32),     y = S^T C + skip[h] * x.
// xbc [T, ld] holds x (H x P), then B (G x N), then C (G x N); dt [T, ldd] one number a head; state float32
// [slots, H, N, P]. Softplus, both exponentials, the state and every sum are float32 in either precision.
//
// A step is a flattened batch: request b's new tokens are rows cu_q[b] .. cu_q[b+1]-1, its state row state_slots[b].
#include "common.h"

namespace {

__device__ __forceinline__ float sigmoidf(float x) { return 1.f / (1.f + expf(-x)); }
__device__ __forceinline__ float softplusf(float x) { return x > 20.f ? x : log1pf(expf(x)); }
__device__ __forceinline__ float activate(float z, int kind) {
  if (kind == 0) {
    const float p = fmaxf(z, 0.f);
    return p * p;
  }
  if (kind == 1) return z / (1.f + expf(-z));
  if (kind == 2) return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
  return fmaxf(z, 0.f);
}

// ---------------------------------------------------------------------------------------------------
// Token by token. A block owns 64 columns p of one head of one request and walks the request's rows in order; thread
// (p, part) keeps rows n = part, part + PARTS, ... of its column in registers, the PARTS partial sums of a column meet
// in LDS. The next row's inputs are asked for before this row's are used.
template <typename X, int PARTS, int ROWS>
__global__ void __launch_bounds__(64 * PARTS)
ssm_scan_kernel(const X* __restrict__ xbc, int64_t ld, const X* __restrict__ dt, int64_t ldd,
                const float* __restrict__ dt_bias, const float* __restrict__ a_log, const float* __restrict__ skip,
                float* __restrict__ state, float* __restrict__ out, const int32_t* __restrict__ cu_q,
                const int32_t* __restrict__ state_slots, int H, int P, int N, int G) {
  __shared__ float b_s[PARTS * ROWS], c_s[PARTS * ROWS];
  __shared__ float partial[PARTS][64];
  const int b = blockIdx.x, head = blockIdx.y;
  const int lane = threadIdx.x % 64, part = threadIdx.x / 64;
  const int p = blockIdx.z * 64 + lane;
  const int group = head / (H / G);
  const int first = cu_q[b], last = cu_q[b + 1];
  if (first >= last) return;
  const float rate = -expf(a_log[head]);
  const float bias = dt_bias[head], through = skip[head];
  float* own = state + (static_cast<int64_t>(state_slots[b]) * H + head) * N * P;
  float s[ROWS];
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    const int n = part + r * PARTS;
    s[r] = (n < N && p < P) ? own[static_cast<int64_t>(n) * P + p] : 0.f;
  }
  const int64_t b_at = static_cast<int64_t>(H) * P + static_cast<int64_t>(group) * N;
  const int64_t c_at = b_at + static_cast<int64_t>(G) * N;
  for (int t = first; t < last; ++t) {
    const X* row = xbc + static_cast<int64_t>(t) * ld;
    __syncthreads();
    for (int n = threadIdx.x; n < N; n += blockDim.x) {
      b_s[n] = to_float(row[b_at + n]);
      c_s[n] = to_float(row[c_at + n]);
    }
    const float x = p < P ? to_float(row[head * P + p]) : 0.f;
    const float d = softplusf(to_float(dt[static_cast<int64_t>(t) * ldd + head]) + bias);
    const float a = expf(rate * d);
    __syncthreads();
    const float dx = d * x;
    float y = 0.f;
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
      const int n = part + r * PARTS;
      if (n < N) {
        s[r] = a * s[r] + b_s[n] * dx;
        y += s[r] * c_s[n];
      }
    }
    partial[part][lane] = y;
    __syncthreads();
    if (part == 0 && p < P) {
      float total = 0.f;
#pragma unroll
      for (int q = 0; q < PARTS; ++q) total += partial[q][lane];
      out[(static_cast<int64_t>(t) * H + head) * P + p] = total + through * x;
    }
  }
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    const int n = part + r * PARTS;
    if (n < N && p < P) own[static_cast<int64_t>(n) * P + p] = s[r];
  }
}

// ---------------------------------------------------------------------------------------------------
// The same recurrence over portions of prompts, in chunks of L rows that run side by side. With l_i the running sum
// of ln a inside the chunk (l_i <= 0, falling), S the state in front of the chunk:
//   sums:     U[n][p]  = sum_j exp(l_L - l_j) d_j B_j[n] x_j[p],  total = exp(l_L)            (each chunk alone)
//   states:   S_next   = total * S + U, chunk after chunk; S (the state in front) takes U's place in the scratch
//   pairs:    (C_i . B_j) for the chunk's rows, once for every group of heads that shares B and C
//   outputs:  y_i[p]   = exp(l_i) sum_n C_i[n] S[n][p] + sum_{j<=i} exp(l_i - l_j) d_j (C_i . B_j) x_j[p] + skip x_i[p]
// Every exponent is <= 0 and no quotient of decays is formed. Float32 throughout, FMAs on tiles held in LDS; a chunk's
// table entry is {request, first row, rows, unused}.
constexpr int SSM_L = 64;
constexpr int SSM_PAD = SSM_L + 1;

// The products of the chunks' tiles run on v_mfma_f32_32x32x2_f32 (float32 operands, products and sums): a lane gives
// A[row = lane % 32][k = lane / 32] and B[k = lane / 32][column = lane % 32], both read from LDS tiles whose rows are an
// odd number of words apart, and holds, in register v, the sum for row tile_row(v, lane) and column lane % 32.
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float ssm_floatx16;
__device__ __forceinline__ int tile_row(int v, int lane) { return 8 * (v / 4) + 4 * (lane / 32) + v % 4; }

// d_j and l_j of a chunk's rows for one head, into LDS (thread 0 adds the logarithms in order)
template <typename X>
__device__ __forceinline__ void chunk_decays(const X* __restrict__ dt, int64_t ldd, int first, int rows, int head,
                                             float bias, float rate, float* d_s, float* l_s) {
  for (int j = threadIdx.x; j < SSM_L; j += blockDim.x)
    d_s[j] = j < rows ? softplusf(to_float(dt[static_cast<int64_t>(first + j) * ldd + head]) + bias) : 0.f;
  __syncthreads();
  if (threadIdx.x == 0) {
    float l = 0.f;
    for (int j = 0; j < SSM_L; ++j) {
      l += rate * d_s[j];
      l_s[j] = l;
    }
  }
  __syncthreads();
}

// blockIdx = (chunk, head, 64 columns p): U and the chunk's total decay
template <typename X>
__global__ void __launch_bounds__(256)
ssm_chunk_sums_kernel(const X* __restrict__ xbc, int64_t ld, const X* __restrict__ dt, int64_t ldd,
                      const float* __restrict__ dt_bias, const float* __restrict__ a_log, float* __restrict__ scratch,
                      float* __restrict__ totals, const int4* __restrict__ chunks, int H, int P, int N, int G) {
  __shared__ float d_s[SSM_L], l_s[SSM_L];
  __shared__ float x_s[SSM_L][SSM_PAD];     // [row][p], times the row's factor
  __shared__ float b_s[SSM_L][SSM_PAD];     // [row][n of this pass]
  const int chunk = blockIdx.x, head = blockIdx.y, p0 = blockIdx.z * 64;
  const int4 entry = chunks[chunk];
  const int first = entry.y, rows = entry.z;
  const int group = head / (H / G);
  chunk_decays(dt, ldd, first, rows, head, dt_bias[head], -expf(a_log[head]), d_s, l_s);
  const float l_end = l_s[rows - 1];
  if (threadIdx.x == 0 && blockIdx.z == 0) totals[static_cast<int64_t>(chunk) * H + head] = expf(l_end);
  for (int i = threadIdx.x; i < SSM_L * 64; i += 256) {
    const int j = i / 64, p = i % 64;
    x_s[j][p] = (j < rows && p0 + p < P)
                    ? expf(l_end - l_s[j]) * d_s[j] * to_float(xbc[static_cast<int64_t>(first + j) * ld + head * P + p0 + p])
                    : 0.f;
  }
  const int64_t b_at = static_cast<int64_t>(H) * P + static_cast<int64_t>(group) * N;
  float* u = scratch + (static_cast<int64_t>(chunk) * H + head) * N * P;
  // a wave: 32 rows n by 32 columns p of the pass's 64 x 64, on float32 matrix products over the rows j
  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  const int nb = 32 * (wave / 2), pb = 32 * (wave % 2);
  for (int n0 = 0; n0 < N; n0 += SSM_L) {
    __syncthreads();
    for (int i = threadIdx.x; i < SSM_L * SSM_L; i += 256) {
      const int j = i / SSM_L, n = i % SSM_L;
      b_s[j][n] = (j < rows && n0 + n < N) ? to_float(xbc[static_cast<int64_t>(first + j) * ld + b_at + n0 + n]) : 0.f;
    }
    __syncthreads();
    ssm_floatx16 acc = {};
    for (int j = 0; j < SSM_L; j += 2)
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(b_s[j + lane / 32][nb + lane % 32], x_s[j + lane / 32][pb + lane % 32],
                                                 acc, 0, 0, 0);
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int n = n0 + nb + tile_row(v, lane), pc = p0 + pb + lane % 32;
      if (n < N && pc < P) u[static_cast<int64_t>(n) * P + pc] = acc[v];
    }
  }
}

// a thread an element of a (request, head)'s state: walks the request's chunks in order; the scratch gets the state
// in front of each chunk, the state tensor the one behind the last
__global__ void ssm_chunk_states_kernel(float* __restrict__ scratch, const float* __restrict__ totals,
                                        float* __restrict__ state, const int32_t* __restrict__ first_chunk,
                                        const int32_t* __restrict__ state_slots, int H, int64_t size) {
  const int b = blockIdx.x, head = blockIdx.y;
  const int begin = first_chunk[b], end = first_chunk[b + 1];
  if (begin >= end) return;
  float* own = state + (static_cast<int64_t>(state_slots[b]) * H + head) * size;
  for (int64_t i = static_cast<int64_t>(blockIdx.z) * blockDim.x + threadIdx.x; i < size;
       i += static_cast<int64_t>(gridDim.z) * blockDim.x) {
    float s = own[i];
    for (int c = begin; c < end; ++c) {
      float* u = scratch + (static_cast<int64_t>(c) * H + head) * size + i;
      const float next = totals[static_cast<int64_t>(c) * H + head] * s + *u;
      *u = s;
      s = next;
    }
    own[i] = s;
  }
}

// blockIdx = (chunk, group): (C_i . B_j) for the chunk's rows i and j, the same for every head of the group
// -> pairs [chunks, G, L, L]. A wave: 32 rows i by 32 columns j.
template <typename X>
__global__ void __launch_bounds__(256)
ssm_chunk_pairs_kernel(const X* __restrict__ xbc, int64_t ld, float* __restrict__ pairs, const int4* __restrict__ chunks,
                       int H, int P, int N, int G) {
  __shared__ float c_s[SSM_L][SSM_PAD];       // [i][n of this pass]
  __shared__ float b_s[SSM_L][SSM_PAD];       // [j][n of this pass]
  const int chunk = blockIdx.x, group = blockIdx.y;
  const int4 entry = chunks[chunk];
  const int first = entry.y, rows = entry.z;
  const int64_t b_at = static_cast<int64_t>(H) * P + static_cast<int64_t>(group) * N;
  const int64_t c_at = b_at + static_cast<int64_t>(G) * N;
  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  const int ib = 32 * (wave / 2), jb = 32 * (wave % 2);
  ssm_floatx16 acc = {};
  for (int n0 = 0; n0 < N; n0 += SSM_L) {
    __syncthreads();
    for (int i = threadIdx.x; i < SSM_L * SSM_L; i += 256) {
      const int j = i / SSM_L, n = i % SSM_L;
      const bool in = j < rows && n0 + n < N;
      b_s[j][n] = in ? to_float(xbc[static_cast<int64_t>(first + j) * ld + b_at + n0 + n]) : 0.f;
      c_s[j][n] = in ? to_float(xbc[static_cast<int64_t>(first + j) * ld + c_at + n0 + n]) : 0.f;
    }
    __syncthreads();
    for (int n = 0; n < SSM_L; n += 2)
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(c_s[ib + lane % 32][n + lane / 32], b_s[jb + lane % 32][n + lane / 32],
                                                 acc, 0, 0, 0);
  }
  float* to = pairs + (static_cast<int64_t>(chunk) * G + group) * SSM_L * SSM_L;
#pragma unroll
  for (int v = 0; v < 16; ++v) to[(ib + tile_row(v, lane)) * SSM_L + jb + lane % 32] = acc[v];
}

// blockIdx = (chunk, head, 64 columns p): the chunk's outputs from the state in front of it and its own rows
template <typename X>
__global__ void __launch_bounds__(256)
ssm_chunk_outputs_kernel(const X* __restrict__ xbc, int64_t ld, const X* __restrict__ dt, int64_t ldd,
                         const float* __restrict__ dt_bias, const float* __restrict__ a_log,
                         const float* __restrict__ skip, const float* __restrict__ scratch,
                         const float* __restrict__ pairs, float* __restrict__ out, const int4* __restrict__ chunks, int H,
                         int P, int N, int G) {
  __shared__ float d_s[SSM_L], l_s[SSM_L];
  __shared__ float a_s[SSM_L][SSM_PAD];     // [i][j]: the pair's weight
  __shared__ float t_s[SSM_L][SSM_PAD];     // a tile of C [i][n], then of x [j][p]
  __shared__ float u_s[SSM_L][SSM_PAD];     // a tile of the state [n][p]
  const int chunk = blockIdx.x, head = blockIdx.y, p0 = blockIdx.z * 64;
  const int4 entry = chunks[chunk];
  const int first = entry.y, rows = entry.z;
  const int group = head / (H / G);
  chunk_decays(dt, ldd, first, rows, head, dt_bias[head], -expf(a_log[head]), d_s, l_s);
  const int64_t c_at = static_cast<int64_t>(H) * P + static_cast<int64_t>(G + group) * N;
  const float* s_in = scratch + (static_cast<int64_t>(chunk) * H + head) * N * P;
  const int col = threadIdx.x % 64, part = threadIdx.x / 64;     // a thread: column col, rows part, part + 4, ...
  // the pairs' weights (zero above the diagonal): (C_i . B_j) exp(l_i - l_j) d_j
  const float* pair = pairs + (static_cast<int64_t>(chunk) * G + group) * SSM_L * SSM_L;
#pragma unroll
  for (int r = 0; r < SSM_L / 4; ++r) {
    const int i = part + 4 * r, j = col;
    a_s[i][j] = (j <= i && i < rows) ? pair[i * SSM_L + j] * expf(l_s[i] - l_s[j]) * d_s[j] : 0.f;
  }
  // a wave: 32 rows i by 32 columns p of the outputs
  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  const int ib = 32 * (wave / 2), pb = 32 * (wave % 2);
  ssm_floatx16 y = {};                 // the state's share: sum_n C_i[n] S[n][p]
  for (int n0 = 0; n0 < N; n0 += SSM_L) {
    __syncthreads();
    for (int i = threadIdx.x; i < SSM_L * SSM_L; i += 256) {
      const int j = i / SSM_L, n = i % SSM_L;
      t_s[j][n] = (j < rows && n0 + n < N) ? to_float(xbc[static_cast<int64_t>(first + j) * ld + c_at + n0 + n]) : 0.f;
    }
    for (int i = threadIdx.x; i < SSM_L * 64; i += 256) {
      const int n = i / 64, p = i % 64;
      u_s[n][p] = (n0 + n < N && p0 + p < P) ? s_in[static_cast<int64_t>(n0 + n) * P + p0 + p] : 0.f;
    }
    __syncthreads();
    for (int n = 0; n < SSM_L; n += 2)
      y = __builtin_amdgcn_mfma_f32_32x32x2f32(t_s[ib + lane % 32][n + lane / 32], u_s[n + lane / 32][pb + lane % 32], y,
                                               0, 0, 0);
  }
  __syncthreads();
  for (int i = threadIdx.x; i < SSM_L * 64; i += 256) {
    const int j = i / 64, p = i % 64;
    t_s[j][p] = (j < rows && p0 + p < P) ? to_float(xbc[static_cast<int64_t>(first + j) * ld + head * P + p0 + p]) : 0.f;
  }
  __syncthreads();
  // the chunk's own rows: sum_{j <= i} a[i][j] x_j[p]; rows j beyond the wave's last i have weight zero
  ssm_floatx16 own = {};
  for (int j = 0; j < ib + 32; j += 2)
    own = __builtin_amdgcn_mfma_f32_32x32x2f32(a_s[ib + lane % 32][j + lane / 32], t_s[j + lane / 32][pb + lane % 32], own,
                                               0, 0, 0);
  const float through = skip[head];
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int i = ib + tile_row(v, lane), pc = pb + lane % 32;
    if (i < rows && p0 + pc < P)
      out[(static_cast<int64_t>(first + i) * H + head) * P + p0 + pc] = expf(l_s[i]) * y[v] + own[v] + through * t_s[i][pc];
  }
}

// ---------------------------------------------------------------------------------------------------
// out = (x * gate) / sqrt(mean((x * gate)^2) + eps) * weight, the mean over each run of N columns of a row by itself
// (`groups` runs side by side in a row of x, of the gates and of out); gate = g * sigmoid(g) (`silu`) or sigmoid(g);
// the weight is each column's own, [groups * N]. The gate stands in front of the norm. One block a (row, run).
// STAGED: the gated values of the run wait in LDS between the two walks, so x and the gates are read once.
template <bool STAGED, typename W, typename G, typename O>
__global__ void gate_rmsnorm_kernel(const float* __restrict__ x, const W* __restrict__ weight, float eps,
                                    const G* __restrict__ gates, int64_t ldg, O* __restrict__ out, int N, int groups,
                                    int silu) {
  extern __shared__ float held[];
  __shared__ float scratch[16];
  const int64_t t = blockIdx.x;
  const int64_t at = static_cast<int64_t>(blockIdx.y) * N;
  const float* row = x + t * N * groups + at;
  const G* g = gates + t * ldg + at;
  float sq = 0.f;
  for (int c = threadIdx.x; c < N; c += blockDim.x) {
    const float z = to_float(g[c]);
    const float v = row[c] * (silu ? z * sigmoidf(z) : sigmoidf(z));
    if constexpr (STAGED) held[c] = v;
    sq += v * v;
  }
  sq = block_sum(sq, scratch);
  const float scale = 1.f / sqrtf(sq / N + eps);
  for (int c = threadIdx.x; c < N; c += blockDim.x) {
    float v;
    if constexpr (STAGED) {
      v = held[c];                       // (written by this same thread)
    } else {
      const float z = to_float(g[c]);
      v = row[c] * (silu ? z * sigmoidf(z) : sigmoidf(z));
    }
    out[t * N * groups + at + c] = from_float<O>(v * scale * to_float(weight[at + c]));
  }
}

// out[t, i] = act(gate_up[t, i]) * gate_up[t, I + i], the input a sum of `slices` partial sums
template <typename X, typename O>
__global__ void glu_mul_kernel(const X* __restrict__ gate_up, int slices, int64_t slice_stride, O* __restrict__ out,
                               int rows, int inter, int kind) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= static_cast<int64_t>(rows) * inter) return;
  const int64_t t = i / inter, c = i % inter;
  const float g = sum_strided(gate_up + t * 2 * inter + c, slices, slice_stride);
  const float u = sum_strided(gate_up + t * 2 * inter + inter + c, slices, slice_stride);
  out[i] = from_float<O>(activate(g, kind) * u);
}

// bfloat16 in and out, one slice, inter a multiple of 8: 16-byte loads and stores
__global__ void glu_mul_bf16x8_kernel(const uint4* __restrict__ gate_up, uint4* __restrict__ out, int64_t rows,
                                      int inter8, int kind) {
  const int64_t total = rows * inter8;
  for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < total;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int64_t r = i / inter8;
    const int c = static_cast<int>(i % inter8);
    const uint4 g4 = gate_up[r * 2 * inter8 + c];
    const uint4 u4 = gate_up[r * 2 * inter8 + inter8 + c];
    const uint32_t gw[4] = {g4.x, g4.y, g4.z, g4.w}, uw[4] = {u4.x, u4.y, u4.z, u4.w};
    uint32_t ow[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float g0 = __uint_as_float(gw[e] << 16), g1 = __uint_as_float(gw[e] & 0xffff0000u);
      const float u0 = __uint_as_float(uw[e] << 16), u1 = __uint_as_float(uw[e] & 0xffff0000u);
      const bf16_t lo = static_cast<bf16_t>(activate(g0, kind) * u0);
      const bf16_t hi = static_cast<bf16_t>(activate(g1, kind) * u1);
      ow[e] = static_cast<uint32_t>(__builtin_bit_cast(uint16_t, lo)) |
              (static_cast<uint32_t>(__builtin_bit_cast(uint16_t, hi)) << 16);
    }
    out[i] = uint4{ow[0], ow[1], ow[2], ow[3]};
  }
}

}  // namespace

extern "C" int distie_ssm_scan_max_state() { return 256; }

extern "C" int distie_ssm_scan(const void* xbc, int dtype, int64_t ld, const void* dt, int64_t ldd, const float* dt_bias,
                               const float* a_log, const float* skip, float* state, float* out, const int32_t* cu_q,
                               const int32_t* state_slots, int B, int H, int P, int N, int G, hipStream_t stream) {
  if (B <= 0) return 0;
  if (H < 1 || P < 1 || N < 1 || G < 1 || H % G || N > 256 || H > 65535 || ldd < H ||
      ld < static_cast<int64_t>(H) * P + 2 * static_cast<int64_t>(G) * N)
    return DISTIE_BAD_ARGUMENT;
  const dim3 grid(B, H, (P + 63) / 64);
#define DISTIE_SSM(PARTS, ROWS)                                                                                     \
  DISTIE_DISPATCH(dtype, X, ssm_scan_kernel<X, PARTS, ROWS><<<grid, 64 * PARTS, 0, stream>>>(                       \
      static_cast<const X*>(xbc), ld, static_cast<const X*>(dt), ldd, dt_bias, a_log, skip, state, out, cu_q,       \
      state_slots, H, P, N, G))
  if (N <= 32) {
    DISTIE_SSM(4, 8);
  } else if (N <= 64) {
    DISTIE_SSM(4, 16);
  } else if (N <= 128) {
    DISTIE_SSM(4, 32);
  } else {
    DISTIE_SSM(8, 32);
  }
#undef DISTIE_SSM
  return launch_status();
}

extern "C" int distie_ssm_scan_chunk_rows() { return SSM_L; }

// scratch float32 [chunks, H, N, P], totals float32 [chunks, H], pairs float32 [chunks, G, L, L]
extern "C" int distie_ssm_scan_chunked(const void* xbc, int dtype, int64_t ld, const void* dt, int64_t ldd,
                                       const float* dt_bias, const float* a_log, const float* skip, float* state,
                                       float* out, float* scratch, float* totals, float* pairs, const void* chunks,
                                       const int32_t* first_chunk, const int32_t* state_slots, int count, int B, int H,
                                       int P, int N, int G, hipStream_t stream) {
  if (B <= 0 || count <= 0) return 0;
  if (H < 1 || P < 1 || N < 1 || G < 1 || H % G || H > 65535 || ldd < H || pairs == nullptr ||
      ld < static_cast<int64_t>(H) * P + 2 * static_cast<int64_t>(G) * N)
    return DISTIE_BAD_ARGUMENT;
  const dim3 grid(count, H, (P + 63) / 64);
  const int64_t size = static_cast<int64_t>(N) * P;
  const int parts = static_cast<int>((size + 255) / 256 < 64 ? (size + 255) / 256 : 64);
  DISTIE_DISPATCH(dtype, X, {
    ssm_chunk_sums_kernel<X><<<grid, 256, 0, stream>>>(static_cast<const X*>(xbc), ld, static_cast<const X*>(dt), ldd,
                                                      dt_bias, a_log, scratch, totals, static_cast<const int4*>(chunks),
                                                      H, P, N, G);
    ssm_chunk_pairs_kernel<X><<<dim3(count, G), 256, 0, stream>>>(static_cast<const X*>(xbc), ld, pairs,
                                                                    static_cast<const int4*>(chunks), H, P, N, G);
    ssm_chunk_states_kernel<<<dim3(B, H, parts), 256, 0, stream>>>(scratch, totals, state, first_chunk, state_slots, H, size);
    ssm_chunk_outputs_kernel<X><<<grid, 256, 0, stream>>>(static_cast<const X*>(xbc), ld, static_cast<const X*>(dt), ldd,
                                                         dt_bias, a_log, skip, scratch, pairs, out,
                                                         static_cast<const int4*>(chunks), H, P, N, G);
  });
  return launch_status();
}

extern "C" int distie_gate_rmsnorm(const float* x, const void* weight, int w_dtype, float eps, const void* gates,
                                   int g_dtype, int64_t ldg, void* out, int out_dtype, int T, int N, int groups, int silu,
                                   hipStream_t stream) {
  if (T <= 0) return 0;
  if (N < 1 || groups < 1 || groups > 65535 || gates == nullptr || ldg < static_cast<int64_t>(N) * groups)
    return DISTIE_BAD_ARGUMENT;
  const int threads = N >= 1024 ? 1024 : (N >= 512 ? 512 : (N >= 256 ? 256 : (N >= 128 ? 128 : 64)));
  if (N <= 12288) {
    DISTIE_DISPATCH(w_dtype, W, DISTIE_DISPATCH(g_dtype, G, DISTIE_DISPATCH(out_dtype, O,
        gate_rmsnorm_kernel<true, W, G, O><<<dim3(T, groups), threads, sizeof(float) * N, stream>>>(
            x, static_cast<const W*>(weight), eps, static_cast<const G*>(gates), ldg, static_cast<O*>(out), N, groups, silu))));
  } else {
    DISTIE_DISPATCH(w_dtype, W, DISTIE_DISPATCH(g_dtype, G, DISTIE_DISPATCH(out_dtype, O,
        gate_rmsnorm_kernel<false, W, G, O><<<dim3(T, groups), threads, 0, stream>>>(
            x, static_cast<const W*>(weight), eps, static_cast<const G*>(gates), ldg, static_cast<O*>(out), N, groups, silu))));
  }
  return launch_status();
}

extern "C" int distie_glu_mul(const void* gate_up, int in_dtype, int slices, void* out, int dtype, int rows, int inter,
                              int kind, hipStream_t stream) {
  if (rows <= 0 || inter <= 0) return 0;
  if (kind < 0 || kind > 3 || slices < 1) return DISTIE_BAD_ARGUMENT;
  if (in_dtype == DISTIE_BF16 && dtype == DISTIE_BF16 && slices == 1 && inter % 8 == 0 &&
      reinterpret_cast<uintptr_t>(gate_up) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0) {
    const int64_t pieces = static_cast<int64_t>(rows) * (inter / 8);
    const int blocks8 = static_cast<int>(pieces / 256 + 1 < 16384 ? pieces / 256 + 1 : 16384);
    glu_mul_bf16x8_kernel<<<blocks8, 256, 0, stream>>>(static_cast<const uint4*>(gate_up), static_cast<uint4*>(out), rows,
                                                       inter / 8, kind);
    return launch_status();
  }
  const int64_t count = static_cast<int64_t>(rows) * inter;
  const int64_t blocks = (count + 255) / 256;
  if (blocks > 0x7fffffff) return DISTIE_BAD_ARGUMENT;
  DISTIE_DISPATCH(in_dtype, X, DISTIE_DISPATCH(dtype, O, glu_mul_kernel<X, O><<<static_cast<unsigned>(blocks), 256, 0, stream>>>(
      static_cast<const X*>(gate_up), slices, static_cast<int64_t>(rows) * 2 * inter, static_cast<O*>(out), rows, inter, kind)));
  return launch_status();
}
