// Routed feed-forward: every token is sent to `top` of E small feed-forward layers.
//
//   moe_route   : scores = f(router logits) per token (sigmoid, or softmax over the experts),
//                 the `top` largest (lowest index among equals), optionally renormalised
//   moe_plan    : the (token, choice) pairs ordered by expert: each expert's pairs take a run
//                 of rows that starts on a multiple of 16, so a tile of 16 rows belongs to one
//                 expert; the row count is bounded by pairs + 15 * E whatever the routing is,
//                 so a step's launches do not depend on the data
//   moe_gather  : the ordered rows of activations, each times its pair's weight when the weight
//                 acts on the expert's input
//   moe_gemm    : C[rows of a tile] = A[rows] * W[expert of the tile]^T for all tiles, with an
//                 optional activation; float32 chains on the vector ALU, or the matrix cores
//                 (v_mfma_f32_16x16x32_bf16) for bfloat16: operands through LDS for the many
//                 tiles of a prompt, K divided among the waves for the few of a single-token step
//   moe_combine : delta[t] = sum of the token's pairs' rows (times the weight when it acts on
//                 the output) + sigmoid(shared gate) * the shared expert's rows
//
// Router scores, weights and all sums are float32.
#include "common.h"

#define MOE_TILE 16

// ------------------------------------------------------------------ routing
// logits: [nt, ld] float32, the first E columns of a row are the router's. mode 0: sigmoid
// scores; 1: softmax over the experts. renorm: the chosen weights are divided by their sum
// (with mode 1 that is the softmax over the chosen logits alone). bias [E] or null: added to
// the logits first. groups > 1: the experts form that many equal groups of neighbours, a group
// counts as its largest score, and only experts of the `keep` best groups (the lowest index
// among equals) can be chosen.
__global__ __launch_bounds__(64) void moe_route_kernel(const float* __restrict__ logits, int ld, int E, int top,
                                                       int mode, int renorm, int* __restrict__ chosen,
                                                       float* __restrict__ weight,
                                                       const float* __restrict__ bias, int groups, int keep) {
  extern __shared__ float sc[];           // [E], then a score per group [groups]
  const size_t t = blockIdx.x;
  const int lane = threadIdx.x;
  float mx = -INFINITY;
  for (int e = lane; e < E; e += 64) mx = fmaxf(mx, logits[t * ld + e] + (bias ? bias[e] : 0.f));
  mx = wave_max(mx);
  float sum = 0.f;
  for (int e = lane; e < E; e += 64) {
    const float z = logits[t * ld + e] + (bias ? bias[e] : 0.f);
    const float s = mode == 0 ? 1.0f / (1.0f + expf(-z)) : expf(z - mx);
    sc[e] = s;
    sum += s;
  }
  sum = wave_sum(sum);
  __syncthreads();
  if (groups > 1) {
    float* gs = sc + E;
    const int size = E / groups;
    for (int g = lane; g < groups; g += 64) {
      float best = -INFINITY;
      for (int e = g * size; e < (g + 1) * size; ++e) best = fmaxf(best, sc[e]);
      gs[g] = best;
    }
    __syncthreads();
    // a group stays when fewer than `keep` groups come before it in the order (score down, index up)
    for (int g = lane; g < groups; g += 64) {
      const float mine = gs[g];
      int ahead = 0;
      for (int o = 0; o < groups; ++o) ahead += (gs[o] > mine || (gs[o] == mine && o < g)) ? 1 : 0;
      if (ahead >= keep)
        for (int e = g * size; e < (g + 1) * size; ++e) sc[e] = -INFINITY;
    }
    __syncthreads();
  }
  float total = 0.f;
  for (int j = 0; j < top; ++j) {
    float best = -INFINITY;
    int at = 0x7fffffff;
    for (int e = lane; e < E; e += 64) {
      const float s = sc[e];
      if (s > best) { best = s; at = e; }       // ascending e: the lowest index among equals
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, TA_WAVE);
      const int oa = __shfl_xor(at, o, TA_WAVE);
      if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
    }
    const float w = mode == 0 ? best : best / sum;
    if (lane == 0) {
      chosen[t * top + j] = at;
      weight[t * top + j] = w;
    }
    total += w;
    __syncthreads();
    if (lane == 0) sc[at] = -INFINITY;
    __syncthreads();
  }
  if (renorm) {
    __syncthreads();
    for (int j = lane; j < top; j += 64) weight[t * top + j] /= total;
  }
}

extern "C" int ta_moe_route_groups(hipStream_t stream, const float* logits, const float* bias, int ld, int nt, int E,
                                   int top, int mode, int renorm, int groups, int keep, int* chosen, float* weight) {
  TA_REQUIRE(nt >= 0 && E >= 1 && E <= 8192 && top >= 1 && top <= E && ld >= E && (mode == 0 || mode == 1),
             "ta_moe_route: bad sizes nt=%d experts=%d top=%d ld=%d", nt, E, top, ld);
  TA_REQUIRE(groups >= 1 && E % groups == 0 && keep >= 1 && keep <= groups && top <= keep * (E / groups),
             "ta_moe_route: %d experts in %d groups of which %d stay do not hold %d choices", E, groups, keep, top);
  if (nt == 0) return 0;
  moe_route_kernel<<<nt, 64, (size_t)(E + groups) * sizeof(float), stream>>>(logits, ld, E, top, mode, renorm, chosen,
                                                                             weight, bias, groups, keep);
  return ta_check_launch("ta_moe_route");
}

extern "C" int ta_moe_route_bias(hipStream_t stream, const float* logits, const float* bias, int ld, int nt, int E,
                                 int top, int mode, int renorm, int* chosen, float* weight) {
  return ta_moe_route_groups(stream, logits, bias, ld, nt, E, top, mode, renorm, 1, 1, chosen, weight);
}

extern "C" int ta_moe_route(hipStream_t stream, const float* logits, int ld, int nt, int E, int top, int mode,
                            int renorm, int* chosen, float* weight) {
  return ta_moe_route_bias(stream, logits, nullptr, ld, nt, E, top, mode, renorm, chosen, weight);
}

// ------------------------------------------------------------------ ordering the pairs by expert
// One workgroup. row_pair: [max_rows] pair index of every ordered row, -1 for a row that only
// fills a tile; tile_expert: [max_rows / 16], -1 for a tile past the last; pair_row: [pairs].
__global__ __launch_bounds__(1024) void moe_plan_kernel(const int* __restrict__ chosen, int pairs, int E,
                                                        int max_rows, int* __restrict__ row_pair,
                                                        int* __restrict__ tile_expert, int* __restrict__ pair_row) {
  extern __shared__ int sh[];             // count [E], start [E + 1]
  int* count = sh;
  int* start = sh + E;
  for (int e = threadIdx.x; e < E; e += 1024) count[e] = 0;
  for (int i = threadIdx.x; i < max_rows; i += 1024) row_pair[i] = -1;
  __syncthreads();
  for (int i = threadIdx.x; i < pairs; i += 1024) atomicAdd(&count[chosen[i]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0;
    for (int e = 0; e < E; ++e) {
      start[e] = at;
      at += (count[e] + MOE_TILE - 1) / MOE_TILE * MOE_TILE;
    }
    start[E] = at;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < max_rows / MOE_TILE; i += 1024) {
    const int r = i * MOE_TILE;
    int e = -1;
    if (r < start[E]) {                   // the last expert whose run starts at or before r
      int lo = 0, hi = E - 1;
      while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (start[mid] <= r) lo = mid; else hi = mid - 1;
      }
      e = lo;
    }
    tile_expert[i] = e;
  }
  for (int e = threadIdx.x; e < E; e += 1024) count[e] = 0;
  __syncthreads();
  // the order of an expert's rows among themselves does not matter: every row is computed alone
  for (int i = threadIdx.x; i < pairs; i += 1024) {
    const int e = chosen[i];
    const int r = start[e] + atomicAdd(&count[e], 1);
    row_pair[r] = i;
    pair_row[i] = r;
  }
}

extern "C" int ta_moe_max_rows(int pairs, int E) {
  const long long n = (long long)pairs + (long long)(MOE_TILE - 1) * E;
  const long long r = (n + MOE_TILE - 1) / MOE_TILE * MOE_TILE;
  return r > 2147483647ll ? -1 : (int)r;
}

extern "C" int ta_moe_plan(hipStream_t stream, const int* chosen, int pairs, int E, int max_rows, int* row_pair,
                           int* tile_expert, int* pair_row) {
  TA_REQUIRE(pairs >= 0 && E >= 1 && E <= 8192, "ta_moe_plan: bad sizes pairs=%d experts=%d", pairs, E);
  TA_REQUIRE(max_rows == ta_moe_max_rows(pairs, E), "ta_moe_plan: %d rows for %d pairs of %d experts", max_rows, pairs, E);
  moe_plan_kernel<<<1, 1024, (size_t)(2 * E + 1) * sizeof(int), stream>>>(chosen, pairs, E, max_rows, row_pair,
                                                                        tile_expert, pair_row);
  return ta_check_launch("ta_moe_plan");
}

// ------------------------------------------------------------------ gathering the rows
template <typename T>
__global__ __launch_bounds__(256) void moe_gather_kernel(const T* __restrict__ h, int d, int top,
                                                         const int* __restrict__ row_pair,
                                                         const float* __restrict__ weight, T* __restrict__ out) {
  const size_t r = blockIdx.x;
  const int pair = row_pair[r];
  T* dst = out + r * d;
  if (pair < 0) {
    for (int c = threadIdx.x; c < d; c += 256) dst[c] = from_f32<T>(0.f);
    return;
  }
  const T* src = h + (size_t)(pair / top) * d;
  if (weight) {
    const float w = weight[pair];
    for (int c = threadIdx.x; c < d; c += 256) dst[c] = from_f32<T>(to_f32(src[c]) * w);
  } else {
    for (int c = threadIdx.x; c < d; c += 256) dst[c] = src[c];
  }
}

// out[r] = h[token of row r] (* weight of its pair; weight null: as it is); filling rows are zero.
extern "C" int ta_moe_gather(hipStream_t stream, int dtype, const void* h, int d, int top, const int* row_pair,
                             const float* weight, void* out, int max_rows) {
  TA_REQUIRE(d > 0 && top >= 1 && max_rows >= 0, "ta_moe_gather: bad sizes");
  if (max_rows == 0) return 0;
  if (dtype == TA_F32)
    moe_gather_kernel<float><<<max_rows, 256, 0, stream>>>((const float*)h, d, top, row_pair, weight, (float*)out);
  else if (dtype == TA_BF16)
    moe_gather_kernel<bf16_t><<<max_rows, 256, 0, stream>>>((const bf16_t*)h, d, top, row_pair, weight, (bf16_t*)out);
  else
    return ta_fail("ta_moe_gather: unknown dtype %d", dtype);
  return ta_check_launch("ta_moe_gather");
}

// ------------------------------------------------------------------ the experts' products
__device__ __forceinline__ float moe_act(int act, float z) {
  switch (act) {
    case 1: return 0.5f * z * (1.0f + erff(z * 0.7071067811865476f));
    case 2: return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
    case 3: { const float r = fmaxf(z, 0.f); return r * r; }
    case 4: return z / (1.0f + expf(-z));
    default: return z;
  }
}

// float32 chains: a workgroup owns a tile of 16 rows and 64 columns; a thread 1 row x 4 columns.
// Every element is one ascending-k chain of fused multiply-adds.
template <typename T, typename TC>
__global__ __launch_bounds__(256) void moe_gemm_fma_kernel(const T* __restrict__ A, const T* __restrict__ W,
                                                           const int* __restrict__ tile_expert, TC* __restrict__ C,
                                                           int N, int K, int act) {
  __shared__ float As[16][MOE_TILE + 1];
  __shared__ float Ws[16][64 + 1];
  const int e = tile_expert[blockIdx.y];
  if (e < 0) return;
  const size_t r0 = (size_t)blockIdx.y * MOE_TILE;
  const int n0 = blockIdx.x * 64;
  const T* We = W + (size_t)e * N * K;
  const int tr = threadIdx.x / 16, tc = threadIdx.x % 16;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < K; k0 += 16) {
    {
      const int r = threadIdx.x / 16, k = k0 + threadIdx.x % 16;
      As[threadIdx.x % 16][r] = k < K ? to_f32(A[(r0 + r) * K + k]) : 0.f;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int idx = threadIdx.x + 256 * i, n = idx / 16, k = k0 + idx % 16;
      Ws[idx % 16][n] = (n0 + n < N && k < K) ? to_f32(We[(size_t)(n0 + n) * K + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < 16; ++kk) {
      const float a = As[kk][tr];
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[j] = fmaf(a, Ws[kk][tc * 4 + j], acc[j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int n = n0 + tc * 4 + j;
    if (n < N) C[(r0 + tr) * N + n] = from_f32<TC>(moe_act(act, acc[j]));
  }
}

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 moe_bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float moe_floatx4;
typedef uint32_t moe_u32x4 __attribute__((ext_vector_type(4)));
union MoeFrag {
  moe_bf16x8 v;
  moe_u32x4 q;
};
static __device__ __forceinline__ moe_u32x4 moe_zero4() { return moe_u32x4{0, 0, 0, 0}; }

// Matrix cores: a workgroup of 4 waves owns four neighbouring tiles of 16 rows, a wave 64
// columns of them (four 16 x 16 tiles). Neighbouring tiles of one expert form a run; a wave
// walks K once per run, in steps of 32 (a lane holds 8 consecutive k of row lane % 16 of its
// operand), and every piece of the expert's matrix that it loads serves all tiles of the run:
// a prompt's rows, of which an expert gets many, read the matrix a quarter as often; a step of
// few tokens has runs of one tile and reads every chosen expert's matrix once. The operands of
// the next step are asked for before the products of this one. K % 8 == 0; the last step's
// missing k are zero.
template <typename TC, int RUN>
__device__ __forceinline__ void moe_run(const bf16_t* __restrict__ A, const bf16_t* __restrict__ We,
                                        TC* __restrict__ C, size_t r0, int n0, int N, int K, int act, int lane) {
  const int r = lane % 16, kb = lane / 16;
  const bf16_t* arow[RUN];
#pragma unroll
  for (int u = 0; u < RUN; ++u) arow[u] = A + (r0 + 16 * u + r) * K + kb * 8;
  const bf16_t* wrow[4];
  bool wok[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const int n = n0 + 16 * t + r;
    wok[t] = n < N;
    wrow[t] = We + (size_t)(wok[t] ? n : 0) * K + kb * 8;
  }
  moe_floatx4 acc[RUN][4];
#pragma unroll
  for (int u = 0; u < RUN; ++u)
#pragma unroll
    for (int t = 0; t < 4; ++t) acc[u][t] = moe_floatx4{0.f, 0.f, 0.f, 0.f};
  // Three steps of 32 k are on their way while one is multiplied: a trip to memory takes several
  // times as long as a step's products. The whole steps load without a condition (a column past
  // N reads row 0 of the matrix and is never stored): a value chosen after its load would be
  // waited for where the load is issued.
  struct Step {
    MoeFrag a[RUN], w[4];
  };
  auto load = [&](Step& s, int k0) {
#pragma unroll
    for (int u = 0; u < RUN; ++u) s.a[u].q = *reinterpret_cast<const moe_u32x4*>(arow[u] + k0);
#pragma unroll
    for (int t = 0; t < 4; ++t) s.w[t].q = *reinterpret_cast<const moe_u32x4*>(wrow[t] + k0);   // other tiles read it again: it stays cached
  };
  auto mma = [&](const Step& s) {
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int u = 0; u < RUN; ++u)
        // register j of a lane: W row 4 * (lane / 16) + j of the tile, activation row lane % 16
        acc[u][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(s.w[t].v, s.a[u].v, acc[u][t], 0, 0, 0);
  };
  const int KF = K / 32 * 32;                           // whole steps
  Step s0, s1, s2;
  if (KF > 0) load(s0, 0);
  if (KF > 32) load(s1, 32);
  for (int k0 = 0; k0 < KF; k0 += 96) {
    if (k0 + 64 < KF) load(s2, k0 + 64);
    mma(s0);
    if (k0 + 32 >= KF) break;
    if (k0 + 96 < KF) load(s0, k0 + 96);
    mma(s1);
    if (k0 + 64 >= KF) break;
    if (k0 + 128 < KF) load(s1, k0 + 128);
    mma(s2);
  }
  if (KF < K) {                                         // the last, partial step
    const bool kok = KF + kb * 8 < K;
#pragma unroll
    for (int u = 0; u < RUN; ++u) s0.a[u].q = kok ? *reinterpret_cast<const moe_u32x4*>(arow[u] + KF) : moe_zero4();
#pragma unroll
    for (int t = 0; t < 4; ++t) s0.w[t].q = kok ? *reinterpret_cast<const moe_u32x4*>(wrow[t] + KF) : moe_zero4();
    mma(s0);
  }
#pragma unroll
  for (int u = 0; u < RUN; ++u)
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int n = n0 + 16 * t + 4 * kb + j;
        if (n < N) C[(r0 + 16 * u + r) * N + n] = from_f32<TC>(moe_act(act, acc[u][t][j]));
      }
}

template <typename TC>
__global__ __launch_bounds__(256) void moe_gemm_mfma_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ W,
                                                            const int* __restrict__ tile_expert, int tiles,
                                                            TC* __restrict__ C, int N, int K, int act) {
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int n0 = (blockIdx.x * 4 + wave) * 64;
  if (n0 >= N) return;
  int t = blockIdx.y * 4;
  const int t_end = t + 4 < tiles ? t + 4 : tiles;
  while (t < t_end) {
    const int e = tile_expert[t];
    if (e < 0) return;                                  // tiles past the last expert's rows
    int run = 1;
    while (t + run < t_end && tile_expert[t + run] == e) ++run;
    const bf16_t* We = W + (size_t)e * N * K;
    const size_t r0 = (size_t)t * MOE_TILE;
    if (run == 4) moe_run<TC, 4>(A, We, C, r0, n0, N, K, act, lane);
    else if (run == 3) moe_run<TC, 3>(A, We, C, r0, n0, N, K, act, lane);
    else if (run == 2) moe_run<TC, 2>(A, We, C, r0, n0, N, K, act, lane);
    else moe_run<TC, 1>(A, We, C, r0, n0, N, K, act, lane);
    t += run;
  }
}

// Few tiles (a step of few tokens): a workgroup owns ONE tile of 16 rows and 64 columns and its
// four waves divide K, so that four times as many loads of the expert's matrix are on their way;
// the partial tiles are added in wave order through LDS.
template <typename TC>
__global__ __launch_bounds__(256) void moe_gemm_mfma_splitk_kernel(const bf16_t* __restrict__ A,
                                                                   const bf16_t* __restrict__ W,
                                                                   const int* __restrict__ tile_expert,
                                                                   TC* __restrict__ C, int N, int K, int act) {
  __shared__ float red[4][16][65];
  const int e = tile_expert[blockIdx.y];
  if (e < 0) return;                                    // the whole workgroup: tiles past the last expert's rows
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int r = lane % 16, kb = lane / 16;
  const int n0 = blockIdx.x * 64;
  const size_t r0 = (size_t)blockIdx.y * MOE_TILE;
  const bf16_t* We = W + (size_t)e * N * K;
  const int steps = (K + 31) / 32;
  const int kbeg = 32 * (steps * wave / 4), kend = 32 * (steps * (wave + 1) / 4);
  const bf16_t* arow = A + (r0 + r) * K + kb * 8;
  const bf16_t* wrow[4];
  bool wok[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const int n = n0 + 16 * t + r;
    wok[t] = n < N;
    wrow[t] = We + (size_t)(wok[t] ? n : 0) * K + kb * 8;
  }
  moe_floatx4 acc[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) acc[t] = moe_floatx4{0.f, 0.f, 0.f, 0.f};
  constexpr int DEPTH = 4;                              // steps of 32 k asked for together
  for (int k0 = kbeg; k0 < kend; k0 += 32 * DEPTH) {
    MoeFrag af[DEPTH], wf[DEPTH][4];
#pragma unroll
    for (int u = 0; u < DEPTH; ++u) {
      const int k = k0 + 32 * u;
      const bool kok = k < kend && k + kb * 8 < K;
      af[u].q = kok ? *reinterpret_cast<const moe_u32x4*>(arow + k) : moe_zero4();
#pragma unroll
      for (int t = 0; t < 4; ++t)
        wf[u][t].q = (kok && wok[t]) ? __builtin_nontemporal_load(reinterpret_cast<const moe_u32x4*>(wrow[t] + k)) : moe_zero4();
    }
#pragma unroll
    for (int u = 0; u < DEPTH; ++u)
#pragma unroll
      for (int t = 0; t < 4; ++t)
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[u][t].v, af[u].v, acc[t], 0, 0, 0);
  }
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int j = 0; j < 4; ++j) red[wave][r][16 * t + 4 * kb + j] = acc[t][j];
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int idx = threadIdx.x + 256 * i, row = idx / 64, col = idx % 64;
    const float v = (red[0][row][col] + red[1][row][col]) + (red[2][row][col] + red[3][row][col]);
    if (n0 + col < N) C[(r0 + row) * N + n0 + col] = from_f32<TC>(moe_act(act, v));
  }
}

// Many tiles (a prompt): operands through LDS. A workgroup owns eight neighbouring tiles of 16
// rows and 128 columns; the runs of one expert among them are multiplied one after the other.
// Every thread brings whole 16-byte pieces of the rows of A and of the expert's matrix (eight
// lanes a row: whole cache lines), a step of 64 k ahead of the one being multiplied, into one of
// two LDS buffers (rows 72 elements apart, so that the operand reads of 16 rows meet 16
// different bank groups); a wave multiplies 64 x 64 of the 128 x 128 (4 x 4 operand tiles: every
// LDS read feeds four products).
#define ML_BM 128
#define ML_BN 128
#define ML_BK 64
#define ML_LD 72

template <typename TC>
__global__ __launch_bounds__(256, 2) void moe_gemm_lds_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ W,
                                                           const int* __restrict__ tile_expert, int tiles, int max_rows,
                                                           TC* __restrict__ C, int N, int K, int act) {
  extern __shared__ __attribute__((aligned(16))) unsigned char ml_lds[];
  bf16_t* As = reinterpret_cast<bf16_t*>(ml_lds);                       // [2][ML_BM][ML_LD]
  bf16_t* Ws = As + 2 * ML_BM * ML_LD;                                  // [2][ML_BN][ML_LD]
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int r = lane % 16, kb = lane / 16, wr = wave / 2, wc = wave % 2;
  // Which (group of eight tiles, block of 128 columns) this workgroup takes. Workgroups go to the
  // eight XCDs in turn, and each XCD has an L2 of its own: the workgroups that one XCD gets one
  // after the other take two neighbouring groups of tiles (mostly one expert) through all blocks
  // of columns, block by block, so that the expert's panel of 128 columns is read from memory once
  // for both groups and the groups' rows once for all blocks.
  const int ncol = (N + ML_BN - 1) / ML_BN;
  const int xcd = blockIdx.x % 8, seq = blockIdx.x / 8;
  const int unit = (seq / (2 * ncol)) * 8 + xcd, within = seq % (2 * ncol);
  const int group = 2 * unit + within % 2;
  const int n0 = (within / 2) * ML_BN;
  int t = group * 8;
  if (t >= tiles) return;
  const int t_end = t + 8 < tiles ? t + 8 : tiles;
  const int nk = (K + ML_BK - 1) / ML_BK;
  while (t < t_end) {
    const int e = tile_expert[t];
    if (e < 0) return;                                  // the whole workgroup: tiles past the last expert's rows
    int run = 1;
    while (t + run < t_end && tile_expert[t + run] == e) ++run;
    const int R = run * MOE_TILE;
    const size_t r0 = (size_t)t * MOE_TILE;
    const bf16_t* We = W + (size_t)e * N * K;
    // this thread's four pieces of A and of W in a step: row p / 8, piece p % 8, p = tid + 256 i
    const bf16_t* asrc[4];
    const bf16_t* wsrc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int p = tid + 256 * i, row = p / 8, pc = p % 8;
      const size_t ar = r0 + (row < R ? row : R - 1);                   // rows past the run: read again, never stored
      const int wn = n0 + row < N ? n0 + row : N - 1;                   // columns past N likewise
      asrc[i] = A + ar * K + pc * 8;
      wsrc[i] = We + (size_t)wn * K + pc * 8;
    }
    // Three steps' pieces wait in registers on their way from memory (a trip takes several times
    // as long as a step's products); the barrier between steps waits for LDS traffic only, not
    // for these loads.
    struct Pieces {
      moe_u32x4 a[4], w[4];
    };
    auto fetch = [&](Pieces& q, int step) {
      const int k0 = step * ML_BK;
      if (step >= nk) return;
      if (k0 + ML_BK <= K) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          q.a[i] = *reinterpret_cast<const moe_u32x4*>(asrc[i] + k0);
          q.w[i] = *reinterpret_cast<const moe_u32x4*>(wsrc[i] + k0);
        }
      } else {                                                          // the last, partial step
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const bool kok = k0 + ((tid + 256 * i) % 8) * 8 < K;
          q.a[i] = kok ? *reinterpret_cast<const moe_u32x4*>(asrc[i] + k0) : moe_zero4();
          q.w[i] = kok ? *reinterpret_cast<const moe_u32x4*>(wsrc[i] + k0) : moe_zero4();
        }
      }
    };
    auto stash = [&](const Pieces& q, int buf) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int p = tid + 256 * i, row = p / 8, pc = p % 8;
        *reinterpret_cast<moe_u32x4*>(As + (buf * ML_BM + row) * ML_LD + pc * 8) = q.a[i];
        *reinterpret_cast<moe_u32x4*>(Ws + (buf * ML_BN + row) * ML_LD + pc * 8) = q.w[i];
      }
    };
    auto lds_barrier = [&]() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };
    moe_floatx4 acc[4][4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[u][v] = moe_floatx4{0.f, 0.f, 0.f, 0.f};
    const bool busy = 64 * wr < R;                      // a run of at most 64 rows leaves two waves only loading
    auto multiply = [&](int buf) {
      if (!busy) return;
#pragma unroll
      for (int kk = 0; kk < ML_BK; kk += 32) {
        MoeFrag af[4], wf[4];
#pragma unroll
        for (int u = 0; u < 4; ++u)
          af[u].q = *reinterpret_cast<const moe_u32x4*>(As + (buf * ML_BM + 64 * wr + 16 * u + r) * ML_LD + kk + 8 * kb);
#pragma unroll
        for (int v = 0; v < 4; ++v)
          wf[v].q = *reinterpret_cast<const moe_u32x4*>(Ws + (buf * ML_BN + 64 * wc + 16 * v + r) * ML_LD + kk + 8 * kb);
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
          for (int v = 0; v < 4; ++v)
            // register j of a lane: column 4 * (lane / 16) + j of the tile, row lane % 16
            acc[u][v] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[v].v, af[u].v, acc[u][v], 0, 0, 0);
      }
    };
    Pieces p0, p1, p2;
    fetch(p0, 0);
    fetch(p1, 1);
    fetch(p2, 2);
    stash(p0, 0);
    fetch(p0, 3);
    lds_barrier();
    // step s multiplies buffer s & 1; the pieces of step s + 1 (in set (s + 1) % 3) then go to the
    // other buffer and their set asks for step s + 4
    for (int step = 0; step < nk; step += 3) {
      multiply(step & 1);
      if (step + 1 < nk) { stash(p1, (step + 1) & 1); fetch(p1, step + 4); }
      lds_barrier();
      if (step + 1 >= nk) break;
      multiply((step + 1) & 1);
      if (step + 2 < nk) { stash(p2, (step + 2) & 1); fetch(p2, step + 5); }
      lds_barrier();
      if (step + 2 >= nk) break;
      multiply((step + 2) & 1);
      if (step + 3 < nk) { stash(p0, (step + 3) & 1); fetch(p0, step + 6); }
      lds_barrier();
    }
    if (busy) {
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        if (64 * wr + 16 * u >= R) break;
#pragma unroll
        for (int v = 0; v < 4; ++v)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int n = n0 + 64 * wc + 16 * v + 4 * kb + j;
            if (n < N) C[(r0 + 64 * wr + 16 * u + r) * N + n] = from_f32<TC>(moe_act(act, acc[u][v][j]));
          }
      }
    }
    t += run;
  }
}

// A: [max_rows, K] ordered rows; W: [E, N, K]; C: [max_rows, N], float32 or the type of A;
// act: 0 none, 1 gelu, 2 gelu (tanh), 3 relu squared, 4 silu. Tiles past the last expert's
// rows are skipped and their rows of C keep what they held.
static int moe_gemm_lds_launch(hipStream_t stream, int out_dtype, const void* A, const void* W, const int* tile_expert,
                               void* C, int max_rows, int tiles, int N, int K, int act) {
  const size_t lds = (size_t)2 * (ML_BM + ML_BN) * ML_LD * sizeof(bf16_t);
  const int ncol = (N + ML_BN - 1) / ML_BN, groups = (tiles + 7) / 8, units = (groups + 1) / 2;
  dim3 g((unsigned)((units + 7) / 8 * 8 * 2 * ncol));      // see the kernel: eight XCDs take units of 2 groups x all column blocks
#define ML_RUN(TC)                                                                                               \
  do {                                                                                                           \
    auto kern = moe_gemm_lds_kernel<TC>;                                                                         \
    static bool allowed = false;                        /* asked for once, not at every launch */                \
    if (!allowed) {                                                                                              \
      const hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),                            \
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);          \
      if (err != hipSuccess) return ta_fail("ta_moe_gemm: %zu bytes of LDS refused (%s)", lds, hipGetErrorString(err)); \
      allowed = true;                                                                                            \
    }                                                                                                            \
    kern<<<g, 256, lds, stream>>>((const bf16_t*)A, (const bf16_t*)W, tile_expert, tiles, max_rows, (TC*)C, N, K, act); \
  } while (0)
  if (out_dtype == TA_BF16) ML_RUN(bf16_t); else ML_RUN(float);
#undef ML_RUN
  return ta_check_launch("ta_moe_gemm");
}

// form: 0 = chosen by the shape; 1 = the waves divide K (few tiles); 2 = runs of tiles with operands
// straight from memory; 3 = operands through LDS (many tiles). 1 to 3 take bfloat16 with K % 8 == 0.
extern "C" int ta_moe_gemm_form(hipStream_t stream, int dtype, int out_dtype, const void* A, const void* W,
                                const int* tile_expert, void* C, int max_rows, int N, int K, int act, int form) {
  TA_REQUIRE(max_rows >= 0 && max_rows % MOE_TILE == 0 && N > 0 && K > 0 && act >= 0 && act <= 4,
             "ta_moe_gemm: bad sizes rows=%d N=%d K=%d act=%d", max_rows, N, K, act);
  TA_REQUIRE(form >= 0 && form <= 3 && (form == 0 || (dtype == TA_BF16 && K % 8 == 0)),
             "ta_moe_gemm: form %d needs bfloat16 and K %% 8 == 0", form);
  if (max_rows == 0) return 0;
  const int tiles = max_rows / MOE_TILE;
  if (dtype == TA_BF16 && K % 8 == 0) {
    if (out_dtype != TA_BF16 && out_dtype != TA_F32) return ta_fail("ta_moe_gemm: unknown output type %d", out_dtype);
    const bool few = (long long)tiles * ((N + 255) / 256) < 1024;
    if (form == 3 || (form == 0 && !few)) return moe_gemm_lds_launch(stream, out_dtype, A, W, tile_expert, C, max_rows, tiles, N, K, act);
    if (form == 1 || (form == 0 && few)) {   // too few workgroups to fill the CUs: the waves divide K
      dim3 gk((N + 63) / 64, tiles);
      if (out_dtype == TA_BF16)
        moe_gemm_mfma_splitk_kernel<bf16_t><<<gk, 256, 0, stream>>>((const bf16_t*)A, (const bf16_t*)W, tile_expert, (bf16_t*)C, N, K, act);
      else
        moe_gemm_mfma_splitk_kernel<float><<<gk, 256, 0, stream>>>((const bf16_t*)A, (const bf16_t*)W, tile_expert, (float*)C, N, K, act);
      return ta_check_launch("ta_moe_gemm");
    }
    dim3 g((N + 255) / 256, (tiles + 3) / 4);
    if (out_dtype == TA_BF16)
      moe_gemm_mfma_kernel<bf16_t><<<g, 256, 0, stream>>>((const bf16_t*)A, (const bf16_t*)W, tile_expert, tiles, (bf16_t*)C, N, K, act);
    else if (out_dtype == TA_F32)
      moe_gemm_mfma_kernel<float><<<g, 256, 0, stream>>>((const bf16_t*)A, (const bf16_t*)W, tile_expert, tiles, (float*)C, N, K, act);
    else
      return ta_fail("ta_moe_gemm: unknown output type %d", out_dtype);
    return ta_check_launch("ta_moe_gemm");
  }
  dim3 g((N + 63) / 64, tiles);
  if (dtype == TA_F32 && out_dtype == TA_F32)
    moe_gemm_fma_kernel<float, float><<<g, 256, 0, stream>>>((const float*)A, (const float*)W, tile_expert, (float*)C, N, K, act);
  else if (dtype == TA_BF16 && out_dtype == TA_BF16)
    moe_gemm_fma_kernel<bf16_t, bf16_t><<<g, 256, 0, stream>>>((const bf16_t*)A, (const bf16_t*)W, tile_expert, (bf16_t*)C, N, K, act);
  else if (dtype == TA_BF16 && out_dtype == TA_F32)
    moe_gemm_fma_kernel<bf16_t, float><<<g, 256, 0, stream>>>((const bf16_t*)A, (const bf16_t*)W, tile_expert, (float*)C, N, K, act);
  else
    return ta_fail("ta_moe_gemm: unsupported types %d -> %d", dtype, out_dtype);
  return ta_check_launch("ta_moe_gemm");
}

extern "C" int ta_moe_gemm(hipStream_t stream, int dtype, int out_dtype, const void* A, const void* W,
                           const int* tile_expert, void* C, int max_rows, int N, int K, int act) {
  return ta_moe_gemm_form(stream, dtype, out_dtype, A, W, tile_expert, C, max_rows, N, K, act, 0);
}

// ------------------------------------------------------------------ putting the rows back
__global__ __launch_bounds__(256) void moe_combine_kernel(const float* __restrict__ rows, int d, int top,
                                                          const int* __restrict__ pair_row,
                                                          const float* __restrict__ weight,
                                                          const float* __restrict__ shared, int planes, size_t plane,
                                                          const float* __restrict__ shared_gate, int gate_ld,
                                                          float* __restrict__ delta,
                                                          const float* __restrict__ extra, int xplanes, size_t xplane) {
  extern __shared__ float cmb[];          // [top] rows of the token's pairs, [top] their weights
  int* prow = reinterpret_cast<int*>(cmb);
  float* pw = cmb + top;
  const size_t t = blockIdx.x;
  for (int j = threadIdx.x; j < top; j += 256) {
    prow[j] = pair_row[t * top + j];
    pw[j] = weight ? weight[t * top + j] : 1.f;
  }
  float sg = 1.f;
  if (shared && shared_gate) sg = 1.0f / (1.0f + expf(-shared_gate[t * gate_ld]));
  __syncthreads();
  for (int c = threadIdx.x; c < d; c += 256) {
    float s = 0.f;
    for (int j = 0; j < top; ++j) s = fmaf(rows[(size_t)prow[j] * d + c], pw[j], s);
    if (shared) {
      float v = shared[t * d + c];
      for (int p = 1; p < planes; ++p) v += shared[t * d + c + p * plane];
      s += sg * v;
    }
    if (extra)      // what another sublayer adds to the stream beside this one, planes in order
      for (int p = 0; p < xplanes; ++p) s += extra[t * d + c + p * xplane];
    delta[t * d + c] = s;
  }
}

// rows: [max_rows, d] float32, the experts' results in the planned order. weight: null when it
// has acted on the inputs. shared (or null): [planes, nt, d] float32 planes that add up to the
// shared expert's result; shared_gate (or null): its gate's pre-activation, one number per
// token, element 0 of a row of gate_ld float32. delta: [nt, d] float32.
// extra (or null): [xplanes, nt, d] float32 planes, ``xplane`` elements apart, added as they are.
extern "C" int ta_moe_combine_extra(hipStream_t stream, const float* rows, int d, int top, const int* pair_row,
                                    const float* weight, const float* shared, int planes, long long plane,
                                    const float* shared_gate, int gate_ld, const float* extra, int xplanes,
                                    long long xplane, float* delta, int nt) {
  TA_REQUIRE(nt >= 0 && d > 0 && top >= 1 && planes >= 1 && planes <= TA_MAX_PLANES, "ta_moe_combine: bad sizes");
  TA_REQUIRE(!extra || (xplanes >= 1 && xplanes <= TA_MAX_PLANES && (xplanes == 1 || xplane > 0)),
             "ta_moe_combine: %d planes of the further addend", xplanes);
  if (nt == 0) return 0;
  moe_combine_kernel<<<nt, 256, (size_t)2 * top * sizeof(float), stream>>>(rows, d, top, pair_row, weight, shared, planes, (size_t)plane,
                                             shared_gate, gate_ld, delta, extra, xplanes, (size_t)xplane);
  return ta_check_launch("ta_moe_combine");
}

extern "C" int ta_moe_combine(hipStream_t stream, const float* rows, int d, int top, const int* pair_row,
                              const float* weight, const float* shared, int planes, long long plane,
                              const float* shared_gate, int gate_ld, float* delta, int nt) {
  return ta_moe_combine_extra(stream, rows, d, top, pair_row, weight, shared, planes, plane, shared_gate, gate_ld,
                              nullptr, 0, 0, delta, nt);
}

// ------------------------------------------------------------------ the limited gated activation
// Rows of [gate | up] (``di`` columns each, ``ld`` elements between rows): g = min(gate, limit),
// u = clamp(up, -limit, limit), out = g * sigmoid(slope * g) * (u + shift). float32 inside.
template <typename T>
__global__ __launch_bounds__(256) void glu_limit_kernel(const T* __restrict__ gu, int ld, T* __restrict__ out, int di,
                                                        float limit, float slope, float shift) {
  const size_t t = blockIdx.y;
  const T* g = gu + t * (size_t)ld;
  T* o = out + t * (size_t)di;
  for (int i = blockIdx.x * 256 + threadIdx.x; i < di; i += gridDim.x * 256) {
    const float a = fminf(to_f32(g[i]), limit);
    const float u = fminf(fmaxf(to_f32(g[di + i]), -limit), limit);
    o[i] = from_f32<T>(a / (1.0f + expf(-slope * a)) * (u + shift));
  }
}

extern "C" int ta_glu_limit(hipStream_t stream, int dtype, const void* gate_up, int ld, void* out, int nt, int di,
                            float limit, float slope, float shift) {
  TA_REQUIRE(nt >= 0 && di > 0 && ld >= 2 * di, "ta_glu_limit: bad sizes nt=%d di=%d ld=%d", nt, di, ld);
  TA_REQUIRE(limit > 0.f, "ta_glu_limit: the limit must be positive, got %g", (double)limit);
  for (int t0 = 0; t0 < nt; t0 += 65535) {
    const int rows = nt - t0 < 65535 ? nt - t0 : 65535;
    dim3 g((di + 1023) / 1024 < 64 ? (di + 1023) / 1024 : 64, rows);
    if (dtype == TA_F32)
      glu_limit_kernel<float><<<g, 256, 0, stream>>>((const float*)gate_up + (size_t)t0 * ld, ld,
                                                    (float*)out + (size_t)t0 * di, di, limit, slope, shift);
    else if (dtype == TA_BF16)
      glu_limit_kernel<bf16_t><<<g, 256, 0, stream>>>((const bf16_t*)gate_up + (size_t)t0 * ld, ld,
                                                     (bf16_t*)out + (size_t)t0 * di, di, limit, slope, shift);
    else
      return ta_fail("ta_glu_limit: unknown dtype %d", dtype);
  }
  return ta_check_launch("ta_glu_limit");
}
