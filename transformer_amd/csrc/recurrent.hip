// Mixers that carry a fixed-size state per sequence instead of a cache of keys.
//
// Gated diagonal recurrence ("rglru"): per channel c
//     u_t = conv_b + sum_j taps[c][j] * xin_{t-(K-1-j)}          (short causal convolution)
//     r_t, i_t = sigmoid(block-diagonal products of u_t + bias)
//     a_t = exp(-c0 * r_t * softplus(lam)),  S_t = a_t S_{t-1} + sqrt(1 - a_t^2) * i_t * u_t
//     out_t = S_t * gelu_tanh(y_t)
//   in two kernels: `rglru_gates` forms a_t and the input term for all tokens at once (they do
//   not depend on S), `rglru_scan` walks each sequence's tokens in order, one thread a channel.
//
// Gated linear attention ("gla"): per head a matrix state S [dk][dv]
//     alpha_t = sigmoid(z_t)^(1/tau) per key channel, z_t = A2 (a1h_t) + bias
//     S_t = diag(alpha_t) S_{t-1} + k_t v_t^T,  o_t = S_t^T q_t
//   `gla_decay` forms alpha for all tokens at once, `gla_recurrent` walks a sequence's tokens in
//   order with S in registers; `gla_out` applies the per-head RMS norm and the output gate.
//
// Selective state space ("ssm"): per head a matrix state S [N][P] with one decay per (token, head),
//     dt_t = softplus(raw_t + bias), S_t = exp(-exp(A) dt_t) S_{t-1} + dt_t B_t x_t^T, o_t = S_t^T C_t
//   `ssm_steps` forms step sizes and decays, the recurrence is `gla_recurrent` with q = C, k = B, v = x
//   (the heads of a group read the same B and C), `gated_group_norm` adds D x, gates and norms.
//
// Short causal convolution (`causal_conv`): per channel over a sequence's tokens, with the last
//   inputs of every sequence kept between steps; used in front of the state space and by the
//   attention variant that convolves its q, k and v.
//
// All state, decays, gates and sums are float32; tokens are walked in the same order however a
// sequence was cut into steps, so the cut does not change a bit of the result.
#include "common.h"

__device__ __forceinline__ int seq_of_token_r(const int* __restrict__ cu_q, int batch, int t) {
  int lo = 0, hi = batch - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (cu_q[mid] <= t) lo = mid; else hi = mid - 1;
  }
  return lo;
}

__device__ __forceinline__ float sigmoidf_(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplusf_(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }
__device__ __forceinline__ float gelu_tanhf_(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

// ------------------------------------------------------------------ rglru: gates
#define RG_TT 8     // tokens per workgroup

template <typename T, typename TW>
__global__ __launch_bounds__(256) void rglru_gates_kernel(
    const T* __restrict__ yx, int stride, int xoff, const float* __restrict__ xbias,
    const float* __restrict__ taps, const float* __restrict__ conv_bias, int K,
    const float* __restrict__ conv_state, const TW* __restrict__ gates_w,
    const float* __restrict__ gates_b, const float* __restrict__ lam, float c0,
    const int* __restrict__ cu_q, const int* __restrict__ slots, int batch, int nt, int C, int nb,
    float* __restrict__ a_out, float* __restrict__ b_out) {
  extern __shared__ float u[];            // [RG_TT][bs]
  __shared__ int s_start[RG_TT], s_slot[RG_TT];
  const int bs = C / nb;
  const int t0 = blockIdx.x * RG_TT, blk = blockIdx.y;
  if (threadIdx.x < RG_TT) {
    const int t = t0 + threadIdx.x;
    int st = 0, sl = 0;
    if (t < nt) {
      const int b = seq_of_token_r(cu_q, batch, t);
      st = cu_q[b];
      sl = slots[b];
    }
    s_start[threadIdx.x] = st;
    s_slot[threadIdx.x] = sl;
  }
  __syncthreads();
  for (int idx = threadIdx.x; idx < RG_TT * bs; idx += 256) {
    const int tt = idx / bs, cc = idx - tt * bs;
    const int t = t0 + tt, c = blk * bs + cc;
    float acc = 0.f;
    if (t < nt) {
      acc = conv_bias[c];
      const int start = s_start[tt];
      const float* cs = conv_state + ((size_t)s_slot[tt] * (K - 1)) * C;
      for (int j = 0; j < K; ++j) {
        const int tp = t - (K - 1 - j);
        float xin;
        if (tp >= start) xin = to_f32(yx[(size_t)tp * stride + xoff + c]) + xbias[c];
        else xin = cs[(size_t)(K - 1 + (tp - start)) * C + c];
        acc = fmaf(taps[(size_t)c * K + j], xin, acc);
      }
    }
    u[idx] = acc;
  }
  __syncthreads();
  for (int o = threadIdx.x; o < bs; o += 256) {
    const int c = blk * bs + o;
    float ar[RG_TT], ai[RG_TT];
#pragma unroll
    for (int tt = 0; tt < RG_TT; ++tt) ar[tt] = ai[tt] = 0.f;
    const TW* wr = gates_w + ((size_t)blk * bs + o) * bs;                 // recurrence gate, block blk
    const TW* wi = gates_w + ((size_t)(nb + blk) * bs + o) * bs;          // input gate
    for (int in = 0; in < bs; ++in) {
      const float a = to_f32(wr[in]), b = to_f32(wi[in]);
#pragma unroll
      for (int tt = 0; tt < RG_TT; ++tt) {
        const float uu = u[tt * bs + in];
        ar[tt] = fmaf(a, uu, ar[tt]);
        ai[tt] = fmaf(b, uu, ai[tt]);
      }
    }
    const float br = gates_b[(size_t)blk * bs + o], bi = gates_b[(size_t)(nb + blk) * bs + o];
    const float sp = softplusf_(lam[c]);
#pragma unroll
    for (int tt = 0; tt < RG_TT; ++tt) {
      const int t = t0 + tt;
      if (t < nt) {
        const float r = sigmoidf_(ar[tt] + br), g = sigmoidf_(ai[tt] + bi);
        const float loga = -c0 * r * sp;
        a_out[(size_t)t * C + c] = expf(loga);
        b_out[(size_t)t * C + c] = sqrtf(-expm1f(2.0f * loga)) * g * u[tt * bs + o];
      }
    }
  }
}

// The same with the gates' weights staged through LDS: a workgroup owns RGT_TT tokens x RGT_OC
// output channels of one block and walks the block's inputs in turns of RGT_KC, each turn's
// weights loaded row by row in whole pieces and laid down transposed, so that a thread reads its
// channel's weight and a wave shares every u. Used whenever a block's inputs fit the LDS.
#define RGT_TT 16
#define RGT_OC 64
#define RGT_KC 32

template <typename T, typename TW>
__global__ __launch_bounds__(256) void rglru_gates_tiled_kernel(
    const T* __restrict__ yx, int stride, int xoff, const float* __restrict__ xbias,
    const float* __restrict__ taps, const float* __restrict__ conv_bias, int K,
    const float* __restrict__ conv_state, const TW* __restrict__ gates_w,
    const float* __restrict__ gates_b, const float* __restrict__ lam, float c0,
    const int* __restrict__ cu_q, const int* __restrict__ slots, int batch, int nt, int C, int nb,
    int bsp, float* __restrict__ a_out, float* __restrict__ b_out) {
  extern __shared__ float sm[];
  float* u = sm;                               // [RGT_TT][bsp], zero beyond bs
  float* wrs = u + RGT_TT * bsp;               // [RGT_KC][RGT_OC]
  float* wis = wrs + RGT_KC * RGT_OC;
  __shared__ int s_start[RGT_TT], s_slot[RGT_TT];
  const int bs = C / nb;
  const int tiles = (bs + RGT_OC - 1) / RGT_OC;
  const int blk = blockIdx.y / tiles, o0 = (blockIdx.y % tiles) * RGT_OC;
  const int t0 = blockIdx.x * RGT_TT;
  if (threadIdx.x < RGT_TT) {
    const int t = t0 + threadIdx.x;
    int st = 0, sl = 0;
    if (t < nt) {
      const int b = seq_of_token_r(cu_q, batch, t);
      st = cu_q[b];
      sl = slots[b];
    }
    s_start[threadIdx.x] = st;
    s_slot[threadIdx.x] = sl;
  }
  __syncthreads();
  // groups of four turns known to lie inside the tile, so that their loads are on their way
  // together (a load is not asked for before the test that guards it)
  auto conv = [&](int idx) {
    const int tt = idx / bsp, cc = idx - tt * bsp;
    const int t = t0 + tt, c = blk * bs + cc;
    // both places a tap may read (this step's rows, the sequence's memory) are asked for
    // whatever the case, at addresses that exist, and one is chosen: no load waits for a branch
    const bool on = t < nt && cc < bs;
    // an entry that is not there computes on token 0 of the step as if it began a sequence,
    // so that every index below stays inside its array
    const int ts = on ? t : 0, cz = on ? c : 0;
    const int start = on ? s_start[tt] : 0;
    const float* cs = conv_state + ((size_t)(on ? s_slot[tt] : s_slot[0]) * (K - 1)) * C;
    const float xb = xbias[cz];
    float acc = conv_bias[cz];
    for (int j = 0; j < K; ++j) {
      const int tp = ts - (K - 1 - j);
      const bool here = tp >= start;
      const float a = to_f32(yx[(size_t)(here ? tp : ts) * stride + xoff + cz]) + xb;
      const float m = K > 1 ? cs[(size_t)(here ? 0 : K - 1 + (tp - start)) * C + cz] : 0.f;
      acc = fmaf(taps[(size_t)cz * K + j], here ? a : m, acc);
    }
    u[idx] = on ? acc : 0.f;
  };
  {
    int idx = threadIdx.x;
    for (; idx + 768 < RGT_TT * bsp; idx += 1024) {
#pragma unroll
      for (int q = 0; q < 4; ++q) conv(idx + 256 * q);
    }
    for (; idx < RGT_TT * bsp; idx += 256) conv(idx);
  }
  const int o = threadIdx.x % RGT_OC, tg = threadIdx.x / RGT_OC;      // tokens tg*4 .. tg*4+3
  const int lr = threadIdx.x / 4, lseg = (threadIdx.x % 4) * 8;       // staging: row lr, 8 inputs from lseg
  float ar[4] = {0.f, 0.f, 0.f, 0.f}, ai[4] = {0.f, 0.f, 0.f, 0.f};
  const bool row_ok = o0 + lr < bs;
  const TW* wr = gates_w + ((size_t)blk * bs + (row_ok ? o0 + lr : 0)) * bs;
  const TW* wi = gates_w + ((size_t)(nb + blk) * bs + (row_ok ? o0 + lr : 0)) * bs;
  float nr[8], ni[8];                           // the next turn's weights, on their way
  auto fetch = [&](int k0) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int in = k0 + lseg + e;
      const bool ok = row_ok && in < bs;
      const float a = to_f32(wr[ok ? in : 0]), b = to_f32(wi[ok ? in : 0]);
      nr[e] = ok ? a : 0.f;
      ni[e] = ok ? b : 0.f;
    }
  };
  fetch(0);
  for (int k0 = 0; k0 < bs; k0 += RGT_KC) {
    __syncthreads();                            // u is complete / the last turn's weights are used up
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      wrs[(lseg + e) * RGT_OC + lr] = nr[e];
      wis[(lseg + e) * RGT_OC + lr] = ni[e];
    }
    __syncthreads();
    if (k0 + RGT_KC < bs) fetch(k0 + RGT_KC);
    const float* ub = u + (tg * 4) * bsp + k0;
#pragma unroll 8
    for (int in = 0; in < RGT_KC; ++in) {
      const float a = wrs[in * RGT_OC + o], b = wis[in * RGT_OC + o];
#pragma unroll
      for (int tk = 0; tk < 4; ++tk) {
        const float uu = ub[tk * bsp + in];
        ar[tk] = fmaf(a, uu, ar[tk]);
        ai[tk] = fmaf(b, uu, ai[tk]);
      }
    }
  }
  if (o0 + o < bs) {
    const int c = blk * bs + o0 + o;
    const float br = gates_b[(size_t)blk * bs + o0 + o], bi = gates_b[(size_t)(nb + blk) * bs + o0 + o];
    const float sp = softplusf_(lam[c]);
#pragma unroll
    for (int tk = 0; tk < 4; ++tk) {
      const int tt = tg * 4 + tk, t = t0 + tt;
      if (t < nt) {
        const float r = sigmoidf_(ar[tk] + br), g = sigmoidf_(ai[tk] + bi);
        const float loga = -c0 * r * sp;
        a_out[(size_t)t * C + c] = expf(loga);
        b_out[(size_t)t * C + c] = sqrtf(-expm1f(2.0f * loga)) * g * u[tt * bsp + o0 + o];
      }
    }
  }
}

// Long steps of a bfloat16 engine take the gates' block-diagonal products to the matrix cores
// without giving up 32-bit inputs: `rglru_conv_split` leaves u in float32 and as two bfloat16
// numbers hi + lo = u (to 16 bits of mantissa), the library multiplies both by the bfloat16
// weights with float32 sums, and `rglru_gates_finish` adds the two products and forms a_t and
// the input term exactly as the kernels above do.
template <typename T>
__global__ __launch_bounds__(256) void rglru_conv_split_kernel(
    const T* __restrict__ yx, int stride, int xoff, const float* __restrict__ xbias,
    const float* __restrict__ taps, const float* __restrict__ conv_bias, int K,
    const float* __restrict__ conv_state, const int* __restrict__ cu_q, const int* __restrict__ slots,
    int batch, int nt, int C, float* __restrict__ u_out, bf16_t* __restrict__ hi, bf16_t* __restrict__ lo) {
  const int t = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= C) return;
  const int b = seq_of_token_r(cu_q, batch, t);
  const int start = cu_q[b];
  const float* cs = conv_state + ((size_t)slots[b] * (K - 1)) * C;
  float acc = conv_bias[c];
  for (int j = 0; j < K; ++j) {
    const int tp = t - (K - 1 - j);
    float xin;
    if (tp >= start) xin = to_f32(yx[(size_t)tp * stride + xoff + c]) + xbias[c];
    else xin = cs[(size_t)(K - 1 + (tp - start)) * C + c];
    acc = fmaf(taps[(size_t)c * K + j], xin, acc);
  }
  const size_t at = (size_t)t * C + c;
  u_out[at] = acc;
  const bf16_t h = from_f32<bf16_t>(acc);
  hi[at] = h;
  lo[at] = from_f32<bf16_t>(acc - to_f32(h));
}

__global__ __launch_bounds__(256) void rglru_gates_finish_kernel(
    const float* __restrict__ g, const float* __restrict__ u, const float* __restrict__ gates_b,
    const float* __restrict__ lam, float c0, int nt, int C, int nb, float* __restrict__ a_out,
    float* __restrict__ b_out) {
  // g: [2 gates][nb][2 halves * nt][bs]: the products of hi (rows 0..nt) and lo (rows nt..2nt)
  const int t = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= C) return;
  const int bs = C / nb, blk = c / bs, cc = c - blk * bs;
  const size_t gate = (size_t)nb * 2 * nt * bs;
  const size_t at = ((size_t)blk * 2 * nt + t) * bs + cc, half = (size_t)nt * bs;
  const float zr = (g[at] + g[at + half]) + gates_b[(size_t)blk * bs + cc];
  const float zi = (g[gate + at] + g[gate + at + half]) + gates_b[(size_t)(nb + blk) * bs + cc];
  const float r = sigmoidf_(zr), gi = sigmoidf_(zi);
  const float loga = -c0 * r * softplusf_(lam[c]);
  a_out[(size_t)t * C + c] = expf(loga);
  b_out[(size_t)t * C + c] = sqrtf(-expm1f(2.0f * loga)) * gi * u[(size_t)t * C + c];
}

extern "C" int ta_rglru_conv_split(hipStream_t stream, int dtype, const void* yx, int stride, int xoff,
                                   const float* xbias, const float* taps, const float* conv_bias, int K,
                                   const float* conv_state, const int* cu_q, const int* slots, int batch,
                                   int nt, int C, float* u_out, void* hi, void* lo) {
  TA_REQUIRE(batch > 0 && nt >= batch && nt <= 65535 && C > 0 && K >= 1, "ta_rglru_conv_split: bad sizes");
  dim3 g((C + 255) / 256, nt);
  if (dtype == TA_F32)
    rglru_conv_split_kernel<float><<<g, 256, 0, stream>>>((const float*)yx, stride, xoff, xbias, taps, conv_bias, K,
        conv_state, cu_q, slots, batch, nt, C, u_out, (bf16_t*)hi, (bf16_t*)lo);
  else if (dtype == TA_BF16)
    rglru_conv_split_kernel<bf16_t><<<g, 256, 0, stream>>>((const bf16_t*)yx, stride, xoff, xbias, taps, conv_bias, K,
        conv_state, cu_q, slots, batch, nt, C, u_out, (bf16_t*)hi, (bf16_t*)lo);
  else
    return ta_fail("ta_rglru_conv_split: unknown dtype %d", dtype);
  return ta_check_launch("ta_rglru_conv_split");
}

extern "C" int ta_rglru_gates_finish(hipStream_t stream, const float* g, const float* u, const float* gates_b,
                                     const float* lam, float c0, int nt, int C, int nb, float* a_out,
                                     float* b_out) {
  TA_REQUIRE(nt > 0 && nt <= 65535 && C > 0 && nb > 0 && C % nb == 0, "ta_rglru_gates_finish: bad sizes");
  dim3 gr((C + 255) / 256, nt);
  rglru_gates_finish_kernel<<<gr, 256, 0, stream>>>(g, u, gates_b, lam, c0, nt, C, nb, a_out, b_out);
  return ta_check_launch("ta_rglru_gates_finish");
}

// yx: [nt, stride] rows holding the y branch at column 0 and the x branch at column xoff (C each);
// xbias [C]; taps [C, K]; conv_state [slots, K-1, C] float32 (inputs of the last K-1 tokens);
// gates_w [2*nb, bs, bs] (recurrence gate blocks, then input gate blocks), gates_b [2*nb, bs];
// a_out, b_out: [nt, C] float32.
extern "C" int ta_rglru_gates(hipStream_t stream, int dtype, int wdtype, const void* yx, int stride, int xoff,
                              const float* xbias, const float* taps, const float* conv_bias, int K,
                              const float* conv_state, const void* gates_w, const float* gates_b,
                              const float* lam, float c0, const int* cu_q, const int* slots, int batch,
                              int nt, int C, int nb, float* a_out, float* b_out) {
  TA_REQUIRE(batch > 0 && nt >= batch && C > 0 && nb > 0 && C % nb == 0 && K >= 1,
             "ta_rglru_gates: bad sizes nt=%d C=%d blocks=%d taps=%d", nt, C, nb, K);
  TA_REQUIRE(nb <= 65535, "ta_rglru_gates: too many blocks");
  const int bs = C / nb;
  const int bsp = (bs + RGT_KC - 1) / RGT_KC * RGT_KC;
  const size_t lds_tiled = ((size_t)RGT_TT * bsp + 2 * RGT_KC * RGT_OC) * sizeof(float);
  const int tiles = (bs + RGT_OC - 1) / RGT_OC;
  if (lds_tiled <= 64000 && (long long)nb * tiles <= 65535) {
    dim3 gt((nt + RGT_TT - 1) / RGT_TT, nb * tiles);
#define RGT_LAUNCH(T, TW)                                                                              \
  rglru_gates_tiled_kernel<T, TW><<<gt, 256, lds_tiled, stream>>>((const T*)yx, stride, xoff, xbias, taps, conv_bias, K, \
      conv_state, (const TW*)gates_w, gates_b, lam, c0, cu_q, slots, batch, nt, C, nb, bsp, a_out, b_out)
    if (dtype == TA_F32 && wdtype == TA_F32) RGT_LAUNCH(float, float);
    else if (dtype == TA_BF16 && wdtype == TA_BF16) RGT_LAUNCH(bf16_t, bf16_t);
    else if (dtype == TA_BF16 && wdtype == TA_F32) RGT_LAUNCH(bf16_t, float);
    else return ta_fail("ta_rglru_gates: unsupported dtypes %d / %d", dtype, wdtype);
#undef RGT_LAUNCH
    return ta_check_launch("ta_rglru_gates");
  }
  const size_t lds = (size_t)RG_TT * bs * sizeof(float);
  TA_REQUIRE(lds <= 60000, "ta_rglru_gates: blocks of %d channels do not fit", bs);
  dim3 g((nt + RG_TT - 1) / RG_TT, nb);
#define RG_LAUNCH(T, TW)                                                                          \
  rglru_gates_kernel<T, TW><<<g, 256, lds, stream>>>((const T*)yx, stride, xoff, xbias, taps, conv_bias, K, \
      conv_state, (const TW*)gates_w, gates_b, lam, c0, cu_q, slots, batch, nt, C, nb, a_out, b_out)
  if (dtype == TA_F32 && wdtype == TA_F32) RG_LAUNCH(float, float);
  else if (dtype == TA_BF16 && wdtype == TA_BF16) RG_LAUNCH(bf16_t, bf16_t);
  else if (dtype == TA_BF16 && wdtype == TA_F32) RG_LAUNCH(bf16_t, float);
  else return ta_fail("ta_rglru_gates: unsupported dtypes %d / %d", dtype, wdtype);
#undef RG_LAUNCH
  return ta_check_launch("ta_rglru_gates");
}

// ------------------------------------------------------------------ rglru: scan
template <typename T>
__global__ __launch_bounds__(256) void rglru_scan_kernel(
    const T* __restrict__ yx, int stride, int xoff, const float* __restrict__ ybias,
    const float* __restrict__ xbias, const float* __restrict__ a_in, const float* __restrict__ b_in,
    float* __restrict__ state, float* __restrict__ conv_state, int K, const int* __restrict__ cu_q,
    const int* __restrict__ slots, int C, T* __restrict__ out) {
  const int b = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= C) return;
  const int start = cu_q[b], end = cu_q[b + 1];
  const size_t slot = (size_t)slots[b];
  float S = state[slot * C + c];
  const float yb = ybias[c];
  int t = start;
  for (; t + 4 <= end; t += 4) {
    float a[4], bb[4], y[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      a[i] = a_in[(size_t)(t + i) * C + c];
      bb[i] = b_in[(size_t)(t + i) * C + c];
      y[i] = to_f32(yx[(size_t)(t + i) * stride + c]);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      S = fmaf(a[i], S, bb[i]);
      out[(size_t)(t + i) * C + c] = from_f32<T>(S * gelu_tanhf_(y[i] + yb));
    }
  }
  for (; t < end; ++t) {
    S = fmaf(a_in[(size_t)t * C + c], S, b_in[(size_t)t * C + c]);
    out[(size_t)t * C + c] = from_f32<T>(S * gelu_tanhf_(to_f32(yx[(size_t)t * stride + c]) + yb));
  }
  state[slot * C + c] = S;
  // the convolution's memory: inputs of the sequence's last K-1 tokens, oldest first
  const int n = end - start;
  float* cs = conv_state + slot * (size_t)(K - 1) * C;
  const float xb = xbias[c];
  for (int j = 0; j < K - 1; ++j) {
    const int src = j + n;            // index into (old memory, then this step's tokens)
    float v;
    if (src < K - 1) v = cs[(size_t)src * C + c];
    else v = to_f32(yx[(size_t)(start + src - (K - 1)) * stride + xoff + c]) + xb;
    cs[(size_t)j * C + c] = v;
  }
}

// ------------------------------------------------------------------ rglru: scan of long steps
// A step that brings many tokens per sequence is cut into segments of RG_SEG tokens that are
// scanned side by side: `rglru_local_kernel` scans each segment from S = 0 and leaves, in place
// of (a_t, b_t), the product of the decays since the segment's start and the locally scanned
// value; `rglru_apply_kernel` forms the state at its segment's start from the segments in front
// of it (S' = P_last S + local_last, in order) and finishes S_t = local_t + P_t S_start.
#define RG_SEG 64

__global__ __launch_bounds__(256) void rglru_local_kernel(float* __restrict__ a_io, float* __restrict__ b_io,
                                                          const float* __restrict__ state, float* __restrict__ s0,
                                                          const int* __restrict__ cu_q,
                                                          const int* __restrict__ slots, int C) {
  const int b = blockIdx.z, seg = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x;
  const int start = cu_q[b] + seg * RG_SEG, end = min(cu_q[b + 1], start + RG_SEG);
  if (c >= C || start >= end) return;
  // the state as the step found it, for every segment's workgroup of the next kernel (whose
  // last segment overwrites the state itself)
  if (seg == 0) s0[(size_t)b * C + c] = state[(size_t)slots[b] * C + c];
  float S = 0.f, P = 1.f;
  int t = start;
  for (; t + 8 <= end; t += 8) {
    float a[8], bb[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      a[i] = a_io[(size_t)(t + i) * C + c];
      bb[i] = b_io[(size_t)(t + i) * C + c];
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      S = fmaf(a[i], S, bb[i]);
      P *= a[i];
      a_io[(size_t)(t + i) * C + c] = P;
      b_io[(size_t)(t + i) * C + c] = S;
    }
  }
  for (; t < end; ++t) {
    S = fmaf(a_io[(size_t)t * C + c], S, b_io[(size_t)t * C + c]);
    P *= a_io[(size_t)t * C + c];
    a_io[(size_t)t * C + c] = P;
    b_io[(size_t)t * C + c] = S;
  }
}

template <typename T>
__global__ __launch_bounds__(256) void rglru_apply_kernel(
    const T* __restrict__ yx, int stride, int xoff, const float* __restrict__ ybias,
    const float* __restrict__ xbias, const float* __restrict__ p_in, const float* __restrict__ l_in,
    const float* __restrict__ s0, float* __restrict__ state, float* __restrict__ conv_state, int K,
    const int* __restrict__ cu_q,
    const int* __restrict__ slots, int C, T* __restrict__ out) {
  const int b = blockIdx.z, seg = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x;
  const int first = cu_q[b], last = cu_q[b + 1];
  const int start = first + seg * RG_SEG, end = min(last, start + RG_SEG);
  if (c >= C || start >= end) return;
  const size_t slot = (size_t)slots[b];
  float S0 = s0[(size_t)b * C + c];
  for (int s = 0; s < seg; ++s) {              // the segments in front, in order
    const size_t e = (size_t)(first + (s + 1) * RG_SEG - 1) * C + c;
    S0 = fmaf(p_in[e], S0, l_in[e]);
  }
  const float yb = ybias[c];
  float S = S0;
  for (int t = start; t < end; ++t) {
    S = fmaf(p_in[(size_t)t * C + c], S0, l_in[(size_t)t * C + c]);
    out[(size_t)t * C + c] = from_f32<T>(S * gelu_tanhf_(to_f32(yx[(size_t)t * stride + c]) + yb));
  }
  if (end != last) return;
  // the sequence's last segment leaves the state and the convolution's memory
  state[slot * C + c] = S;
  const int n = last - first;
  float* cs = conv_state + slot * (size_t)(K - 1) * C;
  const float xb = xbias[c];
  for (int j = 0; j < K - 1; ++j) {
    const int src = j + n;
    float v;
    if (src < K - 1) v = cs[(size_t)src * C + c];
    else v = to_f32(yx[(size_t)(first + src - (K - 1)) * stride + xoff + c]) + xb;
    cs[(size_t)j * C + c] = v;
  }
}

// state [slots, C] float32; out [nt, C]. Runs after ta_rglru_gates of the same step. a_io, b_io
// [nt, C]: what ta_rglru_gates left; overwritten when the step is long (max_qlen > RG_SEG: the
// segments are then scanned side by side, and s0 [batch, C] float32 is scratch for that).
extern "C" int ta_rglru_scan(hipStream_t stream, int dtype, const void* yx, int stride, int xoff,
                             const float* ybias, const float* xbias, float* a_io, float* b_io,
                             float* state, float* conv_state, int K, const int* cu_q, const int* slots,
                             int batch, int max_qlen, int C, float* s0, void* out) {
  TA_REQUIRE(batch > 0 && batch <= 65535 && C > 0 && K >= 1 && max_qlen >= 1, "ta_rglru_scan: bad sizes");
  if (max_qlen > RG_SEG) {
    const int segs = (max_qlen + RG_SEG - 1) / RG_SEG;
    TA_REQUIRE(segs <= 65535 && s0 != nullptr, "ta_rglru_scan: step too long, or no scratch");
    dim3 g((C + 255) / 256, segs, batch);
    rglru_local_kernel<<<g, 256, 0, stream>>>(a_io, b_io, state, s0, cu_q, slots, C);
    if (dtype == TA_F32)
      rglru_apply_kernel<float><<<g, 256, 0, stream>>>((const float*)yx, stride, xoff, ybias, xbias, a_io, b_io, s0,
                                                      state, conv_state, K, cu_q, slots, C, (float*)out);
    else if (dtype == TA_BF16)
      rglru_apply_kernel<bf16_t><<<g, 256, 0, stream>>>((const bf16_t*)yx, stride, xoff, ybias, xbias, a_io, b_io, s0,
                                                       state, conv_state, K, cu_q, slots, C, (bf16_t*)out);
    else
      return ta_fail("ta_rglru_scan: unknown dtype %d", dtype);
    return ta_check_launch("ta_rglru_scan");
  }
  dim3 g((C + 255) / 256, batch);
  if (dtype == TA_F32)
    rglru_scan_kernel<float><<<g, 256, 0, stream>>>((const float*)yx, stride, xoff, ybias, xbias, a_io, b_io, state,
                                                   conv_state, K, cu_q, slots, C, (float*)out);
  else if (dtype == TA_BF16)
    rglru_scan_kernel<bf16_t><<<g, 256, 0, stream>>>((const bf16_t*)yx, stride, xoff, ybias, xbias, a_io, b_io, state,
                                                    conv_state, K, cu_q, slots, C, (bf16_t*)out);
  else
    return ta_fail("ta_rglru_scan: unknown dtype %d", dtype);
  return ta_check_launch("ta_rglru_scan");
}

// ------------------------------------------------------------------ gla: decay per key channel
template <typename T, typename TW>
__global__ __launch_bounds__(256) void gla_decay_kernel(const T* __restrict__ proj, int stride, int aoff, int rank,
                                                        const TW* __restrict__ a2, const float* __restrict__ a2b,
                                                        float inv_tau, int n, float* __restrict__ alpha,
                                                        int mode) {
  extern __shared__ float low[];          // [rank]
  const size_t t = blockIdx.x;
  for (int r = threadIdx.x; r < rank; r += 256) {
    const float v = to_f32(proj[t * stride + aoff + r]);
    low[r] = mode == 1 ? tanhf(v) : v;
  }
  __syncthreads();
  for (int c = blockIdx.y * 256 + threadIdx.x; c < n; c += gridDim.y * 256) {
    const TW* w = a2 + (size_t)c * rank;
    float z = a2b[c];
    for (int r = 0; r < rank; ++r) z = fmaf(to_f32(w[r]), low[r], z);
    if (mode == 1) {                      // the double-exponential decay: exp(-exp(z)), z from tanh(low)
      alpha[t * n + c] = expf(-expf(z));
      continue;
    }
    // sigmoid(z)^(1/tau) = exp(log sigmoid(z) / tau), log sigmoid(z) = min(z, 0) - log1p(exp(-|z|))
    alpha[t * n + c] = expf((fminf(z, 0.f) - log1pf(expf(-fabsf(z)))) * inv_tau);
  }
}

// ------------------------------------------------------------------ gla: recurrence
// A workgroup owns GLA_RT key channels x GLA_CT value columns of one (sequence, head); a thread
// keeps 4 x 2 entries of S in registers, so every operand it reads from LDS feeds two or four
// multiply-adds. A chunk's operands are staged in LDS while the next chunk's are already on
// their way from memory. The readout q.S is summed over a workgroup's rows here and over the
// workgroups that share a head's columns by `gla_out` (o_out holds one plane per group of
// GLA_RT key channels).
// GLA_TC tokens are staged together: 32 for prompts, 8 for steps of few tokens per sequence
// (a chunk always costs all of its turns)
#define GLA_RT 32     // key channels per workgroup
#define GLA_CT 64     // value columns per workgroup

template <int GLA_TC>
struct GlaOperands {  // what one thread brings in for a chunk
  float q[GLA_TC * GLA_RT / 256], k[GLA_TC * GLA_RT / 256], a[GLA_TC * GLA_RT / 256], v[GLA_TC * GLA_CT / 256];
};

// BONUS: the readout comes BEFORE the update and gives the current token a weight of its own,
// o_t = (S_{t-1} + diag(bonus) k_t v_t^T)^T q_t, then S_t = diag(alpha_t) S_{t-1} + k_t v_t^T.
template <typename T, int GLA_TC, bool BONUS>
__global__ __launch_bounds__(256) void gla_recurrent_kernel(
    const T* __restrict__ proj, int stride, int qoff, int koff, int voff, const float* __restrict__ alpha,
    float qscale, float* __restrict__ state, const int* __restrict__ cu_q, const int* __restrict__ slots,
    int H, int dk, int dv, int col_tiles, size_t plane, float* __restrict__ o_out,
    const float* __restrict__ bonus, const float* __restrict__ head_decay,
    int qk_share = 1, const float* __restrict__ tok_decay = nullptr,
    const float* __restrict__ tok_kscale = nullptr) {
  __shared__ float sq[GLA_TC][GLA_RT], sk[GLA_TC][GLA_RT], sa[GLA_TC][GLA_RT];
  __shared__ float sv[GLA_TC][GLA_CT];
  __shared__ float part[GLA_TC][4][GLA_CT];
  constexpr int NQ = GLA_TC * GLA_RT / 256, NV = GLA_TC * GLA_CT / 256;
  const int b = blockIdx.x, h = blockIdx.y;
  const int rpart = blockIdx.z / col_tiles, ctile = blockIdx.z % col_tiles;
  const int row0 = rpart * GLA_RT, col0 = ctile * GLA_CT;
  const int start = cu_q[b], end = cu_q[b + 1];
  const size_t slot = (size_t)slots[b];
  const int tid = threadIdx.x;
  const int rg = tid / 32, cg = tid % 32;          // rows rg*4.., columns cg*2..
  float* st = state + ((slot * H + h) * dk) * (size_t)dv;
  float S[4][2];
#pragma unroll
  for (int r = 0; r < 4; ++r)
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      const int i = row0 + rg * 4 + r, j = col0 + cg * 2 + c;
      S[r][c] = (i < dk && j < dv) ? st[(size_t)i * dv + j] : 0.f;
    }
  float bu[4] = {0.f, 0.f, 0.f, 0.f};
  if (BONUS) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int i = row0 + rg * 4 + r;
      bu[r] = i < dk ? bonus[h * dk + i] : 0.f;
    }
  }
  // one fixed decay for all key channels of the head (``alpha`` is then not read)
  const float fixed = head_decay ? head_decay[h] : 0.f;
  // qk_share consecutive heads read the same q and k (one group of them); tok_decay / tok_kscale
  // [nt, H]: one decay for all key channels of (token, head), and a factor on that token's key
  const int hq = h / qk_share;
  // Loads are asked for two chunks ahead (a trip to memory takes longer than a chunk's
  // arithmetic); a position that is not there reads a harmless address and is replaced.
  auto fetch = [&](GlaOperands<GLA_TC>& o, int t0) {
#pragma unroll
    for (int e = 0; e < NQ; ++e) {
      const int idx = tid + 256 * e, tt = idx / GLA_RT, i = row0 + idx % GLA_RT;
      const bool ok = t0 + tt < end && i < dk;
      const size_t row = (size_t)(ok ? t0 + tt : start);
      const int ii = ok ? i : 0;
      const float qv = to_f32(proj[row * stride + qoff + hq * dk + ii]);
      const float kv = to_f32(proj[row * stride + koff + hq * dk + ii]);
      const float av = head_decay ? fixed : tok_decay ? tok_decay[row * H + h]
                                                      : alpha[row * ((size_t)H * dk) + h * dk + ii];
      const float ks = tok_kscale ? tok_kscale[row * H + h] : 1.f;
      o.q[e] = ok ? qv * qscale : 0.f;
      o.k[e] = ok ? kv * ks : 0.f;
      o.a[e] = ok ? av : 1.f;           // a token that is not there leaves S as it is
    }
#pragma unroll
    for (int e = 0; e < NV; ++e) {
      const int idx = tid + 256 * e, tt = idx / GLA_CT, j = col0 + idx % GLA_CT;
      const bool ok = t0 + tt < end && j < dv;
      const float vv = to_f32(proj[(size_t)(ok ? t0 + tt : start) * stride + voff + h * dv + (ok ? j : 0)]);
      o.v[e] = ok ? vv : 0.f;
    }
  };
  auto turn = [&](GlaOperands<GLA_TC>& o, int t0) {
    const int n = end - t0 < GLA_TC ? end - t0 : GLA_TC;
#pragma unroll
    for (int e = 0; e < NQ; ++e) {
      const int idx = tid + 256 * e;
      (&sq[0][0])[idx] = o.q[e];
      (&sk[0][0])[idx] = o.k[e];
      (&sa[0][0])[idx] = o.a[e];
    }
#pragma unroll
    for (int e = 0; e < NV; ++e) (&sv[0][0])[tid + 256 * e] = o.v[e];
    __syncthreads();
    if (t0 + 2 * GLA_TC < end) fetch(o, t0 + 2 * GLA_TC);
    // all GLA_TC tokens always (those past the end carry k = 0, alpha = 1), in groups of eight
    // whose count is fixed: the compiler asks for the next tokens' operands while it works on
    // this one, and the readouts stay in registers until the group is done, so only the update
    // of S itself is a chain.
#pragma unroll 1
    for (int g0 = 0; g0 < GLA_TC; g0 += 8) {
      float p0[8], p1[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int tt = g0 + u;
        const float4 q4 = *reinterpret_cast<const float4*>(&sq[tt][rg * 4]);
        const float4 k4 = *reinterpret_cast<const float4*>(&sk[tt][rg * 4]);
        const float4 a4 = *reinterpret_cast<const float4*>(&sa[tt][rg * 4]);
        const float2 v2 = *reinterpret_cast<const float2*>(&sv[tt][cg * 2]);
        const float qs[4] = {q4.x, q4.y, q4.z, q4.w}, ks[4] = {k4.x, k4.y, k4.z, k4.w};
        const float as[4] = {a4.x, a4.y, a4.z, a4.w};
        float a0 = 0.f, a1 = 0.f;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          if (BONUS) {
            const float kv0 = ks[r] * v2.x, kv1 = ks[r] * v2.y;
            a0 = fmaf(fmaf(bu[r], kv0, S[r][0]), qs[r], a0);
            a1 = fmaf(fmaf(bu[r], kv1, S[r][1]), qs[r], a1);
            S[r][0] = fmaf(as[r], S[r][0], kv0);
            S[r][1] = fmaf(as[r], S[r][1], kv1);
          } else {
            S[r][0] = fmaf(as[r], S[r][0], ks[r] * v2.x);
            S[r][1] = fmaf(as[r], S[r][1], ks[r] * v2.y);
            a0 = fmaf(S[r][0], qs[r], a0);
            a1 = fmaf(S[r][1], qs[r], a1);
          }
        }
        p0[u] = a0;
        p1[u] = a1;
      }
      // the two row groups of a wave, then the four waves through LDS
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const float a0 = p0[u] + __shfl_xor(p0[u], 32, TA_WAVE);
        const float a1 = p1[u] + __shfl_xor(p1[u], 32, TA_WAVE);
        if ((tid & 32) == 0) {
          part[g0 + u][tid / 64][cg * 2] = a0;
          part[g0 + u][tid / 64][cg * 2 + 1] = a1;
        }
      }
    }
    __syncthreads();
    for (int idx = tid; idx < n * GLA_CT; idx += 256) {
      const int tt = idx / GLA_CT, c = idx % GLA_CT;
      if (col0 + c < dv)
        o_out[rpart * plane + ((size_t)(t0 + tt) * H + h) * dv + col0 + c] =
            (part[tt][0][c] + part[tt][1][c]) + (part[tt][2][c] + part[tt][3][c]);
    }
    // The next turn's stores into sq/sk/sa/sv follow the barrier above, which every thread
    // passes only after its last read of them; `part` is read here and written again only
    // behind the next turn's first barrier.
  };
  GlaOperands<GLA_TC> even, odd;
  if (start < end) fetch(even, start);
  if (start + GLA_TC < end) fetch(odd, start + GLA_TC);
  for (int t0 = start; t0 < end; t0 += 2 * GLA_TC) {
    turn(even, t0);
    if (t0 + GLA_TC < end) turn(odd, t0 + GLA_TC);
  }
#pragma unroll
  for (int r = 0; r < 4; ++r)
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      const int i = row0 + rg * 4 + r, j = col0 + cg * 2 + c;
      if (i < dk && j < dv) st[(size_t)i * dv + j] = S[r][c];
    }
}

extern "C" int ta_gla_row_parts(int dk) { return (dk + GLA_RT - 1) / GLA_RT; }

// proj: [nt, stride] rows holding q (H*dk) at qoff, k (H*dk) at koff, v (H*dv) at voff and the
// low-rank decay input (rank) at aoff. a2: [H*dk, rank], a2b [H*dk]. alpha: scratch [nt, H*dk]
// float32. state: [slots, H, dk, dv] float32. o_out: [ta_gla_row_parts(dk), nt, H, dv] float32,
// planes that add up to the readout (not yet normalised).
static int gla_recurrent_launch(hipStream_t stream, int dtype, int wdtype, const void* proj, int stride,
                                int qoff, int koff, int voff, const void* low, int low_stride, int aoff, int rank,
                                const void* a2, const float* a2b, float inv_tau, float qscale, float* alpha,
                                float* state, const int* cu_q, const int* slots, int batch, int nt, int H, int dk,
                                int dv, float* o_out, int mode, const float* bonus,
                                const float* head_decay = nullptr, int qk_share = 1,
                                const float* tok_decay = nullptr, const float* tok_kscale = nullptr) {
  TA_REQUIRE(batch > 0 && batch <= 65535 && H > 0 && H <= 65535 && nt >= batch,
             "ta_gla_recurrent: bad batch %d / heads %d / tokens %d", batch, H, nt);
  TA_REQUIRE(qk_share >= 1 && H % qk_share == 0, "ta_gla_recurrent: %d heads do not form groups of %d", H, qk_share);
  TA_REQUIRE(dk >= 1 && dv >= 1 && (head_decay || tok_decay || (rank >= 1 && rank <= 8192)),
             "ta_gla_recurrent: bad widths %d / %d / %d", dk, dv, rank);
  const int parts = (dk + GLA_RT - 1) / GLA_RT, tiles = (dv + GLA_CT - 1) / GLA_CT;
  TA_REQUIRE(parts * tiles <= 65535, "ta_gla_recurrent: heads of %d x %d are too large", dk, dv);
  const int n = H * dk;
  dim3 gd(nt, (n + 255) / 256 < 64 ? (n + 255) / 256 : 64);
  const size_t lds = (size_t)rank * sizeof(float);
#define GLA_DECAY(T, TW) \
  gla_decay_kernel<T, TW><<<gd, 256, lds, stream>>>((const T*)low, low_stride, aoff, rank, (const TW*)a2, a2b, inv_tau, n, alpha, mode)
  if (head_decay || tok_decay) {
    TA_REQUIRE(dtype == TA_F32 || dtype == TA_BF16, "ta_gla_recurrent: unknown dtype %d", dtype);
  } else if (dtype == TA_F32 && wdtype == TA_F32) GLA_DECAY(float, float);
  else if (dtype == TA_BF16 && wdtype == TA_BF16) GLA_DECAY(bf16_t, bf16_t);
  else if (dtype == TA_BF16 && wdtype == TA_F32) GLA_DECAY(bf16_t, float);
  else return ta_fail("ta_gla_recurrent: unsupported dtypes %d / %d", dtype, wdtype);
#undef GLA_DECAY
  dim3 g(batch, H, parts * tiles);
  const size_t plane = (size_t)nt * H * dv;
  const bool few = nt <= 8 * batch;         // at most 8 tokens a sequence on average: short chunks
#define GLA_RUN(T, TC, B)                                                                                   \
  gla_recurrent_kernel<T, TC, B><<<g, 256, 0, stream>>>((const T*)proj, stride, qoff, koff, voff, alpha, qscale, \
                                                        state, cu_q, slots, H, dk, dv, tiles, plane, o_out, bonus, \
                                                        head_decay, qk_share, tok_decay, tok_kscale)
  if (bonus) {
    if (dtype == TA_F32) {
      if (few) GLA_RUN(float, 8, true); else GLA_RUN(float, 32, true);
    } else {
      if (few) GLA_RUN(bf16_t, 8, true); else GLA_RUN(bf16_t, 32, true);
    }
  } else if (dtype == TA_F32) {
    if (few) GLA_RUN(float, 8, false); else GLA_RUN(float, 32, false);
  } else {
    if (few) GLA_RUN(bf16_t, 8, false); else GLA_RUN(bf16_t, 32, false);
  }
#undef GLA_RUN
  return ta_check_launch("ta_gla_recurrent");
}

extern "C" int ta_gla_recurrent(hipStream_t stream, int dtype, int wdtype, const void* proj, int stride,
                                int qoff, int koff, int voff, int aoff, int rank, const void* a2,
                                const float* a2b, float inv_tau, float qscale, float* alpha, float* state,
                                const int* cu_q, const int* slots, int batch, int nt, int H, int dk, int dv,
                                float* o_out) {
  return gla_recurrent_launch(stream, dtype, wdtype, proj, stride, qoff, koff, voff, proj, stride, aoff, rank, a2,
                              a2b, inv_tau, qscale, alpha, state, cu_q, slots, batch, nt, H, dk, dv, o_out, 0,
                              nullptr);
}

// The recurrence with the readout before the update and a bonus for the current token (see
// BONUS above) and the decay exp(-exp(a2 tanh(low) + a2b)) per key channel. q, k, v sit at
// element offsets qoff, koff, voff of ``proj`` with ``stride`` elements between tokens (three
// planes of one buffer, or three column ranges of its rows); low: [nt, rank] rows of their own.
extern "C" int ta_wkv_recurrent(hipStream_t stream, int dtype, int wdtype, const void* proj, int stride,
                                int qoff, int koff, int voff, const void* low, int low_stride, int rank,
                                const void* a2, const float* a2b, const float* bonus, float* alpha,
                                float* state, const int* cu_q, const int* slots, int batch, int nt, int H,
                                int dk, int dv, float* o_out) {
  TA_REQUIRE(bonus != nullptr, "ta_wkv_recurrent: the bonus is required");
  return gla_recurrent_launch(stream, dtype, wdtype, proj, stride, qoff, koff, voff, low, low_stride, 0, rank, a2,
                              a2b, 1.0f, 1.0f, alpha, state, cu_q, slots, batch, nt, H, dk, dv, o_out, 1, bonus);
}

// The recurrence with ONE fixed decay per head, S_t = decay_h S_{t-1} + k_t v_t^T, o_t = S_t^T
// (qscale q_t): head_decay [H] float32 on the device; q, k, v at element offsets of the rows of
// ``proj`` as above. No decay input, no scratch for decays.
extern "C" int ta_decay_recurrent(hipStream_t stream, int dtype, const void* proj, int stride, int qoff, int koff,
                                  int voff, const float* head_decay, float qscale, float* state, const int* cu_q,
                                  const int* slots, int batch, int nt, int H, int dk, int dv, float* o_out) {
  TA_REQUIRE(head_decay != nullptr, "ta_decay_recurrent: the heads' decays are required");
  return gla_recurrent_launch(stream, dtype, dtype, proj, stride, qoff, koff, voff, nullptr, 0, 0, 0, nullptr,
                              nullptr, 1.0f, qscale, nullptr, state, cu_q, slots, batch, nt, H, dk, dv, o_out, 0,
                              nullptr, head_decay);
}

// ------------------------------------------------------------------ gla: head norm and output gate
template <typename T>
__global__ __launch_bounds__(64) void gla_out_kernel(const float* __restrict__ o, int parts, size_t plane,
                                                     const T* __restrict__ proj,
                                                     int stride, int goff, const float* __restrict__ w,
                                                     int wstride, float eps, int H, int dv, T* __restrict__ out,
                                                     int gate_act) {
  extern __shared__ float row[];          // [dv]
  const size_t t = blockIdx.x;
  const int h = blockIdx.y;
  const float* src = o + (t * H + h) * dv;
  float ss = 0.f;
  for (int c = threadIdx.x; c < dv; c += 64) {
    float v = src[c];
    for (int p = 1; p < parts; ++p) v += src[p * plane + c];
    row[c] = v;
    ss += v * v;
  }
  const float f = rsqrtf(wave_sum(ss) / (float)dv + eps);
  for (int c = threadIdx.x; c < dv; c += 64) {
    const float g = to_f32(proj[t * stride + goff + h * dv + c]);
    const float sg = 1.0f / (1.0f + expf(-g));
    const float wc = w ? w[h * wstride + c] : 1.0f;                        // no weight: the plain unit norm
    out[t * (size_t)(H * dv) + h * dv + c] = from_f32<T>(row[c] * f * wc * (gate_act == 1 ? sg : g * sg));
  }
}

// The same for wide heads (all heads normed as one row of thousands of columns): eight waves share
// a row, each thread keeps its columns in registers. Four planes are asked for at once, and the
// gate and the weight before the sum over the row is known, so that a row of a single-token step
// waits for memory twice, not once per plane.
template <typename T>
__global__ __launch_bounds__(512) void gla_out_wide_kernel(const float* __restrict__ o, int parts, size_t plane,
                                                           const T* __restrict__ proj, int stride,
                                                           const float* __restrict__ w, int wstride, float eps,
                                                           int H, int dv, T* __restrict__ out, int gate_act) {
  constexpr int PER = 8;                  // columns a thread can own: rows of up to 512 * PER
  __shared__ float red[8];
  const size_t t = blockIdx.x;
  const int h = blockIdx.y;
  const float* src = o + (t * H + h) * dv;
  float v[PER], g[PER], wc[PER];
#pragma unroll
  for (int i = 0; i < PER; ++i) v[i] = 0.f;
  for (int p0 = 0; p0 < parts; p0 += 4) {
    float a[4][PER];
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int i = 0; i < PER; ++i) {
        const int c = threadIdx.x + 512 * i;
        a[q][i] = (c < dv && p0 + q < parts) ? src[(size_t)(p0 + q) * plane + c] : 0.f;
      }
#pragma unroll
    for (int q = 0; q < 4; ++q)           // planes in order: the sum does not depend on how they are fetched
#pragma unroll
      for (int i = 0; i < PER; ++i) v[i] += a[q][i];
  }
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int c = threadIdx.x + 512 * i;
    g[i] = c < dv ? to_f32(proj[t * stride + h * dv + c]) : 0.f;
    wc[i] = (c < dv && w) ? w[h * wstride + c] : 1.0f;
  }
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < PER; ++i) ss += v[i] * v[i];
  ss = wave_sum(ss);
  if (threadIdx.x % TA_WAVE == 0) red[threadIdx.x / TA_WAVE] = ss;
  __syncthreads();
  const float f = rsqrtf((((red[0] + red[1]) + (red[2] + red[3])) + ((red[4] + red[5]) + (red[6] + red[7]))) / (float)dv + eps);
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int c = threadIdx.x + 512 * i;
    if (c < dv) {
      const float sg = 1.0f / (1.0f + expf(-g[i]));
      out[t * (size_t)(H * dv) + h * dv + c] = from_f32<T>(v[i] * f * wc[i] * (gate_act == 1 ? sg : g[i] * sg));
    }
  }
}

// o: [parts, nt, H, dv] float32 planes that add up to the readout; the gate's pre-activation sits
// at element goff of proj, ``stride`` elements between tokens; w [dv] shared by the heads
// (wstride 0) or [H, dv] (wstride dv); out [nt, H*dv] = rms_norm(o per head) * w * silu(gate).
// gate_act 0: silu(gate); 1: sigmoid(gate). w may be null (no weight).
extern "C" int ta_gla_out_act(hipStream_t stream, int dtype, const float* o, int parts, const void* proj, int stride,
                              long long goff, const float* w, int wstride, float eps, int nt, int H, int dv,
                              int gate_act, void* out) {
  TA_REQUIRE(nt >= 0 && H > 0 && H <= 65535 && dv > 0 && dv <= 15000 && parts >= 1, "ta_gla_out: bad sizes");
  TA_REQUIRE(gate_act == 0 || gate_act == 1, "ta_gla_out: unknown gate activation %d", gate_act);
  TA_REQUIRE(wstride == 0 || wstride == dv, "ta_gla_out: weight rows of %d for heads of %d", wstride, dv);
  if (nt == 0) return 0;
  dim3 g(nt, H);
  const size_t plane = (size_t)nt * H * dv, lds = (size_t)dv * sizeof(float);
  if (dv > 512 && dv <= 4096 && (dtype == TA_F32 || dtype == TA_BF16)) {
    if (dtype == TA_F32)
      gla_out_wide_kernel<float><<<g, 512, 0, stream>>>(o, parts, plane, (const float*)proj + goff, stride, w, wstride, eps, H, dv, (float*)out, gate_act);
    else
      gla_out_wide_kernel<bf16_t><<<g, 512, 0, stream>>>(o, parts, plane, (const bf16_t*)proj + goff, stride, w, wstride, eps, H, dv, (bf16_t*)out, gate_act);
    return ta_check_launch("ta_gla_out");
  }
  if (dtype == TA_F32)
    gla_out_kernel<float><<<g, 64, lds, stream>>>(o, parts, plane, (const float*)proj + goff, stride, 0, w, wstride, eps, H, dv, (float*)out, gate_act);
  else if (dtype == TA_BF16)
    gla_out_kernel<bf16_t><<<g, 64, lds, stream>>>(o, parts, plane, (const bf16_t*)proj + goff, stride, 0, w, wstride, eps, H, dv, (bf16_t*)out, gate_act);
  else
    return ta_fail("ta_gla_out: unknown dtype %d", dtype);
  return ta_check_launch("ta_gla_out");
}

extern "C" int ta_gla_out_w(hipStream_t stream, int dtype, const float* o, int parts, const void* proj, int stride,
                            long long goff, const float* w, int wstride, float eps, int nt, int H, int dv,
                            void* out) {
  TA_REQUIRE(w != nullptr, "ta_gla_out: the weight is required");
  return ta_gla_out_act(stream, dtype, o, parts, proj, stride, goff, w, wstride, eps, nt, H, dv, 0, out);
}

extern "C" int ta_gla_out(hipStream_t stream, int dtype, const float* o, int parts, const void* proj, int stride,
                          int goff, const float* w, float eps, int nt, int H, int dv, void* out) {
  return ta_gla_out_w(stream, dtype, o, parts, proj, stride, goff, w, 0, eps, nt, H, dv, out);
}

// ------------------------------------------------------------------ short causal convolution
// y_t[c] = act(bias_out[c] + sum_j taps[c][j] * u_{t-(K-1-j)}[c]) on a range of columns of the rows of
// ``in``; u = in + bias_in (a bias that belongs to the projection in front). Inputs before a
// sequence's first token of the step come from conv_state [slots, K-1, C] float32 (zero for a new
// sequence), which afterwards holds the sequence's last K-1 inputs. Sums are float32; act 0: none,
// 1: silu.
#define CONV_MAX_TAPS 8      // taps a thread keeps in registers; more go through the plain kernel
#define CONV_RUN 16          // tokens a thread of the prompt kernel walks

// the sequence that holds token t: the last b with cu_q[b] <= t
__device__ __forceinline__ int sequence_of(const int* __restrict__ cu_q, int batch, int t) {
  int lo = 0, hi = batch - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (cu_q[mid] <= t) lo = mid; else hi = mid - 1;
  }
  return lo;
}

__device__ __forceinline__ float conv_act(float v, int act) { return act == 1 ? v / (1.0f + expf(-v)) : v; }

// Prompts: a thread owns one channel and walks CONV_RUN consecutive tokens with the last K - 1 inputs
// in registers, so every input is read once; where the walk enters another sequence the registers
// are filled from that sequence's memory. The state is not written here.
template <typename T, int K>
__global__ __launch_bounds__(256) void causal_conv_run_kernel(
    const T* __restrict__ in, int stride, int off, const float* __restrict__ bias_in,
    const float* __restrict__ taps, const float* __restrict__ bias_out, const float* __restrict__ conv_state,
    const int* __restrict__ cu_q, const int* __restrict__ slots, int batch, int nt, int C, int act,
    T* __restrict__ out, int out_stride) {
  const int c = blockIdx.y * 256 + threadIdx.x;
  const int t0 = blockIdx.x * CONV_RUN;
  if (c >= C || t0 >= nt) return;
  float w[K], win[K > 1 ? K - 1 : 1];
#pragma unroll
  for (int j = 0; j < K; ++j) w[j] = taps[(size_t)c * K + j];
  const float bi = bias_in ? bias_in[c] : 0.f, bo = bias_out ? bias_out[c] : 0.f;
  int b = sequence_of(cu_q, batch, t0);
  int start = cu_q[b], end = cu_q[b + 1];
  // the K - 1 inputs in front of t0: rows of the step, or the sequence's memory
#pragma unroll
  for (int r = 0; r < K - 1; ++r) {
    const int src = t0 - (K - 1) + r;
    win[r] = src >= start ? to_f32(in[(size_t)src * stride + off + c]) + bi
                          : conv_state[((size_t)slots[b] * (K - 1) + (r + (t0 - start))) * C + c];
  }
  const int t1 = t0 + CONV_RUN < nt ? t0 + CONV_RUN : nt;
  for (int t = t0; t < t1; ++t) {
    if (t >= end) {                      // the next sequence begins: its memory takes the registers
      ++b;
      start = end;
      end = cu_q[b + 1];
#pragma unroll
      for (int r = 0; r < K - 1; ++r) win[r] = conv_state[((size_t)slots[b] * (K - 1) + r) * C + c];
    }
    const float u = to_f32(in[(size_t)t * stride + off + c]) + bi;
    float acc = bo;
#pragma unroll
    for (int j = 0; j < K - 1; ++j) acc = fmaf(w[j], win[j], acc);
    acc = fmaf(w[K - 1], u, acc);
#pragma unroll
    for (int j = 0; j + 1 < K - 1; ++j) win[j] = win[j + 1];
    if (K > 1) win[K - 2] = u;
    out[(size_t)t * out_stride + c] = from_f32<T>(conv_act(acc, act));
  }
}

// Any number of taps, one thread per (token, channel).
template <typename T>
__global__ __launch_bounds__(256) void causal_conv_kernel(
    const T* __restrict__ in, int stride, int off, const float* __restrict__ bias_in,
    const float* __restrict__ taps, const float* __restrict__ bias_out, const float* __restrict__ conv_state,
    const int* __restrict__ cu_q, const int* __restrict__ slots, int batch, int C, int K,
    int act, T* __restrict__ out, int out_stride) {
  const int t = blockIdx.x;
  const int b = sequence_of(cu_q, batch, t);
  const int start = cu_q[b];
  const size_t slot = (size_t)slots[b];
  for (int c = blockIdx.y * 256 + threadIdx.x; c < C; c += gridDim.y * 256) {
    const float bi = bias_in ? bias_in[c] : 0.f;
    float acc = bias_out ? bias_out[c] : 0.f;
    for (int j = 0; j < K; ++j) {
      const int src = t - (K - 1 - j);
      float u;
      if (src >= start) u = to_f32(in[(size_t)src * stride + off + c]) + bi;
      else u = conv_state[(slot * (K - 1) + (K - 1 - (start - src))) * C + c];
      acc = fmaf(taps[(size_t)c * K + j], u, acc);
    }
    out[(size_t)t * out_stride + c] = from_f32<T>(conv_act(acc, act));
  }
}

template <typename T>
__global__ __launch_bounds__(256) void conv_state_update_kernel(
    const T* __restrict__ in, int stride, int off, const float* __restrict__ bias_in, float* __restrict__ conv_state,
    const int* __restrict__ cu_q, const int* __restrict__ slots, int C, int K) {
  const int b = blockIdx.x;
  const int start = cu_q[b], n = cu_q[b + 1] - start;
  const size_t slot = (size_t)slots[b];
  float* st = conv_state + slot * (K - 1) * C;
  for (int c = blockIdx.y * 256 + threadIdx.x; c < C; c += gridDim.y * 256) {
    const float bi = bias_in ? bias_in[c] : 0.f;
    // new row r holds the input n - (K-1) + r of the step, or the old row r + n where that is negative;
    // rows are rewritten in ascending order and every read is of a row at or behind the one written
    for (int r = 0; r < K - 1; ++r) {
      const int src = n - (K - 1) + r;
      const float v = src >= 0 ? to_f32(in[(size_t)(start + src) * stride + off + c]) + bi : st[(size_t)(r + n) * C + c];
      st[(size_t)r * C + c] = v;
    }
  }
}

// Steps of single tokens (token b belongs to sequence b): a thread reads its channel's memory, forms
// the result and writes the memory back moved on by one, all in one kernel.
template <typename T, int K>
__global__ __launch_bounds__(256) void causal_conv_step_kernel(
    const T* __restrict__ in, int stride, int off, const float* __restrict__ bias_in,
    const float* __restrict__ taps, const float* __restrict__ bias_out, float* __restrict__ conv_state,
    const int* __restrict__ slots, int C, int act, T* __restrict__ out, int out_stride, int update) {
  const int b = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  float* st = conv_state + (size_t)slots[b] * (K - 1) * C + c;
  float win[K > 1 ? K - 1 : 1];
#pragma unroll
  for (int r = 0; r < K - 1; ++r) win[r] = st[(size_t)r * C];
  const float u = to_f32(in[(size_t)b * stride + off + c]) + (bias_in ? bias_in[c] : 0.f);
  float acc = bias_out ? bias_out[c] : 0.f;
#pragma unroll
  for (int j = 0; j < K - 1; ++j) acc = fmaf(taps[(size_t)c * K + j], win[j], acc);
  acc = fmaf(taps[(size_t)c * K + K - 1], u, acc);
  out[(size_t)b * out_stride + c] = from_f32<T>(conv_act(acc, act));
  if (update) {
#pragma unroll
    for (int r = 0; r + 1 < K - 1; ++r) st[(size_t)r * C] = win[r + 1];
    if (K > 1) st[(size_t)(K - 2) * C] = u;
  }
}

// in: [nt, stride] rows, the convolution reads columns off .. off + C; out: [nt, out_stride] rows,
// columns 0 .. C. taps [C, K] float32; bias_in, bias_out [C] float32 or null; conv_state [slots, K-1, C]
// float32 (null with K == 1: no memory). update 0: the state is left as it is. max_qlen: the most
// tokens a sequence brings (1: the single-token kernel).
extern "C" int ta_causal_conv(hipStream_t stream, int dtype, const void* in, int stride, int off,
                              const float* bias_in, const float* taps, const float* bias_out, float* conv_state,
                              const int* cu_q, const int* slots, int batch, int nt, int max_qlen, int C, int K,
                              int act, void* out, int out_stride, int update) {
  TA_REQUIRE(batch > 0 && batch <= 65535 && nt >= batch && nt <= 65535 * CONV_RUN && C >= 1 && K >= 1 && K <= 64,
             "ta_causal_conv: bad sizes batch=%d nt=%d channels=%d taps=%d", batch, nt, C, K);
  TA_REQUIRE(off >= 0 && stride >= off + C && out_stride >= C && (act == 0 || act == 1),
             "ta_causal_conv: columns %d..%d of rows of %d, out rows of %d, act %d", off, off + C, stride, out_stride, act);
  TA_REQUIRE(K == 1 || conv_state != nullptr, "ta_causal_conv: %d taps need the sequences' memory", K);
  TA_REQUIRE(dtype == TA_F32 || dtype == TA_BF16, "ta_causal_conv: unknown dtype %d", dtype);
  const int cb = (C + 255) / 256;
  TA_REQUIRE(cb <= 65535, "ta_causal_conv: too many channels");
  const bool single = max_qlen == 1 && nt == batch && K <= CONV_MAX_TAPS;
#define CONV_STEP(T, KK)                                                                                          \
  causal_conv_step_kernel<T, KK><<<dim3(batch, cb), 256, 0, stream>>>((const T*)in, stride, off, bias_in, taps, \
                                                                       bias_out, conv_state, slots, C, act, (T*)out, \
                                                                       out_stride, update)
#define CONV_RUN_K(T, KK)                                                                                      \
  causal_conv_run_kernel<T, KK><<<dim3((nt + CONV_RUN - 1) / CONV_RUN, cb), 256, 0, stream>>>(                 \
      (const T*)in, stride, off, bias_in, taps, bias_out, conv_state, cu_q, slots, batch, nt, C, act, (T*)out, out_stride)
#define CONV_BY_TAPS(WHAT, T)                \
  switch (K) {                               \
    case 1: WHAT(T, 1); break;               \
    case 2: WHAT(T, 2); break;               \
    case 3: WHAT(T, 3); break;               \
    case 4: WHAT(T, 4); break;               \
    case 5: WHAT(T, 5); break;               \
    case 6: WHAT(T, 6); break;               \
    case 7: WHAT(T, 7); break;               \
    default: WHAT(T, 8); break;              \
  }
  if (single) {
    if (dtype == TA_F32) { CONV_BY_TAPS(CONV_STEP, float) } else { CONV_BY_TAPS(CONV_STEP, bf16_t) }
    return ta_check_launch("ta_causal_conv");
  }
  if (K <= CONV_MAX_TAPS) {
    if (dtype == TA_F32) { CONV_BY_TAPS(CONV_RUN_K, float) } else { CONV_BY_TAPS(CONV_RUN_K, bf16_t) }
  } else {
    const int cbs = cb < 64 ? cb : 64;
    if (dtype == TA_F32)
      causal_conv_kernel<float><<<dim3(nt, cbs), 256, 0, stream>>>((const float*)in, stride, off, bias_in, taps, bias_out,
                                                                   conv_state, cu_q, slots, batch, C, K, act, (float*)out, out_stride);
    else
      causal_conv_kernel<bf16_t><<<dim3(nt, cbs), 256, 0, stream>>>((const bf16_t*)in, stride, off, bias_in, taps, bias_out,
                                                                    conv_state, cu_q, slots, batch, C, K, act, (bf16_t*)out, out_stride);
  }
  if (update && K > 1) {
    const int cbs = cb < 64 ? cb : 64;
    if (dtype == TA_F32)
      conv_state_update_kernel<float><<<dim3(batch, cbs), 256, 0, stream>>>((const float*)in, stride, off, bias_in, conv_state, cu_q, slots, C, K);
    else
      conv_state_update_kernel<bf16_t><<<dim3(batch, cbs), 256, 0, stream>>>((const bf16_t*)in, stride, off, bias_in, conv_state, cu_q, slots, C, K);
  }
#undef CONV_STEP
#undef CONV_RUN_K
#undef CONV_BY_TAPS
  return ta_check_launch("ta_causal_conv");
}

// ------------------------------------------------------------------ selective state space
// Step sizes and decays of every (token, head), float32: dt = softplus(raw + dt_bias[h]) (no clamp),
// decay = exp(-exp(a_log[h]) * dt).
template <typename T>
__global__ __launch_bounds__(256) void ssm_steps_kernel(const T* __restrict__ proj, int stride, int off,
                                                        const float* __restrict__ dt_bias,
                                                        const float* __restrict__ a_log, int nt, int H,
                                                        float* __restrict__ dt, float* __restrict__ decay) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= (size_t)nt * H) return;
  const size_t t = i / H;
  const int h = (int)(i - t * H);
  const float z = to_f32(proj[t * stride + off + h]) + dt_bias[h];
  const float sp = fmaxf(z, 0.f) + log1pf(expf(-fabsf(z)));
  dt[i] = sp;
  decay[i] = expf(-expf(a_log[h]) * sp);
}

extern "C" int ta_ssm_steps(hipStream_t stream, int dtype, const void* proj, int stride, int off,
                            const float* dt_bias, const float* a_log, int nt, int H, float* dt, float* decay) {
  TA_REQUIRE(nt >= 0 && H >= 1 && off >= 0 && stride >= off + H, "ta_ssm_steps: bad sizes nt=%d heads=%d", nt, H);
  if (nt == 0) return 0;
  const unsigned blocks = (unsigned)(((size_t)nt * H + 255) / 256);
  if (dtype == TA_F32)
    ssm_steps_kernel<float><<<blocks, 256, 0, stream>>>((const float*)proj, stride, off, dt_bias, a_log, nt, H, dt, decay);
  else if (dtype == TA_BF16)
    ssm_steps_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)proj, stride, off, dt_bias, a_log, nt, H, dt, decay);
  else return ta_fail("ta_ssm_steps: unknown dtype %d", dtype);
  return ta_check_launch("ta_ssm_steps");
}

// The recurrence S_t = decay_t S_{t-1} + dt_t B_t x_t^T, o_t = S_t^T C_t per head, with B and C shared
// by the ``share`` heads of a group: the kernel of gated linear attention with q = C, k = B, v = x,
// one decay per (token, head) and the step size as a factor on the key. decay, dt: [nt, H] float32.
extern "C" int ta_ssm_recurrent(hipStream_t stream, int dtype, const void* proj, int stride, int coff, int boff,
                                int xoff, int share, const float* decay, const float* dt, float* state,
                                const int* cu_q, const int* slots, int batch, int nt, int H, int N, int P,
                                float* o_out) {
  TA_REQUIRE(decay != nullptr && dt != nullptr, "ta_ssm_recurrent: decays and step sizes are required");
  return gla_recurrent_launch(stream, dtype, dtype, proj, stride, coff, boff, xoff, nullptr, 0, 0, 0, nullptr,
                              nullptr, 1.0f, 1.0f, nullptr, state, cu_q, slots, batch, nt, H, N, P, o_out, 0,
                              nullptr, nullptr, share, decay, dt);
}

// y = (sum of the readout's planes + skip[h] * x) * silu(z), cut into ``groups`` equal parts of the row,
// each divided by its own root mean square, times w: the gate comes BEFORE the norm. A workgroup of
// THREADS a (token, part); a thread keeps up to GGN_KEEP of the part's columns in registers (all planes
// asked for at once), so memory is read once; longer parts are formed a second time for the write.
// float32 inside. o: [parts, nt, n]; x at column xoff of xs rows, z at zoff of zs rows.
#define GGN_KEEP 8
template <typename T, int THREADS>
__global__ __launch_bounds__(THREADS) void gated_group_norm_kernel(
    const float* __restrict__ o, int parts, size_t plane, const T* __restrict__ xs, int x_stride, int xoff,
    const float* __restrict__ skip, int head_dim, const T* __restrict__ zs, int z_stride, int zoff,
    const float* __restrict__ w, float eps, int n, int groups, T* __restrict__ out) {
  __shared__ float red[THREADS / TA_WAVE];
  const size_t t = blockIdx.x;
  const int g = blockIdx.y, len = n / groups, c0 = g * len;
  auto value = [&](int c) {
    float y = 0.f;
    for (int p = 0; p < parts; ++p) y += o[p * plane + t * n + c];
    if (skip) y = fmaf(skip[c / head_dim], to_f32(xs[t * x_stride + xoff + c]), y);
    const float z = to_f32(zs[t * z_stride + zoff + c]);
    return y * (z / (1.0f + expf(-z)));
  };
  float keep[GGN_KEEP];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < GGN_KEEP; ++i) {
    const int c = c0 + threadIdx.x + i * THREADS;
    keep[i] = c < c0 + len ? value(c) : 0.f;
    ss = fmaf(keep[i], keep[i], ss);
  }
  for (int c = c0 + threadIdx.x + GGN_KEEP * THREADS; c < c0 + len; c += THREADS) {
    const float y = value(c);
    ss = fmaf(y, y, ss);
  }
  ss = wave_sum(ss);
  if (THREADS > TA_WAVE) {
    if (threadIdx.x % TA_WAVE == 0) red[threadIdx.x / TA_WAVE] = ss;
    __syncthreads();
    ss = 0.f;
#pragma unroll
    for (int i = 0; i < THREADS / TA_WAVE; ++i) ss += red[i];
  }
  const float f = rsqrtf(ss / (float)len + eps);
#pragma unroll
  for (int i = 0; i < GGN_KEEP; ++i) {
    const int c = c0 + threadIdx.x + i * THREADS;
    if (c < c0 + len) out[t * n + c] = from_f32<T>(keep[i] * f * (w ? w[c] : 1.f));
  }
  for (int c = c0 + threadIdx.x + GGN_KEEP * THREADS; c < c0 + len; c += THREADS)
    out[t * n + c] = from_f32<T>(value(c) * f * (w ? w[c] : 1.f));
}

extern "C" int ta_gated_group_norm(hipStream_t stream, int dtype, const float* o, int parts, const void* xs,
                                   int x_stride, int xoff, const float* skip, int head_dim, const void* zs,
                                   int z_stride, int zoff, const float* w, float eps, int nt, int n, int groups,
                                   void* out) {
  TA_REQUIRE(nt >= 0 && n >= 1 && groups >= 1 && groups <= 65535 && n % groups == 0 && parts >= 1,
             "ta_gated_group_norm: rows of %d in %d parts, %d planes", n, groups, parts);
  TA_REQUIRE(skip == nullptr || (head_dim >= 1 && n % head_dim == 0 && x_stride >= xoff + n),
             "ta_gated_group_norm: heads of %d in rows of %d", head_dim, n);
  TA_REQUIRE(z_stride >= zoff + n, "ta_gated_group_norm: gate rows of %d", z_stride);
  TA_REQUIRE(dtype == TA_F32 || dtype == TA_BF16, "ta_gated_group_norm: unknown dtype %d", dtype);
  if (nt == 0) return 0;
  dim3 g(nt, groups);
  const size_t plane = (size_t)nt * n;
  const int len = n / groups;
#define GGN(T, TH)                                                                                              \
  gated_group_norm_kernel<T, TH><<<g, TH, 0, stream>>>(o, parts, plane, (const T*)xs, x_stride, xoff, skip, head_dim, \
                                                       (const T*)zs, z_stride, zoff, w, eps, n, groups, (T*)out)
  if (dtype == TA_F32) {
    if (len <= 256) GGN(float, 64); else GGN(float, 256);
  } else {
    if (len <= 256) GGN(bf16_t, 64); else GGN(bf16_t, 256);
  }
#undef GGN
  return ta_check_launch("ta_gated_group_norm");
}
