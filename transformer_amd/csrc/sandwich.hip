// Kernels of blocks that norm a sublayer's RESULT before it joins the residual stream, and
// of the small things such blocks hang on the stream:
//
//   postnorm_add     : x += rms_norm(delta) * w   (w = the output norm's weight times the
//                      layer scale), optionally followed in the same pass by a copy of the
//                      new row in the engine's type and by the NEXT norm of the stream,
//                      out = rms_norm(x) * w_next, so that a row is read and written once
//   activation       : out = act(in) (* rows of a float32 side table), act one of gelu (erf),
//                      gelu (tanh), relu squared, silu
//
// All sums, norms and the stream itself are float32; one workgroup owns a row.
#include "common.h"

__device__ __forceinline__ float block_sum4(float v, float* red) {
  v = wave_sum(v);
  const int w = threadIdx.x / TA_WAVE;
  __syncthreads();
  if (threadIdx.x % TA_WAVE == 0) red[w] = v;
  __syncthreads();
  float s = 0.f;
  for (int i = 0; i < (int)(blockDim.x / TA_WAVE); ++i) s += red[i];
  return s;
}

template <typename TO>
__device__ __forceinline__ void store4(TO* p, float a, float b, float c, float d);
template <>
__device__ __forceinline__ void store4<float>(float* p, float a, float b, float c, float d) {
  *reinterpret_cast<float4*>(p) = float4{a, b, c, d};
}
template <>
__device__ __forceinline__ void store4<bf16_t>(bf16_t* p, float a, float b, float c, float d) {
  *reinterpret_cast<uint2*>(p) = uint2{f32x2_to_bf16x2_bits(a, b), f32x2_to_bf16x2_bits(c, d)};
}

// VEC: d % 4 == 0 and a thread owns runs of four columns, kept in registers (rows of up to
// 4 * 256 * VMAX columns); else the row waits in LDS between the passes.
template <typename TO, bool VEC>
__global__ __launch_bounds__(256) void postnorm_add_kernel(
    float* __restrict__ x, const float* __restrict__ delta, int planes, size_t plane,
    const float* __restrict__ w, float eps, TO* __restrict__ xcast, const float* __restrict__ w_next,
    float eps_next, TO* __restrict__ out, int d) {
  extern __shared__ float row[];          // [d] (not VEC)
  __shared__ float red[4];
  const size_t base = (size_t)blockIdx.x * d;
  if (VEC) {
    constexpr int VMAX = 4;
    float4 v[VMAX], xv[VMAX], wv[VMAX];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < VMAX; ++i) {
      const int c = 4 * (threadIdx.x + 256 * i);
      if (c < d) {
        v[i] = *reinterpret_cast<const float4*>(delta + base + c);
        xv[i] = *reinterpret_cast<const float4*>(x + base + c);
        wv[i] = *reinterpret_cast<const float4*>(w + c);
      } else {
        v[i] = xv[i] = wv[i] = float4{0.f, 0.f, 0.f, 0.f};
      }
    }
    for (int p = 1; p < planes; ++p)
#pragma unroll
      for (int i = 0; i < VMAX; ++i) {
        const int c = 4 * (threadIdx.x + 256 * i);
        if (c < d) {
          const float4 a = *reinterpret_cast<const float4*>(delta + base + c + p * plane);
          v[i].x += a.x; v[i].y += a.y; v[i].z += a.z; v[i].w += a.w;
        }
      }
#pragma unroll
    for (int i = 0; i < VMAX; ++i) ss += (v[i].x * v[i].x + v[i].y * v[i].y) + (v[i].z * v[i].z + v[i].w * v[i].w);
    const float f = rsqrtf(block_sum4(ss, red) / (float)d + eps);
    float s2 = 0.f;
#pragma unroll
    for (int i = 0; i < VMAX; ++i) {
      const int c = 4 * (threadIdx.x + 256 * i);
      v[i].x = xv[i].x + v[i].x * f * wv[i].x;
      v[i].y = xv[i].y + v[i].y * f * wv[i].y;
      v[i].z = xv[i].z + v[i].z * f * wv[i].z;
      v[i].w = xv[i].w + v[i].w * f * wv[i].w;
      if (c < d) {
        *reinterpret_cast<float4*>(x + base + c) = v[i];
        if (xcast) store4<TO>(xcast + base + c, v[i].x, v[i].y, v[i].z, v[i].w);
        s2 += (v[i].x * v[i].x + v[i].y * v[i].y) + (v[i].z * v[i].z + v[i].w * v[i].w);
      }
    }
    if (!out) return;
#pragma unroll
    for (int i = 0; i < VMAX; ++i) {
      const int c = 4 * (threadIdx.x + 256 * i);
      if (c < d) wv[i] = *reinterpret_cast<const float4*>(w_next + c);
    }
    const float f2 = rsqrtf(block_sum4(s2, red) / (float)d + eps_next);
#pragma unroll
    for (int i = 0; i < VMAX; ++i) {
      const int c = 4 * (threadIdx.x + 256 * i);
      if (c < d) store4<TO>(out + base + c, v[i].x * f2 * wv[i].x, v[i].y * f2 * wv[i].y, v[i].z * f2 * wv[i].z,
                            v[i].w * f2 * wv[i].w);
    }
    return;
  }
  float ss = 0.f;
  for (int c = threadIdx.x; c < d; c += 256) {
    float s = delta[base + c];
    for (int p = 1; p < planes; ++p) s += delta[base + c + p * plane];
    row[c] = s;
    ss += s * s;
  }
  const float f = rsqrtf(block_sum4(ss, red) / (float)d + eps);
  float s2 = 0.f;
  for (int c = threadIdx.x; c < d; c += 256) {
    const float v = x[base + c] + row[c] * f * w[c];
    x[base + c] = v;
    row[c] = v;
    s2 += v * v;
    if (xcast) xcast[base + c] = from_f32<TO>(v);
  }
  if (!out) return;
  const float f2 = rsqrtf(block_sum4(s2, red) / (float)d + eps_next);
  for (int c = threadIdx.x; c < d; c += 256) out[base + c] = from_f32<TO>(row[c] * f2 * w_next[c]);
}

// x: [nt, d] float32, updated in place. delta: [planes, nt, d] float32 (planes added in order).
// w: [d]. xcast (or null): [nt, d] receives the new rows in the engine's type. w_next / out (or
// null): out [nt, d] = rms_norm(new x, eps_next) * w_next.
extern "C" int ta_postnorm_add(hipStream_t stream, int out_dtype, float* x, const float* delta, int planes,
                               long long plane, const float* w, float eps, void* xcast,
                               const float* w_next, float eps_next, void* out, int nt, int d) {
  TA_REQUIRE(nt >= 0 && d > 0 && d <= 32768 && planes >= 1 && planes <= TA_MAX_PLANES,
             "ta_postnorm_add: bad sizes nt=%d d=%d planes=%d", nt, d, planes);
  TA_REQUIRE((out == nullptr) == (w_next == nullptr), "ta_postnorm_add: w_next and out go together");
  if (nt == 0) return 0;
  const size_t lds = (size_t)d * sizeof(float);
  const bool vec = d % 4 == 0 && d <= 4096 && plane % 4 == 0;
#define PN_RUN(T, V, L) postnorm_add_kernel<T, V><<<nt, 256, L, stream>>>(x, delta, planes, (size_t)plane, w, eps, (T*)xcast, w_next, eps_next, (T*)out, d)
  if (out_dtype == TA_F32) {
    if (vec) PN_RUN(float, true, 0); else PN_RUN(float, false, lds);
  } else if (out_dtype == TA_BF16) {
    if (vec) PN_RUN(bf16_t, true, 0); else PN_RUN(bf16_t, false, lds);
  } else {
    return ta_fail("ta_postnorm_add: unknown dtype %d", out_dtype);
  }
#undef PN_RUN
  return ta_check_launch("ta_postnorm_add");
}

// ------------------------------------------------------------------ activations
__device__ __forceinline__ float act_apply(int act, float z) {
  switch (act) {
    case 0: return 0.5f * z * (1.0f + erff(z * 0.7071067811865476f));                              // gelu
    case 1: return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));   // gelu (tanh)
    case 2: { const float r = fmaxf(z, 0.f); return r * r; }                                       // relu squared
    default: return z / (1.0f + expf(-z));                                                         // silu
  }
}

template <typename T>
__global__ __launch_bounds__(256) void activation_kernel(const T* __restrict__ in, int in_stride,
                                                         T* __restrict__ out, int out_stride, int n, int act,
                                                         const float* __restrict__ side, int side_stride) {
  const size_t t = blockIdx.y;
  for (int c = blockIdx.x * 256 + threadIdx.x; c < n; c += gridDim.x * 256) {
    float v = act_apply(act, to_f32(in[t * in_stride + c]));
    if (side) v *= side[t * side_stride + c];
    out[t * out_stride + c] = from_f32<T>(v);
  }
}

// Rows whose starts and lengths are multiples of 16 bytes, no side table: a thread takes 16 bytes
// of a row at a time.
template <typename T>
__global__ __launch_bounds__(256) void activation_vec_kernel(const T* __restrict__ in, int in_stride,
                                                             T* __restrict__ out, int out_stride, int n, int act) {
  constexpr int W = 16 / sizeof(T);
  const size_t t = blockIdx.y;
  for (int c = (blockIdx.x * 256 + threadIdx.x) * W; c < n; c += gridDim.x * 256 * W) {
    const uint4 raw = *reinterpret_cast<const uint4*>(in + t * in_stride + c);
    T a[W];
    __builtin_memcpy(a, &raw, 16);
    float v[W];
#pragma unroll
    for (int i = 0; i < W; ++i) v[i] = act_apply(act, to_f32(a[i]));
#pragma unroll
    for (int i = 0; i < W; ++i) a[i] = from_f32<T>(v[i]);
    uint4 res;
    __builtin_memcpy(&res, a, 16);
    *reinterpret_cast<uint4*>(out + t * out_stride + c) = res;
  }
}

// out[t, c] = act(in[t, c]) (* side[t, c]); rows may be strided. side: float32 or null.
extern "C" int ta_activation(hipStream_t stream, int dtype, int act, const void* in, int in_stride, void* out,
                             int out_stride, const float* side, int side_stride, int nt, int n) {
  TA_REQUIRE(nt >= 0 && nt <= 65535 * 64 && n > 0 && act >= 0 && act <= 3, "ta_activation: bad sizes nt=%d n=%d act=%d", nt, n, act);
  TA_REQUIRE(in_stride >= n && out_stride >= n && (side == nullptr || side_stride >= n), "ta_activation: strides too small");
  for (int t0 = 0; t0 < nt; t0 += 65535) {
    const int rows = nt - t0 < 65535 ? nt - t0 : 65535;
    int gx = (n + 255) / 256;
    if (gx > 64) gx = 64;
    dim3 g(gx, rows);
    const float* sd = side ? side + (size_t)t0 * side_stride : nullptr;
    const int W = dtype == TA_F32 ? 4 : 8;
    if (!side && (dtype == TA_F32 || dtype == TA_BF16) && n % W == 0 && in_stride % W == 0 && out_stride % W == 0 &&
        (uintptr_t)in % 16 == 0 && (uintptr_t)out % 16 == 0) {
      int vx = (n / W + 255) / 256;
      if (vx > 16) vx = 16;
      dim3 gv(vx, rows);
      if (dtype == TA_F32)
        activation_vec_kernel<float><<<gv, 256, 0, stream>>>((const float*)in + (size_t)t0 * in_stride, in_stride,
                                                             (float*)out + (size_t)t0 * out_stride, out_stride, n, act);
      else
        activation_vec_kernel<bf16_t><<<gv, 256, 0, stream>>>((const bf16_t*)in + (size_t)t0 * in_stride, in_stride,
                                                              (bf16_t*)out + (size_t)t0 * out_stride, out_stride, n, act);
      continue;
    }
    if (dtype == TA_F32)
      activation_kernel<float><<<g, 256, 0, stream>>>((const float*)in + (size_t)t0 * in_stride, in_stride,
                                                      (float*)out + (size_t)t0 * out_stride, out_stride, n, act, sd, side_stride);
    else if (dtype == TA_BF16)
      activation_kernel<bf16_t><<<g, 256, 0, stream>>>((const bf16_t*)in + (size_t)t0 * in_stride, in_stride,
                                                       (bf16_t*)out + (size_t)t0 * out_stride, out_stride, n, act, sd, side_stride);
    else
      return ta_fail("ta_activation: unknown dtype %d", dtype);
  }
  return ta_check_launch("ta_activation");
}

// ------------------------------------------------------------------ the mean of normed branches
// out[t] = (1/n) * sum over branches b of rms_norm(sum of the planes of delta_b[t], eps) * w_b.
// A thread owns the same columns in every pass, so the sum over branches needs no exchange; the
// planes are read a second time (from the caches) once a branch's factor is known.
struct MeanBranch {
  const float* delta;     // [planes, nt, d]
  const float* w;         // [d]
  long long plane;        // elements between planes
  int planes;
};
struct MeanBranches {
  MeanBranch b[4];
};

__global__ __launch_bounds__(256) void normed_mean_kernel(MeanBranches br, int n, float eps, float* __restrict__ out,
                                                          int d) {
  __shared__ float red[4];
  const size_t base = (size_t)blockIdx.x * d;
  const float inv = 1.0f / (float)n;
  for (int k = 0; k < n; ++k) {
    const MeanBranch b = br.b[k];
    float ss = 0.f;
    for (int c = threadIdx.x; c < d; c += 256) {
      float s = b.delta[base + c];
      for (int p = 1; p < b.planes; ++p) s += b.delta[base + c + p * b.plane];
      ss += s * s;
    }
    const float f = rsqrtf(block_sum4(ss, red) / (float)d + eps);
    for (int c = threadIdx.x; c < d; c += 256) {
      float s = b.delta[base + c];
      for (int p = 1; p < b.planes; ++p) s += b.delta[base + c + p * b.plane];
      const float v = s * f * b.w[c] * inv;
      out[base + c] = k == 0 ? v : out[base + c] + v;
    }
  }
}

// d % 4 == 0, d <= 4096, every plane and pointer a multiple of 16 bytes: a thread keeps its runs
// of four columns of a branch and of the mean in registers, so every plane is read once and the
// loads of one branch do not wait for one another.
__global__ __launch_bounds__(256) void normed_mean_vec_kernel(MeanBranches br, int n, float eps,
                                                              float* __restrict__ out, int d) {
  __shared__ float red[4];
  constexpr int VMAX = 4;
  const size_t base = (size_t)blockIdx.x * d;
  const float inv = 1.0f / (float)n;
  float4 acc[VMAX];
#pragma unroll
  for (int i = 0; i < VMAX; ++i) acc[i] = float4{0.f, 0.f, 0.f, 0.f};
  for (int k = 0; k < n; ++k) {
    const MeanBranch b = br.b[k];
    float4 v[VMAX], wv[VMAX];
#pragma unroll
    for (int i = 0; i < VMAX; ++i) {
      const int c = 4 * (threadIdx.x + 256 * i);
      if (c < d) {
        v[i] = *reinterpret_cast<const float4*>(b.delta + base + c);
        wv[i] = *reinterpret_cast<const float4*>(b.w + c);
      } else {
        v[i] = wv[i] = float4{0.f, 0.f, 0.f, 0.f};
      }
    }
    for (int p = 1; p < b.planes; ++p)
#pragma unroll
      for (int i = 0; i < VMAX; ++i) {
        const int c = 4 * (threadIdx.x + 256 * i);
        if (c < d) {
          const float4 a = *reinterpret_cast<const float4*>(b.delta + base + c + p * b.plane);
          v[i].x += a.x; v[i].y += a.y; v[i].z += a.z; v[i].w += a.w;
        }
      }
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < VMAX; ++i) ss += (v[i].x * v[i].x + v[i].y * v[i].y) + (v[i].z * v[i].z + v[i].w * v[i].w);
    const float f = rsqrtf(block_sum4(ss, red) / (float)d + eps);
#pragma unroll
    for (int i = 0; i < VMAX; ++i) {
      acc[i].x += v[i].x * f * wv[i].x * inv;
      acc[i].y += v[i].y * f * wv[i].y * inv;
      acc[i].z += v[i].z * f * wv[i].z * inv;
      acc[i].w += v[i].w * f * wv[i].w * inv;
    }
  }
#pragma unroll
  for (int i = 0; i < VMAX; ++i) {
    const int c = 4 * (threadIdx.x + 256 * i);
    if (c < d) *reinterpret_cast<float4*>(out + base + c) = acc[i];
  }
}

// deltas[i]: [planes[i], nt, d] float32, ``plane[i]`` elements apart; ws[i]: [d]; out [nt, d].
extern "C" int ta_normed_mean(hipStream_t stream, int n, const float* const* deltas, const int* planes,
                              const long long* plane, const float* const* ws, float eps, float* out, int nt, int d) {
  TA_REQUIRE(n >= 1 && n <= 4, "ta_normed_mean: %d branches (1 to 4 are taken)", n);
  TA_REQUIRE(nt >= 0 && d > 0, "ta_normed_mean: bad sizes nt=%d d=%d", nt, d);
  MeanBranches br;
  for (int i = 0; i < 4; ++i) br.b[i] = MeanBranch{nullptr, nullptr, 0, 1};
  for (int i = 0; i < n; ++i) {
    TA_REQUIRE(deltas[i] && ws[i] && planes[i] >= 1 && planes[i] <= TA_MAX_PLANES,
               "ta_normed_mean: branch %d: %d planes", i, planes[i]);
    br.b[i] = MeanBranch{deltas[i], ws[i], plane[i], planes[i]};
  }
  if (nt == 0) return 0;
  bool vec = d % 4 == 0 && d <= 4096 && (uintptr_t)out % 16 == 0;
  for (int i = 0; i < n; ++i)
    vec = vec && plane[i] % 4 == 0 && (uintptr_t)deltas[i] % 16 == 0 && (uintptr_t)ws[i] % 16 == 0;
  if (vec)
    normed_mean_vec_kernel<<<nt, 256, 0, stream>>>(br, n, eps, out, d);
  else
    normed_mean_kernel<<<nt, 256, 0, stream>>>(br, n, eps, out, d);
  return ta_check_launch("ta_normed_mean");
}

// ------------------------------------------------------------------ weighted sum of branches
// out = sum over i of scale[i] * (sum of the planes of deltas[i]); float32, 1 to 4 branches.
struct SumBranches {
  const float* d[4];
  long long plane[4];
  int planes[4];
  float scale[4];
};

__global__ __launch_bounds__(256) void weighted_sum_kernel(SumBranches br, int n, float* __restrict__ out, size_t total) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (size_t)gridDim.x * 256) {
    float acc = 0.f;
    for (int b = 0; b < n; ++b) {
      float s = 0.f;
      for (int p = 0; p < br.planes[b]; ++p) s += br.d[b][(size_t)p * br.plane[b] + i];
      acc = fmaf(br.scale[b], s, acc);
    }
    out[i] = acc;
  }
}

// deltas[i]: [planes[i], nt, d] float32, ``plane[i]`` elements apart; out [nt, d].
extern "C" int ta_weighted_sum(hipStream_t stream, int n, const float* const* deltas, const int* planes,
                               const long long* plane, const float* scales, float* out, int nt, int d) {
  TA_REQUIRE(n >= 1 && n <= 4, "ta_weighted_sum: %d branches (1 to 4 are taken)", n);
  TA_REQUIRE(nt >= 0 && d > 0, "ta_weighted_sum: bad sizes nt=%d d=%d", nt, d);
  SumBranches br;
  for (int i = 0; i < 4; ++i) { br.d[i] = nullptr; br.plane[i] = 0; br.planes[i] = 0; br.scale[i] = 0.f; }
  for (int i = 0; i < n; ++i) {
    TA_REQUIRE(deltas[i] && planes[i] >= 1 && planes[i] <= TA_MAX_PLANES, "ta_weighted_sum: branch %d: %d planes", i, planes[i]);
    br.d[i] = deltas[i]; br.plane[i] = plane[i]; br.planes[i] = planes[i]; br.scale[i] = scales[i];
  }
  if (nt == 0) return 0;
  const size_t total = (size_t)nt * d;
  const unsigned blocks = (unsigned)((total + 255) / 256 < 4096 ? (total + 255) / 256 : 4096);
  weighted_sum_kernel<<<blocks, 256, 0, stream>>>(br, n, out, total);
  return ta_check_launch("ta_weighted_sum");
}
