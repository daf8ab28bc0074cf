// What happens to a token's [q | k | v] projection before attention reads the cache, for the
// attention variant whose queries and keys are normalised over the whole projection and whose
// values have a width of their own:
//
//   q <- rms_norm(q over all heads at once) * wq, k likewise with wk      (float32)
//   the first `rot` coordinates of every head of q and k are rotated in pairs (i, i + rot/2)
//   v <- (1 - lambda) v + lambda v_first      (where the layer mixes in the values of an earlier one)
//   q is written back in place; k and v go to the paged cache (keys [pages][kv heads][PAGE][dk],
//   values [pages][kv heads][dvs][PAGE], dvs >= dv, rows dv.. of a token zero).
//
// One workgroup per token. Everything is float32 until the single rounding of each result.
#include "common.h"

template <typename T>
__global__ __launch_bounds__(256) void qk_prepare_kernel(
    T* __restrict__ qkv, int stride, const float* __restrict__ wq, const float* __restrict__ wk,
    float eps, int normed, const float* __restrict__ angles, int rot,
    const float* __restrict__ lambda, const T* __restrict__ v_first, T* __restrict__ v_keep,
    const int* __restrict__ dest, T* __restrict__ kcache, T* __restrict__ vcache,
    int nh, int nkv, int dk, int dv, int dvs, int k_inplace) {
  extern __shared__ float buf[];          // [nh*dk + nkv*dk], then a factor per head [nh + nkv]
  __shared__ float red[8];
  const int t = blockIdx.x;
  T* row = qkv + (size_t)t * stride;
  const int nq = nh * dk, nk = nkv * dk, nv = nkv * dv;
  // Loops over a row go in groups of four turns that are known to lie inside it: a load is
  // not asked for before the test that guards it, so turn by turn every load would wait for
  // the one before (20 trips to memory for a row of 5,120 where 5 do).
  float sq = 0.f, sk = 0.f;
  auto take = [&](int i) {
    const float v = to_f32(row[i]);
    buf[i] = v;
    if (i < nq) sq += v * v; else sk += v * v;
  };
  {
    int i = threadIdx.x;
    for (; i + 768 < nq + nk; i += 1024) {
#pragma unroll
      for (int u = 0; u < 4; ++u) take(i + 256 * u);
    }
    for (; i < nq + nk; i += 256) take(i);
  }
  sq = wave_sum(sq);
  sk = wave_sum(sk);
  if (threadIdx.x % TA_WAVE == 0) {
    red[threadIdx.x / TA_WAVE] = sq;
    red[4 + threadIdx.x / TA_WAVE] = sk;
  }
  __syncthreads();
  float fq = 1.f, fk = 1.f;
  if (normed == 1) {
    fq = rsqrtf((red[0] + red[1] + red[2] + red[3]) / (float)nq + eps);
    fk = rsqrtf((red[4] + red[5] + red[6] + red[7]) / (float)nk + eps);
  }
  // normed == 2: every head of q and of k has a factor of its own; the weights wq, wk are then
  // [dk], shared by the heads. A wave takes heads in turn.
  float* hf = buf + nq + nk;
  if (normed == 2) {
    for (int hd = threadIdx.x / TA_WAVE; hd < nh + nkv; hd += 4) {
      float ss = 0.f;
      for (int c = threadIdx.x % TA_WAVE; c < dk; c += TA_WAVE) ss += buf[hd * dk + c] * buf[hd * dk + c];
      ss = wave_sum(ss);
      if (threadIdx.x % TA_WAVE == 0) hf[hd] = rsqrtf(ss / (float)dk + eps);
    }
    __syncthreads();
  }
  const int half = rot / 2;
  const float* ang = angles ? angles + (size_t)t * half * 2 : nullptr;
  const int page = dest ? dest[t] / TA_PAGE : 0, off = dest ? dest[t] % TA_PAGE : 0;
  // Every thread reads the LDS copy and writes memory, so nothing it reads is written by another
  // thread. All loads are unconditional (a coordinate that is not rotated reads angle 0 and is
  // not changed by it), so that the loads of several turns are on their way together.
  auto finish = [&](int i) {
    const bool is_q = i < nq;
    const int j = is_q ? i : i - nq;
    const int head = j / dk, c = j - head * dk;
    const float f = normed == 2 ? hf[i / dk] : is_q ? fq : fk;
    const float* w = is_q ? wq : wk;
    const bool turns = ang != nullptr && c < rot;
    const int pi = turns ? (c < half ? c : c - half) : 0;
    const int shift = turns ? (c < half ? half : -half) : 0;
    const float cs = ang ? ang[2 * pi] : 1.f, sn = ang ? ang[2 * pi + 1] : 0.f;
    float wv = 1.f, wo = 1.f;
    if (normed) {                     // the same for every thread
      const int jw = normed == 2 ? c : j;
      wv = w[jw];
      wo = w[jw + shift];
    }
    float v = buf[i] * f * wv;
    const float o = buf[i + shift] * f * wo;
    if (turns) v = c < half ? v * cs - o * sn : v * cs + o * sn;
    if (is_q || k_inplace) {
      row[i] = from_f32<T>(v);
    } else if (dest) {
      kcache[(((size_t)page * nkv + head) * TA_PAGE + off) * dk + c] = from_f32<T>(v);
    }
  };
  {
    int i = threadIdx.x;
    for (; i + 768 < nq + nk; i += 1024) {
#pragma unroll
      for (int u = 0; u < 4; ++u) finish(i + 256 * u);
    }
    for (; i < nq + nk; i += 256) finish(i);
  }
  const float lam = lambda ? lambda[0] : 0.f;
  for (int i = threadIdx.x; i < nv; i += 256) {
    float v = to_f32(row[nq + nk + i]);
    if (v_keep) v_keep[(size_t)t * nv + i] = from_f32<T>(v);
    if (v_first) v = (1.0f - lam) * v + lam * to_f32(v_first[(size_t)t * nv + i]);
    if (dest) {
      const int g = i / dv, c = i - g * dv;
      vcache[(((size_t)page * nkv + g) * dvs + c) * TA_PAGE + off] = from_f32<T>(v);
    }
  }
  // a cache whose value rows are wider than the values (dvs > dv) holds zeros there
  if (dest && dvs > dv) {
    const int pad = dvs - dv;
    for (int i = threadIdx.x; i < nkv * pad; i += 256) {
      const int g = i / pad, c = dv + (i - g * pad);
      vcache[(((size_t)page * nkv + g) * dvs + c) * TA_PAGE + off] = from_f32<T>(0.f);
    }
  }
}

// The same in pieces of eight coordinates (16 bytes of bfloat16) per thread and turn, for head
// widths that are multiples of 8 and rotations whose halves are: a row of 5,120 coordinates is
// then two or three turns per thread instead of twenty.
template <typename T> struct Eight;
template <> struct Eight<float> {
  static __device__ __forceinline__ void load(const float* p, float* v) {
    const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
  }
  static __device__ __forceinline__ void store(float* p, const float* v) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
    *reinterpret_cast<float4*>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
  }
};
template <> struct Eight<bf16_t> {
  static __device__ __forceinline__ void load(const bf16_t* p, float* v) {
    const uint4 r = *reinterpret_cast<const uint4*>(p);
    const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[2 * i] = __uint_as_float(w[i] << 16);
      v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  }
  static __device__ __forceinline__ void store(bf16_t* p, const float* v) {
    uint4 r;
    r.x = f32x2_to_bf16x2_bits(v[0], v[1]);
    r.y = f32x2_to_bf16x2_bits(v[2], v[3]);
    r.z = f32x2_to_bf16x2_bits(v[4], v[5]);
    r.w = f32x2_to_bf16x2_bits(v[6], v[7]);
    *reinterpret_cast<uint4*>(p) = r;
  }
};

template <typename T>
__global__ __launch_bounds__(256) void qk_prepare_vec_kernel(
    T* __restrict__ qkv, int stride, const float* __restrict__ wq, const float* __restrict__ wk,
    float eps, int normed, const float* __restrict__ angles, int rot,
    const float* __restrict__ lambda, const T* __restrict__ v_first, T* __restrict__ v_keep,
    const int* __restrict__ dest, T* __restrict__ kcache, T* __restrict__ vcache,
    int nh, int nkv, int dk, int dv, int dvs, int k_inplace) {
  extern __shared__ float buf[];          // [nh*dk + nkv*dk], then a factor per head [nh + nkv]
  __shared__ float red[8];
  const int t = blockIdx.x;
  T* row = qkv + (size_t)t * stride;
  const int nq = nh * dk, nk = nkv * dk, nv = nkv * dv;
  const int pieces = (nq + nk) / 8;
  float sq = 0.f, sk = 0.f;
  for (int p = threadIdx.x; p < pieces; p += 256) {
    float v[8];
    Eight<T>::load(row + 8 * p, v);
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      buf[8 * p + e] = v[e];
      ss += v[e] * v[e];
    }
    if (8 * p < nq) sq += ss; else sk += ss;
  }
  sq = wave_sum(sq);
  sk = wave_sum(sk);
  if (threadIdx.x % TA_WAVE == 0) {
    red[threadIdx.x / TA_WAVE] = sq;
    red[4 + threadIdx.x / TA_WAVE] = sk;
  }
  __syncthreads();
  float fq = 1.f, fk = 1.f;
  if (normed == 1) {
    fq = rsqrtf((red[0] + red[1] + red[2] + red[3]) / (float)nq + eps);
    fk = rsqrtf((red[4] + red[5] + red[6] + red[7]) / (float)nk + eps);
  }
  // normed == 2: every head of q and of k has a factor of its own; the weights wq, wk are then
  // [dk], shared by the heads. A wave takes heads in turn.
  float* hf = buf + nq + nk;
  if (normed == 2) {
    for (int hd = threadIdx.x / TA_WAVE; hd < nh + nkv; hd += 4) {
      float ss = 0.f;
      for (int c = threadIdx.x % TA_WAVE; c < dk; c += TA_WAVE) ss += buf[hd * dk + c] * buf[hd * dk + c];
      ss = wave_sum(ss);
      if (threadIdx.x % TA_WAVE == 0) hf[hd] = rsqrtf(ss / (float)dk + eps);
    }
    __syncthreads();
  }
  const int half = rot / 2;
  const float* ang = angles ? angles + (size_t)t * half * 2 : nullptr;
  const int page = dest ? dest[t] / TA_PAGE : 0, off = dest ? dest[t] % TA_PAGE : 0;
  for (int p = threadIdx.x; p < pieces; p += 256) {
    const int i = 8 * p;
    const bool is_q = i < nq;
    const int j = is_q ? i : i - nq;
    const int head = j / dk, c = j - head * dk;            // the piece lies inside one head
    const float f = normed == 2 ? hf[i / dk] : is_q ? fq : fk;
    const float* w = is_q ? wq : wk;
    const bool turns = ang != nullptr && c < rot;          // and wholly inside or outside the rotation
    const int shift = turns ? (c < half ? half : -half) : 0;
    float wv[8], wo[8], cs[8], sn[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) wv[e] = wo[e] = cs[e] = 1.f, sn[e] = 0.f;
    if (normed) {
      const int jw = normed == 2 ? c : j;
      Eight<float>::load(w + jw, wv);
      Eight<float>::load(w + jw + shift, wo);
    }
    if (turns) {
      float a[8], b[8];
      const int pi = c < half ? c : c - half;
      Eight<float>::load(ang + 2 * pi, a);
      Eight<float>::load(ang + 2 * pi + 8, b);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        cs[e] = a[2 * e]; sn[e] = a[2 * e + 1];
        cs[4 + e] = b[2 * e]; sn[4 + e] = b[2 * e + 1];
      }
    }
    float out[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float v = buf[i + e] * f * wv[e], o = buf[i + shift + e] * f * wo[e];
      out[e] = turns ? (c < half ? v * cs[e] - o * sn[e] : v * cs[e] + o * sn[e]) : v;
    }
    if (is_q || k_inplace) Eight<T>::store(row + i, out);
    else if (dest) Eight<T>::store(kcache + (((size_t)page * nkv + head) * TA_PAGE + off) * dk + c, out);
  }
  const float lam = lambda ? lambda[0] : 0.f;
  for (int i = threadIdx.x; i < nv; i += 256) {
    float v = to_f32(row[nq + nk + i]);
    if (v_keep) v_keep[(size_t)t * nv + i] = from_f32<T>(v);
    if (v_first) v = (1.0f - lam) * v + lam * to_f32(v_first[(size_t)t * nv + i]);
    if (dest) {
      const int g = i / dv, c = i - g * dv;
      vcache[(((size_t)page * nkv + g) * dvs + c) * TA_PAGE + off] = from_f32<T>(v);
    }
  }
  if (dest && dvs > dv) {
    const int pad = dvs - dv;
    for (int i = threadIdx.x; i < nkv * pad; i += 256) {
      const int g = i / pad, c = dv + (i - g * pad);
      vcache[(((size_t)page * nkv + g) * dvs + c) * TA_PAGE + off] = from_f32<T>(0.f);
    }
  }
}

// qkv: [nt, stride] rows of [nh*dk | nkv*dk | nkv*dv]. normed 1: wq [nh*dk], wk [nkv*dk], one norm over
// all heads of q and one over all of k; normed 2: wq, wk [dk], every head normed on its own; 0: no norm.
// k_inplace (no dest): the keys are written back into their rows as the queries are.
// angles: [nt, rot/2, 2] (cos, sin) or null. lambda: one float on the device, v_first [nt, nkv*dv]
// (both or neither). v_keep [nt, nkv*dv] or null: receives the unmixed values. dest [nt] or null:
// page * PAGE + offset of each token in the cache layer.
extern "C" int ta_qk_prepare(hipStream_t stream, int dtype, void* qkv, int stride, const float* wq,
                             const float* wk, float eps, int normed, const float* angles, int rot,
                             const float* lambda, const void* v_first, void* v_keep, const int* dest,
                             void* kcache, void* vcache, int nt, int nh, int nkv, int dk, int dv,
                             int dvs, int k_inplace) {
  TA_REQUIRE(nt >= 0 && nh > 0 && nkv > 0 && dk > 0 && dv > 0, "ta_qk_prepare: bad sizes");
  TA_REQUIRE(normed >= 0 && normed <= 2, "ta_qk_prepare: unknown norm mode %d", normed);
  TA_REQUIRE(!(k_inplace && dest), "ta_qk_prepare: keys go back in place or to the cache, not both");
  TA_REQUIRE(stride >= (nh + nkv) * dk + nkv * dv, "ta_qk_prepare: row stride %d too small", stride);
  TA_REQUIRE(rot >= 0 && rot <= dk && rot % 2 == 0, "ta_qk_prepare: %d rotated coordinates of %d", rot, dk);
  TA_REQUIRE((lambda == nullptr) == (v_first == nullptr), "ta_qk_prepare: lambda and v_first go together");
  TA_REQUIRE(!normed || (wq && wk), "ta_qk_prepare: norm weights missing");
  TA_REQUIRE(!dest || (kcache && vcache), "ta_qk_prepare: cache layer missing");
  TA_REQUIRE(dvs >= dv, "ta_qk_prepare: cache rows of %d cannot hold values of %d", dvs, dv);
  const size_t lds = ((size_t)(nh + nkv) * dk + nh + nkv) * sizeof(float);
  TA_REQUIRE(lds <= 60000, "ta_qk_prepare: %d + %d heads of %d do not fit", nh, nkv, dk);
  if (nt == 0) return 0;
  if (rot == 0) angles = nullptr;
  // pieces of eight: whole pieces per head and per half of the rotation, rows and tables on
  // 16-byte boundaries (32 for float32 rows)
  const uintptr_t all = (uintptr_t)qkv | (uintptr_t)wq | (uintptr_t)wk | (uintptr_t)angles | (uintptr_t)kcache;
  if (dk % 8 == 0 && rot % 16 == 0 && stride % 8 == 0 && (all & 31) == 0 &&
      (dtype == TA_F32 || dtype == TA_BF16)) {
    if (dtype == TA_F32)
      qk_prepare_vec_kernel<float><<<nt, 256, lds, stream>>>(
          (float*)qkv, stride, wq, wk, eps, normed, angles, rot, lambda, (const float*)v_first, (float*)v_keep,
          dest, (float*)kcache, (float*)vcache, nh, nkv, dk, dv, dvs, k_inplace);
    else
      qk_prepare_vec_kernel<bf16_t><<<nt, 256, lds, stream>>>(
          (bf16_t*)qkv, stride, wq, wk, eps, normed, angles, rot, lambda, (const bf16_t*)v_first, (bf16_t*)v_keep,
          dest, (bf16_t*)kcache, (bf16_t*)vcache, nh, nkv, dk, dv, dvs, k_inplace);
    return ta_check_launch("ta_qk_prepare");
  }
  if (dtype == TA_F32)
    qk_prepare_kernel<float><<<nt, 256, lds, stream>>>(
        (float*)qkv, stride, wq, wk, eps, normed, angles, rot, lambda, (const float*)v_first, (float*)v_keep,
        dest, (float*)kcache, (float*)vcache, nh, nkv, dk, dv, dvs, k_inplace);
  else if (dtype == TA_BF16)
    qk_prepare_kernel<bf16_t><<<nt, 256, lds, stream>>>(
        (bf16_t*)qkv, stride, wq, wk, eps, normed, angles, rot, lambda, (const bf16_t*)v_first, (bf16_t*)v_keep,
        dest, (bf16_t*)kcache, (bf16_t*)vcache, nh, nkv, dk, dv, dvs, k_inplace);
  else
    return ta_fail("ta_qk_prepare: unknown dtype %d", dtype);
  return ta_check_launch("ta_qk_prepare");
}

// ------------------------------------------------------------------ rotation and cache write, no norm
// Rows [q | k | v] (nh*dk, nkv*dk, nkv*dv columns; a layer that reads another layer's keys and values
// has q only: nkv_own = 0). bias [columns] float32 or null is added first. The first `rot` coordinates
// of every head of q and k turn by the token's angles cs [nt, rot/2] (cos, sin): style 0 pairs
// (i, i + rot/2), style 1 pairs (2i, 2i + 1). q goes back in place; k and v go to the paged cache at
// dest[t] (keys [pages][kv heads][PAGE][dk], values [pages][kv heads][dvs][PAGE], dvs >= dv, rows dv.. of
// a token zero). float32 inside, one rounding of each result. One workgroup per token, a thread per pair of coordinates.
template <typename T>
__global__ __launch_bounds__(256) void qk_rotate_store_kernel(
    T* __restrict__ qkv, int stride, const float* __restrict__ bias, const float2* __restrict__ cs, int rot,
    int style, const int* __restrict__ dest, T* __restrict__ kcache, T* __restrict__ vcache, int nh, int nkv,
    int nkv_own, int dk, int dv, int dvs) {
  const int t = blockIdx.x;
  T* row = qkv + (size_t)t * stride;
  const int nq = nh * dk, nk = nkv_own * dk, nv = nkv_own * dv;
  const int half = rot / 2, hd2 = dk / 2;              // dk is even
  const float2* ang = cs ? cs + (size_t)t * half : nullptr;
  const int page = dest ? dest[t] / TA_PAGE : 0, off = dest ? dest[t] % TA_PAGE : 0;
  for (int i = threadIdx.x; i < (nq + nk) / 2; i += 256) {
    const int head = i / hd2, p = i - head * hd2;      // pair p of head (q heads first, then k heads)
    int c0, c1;
    bool turns = ang != nullptr && p < half;
    if (style == 1) { c0 = 2 * p; c1 = 2 * p + 1; }
    else if (p < half) { c0 = p; c1 = p + half; }
    else {                                              // the coordinates that no pair of style 0 covers
      const int r = p - half;                           // rot + 2r, rot + 2r + 1
      c0 = rot + 2 * r; c1 = c0 + 1;
    }
    const int base = head * dk;
    float u = to_f32(row[base + c0]), v = to_f32(row[base + c1]);
    if (bias) { u += bias[base + c0]; v += bias[base + c1]; }
    if (turns) {
      const float2 a = ang[p];
      const float nu = u * a.x - v * a.y, nv2 = v * a.x + u * a.y;
      u = nu; v = nv2;
    }
    if (head < nh) {
      row[base + c0] = from_f32<T>(u);
      row[base + c1] = from_f32<T>(v);
    } else if (dest) {
      T* kd = kcache + (((size_t)page * nkv + (head - nh)) * TA_PAGE + off) * dk;
      kd[c0] = from_f32<T>(u);
      kd[c1] = from_f32<T>(v);
    }
  }
  if (dest) {
    for (int i = threadIdx.x; i < nv; i += 256) {
      float v = to_f32(row[nq + nk + i]);
      if (bias) v += bias[nq + nk + i];
      const int g = i / dv, c = i - g * dv;
      vcache[(((size_t)page * nkv + g) * dvs + c) * TA_PAGE + off] = from_f32<T>(v);
    }
    const int pad = dvs - dv;                          // a cache whose value rows are wider holds zeros there
    for (int i = threadIdx.x; i < nkv_own * pad; i += 256) {
      const int g = i / pad, c = dv + (i - g * pad);
      vcache[(((size_t)page * nkv + g) * dvs + c) * TA_PAGE + off] = from_f32<T>(0.f);
    }
  }
}

extern "C" int ta_qk_rotate_store(hipStream_t stream, int dtype, void* qkv, int stride, const float* bias,
                                  const float* cs, int rot, int style, const int* dest, void* kcache, void* vcache,
                                  int nt, int nh, int nkv, int nkv_own, int dk, int dv, int dvs) {
  TA_REQUIRE(dvs >= dv, "ta_qk_rotate_store: value rows of %d do not hold values of %d", dvs, dv);
  TA_REQUIRE(nt >= 0 && nh >= 1 && nkv >= 1 && (nkv_own == 0 || nkv_own == nkv) && dk >= 2 && dk % 2 == 0 && dv >= 1,
             "ta_qk_rotate_store: bad sizes nt=%d heads=%d/%d (%d own) widths %d/%d", nt, nh, nkv, nkv_own, dk, dv);
  TA_REQUIRE(rot >= 0 && rot % 2 == 0 && rot <= dk && (rot == 0 || cs != nullptr) && (style == 0 || style == 1),
             "ta_qk_rotate_store: %d rotated coordinates of %d, style %d", rot, dk, style);
  TA_REQUIRE(stride >= nh * dk + nkv_own * (dk + dv), "ta_qk_rotate_store: rows of %d are too short", stride);
  TA_REQUIRE(dest == nullptr || (nkv_own == nkv && kcache && vcache), "ta_qk_rotate_store: a cache write needs keys, values and a cache");
  if (nt == 0) return 0;
  if (dtype == TA_F32)
    qk_rotate_store_kernel<float><<<nt, 256, 0, stream>>>((float*)qkv, stride, bias, rot ? (const float2*)cs : nullptr,
                                                          rot, style, dest, (float*)kcache, (float*)vcache, nh, nkv,
                                                          nkv_own, dk, dv, dvs);
  else if (dtype == TA_BF16)
    qk_rotate_store_kernel<bf16_t><<<nt, 256, 0, stream>>>((bf16_t*)qkv, stride, bias, rot ? (const float2*)cs : nullptr,
                                                           rot, style, dest, (bf16_t*)kcache, (bf16_t*)vcache, nh, nkv,
                                                           nkv_own, dk, dv, dvs);
  else return ta_fail("ta_qk_rotate_store: unknown dtype %d", dtype);
  return ta_check_launch("ta_qk_rotate_store");
}
