// Element access shared by the mixer kernels: activations and weights are bf16 (raw bits) or fp32,
// all arithmetic is fp32.
#pragma once
#include "../kernels/common.h"

namespace mxs {

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<bf16_t>(const bf16_t* p) { return bf2f(*p); }
template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stf<bf16_t>(bf16_t* p, float v) { *p = f2bf(v); }

// dot of a fp32 vector in LDS with a row of T in global memory (16-byte loads when `vec`)
template <typename T> __device__ __forceinline__ float dot_row(const float* __restrict__ q, const T* __restrict__ k, int n, bool vec);
template <> __device__ __forceinline__ float dot_row<float>(const float* __restrict__ q, const float* __restrict__ k, int n, bool vec) {
  float s = 0.f;
  if (vec) {
    for (int d = 0; d < n; d += 4) {
      const float4 a = *reinterpret_cast<const float4*>(k + d);
      s += q[d] * a.x + q[d + 1] * a.y + q[d + 2] * a.z + q[d + 3] * a.w;
    }
  } else {
    for (int d = 0; d < n; ++d) s += q[d] * k[d];
  }
  return s;
}
template <> __device__ __forceinline__ float dot_row<bf16_t>(const float* __restrict__ q, const bf16_t* __restrict__ k, int n, bool vec) {
  float s = 0.f;
  if (vec) {
    for (int d = 0; d < n; d += 8) {
      const uint4 a = *reinterpret_cast<const uint4*>(k + d);
      s += q[d] * bf2f_lo(a.x) + q[d + 1] * bf2f_hi(a.x) + q[d + 2] * bf2f_lo(a.y) + q[d + 3] * bf2f_hi(a.y) +
           q[d + 4] * bf2f_lo(a.z) + q[d + 5] * bf2f_hi(a.z) + q[d + 6] * bf2f_lo(a.w) + q[d + 7] * bf2f_hi(a.w);
    }
  } else {
    for (int d = 0; d < n; ++d) s += q[d] * bf2f(k[d]);
  }
  return s;
}

// 16 bytes of a row as floats: 8 bf16 or 4 fp32 (the pointer is 16-byte aligned)
template <typename T> struct El;
template <> struct El<bf16_t> { static constexpr int N = 8; };
template <> struct El<float> { static constexpr int N = 4; };
__device__ __forceinline__ void load16(const bf16_t* p, float* o) {
  const uint4 a = *reinterpret_cast<const uint4*>(p);
  o[0] = bf2f_lo(a.x); o[1] = bf2f_hi(a.x); o[2] = bf2f_lo(a.y); o[3] = bf2f_hi(a.y);
  o[4] = bf2f_lo(a.z); o[5] = bf2f_hi(a.z); o[6] = bf2f_lo(a.w); o[7] = bf2f_hi(a.w);
}
__device__ __forceinline__ void load16(const float* p, float* o) {
  const float4 a = *reinterpret_cast<const float4*>(p);
  o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w;
}
__device__ __forceinline__ void store16(bf16_t* p, const float* v) {
  uint4 a;
  a.x = pack2(v[0], v[1]); a.y = pack2(v[2], v[3]); a.z = pack2(v[4], v[5]); a.w = pack2(v[6], v[7]);
  *reinterpret_cast<uint4*>(p) = a;
}
__device__ __forceinline__ void store16(float* p, const float* v) {
  *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
}

__device__ __forceinline__ float silu_f(float z) { return z / (1.f + expf(-z)); }
__device__ __forceinline__ float sigmoid_f(float z) { return 1.f / (1.f + expf(-z)); }
__device__ __forceinline__ float logsigmoid_f(float z) { return z < 0.f ? z - log1pf(expf(z)) : -log1pf(expf(-z)); }

// sequence of flattened row t: the last s with qsl[s] <= t
__device__ __forceinline__ int seq_of_row(const int* __restrict__ qsl, int S, int t) {
  int lo = 0, hi = S - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (qsl[mid] <= t) lo = mid; else hi = mid - 1;
  }
  return lo;
}

}  // namespace mxs
