// Kernels of a residual stream that keeps what every layer produced (gfx950): the normed embedding,
// the weighted sum over the kept results, and a two-sided activation with learned curvatures.
// Activations and weights are bf16 or fp32 (template T); the stream, norms, sums and the activation's
// arithmetic are fp32.  One workgroup per token row.
#include "mix_common.h"

namespace mxs {

#define MIX_DISPATCH(bf, ...)                      \
  do {                                             \
    if (bf) { using T = bf16_t; __VA_ARGS__; }     \
    else { using T = float; __VA_ARGS__; }         \
  } while (0)

// out[t] = RMSNorm(table[ids[t]]) * (w_offset + w); h (optional) = the same rounded to T; copy (optional) = a
// second fp32 copy (the slab the first layer updates in place).
template <typename T>
__global__ void __launch_bounds__(256) embed_normed_kernel(float* __restrict__ out, float* __restrict__ copy,
                                                           T* __restrict__ h, const int64_t* __restrict__ ids,
                                                           const T* __restrict__ table, const T* __restrict__ w, int W,
                                                           long vocab, float eps, float w_offset) {
  __shared__ float scratch[16];
  const long t = blockIdx.x;
  long id = ids[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);  // padding rows carry any id
  const T* row = table + id * W;
  float s = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) { const float v = ldf(row + c); s += v * v; }
  const float inv = rsqrtf(block_sum(s, scratch) / static_cast<float>(W) + eps);
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float v = ldf(row + c) * inv * (w_offset + ldf(w + c));
    out[t * W + c] = v;
    if (copy) copy[t * W + c] = v;
    if (h) stf(h + t * W + c, v);
  }
}

// slab n <- sum_{j < n} coeffs[j] * slab j, summed in the order of j; h (optional) = the sum rounded to T.
// The coefficients wait in LDS; a thread's loads of the n slabs are independent of one another.
template <typename T>
__global__ void __launch_bounds__(256) depth_mix_kernel(float* __restrict__ hist, long slab, int n,
                                                        const float* __restrict__ coeffs, T* __restrict__ h, int W) {
  extern __shared__ float cf[];
  for (int j = threadIdx.x; j < n; j += blockDim.x) cf[j] = coeffs[j];
  __syncthreads();
  const long t = blockIdx.x;
  const float* src = hist + t * W;
  float* dst = hist + static_cast<long>(n) * slab + t * W;
  if ((W & 3) == 0) {
    for (int c = threadIdx.x * 4; c < W; c += blockDim.x * 4) {
      float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll 4
      for (int j = 0; j < n; ++j) {
        const float4 v = *reinterpret_cast<const float4*>(src + j * slab + c);
        const float a = cf[j];
        acc.x += a * v.x; acc.y += a * v.y; acc.z += a * v.z; acc.w += a * v.w;
      }
      *reinterpret_cast<float4*>(dst + c) = acc;
      if (h) {
        T* hp = h + t * W + c;
        stf(hp, acc.x); stf(hp + 1, acc.y); stf(hp + 2, acc.z); stf(hp + 3, acc.w);
      }
    }
    return;
  }
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float acc = 0.f;
    for (int j = 0; j < n; ++j) acc += cf[j] * src[j * slab + c];
    dst[c] = acc;
    if (h) stf(h + t * W + c, acc);
  }
}

// ab = (a, b):  z > 0: a z^2 + z / 2;  z <= 0: b (e^z - 1 - z) + z / 2.
template <typename T>
__global__ void __launch_bounds__(256) xielu_kernel(T* __restrict__ out, const T* __restrict__ x, long n,
                                                    const float* __restrict__ ab) {
  const float a = ab[0], b = ab[1];
  for (long i = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x; i < n; i += static_cast<long>(gridDim.x) * blockDim.x) {
    const float z = ldf(x + i);
    const float zn = fminf(z, 0.f);
    stf(out + i, z > 0.f ? a * z * z + 0.5f * z : b * (expm1f(zn) - zn) + 0.5f * z);
  }
}

void launch_embed_normed(float* out, float* copy, void* h, const int64_t* ids, const void* table, const void* w, int rows, int W,
                         long vocab, float eps, float w_offset, bool bf, hipStream_t st) {
  if (rows == 0) return;
  MIX_DISPATCH(bf, hipLaunchKernelGGL(embed_normed_kernel<T>, dim3(rows), dim3(256), 0, st, out, copy, (T*)h, ids,
                                      (const T*)table, (const T*)w, W, vocab, eps, w_offset));
  MXS_CHECK_LAUNCH();
}

bool launch_depth_mix(float* hist, long slab, int n, const float* coeffs, void* h, int rows, int W, bool bf,
                      hipStream_t st) {
  if (rows == 0) return true;
  const size_t shm = static_cast<size_t>(n) * sizeof(float);
  if (shm > 60 * 1024) return false;
  MIX_DISPATCH(bf, hipLaunchKernelGGL(depth_mix_kernel<T>, dim3(rows), dim3(256), shm, st, hist, slab, n, coeffs, (T*)h, W));
  MXS_CHECK_LAUNCH();
  return true;
}

void launch_xielu(void* out, const void* x, long n, const float* ab, bool bf, hipStream_t st) {
  if (n == 0) return;
  const int blocks = static_cast<int>(std::min<long>((n + 255) / 256, 8192));
  MIX_DISPATCH(bf, hipLaunchKernelGGL(xielu_kernel<T>, dim3(blocks), dim3(256), 0, st, (T*)out, (const T*)x, n, ab));
  MXS_CHECK_LAUNCH();
}

}  // namespace mxs
