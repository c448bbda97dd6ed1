// Residual-stream, norm, activation and cache-write kernels of the mixer models (gfx950).
// One workgroup per token row; rows are a few KB, so each kernel is one pass over HBM: the row is
// re-read from L1/L2 where a second sweep is needed.
#include "mix_common.h"

namespace mxs {

// x (fp32, in place) <- x + d | d, d built from up to two branch outputs (each optionally RMS-normed
// over the row with its weight, then averaged) and a bias row; h <- RMSNorm(x) * norm_w when asked, or
// h <- x itself (rounded to T) when h is given without norm_w.
template <typename T>
__global__ void __launch_bounds__(256) resid_update_kernel(float* __restrict__ x, const T* __restrict__ a, long a_stride,
                                                           const T* __restrict__ wa, const T* __restrict__ b,
                                                           long b_stride, const T* __restrict__ wb,
                                                           const T* __restrict__ bias, int assign,
                                                           const T* __restrict__ norm_w, T* __restrict__ h, int W,
                                                           float eps, float a_scale, float w_offset, float wa_offset) {
  __shared__ float scratch[16];
  const long row = blockIdx.x;
  float* xr = x + row * W;
  const T* ar = a ? a + row * a_stride : nullptr;
  const T* br = b ? b + row * b_stride : nullptr;
  float ra = 1.f, rb = 1.f;
  if (ar && wa) {
    float s = 0.f;
    for (int c = threadIdx.x; c < W; c += blockDim.x) { const float v = ldf(ar + c); s += v * v; }
    ra = rsqrtf(block_sum(s, scratch) / static_cast<float>(W) + eps);
  }
  if (br) {
    float s = 0.f;
    for (int c = threadIdx.x; c < W; c += blockDim.x) { const float v = ldf(br + c); s += v * v; }
    rb = rsqrtf(block_sum(s, scratch) / static_cast<float>(W) + eps);
  }
  float ss = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float xv = xr[c];
    if (ar) {
      float d = ldf(ar + c) * a_scale;
      if (wa) d = d * ra * (wa_offset + ldf(wa + c));
      if (br) d = 0.5f * (d + ldf(br + c) * rb * ldf(wb + c));
      if (bias) d += ldf(bias + c);
      xv = assign ? d : xv + d;
      xr[c] = xv;
    }
    if (h && !norm_w) stf(h + row * W + c, xv);
    ss += xv * xv;
  }
  if (norm_w == nullptr) return;
  const float inv = rsqrtf(block_sum(ss, scratch) / static_cast<float>(W) + eps);
  T* hr = h + row * W;
  for (int c = threadIdx.x; c < W; c += blockDim.x) stf(hr + c, xr[c] * inv * (w_offset + ldf(norm_w + c)));  // own writes
}

template <typename T>
__global__ void __launch_bounds__(256) cast_into_kernel(T* __restrict__ dst, long dst_stride, const float* __restrict__ x, int W) {
  const long row = blockIdx.x;
  for (int c = threadIdx.x; c < W; c += blockDim.x) stf(dst + row * dst_stride + c, x[row * W + c]);
}

template <typename T>
__global__ void __launch_bounds__(256) relu_sq_kernel(T* __restrict__ out, const T* __restrict__ x, long n) {
  for (long i = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x; i < n; i += static_cast<long>(gridDim.x) * blockDim.x) {
    const float v = fmaxf(ldf(x + i), 0.f);
    stf(out + i, v * v);
  }
}

template <typename T>
__global__ void __launch_bounds__(256) softcap_kernel(float* __restrict__ out, const T* __restrict__ x, long x_stride,
                                                      int V, float cap) {
  const long row = blockIdx.x;
  for (int c = threadIdx.x; c < V; c += blockDim.x) {
    const float v = ldf(x + row * x_stride + c);
    out[row * V + c] = cap > 0.f ? cap * tanhf(v / cap) : v;
  }
}

// out = RMSNorm(o) * w * sigmoid(gate), the norm over each of `groups` equal slices of the row.
// groups == 1: the block reduces the row; otherwise one wave per slice.
template <typename T>
__global__ void __launch_bounds__(256) gated_rms_norm_kernel(T* __restrict__ out, const float* __restrict__ o,
                                                             const T* __restrict__ gate, long g_stride,
                                                             const T* __restrict__ w, int N, int groups, float eps) {
  __shared__ float scratch[16];
  const long row = blockIdx.x;
  const float* orow = o + row * N;
  const T* grow = gate + row * g_stride;
  T* yrow = out + row * N;
  if (groups == 1) {
    float s = 0.f;
    for (int c = threadIdx.x; c < N; c += blockDim.x) s += orow[c] * orow[c];
    const float inv = rsqrtf(block_sum(s, scratch) / static_cast<float>(N) + eps);
    for (int c = threadIdx.x; c < N; c += blockDim.x)
      stf(yrow + c, orow[c] * inv * ldf(w + c) * sigmoid_f(ldf(grow + c)));
    return;
  }
  const int n = N / groups, lane = threadIdx.x & 63, wid = threadIdx.x >> 6, nw = blockDim.x >> 6;
  for (int g = wid; g < groups; g += nw) {
    float s = 0.f;
    for (int c = lane; c < n; c += 64) { const float v = orow[g * n + c]; s += v * v; }
    const float inv = rsqrtf(wave_sum(s) / static_cast<float>(n) + eps);
    for (int c = lane; c < n; c += 64) {
      const int i = g * n + c;
      stf(yrow + i, orow[i] * inv * ldf(w + i) * sigmoid_f(ldf(grow + i)));
    }
  }
}

// out[t, n] = sum_c h[t, c] w[n, c] + bias[n], fp32 products and sums; a wave per output column.
template <typename T>
__global__ void __launch_bounds__(256) gate_linear_kernel(float* __restrict__ out, const T* __restrict__ h, long h_stride,
                                                          const T* __restrict__ w, const T* __restrict__ bias, int N,
                                                          int W, int vec) {
  constexpr int EL = El<T>::N;
  const long row = blockIdx.x;
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const T* hr = h + row * h_stride;
  for (int n = wid; n < N; n += nw) {
    float s = 0.f;
    const T* wr = w + static_cast<long>(n) * W;
    if (vec) {  // rows of whole, aligned 16-byte pieces
      for (int c = lane * EL; c < W; c += 64 * EL) {
        float a[EL], b[EL];
        load16(hr + c, a);
        load16(wr + c, b);
#pragma unroll
        for (int e = 0; e < EL; ++e) s += a[e] * b[e];
      }
    } else {
      for (int c = lane; c < W; c += 64) s += ldf(hr + c) * ldf(wr + c);
    }
    s = wave_sum(s);
    if (lane == 0) out[row * N + n] = s + (bias ? ldf(bias + n) : 0.f);
  }
}

// K [T, G*dk] and V [T, G*dv] rows into the paged pool: block-major, K at koff as [G][BS][dk], V at
// voff as [G][BS][dv].  slot < 0: nothing is written (padding rows).
template <typename T>
__global__ void __launch_bounds__(256) kv_write_kernel(T* __restrict__ cache, long block_stride, const T* __restrict__ k,
                                                       long k_stride, const T* __restrict__ v, long v_stride,
                                                       const int64_t* __restrict__ slots, int koff, int voff, int G,
                                                       int dk, int dv, int bs) {
  const long t = blockIdx.x;
  const int64_t slot = slots[t];
  if (slot < 0) return;
  const long blk = slot / bs;
  const int off = static_cast<int>(slot % bs);
  T* base = cache + blk * block_stride;
  for (int i = threadIdx.x; i < G * dk; i += blockDim.x) {
    const int g = i / dk, d = i - g * dk;
    base[koff + (static_cast<long>(g) * bs + off) * dk + d] = k[t * k_stride + i];
  }
  for (int i = threadIdx.x; i < G * dv; i += blockDim.x) {
    const int g = i / dv, d = i - g * dv;
    base[voff + (static_cast<long>(g) * bs + off) * dv + d] = v[t * v_stride + i];
  }
}

#define MIX_DISPATCH(bf, ...)                      \
  do {                                             \
    if (bf) { using T = bf16_t; __VA_ARGS__; }     \
    else { using T = float; __VA_ARGS__; }         \
  } while (0)

void launch_resid_update(float* x, const void* a, long a_stride, const void* wa, const void* b, long b_stride,
                         const void* wb, const void* bias, int assign, const void* norm_w, void* h, int rows, int W,
                         float eps, float a_scale, float w_offset, float wa_offset, bool bf, hipStream_t st) {
  if (rows == 0) return;
  MIX_DISPATCH(bf, hipLaunchKernelGGL(resid_update_kernel<T>, dim3(rows), dim3(256), 0, st, x, (const T*)a, a_stride,
                                      (const T*)wa, (const T*)b, b_stride, (const T*)wb, (const T*)bias, assign,
                                      (const T*)norm_w, (T*)h, W, eps, a_scale, w_offset, wa_offset));
  MXS_CHECK_LAUNCH();
}

void launch_cast_into(void* dst, long dst_stride, const float* x, int rows, int W, bool bf, hipStream_t st) {
  if (rows == 0) return;
  MIX_DISPATCH(bf, hipLaunchKernelGGL(cast_into_kernel<T>, dim3(rows), dim3(256), 0, st, (T*)dst, dst_stride, x, W));
  MXS_CHECK_LAUNCH();
}

void launch_relu_sq(void* out, const void* x, long n, bool bf, hipStream_t st) {
  if (n == 0) return;
  const int blocks = static_cast<int>(n / 256 + 1 < 4096 ? n / 256 + 1 : 4096);
  MIX_DISPATCH(bf, hipLaunchKernelGGL(relu_sq_kernel<T>, dim3(blocks), dim3(256), 0, st, (T*)out, (const T*)x, n));
  MXS_CHECK_LAUNCH();
}

void launch_softcap(float* out, const void* x, long x_stride, int rows, int V, float cap, bool bf, hipStream_t st) {
  if (rows == 0) return;
  MIX_DISPATCH(bf, hipLaunchKernelGGL(softcap_kernel<T>, dim3(rows), dim3(256), 0, st, out, (const T*)x, x_stride, V, cap));
  MXS_CHECK_LAUNCH();
}

void launch_gated_rms_norm(void* out, const float* o, const void* gate, long g_stride, const void* w, int rows, int N,
                           int groups, float eps, bool bf, hipStream_t st) {
  if (rows == 0) return;
  MIX_DISPATCH(bf, hipLaunchKernelGGL(gated_rms_norm_kernel<T>, dim3(rows), dim3(256), 0, st, (T*)out, o, (const T*)gate,
                                      g_stride, (const T*)w, N, groups, eps));
  MXS_CHECK_LAUNCH();
}

void launch_gate_linear(float* out, const void* h, long h_stride, const void* w, const void* bias, int rows, int N,
                        int W, bool bf, hipStream_t st) {
  if (rows == 0) return;
  const int el = bf ? 8 : 4;
  const int vec = W % el == 0 && h_stride % el == 0 && reinterpret_cast<uintptr_t>(h) % 16 == 0 &&
                  reinterpret_cast<uintptr_t>(w) % 16 == 0;
  MIX_DISPATCH(bf, hipLaunchKernelGGL(gate_linear_kernel<T>, dim3(rows), dim3(256), 0, st, out, (const T*)h, h_stride,
                                      (const T*)w, (const T*)bias, N, W, vec));
  MXS_CHECK_LAUNCH();
}

void launch_kv_write(void* cache, long block_stride, const void* k, long k_stride, const void* v, long v_stride,
                     const int64_t* slots, int rows, int koff, int voff, int G, int dk, int dv, int bs, bool bf,
                     hipStream_t st) {
  if (rows == 0) return;
  MIX_DISPATCH(bf, hipLaunchKernelGGL(kv_write_kernel<T>, dim3(rows), dim3(256), 0, st, (T*)cache, block_stride,
                                      (const T*)k, k_stride, (const T*)v, v_stride, slots, koff, voff, G, dk, dv, bs));
  MXS_CHECK_LAUNCH();
}

}  // namespace mxs
