// Small kernels of the latent attention and of the routed experts (gfx950).  Activations and
// weights are bf16 or fp32 (template T); norms, angles, router scores, routing weights and every sum
// are fp32, with one rounding where a result is stored.
//
//   latent_prep     per token: RMS norm of the query latent; RMS norm of the key/value latent and the
//                   rotary turn (half-split or neighbouring pairs) of the shared key part, both written into the token's page row
//   rope_half_into  per token and head: the rotated part of the query into its columns of the folded query
//   route_topk      sigmoid or softmax scores, the k largest per token (a wave per token)
//   capped_glu      g = min(gate, L), u = clamp(up, -L, L), g * sigmoid(alpha g) * (u + 1)
//   expert_align    counting sort of the (token, slot) pairs by expert: offsets and each pair's sorted row
//   gather_scaled   sorted rows = routing weight * the token's input
//   spread_scaled   [E, T, W] rows = routing weight * input for chosen experts, zero for the others
//   expert_combine  out[t] = sum of the token's k rows (given by place, or by expert inside an [E, T, W] stack), each
//                   optionally times its routing weight (+ a shared expert's row)
#include "mix_common.h"

namespace mxs {

#define MIX_DISPATCH(bf, ...)                      \
  do {                                             \
    if (bf) { using T = bf16_t; __VA_ARGS__; }     \
    else { using T = float; __VA_ARGS__; }         \
  } while (0)

template <typename T>
__global__ void __launch_bounds__(256) latent_prep_kernel(
    T* __restrict__ cq, const T* __restrict__ dq, long dq_stride, const T* __restrict__ dkv, long dkv_stride,
    const int64_t* __restrict__ positions, const int64_t* __restrict__ slots, T* __restrict__ cache, long block_stride,
    int koff, int qr, int rank, int nf, int bs, const float* __restrict__ freqs, const T* __restrict__ qn,
    const T* __restrict__ kvn, float eps, int split) {
  __shared__ float scratch[16];
  const long t = blockIdx.x;
  const T* a = dq + t * dq_stride;
  float s = 0.f;
  for (int c = threadIdx.x; c < qr; c += blockDim.x) { const float v = ldf(a + c); s += v * v; }
  const float rq = rsqrtf(block_sum(s, scratch) / static_cast<float>(qr) + eps);
  for (int c = threadIdx.x; c < qr; c += blockDim.x) stf(cq + t * qr + c, ldf(a + c) * rq * ldf(qn + c));
  const int64_t slot = slots[t];
  if (slot < 0) return;  // a padding row: the whole workgroup leaves
  const T* b = dkv + t * dkv_stride;
  s = 0.f;
  for (int c = threadIdx.x; c < rank; c += blockDim.x) { const float v = ldf(b + c); s += v * v; }
  const float rk = rsqrtf(block_sum(s, scratch) / static_cast<float>(rank) + eps);
  T* row = cache + (slot / bs) * block_stride + koff + (slot % bs) * static_cast<long>(rank + 2 * nf);
  for (int c = threadIdx.x; c < rank; c += blockDim.x) stf(row + c, ldf(b + c) * rk * ldf(kvn + c));
  const float pos = static_cast<float>(positions[t]);
  for (int i = threadIdx.x; i < nf; i += blockDim.x) {
    float sn, cs;
    sincosf(pos * freqs[i], &sn, &cs);
    // the pair's two columns: (i, i + nf) or neighbours (2i, 2i + 1)
    const int cu = split ? i : 2 * i, cv = split ? nf + i : 2 * i + 1;
    const float u = ldf(b + rank + cu), v = ldf(b + rank + cv);
    stf(row + rank + cu, u * cs - v * sn);
    stf(row + rank + cv, v * cs + u * sn);
  }
}

template <typename T>
__global__ void __launch_bounds__(256) rope_half_into_kernel(
    T* __restrict__ out, long out_stride, const T* __restrict__ x, long x_stride, const int64_t* __restrict__ positions,
    int heads, int x_dim, int x_col, int out_dim, int out_col, const float* __restrict__ freqs, int nf, int split) {
  const long t = blockIdx.x;
  const float pos = static_cast<float>(positions[t]);
  for (int idx = threadIdx.x; idx < heads * nf; idx += blockDim.x) {
    const int h = idx / nf, i = idx - h * nf;
    float sn, cs;
    sincosf(pos * freqs[i], &sn, &cs);
    const T* xp = x + t * x_stride + h * x_dim + x_col;
    T* op = out + t * out_stride + h * out_dim + out_col;
    const int cu = split ? i : 2 * i, cv = split ? nf + i : 2 * i + 1;
    const float u = ldf(xp + cu), v = ldf(xp + cv);
    stf(op + cu, u * cs - v * sn);
    stf(op + cv, v * cs + u * sn);
  }
}

// A wave per token.  Scores are sigmoid(logit), or the softmax over all E logits (maximum and sum by
// the wave first); the k largest are found by k passes of a wave-wide arg-max over the lanes' experts
// (ties: the lower index), so E and k are free.
__global__ void __launch_bounds__(256) route_topk_kernel(float* __restrict__ w, int* __restrict__ ids,
                                                         const float* __restrict__ logits, int T, int E, int k,
                                                         int renorm, int softmax) {
  const int lane = threadIdx.x & 63;
  const int t = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (t >= T) return;  // wave-uniform
  const float* z = logits + static_cast<long>(t) * E;
  float zmax = 0.f, zinv = 1.f;
  if (softmax) {
    float mx = -INFINITY;
    for (int e = lane; e < E; e += 64) mx = fmaxf(mx, z[e]);
    zmax = wave_max(mx);
    float sm = 0.f;
    for (int e = lane; e < E; e += 64) sm += expf(z[e] - zmax);
    zinv = 1.f / wave_sum(sm);
  }
  float total = 0.f;
  int last_id = -1;
  float last_s = INFINITY;
  for (int j = 0; j < k; ++j) {
    // the best expert not taken yet: smaller than the last one taken in (score desc, index asc) order
    float best = -INFINITY;
    int bi = 0x7fffffff;
    for (int e = lane; e < E; e += 64) {
      const float sc = softmax ? expf(z[e] - zmax) * zinv : sigmoid_f(z[e]);
      const bool after = sc < last_s || (sc == last_s && e > last_id);
      if (after && (sc > best || (sc == best && e < bi))) { best = sc; bi = e; }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (ob > best || (ob == best && oi < bi)) { best = ob; bi = oi; }
    }
    last_s = best;
    last_id = bi;
    total += best;
    if (lane == 0) {
      w[static_cast<long>(t) * k + j] = best;
      ids[static_cast<long>(t) * k + j] = bi;
    }
  }
  if (renorm && lane == 0) {
    const float inv = 1.f / total;
    for (int j = 0; j < k; ++j) w[static_cast<long>(t) * k + j] *= inv;  // own writes
  }
}

template <typename T>
__global__ void __launch_bounds__(256) capped_glu_kernel(T* __restrict__ out, const T* __restrict__ gu, long gu_stride,
                                                         int F, long n, float limit, float alpha) {
  for (long i = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x; i < n; i += static_cast<long>(gridDim.x) * blockDim.x) {
    const long r = i / F;
    const int c = static_cast<int>(i - r * F);
    const float g = fminf(ldf(gu + r * gu_stride + c), limit);
    const float u = fminf(fmaxf(ldf(gu + r * gu_stride + F + c), -limit), limit);
    stf(out + i, g * sigmoid_f(alpha * g) * (u + 1.f));
  }
}

// One workgroup.  Counts per expert in LDS, an exclusive scan by thread 0 (E is small beside n), then
// every pair takes the next free row of its expert.  The order of an expert's rows is whatever the
// atomics give: a row's result does not depend on its place.
__global__ void __launch_bounds__(1024) expert_align_kernel(int* __restrict__ offs, int* __restrict__ inv,
                                                            const int* __restrict__ ids, int n, int E) {
  extern __shared__ int cnt[];  // [E] counts, then each expert's next free row
  const int tid = threadIdx.x, nt = blockDim.x;
  for (int e = tid; e < E; e += nt) cnt[e] = 0;
  __syncthreads();
  for (int p = tid; p < n; p += nt) {
    const int e = ids[p];
    if (e >= 0 && e < E) atomicAdd(&cnt[e], 1);
  }
  __syncthreads();
  if (tid == 0) {
    int run = 0;
    for (int e = 0; e < E; ++e) { const int c = cnt[e]; offs[e] = run; cnt[e] = run; run += c; }
    offs[E] = run;
  }
  __syncthreads();
  for (int p = tid; p < n; p += nt) {
    const int e = ids[p];
    inv[p] = (e >= 0 && e < E) ? atomicAdd(&cnt[e], 1) : 0;
  }
}

template <typename T>
__global__ void __launch_bounds__(256) gather_scaled_kernel(T* __restrict__ xs, const T* __restrict__ h, long h_stride,
                                                            const float* __restrict__ w, const int* __restrict__ inv,
                                                            int k, int W) {
  const long p = blockIdx.x;
  const float wt = w ? w[p] : 1.f;
  const T* src = h + (p / k) * h_stride;
  T* dst = xs + static_cast<long>(inv[p]) * W;
  for (int c = threadIdx.x; c < W; c += blockDim.x) stf(dst + c, ldf(src + c) * wt);
}

template <typename T>
__global__ void __launch_bounds__(256) spread_scaled_kernel(T* __restrict__ xs, const T* __restrict__ h, long h_stride,
                                                            const float* __restrict__ w, const int* __restrict__ ids,
                                                            int Tn, int k, int W) {
  const int t = blockIdx.x, e = blockIdx.y;
  float wt = 0.f;
  for (int j = 0; j < k; ++j)
    if (ids[t * k + j] == e) wt += w ? w[t * k + j] : 1.f;
  const T* src = h + static_cast<long>(t) * h_stride;
  T* dst = xs + (static_cast<long>(e) * Tn + t) * W;
  for (int c = threadIdx.x; c < W; c += blockDim.x) stf(dst + c, wt == 0.f ? 0.f : ldf(src + c) * wt);
}

template <typename T>
__global__ void __launch_bounds__(256) expert_combine_kernel(T* __restrict__ out, const T* __restrict__ ys,
                                                             const int* __restrict__ index, int k, long row_stride,
                                                             const T* __restrict__ extra, long extra_stride, int W,
                                                             int vec, const float* __restrict__ wts, int by_expert) {
  constexpr int EL = El<T>::N;
  const long t = blockIdx.x;
  if (vec) {  // rows of whole, aligned 16-byte pieces: the k rows' loads of a piece are in flight together
    for (int c = threadIdx.x * EL; c < W; c += blockDim.x * EL) {
      float s[EL];
      if (extra) {
        load16(extra + t * extra_stride + c, s);
      } else {
#pragma unroll
        for (int e = 0; e < EL; ++e) s[e] = 0.f;
      }
#pragma unroll 4
      for (int j = 0; j < k; ++j) {
        const long r = index ? (by_expert ? index[t * k + j] * row_stride + t : index[t * k + j]) : j * row_stride + t;
        float v[EL];
        load16(ys + r * W + c, v);
        const float wt = wts ? wts[t * k + j] : 1.f;
#pragma unroll
        for (int e = 0; e < EL; ++e) s[e] += wt * v[e];
      }
      store16(out + t * W + c, s);
    }
    return;
  }
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float s = extra ? ldf(extra + t * extra_stride + c) : 0.f;
    for (int j = 0; j < k; ++j) {
      const long r = index ? (by_expert ? index[t * k + j] * row_stride + t : index[t * k + j]) : j * row_stride + t;
      s += (wts ? wts[t * k + j] : 1.f) * ldf(ys + r * W + c);
    }
    stf(out + t * W + c, s);
  }
}

void launch_latent_prep(void* cq, const void* dq, long dq_stride, const void* dkv, long dkv_stride,
                        const int64_t* positions, const int64_t* slots, void* cache, long block_stride, int rows, int koff,
                        int qr, int rank, int nf, int bs, const float* freqs, const void* qn, const void* kvn, float eps,
                        bool split, bool bf, hipStream_t st) {
  if (rows == 0) return;
  MIX_DISPATCH(bf, hipLaunchKernelGGL(latent_prep_kernel<T>, dim3(rows), dim3(256), 0, st, (T*)cq, (const T*)dq, dq_stride,
                                      (const T*)dkv, dkv_stride, positions, slots, (T*)cache, block_stride, koff, qr, rank,
                                      nf, bs, freqs, (const T*)qn, (const T*)kvn, eps, split ? 1 : 0));
  MXS_CHECK_LAUNCH();
}

void launch_rope_half_into(void* out, long out_stride, const void* x, long x_stride, const int64_t* positions, int rows,
                           int heads, int x_dim, int x_col, int out_dim, int out_col, const float* freqs, int nf,
                           bool split, bool bf, hipStream_t st) {
  if (rows == 0 || nf == 0) return;
  MIX_DISPATCH(bf, hipLaunchKernelGGL(rope_half_into_kernel<T>, dim3(rows), dim3(256), 0, st, (T*)out, out_stride,
                                      (const T*)x, x_stride, positions, heads, x_dim, x_col, out_dim, out_col, freqs, nf,
                                      split ? 1 : 0));
  MXS_CHECK_LAUNCH();
}

void launch_route_topk(float* w, int* ids, const float* logits, int T, int E, int k, bool renorm, bool softmax,
                       hipStream_t st) {
  if (T == 0) return;
  hipLaunchKernelGGL(route_topk_kernel, dim3((T + 3) / 4), dim3(256), 0, st, w, ids, logits, T, E, k, renorm ? 1 : 0,
                     softmax ? 1 : 0);
  MXS_CHECK_LAUNCH();
}

void launch_capped_glu(void* out, const void* gu, long gu_stride, int rows, int F, float limit, float alpha, bool bf,
                       hipStream_t st) {
  const long n = static_cast<long>(rows) * F;
  if (n == 0) return;
  const int blocks = static_cast<int>(std::min<long>((n + 255) / 256, 8192));
  MIX_DISPATCH(bf, hipLaunchKernelGGL(capped_glu_kernel<T>, dim3(blocks), dim3(256), 0, st, (T*)out, (const T*)gu, gu_stride,
                                      F, n, limit, alpha));
  MXS_CHECK_LAUNCH();
}

bool launch_expert_align(int* offs, int* inv, const int* ids, int n, int E, hipStream_t st) {
  const int nt = n >= 4096 ? 1024 : 256;
  const size_t shm = static_cast<size_t>(E) * sizeof(int);
  if (shm > 60 * 1024) return false;
  hipLaunchKernelGGL(expert_align_kernel, dim3(1), dim3(nt), shm, st, offs, inv, ids, n, E);
  MXS_CHECK_LAUNCH();
  return true;
}

void launch_gather_scaled(void* xs, const void* h, long h_stride, const float* w, const int* inv, int pairs, int k, int W,
                          bool bf, hipStream_t st) {
  if (pairs == 0) return;
  MIX_DISPATCH(bf, hipLaunchKernelGGL(gather_scaled_kernel<T>, dim3(pairs), dim3(256), 0, st, (T*)xs, (const T*)h, h_stride,
                                      w, inv, k, W));
  MXS_CHECK_LAUNCH();
}

void launch_spread_scaled(void* xs, const void* h, long h_stride, const float* w, const int* ids, int Tn, int E, int k,
                          int W, bool bf, hipStream_t st) {
  if (Tn == 0 || E == 0) return;
  MIX_DISPATCH(bf, hipLaunchKernelGGL(spread_scaled_kernel<T>, dim3(Tn, E), dim3(256), 0, st, (T*)xs, (const T*)h,
                                      h_stride, w, ids, Tn, k, W));
  MXS_CHECK_LAUNCH();
}

void launch_expert_combine(void* out, const void* ys, const int* index, int Tn, int k, long row_stride, const void* extra,
                           long extra_stride, int W, const float* wts, bool by_expert, bool bf, hipStream_t st) {
  if (Tn == 0) return;
  const int el = bf ? 8 : 4;
  const int vec = W % el == 0 && extra_stride % el == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0 &&
                  reinterpret_cast<uintptr_t>(ys) % 16 == 0 && reinterpret_cast<uintptr_t>(extra) % 16 == 0;
  MIX_DISPATCH(bf, hipLaunchKernelGGL(expert_combine_kernel<T>, dim3(Tn), dim3(256), 0, st, (T*)out, (const T*)ys, index, k,
                                      row_stride, (const T*)extra, extra_stride, W, vec, wts, by_expert ? 1 : 0));
  MXS_CHECK_LAUNCH();
}

}  // namespace mxs
