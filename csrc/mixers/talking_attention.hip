// Attention whose heads talk to one another before the softmax (gfx950): the scaled scores of a
// (query, key) pair are mixed over the heads, score_h <- sum_g talk[h, g] score_g, then masked (sliding
// window, kept first tokens), softmaxed per head (optionally with a sink in the denominator) and
// applied to the head's values.  Because a mixed score needs every head's raw score, a workgroup
// serves ALL heads of its query rows.
//
//   qkv_prep_cache   per token, one launch: biases, RMS norms of q and k (one over the whole row, or
//                    one per head), rotary turn of part of every head (half-split or neighbouring
//                    pairs, a factor on cos and sin), q rewritten in place, k and v into the pages
//   talking_attention (rows form)   one workgroup per query row, any dtype and size: prompt chunks in
//                    fp32, single decoded tokens
//   talking_attention (MFMA form)   bf16 prompt chunks: a workgroup owns 16 query rows, one wave per head
//                    (or several heads a wave); raw score tiles are exchanged through LDS
//   talking_attention (single-token MFMA form)   bf16 steps of single tokens: a workgroup owns one row, a wave
//                    one kv head (or several), a tile's columns are that kv head's query heads
// Scores, the mix, maxima, sums and output accumulators are fp32.
#include "mix_common.h"

namespace mxs {

#define MIX_DISPATCH(bf, ...)                      \
  do {                                             \
    if (bf) { using T = bf16_t; __VA_ARGS__; }     \
    else { using T = float; __VA_ARGS__; }         \
  } while (0)

// ------------------------------------------------------------------------------------------------
// norm_mode: 0 none, 1 one RMS norm per head (weights [dk]), 2 one over the whole row (weights [heads * dk])
template <typename T>
__device__ __forceinline__ void prep_row(const T* __restrict__ src, T* __restrict__ dst, int heads, int dk,
                                         const T* __restrict__ bias, const T* __restrict__ nw, int norm_mode,
                                         float eps, const float* __restrict__ cs_t, const float* __restrict__ sn_t,
                                         int nf, int split, float* __restrict__ rh, float* __restrict__ scratch, bool write,
                                         long head_stride) {
  // src: the projection's row [heads * dk]; dst: element (hd, c) goes to dst[hd * head_stride + c]
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6, nw_ = blockDim.x >> 6;
  const int n = heads * dk;
  float rall = 1.f;
  if (norm_mode == 2 && nw) {
    float s = 0.f;
    for (int c = threadIdx.x; c < n; c += blockDim.x) {
      const float v = ldf(src + c) + (bias ? ldf(bias + c) : 0.f);
      s += v * v;
    }
    rall = rsqrtf(block_sum(s, scratch) / static_cast<float>(n) + eps);
  } else if (norm_mode == 1 && nw) {
    for (int hd = wid; hd < heads; hd += nw_) {
      float s = 0.f;
      for (int c = lane; c < dk; c += 64) {
        const float v = ldf(src + hd * dk + c) + (bias ? ldf(bias + hd * dk + c) : 0.f);
        s += v * v;
      }
      s = wave_sum(s);
      if (lane == 0) rh[hd] = rsqrtf(s / static_cast<float>(dk) + eps);
    }
    __syncthreads();
  }
  if (!write) return;  // block-uniform
  auto val = [&](int hd, int c) -> float {
    const int i = hd * dk + c;
    float v = ldf(src + i) + (bias ? ldf(bias + i) : 0.f);
    if (nw) v *= norm_mode == 2 ? rall * ldf(nw + i) : (norm_mode == 1 ? rh[hd] * ldf(nw + c) : 1.f);
    return v;
  };
  // every element is read and written by exactly one thread (a pair by the thread that turns it)
  for (int idx = threadIdx.x; idx < heads * nf; idx += blockDim.x) {
    const int hd = idx / nf, p = idx - hd * nf;
    const int cu = split ? p : 2 * p, cv = split ? p + nf : 2 * p + 1;
    const float sn = sn_t[p], cs = cs_t[p];  // the pair's turn, made once per token for all heads
    const float u = val(hd, cu), v = val(hd, cv);
    stf(dst + hd * head_stride + cu, u * cs - v * sn);
    stf(dst + hd * head_stride + cv, v * cs + u * sn);
  }
  const int rest = dk - 2 * nf;
  for (int idx = threadIdx.x; idx < heads * rest; idx += blockDim.x) {
    const int hd = idx / rest, c = 2 * nf + (idx - hd * rest);
    stf(dst + hd * head_stride + c, val(hd, c));
  }
}

template <typename T>
__global__ void __launch_bounds__(256) qkv_prep_cache_kernel(
    T* __restrict__ q, long q_stride, const T* __restrict__ k, long k_stride, const T* __restrict__ v, long v_stride,
    const int64_t* __restrict__ positions, const int64_t* __restrict__ slots, T* __restrict__ cache, long block_stride,
    int koff, int voff, int H, int G, int dk, int dv, int bs, const float* __restrict__ freqs, int nf, float mag,
    int split, const T* __restrict__ bq, const T* __restrict__ bk, const T* __restrict__ bv, const T* __restrict__ qn,
    const T* __restrict__ kn, float eps, int norm_mode) {
  extern __shared__ float rh[];  // [max(H, G)] per-head inverse rms, then cos [nf] and sin [nf] of the token's turns
  __shared__ float scratch[16];
  const long t = blockIdx.x;
  const float pos = static_cast<float>(positions[t]);
  float* cs_t = rh + max(H, G);
  float* sn_t = cs_t + nf;
  for (int p = threadIdx.x; p < nf; p += blockDim.x) {
    float sn, cs;
    sincosf(pos * freqs[p], &sn, &cs);
    cs_t[p] = cs * mag;
    sn_t[p] = sn * mag;
  }
  __syncthreads();
  // blockIdx.y == 0: the queries; 1: keys and values (two workgroups a token, so that single-token steps,
  // which are a chain of dependent passes, run the two chains side by side)
  if (blockIdx.y == 0) {
    T* qr = q + t * q_stride;
    prep_row<T>(qr, qr, H, dk, bq, qn, norm_mode, eps, cs_t, sn_t, nf, split, rh, scratch, true, dk);
    return;
  }
  const int64_t slot = slots[t];
  const bool wr = slot >= 0;  // a padding row writes nothing (block-uniform)
  T* base = cache + (wr ? slot / bs : 0) * block_stride;
  const int off = wr ? static_cast<int>(slot % bs) : 0;
  prep_row<T>(k + t * k_stride, base + koff + static_cast<long>(off) * dk, G, dk, bk, kn, norm_mode, eps, cs_t, sn_t, nf,
              split, rh, scratch, wr, static_cast<long>(bs) * dk);
  if (!wr) return;
  const T* vr = v + t * v_stride;
  for (int i = threadIdx.x; i < G * dv; i += blockDim.x) {
    const int g = i / dv, d = i - g * dv;
    stf(base + voff + (static_cast<long>(g) * bs + off) * dv + d, ldf(vr + i) + (bv ? ldf(bv + i) : 0.f));
  }
}

// ------------------------------------------------------------------------------------------------
// Rows form.  Visible keys are walked in tiles of 64 (one key per lane of a wave in the softmax step):
//   1. raw[h][n] = q_h . k_n for all heads (thread per (head, key), the scaled query in LDS)
//   2. mixed[h][n] = sum_g talk[h][g] raw[g][n]
//   3. per head (a wave each, in turn): running maximum and sum, weights e^(s - m) back into LDS
//   4. every thread owns NACC (head, value column) outputs: rescale, then add weight * value over the tile
constexpr int kTalkTile = 64;

template <typename T, int NACC>
__global__ void __launch_bounds__(256) talking_attention_rows_kernel(
    T* __restrict__ out, const T* __restrict__ q, long q_stride, const T* __restrict__ cache, long block_stride,
    const int* __restrict__ block_tables, int bt_stride, const int* __restrict__ qsl, const int* __restrict__ seq_lens,
    int S, int koff, int voff, int H, int G, int dk, int dv, int bs, float scale, int window, int keep, bool vec,
    const float* __restrict__ sink, const float* __restrict__ talk) {
  extern __shared__ float lds[];
  const int dkp = (dk + 3) & ~3;
  float* qs = lds;                         // [H][dkp]
  float* tk = qs + H * dkp;                // [H][H]
  float* raw = tk + H * H;                 // [H][64]
  float* pw = raw + H * kTalkTile;         // [H][64] mixed scores, then weights
  float* ms = pw + H * kTalkTile;          // [H] running maxima
  float* ls = ms + H;                      // [H] running sums
  float* cr = ls + H;                      // [H] this tile's rescale factors
  const int t = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wid = tid >> 6;
  const int s = seq_of_row(qsl, S, t);
  const int qlen = qsl[s + 1] - qsl[s];
  const int pos = min(max(seq_lens[s] - qlen + (t - qsl[s]), 0), bt_stride * bs - 1);
  const int lo = window > 0 ? max(pos - window + 1, 0) : 0;
  const int nA = window > 0 ? min(keep, lo) : 0;  // kept first tokens that lie below the window
  const int nvis = nA + (pos - lo + 1);
  const int R = H / G;
  const int* bt = block_tables + static_cast<long>(s) * bt_stride;
  for (int i = tid; i < H * dk; i += blockDim.x) {
    const int hd = i / dk, d = i - hd * dk;
    qs[hd * dkp + d] = ldf(q + static_cast<long>(t) * q_stride + i) * scale;
  }
  for (int i = tid; i < H * H; i += blockDim.x) tk[i] = talk[i];
  for (int i = tid; i < H; i += blockDim.x) {
    ms[i] = sink ? sink[i] : -INFINITY;
    ls[i] = sink ? 1.f : 0.f;
  }
  float acc[NACC];
#pragma unroll
  for (int c = 0; c < NACC; ++c) acc[c] = 0.f;
  const int nout = H * dv;
  __syncthreads();
  for (int t0 = 0; t0 < nvis; t0 += kTalkTile) {
    const int nt = min(kTalkTile, nvis - t0);
    // 1. raw scores: neighbouring threads take neighbouring keys of one head
    for (int idx = tid; idx < H * nt; idx += blockDim.x) {
      const int hd = idx / nt, n = idx - hd * nt;
      const int nn = t0 + n;
      const int j = nn < nA ? nn : lo + (nn - nA);
      const T* kp = cache + static_cast<long>(bt[j / bs]) * block_stride + koff + (static_cast<long>(hd / R) * bs + j % bs) * dk;
      raw[hd * kTalkTile + n] = dot_row<T>(qs + hd * dkp, kp, dk, vec);
    }
    __syncthreads();
    // 2. the heads' scores mixed
    for (int idx = tid; idx < H * nt; idx += blockDim.x) {
      const int hd = idx / nt, n = idx - hd * nt;
      float sc = 0.f;
      for (int g = 0; g < H; ++g) sc += tk[hd * H + g] * raw[g * kTalkTile + n];
      pw[hd * kTalkTile + n] = sc;
    }
    __syncthreads();
    // 3. online softmax, a wave per head
    for (int hd = wid; hd < H; hd += 4) {
      const float sc = lane < nt ? pw[hd * kTalkTile + lane] : -INFINITY;
      const float m_old = ms[hd];
      const float m_new = fmaxf(m_old, wave_max(sc));
      const float e = lane < nt ? expf(sc - m_new) : 0.f;
      const float sum = wave_sum(e);
      pw[hd * kTalkTile + lane] = e;
      if (lane == 0) {
        const float corr = m_old == -INFINITY ? 0.f : expf(m_old - m_new);
        cr[hd] = corr;
        ls[hd] = ls[hd] * corr + sum;
        ms[hd] = m_new;
      }
    }
    __syncthreads();
    // 4. values
#pragma unroll
    for (int c = 0; c < NACC; ++c) {
      const int o = tid + 256 * c;
      if (o < nout) {
        const int hd = o / dv, e = o - hd * dv;
        float a = acc[c] * cr[hd];
        const float* pr = pw + hd * kTalkTile;
        const long vcol = static_cast<long>(hd / R) * bs * dv + e;
        for (int n = 0; n < nt; ++n) {
          const int nn = t0 + n;
          const int j = nn < nA ? nn : lo + (nn - nA);
          a += pr[n] * ldf(cache + static_cast<long>(bt[j / bs]) * block_stride + voff + vcol + static_cast<long>(j % bs) * dv);
        }
        acc[c] = a;
      }
    }
    __syncthreads();  // raw, pw and cr are rewritten by the next tile
  }
#pragma unroll
  for (int c = 0; c < NACC; ++c) {
    const int o = tid + 256 * c;
    if (o < nout) stf(out + static_cast<long>(t) * nout + o, acc[c] / ls[o / dv]);
  }
}

// ------------------------------------------------------------------------------------------------
// MFMA form (bf16, 16-token cache blocks, head sizes multiples of 16 up to 128).  A workgroup owns 16
// consecutive query rows of one sequence and all H heads; wave w serves the heads w, w + NW, ...
// (HPW of them).  Per visible 16-key block, with v_mfma_f32_16x16x16_bf16:
//   a. every wave: S_h^T = K_g Q_h^T for its heads (A = the block's key rows, B = Q^T kept in registers),
//      the raw fp32 tile written to LDS [H][16 keys][16 queries]
//   b. barrier; every wave mixes its heads' tiles from all H raw tiles (fp32 on the vector units),
//      masks, and runs the online softmax of its heads (the query on the lane, 4 keys a lane)
//   c. O_h^T += V_g^T P_h^T with every weight as two bf16 halves; the block's value rows go through
//      the wave's LDS area to become the key-contiguous A operand
//   d. barrier (the raw tiles are rewritten by the next block)
// With nsplit > 1 (steps of few rows, e.g. single decoded tokens) the visible blocks are divided over
// nsplit workgroups; each writes (maximum, sum, unnormalised output) per row and head, and the merge
// kernel of the latent attention combines them.
bool launch_attention_combine(void* out, const float* part, long rows, int nsplit, int width, hipStream_t st);

typedef short s4_t __attribute__((ext_vector_type(4)));
typedef float f4_t __attribute__((ext_vector_type(4)));

template <int KSM, int VTM, int HPW, int NW>
__global__ void __launch_bounds__(64 * NW) talking_attention_mfma_kernel(
    bf16_t* __restrict__ out, const bf16_t* __restrict__ q, long q_stride, const bf16_t* __restrict__ cache,
    long block_stride, const int* __restrict__ block_tables, int bt_stride, const int* __restrict__ qsl,
    const int* __restrict__ seq_lens, int koff, int voff, int H, int G, int dk, int dv, float scale, int window,
    int keep, const float* __restrict__ sink, const float* __restrict__ talk, float* __restrict__ part, int nsplit) {
  extern __shared__ __attribute__((aligned(16))) float tlds[];
  // [H][256] raw tiles (lane-major: element (lane, i) at lane * 4 + i), then [H][H] talk, then the waves' value areas
  float* raw = tlds;
  float* tk = raw + H * 256;
  const int DVP = dv + 8;
  bf16_t* vw = reinterpret_cast<bf16_t*>(tk + ((H * H + 3) & ~3)) + (threadIdx.x >> 6) * (16 * DVP);
  const int s = blockIdx.y, sp = blockIdx.z;
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  const int row0 = qsl[s], qlen = qsl[s + 1] - row0;
  const int qt0 = blockIdx.x * 16;
  if (qt0 >= qlen) return;  // workgroup-uniform
  const int nq = min(16, qlen - qt0);
  const int pos0 = min(max(seq_lens[s] - qlen + qt0, 0), bt_stride * 16 - nq);
  const int c = lane & 15, kg = lane >> 4;
  const int KS = dk >> 4, VT = dv >> 4, R = H / G;
  const bool qok = c < nq;
  const int pq = pos0 + c;
  const int* bt = block_tables + static_cast<long>(s) * bt_stride;
  for (int i = threadIdx.x; i < H * H; i += blockDim.x) tk[i] = talk[i];
  s4_t qf[HPW][KSM];
  float m[HPW], l[HPW];
  f4_t o[HPW][VTM];
#pragma unroll
  for (int j = 0; j < HPW; ++j) {
    const int hd = wid + j * NW;
    const bool hok = hd < H;
    const bf16_t* qp = q + static_cast<long>(row0 + qt0 + (qok ? c : 0)) * q_stride + (hok ? hd : 0) * dk + 4 * kg;
#pragma unroll
    for (int ks = 0; ks < KSM; ++ks)
      qf[j][ks] = (ks < KS && qok && hok) ? *reinterpret_cast<const s4_t*>(qp + 16 * ks) : s4_t{0, 0, 0, 0};
    m[j] = (sink && hok && sp == 0) ? sink[hd] * 1.4426950408889634f : -INFINITY;  // the sink counts once: in the first stretch
    l[j] = (sink && hok && sp == 0 && kg == 0) ? 1.f : 0.f;
#pragma unroll
    for (int vt = 0; vt < VTM; ++vt) o[j][vt] = f4_t{0.f, 0.f, 0.f, 0.f};
  }
  const int p_last = pos0 + nq - 1;
  const int lo_first = window > 0 ? max(pos0 - window + 1, 0) : 0;
  const int wb = lo_first >> 4, lastb = p_last >> 4;
  const int kA = window > 0 ? min((keep + 15) >> 4, wb) : 0;
  const float sl2 = scale * 1.4426950408889634f;
  const int nit = kA + (lastb - wb + 1);
  const int it0 = static_cast<int>(static_cast<long>(nit) * sp / nsplit);
  const int it1 = static_cast<int>(static_cast<long>(nit) * (sp + 1) / nsplit);
  __syncthreads();
  for (int it = it0; it < it1; ++it) {
    const int kb = it < kA ? it : wb + (it - kA);
    const bf16_t* blk = cache + static_cast<long>(bt[kb]) * block_stride;
    const int k0 = kb * 16;
    // a. raw tiles of this wave's heads
#pragma unroll
    for (int j = 0; j < HPW; ++j) {
      const int hd = wid + j * NW;
      if (hd < H) {
        f4_t acc = f4_t{0.f, 0.f, 0.f, 0.f};
        const bf16_t* kp = blk + koff + (static_cast<long>(hd / R) * 16 + c) * dk + 4 * kg;
#pragma unroll
        for (int ks = 0; ks < KSM; ++ks)
          if (ks < KS)
            acc = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(*reinterpret_cast<const s4_t*>(kp + 16 * ks), qf[j][ks], acc, 0, 0, 0);
        // key rows past the tile's last position may hold anything (also NaN or inf): they are masked below,
        // but a mix over the heads would spread a NaN through 0 * NaN: store them as 0
        if (k0 + 15 > p_last) {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (k0 + 4 * kg + i > p_last) acc[i] = 0.f;
        }
        if (qok) *reinterpret_cast<f4_t*>(raw + hd * 256 + lane * 4) = acc;  // a 1-row tile moves a sixteenth of the tile
      }
    }
    __syncthreads();
    const bool whole = k0 + 15 <= pos0 && (window <= 0 || k0 >= p_last - window + 1 || k0 + 15 < keep);
    const bool vall = k0 + 15 <= p_last;
#pragma unroll
    for (int j = 0; j < HPW; ++j) {
      const int hd = wid + j * NW;
      if (hd >= H) continue;  // wave-uniform
      // b. mix and softmax
      f4_t mx4 = f4_t{0.f, 0.f, 0.f, 0.f};
      const float* trow = tk + hd * H;
      if (qok) {  // lanes of rows the tile does not have read nothing: single tokens need a sixteenth of the LDS traffic
        for (int g = 0; g < H; ++g) {
          const f4_t r = *reinterpret_cast<const f4_t*>(raw + g * 256 + lane * 4);
          const float tw = trow[g];
#pragma unroll
          for (int i = 0; i < 4; ++i) mx4[i] += tw * r[i];
        }
      }
      float sv[4], mx = -INFINITY;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (whole) {
          sv[i] = mx4[i] * sl2;
        } else {
          const int jk = k0 + 4 * kg + i;
          const bool vis = qok && jk <= pq && (window <= 0 || pq - jk < window || jk < keep);
          sv[i] = vis ? mx4[i] * sl2 : -INFINITY;
        }
        mx = fmaxf(mx, sv[i]);
      }
      mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float m_new = fmaxf(m[j], mx);
      if (__builtin_amdgcn_ballot_w64(m_new > m[j]) != 0) {
        const float corr = m_new == -INFINITY ? 1.f : __builtin_amdgcn_exp2f(m[j] - m_new);
        l[j] *= corr;
#pragma unroll
        for (int vt = 0; vt < VTM; ++vt)
#pragma unroll
          for (int i = 0; i < 4; ++i) o[j][vt][i] *= corr;
        m[j] = m_new;
      }
      s4_t ph, pl;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float pr = (whole || sv[i] != -INFINITY) ? __builtin_amdgcn_exp2f(sv[i] - m[j]) : 0.f;
        l[j] += pr;
        // pr = hi + lo: hi the upper 16 bits (exact), lo = pr - hi rounded to bf16 (pr >= 0, finite)
        const uint32_t u = __float_as_uint(pr), uh = u & 0xFFFF0000u;
        uint32_t ul = __float_as_uint(pr - __uint_as_float(uh));
        ul += 0x7FFFu + ((ul >> 16) & 1u);
        ph[i] = static_cast<short>(uh >> 16);
        pl[i] = static_cast<short>(ul >> 16);
      }
      // c. values of the head's kv head through the wave's LDS area
      const bf16_t* vblk = blk + voff + static_cast<long>(hd / R) * 16 * dv;
      __builtin_amdgcn_wave_barrier();  // the previous head's reads come first
#pragma unroll
      for (int r = 0; r < (VTM + 1) / 2; ++r) {
        const int idx = lane + 64 * r;  // 16-byte piece
        if (idx < 2 * dv) {
          const int e0 = idx * 8, vr = e0 / dv, vc = e0 - vr * dv;
          *reinterpret_cast<uint4*>(vw + vr * DVP + vc) = *reinterpret_cast<const uint4*>(vblk + e0);
        }
      }
      __builtin_amdgcn_wave_barrier();
      const bf16_t* vp = vw + 4 * kg * DVP + c;
#pragma unroll
      for (int vt = 0; vt < VTM; ++vt) {
        if (vt < VT) {
          s4_t a;
#pragma unroll
          for (int i = 0; i < 4; ++i)  // rows past the sequence's last token may hold anything: read them as 0
            a[i] = (vall || k0 + 4 * kg + i <= p_last) ? static_cast<short>(vp[i * DVP + 16 * vt]) : short(0);
          const f4_t t = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, ph, o[j][vt], 0, 0, 0);
          o[j][vt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, pl, t, 0, 0, 0);
        }
      }
    }
    __syncthreads();  // d. the raw tiles are rewritten by the next block
  }
#pragma unroll
  for (int j = 0; j < HPW; ++j) {
    const int hd = wid + j * NW;
    float lj = l[j];
    lj += __shfl_xor(lj, 16, 64);
    lj += __shfl_xor(lj, 32, 64);
    if (hd >= H || !qok) continue;
    if (nsplit > 1) {
      float* pp = part + ((static_cast<long>(row0 + qt0 + c) * H + hd) * nsplit + sp) * (dv + 4);
      if (kg == 0) { pp[0] = m[j]; pp[1] = lj; }
#pragma unroll
      for (int vt = 0; vt < VTM; ++vt)
        if (vt < VT) *reinterpret_cast<f4_t*>(pp + 4 + 16 * vt + 4 * kg) = o[j][vt];
      continue;
    }
    const float inv = 1.f / lj;
    bf16_t* op = out + static_cast<long>(row0 + qt0 + c) * (H * dv) + hd * dv + 4 * kg;
#pragma unroll
    for (int vt = 0; vt < VTM; ++vt) {
      if (vt < VT) {
        uint2 w;
        w.x = pack2(o[j][vt][0] * inv, o[j][vt][1] * inv);
        w.y = pack2(o[j][vt][2] * inv, o[j][vt][3] * inv);
        *reinterpret_cast<uint2*>(op + 16 * vt) = w;
      }
    }
  }
}

// ---- Single-token form (bf16, same sizes): a workgroup owns ONE query row.  The 16 columns of a tile are
// the R = H / G query heads of one kv head (R <= 16) instead of 16 rows of one head, and wave w serves the
// kv heads w, w + NW, ...: a block's keys and values are loaded and multiplied once per kv head, not once
// per query head, and R of the 16 columns do useful work instead of one.  The raw scores are [H][16 keys]
// in LDS; the mix, the softmax and the split over nsplit workgroups are those of the form above.
template <int KSM, int VTM, int GPW, int NW>
__global__ void __launch_bounds__(64 * NW) talking_attention_token_kernel(
    bf16_t* __restrict__ out, const bf16_t* __restrict__ q, long q_stride, const bf16_t* __restrict__ cache,
    long block_stride, const int* __restrict__ block_tables, int bt_stride, const int* __restrict__ qsl,
    const int* __restrict__ seq_lens, int S, int koff, int voff, int H, int G, int dk, int dv, float scale, int window,
    int keep, const float* __restrict__ sink, const float* __restrict__ talk, float* __restrict__ part, int nsplit) {
  extern __shared__ __attribute__((aligned(16))) float tlds[];
  float* raw = tlds;            // [H][16]
  float* tk = raw + H * 16;     // [H][H]
  const int DVP = dv + 8;
  bf16_t* vw = reinterpret_cast<bf16_t*>(tk + ((H * H + 3) & ~3)) + (threadIdx.x >> 6) * (16 * DVP);
  const int t = blockIdx.x, sp = blockIdx.y;
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  const int s = seq_of_row(qsl, S, t);
  const int qlen = qsl[s + 1] - qsl[s];
  const int pos = min(max(seq_lens[s] - qlen + (t - qsl[s]), 0), bt_stride * 16 - 1);
  const int c = lane & 15, kg = lane >> 4;
  const int KS = dk >> 4, VT = dv >> 4, R = H / G;
  const bool qok = c < R;
  const int* bt = block_tables + static_cast<long>(s) * bt_stride;
  for (int i = threadIdx.x; i < H * H; i += blockDim.x) tk[i] = talk[i];
  s4_t qf[GPW][KSM];
  float m[GPW], l[GPW];
  f4_t o[GPW][VTM];
#pragma unroll
  for (int j = 0; j < GPW; ++j) {
    const int g = wid + j * NW;
    const bool ok = qok && g < G;
    const int hd = ok ? g * R + c : 0;
    const bf16_t* qp = q + static_cast<long>(t) * q_stride + hd * dk + 4 * kg;
#pragma unroll
    for (int ks = 0; ks < KSM; ++ks)
      qf[j][ks] = (ks < KS && ok) ? *reinterpret_cast<const s4_t*>(qp + 16 * ks) : s4_t{0, 0, 0, 0};
    m[j] = (sink && ok && sp == 0) ? sink[hd] * 1.4426950408889634f : -INFINITY;
    l[j] = (sink && ok && sp == 0 && kg == 0) ? 1.f : 0.f;
#pragma unroll
    for (int vt = 0; vt < VTM; ++vt) o[j][vt] = f4_t{0.f, 0.f, 0.f, 0.f};
  }
  const int lo_first = window > 0 ? max(pos - window + 1, 0) : 0;
  const int wb = lo_first >> 4, lastb = pos >> 4;
  const int kA = window > 0 ? min((keep + 15) >> 4, wb) : 0;
  const float sl2 = scale * 1.4426950408889634f;
  const int nit = kA + (lastb - wb + 1);
  const int it0 = static_cast<int>(static_cast<long>(nit) * sp / nsplit);
  const int it1 = static_cast<int>(static_cast<long>(nit) * (sp + 1) / nsplit);
  __syncthreads();
  for (int it = it0; it < it1; ++it) {
    const int kb = it < kA ? it : wb + (it - kA);
    const bf16_t* blk = cache + static_cast<long>(bt[kb]) * block_stride;
    const int k0 = kb * 16;
#pragma unroll
    for (int j = 0; j < GPW; ++j) {
      const int g = wid + j * NW;
      if (g < G) {
        f4_t acc = f4_t{0.f, 0.f, 0.f, 0.f};
        const bf16_t* kp = blk + koff + (static_cast<long>(g) * 16 + c) * dk + 4 * kg;
#pragma unroll
        for (int ks = 0; ks < KSM; ++ks)
          if (ks < KS)
            acc = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(*reinterpret_cast<const s4_t*>(kp + 16 * ks), qf[j][ks], acc, 0, 0, 0);
        if (k0 + 15 > pos) {  // stale rows behind the sequence's end: zeros, before they can meet the mix
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (k0 + 4 * kg + i > pos) acc[i] = 0.f;
        }
        if (qok) *reinterpret_cast<f4_t*>(raw + (g * R + c) * 16 + 4 * kg) = acc;
      }
    }
    __syncthreads();
    const bool whole = k0 + 15 <= pos && (window <= 0 || k0 >= pos - window + 1 || k0 + 15 < keep);
    const bool vall = k0 + 15 <= pos;
#pragma unroll
    for (int j = 0; j < GPW; ++j) {
      const int g = wid + j * NW;
      if (g >= G) continue;  // wave-uniform
      f4_t mx4 = f4_t{0.f, 0.f, 0.f, 0.f};
      if (qok) {
        const float* trow = tk + (g * R + c) * H;
        for (int g2 = 0; g2 < H; ++g2) {
          const f4_t r = *reinterpret_cast<const f4_t*>(raw + g2 * 16 + 4 * kg);
          const float tw = trow[g2];
#pragma unroll
          for (int i = 0; i < 4; ++i) mx4[i] += tw * r[i];
        }
      }
      float sv[4], mx = -INFINITY;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int jk = k0 + 4 * kg + i;
        const bool vis = qok && (whole || (jk <= pos && (window <= 0 || pos - jk < window || jk < keep)));
        sv[i] = vis ? mx4[i] * sl2 : -INFINITY;
        mx = fmaxf(mx, sv[i]);
      }
      mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float m_new = fmaxf(m[j], mx);
      if (__builtin_amdgcn_ballot_w64(m_new > m[j]) != 0) {
        const float corr = m_new == -INFINITY ? 1.f : __builtin_amdgcn_exp2f(m[j] - m_new);
        l[j] *= corr;
#pragma unroll
        for (int vt = 0; vt < VTM; ++vt)
#pragma unroll
          for (int i = 0; i < 4; ++i) o[j][vt][i] *= corr;
        m[j] = m_new;
      }
      s4_t ph, pl;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float pr = sv[i] != -INFINITY ? __builtin_amdgcn_exp2f(sv[i] - m[j]) : 0.f;
        l[j] += pr;
        const uint32_t u = __float_as_uint(pr), uh = u & 0xFFFF0000u;
        uint32_t ul = __float_as_uint(pr - __uint_as_float(uh));
        ul += 0x7FFFu + ((ul >> 16) & 1u);
        ph[i] = static_cast<short>(uh >> 16);
        pl[i] = static_cast<short>(ul >> 16);
      }
      const bf16_t* vblk = blk + voff + static_cast<long>(g) * 16 * dv;
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int r = 0; r < (VTM + 1) / 2; ++r) {
        const int idx = lane + 64 * r;
        if (idx < 2 * dv) {
          const int e0 = idx * 8, vr = e0 / dv, vc = e0 - vr * dv;
          *reinterpret_cast<uint4*>(vw + vr * DVP + vc) = *reinterpret_cast<const uint4*>(vblk + e0);
        }
      }
      __builtin_amdgcn_wave_barrier();
      const bf16_t* vp = vw + 4 * kg * DVP + c;
#pragma unroll
      for (int vt = 0; vt < VTM; ++vt) {
        if (vt < VT) {
          s4_t a;
#pragma unroll
          for (int i = 0; i < 4; ++i)
            a[i] = (vall || k0 + 4 * kg + i <= pos) ? static_cast<short>(vp[i * DVP + 16 * vt]) : short(0);
          const f4_t tt = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, ph, o[j][vt], 0, 0, 0);
          o[j][vt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, pl, tt, 0, 0, 0);
        }
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int j = 0; j < GPW; ++j) {
    const int g = wid + j * NW;
    float lj = l[j];
    lj += __shfl_xor(lj, 16, 64);
    lj += __shfl_xor(lj, 32, 64);
    if (g >= G || !qok) continue;
    const int hd = g * R + c;
    if (nsplit > 1) {
      float* pp = part + ((static_cast<long>(t) * H + hd) * nsplit + sp) * (dv + 4);
      if (kg == 0) { pp[0] = m[j]; pp[1] = lj; }
#pragma unroll
      for (int vt = 0; vt < VTM; ++vt)
        if (vt < VT) *reinterpret_cast<f4_t*>(pp + 4 + 16 * vt + 4 * kg) = o[j][vt];
      continue;
    }
    const float inv = 1.f / lj;
    bf16_t* op = out + static_cast<long>(t) * (H * dv) + hd * dv + 4 * kg;
#pragma unroll
    for (int vt = 0; vt < VTM; ++vt) {
      if (vt < VT) {
        uint2 w;
        w.x = pack2(o[j][vt][0] * inv, o[j][vt][1] * inv);
        w.y = pack2(o[j][vt][2] * inv, o[j][vt][3] * inv);
        *reinterpret_cast<uint2*>(op + 16 * vt) = w;
      }
    }
  }
}

void launch_qkv_prep_cache(void* q, long q_stride, const void* k, long k_stride, const void* v, long v_stride,
                           const int64_t* positions, const int64_t* slots, void* cache, long block_stride, int rows,
                           int koff, int voff, int H, int G, int dk, int dv, int bs, const float* freqs, int nf, float mag,
                           bool split, const void* bq, const void* bk, const void* bv, const void* qn, const void* kn,
                           float eps, int norm_mode, bool bf, hipStream_t st) {
  if (rows == 0) return;
  const size_t shm = static_cast<size_t>(std::max(H, G) + 2 * nf) * sizeof(float);
  MIX_DISPATCH(bf, hipLaunchKernelGGL(qkv_prep_cache_kernel<T>, dim3(rows, k ? 2 : 1), dim3(256), shm, st, (T*)q, q_stride, (const T*)k,
                                      k_stride, (const T*)v, v_stride, positions, slots, (T*)cache, block_stride, koff, voff,
                                      H, G, dk, dv, bs, freqs, nf, mag, split ? 1 : 0, (const T*)bq, (const T*)bk,
                                      (const T*)bv, (const T*)qn, (const T*)kn, eps, norm_mode));
  MXS_CHECK_LAUNCH();
}

template <int KSM, int VTM, int HPW, int NW>
static bool launch_talking_mfma(void* out, const void* q, long q_stride, const void* cache, long block_stride,
                                const int* block_tables, int bt_stride, const int* qsl, const int* seq_lens, int S, int koff,
                                int voff, int H, int G, int dk, int dv, float scale, int window, int keep, int max_q,
                                const float* sink, const float* talk, float* part, int nsplit, hipStream_t st) {
  const size_t shm = (static_cast<size_t>(H) * 256 + ((H * H + 3) & ~3)) * sizeof(float) +
                     static_cast<size_t>(NW) * 16 * (dv + 8) * sizeof(bf16_t);
  if (shm > 160 * 1024) return false;
  if (shm > 48 * 1024) {  // beyond the default dynamic LDS of a workgroup: asked for once per kernel
    static bool raised = false;
    if (!raised) {
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(&talking_attention_mfma_kernel<KSM, VTM, HPW, NW>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess) {
        (void)hipGetLastError();
        return false;
      }
      raised = true;
    }
  }
  hipLaunchKernelGGL((talking_attention_mfma_kernel<KSM, VTM, HPW, NW>), dim3((max_q + 15) / 16, S, nsplit), dim3(64 * NW),
                     shm, st, (bf16_t*)out, (const bf16_t*)q, q_stride, (const bf16_t*)cache, block_stride, block_tables,
                     bt_stride, qsl, seq_lens, koff, voff, H, G, dk, dv, scale, window, keep, sink, talk, part, nsplit);
  MXS_CHECK_LAUNCH();
  return true;
}

template <int KSM, int VTM, int GPW, int NW>
static bool launch_talking_token(void* out, const void* q, long q_stride, const void* cache, long block_stride,
                                 const int* block_tables, int bt_stride, const int* qsl, const int* seq_lens, int S, int rows,
                                 int koff, int voff, int H, int G, int dk, int dv, float scale, int window, int keep,
                                 const float* sink, const float* talk, float* part, int nsplit, hipStream_t st) {
  const size_t shm = (static_cast<size_t>(H) * 16 + ((H * H + 3) & ~3)) * sizeof(float) +
                     static_cast<size_t>(NW) * 16 * (dv + 8) * sizeof(bf16_t);
  if (shm > 160 * 1024) return false;
  if (shm > 48 * 1024) {
    static bool raised = false;
    if (!raised) {
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(&talking_attention_token_kernel<KSM, VTM, GPW, NW>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess) {
        (void)hipGetLastError();
        return false;
      }
      raised = true;
    }
  }
  hipLaunchKernelGGL((talking_attention_token_kernel<KSM, VTM, GPW, NW>), dim3(rows, nsplit), dim3(64 * NW), shm, st,
                     (bf16_t*)out, (const bf16_t*)q, q_stride, (const bf16_t*)cache, block_stride, block_tables, bt_stride,
                     qsl, seq_lens, S, koff, voff, H, G, dk, dv, scale, window, keep, sink, talk, part, nsplit);
  MXS_CHECK_LAUNCH();
  return true;
}

bool launch_talking_attention(void* out, const void* q, long q_stride, const void* cache, long block_stride,
                              const int* block_tables, int bt_stride, const int* qsl, const int* seq_lens, int S, int rows,
                              int koff, int voff, int H, int G, int dk, int dv, int bs, float scale, int window, int keep,
                              int max_q, const float* sink, const float* talk, float* part, int nsplit, bool bf,
                              hipStream_t st) {
  if (rows == 0 || S == 0) return true;
  if (nsplit < 1 || (nsplit > 1 && (part == nullptr || reinterpret_cast<uintptr_t>(part) % 16))) return false;
  // bf16 with MFMA-shaped heads: the matrix-core form for prompt chunks and single tokens alike (a single
  // token is a 1-row tile; steps of few rows split every row's keys over nsplit workgroups)
  if (bf && max_q >= 1 && bs == 16 && dk % 16 == 0 && dv % 16 == 0 && dk <= 128 && dv <= 128 && q_stride % 4 == 0 &&
      reinterpret_cast<uintptr_t>(q) % 8 == 0 && koff % 8 == 0 && voff % 8 == 0 && block_stride % 8 == 0 && H <= 64) {
    const bool small = dk <= 64 && dv <= 64;
    bool done = false;
    if (max_q == 1 && H / G <= 16) {  // single tokens only: a tile's columns are the query heads of a kv head
#define MIX_TT(KSM, VTM, GPW, NW)                                                                                       \
  launch_talking_token<KSM, VTM, GPW, NW>(out, q, q_stride, cache, block_stride, block_tables, bt_stride, qsl, seq_lens, S, \
                                          rows, koff, voff, H, G, dk, dv, scale, window, keep, sink, talk, part, nsplit, st)
#define MIX_TT_N(GPW, NW) (small ? MIX_TT(4, 4, GPW, NW) : MIX_TT(8, 8, GPW, NW))
      if (G <= 1) done = MIX_TT_N(1, 1);
      else if (G <= 2) done = MIX_TT_N(1, 2);
      else if (G <= 4) done = MIX_TT_N(1, 4);
      else if (G <= 8) done = MIX_TT_N(1, 8);
      else if (G <= 16) done = MIX_TT_N(1, 16);
      else if (G <= 32) done = MIX_TT_N(2, 16);
      else done = small ? MIX_TT(4, 4, 4, 16) : false;
#undef MIX_TT_N
#undef MIX_TT
      if (done) return nsplit == 1 || launch_attention_combine(out, part, static_cast<long>(rows) * H, nsplit, dv, st);
    }
#define MIX_TA(KSM, VTM, HPW, NW)                                                                                       \
  launch_talking_mfma<KSM, VTM, HPW, NW>(out, q, q_stride, cache, block_stride, block_tables, bt_stride, qsl, seq_lens, S, \
                                         koff, voff, H, G, dk, dv, scale, window, keep, max_q, sink, talk, part, nsplit, st)
    if (H <= 4) done = small ? MIX_TA(4, 4, 1, 4) : MIX_TA(8, 8, 1, 4);
    else if (H <= 8) done = small ? MIX_TA(4, 4, 1, 8) : MIX_TA(8, 8, 1, 8);
    else if (H <= 16) done = small ? MIX_TA(4, 4, 1, 16) : MIX_TA(8, 8, 1, 16);
    else if (H <= 32) done = small ? MIX_TA(4, 4, 2, 16) : MIX_TA(8, 8, 2, 16);
    else done = small ? MIX_TA(4, 4, 4, 16) : false;
#undef MIX_TA
    if (done) return nsplit == 1 || launch_attention_combine(out, part, static_cast<long>(rows) * H, nsplit, dv, st);
  }
  // the rows form walks a row's keys in one workgroup, whatever split was asked for
  const int dkp = (dk + 3) & ~3;
  const size_t shm = (static_cast<size_t>(H) * dkp + static_cast<size_t>(H) * H + 2 * static_cast<size_t>(H) * kTalkTile +
                      3 * static_cast<size_t>(H)) * sizeof(float);
  if (shm > 160 * 1024 || H * dv > 256 * 32) return false;
  const int el = bf ? 8 : 4;
  const bool vec = dk % el == 0 && koff % el == 0 && block_stride % el == 0;
  // many wide heads need more than the default dynamic LDS of a workgroup: asked for once per kernel
#define MIX_TR(TT, NACC)                                                                                              \
  do {                                                                                                                \
    if (shm > 48 * 1024) {                                                                                            \
      static bool raised = false;                                                                                     \
      if (!raised) {                                                                                                  \
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(&talking_attention_rows_kernel<TT, NACC>),              \
                                hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess) {              \
          (void)hipGetLastError();                                                                                    \
          return false;                                                                                               \
        }                                                                                                             \
        raised = true;                                                                                                \
      }                                                                                                               \
    }                                                                                                                 \
    hipLaunchKernelGGL((talking_attention_rows_kernel<TT, NACC>), dim3(rows), dim3(256), shm, st, (TT*)out, (const TT*)q, \
                       q_stride, (const TT*)cache, block_stride, block_tables, bt_stride, qsl, seq_lens, S, koff, voff, H, \
                       G, dk, dv, bs, scale, window, keep, vec, sink, talk);                                           \
  } while (0)
#define MIX_TR_T(TT)                                \
  do {                                              \
    if (H * dv <= 256 * 2) MIX_TR(TT, 2);           \
    else if (H * dv <= 256 * 8) MIX_TR(TT, 8);      \
    else if (H * dv <= 256 * 16) MIX_TR(TT, 16);    \
    else MIX_TR(TT, 32);                            \
  } while (0)
  if (bf) MIX_TR_T(bf16_t);
  else MIX_TR_T(float);
#undef MIX_TR_T
#undef MIX_TR
  MXS_CHECK_LAUNCH();
  return true;
}

}  // namespace mxs
