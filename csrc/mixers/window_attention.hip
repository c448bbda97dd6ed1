// Softmax attention over the paged cache with a sliding window and kept first tokens (gfx950),
// for prompt chunks and single decoded tokens alike: one workgroup per (query row, query head).
// The query at position i sees key j <= i when i - j < window or j < keep (window <= 0: all j <= i).
// Visible keys are walked in tiles of 256: one key per thread for the scores (fp32 dot of the LDS
// query with the key's cache row), a block-wide running maximum and sum (online softmax), then each
// wave takes every fourth key of the tile with its lanes across the value row.  Scores, weights and
// the output sum are fp32; q, K and V are bf16 or fp32.
// A sink (fp32 [H], optional) is one more key per head with the score sink[h], not scaled, and no
// value: the running maximum starts at it and the running sum at 1 instead of -inf and 0.
#include "mix_common.h"

namespace mxs {

constexpr int kKeyTile = 256;
constexpr int kMaxVChunks = 8;  // value size <= 64 * 8

template <typename T>
__global__ void __launch_bounds__(256) window_attention_kernel(
    T* __restrict__ out, const T* __restrict__ q, long q_stride, const T* __restrict__ cache, long block_stride,
    const int* __restrict__ block_tables, int bt_stride, const int* __restrict__ qsl, const int* __restrict__ seq_lens,
    int S, int koff, int voff, int H, int G, int dk, int dv, int bs, float scale, int window, int keep, bool vec,
    const float* __restrict__ sink, int vs) {
  extern __shared__ float lds[];
  float* qs = lds;                      // [dk]
  float* p = qs + ((dk + 3) & ~3);      // [kKeyTile]
  float* red = p + kKeyTile;            // [4][dv]
  __shared__ float scratch[16];
  const int t = blockIdx.x, hd = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wid = tid >> 6;
  const int s = seq_of_row(qsl, S, t);
  const int qlen = qsl[s + 1] - qsl[s];
  // the row's position, kept inside the block table whatever the metadata says
  const int pos = min(max(seq_lens[s] - qlen + (t - qsl[s]), 0), bt_stride * bs - 1);
  const int g = hd / (H / G);
  const int lo = window > 0 ? max(pos - window + 1, 0) : 0;
  const int nA = window > 0 ? min(keep, lo) : 0;  // kept first tokens that lie below the window
  const int nvis = nA + (pos - lo + 1);
  const int* bt = block_tables + static_cast<long>(s) * bt_stride;
  for (int d = tid; d < dk; d += blockDim.x) qs[d] = ldf(q + static_cast<long>(t) * q_stride + hd * dk + d) * scale;
  float m = sink ? sink[hd] : -INFINITY, l = sink ? 1.f : 0.f;
  float acc[kMaxVChunks];
#pragma unroll
  for (int c = 0; c < kMaxVChunks; ++c) acc[c] = 0.f;
  const int nchunk = (dv + 63) >> 6;
  __syncthreads();
  for (int t0 = 0; t0 < nvis; t0 += kKeyTile) {
    const int nt = min(kKeyTile, nvis - t0);
    float sc = -INFINITY;
    if (tid < nt) {
      const int n = t0 + tid;
      const int j = n < nA ? n : lo + (n - nA);
      const T* kp = cache + static_cast<long>(bt[j / bs]) * block_stride + koff + (static_cast<long>(g) * bs + j % bs) * dk;
      sc = dot_row<T>(qs, kp, dk, vec);
    }
    const float m_new = fmaxf(m, block_max(sc, scratch));
    const float e = tid < nt ? expf(sc - m_new) : 0.f;
    p[tid] = e;
    const float tsum = block_sum(e, scratch);  // its barriers also publish p
    const float corr = expf(m - m_new);        // first tile: exp(-inf) = 0, acc and l are 0
    l = l * corr + tsum;
    m = m_new;
#pragma unroll
    for (int c = 0; c < kMaxVChunks; ++c) acc[c] *= corr;
    for (int n = wid; n < nt; n += 4) {
      const int nn = t0 + n;
      const int j = nn < nA ? nn : lo + (nn - nA);
      const T* vp = cache + static_cast<long>(bt[j / bs]) * block_stride + voff + (static_cast<long>(g) * bs + j % bs) * vs;
      const float pn = p[n];
#pragma unroll
      for (int c = 0; c < kMaxVChunks; ++c) {
        const int e2 = lane + 64 * c;
        if (c < nchunk && e2 < dv) acc[c] += pn * ldf(vp + e2);
      }
    }
    __syncthreads();  // p is rewritten by the next tile
  }
#pragma unroll
  for (int c = 0; c < kMaxVChunks; ++c) {
    const int e2 = lane + 64 * c;
    if (c < nchunk && e2 < dv) red[wid * dv + e2] = acc[c];
  }
  __syncthreads();
  const float inv = 1.f / l;
  for (int e2 = tid; e2 < dv; e2 += blockDim.x) {
    const float o = red[e2] + red[dv + e2] + red[2 * dv + e2] + red[3 * dv + e2];
    stf(out + static_cast<long>(t) * (H * dv) + hd * dv + e2, o * inv);
  }
}


// ---- Row form with 16-byte loads (single decoded tokens, short chunks): head sizes that are
// multiples of 16 bytes.  Eight lanes share a key: each loads 16 bytes of every 128-byte stretch of
// the key's row, so a wave's load instruction covers eight whole rows instead of 64 two-byte (or 64
// scattered 16-byte) pieces; the score is summed over the eight lanes.  The value rows are read the
// same way with the weight of their key, and the 32 key slots of the block are summed at the end
// (three lane exchanges, then the four waves through LDS).
// NC: 128-byte stretches of a row (head sizes <= NC * 8 * El<T>::N).  RM: query heads of one kv head that
// a workgroup serves together: a key or value row is loaded once and used for all of them.
template <typename T, int NC, int RM>
__global__ void __launch_bounds__(256) window_attention_rows_kernel(
    T* __restrict__ out, const T* __restrict__ q, long q_stride, const T* __restrict__ cache, long block_stride,
    const int* __restrict__ block_tables, int bt_stride, const int* __restrict__ qsl, const int* __restrict__ seq_lens,
    int S, int koff, int voff, int H, int G, int dk, int dv, int bs, float scale, int window, int keep, int nsplit,
    const float* __restrict__ sink, int vs) {
  constexpr int EL = El<T>::N;
  extern __shared__ float lds[];
  float* p = lds;                      // [RM][kKeyTile]
  float* red = p + RM * kKeyTile;      // [4][RM][dv]
  __shared__ float scratch[RM * 4];
  const int t = blockIdx.x;
  const int g = blockIdx.y / nsplit, hs = blockIdx.y - g * nsplit;
  const int R = H / G;
  const int h0 = g * R + hs * RM;      // first query head of this workgroup
  const int nr = min(RM, R - hs * RM);
  const int tid = threadIdx.x, lane = tid & 63, wid = tid >> 6;
  const int part = tid & 7, slot = tid >> 3;  // the lane's 16 bytes of each stretch; its key slot (0..31)
  const int s = seq_of_row(qsl, S, t);
  const int qlen = qsl[s + 1] - qsl[s];
  const int pos = min(max(seq_lens[s] - qlen + (t - qsl[s]), 0), bt_stride * bs - 1);
  const int lo = window > 0 ? max(pos - window + 1, 0) : 0;
  const int nA = window > 0 ? min(keep, lo) : 0;
  const int nvis = nA + (pos - lo + 1);
  const int* bt = block_tables + static_cast<long>(s) * bt_stride;
  float qf[RM][NC][EL], acc[RM][NC][EL], m[RM], l[RM];
#pragma unroll
  for (int r = 0; r < RM; ++r) {
    m[r] = (sink && r < nr) ? sink[h0 + r] : -INFINITY;
    l[r] = (sink && r < nr) ? 1.f : 0.f;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int d = (c * 8 + part) * EL;
#pragma unroll
      for (int e = 0; e < EL; ++e) {
        qf[r][c][e] = (r < nr && d + e < dk) ? ldf(q + static_cast<long>(t) * q_stride + (h0 + r) * dk + d + e) * scale : 0.f;
        acc[r][c][e] = 0.f;
      }
    }
  }
  for (int t0 = 0; t0 < nvis; t0 += kKeyTile) {
    const int nt = min(kKeyTile, nvis - t0);
    for (int n = slot; n < nt; n += 32) {
      const int nn = t0 + n;
      const int j = nn < nA ? nn : lo + (nn - nA);
      const T* kp = cache + static_cast<long>(bt[j / bs]) * block_stride + koff + (static_cast<long>(g) * bs + j % bs) * dk;
      float sc[RM];
#pragma unroll
      for (int r = 0; r < RM; ++r) sc[r] = 0.f;
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const int d = (c * 8 + part) * EL;
        if (d < dk) {
          float kf[EL];
          load16(kp + d, kf);
#pragma unroll
          for (int r = 0; r < RM; ++r)
#pragma unroll
            for (int e = 0; e < EL; ++e) sc[r] += qf[r][c][e] * kf[e];
        }
      }
#pragma unroll
      for (int r = 0; r < RM; ++r) {
        float v = sc[r];
        v += __shfl_xor(v, 1, 64);
        v += __shfl_xor(v, 2, 64);
        v += __shfl_xor(v, 4, 64);
        if (part == 0) p[r * kKeyTile + n] = v;
      }
    }
    __syncthreads();
    float sv[RM], ev[RM], m_new[RM];
#pragma unroll
    for (int r = 0; r < RM; ++r) {
      sv[r] = tid < nt ? p[r * kKeyTile + tid] : -INFINITY;
      const float wm = wave_max(sv[r]);
      if (lane == 0) scratch[r * 4 + wid] = wm;
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < RM; ++r) {
      const float mx = fmaxf(fmaxf(scratch[r * 4], scratch[r * 4 + 1]), fmaxf(scratch[r * 4 + 2], scratch[r * 4 + 3]));
      m_new[r] = fmaxf(m[r], mx);
      ev[r] = tid < nt ? expf(sv[r] - m_new[r]) : 0.f;
    }
    __syncthreads();  // every score and maximum is read before it is replaced
#pragma unroll
    for (int r = 0; r < RM; ++r) {
      p[r * kKeyTile + tid] = ev[r];
      const float ws = wave_sum(ev[r]);
      if (lane == 0) scratch[r * 4 + wid] = ws;
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < RM; ++r) {
      const float tsum = (scratch[r * 4] + scratch[r * 4 + 1]) + (scratch[r * 4 + 2] + scratch[r * 4 + 3]);
      const float corr = expf(m[r] - m_new[r]);  // first tile: exp(-inf) = 0, acc and l are 0
      l[r] = l[r] * corr + tsum;
      m[r] = m_new[r];
#pragma unroll
      for (int c = 0; c < NC; ++c)
#pragma unroll
        for (int e2 = 0; e2 < EL; ++e2) acc[r][c][e2] *= corr;
    }
    for (int n = slot; n < nt; n += 32) {
      const int nn = t0 + n;
      const int j = nn < nA ? nn : lo + (nn - nA);
      const T* vp = cache + static_cast<long>(bt[j / bs]) * block_stride + voff + (static_cast<long>(g) * bs + j % bs) * vs;
      float pn[RM];
#pragma unroll
      for (int r = 0; r < RM; ++r) pn[r] = p[r * kKeyTile + n];
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const int d = (c * 8 + part) * EL;
        if (d < dv) {
          float vf[EL];
          load16(vp + d, vf);
#pragma unroll
          for (int r = 0; r < RM; ++r)
#pragma unroll
            for (int e2 = 0; e2 < EL; ++e2) acc[r][c][e2] += pn[r] * vf[e2];
        }
      }
    }
    __syncthreads();  // p and scratch are rewritten by the next tile
  }
  // the 8 key slots of a wave that share `part`, then the 4 waves
#pragma unroll
  for (int r = 0; r < RM; ++r) {
#pragma unroll
    for (int c = 0; c < NC; ++c) {
#pragma unroll
      for (int e2 = 0; e2 < EL; ++e2) {
        float v = acc[r][c][e2];
        v += __shfl_xor(v, 8, 64);
        v += __shfl_xor(v, 16, 64);
        v += __shfl_xor(v, 32, 64);
        const int d = (c * 8 + part) * EL + e2;
        if (lane < 8 && d < dv) red[(wid * RM + r) * dv + d] = v;
      }
    }
    if (tid == 0) scratch[r] = 1.f / l[r];
  }
  __syncthreads();
  for (int idx = tid; idx < nr * dv; idx += blockDim.x) {
    const int r = idx / dv, e2 = idx - r * dv;
    const float o = (red[r * dv + e2] + red[(RM + r) * dv + e2]) + (red[(2 * RM + r) * dv + e2] + red[(3 * RM + r) * dv + e2]);
    stf(out + static_cast<long>(t) * (H * dv) + (h0 + r) * dv + e2, o * scratch[r]);
  }
}

// ---- MFMA form for prompt chunks (bf16, 16-token cache blocks, head sizes multiples of 16 up to
// 16 * KSM / 16 * VTM).  A wave owns 16 consecutive query rows of one head and walks the visible
// cache blocks (the kept first blocks, then the window's); no workgroup barriers.  Per block, with
// v_mfma_f32_16x16x16_bf16:
//   S^T = K Q^T      A = the block's 16 key rows (8-byte loads from the token-major cache),
//                    B = Q^T, held in registers for the whole walk.  The accumulator has the query
//                    on the lane (column) and 4 keys per lane, so a row's max and sum are per-lane
//                    work plus two cross-lane exchanges.
//   O^T += V^T P^T   B = P^T straight from the S^T accumulator's registers; every weight is split
//                    into two bf16 halves (p = hi + lo, two MFMAs) so the product keeps 16 mantissa
//                    bits of the fp32 weight; A = V^T: the block's token-major value rows go through
//                    the wave's LDS area (16-byte pieces in, 2-byte reads out, key-contiguous).
// Scores, maxima, sums and the output accumulator are fp32.
typedef short s4_t __attribute__((ext_vector_type(4)));
typedef float f4_t __attribute__((ext_vector_type(4)));

template <int KSM, int VTM>
__global__ void __launch_bounds__(256) window_attention_mfma_kernel(
    bf16_t* __restrict__ out, const bf16_t* __restrict__ q, long q_stride, const bf16_t* __restrict__ cache,
    long block_stride, const int* __restrict__ block_tables, int bt_stride, const int* __restrict__ qsl,
    const int* __restrict__ seq_lens, int koff, int voff, int H, int G, int dk, int dv, float scale, int window,
    int keep, const float* __restrict__ sink) {
  // each wave's own staging area for a block's value rows (token-major in the pages): written with
  // 16-byte pieces, read back as the key-contiguous V^T operand.  Rows are padded by 8 elements so
  // that the four key groups of a read fall into different banks.
  __shared__ __attribute__((aligned(16))) bf16_t vlds[4][16 * (16 * VTM + 8)];
  const int s = blockIdx.z, hd = blockIdx.y;
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  bf16_t* vw = vlds[wid];
  const int DVP = dv + 8;
  const int row0 = qsl[s], qlen = qsl[s + 1] - row0;
  const int qt0 = blockIdx.x * 64 + wid * 16;  // this wave's first query row inside the chunk
  if (qt0 >= qlen) return;                     // wave-uniform (no workgroup barrier is used below)
  const int nq = min(16, qlen - qt0);
  // the tile's first position; its last row stays inside the block table whatever the metadata says
  const int pos0 = min(max(seq_lens[s] - qlen + qt0, 0), bt_stride * 16 - nq);
  const int g = hd / (H / G);
  const int c = lane & 15, kg = lane >> 4;  // the lane's query (column) and its group of 4 keys / dims
  const int KS = dk >> 4, VT = dv >> 4;
  const bool qok = c < nq;
  const int pq = pos0 + c;
  const int* bt = block_tables + static_cast<long>(s) * bt_stride;
  s4_t qf[KSM];
  {
    const bf16_t* qp = q + static_cast<long>(row0 + qt0 + (qok ? c : 0)) * q_stride + hd * dk + 4 * kg;
#pragma unroll
    for (int ks = 0; ks < KSM; ++ks)
      qf[ks] = (ks < KS && qok) ? *reinterpret_cast<const s4_t*>(qp + 16 * ks) : s4_t{0, 0, 0, 0};
  }
  const int p_last = pos0 + nq - 1;
  const int lo_first = window > 0 ? max(pos0 - window + 1, 0) : 0;
  const int wb = lo_first >> 4, lastb = p_last >> 4;
  const int kA = window > 0 ? min((keep + 15) >> 4, wb) : 0;  // kept first blocks below the window's
  // m in log2 units: scores are scaled by scale * log2(e), weights are exp2.  l is a lane's share of the
  // row's sum (its key group's), added up at the end: the sink's 1 goes to the first group.
  float m = sink ? sink[hd] * 1.4426950408889634f : -INFINITY, l = (sink && kg == 0) ? 1.f : 0.f;
  f4_t o[VTM];
#pragma unroll
  for (int vt = 0; vt < VTM; ++vt) o[vt] = f4_t{0.f, 0.f, 0.f, 0.f};
  const float sl2 = scale * 1.4426950408889634f;
  const int nit = kA + (lastb - wb + 1);
  for (int it = 0; it < nit; ++it) {
    const int kb = it < kA ? it : wb + (it - kA);
    const bf16_t* blk = cache + static_cast<long>(bt[kb]) * block_stride;
    f4_t acc = f4_t{0.f, 0.f, 0.f, 0.f};
    const bf16_t* kp = blk + koff + (static_cast<long>(g) * 16 + c) * dk + 4 * kg;
#pragma unroll
    for (int ks = 0; ks < KSM; ++ks)
      if (ks < KS)
        acc = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(*reinterpret_cast<const s4_t*>(kp + 16 * ks), qf[ks], acc, 0, 0, 0);
    // a block that every query of the tile sees whole (the usual case inside a window) needs no mask
    const int k0 = kb * 16;
    const bool whole = k0 + 15 <= pos0 && (window <= 0 || k0 >= p_last - window + 1 || k0 + 15 < keep);
    float sv[4], mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (whole) {
        sv[i] = acc[i] * sl2;
      } else {
        const int j = k0 + 4 * kg + i;
        const bool vis = qok && j <= pq && (window <= 0 || pq - j < window || j < keep);
        sv[i] = vis ? acc[i] * sl2 : -INFINITY;
      }
      mx = fmaxf(mx, sv[i]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m, mx);
    // the running maximum seldom moves after the first blocks: rescale only when some query's did
    if (__builtin_amdgcn_ballot_w64(m_new > m) != 0) {
      const float corr = m_new == -INFINITY ? 1.f : __builtin_amdgcn_exp2f(m - m_new);
      l *= corr;
#pragma unroll
      for (int vt = 0; vt < VTM; ++vt)
#pragma unroll
        for (int i = 0; i < 4; ++i) o[vt][i] *= corr;
      m = m_new;
    }
    s4_t ph, pl;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      // exp2(-inf) = 0; a query with nothing visible yet (m = -inf) must not turn -inf - -inf into a weight
      const float pr = (whole || sv[i] != -INFINITY) ? __builtin_amdgcn_exp2f(sv[i] - m) : 0.f;
      l += pr;
      // pr = hi + lo: hi the upper 16 bits (exact), lo = pr - hi rounded to bf16 (pr >= 0, finite)
      const uint32_t u = __float_as_uint(pr), uh = u & 0xFFFF0000u;
      uint32_t ul = __float_as_uint(pr - __uint_as_float(uh));
      ul += 0x7FFFu + ((ul >> 16) & 1u);
      ph[i] = static_cast<short>(uh >> 16);
      pl[i] = static_cast<short>(ul >> 16);
    }
    // the block's 16 value rows are one contiguous stretch of 16 * dv elements
    const bf16_t* vblk = blk + voff + static_cast<long>(g) * 16 * dv;
    __builtin_amdgcn_wave_barrier();  // the previous block's reads come first
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
    const bool vall = k0 + 15 <= p_last;
#pragma unroll
    for (int vt = 0; vt < VTM; ++vt) {
      if (vt < VT) {
        s4_t a;
#pragma unroll
        for (int j = 0; j < 4; ++j)  // rows past the sequence's last token may hold anything: read them as 0
          a[j] = (vall || k0 + 4 * kg + j <= p_last) ? static_cast<short>(vp[j * DVP + 16 * vt]) : short(0);
        const f4_t t = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, ph, o[vt], 0, 0, 0);
        o[vt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, pl, t, 0, 0, 0);
      }
    }
  }
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);
  if (!qok) return;
  const float inv = 1.f / l;
  bf16_t* op = out + static_cast<long>(row0 + qt0 + c) * (H * dv) + hd * dv + 4 * kg;
#pragma unroll
  for (int vt = 0; vt < VTM; ++vt) {
    if (vt < VT) {
      uint2 w;
      w.x = pack2(o[vt][0] * inv, o[vt][1] * inv);
      w.y = pack2(o[vt][2] * inv, o[vt][3] * inv);
      *reinterpret_cast<uint2*>(op + 16 * vt) = w;
    }
  }
}

bool launch_window_attention(void* out, const void* q, long q_stride, const void* cache, long block_stride,
                             const int* block_tables, int bt_stride, const int* qsl, const int* seq_lens, int S,
                             int rows, int koff, int voff, int H, int G, int dk, int dv, int bs, float scale,
                             int window, int keep, int max_q, const float* sink, int vs, bool bf, hipStream_t st) {
  if (rows == 0 || S == 0) return true;
  if (vs <= 0) vs = dv;  // value rows back to back
  // prompt chunks in bf16 with MFMA-shaped heads: the matrix-core form (rows of a mixed step's single
  // tokens ride along as 1-row tiles); everything else the scalar form below
  if (bf && vs == dv && max_q >= 16 && bs == 16 && dk % 16 == 0 && dv % 16 == 0 && dk <= 128 && dv <= 128 && q_stride % 4 == 0 &&
      reinterpret_cast<uintptr_t>(q) % 8 == 0 && koff % 8 == 0 && voff % 8 == 0 && block_stride % 8 == 0) {
    const dim3 grid((max_q + 63) / 64, H, S);
#define MIX_WA(KSM, VTM)                                                                                              \
  hipLaunchKernelGGL((window_attention_mfma_kernel<KSM, VTM>), grid, dim3(256), 0, st, (bf16_t*)out, (const bf16_t*)q, \
                     q_stride, (const bf16_t*)cache, block_stride, block_tables, bt_stride, qsl, seq_lens, koff, voff, \
                     H, G, dk, dv, scale, window, keep, sink)
    if (dk <= 64 && dv <= 64) MIX_WA(4, 4);
    else MIX_WA(8, 8);
#undef MIX_WA
    MXS_CHECK_LAUNCH();
    return true;
  }
  if (dv > 64 * kMaxVChunks) return false;
  const int el = bf ? 8 : 4;  // elements per 16-byte load
  const bool vec = dk % el == 0 && koff % el == 0 && block_stride % el == 0;
  const size_t shm = (((dk + 3) & ~3) + kKeyTile + 4 * dv) * sizeof(float);
  if (shm > 60 * 1024) return false;
  if (vec && dv % el == 0 && voff % el == 0 && vs % el == 0 && dk <= 256 && dv <= 256) {  // rows of whole 16-byte pieces
    const int stretch = 8 * el, need = (std::max(dk, dv) + stretch - 1) / stretch;  // 128-byte stretches of a row
    const int R = H / G;
#define MIX_ROWS(TT, NC, RM)                                                                                          \
  do {                                                                                                                \
    const int nsplit = (R + RM - 1) / RM;                                                                             \
    const size_t sh = (static_cast<size_t>(RM) * kKeyTile + 4 * RM * dv) * sizeof(float);                             \
    hipLaunchKernelGGL((window_attention_rows_kernel<TT, NC, RM>), dim3(rows, G * nsplit), dim3(256), sh, st, (TT*)out, \
                       (const TT*)q, q_stride, (const TT*)cache, block_stride, block_tables, bt_stride, qsl, seq_lens, \
                       S, koff, voff, H, G, dk, dv, bs, scale, window, keep, nsplit, sink, vs);                        \
  } while (0)
#define MIX_ROWS_T(TT)                                          \
  do {                                                          \
    if (need <= 1) { if (R > 1) MIX_ROWS(TT, 1, 8); else MIX_ROWS(TT, 1, 1); } \
    else if (need <= 2) { if (R > 1) MIX_ROWS(TT, 2, 4); else MIX_ROWS(TT, 2, 1); } \
    else if (need <= 4) { if (R > 1) MIX_ROWS(TT, 4, 2); else MIX_ROWS(TT, 4, 1); } \
    else MIX_ROWS(TT, 8, 1);                                    \
  } while (0)
    if (bf) MIX_ROWS_T(bf16_t);
    else MIX_ROWS_T(float);
#undef MIX_ROWS_T
#undef MIX_ROWS
    MXS_CHECK_LAUNCH();
    return true;
  }
  if (bf)
    hipLaunchKernelGGL(window_attention_kernel<bf16_t>, dim3(rows, H), dim3(256), shm, st, (bf16_t*)out, (const bf16_t*)q,
                       q_stride, (const bf16_t*)cache, block_stride, block_tables, bt_stride, qsl, seq_lens, S, koff,
                       voff, H, G, dk, dv, bs, scale, window, keep, vec, sink, vs);
  else
    hipLaunchKernelGGL(window_attention_kernel<float>, dim3(rows, H), dim3(256), shm, st, (float*)out, (const float*)q,
                       q_stride, (const float*)cache, block_stride, block_tables, bt_stride, qsl, seq_lens, S, koff,
                       voff, H, G, dk, dv, bs, scale, window, keep, vec, sink, vs);
  MXS_CHECK_LAUNCH();
  return true;
}

}  // namespace mxs
