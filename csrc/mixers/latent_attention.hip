// Latent attention on the matrix cores (gfx950, bf16): every query head attends over the same
// cached rows [latent (rank) | rotated key part], dk entries a row, and the values are the rows'
// first `rank` entries.  Prompt chunks and single decoded tokens run the same kernel.
//
// The rows of a sequence's step are its (token, head) pairs, flattened; a wave owns 16 consecutive
// rows and walks the 16-key cache blocks that its rows see (causal; with window > 0 only the last
// `window` positions of each row), or one of `nsplit` stretches of them.  No workgroup barriers: the four waves of a workgroup are independent.  Per block, with
// v_mfma_f32_16x16x32_bf16 (scores) and v_mfma_f32_16x16x16_bf16 (values):
//   S^T = K Q^T      A = the block's 16 key rows, loaded from the pages as 16-byte pieces that are
//                    used as they are: lane (key c, group kg) holds entries 32 kk + 8 kg .. + 7 of its
//                    key, one piece feeds one 32-deep MFMA, and Q^T (held in registers for
//                    the whole walk) is loaded in the same order, so the products pair up.  The accumulator has the row on the lane
//                    and 4 keys per lane: maxima and sums are per-lane work plus two lane exchanges.
//   O^T += V^T P^T   B = P^T straight from the S^T accumulator's registers, every weight split into
//                    two bf16 halves (p = hi + lo, two MFMAs) so that the product keeps 16 mantissa
//                    bits of the fp32 weight.  A = V^T: the same registers that held the key pieces
//                    are written into the wave's LDS area transposed ([entry][key], 2-byte stores)
//                    and read back key-contiguous with one 8-byte load per tile.
// The next block's pieces are loaded while the values are multiplied.  Scores (log2 units), maxima,
// sums and the output accumulator are fp32.  A sink (fp32 [H], optional) starts the running maximum at
// sink[h] and the running sum at 1.  With nsplit > 1 a wave writes its stretch's (maximum, sum,
// unnormalised output) and latent_attention_combine merges the stretches of a row.
#include "mix_common.h"

namespace mxs {

typedef short s4_t __attribute__((ext_vector_type(4)));
typedef float f4_t __attribute__((ext_vector_type(4)));
typedef __bf16 bf8_t __attribute__((ext_vector_type(8)));
// one v_mfma_f32_16x16x32_bf16 per 16-byte piece: lane (c, kg) holds the 8 summed indices 8 kg .. 8 kg + 7
__device__ __forceinline__ f4_t mfma_piece(const uint4& a, const uint4& b, f4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf8_t, a), __builtin_bit_cast(bf8_t, b), c, 0, 0, 0);
}

constexpr int kVtPitch = 20;  // bf16 per transposed row: 16 keys + 4, so that the four key groups fall into different banks

constexpr int kPartHead = 4;  // floats ahead of a stretch's output: maximum, sum, two unused (16-byte rows)

// KKM: 32-entry chunks of a row (dk <= 32 KKM); VTM: 16-entry value tiles (rank <= 16 VTM); NW: waves of
// a workgroup (its LDS is NW transposed value blocks); QLDS: the query pieces wait in LDS, each lane's
// own 16 bytes per chunk side by side, instead of in registers (the widest rows: the output
// accumulator and a block's key pieces already take 200 registers)
// EXACT: dk = 32 KKM and rank = 16 VTM, so no piece or tile needs a bounds test
template <int KKM, int VTM, int NW, bool QLDS, bool EXACT>
__global__ void __launch_bounds__(64 * NW) latent_attention_mfma_kernel(
    bf16_t* __restrict__ out, float* __restrict__ part, const bf16_t* __restrict__ q, long q_stride,
    const bf16_t* __restrict__ cache, long block_stride, const int* __restrict__ block_tables, int bt_stride,
    const int* __restrict__ qsl, const int* __restrict__ seq_lens, int koff, int H, int dk, int rank, float scale,
    const float* __restrict__ sink, int nsplit, int window) {
  extern __shared__ __attribute__((aligned(16))) bf16_t vt_lds[];  // [NW waves][16 VTM entries][kVtPitch] (+ [NW][KKM][64] x 16 B)
  const int s = blockIdx.z;
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  bf16_t* vt_w = vt_lds + wid * (16 * VTM * kVtPitch);
  uint4* q_l = reinterpret_cast<uint4*>(vt_lds + NW * (16 * VTM * kVtPitch)) + wid * (KKM * 64) + lane;
  const int row0 = qsl[s], qlen = qsl[s + 1] - row0;
  const int nrows = qlen * H;
  const int id = blockIdx.x * NW + wid;
  const int tile = id / nsplit, sp = id - tile * nsplit;
  if (tile * 16 >= nrows) return;  // wave-uniform (no workgroup barrier is used below)
  const int c = lane & 15, kg = lane >> 4;
  const int r = tile * 16 + c;
  const bool rok = r < nrows;
  const int rr = rok ? r : nrows - 1;
  const int tok = rr / H, hd = rr - tok * H;
  // positions, kept inside the block table whatever the metadata says
  const int last = bt_stride * 16 - 1;
  const int base = max(seq_lens[s] - qlen, 0);
  const int pq = min(base + tok, last);
  const int p_first = min(base + (tile * 16) / H, last);
  const int p_last = min(base + min(tile * 16 + 15, nrows - 1) / H, last);
  // window > 0: a row at position p sees p - window + 1 .. p; the tile's walk starts at the block of
  // its first row's oldest visible key
  const int wb = window > 0 ? max(p_first - window + 1, 0) >> 4 : 0;
  const int nblk = (p_last >> 4) + 1 - wb;
  const int b0 = wb + static_cast<int>(static_cast<long>(nblk) * sp / nsplit);
  const int b1 = wb + static_cast<int>(static_cast<long>(nblk) * (sp + 1) / nsplit);
  const int KK = EXACT ? KKM : (dk + 31) >> 5, VT = EXACT ? VTM : rank >> 4;
  const int* bt = block_tables + static_cast<long>(s) * bt_stride;
  uint4 qf[QLDS ? 1 : KKM];
  {
    const bf16_t* qp = q + static_cast<long>(row0 + tok) * q_stride + static_cast<long>(hd) * dk + 8 * kg;
#pragma unroll
    for (int kk = 0; kk < KKM; ++kk) {
      const uint4 v = (rok && (EXACT || (kk < KK && 32 * kk + 8 * kg + 8 <= dk))) ? *reinterpret_cast<const uint4*>(qp + 32 * kk)
                                                                                  : make_uint4(0, 0, 0, 0);
      if (QLDS) q_l[kk * 64] = v;  // read back by this lane only
      else qf[kk] = v;
    }
  }
  const float L2E = 1.4426950408889634f;
  float m = (sink && sp == 0) ? sink[hd] * L2E : -INFINITY;
  float l = (sink && sp == 0 && kg == 0) ? 1.f : 0.f;  // a lane's share of its row's sum (its key group's)
  f4_t o[VTM];
#pragma unroll
  for (int vt = 0; vt < VTM; ++vt) o[vt] = f4_t{0.f, 0.f, 0.f, 0.f};
  const float sl2 = scale * L2E;
  uint4 kr[KKM];
  auto load_block = [&](int kb) {
    const bf16_t* kp = cache + static_cast<long>(bt[kb]) * block_stride + koff + static_cast<long>(c) * dk + 8 * kg;
#pragma unroll
    for (int kk = 0; kk < KKM; ++kk)
      kr[kk] = (EXACT || (kk < KK && 32 * kk + 8 * kg + 8 <= dk)) ? *reinterpret_cast<const uint4*>(kp + 32 * kk)
                                                                  : make_uint4(0, 0, 0, 0);
    // key rows past the tile's last position may hold anything (also NaN); no row of the tile sees
    // them, but as values they would be multiplied by their zero weights: read them as zeros.  Only a
    // tile's last block can have such rows.
    if (kb * 16 + 15 > p_last && kb * 16 + c > p_last) {
#pragma unroll
      for (int kk = 0; kk < KKM; ++kk) kr[kk] = make_uint4(0, 0, 0, 0);
    }
  };
  if (b0 < b1) load_block(b0);
  for (int kb = b0; kb < b1; ++kb) {
    const int k0 = kb * 16;
    __builtin_amdgcn_wave_barrier();  // the previous block's LDS reads come before this block's writes
    // four accumulators: consecutive MFMAs do not wait for one another
    f4_t ac[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) ac[i] = f4_t{0.f, 0.f, 0.f, 0.f};
    // the block's values go into the wave's LDS area transposed, piece by piece as the scores are summed
#pragma unroll
    for (int kk = 0; kk < KKM; ++kk) {
      if (EXACT || kk < KK) {
        const uint4 qv = QLDS ? q_l[kk * 64] : qf[QLDS ? 0 : kk];
        ac[kk & 3] = mfma_piece(kr[kk], qv, ac[kk & 3]);
        const int d0 = 32 * kk + 8 * kg;
        if (d0 < rank) {
          const uint4 a = kr[kk];
          bf16_t* w = vt_w + d0 * kVtPitch + c;
          w[0] = static_cast<bf16_t>(a.x & 0xFFFFu);
          w[kVtPitch] = static_cast<bf16_t>(a.x >> 16);
          w[2 * kVtPitch] = static_cast<bf16_t>(a.y & 0xFFFFu);
          w[3 * kVtPitch] = static_cast<bf16_t>(a.y >> 16);
          w[4 * kVtPitch] = static_cast<bf16_t>(a.z & 0xFFFFu);
          w[5 * kVtPitch] = static_cast<bf16_t>(a.z >> 16);
          w[6 * kVtPitch] = static_cast<bf16_t>(a.w & 0xFFFFu);
          w[7 * kVtPitch] = static_cast<bf16_t>(a.w >> 16);
        }
      }
    }
    const f4_t acc = (ac[0] + ac[1]) + (ac[2] + ac[3]);
    if (kb + 1 < b1) load_block(kb + 1);  // in flight while the weights are made and the values multiplied
    // a block that every row of the tile sees whole needs no mask
    const bool whole = k0 + 15 <= p_first && (window <= 0 || k0 >= p_last - window + 1);
    float sv[4], mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (whole) {
        sv[i] = acc[i] * sl2;
      } else {
        const int j = k0 + 4 * kg + i;
        sv[i] = (rok && j <= pq && (window <= 0 || pq - j < window)) ? acc[i] * sl2 : -INFINITY;
      }
      mx = fmaxf(mx, sv[i]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m, mx);
    if (__builtin_amdgcn_ballot_w64(m_new > m) != 0) {  // rescale only when some row's maximum moved
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
      // a row with nothing visible yet (m = -inf) must not turn -inf - -inf into a weight
      const float pr = (whole || sv[i] != -INFINITY) ? __builtin_amdgcn_exp2f(sv[i] - m) : 0.f;
      l += pr;
      // pr = hi + lo: hi the upper 16 bits (exact), lo = pr - hi rounded to bf16 (pr >= 0, finite)
      const uint32_t u = __float_as_uint(pr), uh = u & 0xFFFF0000u;
      uint32_t ul = __float_as_uint(pr - __uint_as_float(uh));
      ul += 0x7FFFu + ((ul >> 16) & 1u);
      ph[i] = static_cast<short>(uh >> 16);
      pl[i] = static_cast<short>(ul >> 16);
    }
    __builtin_amdgcn_wave_barrier();
    const bf16_t* vp = vt_w + c * kVtPitch + 4 * kg;
#pragma unroll
    for (int vt = 0; vt < VTM; ++vt) {
      if (EXACT || vt < VT) {
        const s4_t a = *reinterpret_cast<const s4_t*>(vp + 16 * vt * kVtPitch);
        const f4_t t = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, ph, o[vt], 0, 0, 0);
        o[vt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, pl, t, 0, 0, 0);
      }
    }
  }
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);
  if (!rok) return;
  const long grow = static_cast<long>(row0 + tok) * H + hd;  // the row among all (token, head) pairs of the step
  if (nsplit == 1) {
    const float inv = 1.f / l;
    bf16_t* op = out + grow * rank + 4 * kg;
#pragma unroll
    for (int vt = 0; vt < VTM; ++vt) {
      if (vt < VT) {
        uint2 w;
        w.x = pack2(o[vt][0] * inv, o[vt][1] * inv);
        w.y = pack2(o[vt][2] * inv, o[vt][3] * inv);
        *reinterpret_cast<uint2*>(op + 16 * vt) = w;
      }
    }
  } else {
    float* pp = part + (grow * nsplit + sp) * (rank + kPartHead);
    if (kg == 0) { pp[0] = m; pp[1] = l; }
#pragma unroll
    for (int vt = 0; vt < VTM; ++vt)
      if (vt < VT) *reinterpret_cast<f4_t*>(pp + kPartHead + 16 * vt + 4 * kg) = o[vt];
  }
}

// ---- Pair form for the widest rows: a workgroup of two waves owns one 16-row tile and splits the ROW
// between them.  Wave w multiplies its half of the 32-entry chunks (half of the score products; the two
// partial score tiles meet in LDS and both waves add them in the same order, so both hold the same
// weights), writes its chunks' share of the transposed values into the workgroup's LDS block, and
// accumulates its half of the value tiles.  A wave then holds 64 accumulators, 36 registers of query
// pieces and 36 of key pieces: two such waves fit a SIMD, and one covers the other's waits.  Two
// workgroup barriers per key block (of two waves each): before the transposed values are overwritten, and
// after they and the partial scores are written.  24 KB of LDS a workgroup: four share a CU.
template <int KKM, int VTM, bool EXACT>
__global__ void __launch_bounds__(128) __attribute__((amdgpu_waves_per_eu(2, 2))) latent_attention_pair_kernel(
    bf16_t* __restrict__ out, float* __restrict__ part, const bf16_t* __restrict__ q, long q_stride,
    const bf16_t* __restrict__ cache, long block_stride, const int* __restrict__ block_tables, int bt_stride,
    const int* __restrict__ qsl, const int* __restrict__ seq_lens, int koff, int H, int dk, int rank, float scale,
    const float* __restrict__ sink, int nsplit, int window) {
  constexpr int KHM = KKM / 2, VHM = VTM / 2;
  static_assert(KKM % 2 == 0 && VTM % 2 == 0, "the row is split in two");
  __shared__ __attribute__((aligned(16))) bf16_t vt_s[16 * VTM * kVtPitch];
  __shared__ __attribute__((aligned(16))) f4_t sx[2][2][64];
  const int s = blockIdx.z;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int row0 = qsl[s], qlen = qsl[s + 1] - row0;
  const int nrows = qlen * H;
  const int id = blockIdx.x;
  const int tile = id / nsplit, sp = id - tile * nsplit;
  if (tile * 16 >= nrows) return;  // the same for both waves of the workgroup
  const int c = lane & 15, kg = lane >> 4;
  const int r = tile * 16 + c;
  const bool rok = r < nrows;
  const int rr = rok ? r : nrows - 1;
  const int tok = rr / H, hd = rr - tok * H;
  const int last = bt_stride * 16 - 1;
  const int base = max(seq_lens[s] - qlen, 0);
  const int pq = min(base + tok, last);
  const int p_first = min(base + (tile * 16) / H, last);
  const int p_last = min(base + min(tile * 16 + 15, nrows - 1) / H, last);
  // window > 0: a row at position p sees p - window + 1 .. p; the tile's walk starts at the block of
  // its first row's oldest visible key
  const int wb = window > 0 ? max(p_first - window + 1, 0) >> 4 : 0;
  const int nblk = (p_last >> 4) + 1 - wb;
  const int b0 = wb + static_cast<int>(static_cast<long>(nblk) * sp / nsplit);
  const int b1 = wb + static_cast<int>(static_cast<long>(nblk) * (sp + 1) / nsplit);
  const int KK = EXACT ? KKM : (dk + 31) >> 5, VT = EXACT ? VTM : rank >> 4;
  const int kk0 = w * KHM, vt0 = w * VHM;  // this wave's chunks and value tiles
  const int* bt = block_tables + static_cast<long>(s) * bt_stride;
  uint4 qf[KHM];
  {
    const bf16_t* qp = q + static_cast<long>(row0 + tok) * q_stride + static_cast<long>(hd) * dk + 8 * kg;
#pragma unroll
    for (int j = 0; j < KHM; ++j) {
      const int kk = kk0 + j;
      qf[j] = (rok && (EXACT || (kk < KK && 32 * kk + 8 * kg + 8 <= dk))) ? *reinterpret_cast<const uint4*>(qp + 32 * kk)
                                                                          : make_uint4(0, 0, 0, 0);
    }
  }
  const float L2E = 1.4426950408889634f;
  float m = (sink && sp == 0) ? sink[hd] * L2E : -INFINITY;
  float l = (sink && sp == 0 && kg == 0) ? 1.f : 0.f;
  f4_t o[VHM];
#pragma unroll
  for (int j = 0; j < VHM; ++j) o[j] = f4_t{0.f, 0.f, 0.f, 0.f};
  const float sl2 = scale * L2E;
  uint4 kr[KHM];
  auto load_block = [&](int kb) {
    const bf16_t* kp = cache + static_cast<long>(bt[kb]) * block_stride + koff + static_cast<long>(c) * dk + 8 * kg;
#pragma unroll
    for (int j = 0; j < KHM; ++j) {
      const int kk = kk0 + j;
      kr[j] = (EXACT || (kk < KK && 32 * kk + 8 * kg + 8 <= dk)) ? *reinterpret_cast<const uint4*>(kp + 32 * kk)
                                                                 : make_uint4(0, 0, 0, 0);
    }
    if (kb * 16 + 15 > p_last && kb * 16 + c > p_last) {  // stale rows behind the tile's last position: zeros
#pragma unroll
      for (int j = 0; j < KHM; ++j) kr[j] = make_uint4(0, 0, 0, 0);
    }
  };
  if (b0 < b1) load_block(b0);
  for (int kb = b0; kb < b1; ++kb) {
    const int k0 = kb * 16, buf = (kb - b0) & 1;
    bf16_t* vt_w = vt_s;
    __syncthreads();  // both waves have read the previous block's values
    f4_t ac[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) ac[i] = f4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < KHM; ++j) {
      const int kk = kk0 + j;
      if (EXACT || kk < KK) {
        ac[j & 3] = mfma_piece(kr[j], qf[j], ac[j & 3]);
        const int d0 = 32 * kk + 8 * kg;
        if (d0 < rank) {
          const uint4 a = kr[j];
          bf16_t* wp = vt_w + d0 * kVtPitch + c;
          wp[0] = static_cast<bf16_t>(a.x & 0xFFFFu);
          wp[kVtPitch] = static_cast<bf16_t>(a.x >> 16);
          wp[2 * kVtPitch] = static_cast<bf16_t>(a.y & 0xFFFFu);
          wp[3 * kVtPitch] = static_cast<bf16_t>(a.y >> 16);
          wp[4 * kVtPitch] = static_cast<bf16_t>(a.z & 0xFFFFu);
          wp[5 * kVtPitch] = static_cast<bf16_t>(a.z >> 16);
          wp[6 * kVtPitch] = static_cast<bf16_t>(a.w & 0xFFFFu);
          wp[7 * kVtPitch] = static_cast<bf16_t>(a.w >> 16);
        }
      }
    }
    sx[buf][w][lane] = (ac[0] + ac[1]) + (ac[2] + ac[3]);
    if (kb + 1 < b1) load_block(kb + 1);  // in flight across the barrier, the weights and the value products
    __syncthreads();
    const f4_t acc = sx[buf][0][lane] + sx[buf][1][lane];  // the same sum in both waves
    const bool whole = k0 + 15 <= p_first && (window <= 0 || k0 >= p_last - window + 1);
    float sv[4], mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (whole) {
        sv[i] = acc[i] * sl2;
      } else {
        const int jj = k0 + 4 * kg + i;
        sv[i] = (rok && jj <= pq && (window <= 0 || pq - jj < window)) ? acc[i] * sl2 : -INFINITY;
      }
      mx = fmaxf(mx, sv[i]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m, mx);
    if (__builtin_amdgcn_ballot_w64(m_new > m) != 0) {
      const float corr = m_new == -INFINITY ? 1.f : __builtin_amdgcn_exp2f(m - m_new);
      l *= corr;
#pragma unroll
      for (int j = 0; j < VHM; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) o[j][i] *= corr;
      m = m_new;
    }
    s4_t ph, pl;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float pr = (whole || sv[i] != -INFINITY) ? __builtin_amdgcn_exp2f(sv[i] - m) : 0.f;
      l += pr;
      const uint32_t u = __float_as_uint(pr), uh = u & 0xFFFF0000u;
      uint32_t ul = __float_as_uint(pr - __uint_as_float(uh));
      ul += 0x7FFFu + ((ul >> 16) & 1u);
      ph[i] = static_cast<short>(uh >> 16);
      pl[i] = static_cast<short>(ul >> 16);
    }
    const bf16_t* vp = vt_w + (16 * vt0 + c) * kVtPitch + 4 * kg;
#pragma unroll
    for (int j = 0; j < VHM; ++j) {
      if (EXACT || vt0 + j < VT) {
        const s4_t a = *reinterpret_cast<const s4_t*>(vp + 16 * j * kVtPitch);
        const f4_t t = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, ph, o[j], 0, 0, 0);
        o[j] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, pl, t, 0, 0, 0);
      }
    }
  }
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);
  if (!rok) return;
  const long grow = static_cast<long>(row0 + tok) * H + hd;
  if (nsplit == 1) {
    const float inv = 1.f / l;
    bf16_t* op = out + grow * rank + 16 * vt0 + 4 * kg;
#pragma unroll
    for (int j = 0; j < VHM; ++j) {
      if (EXACT || vt0 + j < VT) {
        uint2 wv;
        wv.x = pack2(o[j][0] * inv, o[j][1] * inv);
        wv.y = pack2(o[j][2] * inv, o[j][3] * inv);
        *reinterpret_cast<uint2*>(op + 16 * j) = wv;
      }
    }
  } else {
    float* pp = part + (grow * nsplit + sp) * (rank + kPartHead);
    if (kg == 0 && w == 0) { pp[0] = m; pp[1] = l; }
#pragma unroll
    for (int j = 0; j < VHM; ++j)
      if (EXACT || vt0 + j < VT) *reinterpret_cast<f4_t*>(pp + kPartHead + 16 * (vt0 + j) + 4 * kg) = o[j];
  }
}

// One workgroup per (token, head) row: the stretches' (m, l, o) merged.  m is in log2 units.  The
// stretches' weights 2^(m_s - M) / L are made once by the first wave's lanes; the sum over the
// stretches is unrolled so that their loads are in flight together.
constexpr int kMaxSplit = 64;
__global__ void __launch_bounds__(128) latent_attention_combine_kernel(bf16_t* __restrict__ out,
                                                                       const float* __restrict__ part, int nsplit,
                                                                       int rank) {
  __shared__ float wsh[kMaxSplit];
  const long row = blockIdx.x;
  const int ps = rank + kPartHead;
  const float* pp = part + row * nsplit * ps;
  if (threadIdx.x < 64) {
    const int s = threadIdx.x;
    const float ms = s < nsplit ? pp[s * ps] : -INFINITY;
    const float ls = s < nsplit ? pp[s * ps + 1] : 0.f;
    const float M = wave_max(ms);
    const float w = ms != -INFINITY ? __builtin_amdgcn_exp2f(ms - M) : 0.f;
    const float L = wave_sum(ls * w);
    wsh[s] = w / L;
  }
  __syncthreads();
  for (int d = threadIdx.x; d < rank; d += blockDim.x) {
    const float* pd = pp + kPartHead + d;
    float a = 0.f;
#pragma unroll 8
    for (int s = 0; s < nsplit; ++s) {
      const float w = wsh[s];
      a += w != 0.f ? pd[s * ps] * w : 0.f;  // a stretch without keys wrote zeros; nothing is read as a number it is not
    }
    out[row * rank + d] = f2bf(a);
  }
}

// The merge alone, for other attention kernels that split a row's keys over workgroups and write the same
// (maximum in log2 units, sum, two unused, unnormalised output[width]) records: rows = (token, head) pairs.
bool launch_attention_combine(void* out, const float* part, long rows, int nsplit, int width, hipStream_t st) {
  if (rows == 0) return true;
  if (nsplit < 1 || nsplit > kMaxSplit || reinterpret_cast<uintptr_t>(part) % 16) return false;
  hipLaunchKernelGGL(latent_attention_combine_kernel, dim3(rows), dim3(128), 0, st, (bf16_t*)out, part, nsplit, width);
  MXS_CHECK_LAUNCH();
  return true;
}

// False: sizes the kernel does not take (the caller runs the general kernel).
bool launch_latent_attention(void* out, float* part, const void* q, long q_stride, const void* cache, long block_stride,
                             const int* block_tables, int bt_stride, const int* qsl, const int* seq_lens, int S, int rows,
                             int koff, int H, int dk, int rank, int bs, float scale, int max_q, const float* sink,
                             int nsplit, bool pair, int window, hipStream_t st) {
  if (rows == 0 || S == 0) return true;
  if (bs != 16 || dk % 8 || rank % 16 || rank > dk || dk > 576 || rank > 512 || q_stride % 8 || koff % 8 ||
      block_stride % 8 || reinterpret_cast<uintptr_t>(q) % 16 || reinterpret_cast<uintptr_t>(cache) % 16 ||
      reinterpret_cast<uintptr_t>(part) % 16 || nsplit < 1 || nsplit > kMaxSplit || (nsplit > 1 && part == nullptr))
    return false;
  const int tiles = (max_q * H + 15) / 16;
#define MIX_LA(KKM, VTM, NW, QLDS, EXACT)                                                                             \
  hipLaunchKernelGGL((latent_attention_mfma_kernel<KKM, VTM, NW, QLDS, EXACT>), dim3((tiles * nsplit + NW - 1) / NW, 1, S), \
                     dim3(64 * NW), NW * (16 * VTM * kVtPitch * sizeof(bf16_t) + (QLDS ? KKM * 64 * 16 : 0)), st,     \
                     (bf16_t*)out, part, (const bf16_t*)q, q_stride, (const bf16_t*)cache, block_stride, block_tables, \
                     bt_stride, qsl, seq_lens, koff, H, dk, rank, scale, sink, nsplit, window)
  if (dk <= 192 && rank <= 128) MIX_LA(6, 8, 4, false, false);
  else if (dk <= 320 && rank <= 256) MIX_LA(10, 16, 4, false, false);
  else if (pair) {
#define MIX_LP(EXACT)                                                                                                  \
  hipLaunchKernelGGL((latent_attention_pair_kernel<18, 32, EXACT>), dim3(tiles * nsplit, 1, S), dim3(128), 0, st,      \
                     (bf16_t*)out, part, (const bf16_t*)q, q_stride, (const bf16_t*)cache, block_stride, block_tables, \
                     bt_stride, qsl, seq_lens, koff, H, dk, rank, scale, sink, nsplit, window)
    if (dk == 576 && rank == 512) MIX_LP(true);
    else MIX_LP(false);
#undef MIX_LP
  }
  else if (dk == 576 && rank == 512) MIX_LA(18, 32, 1, true, true);
  else MIX_LA(18, 32, 1, true, false);  // 38 KB of LDS a wave: four one-wave workgroups share a CU
#undef MIX_LA
  MXS_CHECK_LAUNCH();
  if (nsplit > 1) {
    hipLaunchKernelGGL(latent_attention_combine_kernel, dim3(rows * H), dim3(128), 0, st, (bf16_t*)out, part, nsplit, rank);
    MXS_CHECK_LAUNCH();
  }
  return true;
}

}  // namespace mxs
