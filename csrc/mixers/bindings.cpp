// torch bindings of the mixer kernels (mxserve/_M): shape and dtype checks on the host, so that a
// launch never reads or writes outside what the kernels and their grids assume.
#include <ATen/ATen.h>
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime.h>
#include <torch/extension.h>

#include "column_scan.h"

namespace mxs {
void launch_resid_update(float*, const void*, long, const void*, const void*, long, const void*, const void*, int,
                         const void*, void*, int, int, float, float, float, float, bool, hipStream_t);
void launch_embed_normed(float*, float*, void*, const int64_t*, const void*, const void*, int, int, long, float, float, bool,
                         hipStream_t);
bool launch_depth_mix(float*, long, int, const float*, void*, int, int, bool, hipStream_t);
void launch_xielu(void*, const void*, long, const float*, bool, hipStream_t);
void launch_qkv_prep_cache(void*, long, const void*, long, const void*, long, const int64_t*, const int64_t*, void*, long,
                           int, int, int, int, int, int, int, int, const float*, int, float, bool, const void*, const void*,
                           const void*, const void*, const void*, float, int, bool, hipStream_t);
bool launch_talking_attention(void*, const void*, long, const void*, long, const int*, int, const int*, const int*, int,
                              int, int, int, int, int, int, int, int, float, int, int, int, const float*, const float*, float*,
                              int, bool, hipStream_t);
void launch_cast_into(void*, long, const float*, int, int, bool, hipStream_t);
void launch_relu_sq(void*, const void*, long, bool, hipStream_t);
void launch_softcap(float*, const void*, long, int, int, float, bool, hipStream_t);
void launch_gated_rms_norm(void*, const float*, const void*, long, const void*, int, int, int, float, bool, hipStream_t);
void launch_gate_linear(float*, const void*, long, const void*, const void*, int, int, int, bool, hipStream_t);
void launch_kv_write(void*, long, const void*, long, const void*, long, const int64_t*, int, int, int, int, int, int,
                     int, bool, hipStream_t);
bool launch_window_attention(void*, const void*, long, const void*, long, const int*, int, const int*, const int*, int,
                             int, int, int, int, int, int, int, int, float, int, int, int, const float*, int, bool,
                             hipStream_t);
bool launch_matrix_scan(float*, const void*, long, const void*, long, const void*, long, const float*, const float*,
                        float*, long, const int*, long, const int*, const int*, int, int, int, int, int, int, float,
                        float, bool, bool, int, int, float*, float*, long, hipStream_t);
void launch_embed_scaled(float*, const int64_t*, const void*, int, int, long, float, bool, hipStream_t);
void launch_silu_mul(void*, const void*, long, int, int, bool, hipStream_t);
void launch_rope_qkv_cache(void*, long, const void*, long, const void*, long, const int64_t*, const int64_t*, void*, long,
                           int, int, int, int, int, int, int, int, const float*, int, const void*, const void*, float,
                           const float*, int, bool, hipStream_t);
void launch_rope_rows(void*, long, const void*, long, const int64_t*, int, int, int, const float*, int, float, float, bool,
                      hipStream_t);
void launch_causal_conv(void*, const void*, long, const void*, const void*, float*, long, const int*, long, const int*,
                        const int*, int, int, int, int, int, bool, hipStream_t);
void launch_gated_norm(void*, long, const float*, const void*, long, const void*, int, int, int, int, float, int, int,
                       float, bool, hipStream_t);
bool launch_column_scan(const ScanArgs&, int, bool, bool, hipStream_t);
bool launch_latent_attention(void*, float*, const void*, long, const void*, long, const int*, int, const int*, const int*,
                             int, int, int, int, int, int, int, float, int, const float*, int, bool, int, hipStream_t);
void launch_latent_prep(void*, const void*, long, const void*, long, const int64_t*, const int64_t*, void*, long, int, int,
                        int, int, int, int, const float*, const void*, const void*, float, bool, bool, hipStream_t);
void launch_rope_half_into(void*, long, const void*, long, const int64_t*, int, int, int, int, int, int, const float*, int,
                           bool, bool, hipStream_t);
void launch_route_topk(float*, int*, const float*, int, int, int, bool, bool, hipStream_t);
void launch_capped_glu(void*, const void*, long, int, int, float, float, bool, hipStream_t);
bool launch_expert_align(int*, int*, const int*, int, int, hipStream_t);
void launch_gather_scaled(void*, const void*, long, const float*, const int*, int, int, int, bool, hipStream_t);
void launch_spread_scaled(void*, const void*, long, const float*, const int*, int, int, int, int, bool, hipStream_t);
void launch_expert_combine(void*, const void*, const int*, int, int, long, const void*, long, int, const float*, bool, bool,
                           hipStream_t);
}  // namespace mxs

namespace {

using OptT = c10::optional<at::Tensor>;

hipStream_t stream() { return c10::hip::getCurrentHIPStream().stream(); }

bool is_bf(const at::Tensor& t) {
  TORCH_CHECK(t.scalar_type() == at::kBFloat16 || t.scalar_type() == at::kFloat, "activations must be bf16 or fp32");
  return t.scalar_type() == at::kBFloat16;
}

// a [rows, cols] matrix of dtype `bf`, unit column stride
const void* mat(const at::Tensor& t, bool bf, int64_t rows, int64_t cols, const char* name) {
  TORCH_CHECK(t.is_cuda() && t.dim() == 2 && t.size(0) == rows && t.size(1) == cols && (cols == 1 || t.stride(1) == 1),
              name, ": expected a GPU [", rows, ", ", cols, "] matrix with contiguous rows");
  TORCH_CHECK(is_bf(t) == bf, name, ": dtype differs from the other operands");
  return t.data_ptr();
}

const void* vec(const OptT& t, bool bf, int64_t n, const char* name) {
  if (!t.has_value()) return nullptr;
  TORCH_CHECK(t->is_cuda() && t->is_contiguous() && t->numel() == n, name, ": expected ", n, " contiguous elements");
  TORCH_CHECK(is_bf(*t) == bf, name, ": dtype differs from the other operands");
  return t->data_ptr();
}

const int* i32(const at::Tensor& t, int64_t n, const char* name) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == at::kInt && t.is_contiguous() && t.numel() >= n, name,
              ": expected >= ", n, " contiguous int32");
  return t.data_ptr<int>();
}

float* f32(const at::Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == at::kFloat && t.is_contiguous(), name, ": expected contiguous fp32");
  return t.data_ptr<float>();
}

void resid_update(at::Tensor x, OptT a, OptT wa, OptT b, OptT wb, OptT bias, bool assign, OptT norm_w, OptT h,
                  double eps, double a_scale, double w_offset, double wa_offset) {
  float* xp = f32(x, "x");
  TORCH_CHECK(x.dim() == 2, "x: [T, W]");
  const int64_t T = x.size(0), W = x.size(1);
  const at::Tensor* any = a.has_value() ? &*a : (norm_w.has_value() ? &*norm_w : (h.has_value() ? &*h : nullptr));
  if (any == nullptr || T == 0) return;
  const bool bf = is_bf(*any);
  const void* ap = a.has_value() ? mat(*a, bf, T, W, "a") : nullptr;
  const void* bp = b.has_value() ? mat(*b, bf, T, W, "b") : nullptr;
  TORCH_CHECK(!b.has_value() || (a.has_value() && wa.has_value() && wb.has_value()), "two branches need both weights");
  TORCH_CHECK(!assign || a.has_value(), "assign needs a");
  TORCH_CHECK(!norm_w.has_value() || h.has_value(), "norm_w needs h (h alone: the updated x, cast)");
  void* hp = nullptr;
  if (h.has_value()) {
    TORCH_CHECK(h->is_cuda() && h->is_contiguous() && h->dim() == 2 && h->size(0) == T && h->size(1) == W &&
                is_bf(*h) == bf, "h: contiguous [T, W] of the operands' dtype");
    hp = h->data_ptr();
  }
  mxs::launch_resid_update(xp, ap, a.has_value() ? a->stride(0) : 0, vec(wa, bf, W, "wa"), bp,
                           b.has_value() ? b->stride(0) : 0, vec(wb, bf, W, "wb"), vec(bias, bf, W, "bias"), assign,
                           vec(norm_w, bf, W, "norm_w"), hp, static_cast<int>(T), static_cast<int>(W),
                           static_cast<float>(eps), static_cast<float>(a_scale), static_cast<float>(w_offset),
                           static_cast<float>(wa_offset), bf, stream());
}

void cast_into(at::Tensor dst, at::Tensor x) {
  const float* xp = f32(x, "x");
  TORCH_CHECK(x.dim() == 2 && dst.is_cuda() && dst.dim() == 2 && dst.size(0) == x.size(0) && dst.size(1) >= x.size(1) &&
              dst.stride(1) == 1, "dst: [T, >= W] with contiguous rows");
  mxs::launch_cast_into(dst.data_ptr(), dst.stride(0), xp, static_cast<int>(x.size(0)), static_cast<int>(x.size(1)),
                        is_bf(dst), stream());
}

void relu_sq(at::Tensor out, at::Tensor x) {
  TORCH_CHECK(x.is_cuda() && x.is_contiguous() && out.is_contiguous() && out.numel() == x.numel() &&
              out.scalar_type() == x.scalar_type(), "relu_sq: contiguous tensors of one dtype");
  mxs::launch_relu_sq(out.data_ptr(), x.data_ptr(), x.numel(), is_bf(x), stream());
}

void softcap(at::Tensor out, at::Tensor x, double cap) {
  float* op = f32(out, "out");
  TORCH_CHECK(x.is_cuda() && x.dim() == 2 && x.stride(1) == 1 && out.dim() == 2 && out.size(0) == x.size(0) &&
              out.size(1) == x.size(1), "softcap: [n, V]");
  mxs::launch_softcap(op, x.data_ptr(), x.stride(0), static_cast<int>(x.size(0)), static_cast<int>(x.size(1)),
                      static_cast<float>(cap), is_bf(x), stream());
}

void gated_rms_norm(at::Tensor out, at::Tensor o, at::Tensor gate, at::Tensor w, double eps, int64_t groups) {
  const float* opn = f32(o, "o");
  TORCH_CHECK(o.dim() == 2, "o: [T, N]");
  const int64_t T = o.size(0), N = o.size(1);
  const bool bf = is_bf(out);
  TORCH_CHECK(out.is_cuda() && out.is_contiguous() && out.dim() == 2 && out.size(0) == T && out.size(1) == N, "out: [T, N]");
  TORCH_CHECK(groups >= 1 && N % groups == 0, "groups must divide N");
  mxs::launch_gated_rms_norm(out.data_ptr(), opn, mat(gate, bf, T, N, "gate"), gate.stride(0), vec(OptT(w), bf, N, "w"),
                             static_cast<int>(T), static_cast<int>(N), static_cast<int>(groups), static_cast<float>(eps),
                             bf, stream());
}

void gate_linear(at::Tensor out, at::Tensor h, at::Tensor w, OptT bias) {
  float* op = f32(out, "out");
  TORCH_CHECK(h.is_cuda() && h.dim() == 2 && h.stride(1) == 1 && w.is_cuda() && w.dim() == 2 && w.is_contiguous() &&
              w.size(1) == h.size(1) && out.dim() == 2 && out.size(0) == h.size(0) && out.size(1) == w.size(0),
              "gate_linear: h [T, W], w [N, W], out [T, N]");
  const bool bf = is_bf(h);
  TORCH_CHECK(is_bf(w) == bf, "w: dtype differs from h");
  mxs::launch_gate_linear(op, h.data_ptr(), h.stride(0), w.data_ptr(), vec(bias, bf, w.size(0), "bias"),
                          static_cast<int>(h.size(0)), static_cast<int>(w.size(0)), static_cast<int>(w.size(1)), bf,
                          stream());
}

void check_cache(const at::Tensor& cache, bool bf, int64_t koff, int64_t voff, int64_t G, int64_t dk, int64_t dv,
                 int64_t bs) {
  TORCH_CHECK(cache.is_cuda() && cache.dim() == 2 && cache.is_contiguous() && is_bf(cache) == bf,
              "cache: contiguous [blocks, block_elems] of the operands' dtype");
  TORCH_CHECK(koff >= 0 && voff >= 0 && koff + G * bs * dk <= cache.size(1) && voff + G * bs * dv <= cache.size(1),
              "K/V region outside a cache block");
}

void kv_write(at::Tensor cache, at::Tensor k, at::Tensor v, at::Tensor slots, int64_t koff, int64_t voff, int64_t G,
              int64_t dk, int64_t dv, int64_t bs) {
  const bool bf = is_bf(k);
  const int64_t T = k.size(0);
  check_cache(cache, bf, koff, voff, G, dk, dv, bs);
  TORCH_CHECK(slots.is_cuda() && slots.scalar_type() == at::kLong && slots.is_contiguous() && slots.numel() == T,
              "slot_mapping: int64 [T]");
  mxs::launch_kv_write(cache.data_ptr(), cache.stride(0), mat(k, bf, T, G * dk, "k"), k.stride(0),
                       mat(v, bf, T, G * dv, "v"), v.stride(0), slots.data_ptr<int64_t>(), static_cast<int>(T),
                       static_cast<int>(koff), static_cast<int>(voff), static_cast<int>(G), static_cast<int>(dk),
                       static_cast<int>(dv), static_cast<int>(bs), bf, stream());
}

void window_attention(at::Tensor out, at::Tensor q, at::Tensor cache, at::Tensor block_tables, at::Tensor qsl,
                      at::Tensor seq_lens, int64_t koff, int64_t voff, int64_t H, int64_t G, int64_t dk, int64_t dv,
                      int64_t bs, double scale, int64_t window, int64_t keep, int64_t max_query_len, OptT sink,
                      int64_t v_stride) {
  const bool bf = is_bf(q);
  const float* sinkp = nullptr;
  if (sink.has_value()) {
    sinkp = f32(*sink, "sink");
    TORCH_CHECK(sink->numel() == H, "sink: fp32 [H]");
  }
  const int64_t T = q.size(0), S = seq_lens.numel();
  if (v_stride > 0 && v_stride != dv) {  // values are a slice of a wider cached row of the one kv head
    TORCH_CHECK(G == 1 && v_stride >= dv, "strided value rows: one kv head, stride >= dv");
    check_cache(cache, bf, koff, voff, G, dk, 0, bs);
    TORCH_CHECK(voff >= 0 && voff + (bs - 1) * v_stride + dv <= cache.size(1), "value rows reach past the cache block");
  } else {
    check_cache(cache, bf, koff, voff, G, dk, dv, bs);
  }
  TORCH_CHECK(G >= 1 && H % G == 0, "query heads must divide over kv heads");
  TORCH_CHECK(out.is_cuda() && out.is_contiguous() && out.dim() == 2 && out.size(0) == T && out.size(1) == H * dv &&
              is_bf(out) == bf, "out: [T, H*dv]");
  TORCH_CHECK(block_tables.is_cuda() && block_tables.scalar_type() == at::kInt && block_tables.dim() == 2 &&
              block_tables.size(0) >= S && block_tables.stride(1) == 1, "block_tables: int32 [S, max_blocks]");
  const bool ok = mxs::launch_window_attention(
      out.data_ptr(), mat(q, bf, T, H * dk, "q"), q.stride(0), cache.data_ptr(), cache.stride(0),
      block_tables.data_ptr<int>(), static_cast<int>(block_tables.stride(0)), i32(qsl, S + 1, "qsl"),
      i32(seq_lens, S, "seq_lens"), static_cast<int>(S), static_cast<int>(T), static_cast<int>(koff),
      static_cast<int>(voff), static_cast<int>(H), static_cast<int>(G), static_cast<int>(dk), static_cast<int>(dv),
      static_cast<int>(bs), static_cast<float>(scale), static_cast<int>(window), static_cast<int>(keep),
      static_cast<int>(std::min<int64_t>(max_query_len, T)), sinkp, static_cast<int>(v_stride), bf, stream());
  TORCH_CHECK(ok, "window_attention: head sizes beyond what the kernel holds (dv <= 512)");
}

void scan(bool mlstm, at::Tensor out, at::Tensor q, at::Tensor k, at::Tensor v, const float* decay, const float* gates,
          at::Tensor state, at::Tensor state_rows, int64_t off, at::Tensor qsl, at::Tensor seq_lens, int64_t H,
          int64_t dk, int64_t dv, bool silu, double cap, double q_scale, int64_t piece, int64_t npieces, OptT sc_local,
          OptT sc_start) {
  const bool bf = is_bf(q);
  const int64_t T = q.size(0), S = seq_lens.numel();
  float* op = f32(out, "out");
  TORCH_CHECK(out.dim() == 2 && out.size(0) == T && out.size(1) == H * dv, "out: fp32 [T, H*dv]");
  float* sp = f32(state, "state");
  const int64_t need = mlstm ? H * (dk * dv + dk + 1) : H * dk * dv;
  TORCH_CHECK(state.dim() == 2 && off >= 0 && off + need <= state.size(1), "state slot too small for this layer");
  // time-split launches: two scratch pools of [S, npieces, sc_floats] (a piece's end state; mLSTM: plus [H] sums)
  const int64_t sc_floats = need + (mlstm ? H : 0);
  float *scl = nullptr, *scs = nullptr;
  if (npieces > 1) {
    TORCH_CHECK(piece >= 16 && sc_local.has_value() && sc_start.has_value(), "a split scan needs its scratch pools");
    scl = f32(*sc_local, "sc_local");
    scs = f32(*sc_start, "sc_start");
    TORCH_CHECK(sc_local->numel() >= S * npieces * sc_floats && sc_start->numel() >= S * npieces * sc_floats,
                "scratch pools smaller than [S, npieces, state]");
  } else {
    piece = 1;
    npieces = 1;
  }
  const bool ok = mxs::launch_matrix_scan(
      op, mat(q, bf, T, H * dk, "q"), q.stride(0), mat(k, bf, T, H * dk, "k"), k.stride(0), mat(v, bf, T, H * dv, "v"),
      v.stride(0), decay, gates, sp, state.stride(0), i32(state_rows, S, "state_rows"), off, i32(qsl, S + 1, "qsl"),
      i32(seq_lens, S, "seq_lens"), static_cast<int>(S), static_cast<int>(T), static_cast<int>(H), static_cast<int>(dk),
      static_cast<int>(dv), silu ? 1 : 0, static_cast<float>(cap), static_cast<float>(q_scale), mlstm, bf,
      static_cast<int>(piece), static_cast<int>(npieces), scl, scs, sc_floats, stream());
  TORCH_CHECK(ok, "matrix scan: key size beyond 256");
}

void decay_scan(at::Tensor out, at::Tensor q, at::Tensor k, at::Tensor v, at::Tensor decay, at::Tensor state,
                at::Tensor state_rows, int64_t off, at::Tensor qsl, at::Tensor seq_lens, int64_t H, int64_t dk,
                int64_t dv, bool silu, int64_t piece, int64_t npieces, OptT sc_local, OptT sc_start) {
  TORCH_CHECK(decay.numel() == H, "decay: fp32 [H]");
  scan(false, out, q, k, v, f32(decay, "decay"), nullptr, state, state_rows, off, qsl, seq_lens, H, dk, dv, silu, 0.0, 1.0,
       piece, npieces, sc_local, sc_start);
}

void mlstm_scan(at::Tensor out, at::Tensor q, at::Tensor k, at::Tensor v, at::Tensor gates, at::Tensor state,
                at::Tensor state_rows, int64_t off, at::Tensor qsl, at::Tensor seq_lens, int64_t H, int64_t dk,
                int64_t dv, double cap, double q_scale, int64_t piece, int64_t npieces, OptT sc_local, OptT sc_start) {
  TORCH_CHECK(gates.dim() == 2 && gates.size(0) == q.size(0) && gates.size(1) == 2 * H, "gates: fp32 [T, 2H]");
  scan(true, out, q, k, v, nullptr, f32(gates, "gates"), state, state_rows, off, qsl, seq_lens, H, dk, dv, false, cap,
       q_scale, piece, npieces, sc_local, sc_start);
}

// ---- rotary attention, convolutions, column scans
const int64_t* i64(const at::Tensor& t, int64_t n, const char* name) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == at::kLong && t.is_contiguous() && t.numel() == n, name,
              ": expected ", n, " contiguous int64");
  return t.data_ptr<int64_t>();
}

const float* f32n(const OptT& t, int64_t n, const char* name) {
  if (!t.has_value()) return nullptr;
  TORCH_CHECK(t->numel() == n, name, ": expected ", n, " elements");
  return f32(*t, name);
}

void embed_scaled(at::Tensor out, at::Tensor ids, at::Tensor table, double scale) {
  float* op = f32(out, "out");
  TORCH_CHECK(table.is_cuda() && table.dim() == 2 && table.is_contiguous(), "table: contiguous [vocab, W]");
  const int64_t T = ids.numel(), W = table.size(1);
  TORCH_CHECK(out.dim() == 2 && out.size(0) == T && out.size(1) == W, "out: fp32 [T, W]");
  mxs::launch_embed_scaled(op, i64(ids, T, "ids"), table.data_ptr(), static_cast<int>(T), static_cast<int>(W),
                           table.size(0), static_cast<float>(scale), is_bf(table), stream());
}

void silu_mul(at::Tensor out, at::Tensor gu) {
  const bool bf = is_bf(gu);
  TORCH_CHECK(gu.is_cuda() && gu.dim() == 2 && gu.stride(1) == 1 && gu.size(1) % 2 == 0, "gu: [T, 2F] with contiguous rows");
  const int64_t T = gu.size(0), F = gu.size(1) / 2;
  TORCH_CHECK(out.is_cuda() && out.is_contiguous() && out.dim() == 2 && out.size(0) == T && out.size(1) == F &&
              is_bf(out) == bf, "out: [T, F]");
  mxs::launch_silu_mul(out.data_ptr(), gu.data_ptr(), gu.stride(0), static_cast<int>(T), static_cast<int>(F), bf, stream());
}

void rope_qkv_cache(at::Tensor q, OptT k, OptT v, at::Tensor positions, at::Tensor slots, at::Tensor cache, int64_t koff,
                    int64_t voff, int64_t H, int64_t G, int64_t dk, int64_t dv, int64_t bs, at::Tensor freqs, OptT q_norm,
                    OptT k_norm, double eps, OptT v_freqs) {
  const bool bf = is_bf(q);
  const int64_t T = q.size(0);
  TORCH_CHECK(k.has_value() == v.has_value(), "k and v go together");
  const void *kp = nullptr, *vp = nullptr;
  if (k.has_value()) {
    check_cache(cache, bf, koff, voff, G, dk, dv, bs);
    kp = mat(*k, bf, T, G * dk, "k");
    vp = mat(*v, bf, T, G * dv, "v");
  }
  const int64_t nf = freqs.numel(), nvf = v_freqs.has_value() ? v_freqs->numel() : 0;
  TORCH_CHECK(2 * nf <= dk && 2 * nvf <= dv, "more rotary pairs than the head has dimensions");
  mxs::launch_rope_qkv_cache(const_cast<void*>(mat(q, bf, T, H * dk, "q")), q.stride(0), kp, k.has_value() ? k->stride(0) : 0,
                             vp, v.has_value() ? v->stride(0) : 0, i64(positions, T, "positions"),
                             i64(slots, T, "slot_mapping"), cache.data_ptr(), cache.stride(0), static_cast<int>(T),
                             static_cast<int>(koff), static_cast<int>(voff), static_cast<int>(H), static_cast<int>(G),
                             static_cast<int>(dk), static_cast<int>(dv), static_cast<int>(bs), f32(freqs, "freqs"),
                             static_cast<int>(nf), vec(q_norm, bf, dk, "q_norm"), vec(k_norm, bf, dk, "k_norm"),
                             static_cast<float>(eps), f32n(v_freqs, nvf, "v_freqs"), static_cast<int>(nvf), bf, stream());
}

void rope_rows(at::Tensor out, at::Tensor x, at::Tensor positions, int64_t heads, int64_t dim, at::Tensor freqs,
               double sign, double scale) {
  const bool bf = is_bf(x);
  const int64_t T = x.size(0);
  TORCH_CHECK(2 * freqs.numel() <= dim, "more rotary pairs than the head has dimensions");
  mxs::launch_rope_rows(const_cast<void*>(mat(out, bf, T, heads * dim, "out")), out.stride(0), mat(x, bf, T, heads * dim, "x"),
                        x.stride(0), i64(positions, T, "positions"), static_cast<int>(T), static_cast<int>(heads),
                        static_cast<int>(dim), f32(freqs, "freqs"), static_cast<int>(freqs.numel()),
                        static_cast<float>(sign), static_cast<float>(scale), bf, stream());
}

void causal_conv(at::Tensor out, at::Tensor x, at::Tensor w, OptT bias, at::Tensor state, at::Tensor state_rows,
                 int64_t off, at::Tensor qsl, at::Tensor seq_lens, bool silu) {
  const bool bf = is_bf(x);
  TORCH_CHECK(x.dim() == 2 && w.dim() == 2 && w.is_cuda() && w.is_contiguous() && is_bf(w) == bf && w.size(1) == x.size(1),
              "causal_conv: x [T, C], w [taps, C] of one dtype");
  const int64_t T = x.size(0), C = x.size(1), taps = w.size(0), S = seq_lens.numel();
  TORCH_CHECK(out.is_cuda() && out.is_contiguous() && out.dim() == 2 && out.size(0) == T && out.size(1) == C &&
              is_bf(out) == bf, "out: contiguous [T, C]");
  float* sp = f32(state, "state");
  TORCH_CHECK(state.dim() == 2 && off >= 0 && off + (taps - 1) * C <= state.size(1), "state slot too small for this filter");
  mxs::launch_causal_conv(out.data_ptr(), mat(x, bf, T, C, "x"), x.stride(0), w.data_ptr(), vec(bias, bf, C, "bias"), sp,
                          state.stride(0), i32(state_rows, S, "state_rows"), off, i32(qsl, S + 1, "qsl"),
                          i32(seq_lens, S, "seq_lens"), static_cast<int>(S), static_cast<int>(T), static_cast<int>(C),
                          static_cast<int>(taps), silu ? 1 : 0, bf, stream());
}

void gated_norm(at::Tensor out, at::Tensor o, at::Tensor gate, at::Tensor w, double eps, int64_t groups, bool silu,
                bool gate_first, double scale) {
  const float* opn = f32(o, "o");
  TORCH_CHECK(o.dim() == 2, "o: [T, N]");
  const int64_t T = o.size(0), N = o.size(1), wn = w.numel();
  const bool bf = is_bf(out);
  TORCH_CHECK(groups >= 1 && N % groups == 0 && wn >= 1 && N % wn == 0, "groups and the weight's length must divide N");
  mxs::launch_gated_norm(const_cast<void*>(mat(out, bf, T, N, "out")), out.stride(0), opn, mat(gate, bf, T, N, "gate"),
                         gate.stride(0), vec(OptT(w), bf, wn, "w"), static_cast<int>(wn), static_cast<int>(T),
                         static_cast<int>(N), static_cast<int>(groups), static_cast<float>(eps), silu ? 1 : 0,
                         gate_first ? 1 : 0, static_cast<float>(scale), bf, stream());
}

void column_scan(bool delta, at::Tensor out, at::Tensor q, at::Tensor k, at::Tensor v, at::Tensor beta, OptT a,
                 at::Tensor dt_bias, at::Tensor A_log, OptT D, at::Tensor state, at::Tensor state_rows, int64_t off,
                 at::Tensor qsl, at::Tensor seq_lens, int64_t H, int64_t G, int64_t dk, int64_t dv, double q_scale,
                 double unit_eps, int64_t piece = 1, int64_t npieces = 1, OptT sc_local = OptT(), OptT sc_start = OptT(),
                 OptT sc_decay = OptT(), int64_t mode = 0, int64_t max_q = 0) {
  const bool bf = is_bf(q);
  const int64_t T = q.size(0), S = seq_lens.numel();
  TORCH_CHECK(G >= 1 && H % G == 0, "heads must divide over the q/k heads (groups)");
  mxs::ScanArgs p{};
  p.out = f32(out, "out");
  TORCH_CHECK(out.dim() == 2 && out.size(0) == T && out.size(1) == H * dv, "out: fp32 [T, H*dv]");
  p.q = mat(q, bf, T, G * dk, "q");
  p.q_stride = q.stride(0);
  p.k = mat(k, bf, T, G * dk, "k");
  p.k_stride = k.stride(0);
  p.v = mat(v, bf, T, H * dv, "v");
  p.v_stride = v.stride(0);
  p.beta = mat(beta, bf, T, H, "beta");
  p.beta_stride = beta.stride(0);
  if (delta) {
    TORCH_CHECK(a.has_value(), "the delta rule needs its decay pre-activations");
    p.a = mat(*a, bf, T, H * dk, "a");
    p.a_stride = a->stride(0);
  } else {
    TORCH_CHECK(D.has_value(), "the state-space scan needs D");
  }
  p.dt_bias = f32n(OptT(dt_bias), delta ? H * dk : H, "dt_bias");
  p.A_log = f32n(OptT(A_log), H, "A_log");
  p.D = f32n(D, H, "D");
  p.state = f32(state, "state");
  TORCH_CHECK(state.dim() == 2 && off >= 0 && off + H * dk * dv <= state.size(1), "state slot too small for this layer");
  p.state_stride = state.stride(0);
  p.state_rows = i32(state_rows, S, "state_rows");
  p.off = off;
  p.qsl = i32(qsl, S + 1, "qsl");
  p.seq_lens = i32(seq_lens, S, "seq_lens");
  p.n_rows = static_cast<int>(T);
  p.H = static_cast<int>(H);
  p.G = static_cast<int>(G);
  p.dk = static_cast<int>(dk);
  p.dv = static_cast<int>(dv);
  p.q_scale = static_cast<float>(q_scale);
  p.unit_eps = static_cast<float>(unit_eps);
  p.piece = 1;
  p.npieces = 1;
  p.max_q = (max_q == 1 && T == S) ? 1 : 0;  // every sequence brings one row
  if (npieces > 1) {  // pieces side by side: scratch [S, npieces, state] twice and [S, npieces, H]
    TORCH_CHECK(piece >= 16 && sc_local.has_value() && sc_start.has_value() && (delta || sc_decay.has_value()),
                "a split scan needs its scratch pools");
    TORCH_CHECK(sc_local->numel() >= S * npieces * H * dk * (delta ? dv + dk : dv) &&
                sc_start->numel() >= S * npieces * H * dk * dv && (delta || sc_decay->numel() >= S * npieces * H),
                "scratch pools smaller than [S, npieces, state]");
    TORCH_CHECK(!delta || mode == 1 || mode == 2, "a split delta-rule scan is launched pass by pass");
    p.piece = static_cast<int>(piece);
    p.npieces = static_cast<int>(npieces);
    p.mode = static_cast<int>(mode);
    p.sc_local = f32(*sc_local, "sc_local");
    p.sc_start = f32(*sc_start, "sc_start");
    p.sc_decay = delta ? nullptr : f32(*sc_decay, "sc_decay");
  }
  TORCH_CHECK(mxs::launch_column_scan(p, static_cast<int>(S), delta, bf, stream()), "column scan: key / state size beyond 256");
}

void ssd_scan(at::Tensor out, at::Tensor x, at::Tensor B, at::Tensor C, at::Tensor dt, at::Tensor dt_bias, at::Tensor A_log,
              at::Tensor D, at::Tensor state, at::Tensor state_rows, int64_t off, at::Tensor qsl, at::Tensor seq_lens,
              int64_t H, int64_t G, int64_t N, int64_t P, int64_t piece, int64_t npieces, OptT sc_local, OptT sc_start,
              OptT sc_decay, int64_t max_q) {
  column_scan(false, out, C, B, x, dt, OptT(), dt_bias, A_log, OptT(D), state, state_rows, off, qsl, seq_lens, H, G, N, P,
              1.0, 0.0, piece, npieces, sc_local, sc_start, sc_decay, 0, max_q);
}

void delta_scan(at::Tensor out, at::Tensor q, at::Tensor k, at::Tensor v, at::Tensor beta, at::Tensor a, at::Tensor dt_bias,
                at::Tensor A_log, at::Tensor state, at::Tensor state_rows, int64_t off, at::Tensor qsl, at::Tensor seq_lens,
                int64_t H, int64_t G, int64_t dk, int64_t dv, double q_scale, double unit_eps, int64_t mode, int64_t piece,
                int64_t npieces, OptT sc_local, OptT sc_start, int64_t max_q) {
  column_scan(true, out, q, k, v, beta, OptT(a), dt_bias, A_log, OptT(), state, state_rows, off, qsl, seq_lens, H, G, dk, dv,
              q_scale, unit_eps, piece, npieces, sc_local, sc_start, OptT(), mode, max_q);
}

// ---- latent attention, routed experts (latent_experts.hip)
const int64_t* i64c(const at::Tensor& t, int64_t n, const char* name) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == at::kLong && t.is_contiguous() && t.numel() == n, name,
              ": expected ", n, " contiguous int64");
  return t.data_ptr<int64_t>();
}

void latent_prep(at::Tensor cq, at::Tensor dq, at::Tensor dkv, at::Tensor positions, at::Tensor slots, at::Tensor cache,
                 int64_t koff, int64_t rank, int64_t bs, at::Tensor freqs, at::Tensor q_norm, at::Tensor kv_norm,
                 double eps, bool split_pairs) {
  const bool bf = is_bf(dq);
  const int64_t T = dq.size(0), qr = dq.size(1), nf = freqs.numel(), dk = rank + 2 * nf;
  TORCH_CHECK(rank >= 1 && bs >= 1, "rank and block size must be positive");
  check_cache(cache, bf, koff, koff, 1, dk, 0, bs);
  TORCH_CHECK(cq.is_cuda() && cq.is_contiguous() && cq.dim() == 2 && cq.size(0) == T && cq.size(1) == qr && is_bf(cq) == bf,
              "cq: contiguous [T, q_rank]");
  mxs::launch_latent_prep(cq.data_ptr(), mat(dq, bf, T, qr, "dq"), dq.stride(0), mat(dkv, bf, T, dk, "dkv"), dkv.stride(0),
                          i64c(positions, T, "positions"), i64c(slots, T, "slot_mapping"), cache.data_ptr(), cache.stride(0),
                          static_cast<int>(T), static_cast<int>(koff), static_cast<int>(qr), static_cast<int>(rank),
                          static_cast<int>(nf), static_cast<int>(bs), f32(freqs, "freqs"),
                          vec(OptT(q_norm), bf, qr, "q_norm"), vec(OptT(kv_norm), bf, rank, "kv_norm"),
                          static_cast<float>(eps), split_pairs, bf, stream());
}

// The matrix-core latent attention (bf16).  Returns false when the sizes are not the kernel's: nothing
// was launched and the caller runs window_attention with strided value rows instead.
bool latent_attention(at::Tensor out, at::Tensor q, at::Tensor cache, at::Tensor block_tables, at::Tensor qsl,
                      at::Tensor seq_lens, int64_t koff, int64_t H, int64_t dk, int64_t rank, int64_t bs, double scale,
                      int64_t max_query_len, OptT sink, int64_t nsplit, OptT part, bool pair, int64_t window) {
  if (!is_bf(q)) return false;
  TORCH_CHECK(window >= 0 && window < (1LL << 30), "window out of range");
  const float* sinkp = nullptr;
  if (sink.has_value()) {
    sinkp = f32(*sink, "sink");
    TORCH_CHECK(sink->numel() == H, "sink: fp32 [H]");
  }
  const int64_t T = q.size(0), S = seq_lens.numel();
  TORCH_CHECK(rank >= 1 && rank <= dk && H >= 1, "1 <= rank <= dk");
  check_cache(cache, true, koff, koff, 1, dk, 0, bs);
  TORCH_CHECK(out.is_cuda() && out.is_contiguous() && out.dim() == 2 && out.size(0) == T && out.size(1) == H * rank &&
              is_bf(out), "out: bf16 [T, H*rank]");
  TORCH_CHECK(block_tables.is_cuda() && block_tables.scalar_type() == at::kInt && block_tables.dim() == 2 &&
              block_tables.size(0) >= S && block_tables.stride(1) == 1, "block_tables: int32 [S, max_blocks]");
  float* pp = nullptr;
  if (nsplit > 1) {
    TORCH_CHECK(part.has_value() && part->numel() >= T * H * nsplit * (rank + 4), "part: fp32 [T*H, nsplit, rank + 4]");
    pp = f32(*part, "part");
  }
  return mxs::launch_latent_attention(
      out.data_ptr(), pp, mat(q, true, T, H * dk, "q"), q.stride(0), cache.data_ptr(), cache.stride(0),
      block_tables.data_ptr<int>(), static_cast<int>(block_tables.stride(0)), i32(qsl, S + 1, "qsl"),
      i32(seq_lens, S, "seq_lens"), static_cast<int>(S), static_cast<int>(T), static_cast<int>(koff), static_cast<int>(H),
      static_cast<int>(dk), static_cast<int>(rank), static_cast<int>(bs), static_cast<float>(scale),
      static_cast<int>(std::max<int64_t>(1, std::min<int64_t>(max_query_len, T))), sinkp, static_cast<int>(nsplit), pair,
      static_cast<int>(window), stream());
}

void rope_half_into(at::Tensor out, at::Tensor x, at::Tensor positions, int64_t heads, int64_t x_dim, int64_t x_col,
                    int64_t out_dim, int64_t out_col, at::Tensor freqs, bool split_pairs) {
  const bool bf = is_bf(x);
  const int64_t T = x.size(0), nf = freqs.numel();
  TORCH_CHECK(x_col >= 0 && out_col >= 0 && x_col + 2 * nf <= x_dim && out_col + 2 * nf <= out_dim,
              "the rotated columns lie outside a head");
  mxs::launch_rope_half_into(const_cast<void*>(mat(out, bf, T, heads * out_dim, "out")), out.stride(0),
                             mat(x, bf, T, heads * x_dim, "x"), x.stride(0), i64c(positions, T, "positions"),
                             static_cast<int>(T), static_cast<int>(heads), static_cast<int>(x_dim), static_cast<int>(x_col),
                             static_cast<int>(out_dim), static_cast<int>(out_col), f32(freqs, "freqs"), static_cast<int>(nf),
                             split_pairs, bf, stream());
}

void route_topk(at::Tensor w, at::Tensor ids, at::Tensor logits, bool renorm, bool softmax) {
  const float* lp = f32(logits, "logits");
  TORCH_CHECK(logits.dim() == 2 && w.dim() == 2 && ids.dim() == 2, "logits [T, E], w / ids [T, k]");
  const int64_t T = logits.size(0), E = logits.size(1), k = w.size(1);
  TORCH_CHECK(k >= 1 && k <= E && w.size(0) == T && ids.size(0) == T && ids.size(1) == k, "1 <= k <= E; w, ids [T, k]");
  TORCH_CHECK(ids.is_cuda() && ids.scalar_type() == at::kInt && ids.is_contiguous(), "ids: contiguous int32");
  mxs::launch_route_topk(f32(w, "w"), ids.data_ptr<int>(), lp, static_cast<int>(T), static_cast<int>(E),
                         static_cast<int>(k), renorm, softmax, stream());
}

void capped_glu(at::Tensor out, at::Tensor gu, double limit, double alpha) {
  const bool bf = is_bf(gu);
  TORCH_CHECK(gu.is_cuda() && gu.dim() == 2 && gu.size(1) % 2 == 0 && (gu.size(1) == 1 || gu.stride(1) == 1), "gu: [R, 2F]");
  const int64_t R = gu.size(0), F = gu.size(1) / 2;
  TORCH_CHECK(out.is_cuda() && out.is_contiguous() && out.dim() == 2 && out.size(0) == R && out.size(1) == F &&
              is_bf(out) == bf, "out: contiguous [R, F]");
  mxs::launch_capped_glu(out.data_ptr(), gu.data_ptr(), gu.stride(0), static_cast<int>(R), static_cast<int>(F),
                         static_cast<float>(limit), static_cast<float>(alpha), bf, stream());
}

void expert_align(at::Tensor offs, at::Tensor inv, at::Tensor ids, int64_t E) {
  const int64_t n = ids.numel();
  TORCH_CHECK(ids.is_cuda() && ids.scalar_type() == at::kInt && ids.is_contiguous(), "ids: contiguous int32");
  TORCH_CHECK(E >= 1 && n < (1LL << 30), "expert count / pair count out of range");
  int* op = const_cast<int*>(i32(offs, E + 1, "offs"));
  int* ip = const_cast<int*>(i32(inv, n, "inv"));
  TORCH_CHECK(mxs::launch_expert_align(op, ip, ids.data_ptr<int>(), static_cast<int>(n), static_cast<int>(E), stream()),
              "expert_align: more experts than the kernel's counters hold");
}

void gather_scaled(at::Tensor xs, at::Tensor h, OptT w, at::Tensor inv, int64_t k) {
  const bool bf = is_bf(h);
  TORCH_CHECK(h.dim() == 2 && k >= 1, "h [T, W], k >= 1");
  const int64_t T = h.size(0), W = h.size(1);
  const float* wp = nullptr;
  if (w.has_value()) {
    TORCH_CHECK(w->dim() == 2 && w->size(0) == T && w->size(1) == k, "w [T, k]");
    wp = f32(*w, "w");
  }
  TORCH_CHECK(xs.is_cuda() && xs.is_contiguous() && xs.dim() == 2 && xs.size(0) == T * k && xs.size(1) == W &&
              is_bf(xs) == bf, "xs: contiguous [T*k, W]");
  // inv comes from expert_align over the same pairs: a permutation of 0 .. T*k-1
  mxs::launch_gather_scaled(xs.data_ptr(), mat(h, bf, T, W, "h"), h.stride(0), wp, i32(inv, T * k, "inv"),
                            static_cast<int>(T * k), static_cast<int>(k), static_cast<int>(W), bf, stream());
}

void spread_scaled(at::Tensor xs, at::Tensor h, OptT w, at::Tensor ids) {
  const bool bf = is_bf(h);
  TORCH_CHECK(ids.dim() == 2 && h.dim() == 2 && ids.size(0) == h.size(0) && xs.dim() == 3, "h [T, W], ids [T, k], xs [E, T, W]");
  const int64_t T = h.size(0), W = h.size(1), k = ids.size(1), E = xs.size(0);
  const float* wp = nullptr;
  if (w.has_value()) {
    TORCH_CHECK(w->dim() == 2 && w->size(0) == T && w->size(1) == k, "w [T, k]");
    wp = f32(*w, "w");
  }
  TORCH_CHECK(xs.is_cuda() && xs.is_contiguous() && xs.size(1) == T && xs.size(2) == W && is_bf(xs) == bf,
              "xs: contiguous [E, T, W]");
  TORCH_CHECK(E <= 65535, "more experts than a grid dimension holds");
  mxs::launch_spread_scaled(xs.data_ptr(), mat(h, bf, T, W, "h"), h.stride(0), wp, i32(ids, T * k, "ids"),
                            static_cast<int>(T), static_cast<int>(E), static_cast<int>(k), static_cast<int>(W), bf,
                            stream());
}

void expert_combine(at::Tensor out, at::Tensor ys, OptT index, int64_t k, OptT extra, int64_t row_stride, OptT weights,
                    bool by_expert) {
  const bool bf = is_bf(ys);
  TORCH_CHECK(ys.is_cuda() && ys.is_contiguous() && ys.dim() == 2 && out.is_cuda() && out.is_contiguous() &&
              out.dim() == 2 && out.size(1) == ys.size(1) && is_bf(out) == bf, "ys [R, W], out [T, W]");
  const int64_t T = out.size(0), W = out.size(1), R = ys.size(0);
  const int* ip = nullptr;
  if (index.has_value()) {
    ip = i32(*index, T * k, "index");  // entries are rows of ys: expert_align's places (< T*k), or expert * T + t (< R)
    TORCH_CHECK(T * k <= R, "index reaches past ys");
    // by_expert: entries are experts (route_topk's ids, < R / row_stride) of an [E, row_stride, W] stack
    TORCH_CHECK(!by_expert || (row_stride >= T && R % row_stride == 0), "by_expert: ys is [E, row_stride, W]");
  } else {
    TORCH_CHECK(k >= 1 && row_stride >= T && (k - 1) * row_stride + T <= R, "the k slabs reach past ys");
  }
  const void* ep = extra.has_value() ? mat(*extra, bf, T, W, "extra") : nullptr;
  const float* wp = nullptr;
  if (weights.has_value()) {
    TORCH_CHECK(weights->numel() == T * k, "weights: fp32 [T, k]");
    wp = f32(*weights, "weights");
  }
  mxs::launch_expert_combine(out.data_ptr(), ys.data_ptr(), ip, static_cast<int>(T), static_cast<int>(k), row_stride, ep,
                             extra.has_value() ? extra->stride(0) : 0, static_cast<int>(W), wp, by_expert && index.has_value(), bf,
                             stream());
}

void embed_normed(at::Tensor out, OptT copy, OptT h, at::Tensor ids, at::Tensor table, at::Tensor w, double eps,
                  double w_offset) {
  float* op = f32(out, "out");
  float* cp = nullptr;
  if (copy.has_value()) {
    cp = f32(*copy, "copy");
    TORCH_CHECK(copy->sizes() == out.sizes(), "copy: fp32 [T, W] like out");
  }
  TORCH_CHECK(table.is_cuda() && table.dim() == 2 && table.is_contiguous(), "table: contiguous [vocab, W]");
  const bool bf = is_bf(table);
  const int64_t T = ids.numel(), W = table.size(1);
  TORCH_CHECK(out.dim() == 2 && out.size(0) == T && out.size(1) == W, "out: fp32 [T, W]");
  void* hp = nullptr;
  if (h.has_value()) {
    TORCH_CHECK(h->is_cuda() && h->is_contiguous() && h->dim() == 2 && h->size(0) == T && h->size(1) == W && is_bf(*h) == bf,
                "h: contiguous [T, W] of the table's dtype");
    hp = h->data_ptr();
  }
  mxs::launch_embed_normed(op, cp, hp, i64c(ids, T, "ids"), table.data_ptr(), vec(OptT(w), bf, W, "w"), static_cast<int>(T),
                           static_cast<int>(W), table.size(0), static_cast<float>(eps), static_cast<float>(w_offset), bf,
                           stream());
}

void depth_mix(at::Tensor hist, int64_t n, at::Tensor coeffs, OptT h) {
  float* hp = f32(hist, "hist");
  TORCH_CHECK(hist.dim() == 3 && n >= 1 && n < hist.size(0), "hist: fp32 [L, T, W], 1 <= n < L");
  const int64_t T = hist.size(1), W = hist.size(2);
  const float* cp = f32(coeffs, "coeffs");
  TORCH_CHECK(coeffs.numel() == n, "coeffs: fp32 [n]");
  void* op = nullptr;
  bool bf = false;
  if (h.has_value()) {
    TORCH_CHECK(h->is_cuda() && h->is_contiguous() && h->dim() == 2 && h->size(0) == T && h->size(1) == W, "h: contiguous [T, W]");
    bf = is_bf(*h);
    op = h->data_ptr();
  }
  TORCH_CHECK(mxs::launch_depth_mix(hp, T * W, static_cast<int>(n), cp, op, static_cast<int>(T), static_cast<int>(W), bf,
                                    stream()), "depth_mix: more slabs than the kernel's coefficient table holds");
}

void xielu(at::Tensor out, at::Tensor x, at::Tensor ab) {
  TORCH_CHECK(x.is_cuda() && x.is_contiguous() && out.is_cuda() && out.is_contiguous() && out.numel() == x.numel() &&
              out.scalar_type() == x.scalar_type(), "xielu: contiguous tensors of one dtype");
  const float* ap = f32(ab, "ab");
  TORCH_CHECK(ab.numel() == 2, "ab: fp32 [2]");
  mxs::launch_xielu(out.data_ptr(), x.data_ptr(), x.numel(), ap, is_bf(x), stream());
}

// Biases, q / k norms (norm_whole: one over all of a row's heads), rotary turn, q in place, k and v into the pages.
void qkv_prep_cache(at::Tensor q, OptT k, OptT v, at::Tensor positions, at::Tensor slots, at::Tensor cache, int64_t koff,
                    int64_t voff, int64_t H, int64_t G, int64_t dk, int64_t dv, int64_t bs, at::Tensor freqs, double mag,
                    bool split_pairs, OptT bq, OptT bk, OptT bv, OptT q_norm, OptT k_norm, double eps, bool norm_whole) {
  const bool bf = is_bf(q);
  const int64_t T = q.size(0);
  TORCH_CHECK(k.has_value() == v.has_value(), "k and v go together");
  TORCH_CHECK(H >= 1 && G >= 1 && H <= 4096 && G <= 4096 && dk >= 1 && bs >= 1, "head counts / sizes out of range");
  const void *kp = nullptr, *vp = nullptr;
  if (k.has_value()) {
    check_cache(cache, bf, koff, voff, G, dk, dv, bs);
    kp = mat(*k, bf, T, G * dk, "k");
    vp = mat(*v, bf, T, G * dv, "v");
  }
  const int64_t nf = freqs.numel();
  TORCH_CHECK(2 * nf <= dk, "more rotary pairs than the head has dimensions");
  const int64_t nq = norm_whole ? H * dk : dk, nk = norm_whole ? G * dk : dk;
  mxs::launch_qkv_prep_cache(const_cast<void*>(mat(q, bf, T, H * dk, "q")), q.stride(0), kp, k.has_value() ? k->stride(0) : 0,
                             vp, v.has_value() ? v->stride(0) : 0, i64c(positions, T, "positions"),
                             i64c(slots, T, "slot_mapping"), cache.data_ptr(), cache.stride(0), static_cast<int>(T),
                             static_cast<int>(koff), static_cast<int>(voff), static_cast<int>(H), static_cast<int>(G),
                             static_cast<int>(dk), static_cast<int>(dv), static_cast<int>(bs), f32(freqs, "freqs"),
                             static_cast<int>(nf), static_cast<float>(mag), split_pairs, vec(bq, bf, H * dk, "bias_q"),
                             vec(bk, bf, G * dk, "bias_k"), vec(bv, bf, G * dv, "bias_v"), vec(q_norm, bf, nq, "q_norm"),
                             vec(k_norm, bf, nk, "k_norm"), static_cast<float>(eps), norm_whole ? 2 : 1, bf, stream());
}

void talking_attention(at::Tensor out, at::Tensor q, at::Tensor cache, at::Tensor block_tables, at::Tensor qsl,
                       at::Tensor seq_lens, int64_t koff, int64_t voff, int64_t H, int64_t G, int64_t dk, int64_t dv,
                       int64_t bs, double scale, int64_t window, int64_t keep, int64_t max_query_len, OptT sink,
                       at::Tensor talk, int64_t nsplit, OptT part) {
  const bool bf = is_bf(q);
  const float* sinkp = nullptr;
  if (sink.has_value()) {
    sinkp = f32(*sink, "sink");
    TORCH_CHECK(sink->numel() == H, "sink: fp32 [H]");
  }
  const float* tp = f32(talk, "talk");
  TORCH_CHECK(talk.numel() == H * H, "talk: fp32 [H, H]");
  const int64_t T = q.size(0), S = seq_lens.numel();
  check_cache(cache, bf, koff, voff, G, dk, dv, bs);
  TORCH_CHECK(G >= 1 && H % G == 0, "query heads must divide over kv heads");
  TORCH_CHECK(out.is_cuda() && out.is_contiguous() && out.dim() == 2 && out.size(0) == T && out.size(1) == H * dv &&
              is_bf(out) == bf, "out: [T, H*dv]");
  TORCH_CHECK(block_tables.is_cuda() && block_tables.scalar_type() == at::kInt && block_tables.dim() == 2 &&
              block_tables.size(0) >= S && block_tables.stride(1) == 1, "block_tables: int32 [S, max_blocks]");
  float* pp = nullptr;
  TORCH_CHECK(nsplit >= 1 && nsplit <= 64, "1 <= nsplit <= 64");
  if (nsplit > 1) {
    TORCH_CHECK(part.has_value() && part->numel() >= T * H * nsplit * (dv + 4), "part: fp32 [T*H, nsplit, dv + 4]");
    pp = f32(*part, "part");
  }
  const bool ok = mxs::launch_talking_attention(
      out.data_ptr(), mat(q, bf, T, H * dk, "q"), q.stride(0), cache.data_ptr(), cache.stride(0),
      block_tables.data_ptr<int>(), static_cast<int>(block_tables.stride(0)), i32(qsl, S + 1, "qsl"),
      i32(seq_lens, S, "seq_lens"), static_cast<int>(S), static_cast<int>(T), static_cast<int>(koff),
      static_cast<int>(voff), static_cast<int>(H), static_cast<int>(G), static_cast<int>(dk), static_cast<int>(dv),
      static_cast<int>(bs), static_cast<float>(scale), static_cast<int>(window), static_cast<int>(keep),
      static_cast<int>(std::max<int64_t>(1, std::min<int64_t>(max_query_len, T))), sinkp, tp, pp, static_cast<int>(nsplit), bf,
      stream());
  TORCH_CHECK(ok, "talking_attention: more heads or wider heads than the kernel's LDS tables hold, or a split the sizes do not take");
}

}  // namespace

PYBIND11_MODULE(_M, m) {
  m.def("resid_update", &resid_update);
  m.def("cast_into", &cast_into);
  m.def("relu_sq", &relu_sq);
  m.def("softcap", &softcap);
  m.def("gated_rms_norm", &gated_rms_norm);
  m.def("gate_linear", &gate_linear);
  m.def("kv_write", &kv_write);
  m.def("window_attention", &window_attention);
  m.def("decay_scan", &decay_scan);
  m.def("mlstm_scan", &mlstm_scan);
  m.def("embed_scaled", &embed_scaled);
  m.def("silu_mul", &silu_mul);
  m.def("rope_qkv_cache", &rope_qkv_cache);
  m.def("rope_rows", &rope_rows);
  m.def("causal_conv", &causal_conv);
  m.def("gated_norm", &gated_norm);
  m.def("ssd_scan", &ssd_scan);
  m.def("delta_scan", &delta_scan);
  m.def("latent_prep", &latent_prep);
  m.def("rope_half_into", &rope_half_into);
  m.def("latent_attention", &latent_attention);
  m.def("route_topk", &route_topk);
  m.def("capped_glu", &capped_glu);
  m.def("expert_align", &expert_align);
  m.def("gather_scaled", &gather_scaled);
  m.def("spread_scaled", &spread_scaled);
  m.def("expert_combine", &expert_combine);
  m.def("embed_normed", &embed_normed);
  m.def("depth_mix", &depth_mix);
  m.def("xielu", &xielu);
  m.def("qkv_prep_cache", &qkv_prep_cache);
  m.def("talking_attention", &talking_attention);
}
