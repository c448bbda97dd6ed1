"""Sequence-mixer ops beyond rotary softmax attention: a 32-bit residual stream with fused norms,
paged attention with a sliding window and kept first tokens, decayed linear attention, the mLSTM
matrix memory, gated output norms, squared ReLU and logit soft-capping.

Like mxserve.ops: GPU tensors run the gfx950 kernels of the in-tree extension `mxserve/_M*.so`
(csrc/mixers/*.hip, activations bf16 or fp32; built by `python setup_ext.py --only M` or on first
use), CPU tensors the PyTorch forms below.  Everything the recurrences touch is fp32: the state
pools, decays, gates, scores and the residual stream.

Batch layout (shared with the attention ops): sequence s owns rows qsl[s]:qsl[s+1] of a step's
flattened tokens; they are the LAST rows of its seq_lens[s] tokens.  A sequence whose first row is
position 0 starts from a zero state, whatever its slot held before.

Paged cache of one attention layer inside the block-major pool `cache` [num_blocks, block_elems]:
K at `koff` as [Hkv, BS, dk], V at `voff` as [Hkv, BS, dv], both token-major.
Recurrent state of one layer inside the slot pool `state` [slots, state_floats] (fp32): decayed
linear attention S [H, dk, dv] at `off`; mLSTM S [H, dk, dv], then n [H, dk], then m [H]; the
column scans (state-space duality, gated delta rule) S transposed [H, dv, dk], so that the rows a
lane owns are contiguous; a short causal convolution its last taps - 1 inputs [taps - 1, channels].
"""
from __future__ import annotations

import importlib
import os
import threading
from typing import Optional

import torch
import torch.nn.functional as F

_EXT = None
_LOCK = threading.Lock()


def ext():
    """The mixer kernels' extension; built in-tree on first use when it is missing (hipcc)."""
    global _EXT
    if _EXT is None:
        with _LOCK:
            if _EXT is None:
                try:
                    _EXT = importlib.import_module("mxserve._M")
                except ImportError:
                    import sys
                    root = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
                    if root not in sys.path:
                        sys.path.insert(0, root)
                    import setup_ext
                    setup_ext.build_M()
                    importlib.invalidate_caches()
                    _EXT = importlib.import_module("mxserve._M")
    return _EXT


def _gpu(t: torch.Tensor) -> bool:
    return t.is_cuda and os.environ.get("MXS_FORCE_REFERENCE_OPS", "0") != "1"


def _rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)


# ----------------------------------------------------------------------------- residual stream
def resid_update(x: torch.Tensor, a: Optional[torch.Tensor], eps: float, *, wa: Optional[torch.Tensor] = None,
                 b: Optional[torch.Tensor] = None, wb: Optional[torch.Tensor] = None,
                 bias: Optional[torch.Tensor] = None, assign: bool = False,
                 norm_w: Optional[torch.Tensor] = None, out_dtype: Optional[torch.dtype] = None,
                 a_scale: float = 1.0, w_offset: float = 0.0, wa_offset: float = 0.0,
                 cast_dtype: Optional[torch.dtype] = None):
    """One pass over the fp32 residual stream x [T, W], in place:
        d = a * a_scale            (wa: RMSNorm(a) * (wa_offset + wa))
        d = (d + RMSNorm(b) * wb) / 2      when b is given (two branches, each normed over the width)
        d += bias                  (a [W] vector)
        x = d if assign else x + d
    and, when norm_w is given, returns RMSNorm(x) * (w_offset + norm_w) in out_dtype (the next
    sublayer's input; w_offset = 1 for weights stored as their difference from one, added in fp32).
    Without norm_w, cast_dtype asks for the updated x itself in that dtype (a next sublayer that
    reads the stream un-normed).  a = None leaves x as it is.  All sums and norms in fp32."""
    if _gpu(x):
        h = None
        if norm_w is not None:
            h = torch.empty(x.shape, dtype=out_dtype or norm_w.dtype, device=x.device)
        elif cast_dtype is not None:
            h = torch.empty(x.shape, dtype=cast_dtype, device=x.device)
        ext().resid_update(x, a, wa, b, wb, bias, bool(assign), norm_w, h, float(eps), float(a_scale), float(w_offset),
                           float(wa_offset))
        return h
    if a is not None:
        d = a.float() * a_scale if a_scale != 1.0 else a.float()
        if wa is not None:
            d = _rms(d, eps) * (wa.float() + wa_offset if wa_offset else wa.float())
        if b is not None:
            d = 0.5 * (d + _rms(b.float(), eps) * wb.float())
        if bias is not None:
            d = d + bias.float()
        if assign:
            x.copy_(d)
        else:
            x.add_(d)
    if norm_w is None:
        return None if cast_dtype is None else x.to(cast_dtype, copy=True)
    return (_rms(x, eps) * (norm_w.float() + w_offset if w_offset else norm_w.float())).to(out_dtype or norm_w.dtype)


def embed_normed(ids: torch.Tensor, table: torch.Tensor, w: torch.Tensor, eps: float, w_offset: float,
                 out: torch.Tensor, cast_dtype: Optional[torch.dtype] = None, copy: Optional[torch.Tensor] = None):
    """out (fp32 [T, W], may be one slab of a larger buffer) = RMSNorm(table[ids]) * (w_offset + w): an
    embedding that is normed before it becomes the stream; `copy` receives the same (a second slab that a
    layer then updates in place).  Returns out in cast_dtype when asked."""
    if _gpu(table):
        h = torch.empty(out.shape, dtype=cast_dtype, device=out.device) if cast_dtype is not None else None
        ext().embed_normed(out, copy, h, ids, table, w, float(eps), float(w_offset))
        return h
    out.copy_(_rms(F.embedding(ids, table).float(), eps) * (w.float() + w_offset))
    if copy is not None:
        copy.copy_(out)
    return None if cast_dtype is None else out.to(cast_dtype, copy=True)


def depth_mix(hist: torch.Tensor, n: int, coeffs: torch.Tensor, cast_dtype: Optional[torch.dtype] = None):
    """hist fp32 [L, T, W]: slab n <- sum over j < n of coeffs[j] * slab j (coeffs fp32 [n]): a stream
    that goes on as a weighted sum of everything earlier layers produced.  Returns the new slab in
    cast_dtype when asked.  fp32 products and sums, in the order of j."""
    if not 0 < n < hist.shape[0] or coeffs.numel() != n:
        raise ValueError(f"depth_mix: slab {n} of {hist.shape[0]} with {coeffs.numel()} coefficients")
    if _gpu(hist):
        h = torch.empty(hist.shape[1:], dtype=cast_dtype, device=hist.device) if cast_dtype is not None else None
        ext().depth_mix(hist, int(n), coeffs, h)
        return h
    acc = hist[0] * coeffs[0]
    for j in range(1, n):
        acc = acc + hist[j] * coeffs[j]
    hist[n].copy_(acc)
    return None if cast_dtype is None else hist[n].to(cast_dtype, copy=True)


def cast_into(dst: torch.Tensor, x: torch.Tensor) -> None:
    """dst[:, :W] = x (fp32 -> dst's dtype); dst may be a wider row-strided buffer."""
    if _gpu(x):
        ext().cast_into(dst, x)
    else:
        dst[:, :x.shape[1]].copy_(x)


def relu_sq(x: torch.Tensor) -> torch.Tensor:
    """max(x, 0)^2, computed in fp32."""
    if _gpu(x):
        out = torch.empty_like(x)
        ext().relu_sq(out, x)
        return out
    return F.relu(x.float()).square().to(x.dtype)


def xielu(x: torch.Tensor, ab: torch.Tensor) -> torch.Tensor:
    """ab fp32 [2] = (a, b), both positive:  z > 0: a z^2 + z / 2;  z <= 0: b (e^z - 1 - z) + z / 2.
    Computed in fp32."""
    if _gpu(x):
        out = torch.empty_like(x)
        ext().xielu(out, x, ab)
        return out
    z = x.float()
    zn = z.clamp(max=0.0)
    return torch.where(z > 0, ab[0] * z * z + 0.5 * z, ab[1] * (torch.expm1(zn) - zn) + 0.5 * z).to(x.dtype)


def softcap(x: torch.Tensor, cap: float) -> torch.Tensor:
    """cap * tanh(x / cap) as fp32 (cap <= 0: a plain fp32 copy)."""
    if _gpu(x):
        out = torch.empty(x.shape, dtype=torch.float32, device=x.device)
        ext().softcap(out, x, float(cap))
        return out
    xf = x.float()
    return cap * torch.tanh(xf / cap) if cap > 0 else xf


def gated_rms_norm(o: torch.Tensor, gate: torch.Tensor, w: torch.Tensor, eps: float, groups: int,
                   out_dtype: torch.dtype) -> torch.Tensor:
    """RMSNorm(o) * w * sigmoid(gate).  o fp32 [T, N]; the norm runs over each of `groups` equal
    slices of a row (1: the whole row; H: per head).  gate [T, N] may be a row-strided view."""
    if _gpu(o):
        out = torch.empty(o.shape, dtype=out_dtype, device=o.device)
        ext().gated_rms_norm(out, o, gate, w, float(eps), int(groups))
        return out
    T, N = o.shape
    y = _rms(o.view(T, groups, N // groups), eps).reshape(T, N)
    return (y * w.float() * torch.sigmoid(gate.float())).to(out_dtype)


def gate_linear(h: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor]) -> torch.Tensor:
    """fp32 h @ w.T + bias for a handful of output columns (recurrence gates): inputs of any float
    dtype, products and sums in fp32, fp32 out."""
    if _gpu(h):
        out = torch.empty(h.shape[0], w.shape[0], dtype=torch.float32, device=h.device)
        ext().gate_linear(out, h, w, bias)
        return out
    return F.linear(h.float(), w.float(), None if bias is None else bias.float())


# ----------------------------------------------------------------------------- windowed attention
TALK_TARGET_GROUPS = 512  # workgroups (all heads of 16 rows each) that fill the 256 CUs two deep: steps of few rows split their keys up to this


def kv_write(cache: torch.Tensor, k: torch.Tensor, v: torch.Tensor, slot_mapping: torch.Tensor, koff: int,
             voff: int, num_kv_heads: int, dk: int, dv: int, block_size: int) -> None:
    """k [T, Hkv*dk], v [T, Hkv*dv] (row-strided views) into the paged cache; slot -1 writes nothing."""
    if _gpu(k):
        ext().kv_write(cache, k, v, slot_mapping, int(koff), int(voff), num_kv_heads, dk, dv, block_size)
        return
    ok = slot_mapping >= 0
    slots = slot_mapping[ok]
    blk, off = slots // block_size, slots % block_size
    T = int(slots.numel())
    kc = cache[:, koff:koff + num_kv_heads * block_size * dk].view(-1, num_kv_heads, block_size, dk)
    vc = cache[:, voff:voff + num_kv_heads * block_size * dv].view(-1, num_kv_heads, block_size, dv)
    kc[blk, :, off] = k[ok].reshape(T, num_kv_heads, dk).to(cache.dtype)
    vc[blk, :, off] = v[ok].reshape(T, num_kv_heads, dv).to(cache.dtype)


def window_attention(q: torch.Tensor, cache: torch.Tensor, block_tables: torch.Tensor, qsl: torch.Tensor,
                     seq_lens: torch.Tensor, koff: int, voff: int, num_heads: int, num_kv_heads: int, dk: int,
                     dv: int, block_size: int, scale: float, window: int, keep_first: int,
                     max_query_len: int = 0, sink: Optional[torch.Tensor] = None, v_stride: int = 0,
                     talk: Optional[torch.Tensor] = None, max_seq_len: int = 0) -> torch.Tensor:
    """Softmax attention over the paged cache (this step's keys already written).  The query at
    position i sees key j <= i when i - j < window or j < keep_first (window <= 0: every j <= i).
    q [T, H*dk] (row-strided view) -> [T, H*dv] in q's dtype; scores and weights in fp32.
    Query head h reads kv head h // (H / Hkv).  sink (fp32 [H]): the softmax denominator of head h also
    holds exp(sink[h]), a key without a value whose score is not scaled.  v_stride (elements, 0: dv): the
    distance between two tokens' value rows, for values that are a slice of a wider cached row (then
    num_kv_heads is 1 and voff points at the slice inside the first row).  max_query_len: the longest chunk of the step (host
    int); from 16 rows a bf16 step with head sizes that are multiples of 16 runs the MFMA kernel.
    talk (fp32 [H, H]): the heads' scaled scores of a (query, key) pair are mixed before the softmax,
    score_h <- sum_g talk[h, g] score_g (the mask and the sink act on the mixed scores); a workgroup then
    serves all heads of its rows, and a bf16 step of few rows splits every row's keys over several
    workgroups (max_seq_len, a host int, bounds how many are worth it) whose stretches are merged."""
    T = q.shape[0]
    if _gpu(q) and talk is not None:
        if v_stride and v_stride != dv:
            raise ValueError("mixed heads read value rows back to back")
        out = torch.empty(T, num_heads * dv, dtype=q.dtype, device=q.device)
        nsplit, part = 1, None
        if q.dtype == torch.bfloat16 and T and block_size == 16 and dk % 16 == 0 and dv % 16 == 0 and dk <= 128 and dv <= 128:
            mq = max(1, min(int(max_query_len) or T, T))
            tiles = seq_lens.numel() * (-(-mq // 16))
            span = int(max_seq_len) or 16
            if window > 0:
                span = min(span, int(window) + int(keep_first) + 15)
            nsplit = max(1, min(16, TALK_TARGET_GROUPS // max(tiles, 1), -(-span // 16) // 2))
            if nsplit > 1:
                part = torch.empty(T * num_heads * nsplit * (dv + 4), dtype=torch.float32, device=q.device)
        ext().talking_attention(out, q, cache, block_tables, qsl, seq_lens, int(koff), int(voff), num_heads, num_kv_heads,
                                dk, dv, block_size, float(scale), int(window), int(keep_first), int(max_query_len), sink,
                                talk, nsplit, part)
        return out
    if _gpu(q):
        out = torch.empty(T, num_heads * dv, dtype=q.dtype, device=q.device)
        ext().window_attention(out, q, cache, block_tables, qsl, seq_lens, int(koff), int(voff), num_heads,
                               num_kv_heads, dk, dv, block_size, float(scale), int(window), int(keep_first),
                               int(max_query_len), sink, int(v_stride))
        return out
    out = torch.zeros(T, num_heads, dv, dtype=torch.float32)
    kc = cache[:, koff:koff + num_kv_heads * block_size * dk].view(-1, num_kv_heads, block_size, dk)
    if v_stride and v_stride != dv:
        if num_kv_heads != 1:
            raise ValueError("strided value rows need a single kv head")
        vc = torch.as_strided(cache, (cache.shape[0], 1, block_size, dv), (cache.stride(0), 0, v_stride, 1),
                              cache.storage_offset() + voff)
    else:
        vc = cache[:, voff:voff + num_kv_heads * block_size * dv].view(-1, num_kv_heads, block_size, dv)
    g = num_heads // num_kv_heads
    ql, sl = qsl.tolist(), seq_lens.tolist()
    for s in range(len(sl)):
        a, e = ql[s], ql[s + 1]
        n = sl[s]
        if e <= a:
            continue
        nb = -(-n // block_size)
        blocks = block_tables[s, :nb].long()
        K = kc[blocks].permute(0, 2, 1, 3).reshape(nb * block_size, num_kv_heads, dk)[:n].float()
        V = vc[blocks].permute(0, 2, 1, 3).reshape(nb * block_size, num_kv_heads, dv)[:n].float()
        qs = q[a:e].reshape(e - a, num_heads, dk).float()
        sc = torch.einsum("mhd,nhd->hmn", qs, K.repeat_interleave(g, dim=1)) * scale
        if talk is not None:
            sc = torch.einsum("hg,gmn->hmn", talk.float(), sc)
        i = torch.arange(n - (e - a), n).unsqueeze(1)
        j = torch.arange(n).unsqueeze(0)
        seen = j <= i
        if window > 0:
            seen = seen & ((i - j < window) | (j < keep_first))
        sc = sc.masked_fill(~seen.unsqueeze(0), float("-inf"))
        if sink is not None:  # one more column, dropped after the softmax: it has no value
            sc = torch.cat([sc, sink.float().view(-1, 1, 1).expand(-1, sc.shape[1], 1)], dim=-1)
        p = torch.softmax(sc, dim=-1)[..., :n]
        out[a:e] = torch.einsum("hmn,nhd->mhd", p, V.repeat_interleave(g, dim=1))
    return out.reshape(T, num_heads * dv).to(q.dtype)


# ----------------------------------------------------------------------------- recurrences
SCAN_PIECE = int(os.environ.get("MXS_SCAN_PIECE", "0"))  # tokens per piece of a time-split scan; 0: by the launch's size
SCAN_SCRATCH_BYTES = 512 << 20
SCAN_TARGET_BLOCKS = 1024  # workgroups that fill the 256 CUs four deep


def _scan_split(S: int, T: int, max_query_len: int, floats: int, heads: int, dv: int, device) -> tuple:
    """(piece, npieces, scratch pool, scratch pool) of a scan launch: chunks of 2 pieces or more are cut
    into pieces that run side by side (two passes and a chaining step, csrc/mixers/scan.hip).  Pieces
    are 64 to 256 tokens, as short as it takes to reach SCAN_TARGET_BLOCKS workgroups over the long
    chunks of the step, and grow until both scratch pools [S, npieces, state] fit SCAN_SCRATCH_BYTES."""
    max_query_len = min(max_query_len, T)
    if max_query_len < 128:
        return 1, 1, None, None
    piece = SCAN_PIECE
    if piece <= 0:
        per_piece = heads * -(-dv // 64) * max(1, T // max_query_len)  # workgroups one piece index adds
        want = -(-SCAN_TARGET_BLOCKS // per_piece)
        piece = 256
        while piece > 64 and -(-max_query_len // piece) < want:
            piece //= 2
    while max_query_len >= 2 * piece:
        n = -(-max_query_len // piece)
        if 2 * S * n * floats * 4 <= SCAN_SCRATCH_BYTES:
            pool = torch.empty(2, S * n * floats, dtype=torch.float32, device=device)
            return piece, n, pool[0], pool[1]
        piece *= 2
    return 1, 1, None, None


def decay_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay: torch.Tensor, state: torch.Tensor,
               state_rows: torch.Tensor, off: int, qsl: torch.Tensor, seq_lens: torch.Tensor, num_heads: int,
               dk: int, dv: int, silu: bool = True, max_query_len: int = 0) -> torch.Tensor:
    """Decayed linear attention, token by token per head: S = decay_h S + k v^T, o = S^T q, with q, k, v
    passed through SiLU first when `silu`.  q, k [T, H*dk], v [T, H*dv] (row-strided views); decay
    fp32 [H]; returns o fp32 [T, H*dv] and leaves each sequence's S in its slot.  max_query_len: the
    step's longest chunk (host int); long chunks are cut into pieces that run side by side."""
    T = q.shape[0]
    if _gpu(q):
        out = torch.empty(T, num_heads * dv, dtype=torch.float32, device=q.device)
        plan = _scan_split(seq_lens.numel(), T, max_query_len, num_heads * dk * dv, num_heads, dv, q.device)
        ext().decay_scan(out, q, k, v, decay, state, state_rows, int(off), qsl, seq_lens, num_heads, dk, dv,
                         bool(silu), *plan)
        return out
    out = torch.zeros(T, num_heads, dv, dtype=torch.float32)
    qf, kf, vf = (t.float().reshape(T, num_heads, -1) for t in (q, k, v))
    if silu:
        qf, kf, vf = F.silu(qf), F.silu(kf), F.silu(vf)
    ql, sl, rows = qsl.tolist(), seq_lens.tolist(), state_rows.tolist()
    n = num_heads * dk * dv
    for s in range(len(sl)):
        a, e = ql[s], ql[s + 1]
        if e <= a:
            continue
        S = state[rows[s], off:off + n].view(num_heads, dk, dv)
        if sl[s] - (e - a) == 0:
            S.zero_()
        for t in range(a, e):
            S.mul_(decay.view(-1, 1, 1)).add_(kf[t].unsqueeze(2) * vf[t].unsqueeze(1))
            out[t] = torch.einsum("hdv,hd->hv", S, qf[t])
    return out.reshape(T, num_heads * dv)


def mlstm_state_floats(num_heads: int, dk: int, dv: int) -> int:
    return num_heads * (dk * dv + dk + 1)


def mlstm_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, gates: torch.Tensor, state: torch.Tensor,
               state_rows: torch.Tensor, off: int, qsl: torch.Tensor, seq_lens: torch.Tensor, num_heads: int,
               dk: int, dv: int, gate_cap: float, q_scale: float, max_query_len: int = 0) -> torch.Tensor:
    """mLSTM matrix memory, token by token per head.  gates fp32 [T, 2H]: the input gates' then the
    forget gates' pre-activations.  With i = cap tanh(pre_i / cap), f = logsigmoid(cap tanh(pre_f / cap))
    and a running maximum m (0 at the start):
        m' = max(f + m, i);  S = e^(f + m - m') S + e^(i - m') k v^T;  n likewise with k;
        o = S^T q~ / (max(|n . q~|, e^(-m')) + 1e-6),   q~ = q_scale q.
    Returns o fp32 [T, H*dv] (before any norm)."""
    T = q.shape[0]
    if _gpu(q):
        out = torch.empty(T, num_heads * dv, dtype=torch.float32, device=q.device)
        plan = _scan_split(seq_lens.numel(), T, max_query_len, mlstm_state_floats(num_heads, dk, dv) + num_heads,
                           num_heads, dv, q.device)
        ext().mlstm_scan(out, q, k, v, gates, state, state_rows, int(off), qsl, seq_lens, num_heads, dk, dv,
                         float(gate_cap), float(q_scale), *plan)
        return out
    H = num_heads
    out = torch.zeros(T, H, dv, dtype=torch.float32)
    qf = q.float().reshape(T, H, dk) * q_scale
    kf, vf = k.float().reshape(T, H, dk), v.float().reshape(T, H, dv)
    ig = gate_cap * torch.tanh(gates[:, :H] / gate_cap)
    fg = F.logsigmoid(gate_cap * torch.tanh(gates[:, H:] / gate_cap))
    ql, sl, rows = qsl.tolist(), seq_lens.tolist(), state_rows.tolist()
    nS, nn = H * dk * dv, H * dk
    for s in range(len(sl)):
        a, e = ql[s], ql[s + 1]
        if e <= a:
            continue
        st = state[rows[s]]
        S = st[off:off + nS].view(H, dk, dv)
        n = st[off + nS:off + nS + nn].view(H, dk)
        m = st[off + nS + nn:off + nS + nn + H]
        if sl[s] - (e - a) == 0:
            S.zero_(), n.zero_(), m.zero_()
        for t in range(a, e):
            m_new = torch.maximum(fg[t] + m, ig[t])
            fa, ia = torch.exp(fg[t] + m - m_new), torch.exp(ig[t] - m_new)
            S.mul_(fa.view(H, 1, 1)).add_(ia.view(H, 1, 1) * kf[t].unsqueeze(2) * vf[t].unsqueeze(1))
            n.mul_(fa.view(H, 1)).add_(ia.view(H, 1) * kf[t])
            m.copy_(m_new)
            den = torch.maximum((n * qf[t]).sum(-1).abs(), torch.exp(-m)) + 1e-6
            out[t] = torch.einsum("hdv,hd->hv", S, qf[t]) / den.unsqueeze(1)
    return out.reshape(T, H * dv)


# ----------------------------------------------------------------------------- embedding, feed-forward
def embed_scaled(ids: torch.Tensor, table: torch.Tensor, scale: float) -> torch.Tensor:
    """table[ids] * scale as the fp32 residual stream [T, W]."""
    if _gpu(table):
        out = torch.empty(ids.shape[0], table.shape[1], dtype=torch.float32, device=table.device)
        ext().embed_scaled(out, ids, table, float(scale))
        return out
    return F.embedding(ids, table).float() * scale


def silu_mul(gu: torch.Tensor) -> torch.Tensor:
    """SiLU(gu[:, :F]) * gu[:, F:] of a fused gate/up projection [T, 2F]; fp32 inside."""
    Fh = gu.shape[1] // 2
    if _gpu(gu):
        out = torch.empty(gu.shape[0], Fh, dtype=gu.dtype, device=gu.device)
        ext().silu_mul(out, gu)
        return out
    return (F.silu(gu[:, :Fh].float()) * gu[:, Fh:].float()).to(gu.dtype)


# ----------------------------------------------------------------------------- rotary positions
def _rotate(x: torch.Tensor, pos: torch.Tensor, freqs: torch.Tensor, sign: float, mag: float = 1.0) -> torch.Tensor:
    """x fp32 [T, heads, dim]: pair (2i, 2i+1) turned by sign * pos * freqs[i]; the rest passes."""
    n = freqs.numel()
    ang = pos.to(torch.float32).view(-1, 1, 1) * freqs.float().view(1, 1, n) * sign
    c, s = torch.cos(ang) * mag, torch.sin(ang) * mag
    u, v = x[..., 0:2 * n:2], x[..., 1:2 * n:2]
    y = x.clone()
    y[..., 0:2 * n:2] = u * c - v * s
    y[..., 1:2 * n:2] = v * c + u * s
    return y


def rope_qkv_cache(q: torch.Tensor, k: Optional[torch.Tensor], v: Optional[torch.Tensor], positions: torch.Tensor,
                   slot_mapping: torch.Tensor, cache: torch.Tensor, koff: int, voff: int, num_heads: int,
                   num_kv_heads: int, dk: int, dv: int, block_size: int, freqs: torch.Tensor,
                   q_norm: Optional[torch.Tensor] = None, k_norm: Optional[torch.Tensor] = None, eps: float = 1e-5,
                   v_freqs: Optional[torch.Tensor] = None, *, bias_q: Optional[torch.Tensor] = None,
                   bias_k: Optional[torch.Tensor] = None, bias_v: Optional[torch.Tensor] = None,
                   norm_whole: bool = False, split_pairs: bool = False, mag: float = 1.0) -> None:
    """Queries, keys and values of a step from the fused projection to what attention reads, in one
    launch.  Per head: optional RMS norm over the head (weight [dk], plain), then interleaved rotary
    pairs (2i, 2i+1) on the first 2 * len(freqs) dimensions by position * freqs[i]; values are
    turned over 2 * len(v_freqs) dimensions when v_freqs is given.  q [T, H*dk] is rewritten in place;
    k [T, G*dk] and v [T, G*dv] go into the paged cache (slot -1: not written).  k = v = None: a layer
    that reads another layer's pages.  Angles, norms and rotations in fp32, one rounding at the end.
    The keyword forms (one launch of a workgroup per token): bias_q / bias_k / bias_v are added first;
    norm_whole: ONE RMS norm over all of q's columns and one over all of k's (weights [H*dk], [G*dk]);
    split_pairs: coordinate i pairs with i + len(freqs) instead of its neighbour; mag multiplies cos and sin."""
    general = bias_q is not None or bias_k is not None or bias_v is not None or norm_whole or split_pairs or mag != 1.0
    if _gpu(q) and general:
        if v_freqs is not None:
            raise ValueError("turned values come with the per-head form only")
        ext().qkv_prep_cache(q, k, v, positions, slot_mapping, cache, int(koff), int(voff), num_heads, num_kv_heads, dk, dv,
                             block_size, freqs, float(mag), bool(split_pairs), bias_q, bias_k, bias_v, q_norm, k_norm,
                             float(eps), bool(norm_whole))
        return
    if _gpu(q):
        ext().rope_qkv_cache(q, k, v, positions, slot_mapping, cache, int(koff), int(voff), num_heads, num_kv_heads,
                             dk, dv, block_size, freqs, q_norm, k_norm, float(eps), v_freqs)
        return
    T = q.shape[0]

    def prep(x, heads, dim, norm_w, fr, bias):
        y = x.float()
        if bias is not None:
            y = y + bias.float()
        if norm_w is not None and norm_whole:
            y = _rms(y, eps) * norm_w.float()
        y = y.reshape(T, heads, dim)
        if norm_w is not None and not norm_whole:
            y = _rms(y, eps) * norm_w.float()
        if fr is None:
            return y
        if split_pairs:
            n = fr.numel()
            return torch.cat([_rotate_half(y[..., :2 * n], positions, fr, mag), y[..., 2 * n:]], dim=-1)
        return _rotate(y, positions, fr, 1.0, mag)

    q.copy_(prep(q, num_heads, dk, q_norm, freqs, bias_q).reshape(T, -1).to(q.dtype))
    if k is None:
        return
    kk = prep(k, num_kv_heads, dk, k_norm, freqs, bias_k).reshape(T, -1).to(k.dtype)
    vv = prep(v, num_kv_heads, dv, None, v_freqs, bias_v).reshape(T, -1).to(v.dtype)
    kv_write(cache, kk, vv, slot_mapping, koff, voff, num_kv_heads, dk, dv, block_size)


def rope_rows(x: torch.Tensor, positions: torch.Tensor, heads: int, dim: int, freqs: torch.Tensor, sign: float,
              out_scale: float, out: torch.Tensor) -> None:
    """out = out_scale * (x with every head's pairs (2i, 2i+1) turned by sign * position * freqs[i]).
    x [T, heads*dim]; out may be a row-strided view of the same shape (a slice of a wider buffer)."""
    if _gpu(x):
        ext().rope_rows(out, x, positions, heads, dim, freqs, float(sign), float(out_scale))
        return
    T = x.shape[0]
    out.copy_((_rotate(x.float().reshape(T, heads, dim), positions, freqs, sign) * out_scale).reshape(T, -1).to(out.dtype))


# ----------------------------------------------------------------------------- short causal convolution
def causal_conv(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], state: torch.Tensor,
                state_rows: torch.Tensor, off: int, qsl: torch.Tensor, seq_lens: torch.Tensor,
                silu: bool = True) -> torch.Tensor:
    """Per-channel causal filter over time: y[t, c] = bias[c] + sum_j w[j, c] x[t - (taps-1) + j, c], the
    last row of w weighing the current token, inputs before a sequence's start being zero; then
    SiLU.  x [T, C] (row-strided view), w tap-major [taps, C] (a checkpoint's [C, taps] transposed, so
    that neighbouring channels' weights are neighbours).  The sequence's last taps - 1 inputs live in
    its state slot at `off` as fp32 [taps - 1, C], oldest first, and are replaced by this step's."""
    T, C = x.shape
    taps = w.shape[0]
    if _gpu(x):
        out = torch.empty(T, C, dtype=x.dtype, device=x.device)
        ext().causal_conv(out, x, w, bias, state, state_rows, int(off), qsl, seq_lens, bool(silu))
        return out
    out = torch.zeros(T, C, dtype=torch.float32)
    ql, sl, rows = qsl.tolist(), seq_lens.tolist(), state_rows.tolist()
    wf = w.float()
    for s in range(len(sl)):
        a, e = ql[s], ql[s + 1]
        if e <= a:
            continue
        n = e - a
        st = state[rows[s], off:off + (taps - 1) * C].view(taps - 1, C)
        prev = torch.zeros(taps - 1, C) if sl[s] - n == 0 else st.clone()
        full = torch.cat([prev, x[a:e].float()])
        y = torch.zeros(n, C) if bias is None else bias.float().expand(n, C).clone()
        for j in range(taps):
            y += wf[j] * full[j:j + n]
        out[a:e] = y
        if taps > 1:
            st.copy_(full[n:])
    return (F.silu(out) if silu else out).to(x.dtype)


# ----------------------------------------------------------------------------- column scans
def ssd_scan(x: torch.Tensor, B: torch.Tensor, C: torch.Tensor, dt: torch.Tensor, dt_bias: torch.Tensor,
             A_log: torch.Tensor, D: torch.Tensor, state: torch.Tensor, state_rows: torch.Tensor, off: int,
             qsl: torch.Tensor, seq_lens: torch.Tensor, num_heads: int, groups: int, N: int, P: int,
             max_query_len: int = 0) -> torch.Tensor:
    """Selective state-space recurrence with a scalar decay per head and token (state-space duality):
        d = softplus(dt + dt_bias_h);  S = exp(-exp(A_log_h) d) S + d B_g x_h^T;  y_h = S^T C_g + D_h x_h
    with S [N, P] per head and head h reading group h // (H / G).  x [T, H*P], B, C [T, G*N], dt [T, H]
    (row-strided views of any float dtype); dt_bias, A_log, D fp32 [H].  Returns y fp32 [T, H*P]; the
    state (fp32, stored [H, P, N]) stays in the sequence's slot.  max_query_len: the step's longest
    chunk (host int); the step is a diagonal map of the state, so long chunks are cut into pieces
    that run side by side (a piece's end state from an empty state, the true state at every piece's
    start chained from those and the pieces' decays, then the outputs)."""
    T = x.shape[0]
    H = num_heads
    if _gpu(x):
        out = torch.empty(T, H * P, dtype=torch.float32, device=x.device)
        piece, npieces, loc, start = _scan_split(seq_lens.numel(), T, max_query_len, H * N * P, H, 4 * P, x.device)
        dec = torch.empty(seq_lens.numel() * npieces * H, dtype=torch.float32, device=x.device) if npieces > 1 else None
        ext().ssd_scan(out, x, B, C, dt, dt_bias, A_log, D, state, state_rows, int(off), qsl, seq_lens, H, groups, N, P,
                       piece, npieces, loc, start, dec, int(max_query_len))
        return out
    out = torch.zeros(T, H, P, dtype=torch.float32)
    xf = x.float().reshape(T, H, P)
    rep = H // groups
    Bf = B.float().reshape(T, groups, N).repeat_interleave(rep, dim=1)
    Cf = C.float().reshape(T, groups, N).repeat_interleave(rep, dim=1)
    d = F.softplus(dt.float() + dt_bias.float(), threshold=1e9)
    a = torch.exp(-torch.exp(A_log.float()) * d)
    ql, sl, rows = qsl.tolist(), seq_lens.tolist(), state_rows.tolist()
    for s in range(len(sl)):
        b, e = ql[s], ql[s + 1]
        if e <= b:
            continue
        S = state[rows[s], off:off + H * P * N].view(H, P, N)
        if sl[s] - (e - b) == 0:
            S.zero_()
        for t in range(b, e):
            S.mul_(a[t].view(H, 1, 1)).add_((d[t].view(H, 1) * xf[t]).unsqueeze(2) * Bf[t].unsqueeze(1))
            out[t] = (S * Cf[t].unsqueeze(1)).sum(-1) + D.float().view(H, 1) * xf[t]
    return out.reshape(T, H * P)


DELTA_MIN_PIECES = 4  # a split delta-rule scan does three times the work: fewer pieces do not pay


def delta_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, beta: torch.Tensor, a: torch.Tensor,
               dt_bias: torch.Tensor, A_log: torch.Tensor, state: torch.Tensor, state_rows: torch.Tensor, off: int,
               qsl: torch.Tensor, seq_lens: torch.Tensor, num_heads: int, qk_heads: int, dk: int, dv: int,
               q_scale: float, unit_eps: float = 1e-6, max_query_len: int = 0) -> torch.Tensor:
    """Gated delta rule with one decay per head and key channel.  q, k [T, G*dk] are made unit vectors
    per head (x / sqrt(sum x^2 + unit_eps)), q also times q_scale; head h reads q/k head h // (H / G).
        g = exp(-exp(A_log_h) softplus(a + dt_bias))   [H, dk]      b = sigmoid(beta)   [H]
        S = diag(g) S;   u = b (v - S^T k);   S = S + k u^T;   o = S^T q
    so the read-out sees the token's own write.  v [T, H*dv], beta [T, H], a [T, H*dk] (row-strided
    views); dt_bias fp32 [H*dk], A_log fp32 [H].  Returns o fp32 [T, H*dv]; S (fp32, stored [H, dv, dk])
    stays in the sequence's slot.
    max_query_len: the step's longest chunk (host int).  A token maps the state as S -> A_t S + b_t with
    A_t = (I - b k k^T) diag(g), so a piece of tokens maps it as S -> P S + L: long chunks are cut into
    pieces that run side by side, pass 1 giving every piece's L (end state from an empty start) and P
    (dk more state columns started as the identity and fed no values), the states at the pieces'
    starts following by one fp32 matrix product per piece, pass 2 writing the outputs.  Three times
    the multiply-adds, but DELTA_MIN_PIECES or more pieces at once instead of one serial walk."""
    T = q.shape[0]
    H, G = num_heads, qk_heads
    if _gpu(q):
        out = torch.empty(T, H * dv, dtype=torch.float32, device=q.device)
        S = seq_lens.numel()
        args = (out, q, k, v, beta, a, dt_bias, A_log, state, state_rows, int(off), qsl, seq_lens, H, G, dk, dv,
                float(q_scale), float(unit_eps))
        piece, npieces, _, _ = _scan_split(S, T, max_query_len, H * (dv + dk) * dk, H, 4 * (dv + dk), q.device)
        if npieces < DELTA_MIN_PIECES:
            ext().delta_scan(*args, 0, 1, 1, None, None, int(max_query_len))
            return out
        n = H * dv * dk
        loc = torch.empty(S, npieces, H, dv + dk, dk, dtype=torch.float32, device=q.device)
        start = torch.empty(S, npieces, H * dv, dk, dtype=torch.float32, device=q.device)
        ext().delta_scan(*args, 1, piece, npieces, loc, start, int(max_query_len))
        first = (seq_lens - (qsl[1:] - qsl[:-1]) <= 0).view(S, 1, 1)
        slot = state.index_select(0, state_rows.long())[:, off:off + n].view(S, H * dv, dk)
        start[:, 0] = torch.where(first, torch.zeros((), dtype=torch.float32, device=q.device), slot)
        for p in range(npieces - 1):  # St' = St Pt + Lt in the transposed storage, batched over sequences and heads
            start[:, p + 1] = torch.baddbmm(loc[:, p, :, :dv].reshape(S * H, dv, dk), start[:, p].reshape(S * H, dv, dk),
                                            loc[:, p, :, dv:].reshape(S * H, dk, dk)).view(S, H * dv, dk)
        ext().delta_scan(*args, 2, piece, npieces, loc, start, int(max_query_len))
        return out
    out = torch.zeros(T, H, dv, dtype=torch.float32)
    rep = H // G

    def unit(t):
        t = t.float().reshape(T, G, dk)
        return (t * torch.rsqrt(t.pow(2).sum(-1, keepdim=True) + unit_eps)).repeat_interleave(rep, dim=1)

    qf, kf = unit(q) * q_scale, unit(k)
    vf = v.float().reshape(T, H, dv)
    b = torch.sigmoid(beta.float())
    g = torch.exp(-torch.exp(A_log.float()).view(1, H, 1) *
                  F.softplus(a.float() + dt_bias.float(), threshold=1e9).reshape(T, H, dk))
    ql, sl, rows = qsl.tolist(), seq_lens.tolist(), state_rows.tolist()
    for s in range(len(sl)):
        c, e = ql[s], ql[s + 1]
        if e <= c:
            continue
        S = state[rows[s], off:off + H * dv * dk].view(H, dv, dk)
        if sl[s] - (e - c) == 0:
            S.zero_()
        for t in range(c, e):
            S.mul_(g[t].unsqueeze(1))
            u = b[t].view(H, 1) * (vf[t] - (S * kf[t].unsqueeze(1)).sum(-1))
            S.add_(u.unsqueeze(2) * kf[t].unsqueeze(1))
            out[t] = (S * qf[t].unsqueeze(1)).sum(-1)
    return out.reshape(T, H * dv)


def gated_norm(o: torch.Tensor, gate: torch.Tensor, w: torch.Tensor, eps: float, groups: int, act: str,
               gate_first: bool, out_dtype: torch.dtype, out_scale: float = 1.0,
               out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """A mixer's output norm with its gate.  o fp32 [T, N]; the RMS norm runs over each of `groups`
    equal slices of a row; w has N entries or a divisor of N (then it repeats, e.g. one weight per
    head size shared by the heads); act(gate) with act in silu | sigmoid multiplies before the norm
    (gate_first) or after it.  The result, times out_scale, goes to `out` (may be a row-strided view
    of a wider buffer) or a new [T, N] tensor of out_dtype."""
    T, N = o.shape
    if out is None:
        out = torch.empty(T, N, dtype=out_dtype, device=o.device)
    if _gpu(o):
        ext().gated_norm(out, o, gate, w, float(eps), int(groups), act == "silu", bool(gate_first), float(out_scale))
        return out
    gf = F.silu(gate.float()) if act == "silu" else torch.sigmoid(gate.float())
    wf = w.float().repeat(N // w.numel())
    y = o * gf if gate_first else o
    y = _rms(y.view(T, groups, N // groups), eps).reshape(T, N) * wf
    if not gate_first:
        y = y * gf
    out.copy_((y * out_scale).to(out.dtype))
    return out


# ----------------------------------------------------------------------------- latent attention
def _rotate_half(x: torch.Tensor, pos: torch.Tensor, freqs: torch.Tensor, mag: float = 1.0) -> torch.Tensor:
    """x fp32 [T, heads, 2n]: coordinate i pairs with i + n and the pair turns by pos * freqs[i]."""
    n = freqs.numel()
    ang = pos.to(torch.float32).view(-1, 1, 1) * freqs.float().view(1, 1, n)
    c, s = torch.cos(ang) * mag, torch.sin(ang) * mag
    u, v = x[..., :n], x[..., n:]
    return torch.cat([u * c - v * s, v * c + u * s], dim=-1)


def latent_prep(dq: torch.Tensor, dkv: torch.Tensor, positions: torch.Tensor, slot_mapping: torch.Tensor,
                cache: torch.Tensor, koff: int, rank: int, block_size: int, freqs: torch.Tensor,
                q_norm: torch.Tensor, kv_norm: torch.Tensor, eps: float, split_pairs: bool = True) -> torch.Tensor:
    """The two down-projections of a latent attention, from the fused projection to what the next
    steps read, in one launch.  dq [T, q_rank] (row-strided view): returns RMSNorm(dq) * q_norm as a
    new [T, q_rank].  dkv [T, rank + 2n]: the first `rank` columns RMS-normed times kv_norm, the last
    2n (n = len(freqs)) turned in the half-split layout (i pairs with i + n; split_pairs False: 2i with
    2i + 1) by position * freqs[i]; the row [latent | turned part] goes into the paged cache at `koff` as [BS, rank + 2n] (one shared
    kv head; slot -1: not written).  Norms, angles and turns in fp32, one rounding at the end."""
    T, qr = dq.shape
    n = freqs.numel()
    dk = rank + 2 * n
    if _gpu(dq):
        cq = torch.empty(T, qr, dtype=dq.dtype, device=dq.device)
        ext().latent_prep(cq, dq, dkv, positions, slot_mapping, cache, int(koff), int(rank), int(block_size), freqs,
                          q_norm, kv_norm, float(eps), bool(split_pairs))
        return cq
    cq = (_rms(dq.float(), eps) * q_norm.float()).to(dq.dtype)
    d = dkv.float()
    c = _rms(d[:, :rank], eps) * kv_norm.float()
    turn = _rotate_half if split_pairs else (lambda x, p, f: _rotate(x, p, f, 1.0))
    kr = turn(d[:, rank:].unsqueeze(1), positions, freqs).squeeze(1)
    row = torch.cat([c, kr], dim=-1).to(cache.dtype)
    ok = slot_mapping >= 0
    slots = slot_mapping[ok]
    kc = cache[:, koff:koff + block_size * dk].view(-1, block_size, dk)
    kc[slots // block_size, slots % block_size] = row[ok]
    return cq


def rope_half_into(out: torch.Tensor, x: torch.Tensor, positions: torch.Tensor, heads: int, x_dim: int, x_col: int,
                   out_dim: int, out_col: int, freqs: torch.Tensor, split_pairs: bool = True) -> None:
    """Per token and head: the 2n columns of x's head (x [T, heads*x_dim], from column x_col of the head)
    turned in the half-split layout (split_pairs False: as neighbouring pairs) by position * freqs[i],
    written to columns out_col.. of the same head in out [T, heads*out_dim].  fp32 inside."""
    n = freqs.numel()
    if _gpu(x):
        ext().rope_half_into(out, x, positions, int(heads), int(x_dim), int(x_col), int(out_dim), int(out_col), freqs,
                             bool(split_pairs))
        return
    T = x.shape[0]
    part = x.reshape(T, heads, x_dim)[:, :, x_col:x_col + 2 * n].float()
    turned = _rotate_half(part, positions, freqs) if split_pairs else _rotate(part, positions, freqs, 1.0)
    out.view(T, heads, out_dim)[:, :, out_col:out_col + 2 * n] = turned.to(out.dtype)


LATENT_TARGET_WAVES = 1024  # waves that fill the 256 CUs one deep: single-token steps split their keys up to this
# the widest rows (over 320 entries): "pair" = two waves per 16-row tile, each half of the row; "single" = one wave
# per tile with its queries in LDS; "auto" = pair
LATENT_WIDE_FORM = os.environ.get("MXS_LATENT_WIDE_FORM", "auto")


def latent_attention(q: torch.Tensor, cache: torch.Tensor, block_tables: torch.Tensor, qsl: torch.Tensor,
                     seq_lens: torch.Tensor, koff: int, num_heads: int, dk: int, rank: int, block_size: int, scale: float,
                     max_query_len: int = 0, max_seq_len: int = 0, sink: Optional[torch.Tensor] = None,
                     window: int = 0) -> torch.Tensor:
    """Softmax attention of every head over the same cached rows [latent | rotated part] (dk entries a
    row at `koff`, written by latent_prep), causal, within the last `window` positions when window > 0;
    the values are the rows' first `rank` entries.
    q [T, H*dk] (the folded queries) -> the weighted latents [T, H*rank]; scores and weights fp32; sink as
    in window_attention.  bf16 on the GPU with dk a multiple of 8 up to 576 and rank a multiple of 16 up
    to 512 runs the matrix-core kernel; a step of few rows splits each row's keys over several waves
    (max_seq_len bounds how many are worth it) and merges the stretches.  Everything else runs
    window_attention with one kv head and value rows dk apart."""
    T = q.shape[0]
    if _gpu(q) and q.dtype == torch.bfloat16 and T:
        S = seq_lens.numel()
        mq = max(1, min(int(max_query_len) or T, T))
        tiles = S * (-(-mq * num_heads // 16))
        span = min(int(max_seq_len) or 16, int(window) + 15) if window > 0 else (int(max_seq_len) or 16)
        blocks = max(1, -(-span // 16))
        nsplit = max(1, min(16, LATENT_TARGET_WAVES // max(tiles, 1), blocks // 2))
        out = torch.empty(T, num_heads * rank, dtype=q.dtype, device=q.device)
        part = (torch.empty(T * num_heads * nsplit * (rank + 4), dtype=torch.float32, device=q.device)
                if nsplit > 1 else None)
        if ext().latent_attention(out, q, cache, block_tables, qsl, seq_lens, int(koff), num_heads, dk, rank, block_size,
                                  float(scale), mq, sink, nsplit, part,
                                  LATENT_WIDE_FORM != "single", int(window)):
            return out
    return window_attention(q, cache, block_tables, qsl, seq_lens, koff, koff, num_heads, 1, dk, rank, block_size, scale,
                            int(window), 0, max_query_len, sink=sink, v_stride=dk)


# ----------------------------------------------------------------------------- routed experts
def route_topk(logits: torch.Tensor, k: int, renorm: bool = False, softmax: bool = False) -> tuple:
    """Router: scores = sigmoid(logits), or softmax over all experts (fp32 [T, E]); the k largest per
    token (ties: the lower index first), their scores as weights (renorm: divided by their sum).
    -> (weights fp32 [T, k], ids int32 [T, k])."""
    T, E = logits.shape
    if _gpu(logits):
        w = torch.empty(T, k, dtype=torch.float32, device=logits.device)
        ids = torch.empty(T, k, dtype=torch.int32, device=logits.device)
        ext().route_topk(w, ids, logits, bool(renorm), bool(softmax))
        return w, ids
    s = torch.softmax(logits.float(), dim=-1) if softmax else torch.sigmoid(logits.float())
    order = torch.argsort(s, dim=-1, descending=True, stable=True)[:, :k]
    w = torch.gather(s, 1, order)
    if renorm:
        w = w / w.sum(-1, keepdim=True)
    return w, order.to(torch.int32)


def capped_glu(gu: torch.Tensor, limit: float, alpha: float = 1.702) -> torch.Tensor:
    """A fused [gate | up] projection [R, 2F] -> [R, F]:  g = min(gate, limit), u = clamp(up, -limit, limit),
    g * sigmoid(alpha * g) * (u + 1); fp32 inside."""
    Fh = gu.shape[1] // 2
    if _gpu(gu):
        out = torch.empty(gu.shape[0], Fh, dtype=gu.dtype, device=gu.device)
        ext().capped_glu(out, gu, float(limit), float(alpha))
        return out
    g = gu[:, :Fh].float().clamp(max=limit)
    u = gu[:, Fh:].float().clamp(-limit, limit)
    return (g * torch.sigmoid(alpha * g) * (u + 1.0)).to(gu.dtype)


def expert_align(ids: torch.Tensor, num_experts: int) -> tuple:
    """Counting sort of the (token, slot) pairs by expert.  ids int32 [T, k] -> (offs int32 [E + 1]:
    expert e owns the sorted rows offs[e]:offs[e+1]; inv int32 [T*k]: the sorted row of pair p = t*k + j;
    the order of one expert's rows is free)."""
    T, k = ids.shape
    if _gpu(ids):
        offs = torch.empty(num_experts + 1, dtype=torch.int32, device=ids.device)
        inv = torch.empty(T * k, dtype=torch.int32, device=ids.device)
        ext().expert_align(offs, inv, ids, int(num_experts))
        return offs, inv
    flat = ids.reshape(-1).long()
    order = torch.argsort(flat, stable=True)
    inv = torch.empty_like(order)
    inv[order] = torch.arange(order.numel())
    counts = torch.bincount(flat, minlength=num_experts)
    offs = torch.cat([torch.zeros(1, dtype=torch.long), counts.cumsum(0)])
    return offs.to(torch.int32), inv.to(torch.int32)


def gather_scaled(h: torch.Tensor, weights: Optional[torch.Tensor], inv: torch.Tensor, k: int = 0) -> torch.Tensor:
    """xs[inv[p]] = weights[p] * h[p // k] for every pair p (weights fp32 [T, k]): the experts' inputs,
    sorted by expert, each already times its routing weight (product in fp32, rounded once).
    weights None (then k says how many pairs a token has): the rows themselves."""
    T = h.shape[0]
    k = int(k) if weights is None else weights.shape[1]
    xs = torch.empty(T * k, h.shape[1], dtype=h.dtype, device=h.device)
    if _gpu(h):
        ext().gather_scaled(xs, h, weights, inv, k)
        return xs
    if weights is None:
        rows = h.unsqueeze(1).expand(T, k, h.shape[1]).reshape(T * k, -1)
    else:
        rows = (h.float().unsqueeze(1) * weights.float().unsqueeze(2)).reshape(T * k, -1).to(h.dtype)
    xs[inv.long()] = rows
    return xs


def spread_scaled(h: torch.Tensor, weights: Optional[torch.Tensor], ids: torch.Tensor, num_experts: int) -> torch.Tensor:
    """[E, T, W]: row (e, t) = weights[t, j] * h[t] where ids[t, j] = e, zeros for the experts a token
    did not choose (the experts' inputs for a batched product over all experts, no sorting).
    weights None: the chosen rows are h[t] itself."""
    T, k = ids.shape
    if _gpu(h):
        xs = torch.empty(num_experts, T, h.shape[1], dtype=h.dtype, device=h.device)
        ext().spread_scaled(xs, h, weights, ids)
        return xs
    cw = torch.zeros(T, num_experts, dtype=torch.float32)
    cw.scatter_(1, ids.long(), torch.ones(T, k) if weights is None else weights.float())
    return (cw.t().unsqueeze(2) * h.float().unsqueeze(0)).to(h.dtype)


def expert_combine(ys: torch.Tensor, index: Optional[torch.Tensor], k: int, T: int, extra: Optional[torch.Tensor] = None,
                   row_stride: int = 0, weights: Optional[torch.Tensor] = None, by_expert: bool = False) -> torch.Tensor:
    """out[t] = sum_j ys[index[t*k + j]] (+ extra[t]); index None: row j*row_stride + t (the k slabs
    of a [k, T, W] stack); by_expert: index holds experts and the row is index[t*k + j]*row_stride + t (a
    token's chosen slabs of an [E, T, W] stack).  weights (fp32 [T, k]): row j of token t enters times
    weights[t, j] (routing weights on the experts' outputs).  Summed in fp32, rounded once."""
    W = ys.shape[-1]
    y2 = ys.reshape(-1, W)
    if _gpu(ys):
        out = torch.empty(T, W, dtype=ys.dtype, device=ys.device)
        ext().expert_combine(out, y2, index, int(k), extra, int(row_stride), weights, bool(by_expert))
        return out
    if index is None:
        idx = (torch.arange(k).view(1, k) * row_stride + torch.arange(T).view(T, 1)).reshape(-1)
    elif by_expert:
        idx = (index.long().view(T, k) * row_stride + torch.arange(T).view(T, 1)).reshape(-1)
    else:
        idx = index.long()
    rows = y2[idx].float().view(T, k, W)
    if weights is not None:
        rows = rows * weights.float().view(T, k, 1)
    acc = rows.sum(1)
    if extra is not None:
        acc = acc + extra.float()
    return acc.to(ys.dtype)
