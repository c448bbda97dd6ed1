"""Token mixers that a layer can be built from, beside the rotary softmax attention of
mxserve/models/llama.py.  Each takes its sizes and constants as parameters, names the rows it wants
from the layer's fused input projection, says what it keeps per sequence (paged K/V, or fp32 state
in a slot) and computes its output from a step's flattened token batch.

  WindowAttention       softmax attention without positions over a sliding window plus the
                        sequence's first tokens, grouped kv heads, separate key and value sizes
  DecayLinearAttention  "lightning" linear attention: S = a_h S + k v^T, o = S^T q on SiLU(q, k, v),
                        one RMSNorm over all heads, sigmoid output gate
  MLSTM                 xLSTM's matrix memory with capped exponential gates and a running maximum,
                        per-head unit norm, sigmoid output gate
  ParallelPair          two mixers reading the same input; the layer averages their outputs after
                        an RMSNorm of each over the model width
  RotaryAttention       softmax attention with interleaved rotary pairs on part of each head (plain,
                        linearly scaled or band-scaled frequencies), optional per-head q/k RMS norm,
                        a sink in the softmax denominator (fixed or learned per head), optionally
                        values turned by their position and outputs turned back, optionally reading
                        another layer's pages instead of projecting keys and values
  Mamba2                selective state space with a scalar decay per head and token, short causal
                        convolution, SiLU gate before a grouped RMS norm
  GatedDeltaRule        delta-rule matrix memory with a decay per head and key channel, short
                        convolutions and unit-norm q/k, per-head RMS norm and a sigmoid output gate
  ScaledPair            two mixers reading the same input, summed with fixed scales through one
                        output projection over their concatenated activations
  LatentAttention       softmax attention whose keys and values are expansions of one normed low-rank
                        latent per token plus one rotated key part shared by the heads (half-split
                        or neighbouring rotary pairs), queries through a normed latent of their own,
                        optional learned sink, optional sliding window; only the latent and the rotated
                        part are cached, the expansions are folded into the query and the output
  TalkingAttention      softmax attention whose heads' scores are mixed by a learned [H, H] matrix before
                        the softmax; projections with biases, one RMS norm over all query rows and one
                        over all key rows, half-split rotary pairs on part of each head with
                        ramp-blended frequencies and a factor on cos / sin, sliding window, learned sink

The kernels are in mxserve/ops/seqmix.py (csrc/mixers/*.hip on the GPU).
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional

import torch

from .. import ops
from ..ops import seqmix


@dataclass
class StepContext:
    """What a mixer needs of one engine step."""
    md: object  # AttnMetadata
    cache: Optional[torch.Tensor]  # [num_blocks, block_elems] paged K/V pool
    state: Optional[torch.Tensor]  # [slots, state_floats] fp32
    block_size: int
    eps: float


class Mixer:
    kv_heads = dk = dv = 0  # paged K/V per token (0: none)
    state_floats = 0  # fp32 state per sequence

    def proj_rows(self) -> list:
        """[(tensor name, rows)] of the fused input projection, in the order forward() reads them."""
        raise NotImplementedError

    def extra_shapes(self) -> dict:
        return {}


class WindowAttention(Mixer):
    def __init__(self, prefix: str, width: int, heads: int, kv_heads: int, dim: int, vdim: int, scale: float,
                 window: int, keep_first: int):
        if heads % kv_heads:
            raise ValueError(f"{prefix}: {heads} query heads do not divide over {kv_heads} kv heads")
        self.p, self.width = prefix, width
        self.heads, self.kv_heads, self.dk, self.dv = heads, kv_heads, dim, vdim
        self.scale, self.window, self.keep_first = float(scale), int(window), int(keep_first)

    def proj_rows(self) -> list:
        return [(self.p + "q", self.heads * self.dk), (self.p + "k", self.kv_heads * self.dk),
                (self.p + "v", self.kv_heads * self.dv)]

    def extra_shapes(self) -> dict:
        return {self.p + "o": (self.width, self.heads * self.dv)}

    def forward(self, parts: list, h: torch.Tensor, w: dict, ctx: StepContext, koff: int, voff: int, soff: int):
        q, k, v = parts
        md = ctx.md
        seqmix.kv_write(ctx.cache, k, v, md.slot_mapping, koff, voff, self.kv_heads, self.dk, self.dv, ctx.block_size)
        o = seqmix.window_attention(q, ctx.cache, md.block_tables, md.query_start_loc, md.seq_lens, koff, voff,
                                    self.heads, self.kv_heads, self.dk, self.dv, ctx.block_size, self.scale,
                                    self.window, self.keep_first, md.max_query_len)
        return ops.linear(o, w[self.p + "o"])


class DecayLinearAttention(Mixer):
    def __init__(self, prefix: str, width: int, heads: int, dim: int, vdim: int, decay: list):
        if len(decay) != heads:
            raise ValueError(f"{prefix}: {len(decay)} decays for {heads} heads")
        self.p, self.width, self.heads, self.qk, self.vd = prefix, width, heads, dim, vdim
        self.decay = [float(a) for a in decay]
        self.state_floats = heads * dim * vdim
        self._decay_dev: dict = {}

    def decay_on(self, device) -> torch.Tensor:
        """The per-head decays as an fp32 device tensor (made when the weights are loaded, so that no
        host-to-device copy falls into a graph capture)."""
        a = self._decay_dev.get(device)
        if a is None:
            a = self._decay_dev[device] = torch.tensor(self.decay, dtype=torch.float32, device=device)
        return a

    def finish_weights(self, w: dict) -> None:
        self.decay_on(w[self.p + "o"].device)

    def proj_rows(self) -> list:
        n, m = self.heads * self.qk, self.heads * self.vd
        return [(self.p + "q", n), (self.p + "k", n), (self.p + "v", m), (self.p + "g", m)]

    def extra_shapes(self) -> dict:
        return {self.p + "o": (self.width, self.heads * self.vd), self.p + "norm": (self.heads * self.vd,)}

    def forward(self, parts: list, h: torch.Tensor, w: dict, ctx: StepContext, koff: int, voff: int, soff: int):
        q, k, v, g = parts
        md = ctx.md
        a = self.decay_on(h.device)
        o = seqmix.decay_scan(q, k, v, a, ctx.state, md.state_rows, soff, md.query_start_loc, md.seq_lens,
                              self.heads, self.qk, self.vd, silu=True, max_query_len=md.max_query_len)
        y = seqmix.gated_rms_norm(o, g, w[self.p + "norm"], ctx.eps, 1, h.dtype)
        return ops.linear(y, w[self.p + "o"])


class MLSTM(Mixer):
    def __init__(self, prefix: str, width: int, heads: int, dim: int, vdim: int, gate_cap: float):
        self.p, self.width, self.heads, self.qk, self.vd = prefix, width, heads, dim, vdim
        self.gate_cap = float(gate_cap)
        self.state_floats = seqmix.mlstm_state_floats(heads, dim, vdim)

    def proj_rows(self) -> list:
        n, m = self.heads * self.qk, self.heads * self.vd
        return [(self.p + "q", n), (self.p + "k", n), (self.p + "v", m), (self.p + "g", m)]

    def extra_shapes(self) -> dict:
        H = self.heads
        return {self.p + "o": (self.width, H * self.vd), self.p + "norm": (H * self.vd,),
                self.p + "i": (H, self.width), self.p + "i.b": (H,), self.p + "f": (H, self.width),
                self.p + "f.b": (H,)}

    def finish_weights(self, w: dict) -> None:
        """Input and forget gate rows as one [2H, width] projection with its bias."""
        p = self.p
        w[p + "_if"] = torch.cat([w.pop(p + "i"), w.pop(p + "f")]).contiguous()
        w[p + "_if.b"] = torch.cat([w.pop(p + "i.b"), w.pop(p + "f.b")]).contiguous()

    def forward(self, parts: list, h: torch.Tensor, w: dict, ctx: StepContext, koff: int, voff: int, soff: int):
        q, k, v, g = parts
        md = ctx.md
        gates = seqmix.gate_linear(h, w[self.p + "_if"], w[self.p + "_if.b"])
        o = seqmix.mlstm_scan(q, k, v, gates, ctx.state, md.state_rows, soff, md.query_start_loc, md.seq_lens,
                              self.heads, self.qk, self.vd, self.gate_cap, self.qk ** -0.5,
                              max_query_len=md.max_query_len)
        y = seqmix.gated_rms_norm(o, g, w[self.p + "norm"], ctx.eps, self.heads, h.dtype)
        return ops.linear(y, w[self.p + "o"])


class ParallelPair(Mixer):
    """Two mixers over the same input.  forward() returns both outputs; the layer norms each over
    the width with `<prefix>left.out` / `<prefix>right.out` and adds half their sum to the stream."""

    def __init__(self, prefix: str, width: int, left: Mixer, right: Mixer):
        self.p, self.width, self.left, self.right = prefix, width, left, right
        self.kv_heads, self.dk, self.dv = left.kv_heads, left.dk, left.dv
        if right.kv_heads:
            raise ValueError("ParallelPair: only the left mixer may keep paged K/V")
        if left.state_floats:
            raise ValueError("ParallelPair: only the right mixer may keep a recurrent state")
        self.state_floats = right.state_floats

    def proj_rows(self) -> list:
        return self.left.proj_rows() + self.right.proj_rows()

    def extra_shapes(self) -> dict:
        return {**self.left.extra_shapes(), **self.right.extra_shapes(),
                self.p + "left.out": (self.width,), self.p + "right.out": (self.width,)}

    def finish_weights(self, w: dict) -> None:
        for m in (self.left, self.right):
            if hasattr(m, "finish_weights"):
                m.finish_weights(w)

    def forward(self, parts: list, h: torch.Tensor, w: dict, ctx: StepContext, koff: int, voff: int, soff: int):
        nl = len(self.left.proj_rows())
        a = self.left.forward(parts[:nl], h, w, ctx, koff, voff, soff)
        b = self.right.forward(parts[nl:], h, w, ctx, koff, voff, soff)
        return a, b


def rotary_frequencies(dims: int, base: float, scaling: Optional[dict] = None) -> torch.Tensor:
    """fp32 [dims / 2]: base^(-2i/dims), computed in float64 on the host.  scaling {factor}: every
    frequency divided by factor.  scaling {factor, low, high, original}: by wavelength l = 2 pi / f,
    kept where l < original / high, divided by factor where l > original / low, and in between blended
    with s = (original / l - low) / (high - low) as (1 - s) f / factor + s f.
    scaling {factor, original, fast, slow}: a ramp over the pair index i between the indices at which
    `fast` and `slow` turns fit into `original` positions, x(t) = dims ln(original / (2 pi t)) / (2 ln base):
    lo = max(floor(x(fast)), 0), hi = min(ceil(x(slow)), dims - 1), r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1),
    frequency r_i f / factor + (1 - r_i) f (rotary_magnitude() gives the factor on cos and sin that goes with it)."""
    f = [float(base) ** (-2.0 * i / dims) for i in range(dims // 2)]
    if scaling:
        factor = float(scaling["factor"])
        if "fast" in scaling:
            orig = float(scaling["original"])

            def index_of(turns: float) -> float:
                return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(float(base)))

            lo = max(math.floor(index_of(float(scaling["fast"]))), 0)
            hi = min(math.ceil(index_of(float(scaling["slow"]))), dims - 1)
            out = []
            for i, fi in enumerate(f):
                r = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
                out.append(fi / factor * r + fi * (1.0 - r))
            f = out
        elif "original" in scaling:
            orig, low, high = float(scaling["original"]), float(scaling["low"]), float(scaling["high"])
            out = []
            for fi in f:
                wave = 2.0 * math.pi / fi
                if wave < orig / high:
                    out.append(fi)
                elif wave > orig / low:
                    out.append(fi / factor)
                else:
                    sm = (orig / wave - low) / (high - low)
                    out.append((1.0 - sm) * fi / factor + sm * fi)
            f = out
        else:
            f = [fi / factor for fi in f]
    return torch.tensor(f, dtype=torch.float64).to(torch.float32)


def rotary_magnitude(scaling: Optional[dict]) -> float:
    """The factor on cos and sin that goes with ramp-blended frequencies: 0.1 ln(factor) + 1."""
    if scaling and "fast" in scaling:
        return 0.1 * math.log(float(scaling["factor"])) + 1.0
    return 1.0


def _fp32(w: dict, name: str) -> None:
    """Constants of a recurrence, a sink or a decay are read as fp32 by the kernels."""
    w[name] = w[name].to(torch.float32).contiguous()


class RotaryAttention(Mixer):
    """sink: None (plain softmax) | "zero" (the denominator holds one more exp(0)) | "learned" (tensor
    `<prefix>sink` [heads]).  rot: {dims, base, scaling}.  rotate_values: the cached value of position j
    is turned by j over all of vdim (plain frequencies of rot.base) and a head's output at position i
    is turned back by i.  kv_from: the layer whose pages this mixer reads; it has no k / v tensors."""

    def __init__(self, prefix: str, width: int, heads: int, kv_heads: int, dim: int, vdim: int, scale: float,
                 rot: dict, qk_norm: bool, sink: Optional[str], rotate_values: bool = False,
                 kv_from: Optional[int] = None):
        if heads % kv_heads:
            raise ValueError(f"{prefix}: {heads} query heads do not divide over {kv_heads} kv heads")
        rd = int(rot["dims"])
        if rd % 2 or rd > dim or (rotate_values and vdim % 2):
            raise ValueError(f"{prefix}: rotary pairs need an even number of dimensions inside the head")
        if sink not in (None, "zero", "learned"):
            raise ValueError(f"{prefix}: unknown sink {sink!r}")
        self.p, self.width = prefix, width
        self.heads, self.kv_heads, self.dk, self.dv = heads, kv_heads, dim, vdim
        self.scale, self.qk_norm, self.sink, self.rotate_values = float(scale), bool(qk_norm), sink, bool(rotate_values)
        self.kv_from = None if kv_from is None else int(kv_from)
        self.freqs = rotary_frequencies(rd, float(rot["base"]), rot.get("scaling") or None)
        self.v_freqs = rotary_frequencies(vdim, float(rot["base"]), None) if rotate_values else None
        self.out_cols = heads * vdim

    def proj_rows(self) -> list:
        rows = [(self.p + "q", self.heads * self.dk)]
        if self.kv_from is None:
            rows += [(self.p + "k", self.kv_heads * self.dk), (self.p + "v", self.kv_heads * self.dv)]
        return rows

    def extra_shapes(self) -> dict:
        sh = {self.p + "o": (self.width, self.heads * self.dv)}
        if self.qk_norm:
            sh[self.p + "q.norm"] = (self.dk,)
            if self.kv_from is None:
                sh[self.p + "k.norm"] = (self.dk,)
        if self.sink == "learned":
            sh[self.p + "sink"] = (self.heads,)
        return sh

    def finish_weights(self, w: dict) -> None:
        dev = w[self.p + "o"].device
        self.freqs = self.freqs.to(dev)
        if self.v_freqs is not None:
            self.v_freqs = self.v_freqs.to(dev)
        if self.sink == "learned":
            _fp32(w, self.p + "sink")
        elif self.sink == "zero":
            w[self.p + "sink"] = torch.zeros(self.heads, dtype=torch.float32, device=dev)

    def mix(self, parts: list, h: torch.Tensor, w: dict, ctx: StepContext, koff: int, voff: int, soff: int,
            out: Optional[torch.Tensor] = None, out_scale: float = 1.0) -> torch.Tensor:
        """The heads' outputs [T, H*dv] before the output projection (into `out`, times out_scale)."""
        md, p = ctx.md, self.p
        q = parts[0]
        k, v = (parts[1], parts[2]) if self.kv_from is None else (None, None)
        seqmix.rope_qkv_cache(q, k, v, md.positions, md.slot_mapping, ctx.cache, koff, voff, self.heads, self.kv_heads,
                              self.dk, self.dv, ctx.block_size, self.freqs, w.get(p + "q.norm"), w.get(p + "k.norm"),
                              ctx.eps, self.v_freqs)
        o = seqmix.window_attention(q, ctx.cache, md.block_tables, md.query_start_loc, md.seq_lens, koff, voff,
                                    self.heads, self.kv_heads, self.dk, self.dv, ctx.block_size, self.scale, 0, 0,
                                    md.max_query_len, sink=w.get(p + "sink"))
        if not self.rotate_values and out is None and out_scale == 1.0:
            return o
        if out is None:
            out = torch.empty_like(o)
        fr = self.v_freqs if self.rotate_values else self.freqs[:0]
        seqmix.rope_rows(o, md.positions, self.heads, self.dv, fr, -1.0, out_scale, out)
        return out

    def forward(self, parts: list, h: torch.Tensor, w: dict, ctx: StepContext, koff: int, voff: int, soff: int):
        return ops.linear(self.mix(parts, h, w, ctx, koff, voff, soff), w[self.p + "o"])


class Mamba2(Mixer):
    """in -> [z | x | B | C | dt]; x, B, C through a causal convolution with bias and SiLU; the scan;
    y * SiLU(z), RMS norm in `norm_groups` slices, output projection.  State per sequence: the scan's
    S [heads, vdim, state] and the convolution's last taps - 1 inputs."""

    def __init__(self, prefix: str, width: int, heads: int, vdim: int, state: int, groups: int, conv: int,
                 norm_groups: int):
        inner = heads * vdim
        if heads % groups or inner % norm_groups or conv < 1:
            raise ValueError(f"{prefix}: heads {heads} / groups {groups} / norm_groups {norm_groups} do not divide")
        self.p, self.width = prefix, width
        self.heads, self.P, self.N, self.G, self.taps, self.norm_groups = heads, vdim, state, groups, conv, norm_groups
        self.inner, self.conv_ch = inner, inner + 2 * groups * state
        self.scan_floats = heads * vdim * state
        self.state_floats = self.scan_floats + (conv - 1) * self.conv_ch
        self.out_cols = inner

    def proj_rows(self) -> list:
        return [(self.p + "in", 2 * self.inner + 2 * self.G * self.N + self.heads)]

    def extra_shapes(self) -> dict:
        p, H = self.p, self.heads
        return {p + "conv": (self.conv_ch, self.taps), p + "conv.b": (self.conv_ch,), p + "dt_bias": (H,),
                p + "A_log": (H,), p + "D": (H,), p + "norm": (self.inner,), p + "o": (self.width, self.inner)}

    def finish_weights(self, w: dict) -> None:
        for n in ("dt_bias", "A_log", "D"):
            _fp32(w, self.p + n)
        w[self.p + "conv"] = w[self.p + "conv"].t().contiguous()  # tap-major for the kernel

    def mix(self, parts: list, h: torch.Tensor, w: dict, ctx: StepContext, koff: int, voff: int, soff: int,
            out: Optional[torch.Tensor] = None, out_scale: float = 1.0) -> torch.Tensor:
        md, p = ctx.md, self.p
        y = parts[0]
        I, GN = self.inner, self.G * self.N
        z, xbc, dt = y[:, :I], y[:, I:I + self.conv_ch], y[:, I + self.conv_ch:]
        c = seqmix.causal_conv(xbc, w[p + "conv"], w[p + "conv.b"], ctx.state, md.state_rows, soff + self.scan_floats,
                               md.query_start_loc, md.seq_lens, silu=True)
        o = seqmix.ssd_scan(c[:, :I], c[:, I:I + GN], c[:, I + GN:], dt, w[p + "dt_bias"], w[p + "A_log"], w[p + "D"],
                            ctx.state, md.state_rows, soff, md.query_start_loc, md.seq_lens, self.heads, self.G,
                            self.N, self.P, max_query_len=md.max_query_len)
        return seqmix.gated_norm(o, z, w[p + "norm"], ctx.eps, self.norm_groups, "silu", True, h.dtype, out_scale, out)

    def forward(self, parts: list, h: torch.Tensor, w: dict, ctx: StepContext, koff: int, voff: int, soff: int):
        return ops.linear(self.mix(parts, h, w, ctx, koff, voff, soff), w[self.p + "o"])


class GatedDeltaRule(Mixer):
    """q, k (qk_heads x dim) and v (heads x vdim) through short convolutions (no bias) and SiLU; q, k
    unit vectors per head, q times dim^-1/2; write strength sigmoid(b h) per head; decay per head and
    key channel from the low-rank pair a1, a2 with dt_bias and A_log; per-head RMS norm of the
    read-out with a weight shared by the heads, times sigmoid of the low-rank gate g1, g2.  State per
    sequence: S [heads, vdim, dim] and the three convolutions' last taps - 1 inputs (one block)."""

    def __init__(self, prefix: str, width: int, heads: int, qk_heads: int, dim: int, vdim: int, conv: int,
                 unit_eps: float = 1e-6):
        if heads % qk_heads or conv < 1:
            raise ValueError(f"{prefix}: {heads} heads do not divide over {qk_heads} q/k heads")
        self.p, self.width = prefix, width
        self.heads, self.G, self.dk, self.dv, self.taps = heads, qk_heads, dim, vdim, conv
        self.unit_eps = float(unit_eps)
        self.conv_ch = 2 * qk_heads * dim + heads * vdim
        self.scan_floats = heads * vdim * dim
        self.state_floats = self.scan_floats + (conv - 1) * self.conv_ch
        # the low-rank pairs' inner sizes are no config entries: a checkpoint's tensors give them
        # (adopt_shapes); these are what random weights are made with
        self.rank_a = self.rank_g = 16
        self.out_cols = heads * vdim

    def adopt_shapes(self, full: dict) -> None:
        a1, g1 = full.get(self.p + "a1"), full.get(self.p + "g1")
        if a1 is not None and a1.dim() == 2:
            self.rank_a = int(a1.shape[0])
        if g1 is not None and g1.dim() == 2:
            self.rank_g = int(g1.shape[0])

    def proj_rows(self) -> list:
        p, n = self.p, self.G * self.dk
        return [(p + "q", n), (p + "k", n), (p + "v", self.heads * self.dv), (p + "a1", self.rank_a),
                (p + "g1", self.rank_g), (p + "b", self.heads)]

    def extra_shapes(self) -> dict:
        p, H, n = self.p, self.heads, self.G * self.dk
        return {p + "q.conv": (n, self.taps), p + "k.conv": (n, self.taps), p + "v.conv": (H * self.dv, self.taps),
                p + "a2": (H * self.dk, self.rank_a), p + "g2": (H * self.dv, self.rank_g), p + "dt_bias": (H * self.dk,),
                p + "A_log": (H,), p + "norm": (self.dv,), p + "o": (self.width, H * self.dv)}

    def finish_weights(self, w: dict) -> None:
        p = self.p
        # one filter over q, k, v's channels, tap-major for the kernel
        w[p + "_conv"] = torch.cat([w.pop(p + "q.conv"), w.pop(p + "k.conv"), w.pop(p + "v.conv")]).t().contiguous()
        # the second halves of the two low-rank pairs as one projection of [a1 h | g1 h]: a2 and g2 on the
        # diagonal, zeros beside them (their products add exactly nothing)
        a2, g2 = w.pop(p + "a2"), w.pop(p + "g2")
        both = torch.zeros(a2.shape[0] + g2.shape[0], a2.shape[1] + g2.shape[1], dtype=a2.dtype, device=a2.device)
        both[:a2.shape[0], :a2.shape[1]] = a2
        both[a2.shape[0]:, a2.shape[1]:] = g2
        w[p + "_ag2"] = both
        _fp32(w, p + "dt_bias")
        _fp32(w, p + "A_log")

    def mix(self, parts: list, h: torch.Tensor, w: dict, ctx: StepContext, koff: int, voff: int, soff: int,
            out: Optional[torch.Tensor] = None, out_scale: float = 1.0) -> torch.Tensor:
        md, p = ctx.md, self.p
        q, k, v, a1, g1, b = parts
        n = self.G * self.dk
        # q, k, v are neighbours in the fused projection (proj_rows): one convolution over all their channels
        qkv = torch.as_strided(q, (q.shape[0], self.conv_ch), q.stride(), q.storage_offset())
        c = seqmix.causal_conv(qkv, w[p + "_conv"], None, ctx.state, md.state_rows, soff + self.scan_floats,
                               md.query_start_loc, md.seq_lens, silu=True)
        # a1 and g1 are neighbours too: one projection gives the decay pre-activations and the gate's
        ra = a1.shape[1]
        ag = ops.linear(torch.as_strided(a1, (a1.shape[0], ra + g1.shape[1]), a1.stride(), a1.storage_offset()).contiguous(),
                        w[p + "_ag2"])
        a, g = ag[:, :self.heads * self.dk], ag[:, self.heads * self.dk:]
        o = seqmix.delta_scan(c[:, :n], c[:, n:2 * n], c[:, 2 * n:], b, a, w[p + "dt_bias"], w[p + "A_log"], ctx.state,
                              md.state_rows, soff, md.query_start_loc, md.seq_lens, self.heads, self.G, self.dk, self.dv,
                              self.dk ** -0.5, self.unit_eps, max_query_len=md.max_query_len)
        return seqmix.gated_norm(o, g, w[p + "norm"], ctx.eps, self.heads, "sigmoid", False, h.dtype, out_scale, out)

    def forward(self, parts: list, h: torch.Tensor, w: dict, ctx: StepContext, koff: int, voff: int, soff: int):
        return ops.linear(self.mix(parts, h, w, ctx, koff, voff, soff), w[self.p + "o"])


class ScaledPair(Mixer):
    """left_scale * left + right_scale * right.  Both output projections are one GEMM: each mixer
    writes its activations, times its scale, into its columns of a shared buffer, and the two
    projection weights stand side by side."""

    def __init__(self, prefix: str, width: int, left: Mixer, right: Mixer, left_scale: float, right_scale: float):
        if right.kv_heads:
            raise ValueError("ScaledPair: only the left mixer may keep paged K/V")
        if left.state_floats:
            raise ValueError("ScaledPair: only the right mixer may keep a recurrent state")
        self.p, self.width, self.left, self.right = prefix, width, left, right
        self.ls, self.rs = float(left_scale), float(right_scale)
        self.kv_heads, self.dk, self.dv = left.kv_heads, left.dk, left.dv
        self.kv_from = getattr(left, "kv_from", None)
        self.state_floats = right.state_floats

    def proj_rows(self) -> list:
        return self.left.proj_rows() + self.right.proj_rows()

    def extra_shapes(self) -> dict:
        return {**self.left.extra_shapes(), **self.right.extra_shapes()}

    def adopt_shapes(self, full: dict) -> None:
        for m in (self.left, self.right):
            if hasattr(m, "adopt_shapes"):
                m.adopt_shapes(full)

    def finish_weights(self, w: dict) -> None:
        for m in (self.left, self.right):
            m.finish_weights(w)
        w[self.p + "_o"] = torch.cat([w.pop(self.left.p + "o"), w.pop(self.right.p + "o")], dim=1).contiguous()

    def forward(self, parts: list, h: torch.Tensor, w: dict, ctx: StepContext, koff: int, voff: int, soff: int):
        nl, cl = len(self.left.proj_rows()), self.left.out_cols
        buf = torch.empty(h.shape[0], cl + self.right.out_cols, dtype=h.dtype, device=h.device)
        self.left.mix(parts[:nl], h, w, ctx, koff, voff, soff, out=buf[:, :cl], out_scale=self.ls)
        self.right.mix(parts[nl:], h, w, ctx, koff, voff, soff, out=buf[:, cl:], out_scale=self.rs)
        return ops.linear(buf, w[self.p + "_o"])


class LatentAttention(Mixer):
    """Per head the query and key are [dim plain | rot_dim rotated], the value has vdim entries.
        c_q = RMSNorm(W_dq h) * w_qn,  q = W_uq c_q
        [c | r] = W_dkv h,  c <- RMSNorm(c) * w_kvn (kv_rank entries),  r rotated (rot_dim entries, one for all heads)
        k_h = [W_uk,h c | r],  v_h = W_uv,h c,  score = scale * q_h . k_h,  out = W_o [softmax-weighted v_h]_h
    The pages hold the row [c | r] per token (one kv head of kv_rank + rot_dim entries); values are the
    row's first kv_rank entries, so nothing is stored twice.  W_uk is folded into the query
    (q'_h = [W_uk,h^T q_h,plain | q_h,rot], score = scale * q'_h . [c | r]) and W_uv is applied to the
    weighted sum of latents: every head attends over the same rows, with head sizes kv_rank + rot_dim
    and kv_rank.  sink: None | "learned" (tensor `<prefix>sink` [heads]).  window > 0: position i sees the
    positions i - window + 1 .. i.  split_pairs: coordinate i of the rotated part pairs with i + rot_dim / 2
    (False: 2i with 2i + 1)."""

    def __init__(self, prefix: str, width: int, heads: int, dim: int, rot_dim: int, vdim: int, kv_rank: int,
                 q_rank: int, scale: float, rot: dict, sink: Optional[str] = "learned", window: int = 0,
                 split_pairs: bool = True):
        if int(rot["dims"]) != rot_dim or rot_dim % 2:
            raise ValueError(f"{prefix}: the rotated part has rot_dim = rot.dims entries, an even number")
        if sink not in (None, "learned"):
            raise ValueError(f"{prefix}: unknown sink {sink!r}")
        if window < 0:
            raise ValueError(f"{prefix}: window {window}")
        self.window, self.split_pairs = int(window), bool(split_pairs)
        self.p, self.width = prefix, width
        self.heads, self.dn, self.dr, self.vd = int(heads), int(dim), int(rot_dim), int(vdim)
        self.rank, self.q_rank, self.scale, self.sink = int(kv_rank), int(q_rank), float(scale), sink
        self.kv_heads, self.dk, self.dv = 1, self.rank + self.dr, 0  # the page row; values are a slice of it
        self.freqs = rotary_frequencies(self.dr, float(rot["base"]), None)

    def proj_rows(self) -> list:
        return [(self.p + "dq", self.q_rank), (self.p + "dkv", self.rank + self.dr)]

    def extra_shapes(self) -> dict:
        p, H = self.p, self.heads
        sh = {p + "dq.norm": (self.q_rank,), p + "dkv.norm": (self.rank,), p + "uq": (H * (self.dn + self.dr), self.q_rank),
              p + "uk": (H * self.dn, self.rank), p + "uv": (H * self.vd, self.rank), p + "o": (self.width, H * self.vd)}
        if self.sink == "learned":
            sh[p + "sink"] = (H,)
        return sh

    def finish_weights(self, w: dict) -> None:
        p, H = self.p, self.heads
        self.freqs = self.freqs.to(w[p + "o"].device)
        if self.sink == "learned":
            _fp32(w, p + "sink")
        # per-head factors of the two batched products: q'_plain = q_plain @ uk[h], out_h = latent_h @ uv[h]^T
        w[p + "uk"] = w[p + "uk"].view(H, self.dn, self.rank).contiguous()
        w[p + "uv"] = w[p + "uv"].view(H, self.vd, self.rank).transpose(1, 2).contiguous()

    def forward(self, parts: list, h: torch.Tensor, w: dict, ctx: StepContext, koff: int, voff: int, soff: int):
        md, p, H = ctx.md, self.p, self.heads
        dq, dkv = parts
        T = h.shape[0]
        cq = seqmix.latent_prep(dq, dkv, md.positions, md.slot_mapping, ctx.cache, koff, self.rank, ctx.block_size,
                                self.freqs, w[p + "dq.norm"], w[p + "dkv.norm"], ctx.eps, self.split_pairs)
        q = ops.linear(cq, w[p + "uq"])  # [T, H * (dn + dr)]
        dq_, dk = self.dn + self.dr, self.dk
        qf = torch.empty(T, H * dk, dtype=q.dtype, device=q.device)
        # the plain part through W_uk^T, head by head, straight into its columns of the folded query
        torch.bmm(q.view(T, H, dq_)[:, :, :self.dn].transpose(0, 1), w[p + "uk"],
                  out=qf.view(T, H, dk)[:, :, :self.rank].transpose(0, 1))
        seqmix.rope_half_into(qf, q, md.positions, H, dq_, self.dn, dk, self.rank, self.freqs, self.split_pairs)
        lat = seqmix.latent_attention(qf, ctx.cache, md.block_tables, md.query_start_loc, md.seq_lens, koff, H, dk,
                                      self.rank, ctx.block_size, self.scale, md.max_query_len,
                                      getattr(md, "max_seq_len", 0), sink=w.get(p + "sink"), window=self.window)
        o = torch.empty(T, H * self.vd, dtype=q.dtype, device=q.device)
        torch.bmm(lat.view(T, H, self.rank).transpose(0, 1), w[p + "uv"], out=o.view(T, H, self.vd).transpose(0, 1))
        return ops.linear(o, w[p + "o"])


class TalkingAttention(Mixer):
    """q = W_q h + b_q, k, v likewise; q and k each RMS-normed over ALL their rows at once (weights
    `<prefix>q.norm` [H dk], `<prefix>k.norm` [G dk]); the first rot.dims coordinates of every head turned as
    pairs (i, i + rot.dims / 2); score_h = sum_g talk[h, g] scale q_g . k_g (`<prefix>talk` [H, H], mixed
    before the mask and the softmax); window > 0: position i sees i - window + 1 .. i; sink: None | "learned"
    (`<prefix>sink` [H], one more term exp(sink_h) in the denominator).  bias / whole_norm / talk can each
    be switched off for a design that lacks them."""

    def __init__(self, prefix: str, width: int, heads: int, kv_heads: int, dim: int, vdim: int, scale: float, rot: dict,
                 window: int = 0, sink: Optional[str] = "learned", bias: bool = True, whole_norm: bool = True,
                 talk: bool = True):
        if heads % kv_heads:
            raise ValueError(f"{prefix}: {heads} query heads do not divide over {kv_heads} kv heads")
        rd = int(rot["dims"])
        if rd % 2 or rd > dim:
            raise ValueError(f"{prefix}: rotary pairs need an even number of dimensions inside the head")
        if sink not in (None, "learned") or window < 0:
            raise ValueError(f"{prefix}: sink {sink!r}, window {window}")
        self.p, self.width = prefix, width
        self.heads, self.kv_heads, self.dk, self.dv = heads, kv_heads, dim, vdim
        self.scale, self.window, self.sink = float(scale), int(window), sink
        self.bias, self.whole_norm, self.talk = bool(bias), bool(whole_norm), bool(talk)
        sc = rot.get("scaling") or None
        self.freqs = rotary_frequencies(rd, float(rot["base"]), sc)
        self.mag = rotary_magnitude(sc)

    def proj_rows(self) -> list:
        return [(self.p + "q", self.heads * self.dk), (self.p + "k", self.kv_heads * self.dk),
                (self.p + "v", self.kv_heads * self.dv)]

    def extra_shapes(self) -> dict:
        p, H, G = self.p, self.heads, self.kv_heads
        sh = {p + "o": (self.width, H * self.dv)}
        if self.bias:
            sh.update({p + "q.b": (H * self.dk,), p + "k.b": (G * self.dk,), p + "v.b": (G * self.dv,)})
        if self.whole_norm:
            sh.update({p + "q.norm": (H * self.dk,), p + "k.norm": (G * self.dk,)})
        if self.talk:
            sh[p + "talk"] = (H, H)
        if self.sink == "learned":
            sh[p + "sink"] = (H,)
        return sh

    def finish_weights(self, w: dict) -> None:
        self.freqs = self.freqs.to(w[self.p + "o"].device)
        if self.talk:
            _fp32(w, self.p + "talk")
        if self.sink == "learned":
            _fp32(w, self.p + "sink")

    def forward(self, parts: list, h: torch.Tensor, w: dict, ctx: StepContext, koff: int, voff: int, soff: int):
        q, k, v = parts
        md, p = ctx.md, self.p
        seqmix.rope_qkv_cache(q, k, v, md.positions, md.slot_mapping, ctx.cache, koff, voff, self.heads, self.kv_heads,
                              self.dk, self.dv, ctx.block_size, self.freqs, w.get(p + "q.norm"), w.get(p + "k.norm"),
                              ctx.eps, bias_q=w.get(p + "q.b"), bias_k=w.get(p + "k.b"), bias_v=w.get(p + "v.b"),
                              norm_whole=self.whole_norm, split_pairs=True, mag=self.mag)
        o = seqmix.window_attention(q, ctx.cache, md.block_tables, md.query_start_loc, md.seq_lens, koff, voff,
                                    self.heads, self.kv_heads, self.dk, self.dv, ctx.block_size, self.scale, self.window,
                                    0, md.max_query_len, sink=w.get(p + "sink"), talk=w.get(p + "talk"),
                                    max_seq_len=getattr(md, "max_seq_len", 0))
        return ops.linear(o, w[p + "o"])


def build_mixer(kind: str, prefix: str, width: int, mc: dict) -> Mixer:
    """A layer's mixer from its config entry (`type` and `mixer` of a Voletar layer)."""
    if kind == "lightning":
        return DecayLinearAttention(prefix, width, int(mc["heads"]), int(mc["dim"]), int(mc["vdim"]), mc["decay"])
    if kind == "parallel":
        l, r = mc["left"], mc["right"]
        mask = l.get("mask") or {}
        left = WindowAttention(prefix + "left.", width, int(l["heads"]), int(l.get("kv_heads", l["heads"])),
                               int(l["dim"]), int(l["vdim"]), float(l["scale"]), int(mask.get("size", 0) or 0),
                               int(mask.get("keep_first", 0) or 0))
        right = MLSTM(prefix + "right.", width, int(r["heads"]), int(r["dim"]), int(r["vdim"]), float(r["gate_cap"]))
        return ParallelPair(prefix, width, left, right)
    raise ValueError(f"unknown mixer type {kind!r}")
