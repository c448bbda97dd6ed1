"""Feed-forward sublayers that a layer-list design can be built from, each with its sizes and
constants as parameters.  Like the mixers (mxserve/models/mixers.py) they name their checkpoint
tensors, re-pack them once when the weights are loaded, and compute from a step's flattened batch.

  GatedFF        W_down(act(W_gate h) * W_up h), gate and up as one projection; act = silu
  CurvedFF       W_down(act(W_up h)) without a gate; act is a parabola above zero and an exponential
                 below it, with two learned numbers (`<p>act`)
  CappedExpert   one small gated unit with clipped pre-activations: g = min(W_gate x, limit),
                 u = clamp(W_up x, -limit, limit), W_down(g * sigmoid(alpha g) * (u + 1))
  RoutedExperts  a router (fp32; sigmoid scores, or a softmax over all experts) picks `top` of `experts`
                 small gated units per token (CappedExperts, or plain SiLU units when no limit is
                 given); the chosen scores (optionally renormalised) weigh each expert's INPUT or its
                 OUTPUT; an optional shared CappedExpert with its own size and limit sees every token
                 unweighted

The kernels are in mxserve/ops/seqmix.py (csrc/mixers/latent_experts.hip on the GPU); the matrix products go
through ops.linear and torch.bmm (hipBLASLt).
"""
from __future__ import annotations

from typing import Optional

import torch

from .. import ops
from ..ops import seqmix


class FeedForward:
    def shapes(self) -> dict:
        """Checkpoint tensor names -> shapes."""
        raise NotImplementedError

    def finish_weights(self, w: dict) -> None:
        pass

    def forward(self, h: torch.Tensor, w: dict) -> torch.Tensor:
        raise NotImplementedError


class GatedFF(FeedForward):
    def __init__(self, prefix: str, width: int, ff: int):
        self.p, self.width, self.ff = prefix, width, int(ff)

    def shapes(self) -> dict:
        p = self.p
        return {p + "gate": (self.ff, self.width), p + "up": (self.ff, self.width), p + "down": (self.width, self.ff)}

    def finish_weights(self, w: dict) -> None:
        p = self.p
        w[p + "_gu"] = torch.cat([w.pop(p + "gate"), w.pop(p + "up")]).contiguous()

    def forward(self, h: torch.Tensor, w: dict) -> torch.Tensor:
        p = self.p
        return ops.linear(seqmix.silu_mul(ops.linear(h, w[p + "_gu"])), w[p + "down"])


class CurvedFF(FeedForward):
    """act(z) = softplus(p) z^2 + z / 2 for z > 0, (1/2 + softplus(q)) (e^z - 1 - z) + z / 2 otherwise, with
    (p, q) = `<p>act`; the two softplus values are formed once, in fp32, when the weights are loaded."""

    def __init__(self, prefix: str, width: int, ff: int):
        self.p, self.width, self.ff = prefix, width, int(ff)

    def shapes(self) -> dict:
        p = self.p
        return {p + "up": (self.ff, self.width), p + "down": (self.width, self.ff), p + "act": (2,)}

    def finish_weights(self, w: dict) -> None:
        sp = torch.nn.functional.softplus(w.pop(self.p + "act").to(torch.float32), threshold=1e9)
        w[self.p + "_act"] = torch.stack([sp[0], 0.5 + sp[1]]).contiguous()

    def forward(self, h: torch.Tensor, w: dict) -> torch.Tensor:
        p = self.p
        return ops.linear(seqmix.xielu(ops.linear(h, w[p + "up"]), w[p + "_act"]), w[p + "down"])


class CappedExpert(FeedForward):
    def __init__(self, prefix: str, width: int, ff: int, limit: float, alpha: float = 1.702):
        self.p, self.width, self.ff = prefix, width, int(ff)
        self.limit, self.alpha = float(limit), float(alpha)

    def shapes(self) -> dict:
        p = self.p
        return {p + "gate": (self.ff, self.width), p + "up": (self.ff, self.width), p + "down": (self.width, self.ff)}

    def finish_weights(self, w: dict) -> None:
        p = self.p
        w[p + "_gu"] = torch.cat([w.pop(p + "gate"), w.pop(p + "up")]).contiguous()

    def forward(self, h: torch.Tensor, w: dict) -> torch.Tensor:
        p = self.p
        return ops.linear(seqmix.capped_glu(ops.linear(h, w[p + "_gu"]), self.limit, self.alpha), w[p + "down"])


class RoutedExperts(FeedForward):
    """Tensors: `<p>router` [E, width], `<p>e<i>.{gate,up,down}`, optionally `<p>shared.{gate,up,down}`.
    Loaded as `<p>_gu` [E, 2 ff, width] and `<p>_down` [E, width, ff].

    Two ways through the experts, both exact (a token never meets an expert it did not choose with
    anything but a zero row, and a zero row gives a zero output: g = 0):
      batched   every expert over all T rows of `spread_scaled` in two batched products -- no sorting
                and no host round trip, so a captured single-token step can replay it; E / top times
                the needed products, which steps of a few tokens do not feel (they stream the
                experts' weights either way)
      sorted    rows sorted by expert (expert_align, gather_scaled), one product pair per expert that
                got rows (one host read of the E + 1 offsets), expert_combine gathers each token's rows
    """

    BATCHED_MAX_TOKENS = 32    # always batched up to this many tokens ...
    BATCHED_MAX_ROWS = 1024    # ... and beyond while experts x tokens stays within this many rows

    def __init__(self, prefix: str, width: int, experts: int, top: int, ff: int, limit: Optional[float],
                 shared: Optional[CappedExpert] = None, alpha: float = 1.702, renorm: bool = False,
                 score: str = "sigmoid", weigh: str = "input"):
        """limit None: an expert is W_down(SiLU(W_gate x) * W_up x).  score: sigmoid | softmax (over all
        experts, before the choice).  weigh: input | output (what a chosen score multiplies)."""
        if not 1 <= top <= experts:
            raise ValueError(f"{prefix}: top {top} of {experts} experts")
        if score not in ("sigmoid", "softmax") or weigh not in ("input", "output"):
            raise ValueError(f"{prefix}: score {score!r}, weigh {weigh!r}")
        self.p, self.width, self.E, self.top, self.ff = prefix, width, int(experts), int(top), int(ff)
        self.limit = None if limit is None else float(limit)
        self.alpha, self.renorm, self.shared = float(alpha), bool(renorm), shared
        self.softmax, self.on_output = score == "softmax", weigh == "output"

    def act(self, gu: torch.Tensor) -> torch.Tensor:
        if self.limit is None:
            return seqmix.silu_mul(gu)
        return seqmix.capped_glu(gu, self.limit, self.alpha)

    def shapes(self) -> dict:
        p, sh = self.p, {self.p + "router": (self.E, self.width)}
        for e in range(self.E):
            sh[f"{p}e{e}.gate"] = sh[f"{p}e{e}.up"] = (self.ff, self.width)
            sh[f"{p}e{e}.down"] = (self.width, self.ff)
        if self.shared is not None:
            sh.update(self.shared.shapes())
        return sh

    def finish_weights(self, w: dict) -> None:
        p = self.p
        w[p + "_gu"] = torch.stack([torch.cat([w.pop(f"{p}e{e}.gate"), w.pop(f"{p}e{e}.up")]) for e in range(self.E)]).contiguous()
        w[p + "_down"] = torch.stack([w.pop(f"{p}e{e}.down") for e in range(self.E)]).contiguous()
        if self.shared is not None:
            self.shared.finish_weights(w)

    def route(self, h: torch.Tensor, w: dict) -> tuple:
        logits = seqmix.gate_linear(h, w[self.p + "router"], None)  # fp32 products and sums
        return seqmix.route_topk(logits, self.top, self.renorm, self.softmax)

    def forward(self, h: torch.Tensor, w: dict) -> torch.Tensor:
        p, T = self.p, h.shape[0]
        tw, ids = self.route(h, w)
        w_in, w_out = (None, tw) if self.on_output else (tw, None)
        extra = self.shared.forward(h, w) if self.shared is not None else None
        gu, down = w[p + "_gu"], w[p + "_down"]
        capturing = h.is_cuda and torch.cuda.is_current_stream_capturing()
        if T <= self.BATCHED_MAX_TOKENS or T * self.E <= self.BATCHED_MAX_ROWS or capturing:
            xs = seqmix.spread_scaled(h, w_in, ids, self.E)  # [E, T, W]
            a = self.act(torch.bmm(xs, gu.transpose(1, 2)).view(self.E * T, -1))
            ys = torch.bmm(a.view(self.E, T, -1), down.transpose(1, 2))  # [E, T, W]
            if w_out is None:
                return seqmix.expert_combine(ys, None, self.E, T, extra, row_stride=T)
            # weights on the outputs: a token's k chosen slabs, row (expert, t) of the stack
            return seqmix.expert_combine(ys, ids.reshape(-1), self.top, T, extra, row_stride=T, weights=w_out, by_expert=True)
        offs, inv = seqmix.expert_align(ids, self.E)
        xs = seqmix.gather_scaled(h, w_in, inv, self.top)
        ys = torch.empty_like(xs)
        o = offs.tolist()  # the one host read of this path
        for e in range(self.E):
            a0, a1 = o[e], o[e + 1]
            if a1 > a0:
                ys[a0:a1] = ops.linear(self.act(ops.linear(xs[a0:a1], gu[e])), down[e])
        return seqmix.expert_combine(ys, inv, self.top, T, extra, weights=w_out)
