"""Momuvik: a decoder whose config.json lists its layers.  A layer is
    x <- x + m * mixer(norm1(x)),   x <- x + m * ff(norm2(x))        (the second when it has a feed-forward)
with m = `residual_mult` and RMS norms whose weights are stored as their difference from one.  The
mixer is a latent attention with a learned sink per head (mixers.LatentAttention); the feed-forward is
a gated SiLU unit or a sigmoid-routed mixture of capped experts with an optional shared expert
(feedforward.GatedFF, RoutedExperts).  A layer with `weights_of: j` runs layer j's tensors (mixer,
feed-forward and norms) over pages of its own.

The embedding is multiplied by `embedding.scale`; the logits are embed (unscaled) times the final norm
of x.  The residual stream is fp32 from the embedding to the final norm: a sublayer's output is scaled,
added, and the next norm taken in one kernel (seqmix.resid_update).  A layer's two down-projections are
one GEMM, so are a feed-forward's gate and up.  One forward = one engine step over a flattened token
batch, paged latents through the block tables.
"""
from __future__ import annotations

import sys
from typing import Optional

import torch

from .. import ops
from ..ops import seqmix
from .config import ModelConfig
from .feedforward import CappedExpert, FeedForward, GatedFF, RoutedExperts
from .hybrid import HybridLM, LayerPlan, plan_runs
from .mixers import LatentAttention, Mixer, StepContext


def owners(ac: dict) -> list:
    """For every layer, the layer whose tensors it runs (itself unless it names another)."""
    layers = ac["layers"]
    out = []
    for i, l in enumerate(layers):
        j, seen = i, set()
        while layers[j].get("weights_of") is not None:
            if j in seen:
                raise ValueError(f"layer {i}: weights_of goes in a circle")
            seen.add(j)
            j = int(layers[j]["weights_of"])
            if not 0 <= j < len(layers):
                raise ValueError(f"layer {i}: weights_of names no layer")
        out.append(j)
    return out


def build_mixer(kind: str, prefix: str, width: int, mc: dict) -> Mixer:
    if kind == "latent_attention":
        return LatentAttention(prefix, width, int(mc["heads"]), int(mc["dim"]), int(mc["rot_dim"]), int(mc["vdim"]),
                               int(mc["kv_rank"]), int(mc["q_rank"]), float(mc["scale"]), mc["rot"], sink="learned")
    raise ValueError(f"unknown mixer type {kind!r}")


def build_ff(prefix: str, width: int, mlp: Optional[dict]) -> Optional[FeedForward]:
    if not mlp:
        return None
    kind = mlp.get("kind", "dense")
    if kind == "dense":
        return GatedFF(prefix, width, int(mlp["ff"]))
    if kind == "moe":
        sh = mlp.get("shared")
        shared = CappedExpert(prefix + "shared.", width, int(sh["ff"]), float(sh["limit"])) if sh else None
        return RoutedExperts(prefix, width, int(mlp["router"]["experts"]), int(mlp["router"]["top"]),
                             int(mlp["expert"]["ff"]), float(mlp["expert"]["limit"]), shared)
    raise ValueError(f"unknown feed-forward kind {kind!r}")


def mixers_of(ac: dict) -> list:
    """One mixer per layer; a layer that runs another's tensors has that layer's mixer object."""
    own, W, out = owners(ac), int(ac["width"]), []
    for i, l in enumerate(ac["layers"]):
        out.append(build_mixer(l["type"], f"l{i}.mix.", W, l["mixer"]) if own[i] == i else None)
    return [out[j] for j in own]


def ffs_of(ac: dict) -> list:
    own, W, out = owners(ac), int(ac["width"]), []
    for i, l in enumerate(ac["layers"]):
        out.append(build_ff(f"l{i}.mlp.", W, l.get("mlp")) if own[i] == i else None)
    return [out[j] for j in own]


def layer_plan(ac: dict, block_size: int = 16, mixers: Optional[list] = None) -> LayerPlan:
    """Every layer runs once, in order, each over pages of its own."""
    mixers = mixers or mixers_of(ac)
    return plan_runs([(i, None, False) for i in range(len(mixers))], mixers, block_size)


def weight_shapes(ac: dict, mixers: Optional[list] = None) -> dict:
    """Checkpoint tensor names and shapes; layers that run another's tensors have none."""
    W, V = int(ac["width"]), int(ac["vocab"])
    mixers = mixers or mixers_of(ac)
    ffs, own = ffs_of(ac), owners(ac)
    sh = {"embed": (V, W), "final.norm": (W,)}
    for i, m in enumerate(mixers):
        if own[i] != i:
            continue
        p = f"l{i}."
        sh[p + "norm1"] = (W,)
        for name, rows in m.proj_rows():
            sh[name] = (rows, W)
        sh.update(m.extra_shapes())
        if ffs[i] is not None:
            sh[p + "norm2"] = (W,)
            sh.update(ffs[i].shapes())
    return sh


def random_state(ac: dict, seed: int = 0, device="cpu") -> dict:
    """Random weights in checkpoint naming (fp32): projections ~ N(0, 1/fan_in), norm weights around
    their neutral value, sinks and routers spread so that they matter."""
    g = torch.Generator(device=device).manual_seed(seed)
    rnd = lambda shape: torch.randn(shape, generator=g, device=device)  # noqa: E731
    out = {}
    for name, shape in weight_shapes(ac).items():
        leaf = name.rsplit(".", 1)[-1]
        if leaf in ("norm1", "norm2") or name == "final.norm":
            t = 0.1 * rnd(shape)
        elif leaf == "norm":
            t = 1.0 + 0.1 * rnd(shape)
        elif leaf == "sink":
            t = rnd(shape)
        elif leaf == "router":
            t = 2.0 * rnd(shape) * shape[1] ** -0.5
        else:
            t = rnd(shape) * shape[1] ** -0.5
        out[name] = t
    return out


class MomuvikLM(HybridLM):
    design = sys.modules[__name__]

    def __init__(self, cfg: ModelConfig, device, dtype: torch.dtype = torch.bfloat16, block_size: int = 16):
        super().__init__(cfg, device, dtype, block_size)
        self.embed_scale = float((self.ac.get("embedding") or {}).get("scale", 1.0))
        self.mult = float(self.ac.get("residual_mult", 1.0))
        self.own = owners(self.ac)
        self.ffs = ffs_of(self.ac)

    def weight_owner(self, i: int) -> int:
        return self.own[i]

    def finish_weights(self, w: dict) -> None:
        for i, f in enumerate(self.ffs):
            if f is not None and self.own[i] == i:
                f.finish_weights(w)

    def lm_head_weight(self) -> torch.Tensor:
        return self.w["embed"]

    def forward(self, input_ids: torch.Tensor, md, kv_cache: torch.Tensor) -> torch.Tensor:
        """Final-normed hidden states of the rows md.logits_indices."""
        w, eps, dt, m = self.w, self.eps, self.dtype, self.mult
        ctx = StepContext(md=md, cache=kv_cache, state=md.state, block_size=self.block_size, eps=eps)
        x = seqmix.embed_scaled(input_ids, w["embed"], self.embed_scale)
        tap = self.layer_tap
        runs = self.plan.runs
        h = seqmix.resid_update(x, None, eps, norm_w=w[f"l{self.own[0]}.norm1"], out_dtype=dt, w_offset=1.0) if runs else None
        for n, run in enumerate(runs):
            i = run.layer
            p = f"l{self.own[i]}."
            nxt = w[f"l{self.own[runs[n + 1].layer]}.norm1"] if n + 1 < len(runs) else None
            mx, ff = self.mixers[i], self.ffs[i]
            y = mx.forward(self._split(ops.linear(h, w[p + "mix._in"]), mx), h, w, ctx, run.koff, run.voff, run.soff)
            if ff is not None:
                h = seqmix.resid_update(x, y, eps, norm_w=w[p + "norm2"], out_dtype=dt, a_scale=m, w_offset=1.0)
                y = ff.forward(h, w)
            h = seqmix.resid_update(x, y, eps, norm_w=nxt, out_dtype=dt, a_scale=m, w_offset=1.0)
            if tap is not None:
                tap.append(x.clone())
        xs = x.index_select(0, md.logits_indices)
        return seqmix.resid_update(xs, None, eps, norm_w=w["final.norm"], out_dtype=dt, w_offset=1.0)

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        """fp32 logits: the embedding table itself (without its scale) is the output projection."""
        return seqmix.softcap(ops.linear(hidden, self.w["embed"]), 0.0)
