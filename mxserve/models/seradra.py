"""Seradra: a decoder whose config.json lists its layers.  The sublayers read the stream itself and
only their OUTPUT is normed:
    x <- x + norm1(mixer(x)),   x <- x + norm2(ff(x))        (the second when the layer has a feed-forward)
with RMS norms whose weights are stored as their difference from one (so is the norm of the embedding,
which comes before everything, and the final one).  After layer i the stream goes on as a weighted sum
of the embedding output X_0 and every layer's result X_1 .. X_(i+1) so far, with the layer's own
coefficients `l<i>.dwa` (i + 2 numbers); X_(i+1) itself stays what the layer produced.

  attention          mixers.TalkingAttention: biased projections, one RMS norm over all of q and one over
                     all of k, half-split rotary pairs on part of each head with ramp-blended frequencies,
                     the heads' scores mixed by `talk` before the softmax, sliding window, learned sink
  latent_attention   mixers.LatentAttention with neighbouring rotary pairs, a sliding window and no sink
  mlp dense          feedforward.CurvedFF (no gate, a two-parameter activation)
  mlp moe            feedforward.RoutedExperts: softmax over all experts, the `top` largest scores as they
                     are weigh the outputs of plain SiLU units

The stream is fp32 from the embedding's norm to the final norm and lives, with every earlier result, in
one buffer [layers + 2, T, width]: a layer updates its slab in place (seqmix.resid_update: norm of the
sublayer's output, weight, add, and the next sublayer's input as one cast), and seqmix.depth_mix writes
the weighted sum into the next slab.  A layer's input projections are one GEMM, so are an expert's gate
and up.  One forward = one engine step over a flattened token batch, paged keys / values / latents
through the block tables.
"""
from __future__ import annotations

import sys
from typing import Optional

import torch

from .. import ops
from ..ops import seqmix
from .config import ModelConfig
from .feedforward import CurvedFF, FeedForward, RoutedExperts
from .hybrid import HybridLM, LayerPlan, plan_runs
from .mixers import LatentAttention, Mixer, StepContext, TalkingAttention


def build_mixer(kind: str, prefix: str, width: int, mc: dict) -> Mixer:
    window = int((mc.get("mask") or {}).get("size", 0) or 0)
    if kind == "attention":
        return TalkingAttention(prefix, width, int(mc["heads"]), int(mc.get("kv_heads", mc["heads"])), int(mc["dim"]),
                                int(mc["vdim"]), float(mc["scale"]), mc["rot"], window=window, sink="learned")
    if kind == "latent_attention":
        return LatentAttention(prefix, width, int(mc["heads"]), int(mc["dim"]), int(mc["rot_dim"]), int(mc["vdim"]),
                               int(mc["kv_rank"]), int(mc["q_rank"]), float(mc["scale"]), mc["rot"], sink=None,
                               window=window, split_pairs=False)
    raise ValueError(f"unknown mixer type {kind!r}")


def build_ff(prefix: str, width: int, mlp: Optional[dict]) -> Optional[FeedForward]:
    if not mlp:
        return None
    kind = mlp.get("kind", "dense")
    if kind == "dense":
        return CurvedFF(prefix, width, int(mlp["ff"]))
    if kind == "moe":
        return RoutedExperts(prefix, width, int(mlp["router"]["experts"]), int(mlp["router"]["top"]),
                             int(mlp["expert"]["ff"]), None, score="softmax", weigh="output")
    raise ValueError(f"unknown feed-forward kind {kind!r}")


def mixers_of(ac: dict) -> list:
    return [build_mixer(l["type"], f"l{i}.mix.", int(ac["width"]), l["mixer"]) for i, l in enumerate(ac["layers"])]


def ffs_of(ac: dict) -> list:
    return [build_ff(f"l{i}.mlp.", int(ac["width"]), l.get("mlp")) for i, l in enumerate(ac["layers"])]


def layer_plan(ac: dict, block_size: int = 16, mixers: Optional[list] = None) -> LayerPlan:
    """Every layer runs once, in order, each over pages of its own."""
    mixers = mixers or mixers_of(ac)
    return plan_runs([(i, None, False) for i in range(len(mixers))], mixers, block_size)


def weight_shapes(ac: dict, mixers: Optional[list] = None) -> dict:
    """Checkpoint tensor names and shapes."""
    W, V = int(ac["width"]), int(ac["vocab"])
    mixers = mixers or mixers_of(ac)
    ffs = ffs_of(ac)
    sh = {"embed": (V, W), "embed.norm": (W,), "final.norm": (W,), "head": (V, W)}
    for i, m in enumerate(mixers):
        p = f"l{i}."
        sh[p + "norm1"] = (W,)
        for name, rows in m.proj_rows():
            sh[name] = (rows, W)
        sh.update(m.extra_shapes())
        if ffs[i] is not None:
            sh[p + "norm2"] = (W,)
            sh.update(ffs[i].shapes())
        sh[p + "dwa"] = (i + 2,)
    return sh


def random_state(ac: dict, seed: int = 0, device="cpu") -> dict:
    """Random weights in checkpoint naming (fp32): projections ~ N(0, 1/fan_in); stream norms around
    zero, inner norms around one; biases, sinks, the head-mixing matrix (identity plus noise), routers
    and the depth coefficients (mostly the newest result, some of every older one) spread so that each
    mechanism matters."""
    g = torch.Generator(device=device).manual_seed(seed)
    rnd = lambda shape: torch.randn(shape, generator=g, device=device)  # noqa: E731
    out = {}
    for name, shape in weight_shapes(ac).items():
        leaf = name.rsplit(".", 1)[-1]
        if leaf in ("norm1", "norm2") or name in ("final.norm", "embed.norm"):
            t = 0.1 * rnd(shape)
        elif leaf == "norm":
            t = 1.0 + 0.1 * rnd(shape)
        elif leaf == "b":
            t = 0.3 * rnd(shape)
        elif leaf in ("sink", "act"):
            t = rnd(shape)
        elif leaf == "talk":
            t = torch.eye(shape[0], device=device) + 0.4 * rnd(shape) * shape[0] ** -0.5
        elif leaf == "dwa":
            t = 0.2 * rnd(shape)
            t[-1] += 1.0
        elif leaf == "router":
            t = 2.0 * rnd(shape) * shape[1] ** -0.5
        elif name == "embed":
            t = rnd(shape)
        else:
            t = rnd(shape) * shape[1] ** -0.5
        out[name] = t
    return out


class SeradraLM(HybridLM):
    design = sys.modules[__name__]

    def __init__(self, cfg: ModelConfig, device, dtype: torch.dtype = torch.bfloat16, block_size: int = 16):
        super().__init__(cfg, device, dtype, block_size)
        self.ffs = ffs_of(self.ac)

    def finish_weights(self, w: dict) -> None:
        for i, f in enumerate(self.ffs):
            if f is not None:
                f.finish_weights(w)
            w[f"l{i}.dwa"] = w[f"l{i}.dwa"].to(torch.float32).contiguous()

    def forward(self, input_ids: torch.Tensor, md, kv_cache: torch.Tensor) -> torch.Tensor:
        """Final-normed hidden states of the rows md.logits_indices."""
        w, eps, dt = self.w, self.eps, self.dtype
        ctx = StepContext(md=md, cache=kv_cache, state=md.state, block_size=self.block_size, eps=eps)
        runs = self.plan.runs
        T = input_ids.shape[0]
        # slab 0: the embedding output; slab n + 1: what run n produced; a run starts from the weighted sum
        # that the run before it left in its slab
        hist = torch.empty(len(runs) + 2, T, self.width, dtype=torch.float32, device=w["embed"].device)
        h = seqmix.embed_normed(input_ids, w["embed"], w["embed.norm"], eps, 1.0, hist[0], cast_dtype=dt, copy=hist[1])
        tap = self.layer_tap
        for n, run in enumerate(runs):
            i = run.layer
            p = f"l{i}."
            x = hist[n + 1]
            mx, ff = self.mixers[i], self.ffs[i]
            y = mx.forward(self._split(ops.linear(h, w[p + "mix._in"]), mx), h, w, ctx, run.koff, run.voff, run.soff)
            if ff is not None:
                h = seqmix.resid_update(x, y, eps, wa=w[p + "norm1"], wa_offset=1.0, cast_dtype=dt)
                seqmix.resid_update(x, ff.forward(h, w), eps, wa=w[p + "norm2"], wa_offset=1.0)
            else:
                seqmix.resid_update(x, y, eps, wa=w[p + "norm1"], wa_offset=1.0)
            h = seqmix.depth_mix(hist, n + 2, w[p + "dwa"], cast_dtype=dt if n + 1 < len(runs) else None)
            if tap is not None:
                tap.append(hist[n + 2].clone())
        xs = hist[len(runs) + 1].index_select(0, md.logits_indices)
        return seqmix.resid_update(xs, None, eps, norm_w=w["final.norm"], out_dtype=dt, w_offset=1.0)

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        """fp32 logits."""
        return seqmix.softcap(ops.linear(hidden, self.w["head"]), 0.0)
