"""What the designs whose config lists their layers share (mxserve/models/voletar.py,
mxserve/models/tapasun.py, mxserve/models/momuvik.py, mxserve/models/seradra.py): the plan of layer runs with every run's place inside a cache block and a
state slot, and the model surface the runner expects (weights in a flat dict, the mixers' input
projections fused into one GEMM per layer, cache geometry from the plan).

A design's module provides `mixers_of(ac)` (its config's layers as mxserve/models/mixers.py objects),
`layer_plan(ac, block_size, mixers)` and `weight_shapes(ac, mixers)`; `design_module(arch)` finds it.
"""
from __future__ import annotations

import importlib
from dataclasses import dataclass, field
from typing import Optional

import torch

from ..parallel.comm import get_tp
from .config import ModelConfig
from .mixers import Mixer

HYBRID_ARCHS = ("voletar", "tapasun", "momuvik", "seradra")


def design_module(arch: str):
    if arch not in HYBRID_ARCHS:
        raise ValueError(f"{arch!r} is not a design with a layer list")
    return importlib.import_module(f"{__package__}.{arch}")


@dataclass
class LayerRun:
    """One execution of a layer: a looped span's layers appear once per pass."""
    layer: int
    loop_pass: Optional[int]  # pass number inside the looped span, None outside it
    first_of_pass: bool
    kv_heads: int = 0
    dk: int = 0
    dv: int = 0
    koff: int = 0  # element offsets inside a cache block
    voff: int = 0
    soff: int = 0  # float offset inside a state slot
    owns_kv: bool = True  # False: the run reads the pages of another layer's run (koff / voff are that run's)


@dataclass
class LayerPlan:
    runs: list = field(default_factory=list)
    block_elems: int = 0  # K/V elements one block holds over all runs
    state_floats: int = 0

    @property
    def attn_runs(self) -> list:
        """The runs that keep pages of their own."""
        return [r for r in self.runs if r.kv_heads and r.owns_kv]


def plan_runs(order: list, mixers: list, block_size: int) -> LayerPlan:
    """order: [(layer, loop pass or None, first of its pass)] in execution order.  A mixer with
    `kv_from = j` gets the offsets of layer j's run of the same pass, which must come earlier and keep
    pages of the same geometry."""
    plan = LayerPlan()
    done: dict = {}
    for i, t, first in order:
        m: Mixer = mixers[i]
        r = LayerRun(i, t, first, m.kv_heads, m.dk, m.dv)
        src = getattr(m, "kv_from", None)
        if src is not None:
            o = done.get((int(src), t))
            if o is None or not o.owns_kv:
                raise ValueError(f"layer {i}: kv_from {src} is not an earlier layer with keys and values of its own")
            if (o.kv_heads, o.dk, o.dv) != (m.kv_heads, m.dk, m.dv):
                raise ValueError(f"layer {i}: its key/value heads differ from layer {src}'s")
            r.koff, r.voff, r.owns_kv = o.koff, o.voff, False
        elif m.kv_heads:
            r.koff = plan.block_elems
            r.voff = r.koff + m.kv_heads * block_size * m.dk
            plan.block_elems = r.voff + m.kv_heads * block_size * m.dv
        r.soff = plan.state_floats
        plan.state_floats += m.state_floats
        plan.runs.append(r)
        done[(i, t)] = r
    return plan


class HybridLM:
    """Same surface as TransformerLM for the model runner: weights in a flat dict, forward() over a
    step's batch, compute_logits().  A subclass sets `design` (its module) and writes forward()."""

    is_recurrent = True
    design = None

    def __init__(self, cfg: ModelConfig, device, dtype: torch.dtype = torch.bfloat16, block_size: int = 16):
        name = type(self).__name__
        if cfg.arch_config is None:
            raise ValueError(f"{name} needs the checkpoint's layer list (ModelConfig.arch_config)")
        if get_tp().tp_size != 1:
            raise ValueError(f"{name} runs on one GPU per replica (its state and pages are not sharded)")
        self.cfg, self.ac = cfg, cfg.arch_config
        self.device, self.dtype = torch.device(device), dtype
        self.tp_rank, self.tp_size = 0, 1
        self.block_size = block_size
        self.width = int(self.ac["width"])
        self.eps = float((self.ac.get("norm") or {}).get("eps", 1e-5))
        self.mixers = self.design.mixers_of(self.ac)
        self.plan = self.design.layer_plan(self.ac, block_size, self.mixers)
        self.state_floats = self.plan.state_floats
        self.vocab_local = cfg.vocab_size
        self.w: dict[str, torch.Tensor] = {}
        self.kv_scales = [{"k_scale": 1.0, "v_scale": 1.0}]
        self.pf_chain = False
        # debugging tap: a list here receives the residual stream after every layer run (fp32 copies)
        self.layer_tap: Optional[list] = None

    # ------------------------------------------------------------------ cache / state geometry
    def kv_cache_shape(self, num_blocks: int, block_size: int) -> tuple:
        if block_size != self.block_size:
            self.block_size = block_size
            self.plan = self.design.layer_plan(self.ac, block_size, self.mixers)
        return (num_blocks, max(self.plan.block_elems, 1))

    # ------------------------------------------------------------------ weights
    def init_random(self, seed: int = 0, std: float = 0.02) -> None:
        self.load_full_state(self.design.random_state(self.ac, seed, device=self.device))

    def load_full_state(self, full: dict) -> None:
        """Checkpoint tensors (any float dtype; integer tables stay integers) -> this model's dtype, the
        mixers' input projections concatenated into one weight per layer."""
        for m in self.mixers:  # sizes that only the tensors give
            if hasattr(m, "adopt_shapes"):
                m.adopt_shapes(full)
        shapes = self.design.weight_shapes(self.ac, self.mixers)
        missing = [k for k in shapes if k not in full]
        if missing:
            raise KeyError(f"checkpoint lacks {missing[:4]}{' ...' if len(missing) > 4 else ''}")
        w = {}
        for name, shape in shapes.items():
            t = full[name]
            if tuple(t.shape) != tuple(shape):
                raise ValueError(f"{name}: shape {tuple(t.shape)}, the config gives {tuple(shape)}")
            w[name] = t.to(device=self.device, dtype=self.dtype if t.is_floating_point() else t.dtype).contiguous()
        for i, m in enumerate(self.mixers):
            if self.weight_owner(i) != i:  # the layer runs another layer's tensors (and its mixer object)
                continue
            rows = m.proj_rows()
            w[f"l{i}.mix._in"] = torch.cat([w.pop(name) for name, _ in rows]).contiguous()
            if hasattr(m, "finish_weights"):
                m.finish_weights(w)
        self.finish_weights(w)
        self.w = w

    def weight_owner(self, i: int) -> int:
        """The layer whose tensors layer i runs: itself, unless the design lets layers share weights."""
        return i

    def finish_weights(self, w: dict) -> None:
        """A design's own re-packing of its non-mixer weights."""

    def prepare_fused_prefill(self, tuning: bool = True, max_rows: int = 8192) -> bool:
        return False

    def calibrate_kv_scales(self, block_size: int = 16, n: int = 256, headroom: float = 2.0) -> None:
        raise ValueError(f"{type(self).__name__} keeps its K/V pages in the model dtype (no fp8 KV cache)")

    def lm_head_weight(self) -> torch.Tensor:
        return self.w["head"]

    def tunable_shapes(self) -> dict:
        """Decode-GEMM shapes for the start-up tuner: none, the projections run hipBLASLt's own choice."""
        return {}

    def _split(self, y: torch.Tensor, mixer: Mixer) -> list:
        parts, c = [], 0
        for _, rows in mixer.proj_rows():
            parts.append(y[:, c:c + rows])
            c += rows
        return parts
