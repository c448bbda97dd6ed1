"""Model architecture configs and the built-in model registry.

The reference never ships model code; it names models in its manifests
(`examples/deploy/vllm/agg.yaml:35` Llama-3.2-1B-Instruct, `examples/dgdr/trtllm/dgdr.yaml:11`
Qwen3-0.6B) and BASELINE.json names Llama-3-8B, Llama-3-70B and Mixtral-8x7B.  The GPU box has no
network, so every model can be instantiated from the shapes below with random weights; if a
`config.json` is found on disk (HF_HOME / a local path) it overrides the built-in entry.
"""
from __future__ import annotations

import dataclasses
import json
import os
from dataclasses import dataclass, field
from typing import Optional


@dataclass
class ModelConfig:
    name: str
    arch: str  # "llama" | "qwen3" | "mixtral" | "voletar" | "tapasun" | "momuvik" | "seradra"
    hidden_size: int
    intermediate_size: int
    num_layers: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    vocab_size: int
    rope_theta: float = 10000.0
    rms_norm_eps: float = 1e-5
    tie_word_embeddings: bool = False
    max_position_embeddings: int = 8192
    # llama3 rope scaling (factor, low_freq_factor, high_freq_factor, original_max_pos) or None
    rope_scaling: Optional[dict] = None
    qk_norm: bool = False
    # MoE
    num_experts: int = 0
    num_experts_per_tok: int = 0
    # tokenizer / chat
    bos_token_id: Optional[int] = None
    eos_token_ids: list = field(default_factory=list)
    chat_template: str = "llama3"
    # designs whose config lists their layers (arch "voletar", "tapasun", "momuvik", "seradra"): the checkpoint's own
    # config.json structure -- per-layer mixer type and sizes, norm eps and the design's other
    # constants -- as the design's module (mxserve/models/<arch>.py) reads it.  None for the uniform
    # transformer families.
    arch_config: Optional[dict] = None

    @property
    def is_moe(self) -> bool:
        return self.num_experts > 0

    @property
    def has_recurrent_state(self) -> bool:
        """Layers that carry a per-sequence state from token to token (linear attention, mLSTM, state
        spaces, delta rule, short convolutions): no prefix caching (a cached block has no state to
        resume from) and one state slot per request."""
        return self.arch in ("voletar", "tapasun")

    @property
    def q_size(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_kv_heads * self.head_dim

    def kv_bytes_per_token(self, dtype_bytes: int = 2) -> int:
        if self.arch_config is not None:
            from .hybrid import design_module
            plan = design_module(self.arch).layer_plan(self.arch_config)
            return sum(r.kv_heads * (r.dk + r.dv) for r in plan.attn_runs) * dtype_bytes
        return self.num_layers * 2 * self.num_kv_heads * self.head_dim * dtype_bytes

    def num_params(self) -> int:
        if self.arch_config is not None:
            from .hybrid import design_module
            shapes = design_module(self.arch).weight_shapes(self.arch_config)
            return sum(int(__import__("math").prod(v)) for v in shapes.values())
        h, i, L = self.hidden_size, self.intermediate_size, self.num_layers
        attn = h * (self.q_size + 2 * self.kv_size) + self.q_size * h
        if self.is_moe:
            mlp = self.num_experts * 3 * h * i + h * self.num_experts
        else:
            mlp = 3 * h * i
        per_layer = attn + mlp + 2 * h + (2 * self.head_dim if self.qk_norm else 0)
        emb = self.vocab_size * h
        return L * per_layer + emb + (0 if self.tie_word_embeddings else emb) + h

    def to_dict(self) -> dict:
        return dataclasses.asdict(self)


_LLAMA3_EOS = [128001, 128008, 128009]
_LLAMA31_ROPE = {"rope_type": "llama3", "factor": 32.0, "low_freq_factor": 1.0,
                 "high_freq_factor": 4.0, "original_max_position_embeddings": 8192}

# Shapes: public HF config.json of each model.
REGISTRY: dict[str, ModelConfig] = {}


def _reg(cfg: ModelConfig, *aliases: str) -> None:
    REGISTRY[cfg.name.lower()] = cfg
    for a in aliases:
        REGISTRY[a.lower()] = cfg


_reg(ModelConfig(
    name="meta-llama/Llama-3.2-1B-Instruct", arch="llama", hidden_size=2048, intermediate_size=8192,
    num_layers=16, num_heads=32, num_kv_heads=8, head_dim=64, vocab_size=128256, rope_theta=500000.0,
    rms_norm_eps=1e-5, tie_word_embeddings=True, max_position_embeddings=131072,
    rope_scaling=dict(_LLAMA31_ROPE), bos_token_id=128000, eos_token_ids=list(_LLAMA3_EOS),
    chat_template="llama3"), "llama-3.2-1b", "meta-llama/Llama-3.2-1B", "llama-3.2-1b-instruct")

_reg(ModelConfig(
    name="Qwen/Qwen3-0.6B", arch="qwen3", hidden_size=1024, intermediate_size=3072, num_layers=28,
    num_heads=16, num_kv_heads=8, head_dim=128, vocab_size=151936, rope_theta=1000000.0,
    rms_norm_eps=1e-6, tie_word_embeddings=True, max_position_embeddings=40960, qk_norm=True,
    bos_token_id=None, eos_token_ids=[151645, 151643], chat_template="chatml"), "qwen3-0.6b")

_reg(ModelConfig(
    name="meta-llama/Meta-Llama-3-8B-Instruct", arch="llama", hidden_size=4096, intermediate_size=14336,
    num_layers=32, num_heads=32, num_kv_heads=8, head_dim=128, vocab_size=128256, rope_theta=500000.0,
    rms_norm_eps=1e-5, max_position_embeddings=8192, bos_token_id=128000,
    eos_token_ids=[128001, 128009], chat_template="llama3"),
    "llama-3-8b", "meta-llama/Meta-Llama-3-8B", "meta-llama/Llama-3.1-8B-Instruct")

_reg(ModelConfig(
    name="meta-llama/Meta-Llama-3-70B-Instruct", arch="llama", hidden_size=8192, intermediate_size=28672,
    num_layers=80, num_heads=64, num_kv_heads=8, head_dim=128, vocab_size=128256, rope_theta=500000.0,
    rms_norm_eps=1e-5, max_position_embeddings=8192, bos_token_id=128000,
    eos_token_ids=[128001, 128009], chat_template="llama3"),
    "llama-3-70b", "meta-llama/Meta-Llama-3-70B", "meta-llama/Llama-3.1-70B-Instruct")

_reg(ModelConfig(
    name="mistralai/Mixtral-8x7B-Instruct-v0.1", arch="mixtral", hidden_size=4096, intermediate_size=14336,
    num_layers=32, num_heads=32, num_kv_heads=8, head_dim=128, vocab_size=32000, rope_theta=1000000.0,
    rms_norm_eps=1e-5, max_position_embeddings=32768, num_experts=8, num_experts_per_tok=2,
    bos_token_id=1, eos_token_ids=[2], chat_template="mistral"),
    "mixtral-8x7b", "mistralai/Mixtral-8x7B-v0.1")

# Tiny configs with the same code paths, used by CPU tests.
_reg(ModelConfig(
    name="tiny-llama", arch="llama", hidden_size=128, intermediate_size=256, num_layers=2, num_heads=4,
    num_kv_heads=2, head_dim=32, vocab_size=512, rope_theta=10000.0, tie_word_embeddings=True,
    max_position_embeddings=2048, rope_scaling=dict(_LLAMA31_ROPE, original_max_position_embeddings=64),
    bos_token_id=1, eos_token_ids=[2], chat_template="llama3"))
_reg(ModelConfig(
    name="tiny-qwen3", arch="qwen3", hidden_size=128, intermediate_size=256, num_layers=2, num_heads=4,
    num_kv_heads=2, head_dim=64, vocab_size=512, rope_theta=1000000.0, rms_norm_eps=1e-6,
    tie_word_embeddings=True, max_position_embeddings=2048, qk_norm=True, eos_token_ids=[2],
    chat_template="chatml"))
_reg(ModelConfig(
    name="tiny-mixtral", arch="mixtral", hidden_size=128, intermediate_size=192, num_layers=2, num_heads=4,
    num_kv_heads=2, head_dim=32, vocab_size=512, rope_theta=1000000.0, max_position_embeddings=2048,
    num_experts=4, num_experts_per_tok=2, bos_token_id=1, eos_token_ids=[2], chat_template="mistral"))
_reg(ModelConfig(
    name="tiny-qwen3-gpu", arch="qwen3", hidden_size=256, intermediate_size=512, num_layers=2, num_heads=4,
    num_kv_heads=2, head_dim=128, vocab_size=1024, rope_theta=1000000.0, rms_norm_eps=1e-6,
    tie_word_embeddings=True, max_position_embeddings=4096, qk_norm=True, eos_token_ids=[2],
    chat_template="chatml"))
_reg(ModelConfig(
    name="tiny-mixtral-gpu", arch="mixtral", hidden_size=256, intermediate_size=512, num_layers=2, num_heads=8,
    num_kv_heads=2, head_dim=64, vocab_size=1024, rope_theta=1000000.0, max_position_embeddings=4096,
    num_experts=4, num_experts_per_tok=2, bos_token_id=1, eos_token_ids=[2], chat_template="mistral"))
# A GPU-test config: real head dims (64/128) and GQA ratios, few layers.
_reg(ModelConfig(
    name="small-llama", arch="llama", hidden_size=1024, intermediate_size=2816, num_layers=4, num_heads=16,
    num_kv_heads=4, head_dim=64, vocab_size=32000, rope_theta=500000.0, tie_word_embeddings=True,
    max_position_embeddings=8192, bos_token_id=1, eos_token_ids=[2], chat_template="llama3"))


def voletar_config(name: str, d: dict) -> ModelConfig:
    """A Voletar checkpoint's config.json: `width`, `vocab`, `layers` (each with `type`, `mixer`, `mlp`),
    optional `loop` {start, stop, times}, `norm.eps`, optional `logit_softcap`.  The uniform fields are
    filled from the first layer for the code that sizes things from them (profiler, planner)."""
    layers = d["layers"]
    mx = layers[0]["mixer"]
    att = mx.get("left", mx)
    ffs = [l["mlp"]["ff"] for l in layers if l.get("mlp")]
    keep = {k: d[k] for k in ("layers", "loop", "norm", "logit_softcap", "width", "vocab") if k in d}
    return ModelConfig(
        name=name, arch="voletar", hidden_size=int(d["width"]), intermediate_size=max(ffs) if ffs else 0,
        num_layers=len(layers), num_heads=int(att["heads"]), num_kv_heads=int(att.get("kv_heads", att["heads"])),
        head_dim=int(att["dim"]), vocab_size=int(d["vocab"]), rms_norm_eps=float(d.get("norm", {}).get("eps", 1e-5)),
        tie_word_embeddings=False, max_position_embeddings=int(d.get("max_position_embeddings", 1 << 20)),
        bos_token_id=d.get("bos_token_id"), eos_token_ids=list(d.get("eos_token_ids") or []),
        chat_template="chatml", arch_config=keep)


# A small Voletar (random weights) with every kind of layer and a looped span, for tests and smoke runs.
_reg(voletar_config("tiny-voletar", {
    "architecture": "Voletar", "width": 128, "vocab": 512, "norm": {"eps": 1e-5}, "logit_softcap": 25.0,
    "loop": {"start": 1, "stop": 3, "times": 2},
    "layers": [
        {"type": "lightning", "mlp": None,
         "mixer": {"heads": 2, "dim": 32, "vdim": 64, "decay": [0.9, 0.99]}},
        {"type": "parallel", "mlp": {"kind": "dense", "ff": 256},
         "mixer": {"left": {"heads": 4, "kv_heads": 2, "dim": 32, "vdim": 48, "scale": 0.18,
                            "mask": {"size": 40, "keep_first": 3}},
                   "right": {"heads": 2, "dim": 16, "vdim": 32, "gate_cap": 10.0}}},
        {"type": "lightning", "mlp": {"kind": "dense", "ff": 192},
         "mixer": {"heads": 4, "dim": 16, "vdim": 16, "decay": [0.7, 0.9, 0.97, 0.995]}},
        {"type": "parallel", "mlp": None,
         "mixer": {"left": {"heads": 2, "kv_heads": 2, "dim": 64, "vdim": 64, "scale": 0.125,
                            "mask": {"size": 16, "keep_first": 0}},
                   "right": {"heads": 4, "dim": 32, "vdim": 16, "gate_cap": 8.0}}}]}))


def tapasun_config(name: str, d: dict) -> ModelConfig:
    """A Tapasun checkpoint's config.json: `width`, `vocab`, `embedding.scale`, `norm.eps`, `layers` (each
    with `type` mamba2 | attention | parallel, `mixer`, `mlp` or null).  The uniform fields are filled
    from the first attention for the code that sizes things from them (profiler, planner)."""
    layers = d["layers"]
    atts = [l["mixer"].get("left", l["mixer"]) for l in layers if l["type"] in ("attention", "parallel")]
    att = atts[0] if atts else {"heads": 1, "kv_heads": 1, "dim": int(d["width"])}
    ffs = [l["mlp"]["ff"] for l in layers if l.get("mlp")]
    keep = {k: d[k] for k in ("layers", "norm", "embedding", "width", "vocab") if k in d}
    return ModelConfig(
        name=name, arch="tapasun", hidden_size=int(d["width"]), intermediate_size=max(ffs) if ffs else 0,
        num_layers=len(layers), num_heads=int(att["heads"]), num_kv_heads=int(att.get("kv_heads", att["heads"])),
        head_dim=int(att["dim"]), vocab_size=int(d["vocab"]), rms_norm_eps=float((d.get("norm") or {}).get("eps", 1e-5)),
        tie_word_embeddings=False, max_position_embeddings=int(d.get("max_position_embeddings", 1 << 20)),
        bos_token_id=d.get("bos_token_id"), eos_token_ids=list(d.get("eos_token_ids") or []),
        chat_template="chatml", arch_config=keep)


# A small Tapasun (random weights) with every kind of layer, a layer without feed-forward and shared pages.
_reg(tapasun_config("tiny-tapasun", {
    "architecture": "Tapasun", "width": 96, "vocab": 384, "norm": {"eps": 1e-5}, "embedding": {"scale": 4.0},
    "layers": [
        {"type": "attention", "mlp": {"kind": "dense", "ff": 160},
         "mixer": {"heads": 4, "kv_heads": 2, "dim": 32, "vdim": 16, "scale": 0.2,
                   "rot": {"dims": 16, "base": 10000.0,
                           "scaling": {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64}}}},
        {"type": "mamba2", "mlp": None,
         "mixer": {"heads": 3, "vdim": 16, "state": 24, "groups": 1, "conv": 4, "norm_groups": 3}},
        {"type": "parallel", "mlp": {"kind": "dense", "ff": 128}, "mixer": {
            "left": {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 32, "scale": 0.3,
                     "rot": {"dims": 8, "base": 10000.0, "scaling": {"factor": 2.0}}},
            "right": {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 24, "conv": 3},
            "left_scale": 0.7, "right_scale": 1.3}},
        {"type": "attention", "mlp": {"kind": "dense", "ff": 160},
         "mixer": {"heads": 4, "kv_heads": 2, "dim": 32, "vdim": 16, "scale": 0.2, "kv_from": 0,
                   "rot": {"dims": 16, "base": 10000.0,
                           "scaling": {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64}}}}]}))


def momuvik_config(name: str, d: dict) -> ModelConfig:
    """A Momuvik checkpoint's config.json: `width`, `vocab`, `embedding.scale`, `norm.eps`, `residual_mult`,
    `layers` (each with `type` latent_attention, `mixer`, `mlp` dense | moe | null, optionally `weights_of`).
    The uniform fields are filled from the first layer for the code that sizes things from them."""
    layers = d["layers"]
    att = layers[0]["mixer"]
    ffs = [int(l["mlp"]["ff"]) if l["mlp"].get("kind", "dense") == "dense" else int(l["mlp"]["expert"]["ff"])
           for l in layers if l.get("mlp")]
    moes = [l["mlp"]["router"] for l in layers if l.get("mlp") and l["mlp"].get("kind") == "moe"]
    keep = {k: d[k] for k in ("layers", "norm", "embedding", "residual_mult", "width", "vocab") if k in d}
    return ModelConfig(
        name=name, arch="momuvik", hidden_size=int(d["width"]), intermediate_size=max(ffs) if ffs else 0,
        num_layers=len(layers), num_heads=int(att["heads"]), num_kv_heads=1,
        head_dim=int(att["dim"]) + int(att["rot_dim"]), vocab_size=int(d["vocab"]),
        rms_norm_eps=float((d.get("norm") or {}).get("eps", 1e-5)), tie_word_embeddings=True,
        max_position_embeddings=int(d.get("max_position_embeddings", 1 << 20)),
        num_experts=max((int(r["experts"]) for r in moes), default=0),
        num_experts_per_tok=max((int(r["top"]) for r in moes), default=0),
        bos_token_id=d.get("bos_token_id"), eos_token_ids=list(d.get("eos_token_ids") or []),
        chat_template="chatml", arch_config=keep)


def _latent(heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, base=10000.0):
    return {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
            "scale": scale, "rot": {"dims": rot_dim, "base": base}}


# A small Momuvik (random weights): a dense and a routed feed-forward, a layer without one, shared weights.
_reg(momuvik_config("tiny-momuvik", {
    "architecture": "Momuvik", "width": 96, "vocab": 384, "norm": {"eps": 1e-5}, "embedding": {"scale": 6.0},
    "residual_mult": 0.8,
    "layers": [
        {"type": "latent_attention", "mixer": _latent(4, 16, 8, 24, 32, 40, 0.2), "mlp": {"kind": "dense", "ff": 160}},
        {"type": "latent_attention", "mixer": _latent(3, 24, 16, 16, 48, 24, 0.16, 5000.0),
         "mlp": {"kind": "moe", "router": {"experts": 6, "top": 2}, "expert": {"ff": 48, "limit": 2.0},
                 "shared": {"ff": 64, "limit": 1.2}}},
        {"type": "latent_attention", "mixer": _latent(4, 16, 8, 24, 32, 40, 0.2), "mlp": {"kind": "dense", "ff": 160},
         "weights_of": 0},
        {"type": "latent_attention", "mixer": _latent(2, 32, 8, 32, 24, 32, 0.15), "mlp": None}]}))


def seradra_config(name: str, d: dict) -> ModelConfig:
    """A Seradra checkpoint's config.json: `width`, `vocab`, `norm.eps`, `layers` (each with `type` attention |
    latent_attention, `mixer`, `mlp` dense | moe | null).  The uniform fields are filled from the first layer
    for the code that sizes things from them."""
    layers = d["layers"]
    att = layers[0]["mixer"] if layers else {"heads": 1, "dim": int(d["width"])}
    latent = bool(layers) and layers[0]["type"] == "latent_attention"
    ffs = [int(l["mlp"]["ff"]) if l["mlp"].get("kind", "dense") == "dense" else int(l["mlp"]["expert"]["ff"])
           for l in layers if l.get("mlp")]
    moes = [l["mlp"]["router"] for l in layers if l.get("mlp") and l["mlp"].get("kind") == "moe"]
    keep = {k: d[k] for k in ("layers", "norm", "width", "vocab") if k in d}
    return ModelConfig(
        name=name, arch="seradra", hidden_size=int(d["width"]), intermediate_size=max(ffs) if ffs else 0,
        num_layers=len(layers), num_heads=int(att["heads"]),
        num_kv_heads=1 if latent else int(att.get("kv_heads", att["heads"])),
        head_dim=int(att["dim"]) + (int(att["rot_dim"]) if latent else 0), vocab_size=int(d["vocab"]),
        rms_norm_eps=float((d.get("norm") or {}).get("eps", 1e-5)), tie_word_embeddings=False,
        max_position_embeddings=int(d.get("max_position_embeddings", 1 << 20)),
        num_experts=max((int(r["experts"]) for r in moes), default=0),
        num_experts_per_tok=max((int(r["top"]) for r in moes), default=0),
        bos_token_id=d.get("bos_token_id"), eos_token_ids=list(d.get("eos_token_ids") or []),
        chat_template="chatml", arch_config=keep)


def _talking(heads, kv_heads, dim, vdim, scale, window, rot_dims, base=10000.0, scaling=None):
    rot = {"dims": rot_dims, "base": base}
    if scaling:
        rot["scaling"] = scaling
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "mask": {"size": window},
            "rot": rot}


# A small Seradra (random weights): both mixers, a dense and a routed feed-forward, a layer without one.
_reg(seradra_config("tiny-seradra", {
    "architecture": "Seradra", "width": 96, "vocab": 384, "norm": {"eps": 1e-5},
    "layers": [
        {"type": "attention", "mlp": {"kind": "dense", "ff": 160},
         "mixer": _talking(4, 2, 32, 16, 0.2, 24, 16, 10000.0,
                           {"factor": 4.0, "original": 64, "fast": 16.0, "slow": 1.0})},
        {"type": "latent_attention", "mlp": {"kind": "moe", "router": {"experts": 6, "top": 2}, "expert": {"ff": 48}},
         "mixer": dict(_latent(3, 24, 16, 16, 48, 24, 0.16, 5000.0), mask={"size": 20})},
        {"type": "attention", "mlp": None, "mixer": _talking(3, 3, 16, 32, 0.25, 40, 8, 3000.0)},
        {"type": "latent_attention", "mlp": {"kind": "dense", "ff": 128},
         "mixer": dict(_latent(4, 16, 8, 24, 32, 40, 0.2), mask={"size": 33})}]}))


def _from_hf_json(name: str, d: dict) -> ModelConfig:
    if d.get("architecture") == "Seradra":
        return seradra_config(name, d)
    if d.get("architecture") == "Momuvik":
        return momuvik_config(name, d)
    if d.get("architecture") == "Voletar":
        return voletar_config(name, d)
    if d.get("architecture") == "Tapasun":
        return tapasun_config(name, d)
    arch_list = d.get("architectures") or []
    mt = d.get("model_type", "")
    if "qwen3" in mt or any("Qwen3" in a for a in arch_list):
        arch = "qwen3"
    elif "mixtral" in mt or d.get("num_local_experts"):
        arch = "mixtral"
    else:
        arch = "llama"
    nh = d["num_attention_heads"]
    hd = d.get("head_dim") or d["hidden_size"] // nh
    eos = d.get("eos_token_id")
    eos = eos if isinstance(eos, list) else ([eos] if eos is not None else [])
    rs = d.get("rope_scaling")
    if rs is not None and rs.get("rope_type", rs.get("type")) != "llama3":
        rs = None
    return ModelConfig(
        name=name, arch=arch, hidden_size=d["hidden_size"], intermediate_size=d["intermediate_size"],
        num_layers=d["num_hidden_layers"], num_heads=nh, num_kv_heads=d.get("num_key_value_heads", nh),
        head_dim=hd, vocab_size=d["vocab_size"], rope_theta=float(d.get("rope_theta", 10000.0)),
        rms_norm_eps=float(d.get("rms_norm_eps", 1e-5)),
        tie_word_embeddings=bool(d.get("tie_word_embeddings", False)),
        max_position_embeddings=int(d.get("max_position_embeddings", 8192)), rope_scaling=rs,
        qk_norm=(arch == "qwen3"), num_experts=int(d.get("num_local_experts", 0) or 0),
        num_experts_per_tok=int(d.get("num_experts_per_tok", 0) or 0), bos_token_id=d.get("bos_token_id"),
        eos_token_ids=eos,
        chat_template={"qwen3": "chatml", "mixtral": "mistral"}.get(arch, "llama3"))


def find_local_model_dir(name: str) -> Optional[str]:
    """Locate a HF snapshot for `name` on disk (a path, or HF_HOME hub cache). No network."""
    if os.path.isdir(name) and os.path.exists(os.path.join(name, "config.json")):
        return name
    home = os.environ.get("HF_HOME") or os.path.join(os.path.expanduser("~"), ".cache", "huggingface")
    repo_dir = os.path.join(home, "hub", "models--" + name.replace("/", "--"), "snapshots")
    if os.path.isdir(repo_dir):
        for snap in sorted(os.listdir(repo_dir)):
            p = os.path.join(repo_dir, snap)
            if os.path.exists(os.path.join(p, "config.json")):
                return p
    return None


def get_model_config(name: str) -> ModelConfig:
    """`name@layers=N` keeps a model's real shapes with only its first N layers (tests and probes of
    big models on one GPU, e.g. Llama-3-70B TP=8 with 8 ranks sharing the test box's GPU)."""
    if "@layers=" in name:
        base, n = name.split("@layers=", 1)
        cfg = get_model_config(base)
        return dataclasses.replace(cfg, num_layers=int(n), name=name)
    local = find_local_model_dir(name)
    if local is not None:
        with open(os.path.join(local, "config.json")) as f:
            return _from_hf_json(name, json.load(f))
    key = name.lower()
    if key in REGISTRY:
        cfg = REGISTRY[key]
        return dataclasses.replace(cfg, name=name if "/" in name else cfg.name)
    # tolerate org-less or path-like names ("/models/Llama-3.2-1B-Instruct")
    base = os.path.basename(key.rstrip("/"))
    for k, cfg in REGISTRY.items():
        if k.split("/")[-1] == base:
            return dataclasses.replace(cfg, name=name)
    raise KeyError(f"unknown model {name!r}; known: {sorted(set(c.name for c in REGISTRY.values()))}")
