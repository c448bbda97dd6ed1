"""Helpers of the Seradra tests: small configurations and checkpoints on disk.  The engine, replay
and error helpers are those of the Voletar tests (they know nothing of a design)."""
from __future__ import annotations

import json
import os

import torch

from mxserve.models.seradra import random_state
from tests.voletar_utils import cut, engine, rel_err, replay  # noqa: F401

RAMP = {"factor": 3.0, "original": 48, "fast": 8.0, "slow": 1.0}


def talking(heads=4, kv_heads=2, dim=24, vdim=40, scale=0.2, window=21, rot_dims=12, base=10000.0, scaling=RAMP):
    rot = {"dims": rot_dims, "base": base}
    if scaling:
        rot["scaling"] = dict(scaling)
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "mask": {"size": window},
            "rot": rot}


def latent(heads=3, dim=24, rot_dim=16, vdim=40, kv_rank=48, q_rank=56, scale=0.2, window=27, base=5000.0):
    return {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
            "scale": scale, "mask": {"size": window}, "rot": {"dims": rot_dim, "base": base}}


def dense(ff=96):
    return {"kind": "dense", "ff": ff}


def moe(experts=6, top=2, ff=40):
    return {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}


def layer(mixer, mlp=None):
    kind = "latent_attention" if "kv_rank" in mixer else "attention"
    return {"type": kind, "mixer": mixer, "mlp": mlp}


def config(layers, width=112, vocab=320, eps=1e-5):
    return {"architecture": "Seradra", "width": width, "vocab": vocab, "layers": layers, "norm": {"eps": eps}}


BASE = config([layer(talking(), dense()), layer(latent(), moe()), layer(talking(heads=6, kv_heads=6, dim=16, vdim=16, window=40,
                                                                                rot_dims=16, base=300.0, scaling=None)),
               layer(latent(heads=5, dim=16, rot_dim=8, vdim=24, kv_rank=40, q_rank=24, scale=0.17, window=19), dense(64)),
               layer(talking(heads=3, kv_heads=1, dim=32, vdim=24, scale=0.15, window=33, rot_dims=8), moe(experts=5, top=3, ff=32))])


def write_checkpoint(path, cfg: dict, seed: int = 0, tweak=None) -> dict:
    """config.json + model.safetensors (bf16) under `path`; returns the stored weights as float64 arrays."""
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    sd = {k: v.to(torch.bfloat16).contiguous() for k, v in random_state(cfg, seed).items()}
    if tweak:
        tweak(sd)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file(sd, os.path.join(path, "model.safetensors"))
    return {k: v.double().numpy() for k, v in sd.items()}
