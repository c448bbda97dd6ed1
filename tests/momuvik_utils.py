"""Helpers of the Momuvik tests: small configurations and checkpoints on disk.  The engine, replay
and error helpers are those of the Voletar tests (they know nothing of a design)."""
from __future__ import annotations

import json
import os

import torch

from mxserve.models.momuvik import random_state
from tests.voletar_utils import cut, engine, rel_err, replay  # noqa: F401


def latent(heads=4, dim=24, rot_dim=16, vdim=40, kv_rank=48, q_rank=56, scale=0.2, base=10000.0):
    return {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
            "scale": scale, "rot": {"dims": rot_dim, "base": base}}


def dense(ff=96):
    return {"kind": "dense", "ff": ff}


def moe(experts=6, top=2, ff=40, limit=1.5, shared=(56, 1.0)):
    m = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff, "limit": limit}}
    if shared:
        m["shared"] = {"ff": shared[0], "limit": shared[1]}
    return m


def layer(mixer=None, mlp=None, weights_of=None):
    l = {"type": "latent_attention", "mixer": mixer or latent(), "mlp": mlp}
    if weights_of is not None:
        l["weights_of"] = weights_of
    return l


def config(layers, width=112, vocab=320, eps=1e-5, embed_scale=5.0, mult=0.6):
    return {"architecture": "Momuvik", "width": width, "vocab": vocab, "layers": layers, "norm": {"eps": eps},
            "embedding": {"scale": embed_scale}, "residual_mult": mult}


_A, _B = latent(), latent(heads=3, dim=16, rot_dim=24, vdim=16, kv_rank=40, q_rank=24, scale=0.17, base=3000.0)
BASE = config([layer(_A, dense()), layer(_B, moe()), layer(_A, dense(), weights_of=0), layer(_B, moe(), weights_of=1),
               layer(latent(heads=2, dim=32, rot_dim=8, vdim=24, kv_rank=24, q_rank=32), None),
               layer(_B, moe(experts=5, top=3, ff=32, limit=0.8, shared=None))])


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
