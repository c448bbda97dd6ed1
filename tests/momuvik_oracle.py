"""A plain float64 implementation of the Momuvik design, one function per mechanism, one token at a
time.  It shares no code with mxserve: the tests compare the engine against it.

A model is (config dict, {tensor name: float64 numpy array}).  `Oracle.step(token)` feeds one token
of one sequence and returns (logits, the residual stream after every layer).

Notation: h is a sublayer's input [width]; rms(x) = x / sqrt(mean(x^2) + eps).  Keys and values are
kept per head here, expanded from the latent at once (the engine keeps the latent only).
"""
from __future__ import annotations

import math

import numpy as np


# ------------------------------------------------------------------------------------- small pieces
def rms(x, eps):
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def offset_norm(x, w, eps):
    """The layers' norm: its weight is stored as the difference from one."""
    return rms(x, eps) * (1.0 + w)


def plain_norm(x, w, eps):
    return rms(x, eps) * w


def rotate_halves(x, pos, base):
    """x [..., n], n even: coordinate i pairs with i + n/2; the pair turns by pos * base^(-2i/n)."""
    n = x.shape[-1]
    half = n // 2
    f = np.array([float(base) ** (-2.0 * i / n) for i in range(half)])
    a = pos * f
    c, s = np.cos(a), np.sin(a)
    u, v = x[..., :half], x[..., half:]
    return np.concatenate([u * c - v * s, v * c + u * s], axis=-1)


# ------------------------------------------------------------------------------------- attention
def sink_softmax_mix(scores, values, sink):
    """scores [n], values [n, dv]: softmax weights whose denominator holds exp(sink) as well."""
    m = max(float(scores.max()), float(sink))
    e = np.exp(scores - m)
    return (e[:, None] * values).sum(0) / (e.sum() + math.exp(sink - m))


class LatentAttention:
    """Queries through a normed low-rank latent; keys and values expanded from a normed shared latent
    c, plus one rotated key part that all heads share.  Per head the query and key are
    [dim unrotated | rot_dim rotated]."""

    def __init__(self, mc: dict, w: dict, p: str, eps: float):
        self.H, self.dn, self.dr, self.dv, self.rank = (int(mc[k]) for k in ("heads", "dim", "rot_dim", "vdim", "kv_rank"))
        self.scale, self.base, self.eps = float(mc["scale"]), float(mc["rot"]["base"]), eps
        if int(mc["rot"]["dims"]) != self.dr:
            raise ValueError("the rotated part is rot_dim wide")
        self.w = {k: w[p + k] for k in ("dq", "dq.norm", "uq", "dkv", "dkv.norm", "uk", "uv", "sink", "o")}
        self.keys, self.vals = [], []  # per token: [H, dn + dr], [H, dv]

    def step(self, h, pos):
        w, H = self.w, self.H
        cq = plain_norm(w["dq"] @ h, w["dq.norm"], self.eps)
        q = (w["uq"] @ cq).reshape(H, self.dn + self.dr)
        q = np.concatenate([q[:, :self.dn], rotate_halves(q[:, self.dn:], pos, self.base)], axis=-1)
        d = w["dkv"] @ h
        c = plain_norm(d[:self.rank], w["dkv.norm"], self.eps)
        kr = rotate_halves(d[self.rank:], pos, self.base)
        kn = (w["uk"] @ c).reshape(H, self.dn)
        self.keys.append(np.concatenate([kn, np.broadcast_to(kr, (H, self.dr))], axis=-1))
        self.vals.append((w["uv"] @ c).reshape(H, self.dv))
        K, V = np.stack(self.keys), np.stack(self.vals)  # [n, H, .]
        out = np.empty((H, self.dv))
        for hd in range(H):
            out[hd] = sink_softmax_mix((K[:, hd] @ q[hd]) * self.scale, V[:, hd], float(w["sink"][hd]))
        return w["o"] @ out.reshape(-1)


# ------------------------------------------------------------------------------------- feed-forward
def dense_ff(h, w, p):
    return w[p + "down"] @ (silu(w[p + "gate"] @ h) * (w[p + "up"] @ h))


def capped_expert(x, w, p, limit):
    g = np.minimum(w[p + "gate"] @ x, limit)
    u = np.clip(w[p + "up"] @ x, -limit, limit)
    return w[p + "down"] @ (g * sigmoid(1.702 * g) * (u + 1.0))


def routed_ff(h, w, p, mlp):
    """Sigmoid scores; the `top` largest are taken as they are and weigh each chosen expert's INPUT;
    a shared expert, if the layer has one, sees h itself."""
    E, top = int(mlp["router"]["experts"]), int(mlp["router"]["top"])
    s = sigmoid(w[p + "router"] @ h)
    chosen = np.argsort(-s, kind="stable")[:top]
    y = np.zeros_like(h)
    for e in chosen:
        y = y + capped_expert(s[e] * h, w, f"{p}e{int(e)}.", float(mlp["expert"]["limit"]))
    if mlp.get("shared"):
        y = y + capped_expert(h, w, p + "shared.", float(mlp["shared"]["limit"]))
    return y, s


# ------------------------------------------------------------------------------------- the model
class Oracle:
    def __init__(self, cfg: dict, w: dict):
        self.cfg, self.w = cfg, w
        self.eps = float(cfg["norm"]["eps"])
        self.m = float(cfg.get("residual_mult", 1.0))
        self.escale = float((cfg.get("embedding") or {}).get("scale", 1.0))
        self.src = []  # the layer whose tensors layer i runs (a named layer may itself name another)
        for i in range(len(cfg["layers"])):
            j = i
            while cfg["layers"][j].get("weights_of") is not None:
                j = int(cfg["layers"][j]["weights_of"])
            self.src.append(j)
        self.mixers = []
        for i, l in enumerate(cfg["layers"]):
            if l["type"] != "latent_attention":
                raise ValueError(l["type"])
            self.mixers.append(LatentAttention(l["mixer"], w, f"l{self.src[i]}.mix.", self.eps))
        self.pos = 0
        # per token: the smallest gap, over its routed layers, between the last chosen score and the best one left out
        self.margins = []

    def step(self, token: int):
        w, eps, m = self.w, self.eps, self.m
        x = w["embed"][token] * self.escale
        streams, margin = [], math.inf
        for i, l in enumerate(self.cfg["layers"]):
            p = f"l{self.src[i]}."
            x = x + m * self.mixers[i].step(offset_norm(x, w[p + "norm1"], eps), self.pos)
            mlp = l.get("mlp")
            if mlp:
                h = offset_norm(x, w[p + "norm2"], eps)
                if mlp.get("kind", "dense") == "dense":
                    y = dense_ff(h, w, p + "mlp.")
                else:
                    y, sc = routed_ff(h, w, p + "mlp.", mlp)
                    top = int(mlp["router"]["top"])
                    if top < len(sc):
                        srt = np.sort(sc)[::-1]
                        margin = min(margin, float(srt[top - 1] - srt[top]))
                x = x + m * y
            streams.append(x.copy())
        self.pos += 1
        self.margins.append(margin)
        logits = w["embed"] @ offset_norm(x, w["final.norm"], eps)
        return logits, streams


def run(cfg: dict, w: dict, tokens, margins=None) -> tuple:
    """(logits [n, vocab], streams [layers, n, width]) of one sequence; a list passed as `margins`
    receives every token's routing margin."""
    o = Oracle(cfg, w)
    lg, st = [], []
    for t in tokens:
        a, b = o.step(int(t))
        lg.append(a)
        st.append(b)
    if margins is not None:
        margins.extend(o.margins)
    return np.stack(lg), np.stack([np.stack(s) for s in st]).transpose(1, 0, 2)
