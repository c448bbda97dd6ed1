"""A plain float64 implementation of the Seradra design, one function per mechanism, one token at a
time.  It shares no code with mxserve: the tests compare the engine against it.

A model is (config dict, {tensor name: float64 numpy array}).  `Oracle.step(token)` feeds one token
of one sequence and returns (logits, the stream that leaves every layer).

Notation: x is the stream [width]; rms(v) = v / sqrt(mean(v^2) + eps).  Keys and values are kept per
head and per token here, in plain lists (the engine pages them, and for the latent attention keeps
the latent only).
"""
from __future__ import annotations

import math

import numpy as np


# ------------------------------------------------------------------------------------- small pieces
def rms(x, eps):
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def offset_norm(x, w, eps):
    """The stream's norms: the weight is stored as its difference from one."""
    return rms(x, eps) * (1.0 + w)


def plain_norm(x, w, eps):
    return rms(x, eps) * w


def softplus(z):
    return math.log1p(math.exp(-abs(z))) + max(z, 0.0)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def xielu(z, p, q):
    """Positive side: a parabola softplus(p) z^2 + z/2.  Negative side: (1/2 + softplus(q)) (e^z - 1 - z) + z/2.
    Both sides and their slopes meet at 0."""
    ap, an = softplus(p), 0.5 + softplus(q)
    zn = np.minimum(z, 0.0)
    return np.where(z > 0.0, ap * z * z + 0.5 * z, an * (np.expm1(zn) - zn) + 0.5 * z)


# ------------------------------------------------------------------------------------- rotations
def plain_frequencies(dims, base):
    return np.array([float(base) ** (-2.0 * i / dims) for i in range(dims // 2)])


def ramp_frequencies(dims, base, sc):
    """Frequencies blended between f and f / factor by a ramp over the pair index, whose two ends are the
    pair indices at which `fast` and `slow` turns fit into `original` positions; the second result is
    the factor on cos and sin."""
    f = plain_frequencies(dims, base)
    factor, orig = float(sc["factor"]), float(sc["original"])

    def pair_index(turns):
        return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(pair_index(float(sc["fast"]))), 0)
    hi = min(math.ceil(pair_index(float(sc["slow"]))), dims - 1)
    i = np.arange(dims // 2, dtype=np.float64)
    ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def turn_pairs(u, v, pos, freqs, mag=1.0):
    a = pos * freqs
    c, s = np.cos(a) * mag, np.sin(a) * mag
    return u * c - v * s, v * c + u * s


def rotate_split(x, pos, freqs, mag=1.0):
    """x [..., d]: the first 2n coordinates (n = len(freqs)) as pairs (i, i + n); the rest passes."""
    n = len(freqs)
    u, v = turn_pairs(x[..., :n], x[..., n:2 * n], pos, freqs, mag)
    return np.concatenate([u, v, x[..., 2 * n:]], axis=-1)


def rotate_neighbours(x, pos, freqs, mag=1.0):
    """x [..., d]: the first 2n coordinates as pairs (2i, 2i + 1); the rest passes."""
    n = len(freqs)
    y = x.copy()
    u, v = turn_pairs(x[..., 0:2 * n:2], x[..., 1:2 * n:2], pos, freqs, mag)
    y[..., 0:2 * n:2], y[..., 1:2 * n:2] = u, v
    return y


# ------------------------------------------------------------------------------------- attention
def softmax_mix(scores, values, sink=None):
    """scores [n], values [n, dv]; with a sink the denominator holds exp(sink) as well."""
    m = float(scores.max()) if sink is None else max(float(scores.max()), float(sink))
    e = np.exp(scores - m)
    den = e.sum() + (0.0 if sink is None else math.exp(sink - m))
    return (e[:, None] * values).sum(0) / den


class TalkingAttention:
    """Projections with biases, one RMS norm over ALL query rows and one over all key rows, split-pair
    rotation of a part of every head with ramp-blended frequencies, the heads' scores mixed by a
    matrix before the softmax, a sliding window, a learned sink per head."""

    def __init__(self, mc: dict, w: dict, p: str, eps: float):
        self.H, self.G, self.dk, self.dv = (int(mc[k]) for k in ("heads", "kv_heads", "dim", "vdim"))
        self.scale, self.eps = float(mc["scale"]), eps
        self.window = int(mc["mask"]["size"])
        rot = mc["rot"]
        if rot.get("scaling"):
            self.freqs, self.mag = ramp_frequencies(int(rot["dims"]), float(rot["base"]), rot["scaling"])
        else:
            self.freqs, self.mag = plain_frequencies(int(rot["dims"]), float(rot["base"])), 1.0
        self.w = {k: w[p + k] for k in ("q", "q.b", "k", "k.b", "v", "v.b", "q.norm", "k.norm", "talk", "sink", "o")}
        self.keys, self.vals = [], []  # per token [G, dk], [G, dv]

    def step(self, h, pos):
        w, H, G = self.w, self.H, self.G
        q = plain_norm(w["q"] @ h + w["q.b"], w["q.norm"], self.eps).reshape(H, self.dk)
        k = plain_norm(w["k"] @ h + w["k.b"], w["k.norm"], self.eps).reshape(G, self.dk)
        v = (w["v"] @ h + w["v.b"]).reshape(G, self.dv)
        q = rotate_split(q, pos, self.freqs, self.mag)
        k = rotate_split(k, pos, self.freqs, self.mag)
        self.keys.append(k)
        self.vals.append(v)
        first = max(0, pos - self.window + 1)
        K, V = np.stack(self.keys[first:]), np.stack(self.vals[first:])  # [n, G, .]
        rep = H // G
        raw = np.stack([(K[:, hd // rep] @ q[hd]) * self.scale for hd in range(H)])  # [H, n]
        mixed = w["talk"] @ raw
        out = np.stack([softmax_mix(mixed[hd], V[:, hd // rep], float(w["sink"][hd])) for hd in range(H)])
        return w["o"] @ out.reshape(-1)


class LatentAttention:
    """Queries through a normed low-rank latent; keys and values expanded from a normed shared latent,
    plus one rotated key part that all heads share (neighbouring pairs).  Per head the query and key are
    [dim unrotated | rot_dim rotated].  Sliding window, plain softmax."""

    def __init__(self, mc: dict, w: dict, p: str, eps: float):
        self.H, self.dn, self.dr, self.dv, self.rank = (int(mc[k]) for k in ("heads", "dim", "rot_dim", "vdim", "kv_rank"))
        self.scale, self.eps = float(mc["scale"]), eps
        self.window = int(mc["mask"]["size"])
        if int(mc["rot"]["dims"]) != self.dr:
            raise ValueError("the rotated part is rot_dim wide")
        self.freqs = plain_frequencies(self.dr, float(mc["rot"]["base"]))
        self.w = {k: w[p + k] for k in ("dq", "dq.norm", "uq", "dkv", "dkv.norm", "uk", "uv", "o")}
        self.keys, self.vals = [], []  # per token: [H, dn + dr], [H, dv]

    def step(self, h, pos):
        w, H = self.w, self.H
        cq = plain_norm(w["dq"] @ h, w["dq.norm"], self.eps)
        q = (w["uq"] @ cq).reshape(H, self.dn + self.dr)
        q = np.concatenate([q[:, :self.dn], rotate_neighbours(q[:, self.dn:], pos, self.freqs)], axis=-1)
        d = w["dkv"] @ h
        c = plain_norm(d[:self.rank], w["dkv.norm"], self.eps)
        kr = rotate_neighbours(d[self.rank:], pos, self.freqs)
        kn = (w["uk"] @ c).reshape(H, self.dn)
        self.keys.append(np.concatenate([kn, np.broadcast_to(kr, (H, self.dr))], axis=-1))
        self.vals.append((w["uv"] @ c).reshape(H, self.dv))
        first = max(0, pos - self.window + 1)
        K, V = np.stack(self.keys[first:]), np.stack(self.vals[first:])
        out = np.stack([softmax_mix((K[:, hd] @ q[hd]) * self.scale, V[:, hd]) for hd in range(H)])
        return w["o"] @ out.reshape(-1)


# ------------------------------------------------------------------------------------- feed-forward
def dense_ff(h, w, p):
    a = w[p + "act"]
    return w[p + "down"] @ xielu(w[p + "up"] @ h, float(a[0]), float(a[1]))


def gated_expert(h, w, p):
    return w[p + "down"] @ (silu(w[p + "gate"] @ h) * (w[p + "up"] @ h))


def routed_ff(h, w, p, mlp):
    """Softmax over all experts; the `top` largest weigh their experts' OUTPUTS as they are (their sum is
    below one).  Also returns the scores."""
    top = int(mlp["router"]["top"])
    z = w[p + "router"] @ h
    s = np.exp(z - z.max())
    s = s / s.sum()
    y = np.zeros_like(h)
    for e in np.argsort(-s, kind="stable")[:top]:
        y = y + s[e] * gated_expert(h, w, f"{p}e{int(e)}.")
    return y, s


# ------------------------------------------------------------------------------------- the model
class Oracle:
    def __init__(self, cfg: dict, w: dict):
        self.cfg, self.w = cfg, w
        self.eps = float(cfg["norm"]["eps"])
        self.mixers = []
        for i, l in enumerate(cfg["layers"]):
            kind = {"attention": TalkingAttention, "latent_attention": LatentAttention}[l["type"]]
            self.mixers.append(kind(l["mixer"], w, f"l{i}.mix.", self.eps))
        self.pos = 0
        # per token: the smallest gap, over its routed layers, between the last chosen score and the best one left out
        self.margins = []

    def step(self, token: int):
        w, eps = self.w, self.eps
        x = offset_norm(w["embed"][token], w["embed.norm"], eps)
        results = [x]  # what the embedding and every layer produced, before any averaging
        streams, margin = [], math.inf
        for i, l in enumerate(self.cfg["layers"]):
            p = f"l{i}."
            x = x + offset_norm(self.mixers[i].step(x, self.pos), w[p + "norm1"], eps)
            mlp = l.get("mlp")
            if mlp:
                if mlp.get("kind", "dense") == "dense":
                    y = dense_ff(x, w, p + "mlp.")
                else:
                    y, sc = routed_ff(x, w, p + "mlp.", mlp)
                    top = int(mlp["router"]["top"])
                    if top < len(sc):
                        srt = np.sort(sc)[::-1]
                        margin = min(margin, float(srt[top - 1] - srt[top]))
                x = x + offset_norm(y, w[p + "norm2"], eps)
            results.append(x)
            x = sum(float(a) * r for a, r in zip(w[p + "dwa"], results))
            streams.append(x.copy())
        self.pos += 1
        self.margins.append(margin)
        logits = w["head"] @ offset_norm(x, w["final.norm"], eps)
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
