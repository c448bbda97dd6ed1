"""Seradra through the engine (paged keys / values / latents, forced and scheduled steps) against the
plain float64 oracle of tests/seradra_oracle.py: on the PyTorch forms of the ops here, on the HIP
kernels under `-m gpu`.  Every test makes its own small configuration and random weights."""
import math
import types

import numpy as np
import pytest
import torch

from tests import seradra_oracle as so
from tests.seradra_utils import (BASE, RAMP, config, cut, dense, engine, latent, layer, moe, rel_err, replay, talking,
                                 write_checkpoint)

DEVS = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
DEV_DTYPE = [("cpu", torch.float32), pytest.param("cuda", torch.float32, marks=pytest.mark.gpu),
             pytest.param("cuda", torch.bfloat16, marks=pytest.mark.gpu)]
DEV_DTYPE_TOL = [("cpu", "float32", 1e-4), pytest.param("cuda", "float32", 1e-4, marks=pytest.mark.gpu),
                 pytest.param("cuda", "bfloat16", 0.1, marks=pytest.mark.gpu)]
EPS = 1e-5
CLOSE = 0.02  # a routing margin below this may fall either way in bf16


def _skip(dev):
    if dev == "cuda" and not torch.cuda.is_available():
        pytest.skip("no GPU")


def _tokens(n, vocab, seed):
    return np.random.default_rng(seed).integers(0, vocab, n).tolist()


def _row_errors(got, want):
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    return np.sqrt((d ** 2).mean(-1)) / np.sqrt((want ** 2).mean())


def _check(got, want, tol, margins=None):
    """fp32 (tol well below 1e-2): every row within tol.  bf16: the mean over the rows (of eight or
    more) within tol / 4 and the worst row within 2.5 tol -- up to the sequence's first token whose
    routing was a close call in the oracle: rounding may send that token to another expert, and later
    tokens attend to what it left in the pages while it is inside their window.  From there on the rows
    must stay near (median within tol, none beyond 1): a mechanism that fails does not."""
    if tol < 1e-2:
        e = rel_err(got, want)
        assert e < tol, f"relative error {e:.3g} >= {tol}"
        return
    e = _row_errors(got, want)
    assert np.isfinite(e).all()
    if margins is not None and (np.asarray(margins) < CLOSE).any():
        first = int(np.argmax(np.asarray(margins) < CLOSE))
        after = e[first:]
        assert np.median(after) < tol and after.max() < 1.0, f"rows after a close call: median {np.median(after):.3g}, worst {after.max():.3g}"
        e = e[:first]
    assert (len(e) < 8 or e.mean() < tol / 4) and (len(e) == 0 or e.max() < 2.5 * tol), \
        f"row errors: mean {e.mean():.3g}, worst {e.max():.3g} (tol {tol})"


def _oracle_model(cfg, w, tokens):
    m = []
    lg, _ = so.run(cfg, w, tokens, m)
    return lg, m


# ----------------------------------------------------------------------------- the mixers alone
def _mixer_setup(kind, mc, width, seed=0):
    from mxserve.models.seradra import build_mixer
    m = build_mixer(kind, "m.", width, mc)
    g = torch.Generator().manual_seed(seed)
    shapes = {name: (rows, width) for name, rows in m.proj_rows()}
    shapes.update(m.extra_shapes())
    w = {k: torch.randn(s, generator=g) * (s[-1] ** -0.5 if len(s) > 1 else 1.0) for k, s in shapes.items()}
    for k in w:
        if k.endswith(".norm"):
            w[k] = 1.0 + 0.2 * w[k]
        elif k.endswith(".b"):
            w[k] = 0.3 * w[k]
        elif k.endswith("talk"):
            H = w[k].shape[0]
            w[k] = torch.eye(H) + 0.5 * w[k]
    return m, w


class _Pages:
    """One sequence's pages, scattered over a pool that holds stale numbers (also NaN behind the end)."""

    def __init__(self, T, elems, dev, dtype, bs=16):
        nb = -(-T // bs) + 3
        self.bs, self.dev = bs, dev
        self.cache = torch.randn(nb, elems + 16, device=dev).to(dtype)
        self.cache[:, ::7] = float("nan")
        self.blocks = torch.randperm(nb, generator=torch.Generator().manual_seed(3))[:-(-T // bs)].to(torch.int32)

    def ctx(self, at, n):
        from mxserve.models.mixers import StepContext
        dev, bs = self.dev, self.bs
        pos = torch.arange(at, at + n)
        md = types.SimpleNamespace(
            positions=pos.to(dev), slot_mapping=(self.blocks[pos // bs].long() * bs + pos % bs).to(dev),
            block_tables=self.blocks[None].to(dev), query_start_loc=torch.tensor([0, n], dtype=torch.int32, device=dev),
            seq_lens=torch.tensor([at + n], dtype=torch.int32, device=dev), max_query_len=n, max_seq_len=at + n,
            state_rows=None)
        return StepContext(md=md, cache=self.cache, state=None, block_size=bs, eps=EPS)


def _run_mixer(m, w, h, dev, portions, dtype=torch.float32, koff=8):
    """The mixer over one sequence cut into portions, through pages that start at an offset inside the block."""
    T = h.shape[0]
    wt = {k: v.to(dev).to(dtype) for k, v in w.items()}
    w_in = torch.cat([wt[name] for name, _ in m.proj_rows()])
    m.finish_weights(wt)
    elems = 16 * m.kv_heads * (m.dk + m.dv)
    voff = koff + 16 * m.kv_heads * m.dk
    pg = _Pages(T, koff + elems, dev, dtype)
    outs, at, i = [], 0, 0
    while at < T:
        n = min(portions[min(i, len(portions) - 1)], T - at)
        i += 1
        hp = h[at:at + n].to(dev).to(dtype)
        y = hp @ w_in.T
        parts, c = [], 0
        for _, rows in m.proj_rows():
            parts.append(y[:, c:c + rows])
            c += rows
        outs.append(m.forward(parts, hp, wt, pg.ctx(at, n), koff, voff, 0))
        at += n
    return torch.cat(outs).double().cpu().numpy()


def _oracle_mixer(kind, mc, w, h):
    wn = {k: v.double().numpy() for k, v in w.items()}
    cls = {"attention": so.TalkingAttention, "latent_attention": so.LatentAttention}[kind]
    o = cls(mc, wn, "m.", EPS)
    hn = h.double().numpy()
    return np.stack([o.step(hn[t], t) for t in range(h.shape[0])])


def _bf(w, h):
    """Weights and inputs rounded to bf16, so that the oracle and a bf16 run start from the same numbers."""
    return {k: v.to(torch.bfloat16).float() for k, v in w.items()}, h.to(torch.bfloat16).float()


PORTIONS = [[1000], [1], [2], [5, 1, 9, 2, 30]]
TALKING_SHAPES = [
    talking(),
    talking(heads=1, kv_heads=1, dim=2, vdim=3, scale=0.7, window=1, rot_dims=2, base=50.0, scaling=None),
    talking(heads=6, kv_heads=2, dim=20, vdim=12, scale=0.15, window=16, rot_dims=20, base=200000.0,
            scaling={"factor": 8.0, "original": 32, "fast": 4.0, "slow": 0.5}),
    talking(heads=5, kv_heads=5, dim=32, vdim=16, scale=0.12, window=1000, rot_dims=6, scaling=None),
    talking(heads=20, kv_heads=4, dim=16, vdim=16, scale=0.2, window=35, rot_dims=8),
    talking(heads=8, kv_heads=8, dim=80, vdim=96, scale=0.1, window=17, rot_dims=32),
    talking(heads=18, kv_heads=6, dim=96, vdim=80, scale=0.1, window=30, rot_dims=64),
    talking(heads=40, kv_heads=10, dim=16, vdim=32, scale=0.25, window=50, rot_dims=4, scaling=None),
    talking(heads=34, kv_heads=2, dim=16, vdim=16, scale=0.25, window=28, rot_dims=16, scaling=None),
    talking(heads=2, kv_heads=1, dim=144, vdim=136, scale=0.08, window=45, rot_dims=100),
]


@pytest.mark.parametrize("dev,dtype", DEV_DTYPE)
@pytest.mark.parametrize("portions", PORTIONS)
def test_talking_attention_mixer(dev, dtype, portions):
    """Several shapes: grouped key/value heads, one head of one rotary pair that sees itself only, a
    rotation over the whole head, a window longer than the sequence, more heads than a workgroup has
    waves (two and four heads a wave), heads wider than 64, more query heads per kv head than a tile has columns, heads wider than the
    matrix-core forms take."""
    _skip(dev)
    width, T = 72, 70
    h = torch.randn(T, width, generator=torch.Generator().manual_seed(1))
    for n, mc in enumerate(TALKING_SHAPES):
        m, w = _mixer_setup("attention", mc, width, seed=n)
        w["m.sink"] = w["m.sink"] * 2.0
        if dtype == torch.bfloat16:
            w, hh = _bf(w, h)
            got, want = _run_mixer(m, w, hh, dev, portions, dtype), _oracle_mixer("attention", mc, w, hh)
            assert _row_errors(got, want).max() < 0.05, (mc, _row_errors(got, want).max())
        else:
            _check(_run_mixer(m, w, h, dev, portions), _oracle_mixer("attention", mc, w, h), 1e-4)


LATENT_SHAPES = [
    latent(),
    latent(heads=1, dim=8, rot_dim=2, vdim=8, kv_rank=8, q_rank=8, scale=0.5, window=1, base=50.0),
    latent(heads=6, dim=16, rot_dim=32, vdim=24, kv_rank=136, q_rank=16, scale=0.1, window=16, base=200000.0),
    latent(heads=2, dim=72, rot_dim=8, vdim=8, kv_rank=24, q_rank=100, scale=0.12, window=500),
    latent(heads=4, dim=32, rot_dim=16, vdim=32, kv_rank=64, q_rank=48, scale=0.15, window=37),
    latent(heads=3, dim=10, rot_dim=6, vdim=7, kv_rank=13, q_rank=9, scale=0.3, window=20),
]


@pytest.mark.parametrize("dev,dtype", DEV_DTYPE)
@pytest.mark.parametrize("portions", PORTIONS)
def test_latent_attention_mixer(dev, dtype, portions):
    """Plain, rotated and value sizes all different; one head that sees itself only; a latent wider than
    the heads it feeds; a window longer than the sequence; sizes the matrix-core kernel takes in bf16 and
    sizes that fit no vector load."""
    _skip(dev)
    width, T = 80, 70
    h = torch.randn(T, width, generator=torch.Generator().manual_seed(1))
    for n, mc in enumerate(LATENT_SHAPES):
        m, w = _mixer_setup("latent_attention", mc, width, seed=n)
        if dtype == torch.bfloat16:
            w, hh = _bf(w, h)
            got, want = _run_mixer(m, w, hh, dev, portions, dtype), _oracle_mixer("latent_attention", mc, w, hh)
            assert _row_errors(got, want).max() < 0.05, (mc, _row_errors(got, want).max())
        else:
            _check(_run_mixer(m, w, h, dev, portions), _oracle_mixer("latent_attention", mc, w, h), 1e-4)


def _picking_talking(window, heads=1, scale=4.0, sink=-30.0):
    """Every head's query reads h[0:8], its key h[8:16] and its value h[16:24] (head sizes 10 and 8; the two
    rotated entries are zero); norms with unit weights, no biases, an identity mix."""
    mc = talking(heads=heads, kv_heads=1, dim=10, vdim=8, scale=scale, window=window, rot_dims=2, base=100.0, scaling=None)
    from mxserve.models.seradra import build_mixer
    m = build_mixer("attention", "m.", 24, mc)
    eye, z = torch.eye(8), torch.zeros(8, 8)
    rd = lambda cols: torch.cat([torch.zeros(2, 24), torch.cat(cols, 1)])  # noqa: E731
    w = {"m.q": torch.cat([rd([eye, z, z])] * heads), "m.k": rd([z, eye, z]), "m.v": torch.cat([z, z, eye], 1),
         "m.q.b": torch.zeros(10 * heads), "m.k.b": torch.zeros(10), "m.v.b": torch.zeros(8),
         "m.q.norm": torch.ones(10 * heads), "m.k.norm": torch.ones(10), "m.talk": torch.eye(heads),
         "m.sink": torch.full((heads,), sink), "m.o": torch.cat([torch.cat([eye, torch.zeros(16, 8)])] + [torch.zeros(24, 8)] * (heads - 1), 1)}
    return mc, m, w


def _picking_latent(window, scale=4.0):
    """One head whose query reads h[:8], whose latent reads h[8:16] and whose key and value are the normed
    latent itself; the rotated parts are zero."""
    mc = latent(heads=1, dim=8, rot_dim=2, vdim=8, kv_rank=8, q_rank=8, scale=scale, window=window, base=100.0)
    from mxserve.models.seradra import build_mixer
    m = build_mixer("latent_attention", "m.", 24, mc)
    eye = torch.eye(8)
    w = {"m.dq": torch.cat([eye, torch.zeros(8, 16)], 1), "m.dq.norm": torch.ones(8),
         "m.uq": torch.cat([eye, torch.zeros(2, 8)]),
         "m.dkv": torch.cat([torch.cat([torch.zeros(8, 8), eye, torch.zeros(8, 8)], 1), torch.zeros(2, 24)]),
         "m.dkv.norm": torch.ones(8), "m.uk": eye.clone(), "m.uv": eye.clone(), "m.o": torch.cat([eye, torch.zeros(16, 8)])}
    return mc, m, w


WINDOW = 150


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("kind", ["attention", "latent_attention"])
@pytest.mark.parametrize("back", [0, 1, 12, 13, 28, 29, 60, 140, 141, 148, 149, 150, 151, 156, 157, 300])
def test_one_key_stands_out_inside_the_window_only(dev, kind, back):
    """One key `back` positions before the last query matches it so strongly that, when the window holds
    it, the output is that key's value: the query's own position, both sides of page borders, the
    window's last position and the first one outside (where the output must be what the others give), in
    a whole prompt, when the last token is decoded alone, and in uneven portions."""
    _skip(dev)
    T = 301
    mc, m, w = (_picking_talking if kind == "attention" else _picking_latent)(WINDOW)
    target = T - 1 - back
    g = torch.Generator().manual_seed(5)
    h = 0.1 * torch.randn(T, 24, generator=g)
    h[:, 8] += 8.0           # every key points along its first coordinate ...
    h[target, 8] -= 8.0
    h[target, 13] += 8.0     # ... but the target's, which points along the one the last query asks for
    h[T - 1, :8] = 0.0
    h[T - 1, 5] = 8.0
    h[:, 16:] = torch.randn(T, 8, generator=g)
    if kind == "attention":
        h[target, 16:] = 3.0
        shown = np.full(8, 3.0)
    else:  # the value is the normed latent itself
        lat = h[target, 8:16].double().numpy()
        shown = lat / np.sqrt((lat ** 2).mean() + EPS)
    if back == 0:            # the last token is the target: its own key must match its own query
        h[T - 1, 5] = 8.0
    want = _oracle_mixer(kind, mc, w, h)
    near = np.abs(want[T - 1, :8] - shown).max()
    assert near < 0.05 if back < WINDOW else near > 0.5  # the oracle itself shows the case
    for portions in ([T], [T - 1, 1], [7, 2, 160, 3, 100, 1]):
        got = _run_mixer(m, dict(w), h, dev, portions)
        assert np.abs(got - want).max() < 1e-4


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("level,weight", [(0.0, 0.5), (2.0, 1.0 / (1.0 + np.e ** 2)), (-30.0, 1.0)])
def test_sink_counts_once_and_is_not_scaled(dev, level, weight):
    """Keys whose scores are exactly 0: position t's output is the sum of the values in its window over
    (their number + exp(sink)); the first token alone gives value / (1 + exp(sink))."""
    _skip(dev)
    win = 9
    mc, m, w = _picking_talking(win, scale=7.0, sink=level)
    w["m.q"] = torch.zeros_like(w["m.q"])
    h = torch.randn(40, 24, generator=torch.Generator().manual_seed(2))
    v = h[:, 16:].double().numpy()
    want = np.stack([v[max(0, t - win + 1):t + 1].sum(0) / (min(t + 1, win) + np.exp(level)) for t in range(40)])
    assert abs(want[0, 0] - weight * v[0, 0]) < 1e-9
    got = _run_mixer(m, w, h, dev, [1, 32, 1])
    assert np.abs(got[:, :8] - want).max() < 1e-5 and np.abs(got[:, 8:]).max() == 0.0


@pytest.mark.parametrize("dev", DEVS)
def test_heads_talk_before_the_softmax(dev):
    """Two heads over the same keys: head 0 asks for one key, head 1 for another.  With the mixing matrix
    [[0, 1], [1, 0]] each head attends where the OTHER one asked; with [[1, 1], [0, 1]] head 0 splits
    between both keys.  The identity gives neither."""
    _skip(dev)
    T = 40
    mc, m, w = _picking_talking(1000, heads=2, scale=4.0)
    w["m.q"] = torch.zeros(20, 24)
    w["m.q"][2 + 5, 5] = 1.0       # head 0's query reads h[5] into its entry 5, head 1's reads h[6] into entry 6
    w["m.q"][10 + 2 + 6, 6] = 1.0
    w["m.o"] = torch.cat([torch.cat([torch.eye(8), torch.zeros(8, 8)], 1), torch.cat([torch.zeros(8, 8), torch.eye(8)], 1),
                          torch.zeros(8, 16)])
    h = torch.zeros(T, 24)
    h[:, 8] = 8.0
    h[:, 16:] = torch.randn(T, 8, generator=torch.Generator().manual_seed(4))
    h[10, 8], h[10, 13] = 0.0, 8.0  # key 10 answers entry 5
    h[20, 8], h[20, 14] = 0.0, 8.0  # key 20 answers entry 6
    h[T - 1, 5] = h[T - 1, 6] = 1.0
    v = h[:, 16:].double().numpy()
    outs = {}
    for name, talk in (("swap", [[0.0, 1.0], [1.0, 0.0]]), ("both", [[1.0, 1.0], [0.0, 1.0]]), ("plain", [[1.0, 0.0], [0.0, 1.0]])):
        w["m.talk"] = torch.tensor(talk)
        want = _oracle_mixer("attention", mc, w, h)
        got = _run_mixer(m, dict(w), h, dev, [T - 1, 1])
        assert np.abs(got - want).max() < 1e-4
        outs[name] = want[T - 1]
    assert np.abs(outs["plain"][:8] - v[10]).max() < 0.05 and np.abs(outs["plain"][8:16] - v[20]).max() < 0.05
    assert np.abs(outs["swap"][:8] - v[20]).max() < 0.05 and np.abs(outs["swap"][8:16] - v[10]).max() < 0.05
    assert np.abs(outs["both"][:8] - 0.5 * (v[10] + v[20])).max() < 0.05 and np.abs(outs["both"][8:16] - v[20]).max() < 0.05


def test_ramp_frequencies_by_hand():
    """dims 8, base 100, original 40, fast 4, slow 0.5, factor 5: the pair indices where 4 and 0.5 turns
    fit into 40 positions are 8 ln(40 / (2 pi t)) / (2 ln 100) = 0.404 and 2.210, so lo = 0, hi = 3 and the
    ramp is i / 3; cos and sin carry 0.1 ln 5 + 1."""
    from mxserve.models.mixers import rotary_frequencies, rotary_magnitude
    sc = {"factor": 5.0, "original": 40, "fast": 4.0, "slow": 0.5}
    f = [100.0 ** (-2.0 * i / 8) for i in range(4)]
    want = [f[i] * (1 - i / 3) + f[i] / 5.0 * (i / 3) for i in range(4)]
    got = rotary_frequencies(8, 100.0, sc).double().numpy()
    assert np.abs(got - np.array(want)).max() < 1e-7
    assert abs(rotary_magnitude(sc) - (0.1 * math.log(5.0) + 1.0)) < 1e-12 and rotary_magnitude(None) == 1.0
    assert np.abs(so.ramp_frequencies(8, 100.0, sc)[0] - np.array(want)).max() < 1e-12
    # a ramp that is cut at both ends: lo from a negative index, hi beyond the last dimension
    sc2 = {"factor": 2.0, "original": 8, "fast": 64.0, "slow": 0.001}
    assert np.abs(rotary_frequencies(4, 10.0, sc2).double().numpy() - so.ramp_frequencies(4, 10.0, sc2)[0]).max() < 1e-7


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("kind", ["attention", "latent_attention"])
def test_rotation_pairs_and_shows_the_distance(dev, kind):
    """Four rotated entries.  The attention pairs entry 1 with entry 3 (halves), the latent attention
    entry 2 with entry 3 (neighbours); both at the second frequency.  One key at position 4 and the last
    query carry a single non-zero rotated entry: the score is a cosine of the distance times the
    frequency, and the output follows in closed form."""
    _skip(dev)
    T, scale, base = 41, 2.0, 100.0
    f1 = base ** (-2.0 / 4)
    g = torch.Generator().manual_seed(3)
    if kind == "attention":
        mc = talking(heads=1, kv_heads=1, dim=4, vdim=8, scale=scale, window=1000, rot_dims=4, base=base, scaling=None)
        from mxserve.models.seradra import build_mixer
        m = build_mixer("attention", "m.", 24, mc)
        w = {"m.q": torch.zeros(4, 24), "m.k": torch.zeros(4, 24), "m.v": torch.cat([torch.zeros(8, 16), torch.eye(8)], 1),
             "m.q.b": torch.zeros(4), "m.k.b": torch.zeros(4), "m.v.b": torch.zeros(8), "m.q.norm": torch.ones(4),
             "m.k.norm": torch.ones(4), "m.talk": torch.ones(1, 1), "m.sink": torch.tensor([0.3]),
             "m.o": torch.cat([torch.eye(8), torch.zeros(16, 8)])}
        w["m.q"][1, 0] = 1.0   # rotated entry 1 of the query reads h[0], of the key h[1]
        w["m.k"][1, 1] = 1.0
        h = torch.zeros(T, 24)
        h[:, 16:] = torch.randn(T, 8, generator=g)
        h[4, 1] = 1.5
        h[T - 1, 0] = 1.0
        vals = h[:, 16:].double().numpy()
        unit = math.sqrt(4.0 / (1.0 + 4 * EPS / 1.0))      # a lone entry 1 after the norm over four entries
        unit_k = math.sqrt(4.0 / (1.0 + 4 * EPS / 1.5 ** 2))
        sc = np.zeros(T)
        sc[4] = scale * unit * unit_k * math.cos((T - 1 - 4) * f1)
        sink = math.exp(0.3)
    else:
        mc, m, w = _picking_latent(1000, scale=scale)
        mc["rot_dim"] = mc["rot"]["dims"] = 4
        from mxserve.models.seradra import build_mixer
        m = build_mixer("latent_attention", "m.", 24, mc)
        w["m.uq"] = torch.zeros(8 + 4, 8)
        w["m.dkv"] = torch.cat([w["m.dkv"][:8], torch.zeros(4, 24)])
        w["m.uq"][8 + 2, 0] = 1.0    # rotated entry 2 of the query reads the query latent's entry 0
        w["m.dkv"][8 + 2, 1] = 1.0   # rotated entry 2 of the key reads h[1]
        h = torch.zeros(T, 24)
        h[:, 8:16] = torch.randn(T, 8, generator=g)
        h[4, 1] = 1.5
        h[T - 1, 0] = 1.0
        lat = h[:, 8:16].double().numpy()
        vals = lat / np.sqrt((lat ** 2).mean(-1, keepdims=True) + EPS)
        qb = math.sqrt(8.0 / (1.0 + 8 * EPS))  # the query latent (1, 0, ...) after its norm
        sc = np.zeros(T)
        sc[4] = scale * qb * 1.5 * math.cos((T - 1 - 4) * f1)
        sink = 0.0
    want = _oracle_mixer(kind, mc, w, h)
    e = np.exp(sc)
    closed = (e[:, None] * vals).sum(0) / (e.sum() + sink)
    assert np.abs(want[T - 1, :8] - closed).max() < 1e-6
    for portions in ([T], [T - 1, 1], [3, 2]):
        assert np.abs(_run_mixer(m, dict(w), h, dev, portions) - want).max() < 1e-4


# ----------------------------------------------------------------------------- feed-forwards and the stream alone
def _ff_setup(mlp, width, seed=0, router_gain=3.0):
    from mxserve.models.seradra import build_ff
    f = build_ff("f.", width, mlp)
    g = torch.Generator().manual_seed(seed)
    w = {k: torch.randn(s, generator=g) * (s[-1] ** -0.5 if len(s) > 1 else 1.0) for k, s in f.shapes().items()}
    if "f.router" in w:
        w["f.router"] = w["f.router"] * router_gain
    return f, w


@pytest.mark.parametrize("dev", DEVS)
def test_two_sided_activation(dev):
    """Values on both sides of zero, at zero, and far out; learned numbers of both signs."""
    _skip(dev)
    from mxserve.ops import seqmix
    z = torch.cat([torch.linspace(-30, 30, 241), torch.tensor([0.0, -0.0, 1e-6, -1e-6])])
    for p, q in ((0.0, 0.0), (-2.5, 1.5), (3.0, -4.0)):
        ab = torch.tensor([so.softplus(p), 0.5 + so.softplus(q)], dtype=torch.float32)
        got = seqmix.xielu(z.to(dev), ab.to(dev)).double().cpu().numpy()
        want = so.xielu(z.double().numpy(), p, q)
        assert np.abs(got - want).max() < 1e-5 * max(1.0, np.abs(want).max())
    f, w = _ff_setup(dense(40), 24, seed=3)
    h = 2.0 * torch.randn(9, 24, generator=torch.Generator().manual_seed(1))
    wn = {k: v.double().numpy() for k, v in w.items()}
    want = np.stack([so.dense_ff(x, wn, "f.") for x in h.double().numpy()])
    wt = {k: v.to(dev) for k, v in w.items()}
    f.finish_weights(wt)
    assert np.abs(f.forward(h.to(dev), wt).double().cpu().numpy() - want).max() < 1e-4 * max(1.0, np.abs(want).max())


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("T", [1, 5, 33, 150])
def test_routed_experts_alone(dev, T):
    """Both ways through the experts (batched over all experts for a few tokens, sorted rows otherwise);
    top of one, of several and of all; many experts."""
    _skip(dev)
    width = 48
    h = 1.5 * torch.randn(T, width, generator=torch.Generator().manual_seed(T))
    for mlp in (moe(experts=6, top=2, ff=40), moe(experts=5, top=1, ff=24), moe(experts=3, top=3, ff=72),
                moe(experts=70, top=4, ff=16)):
        f, w = _ff_setup(mlp, width)
        wn = {k: v.double().numpy() for k, v in w.items()}
        want = np.stack([so.routed_ff(x, wn, "f.", mlp)[0] for x in h.double().numpy()])
        wt = {k: v.to(dev) for k, v in w.items()}
        f.finish_weights(wt)
        got = f.forward(h.to(dev), wt).double().cpu().numpy()
        assert np.abs(got - want).max() < 2e-4 * max(1.0, np.abs(want).max())


def test_scores_weigh_the_outputs_and_are_not_renormalised():
    """Softmax over ALL experts before the choice: the chosen weights sum to less than one.  The
    alternatives (weights renormalised over the chosen, softmax over the chosen logits only, sigmoid
    scores) differ visibly."""
    width = 32
    mlp = moe(experts=4, top=2, ff=24)
    f, w = _ff_setup(mlp, width, seed=4, router_gain=0.3)
    h = 2.0 * torch.randn(6, width, generator=torch.Generator().manual_seed(9))
    wn = {k: v.double().numpy() for k, v in w.items()}
    hn = h.double().numpy()
    want = np.stack([so.routed_ff(x, wn, "f.", mlp)[0] for x in hn])
    renorm, sig = [], []
    for x in hn:
        z = wn["f.router"] @ x
        s = np.exp(z) / np.exp(z).sum()
        top = np.argsort(-s)[:2]
        assert s[top].sum() < 0.9
        renorm.append(sum(s[e] / s[top].sum() * so.gated_expert(x, wn, f"f.e{e}.") for e in top))
        sig.append(sum(so.sigmoid(z[e]) * so.gated_expert(x, wn, f"f.e{e}.") for e in top))
    assert np.abs(np.stack(renorm) - want).max() > 0.02 and np.abs(np.stack(sig) - want).max() > 0.02
    f.finish_weights(w)
    assert np.abs(f.forward(h, w).double().numpy() - want).max() < 1e-4


@pytest.mark.parametrize("dev", DEVS)
def test_softmax_top_k_order_ties_and_weighted_sum(dev):
    _skip(dev)
    from mxserve.ops import seqmix
    z = torch.tensor([[0.0, 2.0, 2.0, -1.0, 2.0], [5.0, -5.0, 0.0, 0.0, 1.0]], device=dev)
    w, ids = seqmix.route_topk(z, 3, softmax=True)
    assert ids.cpu().tolist() == [[1, 2, 4], [0, 4, 2]]  # ties go to the lower index
    s = torch.softmax(z.double().cpu(), -1)
    assert torch.allclose(w.double().cpu(), torch.gather(s, 1, ids.cpu().long()), atol=1e-6)
    g = torch.Generator().manual_seed(0)
    T, k, W = 7, 3, 40
    ys = torch.randn(T * k, W, generator=g).to(dev)
    idx = torch.randperm(T * k, generator=g).to(torch.int32).to(dev)
    wts = torch.rand(T, k, generator=g).to(dev)
    got = seqmix.expert_combine(ys, idx, k, T, weights=wts).cpu()
    want = (ys.cpu()[idx.cpu().long()].view(T, k, W) * wts.cpu().view(T, k, 1)).sum(1)
    assert torch.allclose(got, want, atol=1e-5)
    hh = torch.randn(T, W, generator=g).to(dev)
    ids2 = torch.stack([torch.randperm(5, generator=g)[:k] for _ in range(T)]).to(torch.int32).to(dev)
    sp = seqmix.spread_scaled(hh, None, ids2, 5).cpu()
    chosen = torch.zeros(T, 5).scatter_(1, ids2.cpu().long(), 1.0)
    assert torch.equal(sp, chosen.t().unsqueeze(2) * hh.cpu().unsqueeze(0))
    offs, inv = seqmix.expert_align(ids2, 5)
    xs = seqmix.gather_scaled(hh, None, inv, k).cpu()
    assert torch.equal(xs[inv.cpu().long()], hh.cpu().repeat_interleave(k, 0))


@pytest.mark.parametrize("dev", DEVS)
def test_stream_of_kept_results(dev):
    """The normed embedding, a sublayer's normed output added with a weight stored around zero and handed on
    un-normed, and the weighted sum over everything kept so far -- widths with and without whole vector loads."""
    _skip(dev)
    from mxserve.ops import seqmix
    g = torch.Generator().manual_seed(2)
    for W in (24, 37):
        table = torch.randn(11, W, generator=g)
        wn = 0.2 * torch.randn(W, generator=g)
        ids = torch.tensor([3, 0, 10, 3, 7])
        hist = torch.full((4, 5, W), float("nan"))
        hs = hist.to(dev)
        h0 = seqmix.embed_normed(ids.to(dev), table.to(dev), wn.to(dev), 1e-3, 1.0, hs[0], cast_dtype=torch.float32, copy=hs[1])
        e = table[ids].double()
        x0 = e / torch.sqrt((e ** 2).mean(-1, keepdim=True) + 1e-3) * (1.0 + wn.double())
        assert torch.allclose(hs[0].cpu().double(), x0, atol=1e-5) and torch.allclose(h0.cpu().double(), x0, atol=1e-5)
        assert torch.equal(hs[1], hs[0])
        a = 3.0 * torch.randn(5, W, generator=g)
        hn = seqmix.resid_update(hs[1], a.to(dev), 1e-3, wa=wn.to(dev), wa_offset=1.0, cast_dtype=torch.float32)
        x1 = x0 + a.double() / torch.sqrt((a.double() ** 2).mean(-1, keepdim=True) + 1e-3) * (1.0 + wn.double())
        assert torch.allclose(hs[1].cpu().double(), x1, atol=1e-5) and torch.allclose(hn.cpu().double(), x1, atol=1e-5)
        assert seqmix.resid_update(hs[1], None, 1e-3) is None
        c = torch.tensor([0.3, -1.2])
        h2 = seqmix.depth_mix(hs, 2, c.to(dev), cast_dtype=torch.float32)
        x2 = 0.3 * x0 - 1.2 * x1
        assert torch.allclose(hs[2].cpu().double(), x2, atol=1e-5) and torch.allclose(h2.cpu().double(), x2, atol=1e-5)
        assert seqmix.depth_mix(hs, 3, torch.tensor([1.0, 0.0, 2.0]).to(dev)) is None
        assert torch.allclose(hs[3].cpu().double(), x0 + 2.0 * x2, atol=1e-5)
        assert torch.allclose(hs[0].cpu().double(), x0, atol=1e-5)  # older slabs stay what they were


# ----------------------------------------------------------------------------- whole models, schedules
@pytest.fixture(scope="module")
def base(tmp_path_factory):
    path = tmp_path_factory.mktemp("seradra_base")
    w = write_checkpoint(path, BASE, seed=11)
    toks = {f"r{i}": _tokens(n, BASE["vocab"], 20 + i) for i, n in enumerate([90, 37, 1, 64, 130, 16])}
    want = {rid: _oracle_model(BASE, w, t) for rid, t in toks.items()}
    return path, w, toks, want


@pytest.mark.parametrize("dev,dtype,tol", DEV_DTYPE_TOL)
def test_portions_and_decoding(base, dev, dtype, tol):
    """Whole prompt, token by token, and portions of several sizes down to two tokens; every window of the
    model is shorter than the prompt, so keys leave the windows inside portions and while decoding."""
    _skip(dev)
    path, _, toks, want = base
    eng = engine(path, dev, dtype, max_tokens=256)
    for sizes in ([1000], [1], [2], [40, 1], [3, 16, 2, 17, 1, 32, 5]):
        steps = [[("a", p, False)] for p in cut(toks["r0"], sizes)]
        steps[-1] = [("a", steps[-1][0][1], True)]
        _check(replay(eng, steps)["a"], *want["r0"][:1], tol, want["r0"][1])
    assert eng.kv.num_free() == eng.kv.num_blocks


@pytest.mark.parametrize("dev,dtype,tol", DEV_DTYPE_TOL)
def test_long_decoding(base, dev, dtype, tol):
    """A short prompt, then well over a hundred tokens one by one (through the decode graphs on the
    GPU): pages fill, new ones start, and every window passes over decoded tokens."""
    _skip(dev)
    path, _, toks, want = base
    eng = engine(path, dev, dtype, max_tokens=192, eager=(dev == "cpu"))
    steps = [[("a", p, False)] for p in cut(toks["r4"], [10, 1])]
    steps[-1] = [("a", steps[-1][0][1], True)]
    _check(replay(eng, steps)["a"], want["r4"][0], tol, want["r4"][1])
    assert eng.kv.num_free() == eng.kv.num_blocks


@pytest.mark.parametrize("dev,dtype,tol", DEV_DTYPE_TOL)
@pytest.mark.parametrize("eager", [True, False])
def test_mixed_batches_reuse_pages_and_slots(base, dev, dtype, tol, eager):
    """Six unequal requests through four rows and a pool that cannot hold them all at once: portions of
    some beside single tokens of others; each must equal the request run alone (the oracle)."""
    _skip(dev)
    if dev == "cpu" and not eager:
        pytest.skip("graphs are a GPU path")
    path, _, toks, want = base
    eng = engine(path, dev, dtype, max_tokens=384, eager=eager)
    rng = np.random.default_rng(3)
    at = {r: 0 for r in toks}
    waiting, live, steps = list(toks), [], []
    while waiting or live:
        while waiting and len(live) < 4 and sum(-(-len(toks[r]) // 64) * 64 for r in live + waiting[:1]) <= 384:
            live.append(waiting.pop(0))
        step = []
        for r in list(live):
            if rng.random() < 0.2 and len(live) > 1:
                continue  # left out of this step
            left = len(toks[r]) - at[r]
            n = min(left, int(rng.choice([1, 1, 2, 3, 16, 29])))
            end = n == left
            step.append((r, toks[r][at[r]:at[r] + n], end))
            at[r] += n
            if end:
                live.remove(r)
        if step:
            steps.append(step)
    got = replay(eng, steps)
    for r in toks:
        _check(got[r], want[r][0], tol, want[r][1])
    assert eng.kv.num_free() == eng.kv.num_blocks and not eng.runner._row_of


@pytest.mark.parametrize("dev,dtype,tol", DEV_DTYPE_TOL)
def test_request_that_fills_the_pool(tmp_path, dev, dtype, tol):
    """A request three tokens short of the pool and of the longest sequence the engine admits, with
    head sizes that are multiples of 16 (what the matrix-core kernels take in bf16): its last portions
    end in partial tiles on the last page of the block table."""
    _skip(dev)
    cfg = config([layer(talking(heads=4, kv_heads=2, dim=32, vdim=32, scale=0.15, window=50, rot_dims=16), dense(128)),
                  layer(latent(heads=4, dim=32, rot_dim=16, vdim=32, kv_rank=64, q_rank=48, scale=0.15, window=70), moe(4, 2, 32)),
                  layer(talking(heads=16, kv_heads=4, dim=16, vdim=16, scale=0.2, window=120, rot_dims=16), None)],
                 width=128, vocab=200)
    w = write_checkpoint(tmp_path, cfg, seed=8)
    t = _tokens(125, cfg["vocab"], 9)
    want, margins = _oracle_model(cfg, w, t)
    eng = engine(tmp_path, dev, dtype, max_tokens=128)
    for sizes in ([1000], [90, 35], [100, 19, 1], [64, 40, 21]):
        steps = [[("a", p, False)] for p in cut(t, sizes)]
        steps[-1] = [("a", steps[-1][0][1], True)]
        _check(replay(eng, steps)["a"], want, tol, margins)
    assert eng.kv.num_free() == eng.kv.num_blocks


_T1 = talking(heads=1, kv_heads=1, dim=2, vdim=2, scale=1.0, window=1, rot_dims=2, base=10.0, scaling=None)
_L1 = latent(heads=1, dim=8, rot_dim=2, vdim=2, kv_rank=8, q_rank=8, scale=1.0, window=2, base=10.0)
VARIANTS = {
    "one_head_one_pair_smallest_windows": config([layer(_T1, dense(24)), layer(_L1, moe(experts=2, top=2, ff=8))],
                                                 width=40, vocab=50, eps=1e-3),
    "latent_layers_first_and_no_feed_forward": config([layer(latent(), None), layer(latent(heads=5, dim=8, rot_dim=8, vdim=8,
                                                       kv_rank=8, q_rank=8, window=11), None), layer(talking(), None)],
                                                      width=64, vocab=70),
    "a_single_layer": config([layer(talking(heads=2, kv_heads=1, dim=16, vdim=8, window=13, rot_dims=4), moe(3, 1, 24))],
                             width=32, vocab=33),
    "equal_sizes_everywhere": config([layer(talking(heads=2, kv_heads=2, dim=16, vdim=16, scale=0.25, window=16, rot_dims=16,
                                                    scaling={"factor": 1.0, "original": 16, "fast": 16.0, "slow": 16.0}), dense(16)),
                                      layer(latent(heads=2, dim=16, rot_dim=16, vdim=16, kv_rank=16, q_rank=16, window=16),
                                            moe(experts=16, top=16, ff=16))], width=16, vocab=16),
    "sizes_that_fit_no_vector_load": config([layer(talking(heads=3, kv_heads=1, dim=10, vdim=7, scale=0.3, window=9, rot_dims=6),
                                                   moe(experts=3, top=2, ff=14)),
                                             layer(latent(heads=5, dim=6, rot_dim=2, vdim=9, kv_rank=21, q_rank=11, scale=0.4, window=14),
                                                   dense(22))], width=50, vocab=37),
    "many_heads_wide_heads_long_windows": config([layer(talking(heads=12, kv_heads=3, dim=48, vdim=80, scale=0.07, window=400,
                                                                rot_dims=48), moe(experts=9, top=4, ff=40)),
                                                  layer(latent(heads=12, dim=8, rot_dim=40, vdim=72, kv_rank=264, q_rank=136,
                                                               scale=0.07, window=300), dense(100))], width=72, vocab=60),
}


@pytest.mark.parametrize("dev,dtype,tol", DEV_DTYPE_TOL)
@pytest.mark.parametrize("name", list(VARIANTS))
def test_other_sizes(tmp_path, dev, dtype, tol, name):
    _skip(dev)
    cfg = VARIANTS[name]
    w = write_checkpoint(tmp_path, cfg, seed=5)
    t = _tokens(45, cfg["vocab"], 6)
    want, margins = _oracle_model(cfg, w, t)
    eng = engine(tmp_path, dev, dtype, max_tokens=128)
    for sizes in ([1000], [20, 2, 1, 7, 1]):
        steps = [[("a", p, False)] for p in cut(t, sizes)]
        steps[-1] = [("a", steps[-1][0][1], True)]
        _check(replay(eng, steps)["a"], want, tol, margins)


@pytest.mark.parametrize("dev", DEVS)
def test_layer_tap_matches_oracle_streams(base, dev):
    """What leaves every layer (the weighted sum over the kept results), layer by layer."""
    _skip(dev)
    path, w, toks, _ = base
    eng = engine(path, dev, "float32", max_tokens=128)
    tap = eng.runner.model.layer_tap = []
    replay(eng, [[("a", toks["r1"], True)]])
    ref = so.run(BASE, w, toks["r1"])[1]
    assert len(tap) == len(ref) == len(BASE["layers"])
    for a, b in zip(tap, ref):
        assert np.abs(a.double().cpu().numpy() - b).max() < 1e-3 * max(1.0, np.abs(b).max())


def test_depth_coefficients_matter(tmp_path):
    """Coefficients that take ONLY the embedding output after the first layer, and three quarters of it after
    the second (what the layers themselves produced is dropped): the oracle's streams say so, and the engine
    agrees with it."""
    cfg = config([layer(talking(), dense()), layer(latent(), None), layer(talking(), None)], width=48, vocab=40)

    def tweak(sd):
        sd["l0.dwa"] = torch.tensor([1.0, 0.0], dtype=torch.bfloat16)
        sd["l1.dwa"] = torch.tensor([0.75, 0.0, 0.0], dtype=torch.bfloat16)

    w = write_checkpoint(tmp_path, cfg, seed=2, tweak=tweak)
    t = _tokens(20, 40, 1)
    lg, streams = so.run(cfg, w, t)
    emb = np.stack([so.offset_norm(w["embed"][tok], w["embed.norm"], EPS) for tok in t])
    assert np.abs(streams[0] - emb).max() < 1e-12 and np.abs(streams[1] - 0.75 * emb).max() < 1e-12
    eng = engine(tmp_path, "cpu", "float32", max_tokens=64)
    _check(replay(eng, [[("a", t, True)]])["a"], lg, 1e-4)


def test_pages_and_tensors_of_the_plan():
    """An attention layer pages keys and values per kv head, a latent layer one row of latent plus rotated
    part per token; every layer has pages of its own and i + 2 depth coefficients."""
    from mxserve.models.config import seradra_config
    from mxserve.models.seradra import layer_plan, weight_shapes
    plan = layer_plan(BASE, 16)
    per_token = []
    for l in BASE["layers"]:
        mc = l["mixer"]
        per_token.append(mc["kv_rank"] + mc["rot_dim"] if l["type"] == "latent_attention" else mc["kv_heads"] * (mc["dim"] + mc["vdim"]))
    assert all(r.owns_kv for r in plan.runs) and len({r.koff for r in plan.runs}) == len(plan.runs)
    assert plan.block_elems == 16 * sum(per_token) and plan.state_floats == 0
    sh = weight_shapes(BASE)
    assert [sh[f"l{i}.dwa"] for i in range(5)] == [(2,), (3,), (4,), (5,), (6,)]
    assert sh["l0.mix.q.norm"] == (4 * 24,) and sh["l0.mix.k.norm"] == (2 * 24,) and sh["l0.mix.talk"] == (4, 4)
    assert sh["l0.mlp.act"] == (2,) and "l2.norm2" not in sh and sh["l4.mlp.e4.down"] == (BASE["width"], 32)
    assert "l1.mix.sink" not in sh and sh["l1.mix.dkv"] == (48 + 16, BASE["width"]) and sh["embed.norm"] == (BASE["width"],)
    cfg = seradra_config("m", BASE)
    assert not cfg.has_recurrent_state and cfg.kv_bytes_per_token(2) == 2 * sum(per_token)


@pytest.mark.parametrize("dev,dtype", [("cpu", "float32"), pytest.param("cuda", "float32", marks=pytest.mark.gpu),
                                       pytest.param("cuda", "bfloat16", marks=pytest.mark.gpu)])
@pytest.mark.parametrize("caching", [False, True])
def test_greedy_generation_through_the_scheduler(base, dev, dtype, caching):
    """LLMEngine.generate: the scheduler chunks the prompts (a small token budget), batches the
    requests and decodes; every generated token must be the oracle's choice given the same prefix
    (or within its near-ties).  With prefix caching two prompts share their first pages."""
    _skip(dev)
    from mxserve.config import EngineArgs
    from mxserve.engine.engine import LLMEngine
    from mxserve.engine.request import SamplingParams
    path, w, toks, _ = base
    args = EngineArgs(model=str(path), device=dev, dtype=dtype, num_gpu_blocks=40, cpu_num_blocks=40, max_model_len=256,
                      max_num_seqs=3, max_num_batched_tokens=48, load_format="safetensors", cuda_graph_max_bs=2,
                      enable_prefix_caching=caching)
    eng = LLMEngine(args)
    assert eng.kv.caching == caching  # nothing recurrent: pages can be reused by prefix
    prompts = [toks["r1"], toks["r3"], toks["r2"], toks["r5"], toks["r3"][:40] + toks["r5"]]
    outs = eng.generate(prompts, SamplingParams(max_tokens=12, temperature=0.0, ignore_eos=True))
    margin = 1e-3 if dtype == "float32" else 0.25
    for p, o in zip(prompts, outs):
        assert len(o) == 12
        lg = so.run(BASE, w, p + o[:-1])[0][len(p) - 1:]
        for row, tok in zip(lg, o):
            assert row[tok] >= row.max() - margin * (row.max() - row.min())


def test_registered_small_model_runs():
    """The registry's small Seradra with random weights, by name, as a served model would start."""
    from mxserve.config import EngineArgs
    from mxserve.engine.engine import LLMEngine
    from mxserve.engine.request import SamplingParams
    eng = LLMEngine(EngineArgs(model="tiny-seradra", device="cpu", dtype="float32", num_gpu_blocks=16, cpu_num_blocks=16,
                               max_model_len=128, max_num_seqs=2, max_num_batched_tokens=64))
    outs = eng.generate([[1, 2, 3, 4, 5], [7] * 20], SamplingParams(max_tokens=5, temperature=0.0, ignore_eos=True))
    assert [len(o) for o in outs] == [5, 5]


def test_trace_runner_command_line(base, tmp_path):
    """bin/trace_run as a user starts it: steps on stdin, `done <step>` after each, logits files for the
    steps that want some, pages given back under --max-tokens."""
    import json
    import os
    import subprocess
    import sys
    path, _, toks, want = base
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    t = toks["r1"]
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": t[:20], "want": [0, 19]}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": t[20:22], "want": []}, {"id": "y", "tokens": toks["r2"], "want": [0]}],
              "end": ["y"]},
             {"step": 2, "entries": [{"id": "x", "tokens": t[22:], "want": [len(t) - 23]}], "end": ["x"]}]
    out = tmp_path / "out"
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", str(path), "--dtype", "float32",
                        "--out", str(out), "--max-tokens", "128", "--device", "cpu"],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    V = BASE["vocab"]
    a = np.fromfile(out / "0.f32", dtype="<f4").reshape(-1, V)
    b = np.fromfile(out / "1.f32", dtype="<f4").reshape(-1, V)
    c = np.fromfile(out / "2.f32", dtype="<f4").reshape(-1, V)
    _check(a.astype(np.float64), want["r1"][0][[0, 19]], 1e-4)
    _check(b.astype(np.float64), want["r2"][0][[0]], 1e-4)
    _check(c.astype(np.float64), want["r1"][0][[len(t) - 1]], 1e-4)
