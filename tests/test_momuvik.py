"""Momuvik through the engine (paged latents, layers that share weights, forced and scheduled steps)
against the plain float64 oracle of tests/momuvik_oracle.py: on the PyTorch forms of the ops here, on
the HIP kernels under `-m gpu`.  Every test makes its own small configuration and random weights."""
import types

import numpy as np
import pytest
import torch

from tests import momuvik_oracle as mo
from tests.momuvik_utils import BASE, config, cut, dense, engine, latent, layer, moe, rel_err, replay, write_checkpoint

DEVS = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
DEV_DTYPE_TOL = [("cpu", "float32", 1e-4), pytest.param("cuda", "float32", 1e-4, marks=pytest.mark.gpu),
                 pytest.param("cuda", "bfloat16", 0.1, marks=pytest.mark.gpu)]
EPS = 1e-5
CLOSE = 0.03  # a routing margin below this may fall either way in bf16


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
    routing was a close call in the oracle: rounding may send that token to another expert, and every
    later token attends to what it left in the pages.  From there on the rows must stay near (median
    within tol, none beyond 1): a mechanism that fails does not."""
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
    lg, _ = mo.run(cfg, w, tokens, m)
    return lg, m


# ----------------------------------------------------------------------------- the mixer alone
def _mixer_setup(mc, width, seed=0):
    from mxserve.models.momuvik import build_mixer
    m = build_mixer("latent_attention", "m.", width, mc)
    g = torch.Generator().manual_seed(seed)
    shapes = {name: (rows, width) for name, rows in m.proj_rows()}
    shapes.update(m.extra_shapes())
    w = {k: torch.randn(s, generator=g) * (s[-1] ** -0.5 if len(s) > 1 else 1.0) for k, s in shapes.items()}
    for k in w:
        if k.endswith(".norm"):
            w[k] = 1.0 + 0.2 * w[k]
    return m, w


class _Pages:
    """One sequence's pages, scattered over a pool that holds stale numbers."""

    def __init__(self, T, elems, dev, bs=16):
        nb = -(-T // bs) + 3
        self.bs, self.dev = bs, dev
        self.cache = torch.randn(nb, elems + 16, device=dev)
        self.blocks = torch.randperm(nb, generator=torch.Generator().manual_seed(3))[:-(-T // bs)].to(torch.int32)

    def ctx(self, at, n):
        from mxserve.models.mixers import StepContext
        dev, bs = self.dev, self.bs
        pos = torch.arange(at, at + n)
        md = types.SimpleNamespace(
            positions=pos.to(dev), slot_mapping=(self.blocks[pos // bs].long() * bs + pos % bs).to(dev),
            block_tables=self.blocks[None].to(dev), query_start_loc=torch.tensor([0, n], dtype=torch.int32, device=dev),
            seq_lens=torch.tensor([at + n], dtype=torch.int32, device=dev), max_query_len=n, state_rows=None)
        return StepContext(md=md, cache=self.cache, state=None, block_size=bs, eps=EPS)


def _run_mixer(m, w, h, dev, portions, koff=8):
    """The mixer over one sequence cut into portions, through pages that start at an offset inside the block."""
    T = h.shape[0]
    wt = {k: v.to(dev) for k, v in w.items()}
    w_in = torch.cat([wt[name] for name, _ in m.proj_rows()])
    m.finish_weights(wt)
    pg = _Pages(T, koff + 16 * m.dk, dev)
    outs, at, i = [], 0, 0
    while at < T:
        n = min(portions[min(i, len(portions) - 1)], T - at)
        i += 1
        hp = h[at:at + n].to(dev)
        y = hp @ w_in.T
        parts, c = [], 0
        for _, rows in m.proj_rows():
            parts.append(y[:, c:c + rows])
            c += rows
        outs.append(m.forward(parts, hp, wt, pg.ctx(at, n), koff, koff, 0))
        at += n
    return torch.cat(outs).double().cpu().numpy()


def _oracle_mixer(mc, w, h):
    wn = {k: v.double().numpy() for k, v in w.items()}
    o = mo.LatentAttention(mc, wn, "m.", EPS)
    hn = h.double().numpy()
    return np.stack([o.step(hn[t], t) for t in range(h.shape[0])])


PORTIONS = [[1000], [1], [2], [5, 1, 9, 2, 30]]


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("portions", PORTIONS)
def test_latent_attention_mixer(dev, portions):
    """Several shapes: plain, rotated and value sizes all different; one head; a rotated part of one
    pair; a latent wider than the heads it feeds."""
    _skip(dev)
    width, T = 80, 70
    h = torch.randn(T, width, generator=torch.Generator().manual_seed(1))
    for mc in (latent(), latent(heads=1, dim=8, rot_dim=2, vdim=8, kv_rank=8, q_rank=8, scale=0.5, base=50.0),
               latent(heads=6, dim=16, rot_dim=32, vdim=24, kv_rank=136, q_rank=16, scale=0.1, base=250000.0),
               latent(heads=2, dim=72, rot_dim=8, vdim=8, kv_rank=24, q_rank=100, scale=0.12)):
        m, w = _mixer_setup(mc, width)
        w["m.sink"] = w["m.sink"] * 2.0
        _check(_run_mixer(m, w, h, dev, portions), _oracle_mixer(mc, w, h), 1e-4)


def _picking_head(width=16, rot_dim=2, scale=4.0, sink=-30.0):
    """One head whose query reads h[:8] (coordinates 3 and 5 swapped), whose latent reads h[8:16] and whose
    key and value are the normed latent itself; the rotated parts are zero."""
    mc = latent(heads=1, dim=8, rot_dim=rot_dim, vdim=8, kv_rank=8, q_rank=8, scale=scale, base=100.0)
    from mxserve.models.momuvik import build_mixer
    m = build_mixer("latent_attention", "m.", width, mc)
    eye = torch.eye(8)
    perm = eye.clone()
    perm[[3, 5]] = perm[[5, 3]]
    w = {"m.dq": torch.cat([eye, torch.zeros(8, 8)], 1), "m.dq.norm": torch.ones(8),
         "m.uq": torch.cat([perm, torch.zeros(rot_dim, 8)]),
         "m.dkv": torch.cat([torch.cat([torch.zeros(8, 8), eye], 1), torch.zeros(rot_dim, width)]),
         "m.dkv.norm": torch.ones(8), "m.uk": eye.clone(), "m.uv": eye.clone(), "m.sink": torch.tensor([sink]),
         "m.o": torch.cat([eye, torch.zeros(8, 8)])}
    return mc, m, w


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("target", [0, 1, 15, 16, 17, 31, 32, 47, 48, 200, 255, 256, 299])
def test_one_far_key_stands_out(dev, target):
    """One key among three hundred matches the last query so strongly that the output is that key's
    value: the first token, both sides of page borders and keys far back, in a whole prompt, when the
    last token is decoded alone, and in uneven portions."""
    _skip(dev)
    T = 301
    mc, m, w = _picking_head()
    g = torch.Generator().manual_seed(5)
    h = 0.1 * torch.randn(T, 16, generator=g)
    h[:, 8] += 8.0           # every latent points along its first coordinate ...
    h[target, 8] -= 8.0
    h[target, 13] += 8.0     # ... but the target's, which points along the one the last query asks for
    h[T - 1, :8] = 0.0
    h[T - 1, 3] = 8.0
    want = _oracle_mixer(mc, w, h)
    lat = h[target, 8:].double().numpy()
    lat = lat / np.sqrt((lat ** 2).mean() + EPS)
    assert np.abs(want[T - 1, :8] - lat).max() < 0.05  # the oracle itself shows the case
    for portions in ([T], [T - 1, 1], [7, 2, 160, 3, 100, 1]):
        got = _run_mixer(m, dict(w), h, dev, portions)
        assert np.abs(got - want).max() < 1e-4


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("level,weight", [(0.0, 0.5), (2.0, 1.0 / (1.0 + np.e ** 2)), (-30.0, 1.0)])
def test_sink_takes_its_share(dev, level, weight):
    """A single key whose score is exactly 0: the output is the value times 1 / (1 + exp(sink)).  With
    many keys of score 0 the sink counts once, not once per key, and is not scaled."""
    _skip(dev)
    mc, m, w = _picking_head(scale=7.0, sink=level)
    w["m.uq"] = torch.zeros_like(w["m.uq"])
    h = torch.randn(40, 16, generator=torch.Generator().manual_seed(2))
    lat = h[:, 8:].double().numpy()
    lat = lat / np.sqrt((lat ** 2).mean(-1, keepdims=True) + EPS)
    want = np.cumsum(lat, 0) / (np.arange(1, 41)[:, None] + np.exp(level))
    assert abs(want[0, 0] - weight * lat[0, 0]) < 1e-9
    got = _run_mixer(m, w, h, dev, [1, 32, 1])
    assert np.abs(got[:, :8] - want).max() < 1e-5 and np.abs(got[:, 8:]).max() == 0.0


@pytest.mark.parametrize("dev", DEVS)
def test_rotation_pairs_halves_and_shows_the_distance(dev):
    """A rotated part of four entries: entry 1 pairs with entry 3 and turns at the second frequency.
    One key at position 4 carries (0, b, 0, 0), the last query (0, b, 0, 0): the score is
    scale * b^2 * cos(distance * f_1), and the output follows from it in closed form."""
    _skip(dev)
    T, b, scale, base = 41, 1.5, 2.0, 100.0
    mc, m, w = _picking_head(rot_dim=4, scale=scale, sink=0.3)
    w["m.uq"] = torch.zeros_like(w["m.uq"])
    w["m.uq"][8 + 1, 0] = 1.0        # the query's rotated entry 1 reads the query latent's entry 0
    w["m.dkv"][8 + 1, 0] = 1.0       # the key's rotated entry 1 reads h[0]
    h = torch.zeros(T, 16)
    h[:, 8:] = torch.randn(T, 8, generator=torch.Generator().manual_seed(3))
    h[4, 0] = b
    h[T - 1, 0] = 1.0                # the query latent is (sqrt(8), 0, ...) after its norm
    h[T - 1, 1] = 0.0
    want = _oracle_mixer(mc, w, h)
    lat = h[:, 8:].double().numpy()
    lat = lat / np.sqrt((lat ** 2).mean(-1, keepdims=True) + EPS)
    f1 = base ** (-2.0 / 4)
    qb = np.sqrt(8.0 / (1.0 + 8 * EPS))
    sc = np.zeros(T)
    sc[4] = scale * qb * b * np.cos((T - 1 - 4) * f1)
    sc[T - 1] = scale * qb * 1.0     # the last token's own key carries h[0] = 1 at distance 0
    e = np.exp(sc)
    closed = (e[:, None] * lat).sum(0) / (e.sum() + np.exp(0.3))
    assert np.abs(want[T - 1, :8] - closed).max() < 1e-6
    for portions in ([T], [T - 1, 1], [3, 2]):
        assert np.abs(_run_mixer(m, dict(w), h, dev, portions) - want).max() < 1e-4


# ----------------------------------------------------------------------------- feed-forwards and norms alone
def _ff_setup(mlp, width, seed=0, router_gain=3.0):
    from mxserve.models.momuvik import build_ff
    f = build_ff("f.", width, mlp)
    g = torch.Generator().manual_seed(seed)
    w = {k: torch.randn(s, generator=g) * s[-1] ** -0.5 for k, s in f.shapes().items()}
    if "f.router" in w:
        w["f.router"] = w["f.router"] * router_gain
    return f, w


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("T", [1, 5, 33, 150])
def test_routed_experts_alone(dev, T):
    """Both ways through the experts (batched over all experts for a few tokens, sorted rows otherwise);
    top of one, of several and of all; with and without the shared expert; limits that bite."""
    _skip(dev)
    width = 48
    h = 1.5 * torch.randn(T, width, generator=torch.Generator().manual_seed(T))
    for mlp in (moe(experts=6, top=2, ff=40, limit=0.7, shared=(56, 0.4)), moe(experts=5, top=1, ff=24, limit=2.0, shared=None),
                moe(experts=3, top=3, ff=72, limit=1.0, shared=(8, 3.0)), moe(experts=70, top=4, ff=16, limit=1.2, shared=None)):
        f, w = _ff_setup(mlp, width)
        wn = {k: v.double().numpy() for k, v in w.items()}
        want = np.stack([mo.routed_ff(x, wn, "f.", mlp)[0] for x in h.double().numpy()])
        wt = {k: v.to(dev) for k, v in w.items()}
        f.finish_weights(wt)
        got = f.forward(h.to(dev), wt).double().cpu().numpy()
        assert np.abs(got - want).max() < 2e-4 * max(1.0, np.abs(want).max())


def test_routing_weight_scales_the_input_not_the_output():
    """The clipped activation is not homogeneous: expert(s h) differs from s expert(h), and the scores
    are used as they are (they do not sum to one)."""
    width = 32
    mlp = moe(experts=4, top=2, ff=24, limit=0.5, shared=None)
    f, w = _ff_setup(mlp, width, seed=4)
    h = 2.0 * torch.randn(6, width, generator=torch.Generator().manual_seed(9))
    wn = {k: v.double().numpy() for k, v in w.items()}
    hn = h.double().numpy()
    want = np.stack([mo.routed_ff(x, wn, "f.", mlp)[0] for x in hn])
    outside, renorm = [], []
    for x in hn:
        s = mo.sigmoid(wn["f.router"] @ x)
        top = np.argsort(-s)[:2]
        outside.append(sum(s[e] * mo.capped_expert(x, wn, f"f.e{e}.", 0.5) for e in top))
        renorm.append(sum(mo.capped_expert(s[e] / s[top].sum() * x, wn, f"f.e{e}.", 0.5) for e in top))
    assert np.abs(np.stack(outside) - want).max() > 0.05 and np.abs(np.stack(renorm) - want).max() > 0.05
    f.finish_weights(w)
    assert np.abs(f.forward(h, w).double().numpy() - want).max() < 1e-4


@pytest.mark.parametrize("dev", DEVS)
def test_route_topk_order_ties_and_weights(dev):
    _skip(dev)
    from mxserve.ops import seqmix
    z = torch.tensor([[0.1, 2.0, -1.0, 2.0, 0.5], [-3.0, -3.0, -3.0, -3.0, -3.0], [9.0, -9.0, 0.0, 1.0, 8.0]], device=dev)
    w, ids = seqmix.route_topk(z, 3)
    assert ids.cpu().tolist() == [[1, 3, 4], [0, 1, 2], [0, 4, 3]]
    assert torch.allclose(w.cpu(), torch.sigmoid(torch.tensor([[2.0, 2.0, 0.5], [-3.0] * 3, [9.0, 8.0, 1.0]])), atol=1e-6)
    w, _ = seqmix.route_topk(z, 2, renorm=True)
    assert torch.allclose(w.sum(-1).cpu(), torch.ones(3), atol=1e-6)
    g = torch.Generator().manual_seed(0)
    z = torch.randn(50, 130, generator=g).to(dev)  # more experts than a wave has lanes
    w, ids = seqmix.route_topk(z, 7)
    ref = torch.topk(torch.sigmoid(z.cpu()), 7)
    assert torch.equal(ids.cpu().long(), ref.indices) and torch.allclose(w.cpu(), ref.values, atol=1e-6)


@pytest.mark.parametrize("dev", DEVS)
def test_capped_activation(dev):
    """The gate is capped from above only, the other branch from both sides, and one is added to it."""
    _skip(dev)
    from mxserve.ops import seqmix
    g = torch.tensor([-5.0, -0.5, 0.0, 0.4, 1.0, 7.0])
    u = torch.tensor([-9.0, -1.0, 0.3, 1.0, 1.2, 9.0])
    L = 1.0
    gu = torch.cat([g.repeat(6, 1), u.view(6, 1).expand(6, 6)], 1).to(dev)
    got = seqmix.capped_glu(gu, L).double().cpu().numpy()
    gc = np.minimum(g.double().numpy(), L)
    want = (gc * mo.sigmoid(1.702 * gc))[None, :] * (np.clip(u.double().numpy(), -L, L) + 1.0)[:, None]
    assert np.abs(got - want).max() < 1e-6
    assert got[0, 0] == 0.0 * got[0, 0] and abs(got[0, 0]) < 1e-12  # up = -limit: u + 1 = 0
    assert got[5, 0] < 0  # a very negative gate passes uncapped (and is tiny), times u + 1 = 2


@pytest.mark.parametrize("dev", DEVS)
def test_expert_rows_sorted_and_gathered(dev):
    _skip(dev)
    from mxserve.ops import seqmix
    g = torch.Generator().manual_seed(1)
    T, k, E, W = 37, 3, 9, 20
    ids = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32).to(dev)
    wts = torch.rand(T, k, generator=g).to(dev)
    h = torch.randn(T, W, generator=g).to(dev)
    offs, inv = seqmix.expert_align(ids, E)
    o, iv = offs.cpu().tolist(), inv.cpu().long()
    assert o[0] == 0 and o[-1] == T * k and sorted(iv.tolist()) == list(range(T * k))
    flat = ids.cpu().reshape(-1).long()
    for p in range(T * k):
        assert o[flat[p]] <= iv[p] < o[flat[p] + 1]
    xs = seqmix.gather_scaled(h, wts, inv).cpu()
    for p in (0, 5, T * k - 1):
        assert torch.allclose(xs[iv[p]], (h[p // k] * wts[p // k, p % k]).cpu(), atol=1e-6)
    sp = seqmix.spread_scaled(h, wts, ids, E).cpu()
    assert sp.shape == (E, T, W)
    dense_w = torch.zeros(T, E).scatter_(1, ids.cpu().long(), wts.cpu())
    assert torch.allclose(sp, dense_w.t().unsqueeze(2) * h.cpu().unsqueeze(0), atol=1e-6)
    back = seqmix.expert_combine(xs.to(dev), inv, k, T, extra=h).cpu()
    assert torch.allclose(back, h.cpu() * (1.0 + wts.cpu().sum(1, keepdim=True)), atol=1e-5)


@pytest.mark.parametrize("dev", DEVS)
def test_residual_scale_and_norm_weights_around_zero(dev):
    _skip(dev)
    from mxserve.ops import seqmix
    g = torch.Generator().manual_seed(2)
    x = torch.randn(5, 24, generator=g)
    a = torch.randn(5, 24, generator=g)
    wn = 0.1 * torch.randn(24, generator=g)
    xs = x.clone().to(dev)
    hh = seqmix.resid_update(xs, a.to(dev), 1e-3, norm_w=wn.to(dev), out_dtype=torch.float32, a_scale=0.6, w_offset=1.0)
    x2 = x.double() + 0.6 * a.double()
    want = x2 / torch.sqrt((x2 ** 2).mean(-1, keepdim=True) + 1e-3) * (1.0 + wn.double())
    assert torch.allclose(xs.cpu().double(), x2, atol=1e-6) and torch.allclose(hh.cpu().double(), want, atol=1e-5)


# ----------------------------------------------------------------------------- whole models, schedules
@pytest.fixture(scope="module")
def base(tmp_path_factory):
    path = tmp_path_factory.mktemp("momuvik_base")
    w = write_checkpoint(path, BASE, seed=11)
    toks = {f"r{i}": _tokens(n, BASE["vocab"], 20 + i) for i, n in enumerate([90, 37, 1, 64, 130, 16])}
    want = {rid: _oracle_model(BASE, w, t) for rid, t in toks.items()}
    return path, w, toks, want


@pytest.mark.parametrize("dev,dtype,tol", DEV_DTYPE_TOL)
def test_portions_and_decoding(base, dev, dtype, tol):
    """Whole prompt, token by token, and portions of several sizes down to two tokens."""
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
    GPU): pages fill and new ones start."""
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
    sizes that are multiples of 16 (what the matrix-core attention takes in bf16): its last portions
    end in partial tiles on the last page of the block table."""
    _skip(dev)
    a = latent(heads=4, dim=32, rot_dim=16, vdim=32, kv_rank=64, q_rank=48, scale=0.15)
    cfg = config([layer(a, dense(128)), layer(latent(heads=16, dim=16, rot_dim=32, vdim=16, kv_rank=32, q_rank=32, scale=0.2),
                                              moe(experts=4, top=2, ff=32, limit=1.0)), layer(a, dense(128), weights_of=0)],
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


_T = latent(heads=1, dim=8, rot_dim=2, vdim=2, kv_rank=8, q_rank=8, scale=1.0, base=10.0)
VARIANTS = {
    "one_head_one_pair_no_scales": config([layer(_T, dense(24)), layer(_T, moe(experts=2, top=2, ff=8, limit=5.0, shared=None))],
                                          width=40, vocab=50, eps=1e-3, embed_scale=1.0, mult=1.0),
    "a_chain_of_shared_weights": config([layer(latent(), moe(experts=3, top=1, ff=24, limit=0.6, shared=(16, 2.0))),
                                         layer(latent(), moe(experts=3, top=1, ff=24, limit=0.6, shared=(16, 2.0)), weights_of=0),
                                         layer(latent(), moe(experts=3, top=1, ff=24, limit=0.6, shared=(16, 2.0)), weights_of=1),
                                         layer(latent(heads=5, dim=8, rot_dim=8, vdim=8, kv_rank=8, q_rank=8), None)],
                                        width=64, vocab=70, embed_scale=7.5, mult=0.3),
    "equal_sizes_everywhere": config([layer(latent(heads=2, dim=16, rot_dim=16, vdim=16, kv_rank=16, q_rank=16), dense(16)),
                                      layer(latent(heads=2, dim=16, rot_dim=16, vdim=16, kv_rank=16, q_rank=16),
                                            moe(experts=16, top=16, ff=16, limit=1.0, shared=(16, 1.0)))], width=16, vocab=16),
    "sizes_that_fit_no_vector_load": config([layer(latent(heads=3, dim=10, rot_dim=6, vdim=7, kv_rank=12, q_rank=9, scale=0.3),
                                                   moe(experts=3, top=2, ff=14, limit=1.1, shared=(5, 0.9))),
                                             layer(latent(heads=5, dim=6, rot_dim=2, vdim=9, kv_rank=21, q_rank=11, scale=0.4), dense(22))],
                                            width=50, vocab=37),
    "wide_latent_many_heads": config([layer(latent(heads=12, dim=8, rot_dim=40, vdim=72, kv_rank=264, q_rank=136, scale=0.07),
                                            moe(experts=9, top=4, ff=40, limit=1.5, shared=(72, 0.5)))], width=72, vocab=60),
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
    _skip(dev)
    path, w, toks, _ = base
    eng = engine(path, dev, "float32", max_tokens=128)
    tap = eng.runner.model.layer_tap = []
    replay(eng, [[("a", toks["r1"], True)]])
    ref = mo.run(BASE, w, toks["r1"])[1]
    assert len(tap) == len(ref) == len(BASE["layers"])
    for a, b in zip(tap, ref):
        assert np.abs(a.double().cpu().numpy() - b).max() < 1e-3 * max(1.0, np.abs(b).max())


def test_pages_and_tensors_of_the_plan():
    """Every layer has pages of its own -- a row of latent plus rotated part per token -- also a layer
    that runs another's tensors; such a layer has no tensors and shares the mixer object."""
    from mxserve.models.config import momuvik_config
    from mxserve.models.momuvik import layer_plan, mixers_of, owners, weight_shapes
    plan, ms = layer_plan(BASE, 16), mixers_of(BASE)
    assert owners(BASE) == [0, 1, 0, 1, 4, 5] and ms[2] is ms[0] and ms[3] is ms[1] and ms[4] is not ms[0]
    assert all(r.owns_kv and r.kv_heads == 1 for r in plan.runs) and len({r.koff for r in plan.runs}) == len(plan.runs)
    rows = [l["mixer"]["kv_rank"] + l["mixer"]["rot_dim"] for l in BASE["layers"]]
    assert plan.block_elems == 16 * sum(rows) and plan.state_floats == 0
    sh = weight_shapes(BASE)
    assert not any(k.startswith(("l2.", "l3.")) for k in sh) and "l1.mlp.shared.up" in sh and "l5.mlp.shared.up" not in sh
    assert sh["l1.mlp.e5.down"] == (BASE["width"], 40) and "l4.norm2" not in sh and sh["l4.mix.sink"] == (2,)
    cfg = momuvik_config("m", BASE)
    assert not cfg.has_recurrent_state and cfg.kv_bytes_per_token(2) == 2 * sum(rows)
    with pytest.raises(ValueError):
        owners(config([layer(weights_of=1), layer(weights_of=0)]))


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
        lg = mo.run(BASE, w, p + o[:-1])[0][len(p) - 1:]
        for row, tok in zip(lg, o):
            assert row[tok] >= row.max() - margin * (row.max() - row.min())


def test_registered_small_model_runs():
    """The registry's small Momuvik with random weights, by name, as a served model would start."""
    from mxserve.config import EngineArgs
    from mxserve.engine.engine import LLMEngine
    from mxserve.engine.request import SamplingParams
    eng = LLMEngine(EngineArgs(model="tiny-momuvik", device="cpu", dtype="float32", num_gpu_blocks=16, cpu_num_blocks=16,
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
