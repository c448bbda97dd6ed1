"""The matrix-core latent attention (csrc/mixers/latent_attention.hip) against the PyTorch form of the
same op on the CPU: every size class of the kernel, head counts that do not divide a 16-row tile,
prompt chunks that end in partial tiles, single-token steps whose keys are split over several waves,
mixed steps, sinks, scattered pages with stale rows behind a sequence's end."""
import pytest
import torch

from mxserve.ops import seqmix

pytestmark = pytest.mark.gpu


def _case(H, dk, rank, lens, qlens, seed=0, sink=True, stale=float("nan")):
    """Sequences of `lens` tokens whose last `qlens` are this step's rows; pages in random order."""
    g = torch.Generator().manual_seed(seed)
    bs, S = 16, len(lens)
    nbs = [-(-n // bs) for n in lens]
    total = sum(nbs) + 2
    perm = torch.randperm(total, generator=g)
    mb = max(nbs) + 1
    bt = torch.zeros(S, mb, dtype=torch.int32)
    cache = torch.full((total, 8 + bs * dk), stale)
    at = 0
    for s, (n, nb) in enumerate(zip(lens, nbs)):
        bt[s, :nb] = perm[at:at + nb].to(torch.int32)
        at += nb
        rows = torch.randn(nb * bs, dk, generator=g) * 0.5
        rows[n:] = stale  # what lies behind the sequence's end must not matter
        cache[bt[s, :nb].long(), 8:] = rows.view(nb, bs * dk)
    cache = torch.nan_to_num(cache, nan=stale) if stale == stale else cache
    T = sum(qlens)
    q = torch.randn(T, H * dk, generator=g) * 0.5
    qsl = torch.tensor([0] + list(torch.tensor(qlens).cumsum(0)), dtype=torch.int32)
    sk = torch.randn(H, generator=g) if sink else None
    return q, cache, bt, qsl, torch.tensor(lens, dtype=torch.int32), sk


@pytest.mark.parametrize("H,dk,rank", [(10, 184, 96), (3, 48, 32), (16, 576, 512), (12, 320, 256), (5, 136, 112), (40, 64, 64),
                                       (6, 408, 352), (2, 552, 512)])
@pytest.mark.parametrize("lens,qlens", [([300], [300]), ([77, 130, 16, 250], [1, 1, 1, 1]), ([100, 45, 333], [1, 45, 21]),
                                         ([17], [2])])
def test_latent_attention_kernel(H, dk, rank, lens, qlens, monkeypatch):
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    q, cache, bt, qsl, sl, sk = _case(H, dk, rank, lens, qlens, seed=H + dk)
    qb, cb = q.to(torch.bfloat16), torch.nan_to_num(cache).to(torch.bfloat16)
    want = seqmix.window_attention(qb.float(), cb.float(), bt, qsl, sl, 8, 8, H, 1, dk, rank, 16, 0.11, 0, 0, max(qlens),
                                   sink=sk, v_stride=dk)
    dev = torch.device("cuda")
    cg = cache.to(torch.bfloat16).to(dev)  # with the stale rows as they are
    args = (qb.to(dev), cg, bt.to(dev), qsl.to(dev), sl.to(dev), 8, H, dk, rank, 16, 0.11)
    for form in ("single", "pair"):  # the two forms of the widest size class (the others have one)
        monkeypatch.setattr(seqmix, "LATENT_WIDE_FORM", form)
        for max_seq in (max(lens), 16):  # keys split over several waves where the step is small, and never
            got = seqmix.latent_attention(*args, max(qlens), max_seq, sink=None if sk is None else sk.to(dev))
            err = (got.float().cpu() - want).abs().max().item()
            assert err < 0.02, f"{form}: max abs error {err}"
    # the general kernel on the same operands (strided value rows)
    got = seqmix.window_attention(args[0], cg, args[2], args[3], args[4], 8, 8, H, 1, dk, rank, 16, 0.11, 0, 0, max(qlens),
                                  sink=None if sk is None else sk.to(dev), v_stride=dk)
    assert (got.float().cpu() - want).abs().max().item() < 0.02


def test_latent_attention_without_sink_and_fp32():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    q, cache, bt, qsl, sl, _ = _case(4, 96, 64, [50, 9], [50, 1], seed=3, sink=False, stale=7.0)
    want = seqmix.window_attention(q, cache, bt, qsl, sl, 8, 8, 4, 1, 96, 64, 16, 0.2, 0, 0, 50, v_stride=96)
    dev = torch.device("cuda")
    got = seqmix.latent_attention(q.to(dev), cache.to(dev), bt.to(dev), qsl.to(dev), sl.to(dev), 8, 4, 96, 64, 16, 0.2, 50, 50)
    assert (got.cpu() - want).abs().max().item() < 1e-4  # fp32 runs the general kernel
    got = seqmix.latent_attention(q.to(dev).bfloat16(), cache.to(dev).bfloat16(), bt.to(dev), qsl.to(dev), sl.to(dev), 8, 4,
                                  96, 64, 16, 0.2, 50, 50)
    assert (got.float().cpu() - want).abs().max().item() < 0.03
