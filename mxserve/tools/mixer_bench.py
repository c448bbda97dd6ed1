"""Prefill and decode throughput of a layer-list design (Voletar, Tapasun, Momuvik, Seradra) beside the models
closest to it at equal width, depth and feed-forward size (random weights), through the same engine
path: forced steps of the scheduler, the model runner, paged K/V and state slots, decode through the
captured graphs.  Voletar stands beside a Llama-shaped model; Tapasun beside Voletar and that model;
Momuvik beside a Mixtral-shaped model (softmax attention and routed experts of the same sizes); Seradra
beside Momuvik and that model.

  python bench.py --mixer-bench [--mixer-design voletar|tapasun|momuvik|seradra] [--mixer-sizes 1024,2048]
                  [--mixer-prompt 4096] [--mixer-batch 64]

Prints one JSON line per (size, model): prefill tokens/s of one prompt in one step, decode tokens/s
of a batch of sequences at that context, and per-kernel times of the mixers against their
roofline (FLOP and byte counts are the algorithm's own, stated next to each entry)."""
from __future__ import annotations

import dataclasses
import json
import time

import torch

from ..config import EngineArgs
from ..engine.engine import LLMEngine
from ..engine.replay import TraceReplayer
from ..models import config as mcfg

PEAK_BF16 = 2.5e15  # dense MFMA bf16 FLOP/s
PEAK_F32 = 157e12  # VALU / fp32 MFMA FLOP/s
PEAK_HBM = 8e12  # bytes/s


def voletar_shape(width: int, layers: int = 4, window: int = 1024) -> dict:
    """Alternating parallel / lightning layers with the head sizes of a model of this width."""
    heads = width // 128
    par = {"type": "parallel",
           "mixer": {"left": {"heads": heads * 2, "kv_heads": max(heads // 2, 1), "dim": 64, "vdim": 64, "scale": 0.125,
                              "mask": {"size": window, "keep_first": 4}},
                     "right": {"heads": max(heads // 2, 1), "dim": 64, "vdim": 128, "gate_cap": 15.0}},
           "mlp": {"kind": "dense", "ff": 4 * width}}
    lig = {"type": "lightning", "mixer": {"heads": heads, "dim": 128, "vdim": 128,
                                          "decay": [1.0 - 2.0 ** -(3 + 5 * i / max(heads - 1, 1)) for i in range(heads)]},
           "mlp": {"kind": "dense", "ff": 4 * width}}
    return {"architecture": "Voletar", "width": width, "vocab": 32000, "norm": {"eps": 1e-5}, "logit_softcap": 30.0,
            "layers": [par if i % 2 == 0 else lig for i in range(layers)]}


def tapasun_shape(width: int, layers: int = 4) -> dict:
    """State space, attention, parallel (attention + delta rule), attention on the second layer's pages,
    with the head sizes of a model of this width and a gated feed-forward of 8/3 width."""
    hq = width // 64
    ffn = {"kind": "dense", "ff": (8 * width // 3) // 256 * 256}
    bands = {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192}
    att = {"heads": hq, "kv_heads": max(hq // 4, 1), "dim": 64, "vdim": 64, "scale": 0.125,
           "rot": {"dims": 64, "base": 500000.0, "scaling": bands}}
    ssm = {"type": "mamba2", "mlp": ffn, "mixer": {"heads": width // 32, "vdim": 64, "state": 128,
                                                  "groups": min(8, width // 32), "conv": 4, "norm_groups": min(8, width // 32)}}
    gh = max(width // 128, 1)
    par = {"type": "parallel", "mlp": ffn, "mixer": {
        "left": {"heads": hq, "kv_heads": max(hq // 8, 1), "dim": 64, "vdim": 64, "scale": 0.125,
                 "rot": {"dims": 32, "base": 500000.0, "scaling": {"factor": 4.0}}},
        "right": {"heads": gh, "kv_heads": gh, "dim": 128, "vdim": 128, "conv": 4}, "left_scale": 0.5, "right_scale": 1.0}}
    kinds = [ssm, {"type": "attention", "mlp": ffn, "mixer": att}, par,
             {"type": "attention", "mlp": ffn, "mixer": dict(att, kv_from=1)}]
    return {"architecture": "Tapasun", "width": width, "vocab": 32000, "norm": {"eps": 1e-5}, "embedding": {"scale": 1.0},
            "layers": [kinds[i % 4] for i in range(layers)]}


MOE_EXPERTS, MOE_TOP = 8, 2


def momuvik_shape(width: int, layers: int = 4) -> dict:
    """Latent attention with 128 + 64 wide query/key heads, 128-wide values and a 512-wide latent; eight
    experts of 4/3 width, two per token, and a shared expert of a third of the width."""
    ff = (4 * width // 3) // 256 * 256
    att = {"heads": width // 128, "dim": 128, "rot_dim": 64, "vdim": 128, "kv_rank": 512, "q_rank": max(3 * width // 8, 256),
           "scale": 192 ** -0.5, "rot": {"dims": 64, "base": 10000.0}}
    mlp = {"kind": "moe", "router": {"experts": MOE_EXPERTS, "top": MOE_TOP}, "expert": {"ff": ff, "limit": 7.0},
           "shared": {"ff": max(width // 3 // 128 * 128, 128), "limit": 7.0}}
    return {"architecture": "Momuvik", "width": width, "vocab": 32000, "norm": {"eps": 1e-5}, "embedding": {"scale": 1.0},
            "residual_mult": 1.0, "layers": [{"type": "latent_attention", "mixer": att, "mlp": mlp} for _ in range(layers)]}


def seradra_shape(width: int, layers: int = 4, window: int = 1024) -> dict:
    """Head-mixing attention (128-wide heads, 4 query heads per kv head, half of each head rotated with
    ramp-blended frequencies) and windowed latent attention (the sizes of momuvik_shape) in turn; the first
    layer's feed-forward is the ungated one of 4 width, the others eight experts of 4/3 width, two per token."""
    heads = max(width // 128, 1)
    ff = (4 * width // 3) // 256 * 256
    att = {"heads": heads, "kv_heads": max(heads // 4, 1), "dim": 128, "vdim": 128, "scale": 128 ** -0.5,
           "mask": {"size": window}, "rot": {"dims": 64, "base": 500000.0,
                                             "scaling": {"factor": 8.0, "original": 8192, "fast": 32.0, "slow": 1.0}}}
    lat = {"heads": heads, "dim": 128, "rot_dim": 64, "vdim": 128, "kv_rank": 512, "q_rank": max(3 * width // 8, 256),
           "scale": 192 ** -0.5, "mask": {"size": window}, "rot": {"dims": 64, "base": 10000.0}}
    moe = {"kind": "moe", "router": {"experts": MOE_EXPERTS, "top": MOE_TOP}, "expert": {"ff": ff}}
    kinds = [{"type": "attention", "mixer": att, "mlp": {"kind": "dense", "ff": 4 * width}},
             {"type": "latent_attention", "mixer": lat, "mlp": moe}, {"type": "attention", "mixer": att, "mlp": moe},
             {"type": "latent_attention", "mixer": lat, "mlp": moe}]
    return {"architecture": "Seradra", "width": width, "vocab": 32000, "norm": {"eps": 1e-5},
            "layers": [kinds[i % 4] for i in range(layers)]}


def register(width: int, layers: int, design: str = "voletar") -> tuple:
    if design == "seradra":
        sd = mcfg.seradra_config(f"seradra-w{width}", seradra_shape(width, layers))
        mcfg.REGISTRY[sd.name.lower()] = sd
        return (sd.name,) + register(width, layers, "momuvik")
    if design == "momuvik":
        m = mcfg.momuvik_config(f"momuvik-w{width}", momuvik_shape(width, layers))
        mcfg.REGISTRY[m.name.lower()] = m
        base = mcfg.REGISTRY["small-llama"]
        x = dataclasses.replace(base, name=f"mixtral-w{width}", arch="mixtral", hidden_size=width,
                                intermediate_size=(4 * width // 3) // 256 * 256, num_layers=layers, num_heads=width // 128,
                                num_kv_heads=max(width // 512, 1), head_dim=128, vocab_size=32000, tie_word_embeddings=False,
                                num_experts=MOE_EXPERTS, num_experts_per_tok=MOE_TOP)
        mcfg.REGISTRY[x.name.lower()] = x
        return (m.name, x.name)
    if design == "tapasun":
        t = mcfg.tapasun_config(f"tapasun-w{width}", tapasun_shape(width, layers))
        mcfg.REGISTRY[t.name.lower()] = t
    v = mcfg.voletar_config(f"voletar-w{width}", voletar_shape(width, layers))
    mcfg.REGISTRY[v.name.lower()] = v
    base = mcfg.REGISTRY["small-llama"]
    # gated feed-forward of 8/3 width has the parameters of a dense one of 4 width
    l = dataclasses.replace(base, name=f"llama-w{width}", hidden_size=width, intermediate_size=(8 * width // 3) // 256 * 256,
                            num_layers=layers, num_heads=width // 64, num_kv_heads=max(width // 256, 1), head_dim=64,
                            vocab_size=32000, tie_word_embeddings=False)
    mcfg.REGISTRY[l.name.lower()] = l
    return (t.name, v.name, l.name) if design == "tapasun" else (v.name, l.name)


def _time(fn, reps: int) -> float:
    fn()  # code objects loaded, allocator warm
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / reps


def run_model(name: str, prompt: int, batch: int, context: int, reps: int = 5) -> dict:
    bs = 16
    blocks = (batch * (context + 64) + prompt) // bs + batch + 8
    args = EngineArgs(model=name, device="cuda", dtype="bfloat16", block_size=bs, num_gpu_blocks=blocks,
                      max_model_len=max(prompt, context) + 128, max_num_seqs=batch, max_num_batched_tokens=max(prompt, batch * 64),
                      enable_prefix_caching=False, async_scheduling=False, load_format="random", cuda_graph_max_bs=batch)
    eng = LLMEngine(args)
    rp = TraceReplayer(eng)
    g = torch.Generator().manual_seed(0)
    V = eng.model_config.vocab_size
    toks = lambda n: torch.randint(3, V, (n,), generator=g).tolist()  # noqa: E731
    n_pf = [0]

    def prefill():
        n_pf[0] += 1
        rid = f"p{n_pf[0]}"
        rp.step([{"id": rid, "tokens": toks(prompt), "want": [prompt - 1]}], [rid])
    prefill()
    t_pf = _time(prefill, reps)
    # decode: `batch` sequences brought to `context` tokens in chunks, then single tokens through the graphs
    ids = [f"d{i}" for i in range(batch)]
    per = max(1, min(batch, args.max_num_batched_tokens // context))
    for i in range(0, batch, per):
        rp.step([{"id": r, "tokens": toks(context), "want": []} for r in ids[i:i + per]], [])

    def decode():
        rp.step([{"id": r, "tokens": toks(1), "want": [0]} for r in ids], [])
    decode()
    t_dec = _time(decode, 4 * reps)
    out = {"model": name, "params_m": round(eng.model_config.num_params() / 1e6, 1), "prompt": prompt,
           "prefill_tok_s": round(prompt / t_pf), "prefill_ms": round(1e3 * t_pf, 3), "decode_batch": batch,
           "decode_context": context, "decode_tok_s": round(batch / t_dec), "decode_step_ms": round(1e3 * t_dec, 3),
           "decode_graph": bool(eng.runner.graphs)}
    rp.step([], ids)
    eng.close()
    return out


def kernel_rooflines(width: int, prompt: int, batch: int, context: int) -> list:
    """The mixers' own kernels alone, at this size: time, and time over the roofline time."""
    from .. import ops
    from ..ops import seqmix
    dev = torch.device("cuda")
    dt = torch.bfloat16
    bs, out = 16, []
    heads = width // 128
    i32 = dict(dtype=torch.int32, device=dev)

    def entry(name, t, flops, peak, bytes_, note):
        roof = max(flops / peak, bytes_ / PEAK_HBM)
        out.append({"kernel": name, "width": width, "ms": round(1e3 * t, 4), "roofline_ms": round(1e3 * roof, 4),
                    "x_roofline": round(t / roof, 1), "counts": note})

    for mode, T, S, ctx in (("prefill", prompt, 1, prompt), ("decode", batch, batch, context)):
        qsl = torch.arange(0, T + 1, T // S, **i32)
        seq = torch.full((S,), ctx, **i32)
        nb = -(-ctx // bs)
        bt = torch.arange(S * nb, **i32).view(S, nb)
        # window attention of the parallel layers
        H, G, dk, dv, win = heads * 2, max(heads // 2, 1), 64, 64, 1024
        cache = torch.randn(S * nb, G * bs * (dk + dv), device=dev).to(dt)
        q = torch.randn(T, H * dk, device=dev).to(dt)
        t = _time(lambda: seqmix.window_attention(q, cache, bt, qsl, seq, 0, G * bs * dk, H, G, dk, dv, bs, 0.125, win, 4,
                                                  max_query_len=T // S), 5)
        keys = min(win, ctx) if mode == "decode" else min(win, ctx / 2)
        entry(f"window_attention/{mode}", t, 2.0 * T * H * keys * (dk + dv), PEAK_BF16,
              2.0 * (S * min(win, ctx) * G * (dk + dv) + 2 * T * H * dk), f"{T} rows x {H} heads x ~{int(keys)} keys, bf16 MFMA peak")
        # the closest kernel of the Llama path at the same head layout, full causal
        kv = torch.randn(S * nb, 1, 2, G, bs, 64, device=dev).to(dt)
        q3 = q.view(T, H, dk)
        if mode == "prefill":
            fn = lambda: ops.paged_attention_prefill(q3, kv[:, 0], bt, qsl, seq, 0.125, T)  # noqa: E731
            keys_l = ctx / 2
        else:
            fn = lambda: ops.paged_attention_decode(q3, kv[:, 0], bt, seq, 0.125, ctx)  # noqa: E731
            keys_l = ctx
        t = _time(fn, 5)
        entry(f"paged_attention/{mode} (llama)", t, 2.0 * T * H * keys_l * 128, PEAK_BF16,
              2.0 * (S * ctx * G * 128 + 2 * T * H * dk), f"{T} rows x {H} heads x ~{int(keys_l)} keys, bf16 MFMA peak")
        # the recurrences: fp32 state, two multiply-adds per state element and token
        for name, Hh, d1, d2, mlstm in (("decay_scan", heads, 128, 128, False), ("mlstm_scan", max(heads // 2, 1), 64, 128, True)):
            n = Hh * d1 * d2 + (Hh * (d1 + 1) if mlstm else 0)
            state = torch.zeros(S, n, device=dev)
            rows = torch.arange(S, **i32)
            qq, kk = (torch.randn(T, Hh * d1, device=dev).to(dt) for _ in range(2))
            vv = torch.randn(T, Hh * d2, device=dev).to(dt)
            if mlstm:
                gates = torch.randn(T, 2 * Hh, device=dev)
                fn = lambda: seqmix.mlstm_scan(qq, kk, vv, gates, state, rows, 0, qsl, seq, Hh, d1, d2, 15.0, d1 ** -0.5,  # noqa: E731
                                               max_query_len=T // S)
            else:
                dec = torch.full((Hh,), 0.99, device=dev)
                fn = lambda: seqmix.decay_scan(qq, kk, vv, dec, state, rows, 0, qsl, seq, Hh, d1, d2, max_query_len=T // S)  # noqa: E731
            t = _time(fn, 5)
            entry(f"{name}/{mode}", t, 4.0 * T * Hh * d1 * d2, PEAK_F32, 8.0 * S * n + 2.0 * T * Hh * (2 * d1 + 3 * d2),
                  f"{T} rows x {Hh} heads x {d1}x{d2} state, fp32 peak; state read and written once")
    return out


def tapasun_rooflines(width: int, prompt: int, batch: int, context: int) -> list:
    """Tapasun's own kernels alone, at the sizes of tapasun_shape(width): time over roofline time.  The
    like kernels of Voletar (kernel_rooflines) are what they stand beside: its scans for the column
    scans, its windowed attention for the attention with a sink, its gated norm and cache write for
    the small kernels."""
    from ..models.mixers import rotary_frequencies
    from ..ops import seqmix
    dev = torch.device("cuda")
    dt = torch.bfloat16
    bs, out = 16, []
    i32 = dict(dtype=torch.int32, device=dev)
    rnd = lambda *sh: torch.randn(*sh, device=dev).to(dt)  # noqa: E731

    def entry(name, t, flops, peak, bytes_, note):
        roof = max(flops / peak, bytes_ / PEAK_HBM)
        out.append({"kernel": name, "width": width, "ms": round(1e3 * t, 4), "roofline_ms": round(1e3 * roof, 4),
                    "x_roofline": round(t / roof, 1), "counts": note})

    for mode, T, S, ctx in (("prefill", prompt, 1, prompt), ("decode", batch, batch, context)):
        qsl = torch.arange(0, T + 1, T // S, **i32)
        seq = torch.full((S,), ctx, **i32)
        rows = torch.arange(S, **i32)
        nb = -(-ctx // bs)
        bt = torch.arange(S * nb, **i32).view(S, nb)
        pos = torch.cat([torch.arange(ctx - T // S, ctx, device=dev) for _ in range(S)])
        slots = torch.cat([bt[s_].long().repeat_interleave(bs)[ctx - T // S:ctx] * bs + pos[:T // S] % bs for s_ in range(S)])
        # attention with a sink, every earlier key visible
        H, G, dk, dv = width // 64, max(width // 256, 1), 64, 64
        cache = rnd(S * nb, G * bs * (dk + dv))
        q, k, v = rnd(T, H * dk), rnd(T, G * dk), rnd(T, G * dv)
        sink = torch.zeros(H, device=dev)
        t = _time(lambda: seqmix.window_attention(q, cache, bt, qsl, seq, 0, G * bs * dk, H, G, dk, dv, bs, 0.125, 0, 0,
                                                  max_query_len=T // S, sink=sink), 5)
        keys = ctx if mode == "decode" else ctx / 2
        entry(f"sink_attention/{mode}", t, 2.0 * T * H * keys * (dk + dv), PEAK_BF16,
              2.0 * (S * ctx * G * (dk + dv) + 2 * T * H * dk), f"{T} rows x {H} heads x ~{int(keys)} keys, bf16 MFMA peak")
        fr = rotary_frequencies(dk, 500000.0, None).to(dev)
        nw = torch.ones(dk, device=dev).to(dt)
        t = _time(lambda: seqmix.rope_qkv_cache(q, k, v, pos, slots, cache, 0, G * bs * dk, H, G, dk, dv, bs, fr, nw, nw,
                                                1e-5, None), 5)
        entry(f"rope_qkv_cache/{mode}", t, 0.0, PEAK_F32, 2.0 * T * (2 * H * dk + 2 * G * (dk + dv)),
              f"{T} rows: q read and written, k and v read and written to the pages")
        # column scans: fp32 state; 4 (state space) or 7 (delta rule) flops per state element and token
        for name, Hh, Gg, d1, d2, fl in (("ssd_scan", width // 32, min(8, width // 32), 128, 64, 4.0),
                                         ("delta_scan", max(width // 128, 1), max(width // 128, 1), 128, 128, 7.0)):
            n = Hh * d1 * d2
            state = torch.zeros(S, n, device=dev)
            qq, kk, vv, bb = rnd(T, Gg * d1), rnd(T, Gg * d1), rnd(T, Hh * d2), rnd(T, Hh)
            hb = torch.zeros(Hh, device=dev)
            if name == "ssd_scan":
                fn = lambda: seqmix.ssd_scan(vv, kk, qq, bb, hb, hb, hb, state, rows, 0, qsl, seq, Hh, Gg, d1, d2,  # noqa: E731
                                             max_query_len=T // S)
                extra = 0
            else:
                aa = rnd(T, Hh * d1)
                cb = torch.zeros(Hh * d1, device=dev)
                fn = lambda: seqmix.delta_scan(qq, kk, vv, bb, aa, cb, hb, state, rows, 0, qsl, seq, Hh, Gg, d1, d2,  # noqa: E731
                                               d1 ** -0.5, max_query_len=T // S)
                extra = T * Hh * d1
            t = _time(fn, 5)
            entry(f"{name}/{mode}", t, fl * T * Hh * d1 * d2, PEAK_F32,
                  8.0 * S * n + 2.0 * (T * (2 * Gg * d1 + Hh * d2) + extra) + 4.0 * T * Hh * d2,
                  f"{T} rows x {Hh} heads x {d1}x{d2} state, fp32 peak; state read and written once")
        # short convolution over the state-space layer's channels, and its gated norm
        C = 2 * width + 2 * min(8, width // 32) * 128
        x, wc, bc = rnd(T, C), rnd(4, C), rnd(C)
        cst = torch.zeros(S, 3 * C, device=dev)
        t = _time(lambda: seqmix.causal_conv(x, wc, bc, cst, rows, 0, qsl, seq), 5)
        entry(f"causal_conv/{mode}", t, 0.0, PEAK_F32, 4.0 * T * C + 24.0 * S * C, f"{T} rows x {C} channels, 4 taps; rows read and written once")
        N = 2 * width
        o, gate, wn = torch.randn(T, N, device=dev), rnd(T, N), rnd(N)
        t = _time(lambda: seqmix.gated_norm(o, gate, wn, 1e-5, 8, "silu", True, dt), 5)
        entry(f"gated_norm/{mode}", t, 0.0, PEAK_F32, 8.0 * T * N, f"{T} rows x {N}: fp32 in, gate in, bf16 out")
        t = _time(lambda: seqmix.gated_rms_norm(o, gate, wn, 1e-5, 8, dt), 5)
        entry(f"gated_rms_norm/{mode} (voletar)", t, 0.0, PEAK_F32, 8.0 * T * N, f"{T} rows x {N}: fp32 in, gate in, bf16 out")
    return out


def momuvik_rooflines(width: int, prompt: int, batch: int, context: int) -> list:
    """Momuvik's own kernels alone, at the sizes of momuvik_shape(width): time over roofline time, each
    beside the like kernel of the Mixtral-shaped model (its paged attention, its routed experts)."""
    from .. import ops
    from ..models.feedforward import RoutedExperts
    from ..models.mixers import rotary_frequencies
    from ..ops import moe as moe_ops
    from ..ops import seqmix
    dev = torch.device("cuda")
    dt = torch.bfloat16
    bs, out = 16, []
    i32 = dict(dtype=torch.int32, device=dev)
    rnd = lambda *sh: torch.randn(*sh, device=dev).to(dt)  # noqa: E731

    def entry(name, t, flops, peak, bytes_, note):
        roof = max(flops / peak, bytes_ / PEAK_HBM)
        out.append({"kernel": name, "width": width, "ms": round(1e3 * t, 4), "roofline_ms": round(1e3 * roof, 4),
                    "x_roofline": round(t / roof, 1), "counts": note})

    shape = momuvik_shape(width)["layers"][0]
    mc, mlp = shape["mixer"], shape["mlp"]
    H, rank, dr, qr = mc["heads"], mc["kv_rank"], mc["rot_dim"], mc["q_rank"]
    dk = rank + dr
    E, top, ff = MOE_EXPERTS, MOE_TOP, mlp["expert"]["ff"]
    for mode, T, S, ctx in (("prefill", prompt, 1, prompt), ("decode", batch, batch, context)):
        qsl = torch.arange(0, T + 1, T // S, **i32)
        seq = torch.full((S,), ctx, **i32)
        nb = -(-ctx // bs)
        bt = torch.arange(S * nb, **i32).view(S, nb)
        pos = torch.cat([torch.arange(ctx - T // S, ctx, device=dev) for _ in range(S)])
        slots = torch.cat([bt[s_].long().repeat_interleave(bs)[ctx - T // S:ctx] * bs + pos[:T // S] % bs for s_ in range(S)])
        keys = ctx if mode == "decode" else ctx / 2
        # latent attention: every head over the same rows [latent | rotated part]; values are the latent
        cache = rnd(S * nb, bs * dk)
        q = rnd(T, H * dk)
        sink = torch.zeros(H, device=dev)
        t = _time(lambda: seqmix.latent_attention(q, cache, bt, qsl, seq, 0, H, dk, rank, bs, 0.07, T // S, ctx, sink=sink), 5)
        entry(f"latent_attention/{mode}", t, 2.0 * T * H * keys * (dk + rank), PEAK_BF16,
              2.0 * (S * ctx * dk + T * H * (dk + rank)), f"{T} rows x {H} heads x ~{int(keys)} keys of {dk}+{rank}, bf16 MFMA peak")
        # the Mixtral-shaped model's attention: 128-wide heads, 4 query heads per kv head
        G = max(width // 512, 1)
        kv = rnd(S * nb, 1, 2, G, bs, 128)
        q3 = rnd(T, H, 128)
        if mode == "prefill":
            fn = lambda: ops.paged_attention_prefill(q3, kv[:, 0], bt, qsl, seq, 0.09, T)  # noqa: E731
        else:
            fn = lambda: ops.paged_attention_decode(q3, kv[:, 0], bt, seq, 0.09, ctx)  # noqa: E731
        t = _time(fn, 5)
        entry(f"paged_attention/{mode} (mixtral)", t, 2.0 * T * H * keys * 256, PEAK_BF16,
              2.0 * (S * ctx * G * 256 + 2 * T * H * 128), f"{T} rows x {H} heads x ~{int(keys)} keys of 128+128, bf16 MFMA peak")
        fr = rotary_frequencies(dr, 10000.0, None).to(dev)
        dqv, dkvv = rnd(T, qr), rnd(T, dk)
        qn, kn = torch.ones(qr, device=dev).to(dt), torch.ones(rank, device=dev).to(dt)
        t = _time(lambda: seqmix.latent_prep(dqv, dkvv, pos, slots, cache, 0, rank, bs, fr, qn, kn, 1e-5), 5)
        entry(f"latent_prep/{mode}", t, 0.0, PEAK_F32, 4.0 * T * (qr + dk), f"{T} rows: both latents read, normed / turned, written")
        qh = rnd(T, H * 192)
        t = _time(lambda: seqmix.rope_half_into(q, qh, pos, H, 192, 128, dk, rank, fr), 5)
        entry(f"rope_half_into/{mode}", t, 0.0, PEAK_F32, 4.0 * T * H * dr, f"{T} rows x {H} heads x {dr} turned entries")
        # routed experts: router, the two expert products with the capped activation, the sum
        f = RoutedExperts("f.", width, E, top, ff, 7.0)
        w = {"f.router": rnd(E, width), "f._gu": rnd(E, 2 * ff, width) * width ** -0.5, "f._down": rnd(E, width, ff) * ff ** -0.5}
        h = rnd(T, width)
        t = _time(lambda: f.forward(h, w), 5)
        act = min(E, T * top)
        entry(f"routed_experts/{mode}", t, 6.0 * T * top * width * ff, PEAK_BF16, 2.0 * (3 * act * width * ff + 2 * T * width),
              f"{T} rows x {top} of {E} experts of {ff}, bf16 MFMA peak; {act} experts' weights read once")
        w13 = rnd(E, 2 * ff, width) * width ** -0.5
        w2 = rnd(E, width, ff) * ff ** -0.5
        gate = rnd(E, width)

        def mixtral_moe():
            tw, ti = ops.moe_topk_softmax(ops.linear(h, gate), top)
            return moe_ops.fused_experts(h, w13, w2, tw, ti, 0)
        t = _time(mixtral_moe, 5)
        entry(f"routed_experts/{mode} (mixtral)", t, 6.0 * T * top * width * ff, PEAK_BF16,
              2.0 * (3 * act * width * ff + 2 * T * width), f"{T} rows x {top} of {E} experts of {ff}, bf16 MFMA peak")
        gu = rnd(T * top, 2 * ff)
        t = _time(lambda: seqmix.capped_glu(gu, 7.0), 5)
        entry(f"capped_glu/{mode}", t, 0.0, PEAK_F32, 6.0 * T * top * ff, f"{T * top} rows x {ff}: gate and up in, product out")
        t = _time(lambda: seqmix.silu_mul(gu), 5)
        entry(f"silu_mul/{mode} (tapasun)", t, 0.0, PEAK_F32, 6.0 * T * top * ff, f"{T * top} rows x {ff}: gate and up in, product out")
    return out


def seradra_rooflines(width: int, prompt: int, batch: int, context: int) -> list:
    """Seradra's own kernels alone, at the sizes of seradra_shape(width): time over roofline time, each beside
    the like kernel of an existing model: the windowed attention with a sink (Voletar's / Tapasun's kernel)
    for the head-mixing attention, Momuvik's unwindowed latent attention for the windowed one, the per-head
    q/k/v preparation for the whole-row one, Momuvik's routed experts for the softmax-routed ones, the gated
    activation and the fused residual kernel for the activation and the weighted sum over kept results."""
    from ..models.feedforward import RoutedExperts
    from ..models.mixers import rotary_frequencies
    from ..ops import seqmix
    dev = torch.device("cuda")
    dt = torch.bfloat16
    bs, out = 16, []
    i32 = dict(dtype=torch.int32, device=dev)
    rnd = lambda *sh: torch.randn(*sh, device=dev).to(dt)  # noqa: E731

    def entry(name, t, flops, peak, bytes_, note):
        roof = max(flops / peak, bytes_ / PEAK_HBM)
        out.append({"kernel": name, "width": width, "ms": round(1e3 * t, 4), "roofline_ms": round(1e3 * roof, 4),
                    "x_roofline": round(t / roof, 1), "counts": note})

    shape = seradra_shape(width)["layers"]
    ac, lc, mlp = shape[0]["mixer"], shape[1]["mixer"], shape[1]["mlp"]
    H, G, dk, dv, win = ac["heads"], ac["kv_heads"], ac["dim"], ac["vdim"], ac["mask"]["size"]
    rank, dr = lc["kv_rank"], lc["rot_dim"]
    ldk = rank + dr
    E, top, ff = MOE_EXPERTS, MOE_TOP, mlp["expert"]["ff"]
    for mode, T, S, ctx in (("prefill", prompt, 1, prompt), ("decode", batch, batch, context)):
        qsl = torch.arange(0, T + 1, T // S, **i32)
        seq = torch.full((S,), ctx, **i32)
        nb = -(-ctx // bs)
        bt = torch.arange(S * nb, **i32).view(S, nb)
        pos = torch.cat([torch.arange(ctx - T // S, ctx, device=dev) for _ in range(S)])
        slots = torch.cat([bt[s_].long().repeat_interleave(bs)[ctx - T // S:ctx] * bs + pos[:T // S] % bs for s_ in range(S)])
        keys = min(win, ctx) if mode == "decode" else min(win, ctx / 2)
        # head-mixing attention beside the windowed attention with a sink at the same head layout
        cache = rnd(S * nb, G * bs * (dk + dv))
        q, k, v = rnd(T, H * dk), rnd(T, G * dk), rnd(T, G * dv)
        sink = torch.zeros(H, device=dev)
        talk = torch.eye(H, device=dev) + 0.1 * torch.randn(H, H, device=dev)
        for name, tk, extra in (("talking_attention", talk, 2.0 * H), ("window_attention", None, 0.0)):
            t = _time(lambda: seqmix.window_attention(q, cache, bt, qsl, seq, 0, G * bs * dk, H, G, dk, dv, bs, 0.09, win, 0,
                                                      max_query_len=T // S, sink=sink, talk=tk, max_seq_len=ctx), 5)
            entry(f"{name}/{mode}" + ("" if tk is not None else " (voletar, tapasun)"), t, 2.0 * T * H * keys * (dk + dv), PEAK_BF16,
                  2.0 * (S * min(win, ctx) * G * (dk + dv) + 2 * T * H * dk),
                  f"{T} rows x {H} heads x ~{int(keys)} keys of {dk}+{dv}, bf16 MFMA peak" +
                  (f" (the mix adds {int(extra)} fp32 multiply-adds per score, not priced)" if extra else ""))
        fr = rotary_frequencies(64, 500000.0, ac["rot"]["scaling"]).to(dev)
        ones = lambda n: torch.ones(n, device=dev).to(dt)  # noqa: E731
        oq, ok_, ov, od, ow = ones(H * dk), ones(G * dk), ones(G * dv), ones(dk), ones(width)
        t = _time(lambda: seqmix.rope_qkv_cache(q, k, v, pos, slots, cache, 0, G * bs * dk, H, G, dk, dv, bs, fr, oq, ok_, 1e-5,
                                                bias_q=oq, bias_k=ok_, bias_v=ov, norm_whole=True, split_pairs=True, mag=1.2), 5)
        pbytes = 2.0 * T * (2 * H * dk + 2 * G * (dk + dv))
        entry(f"qkv_prep_cache/{mode}", t, 0.0, PEAK_F32, pbytes, f"{T} rows: q read and written, k and v read and written to the pages")
        fr2 = rotary_frequencies(64, 500000.0, None).to(dev)
        t = _time(lambda: seqmix.rope_qkv_cache(q, k, v, pos, slots, cache, 0, G * bs * dk, H, G, dk, dv, bs, fr2, od, od, 1e-5, None), 5)
        entry(f"rope_qkv_cache/{mode} (tapasun)", t, 0.0, PEAK_F32, pbytes, f"{T} rows: q read and written, k and v read and written to the pages")
        # latent attention inside the window beside the unwindowed one over the whole context
        lcache = rnd(S * nb, bs * ldk)
        lq = rnd(T, H * ldk)
        for name, w_, kk in (("latent_attention(window)", win, keys), ("latent_attention", 0, ctx if mode == "decode" else ctx / 2)):
            t = _time(lambda: seqmix.latent_attention(lq, lcache, bt, qsl, seq, 0, H, ldk, rank, bs, 0.07, T // S, ctx,
                                                      sink=None if w_ else sink, window=w_), 5)
            entry(f"{name}/{mode}" + ("" if w_ else " (momuvik)"), t, 2.0 * T * H * kk * (ldk + rank), PEAK_BF16,
                  2.0 * (S * (min(win, ctx) if w_ else ctx) * ldk + T * H * (ldk + rank)),
                  f"{T} rows x {H} heads x ~{int(kk)} keys of {ldk}+{rank}, bf16 MFMA peak")
        # routed experts: softmax scores on the outputs of plain SiLU units beside sigmoid scores on the inputs of capped ones
        h = rnd(T, width)
        w = {"f.router": rnd(E, width), "f._gu": rnd(E, 2 * ff, width) * width ** -0.5, "f._down": rnd(E, width, ff) * ff ** -0.5}
        act = min(E, T * top)
        for name, f in (("routed_experts", RoutedExperts("f.", width, E, top, ff, None, score="softmax", weigh="output")),
                        ("routed_experts (momuvik)", RoutedExperts("f.", width, E, top, ff, 7.0))):
            t = _time(lambda: f.forward(h, w), 5)
            nm = name.split(" ")
            entry(f"{nm[0]}/{mode}" + (" " + nm[1] if len(nm) > 1 else ""), t, 6.0 * T * top * width * ff, PEAK_BF16,
                  2.0 * (3 * act * width * ff + 2 * T * width),
                  f"{T} rows x {top} of {E} experts of {ff}, bf16 MFMA peak; {act} experts' weights read once")
        # the ungated activation beside the gated one; the weighted sum over five kept results beside one
        # pass of the fused residual kernel
        z = rnd(T, 4 * width)
        ab = torch.tensor([0.7, 1.2], device=dev)
        t = _time(lambda: seqmix.xielu(z, ab), 5)
        entry(f"xielu/{mode}", t, 0.0, PEAK_F32, 4.0 * T * 4 * width, f"{T} rows x {4 * width}: in and out")
        t = _time(lambda: seqmix.silu_mul(z), 5)
        entry(f"silu_mul/{mode} (tapasun)", t, 0.0, PEAK_F32, 3.0 * T * 4 * width, f"{T} rows x {2 * width}: gate and up in, product out")
        hist = torch.randn(6, T, width, device=dev)
        cf = torch.randn(5, device=dev)
        t = _time(lambda: seqmix.depth_mix(hist, 5, cf, cast_dtype=dt), 5)
        entry(f"depth_mix/{mode}", t, 0.0, PEAK_F32, T * width * (5 * 4.0 + 4.0 + 2.0), f"{T} rows x {width}: five fp32 slabs in, one out, one bf16 copy")
        x = torch.randn(T, width, device=dev)
        a = rnd(T, width)
        t = _time(lambda: seqmix.resid_update(x, a, 1e-5, wa=ow, wa_offset=1.0, cast_dtype=dt), 5)
        entry(f"resid_update/{mode}", t, 0.0, PEAK_F32, T * width * (4.0 + 2.0 + 4.0 + 2.0), f"{T} rows x {width}: stream in and out, branch in, bf16 copy out")
        t = _time(lambda: seqmix.resid_update(x, a, 1e-5, norm_w=ow, out_dtype=dt, w_offset=1.0), 5)
        entry(f"resid_update/{mode} (momuvik)", t, 0.0, PEAK_F32, T * width * (4.0 + 2.0 + 4.0 + 2.0), f"{T} rows x {width}: stream in and out, branch in, normed bf16 out")
    return out


def main(sizes: list, prompt: int, batch: int, context: int, layers: int = 4, only: str = "all",
         design: str = "voletar") -> int:
    """only: all | seradra | momuvik | mixtral | tapasun | voletar | llama | kernels (e.g. one model alone under a profiler)."""
    from .. import ops
    ops.ext()
    for width in sizes:
        names = register(width, layers, design)
        for name in names:
            if only in ("all", name.split("-")[0]):
                print(json.dumps(run_model(name, prompt, batch, context)), flush=True)
        if only in ("all", "kernels"):
            if design == "seradra":
                rows = seradra_rooflines(width, prompt, batch, context)
            elif design == "momuvik":
                rows = momuvik_rooflines(width, prompt, batch, context)
            else:
                rows = (tapasun_rooflines(width, prompt, batch, context) if design == "tapasun" else []) + \
                    kernel_rooflines(width, prompt, batch, context)
            for e in rows:
                print(json.dumps(e), flush=True)
    return 0
