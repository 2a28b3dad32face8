"""Throughput of a hybrid design (Zokunex, Kalesun, Tugovik, Vogerax) beside the framework's other models at equal width and depth:
whole-model prefill and decode steps, and each of the design's kernels beside its closest existing kernel with the
fraction of its roofline it reaches.

``python bench.py --design-compare [--design zokunex|kalesun|tugovik|vogerax] [--design-sizes 1k,2k,4k]`` prints one JSON line
(the default benchmark and its output line are untouched).  Zokunex stands beside Llama; Kalesun beside Zokunex (the
closest family: recurrent layers, attention and mixtures of experts on a float32 stream) and Llama; Tugovik beside
Kalesun (masked grouped-query attention over paged keys and values, linear-state scans behind a short convolution,
gated experts, RMS norms on the stream) and Llama; Vogerax beside Kalesun too (windowed and causal sink attention on
the same kernels, a linear-state scan, RMS norms joined to a float32 stream) and Llama.  Weights are random; every number is measured on the GPU this
process runs on.

Rooflines: HBM 8 TB/s for kernels bound by the bytes they must move, 2.5 PFLOP/s dense bf16 for the matrix-shaped
ones (the attention kernels over a long context are priced by their FLOPs in prefill and by their cache bytes in
decode, like the Llama kernels they stand beside).
"""
from __future__ import annotations

import json
import math
import sys
import time

import torch

HBM_BPS = 8.0e12
BF16_FLOPS = 2.5e15

# width -> (mlstm heads, dim, vdim | latent heads, dim, rot, vdim, rank | dense ff | experts, identity, top, expert ff)
SIZES = {
    "1k": dict(width=1024, m=(4, 128, 256), a=(8, 64, 32, 64, 256), ff=4096, moe=(8, 2, 2, 512)),
    "2k": dict(width=2048, m=(4, 256, 512), a=(16, 128, 64, 128, 512), ff=8192, moe=(16, 2, 4, 1408)),
    "4k": dict(width=4096, m=(8, 256, 512), a=(32, 128, 64, 128, 512), ff=14336, moe=(32, 2, 4, 2048)),
}
LAYERS = 4
VOCAB = 32768


def zokunex_config(size: dict) -> dict:
    mh, md, mv = size["m"]
    ah, ad, ar, av, rank = size["a"]
    ne, ni, top, eff = size["moe"]
    mix_m = dict(type="mlstm", mixer=dict(heads=mh, dim=md, vdim=mv, gate_cap=10.0))
    mix_a = dict(type="latent_attention", mixer=dict(heads=ah, dim=ad, rot_dim=ar, vdim=av, kv_rank=rank,
                                                     scale=(ad + ar) ** -0.5, rot=dict(base=10000.0, dims=ar)))
    dense = dict(kind="dense", ff=size["ff"])
    moe = dict(kind="moe", expert=dict(ff=eff), router=dict(experts=ne, identity=ni, top=top))
    layers = [dict(mix_m, mlp=dense), dict(mix_a, mlp=moe), dict(mix_m, mlp=moe), dict(mix_a, mlp=dense)][:LAYERS]
    return dict(architecture="Zokunex", vocab=VOCAB, width=size["width"], logit_scale=1.0, norm=dict(eps=1e-5),
                layers=layers)


# Kalesun: width -> (attention heads, kv heads, dim, vdim, window, kept | delta heads, qk heads, dim, vdim |
#                    gla heads, dim, vdim | dense ff | experts, top, expert ff)
KALESUN_SIZES = {
    "1k": dict(width=1024, a=(8, 2, 128, 128, 512, 4), d=(8, 4, 128, 128), g=(4, 128, 256), ff=2816, moe=(8, 2, 512)),
    "2k": dict(width=2048, a=(16, 4, 128, 128, 1024, 4), d=(16, 8, 128, 128), g=(8, 128, 256), ff=5632, moe=(16, 4, 1024)),
    "4k": dict(width=4096, a=(32, 8, 128, 128, 1024, 4), d=(32, 16, 128, 128), g=(16, 128, 256), ff=11008, moe=(32, 4, 1536)),
}


def kalesun_config(size: dict) -> dict:
    ah, ag, ad, av, win, keep = size["a"]
    dh, dk, dd, dv = size["d"]
    gh, gd, gv = size["g"]
    ne, top, eff = size["moe"]
    mix_a = dict(type="attention", mixer=dict(heads=ah, kv_heads=ag, dim=ad, vdim=av, scale=ad ** -0.5, v_mix=True,
                                              mask=dict(size=win, keep_first=keep),
                                              rot=dict(base=500000.0, dims=ad // 2,
                                                       scaling=dict(factor=8.0, low=1.0, high=4.0, original=8192))))
    mix_d = dict(type="delta", mixer=dict(heads=dh, kv_heads=dk, dim=dd, vdim=dv, conv=4))
    mix_g = dict(type="gla", mixer=dict(heads=gh, dim=gd, vdim=gv, tau=16.0, rank=16))
    dense = dict(kind="dense", ff=size["ff"], limit=7.0)
    moe = dict(kind="moe", expert=dict(ff=eff, limit=7.0), router=dict(experts=ne, top=top))
    layers = [dict(mix_d, mlp=dense), dict(mix_a, mlp=moe), dict(mix_g, mlp=moe), dict(mix_a, mlp=dense)][:LAYERS]
    return dict(architecture="Kalesun", vocab=VOCAB, width=size["width"], postln_alpha=2.0, norm=dict(eps=1e-6),
                layers=layers)

# Tugovik: width -> (attention heads, kv heads, dim, vdim, chunk | state-space heads, vdim, state, groups |
#                    recurrence width, blocks | experts, top, groups, kept, expert ff, shared ff | token-input columns)
TUGOVIK_SIZES = {
    "1k": dict(width=1024, a=(8, 2, 128, 128, 512), m=(32, 64, 128, 4), r=(1024, 4), moe=(8, 2, 4, 2, 512, 1024), side=128),
    "2k": dict(width=2048, a=(16, 4, 128, 128, 1024), m=(64, 64, 128, 8), r=(2048, 8), moe=(16, 4, 4, 2, 1024, 2048), side=256),
    "4k": dict(width=4096, a=(32, 8, 128, 128, 1024), m=(128, 64, 128, 8), r=(4096, 16), moe=(32, 4, 8, 4, 1536, 4096), side=256),
}


def tugovik_config(size: dict) -> dict:
    ah, ag, ad, av, chunk = size["a"]
    mh, mv, mn, mg = size["m"]
    rw, rb = size["r"]
    ne, top, ng, keep, eff, sff = size["moe"]
    mix_a = dict(type="attention", mixer=dict(heads=ah, kv_heads=ag, dim=ad, vdim=av, scale=ad ** -0.5, mask=dict(size=chunk)))
    mix_m = dict(type="mamba2", mixer=dict(heads=mh, vdim=mv, state=mn, groups=mg, conv=4, norm_groups=mg))
    mix_r = dict(type="rglru", mixer=dict(width=rw, blocks=rb, conv=4))
    moe = dict(kind="moe", expert=dict(ff=eff), shared=dict(ff=sff),
               router=dict(experts=ne, top=top, scale=2.5, groups=dict(count=ng, keep=keep)))
    layers = [dict(mix_m, mlp=moe), dict(mix_a, mlp=moe), dict(mix_r, mlp=moe), dict(mix_a, mlp=moe)][:LAYERS]
    return dict(architecture="Tugovik", vocab=VOCAB, width=size["width"], norm=dict(eps=1e-6), layers=layers,
                token_side=dict(dim=size["side"]))

# Vogerax: width -> (pooled attention heads, kv heads, dim, window, pool | sink attention heads, kv heads, dim, vdim |
#                    retention heads, dim, vdim | dense ff | experts, top, expert ff, shared ff | norm groups)
VOGERAX_SIZES = {
    "1k": dict(width=1024, a=(8, 2, 128, 512, 64), l=(8, 2, 128, 128), r=(8, 128, 128), ff=4096, moe=(8, 2, 512, 1024), groups=4),
    "2k": dict(width=2048, a=(16, 4, 128, 1024, 64), l=(16, 4, 128, 128), r=(16, 128, 128), ff=8192, moe=(16, 4, 1024, 2048), groups=4),
    "4k": dict(width=4096, a=(32, 8, 128, 1024, 64), l=(32, 8, 128, 128), r=(32, 128, 128), ff=14336, moe=(32, 4, 1536, 4096), groups=4),
}


def vogerax_config(size: dict) -> dict:
    ah, ag, ad, win, pool = size["a"]
    lh, lg, ld, lv = size["l"]
    rh, rd, rv = size["r"]
    ne, top, eff, sff = size["moe"]
    mix_a = dict(type="attention", mixer=dict(heads=ah, kv_heads=ag, dim=ad, vdim=ad, scale=ad ** -0.5,
                                              mask=dict(size=win, pool=pool),
                                              rot=dict(base=5e5, dims=ad // 2, scaling=dict(factor=4.0))))
    left = dict(heads=lh, kv_heads=lg, dim=ld, vdim=lv, scale=ld ** -0.5,
                rot=dict(base=1e5, dims=ld // 2, scaling=dict(factor=8.0, original=4096, fast=16.0, slow=2.0)))
    right = dict(heads=rh, dim=rd, vdim=rv, rot=dict(base=1e4, dims=rd),
                 decay=[math.exp(-1.0 / (16.0 * 128.0 ** (h / max(1, rh - 1)))) for h in range(rh)])
    mix_p = dict(type="parallel", mixer=dict(left=left, right=right))
    dense = dict(kind="dense", ff=size["ff"])
    moe = dict(kind="moe", expert=dict(ff=eff), shared=dict(ff=sff), router=dict(experts=ne, top=top))
    layers = [dict(mix_a, mlp=dense), dict(mix_p, mlp=moe), dict(mix_a, mlp=moe), dict(mix_p, mlp=dense)][:LAYERS]
    return dict(architecture="Vogerax", vocab=VOCAB, width=size["width"], norm=dict(eps=1e-6, groups=size["groups"]),
                embedding=dict(scale=8.0), layers=layers)


def _say(msg: str) -> None:
    print(f"[design-compare] {time.strftime('%H:%M:%S')} {msg}", file=sys.stderr, flush=True)


def _time(fn, iters: int = 10, warm: int = 2) -> float:
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(iters):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / iters * 1e-3


def _graph(fn):
    fn()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        fn()
    return g.replay


def _model_steps(model, dev, seqs: int, plen: int, rows: int, ctx: int) -> dict:
    """Prefill of ``seqs`` prompts of ``plen`` tokens in one step; then decode steps of ``rows`` rows at context
    ``ctx`` (captured into a graph, as the engine runs them)."""
    from chronos.models.llama import StepBatch

    bs = 16
    need = max(seqs * plen, rows * (ctx + 1))
    nb = need // bs + rows + seqs + 2
    cache = model.make_cache(nb, bs, max(rows, seqs))
    vocab = model.cfg.vocab_size
    g = torch.Generator().manual_seed(0)
    per = (plen + bs - 1) // bs
    chunks = [torch.randint(0, vocab, (plen,), generator=g).tolist() for _ in range(seqs)]
    bts = [list(range(1 + b * per, 1 + (b + 1) * per)) for b in range(seqs)]
    sb = model.prefill_batch(chunks, [0] * seqs, bts, list(range(seqs)), max_blocks=per, nqt=8)
    t_pre = _time(lambda: model.forward(sb, cache), iters=3, warm=1)
    per = (ctx + 1 + bs - 1) // bs
    i32 = dict(dtype=torch.int32, device=dev)
    bt = torch.arange(1, 1 + rows * per, **i32).view(rows, per)
    ar = torch.arange(rows + 1, **i32)
    from chronos import ops

    dsb = StepBatch(torch.randint(0, vocab, (rows,), generator=g).to(dev).int(), torch.full((rows,), ctx, **i32),
                    ar[:rows], bt, ar, torch.full((rows,), ctx + 1, **i32), torch.arange(rows, device=dev), None, rows, 1,
                    ops.pick_nsplit(rows * model.hkv, ctx + 1), slots=ar[:rows].clone(), max_q=1)
    t_dec = _time(_graph(lambda: model.forward(dsb, cache)), iters=20)
    return dict(prefill_tokens_s=seqs * plen / t_pre, prefill_ms=t_pre * 1e3, decode_tokens_s=rows / t_dec,
                decode_ms=t_dec * 1e3)


def _kernels(size: dict, dev, T: int, ctx: int, rows: int) -> dict:
    """Each new kernel and its Llama counterpart at this size: seconds, and the fraction of the roofline reached."""
    from chronos import ops
    from chronos.models.hybrid import rope_cos_sin
    from chronos.ops import hybrid as hops

    out = {}
    bf = torch.bfloat16
    d = size["width"]
    g = torch.Generator(device=dev).manual_seed(1)
    rnd = lambda *s, dt=bf, sc=1.0: (torch.randn(*s, device=dev, generator=g) * sc).to(dt)  # noqa: E731
    i32 = dict(dtype=torch.int32, device=dev)

    def rec(name, secs, nbytes=0.0, flops=0.0):
        roof = max(nbytes / HBM_BPS, flops / BF16_FLOPS)
        _say(f"  {name}: {secs * 1e6:.1f} us, roofline {roof * 1e6:.2f} us")
        out[name] = dict(us=round(secs * 1e6, 1), roofline_us=round(roof * 1e6, 2), of_roofline=round(roof / secs, 4))

    # ---- norms on the residual stream
    y, x32, w32 = rnd(T, d), rnd(T, d, dt=torch.float32), rnd(d, dt=torch.float32)
    rec("add_layer_norm", _time(lambda: hops.add_layer_norm(y, x32, w32, 1e-5, bf)), T * d * (2 + 4 + 4 + 2))
    xb, wb = rnd(T, d), rnd(d)
    rec("llama.add_rmsnorm", _time(lambda: ops.add_rmsnorm(y, xb, wb, 1e-5)), T * d * (2 + 2 + 2 + 2))
    # ---- attention: prefill of T tokens (seqs of `ctx`), decode of `rows` rows at context ctx
    H, D, R, Dv, rank = size["a"]
    DK, bs = rank + R, 16
    seqs = max(1, T // ctx)
    per = ctx // bs + 1
    nb = max(seqs, rows) * per + 1
    cache = rnd(nb, bs, DK, sc=0.3)
    qa = rnd(seqs * ctx, H, DK, sc=0.3)
    gate = rnd(seqs * ctx, H, dt=torch.float32)
    bt = torch.arange(1, 1 + seqs * per, **i32).view(seqs, per)
    qs = torch.arange(0, (seqs + 1) * ctx, ctx, **i32)
    pos = torch.arange(ctx, **i32).repeat(seqs)
    pairs = seqs * ctx * (ctx + 1) / 2
    rec("latent_attention.prefill", _time(lambda: hops.latent_attention(qa, cache, bt, qs, pos, gate, 0.1, rank, bf, ctx), iters=3, warm=1),
        flops=2.0 * pairs * H * (DK + rank))
    btd = torch.arange(1, 1 + rows * per, **i32).view(rows, per)
    qsd = torch.arange(rows + 1, **i32)
    posd = torch.full((rows,), ctx, **i32)
    qad, gated = rnd(rows, H, DK, sc=0.3), rnd(rows, H, dt=torch.float32)
    rec("latent_attention.decode", _time(lambda: hops.latent_attention(qad, cache, btd, qsd, posd, gated, 0.1, rank, bf, 1)),
        nbytes=rows * (ctx + 1) * DK * 2.0)
    hq = d // 128
    hkv = max(1, hq // 4)
    kc, vc = rnd(nb, hkv, bs, 128, sc=0.3), rnd(nb, hkv, 128, bs, sc=0.3)
    q = rnd(seqs * ctx, hq, 128, sc=0.3)
    ctxl = torch.full((seqs,), ctx, **i32)
    tiles = torch.tensor(ops.attention_tiles([ctx] * seqs, hq, hkv, 8), **i32).view(-1, 2)
    rec("llama.attention.prefill", _time(lambda: ops.paged_attention(q, kc, vc, bt, qs, ctxl, tiles, tiles.shape[0], 8, 1), iters=3, warm=1),
        flops=4.0 * pairs * hq * 128)
    qd = rnd(rows, hq, 128, sc=0.3)
    ctxd = torch.full((rows,), ctx + 1, **i32)
    ns = ops.pick_nsplit(rows * hkv, ctx + 1)
    rec("llama.attention.decode", _time(lambda: ops.paged_attention(qd, kc, vc, btd, qsd, ctxd, None, rows, 1, ns)),
        nbytes=rows * (ctx + 1) * hkv * 128 * 2 * 2.0)
    # ---- the recurrence: prefill (FLOPs of the state update and read-out), decode (state bytes in and out)
    mh, md, mv = size["m"]
    C = 2 * mh * md + 2 * mh * mv
    proj = rnd(seqs * ctx, C, sc=0.5)
    gp = rnd(seqs * ctx, 2 * mh, dt=torch.float32)
    NS = max(seqs, rows) + 1
    S, n, m = (torch.zeros(NS, mh, md, mv, device=dev), torch.zeros(NS, mh, md, device=dev), torch.zeros(NS, mh, device=dev))
    p0 = torch.zeros(seqs, **i32)
    sl = torch.arange(seqs, **i32)
    rec("mlstm_scan.prefill", _time(lambda: hops.mlstm_scan(proj, gp, qs, p0, sl, S, n, m, mh, md, mv, 10.0, ctx), iters=3, warm=1),
        nbytes=seqs * ctx * C * 2.0, flops=seqs * ctx * mh * md * mv * 6.0)
    projd, gpd = rnd(rows, C, sc=0.5), rnd(rows, 2 * mh, dt=torch.float32)
    sld = torch.arange(rows, **i32)
    rec("mlstm_scan.decode", _time(lambda: hops.mlstm_scan(projd, gpd, qsd, posd, sld, S, n, m, mh, md, mv, 10.0, 1)),
        nbytes=rows * mh * md * mv * 4 * 2.0)
    # ---- feed-forwards: the mixture of experts beside a dense SwiGLU of the Llama model at this width
    ne, ni, top, eff = size["moe"]
    wr, corr = rnd(ne + ni, d, sc=0.05), rnd(ne + ni, dt=torch.float32, sc=0.01)
    wu, wd = rnd(ne, eff, d, sc=d ** -0.5), rnd(ne, d, eff, sc=eff ** -0.5)
    for name, tk in (("prefill", T), ("decode", rows)):
        h = rnd(tk, d)
        idx, wt = hops.moe_route(h, wr, corr, top)
        rec(f"moe_route.{name}", _time(lambda: hops.moe_route(h, wr, corr, top)), nbytes=tk * d * 2.0 + (ne + ni) * d * 2.0)
        real = float((idx < ne).sum())
        used = min(ne, real) * 2 * eff * d * 2.0
        rec(f"moe_ffn.{name}", _time(lambda: hops.moe_ffn(h, idx, wt, wu, wd, 1, bf), iters=3, warm=1),
            nbytes=used + tk * d * 4.0, flops=real * 4.0 * eff * d)
        f = int(3.5 * d)
        wgu, wdn = rnd(2 * f, d, sc=d ** -0.5), rnd(d, f, sc=f ** -0.5)
        rec(f"llama.mlp.{name}", _time(lambda: ops.linear(ops.gate_up_silu(h, wgu), wdn), iters=3, warm=1),
            nbytes=3 * f * d * 2.0 + tk * d * 4.0, flops=tk * 6.0 * f * d)
    return out


def _kernels_kalesun(size: dict, zsize: dict, dev, T: int, ctx: int, rows: int) -> dict:
    """Kalesun's kernels and their closest existing kernels at this size: seconds, and the fraction of the roofline
    reached.  ``zsize``: the Zokunex sizes of the same width (for the kernels it stands beside)."""
    from chronos import ops
    from chronos.models.hybrid import rope_cos_sin
    from chronos.ops import hybrid as hops

    out = {}
    bf = torch.bfloat16
    d = size["width"]
    g = torch.Generator(device=dev).manual_seed(1)
    rnd = lambda *s, dt=bf, sc=1.0: (torch.randn(*s, device=dev, generator=g) * sc).to(dt)  # noqa: E731
    i32 = dict(dtype=torch.int32, device=dev)

    def rec(name, secs, nbytes=0.0, flops=0.0):
        roof = max(nbytes / HBM_BPS, flops / BF16_FLOPS)
        _say(f"  {name}: {secs * 1e6:.1f} us, roofline {roof * 1e6:.2f} us")
        out[name] = dict(us=round(secs * 1e6, 1), roofline_us=round(roof * 1e6, 2), of_roofline=round(roof / secs, 4))

    # ---- norms on the residual stream
    y, x32, w32 = rnd(T, d), rnd(T, d, dt=torch.float32), rnd(d, dt=torch.float32)
    rec("scale_add_rms_norm", _time(lambda: hops.scale_add_rms_norm(y, x32, w32, 2.0, 1e-6, bf)), T * d * (2 + 4 + 4 + 2))
    rec("zokunex.add_layer_norm", _time(lambda: hops.add_layer_norm(y, x32, w32, 1e-5, bf)), T * d * (2 + 4 + 4 + 2))
    xb, wb = rnd(T, d), rnd(d)
    rec("llama.add_rmsnorm", _time(lambda: ops.add_rmsnorm(y, xb, wb, 1e-5)), T * d * (2 + 2 + 2 + 2))
    # ---- attention: prefill of T tokens (seqs of `ctx`), decode of `rows` rows at context ctx
    H, G, D, Dv, win, keep = size["a"]
    bs = 16
    seqs = max(1, T // ctx)
    per = ctx // bs + 1
    nb = max(seqs, rows) * per + 1
    kc, vc = rnd(nb, bs, G, D, sc=0.3), rnd(nb, bs, G, Dv, sc=0.3)
    C = (H + G) * D + G * Dv
    qkv = rnd(seqs * ctx, C, sc=0.3)
    gate, sink = rnd(seqs * ctx, H, dt=torch.float32), rnd(H, dt=torch.float32)
    bt = torch.arange(1, 1 + seqs * per, **i32).view(seqs, per)
    qs = torch.arange(0, (seqs + 1) * ctx, ctx, **i32)
    pos = torch.arange(ctx, **i32).repeat(seqs)
    tseq = torch.arange(seqs, **i32).repeat_interleave(ctx)
    vis = sum(min(i + 1, win) + max(0, min(keep, i + 1 - win)) for i in range(ctx))  # visible (query, key) pairs
    pairs = seqs * vis
    rec("window_attention.prefill", _time(lambda: hops.window_attention(qkv, kc, vc, bt, qs, pos, sink, gate, D ** -0.5, win, keep, H, bf, ctx), iters=3, warm=1),
        flops=2.0 * pairs * H * (D + Dv))
    cs = rope_cos_sin(500000.0, D // 2, ctx + 1, dev, (8.0, 1.0, 4.0, 8192.0))
    qn, vf, lam = rnd(D, dt=torch.float32), rnd(seqs * ctx, G * Dv), torch.tensor([0.3], device=dev)
    rec("window_prep.prefill", _time(lambda: hops.window_prep(qkv, H, G, D, Dv, vf, lam, pos, tseq, bt, qn, qn, 1e-6, cs, D // 2, kc, vc, False)),
        nbytes=seqs * ctx * (C * 2 + H * D * 2 + 2 * G * (D + Dv) * 2.0))
    btd = torch.arange(1, 1 + rows * per, **i32).view(rows, per)
    qsd = torch.arange(rows + 1, **i32)
    posd = torch.full((rows,), ctx, **i32)
    qkvd, gated = rnd(rows, C, sc=0.3), rnd(rows, H, dt=torch.float32)
    rec("window_attention.decode", _time(lambda: hops.window_attention(qkvd, kc, vc, btd, qsd, posd, sink, gated, D ** -0.5, win, keep, H, bf, 1)),
        nbytes=rows * (min(ctx + 1, win) + keep) * G * (D + Dv) * 2.0)
    # beside: Llama's paged GQA attention (full causal) and Zokunex's latent attention at this width
    hq = d // 128
    hkv = max(1, hq // 4)
    lkc, lvc = rnd(nb, hkv, bs, 128, sc=0.3), rnd(nb, hkv, 128, bs, sc=0.3)
    q = rnd(seqs * ctx, hq, 128, sc=0.3)
    ctxl = torch.full((seqs,), ctx, **i32)
    tiles = torch.tensor(ops.attention_tiles([ctx] * seqs, hq, hkv, 8), **i32).view(-1, 2)
    full_pairs = seqs * ctx * (ctx + 1) / 2
    rec("llama.attention.prefill", _time(lambda: ops.paged_attention(q, lkc, lvc, bt, qs, ctxl, tiles, tiles.shape[0], 8, 1), iters=3, warm=1),
        flops=4.0 * full_pairs * hq * 128)
    qd = rnd(rows, hq, 128, sc=0.3)
    ctxd = torch.full((rows,), ctx + 1, **i32)
    ns = ops.pick_nsplit(rows * hkv, ctx + 1)
    rec("llama.attention.decode", _time(lambda: ops.paged_attention(qd, lkc, lvc, btd, qsd, ctxd, None, rows, 1, ns)),
        nbytes=rows * (ctx + 1) * hkv * 128 * 2 * 2.0)
    zh, zd, zr, zv, rank = zsize["a"]
    DK = rank + zr
    lat = rnd(nb, bs, DK, sc=0.3)
    qa, zg = rnd(seqs * ctx, zh, DK, sc=0.3), rnd(seqs * ctx, zh, dt=torch.float32)
    rec("zokunex.latent_attention.prefill", _time(lambda: hops.latent_attention(qa, lat, bt, qs, pos, zg, 0.1, rank, bf, ctx), iters=3, warm=1),
        flops=2.0 * full_pairs * zh * (DK + rank))
    qad, zgd = rnd(rows, zh, DK, sc=0.3), rnd(rows, zh, dt=torch.float32)
    rec("zokunex.latent_attention.decode", _time(lambda: hops.latent_attention(qad, lat, btd, qsd, posd, zgd, 0.1, rank, bf, 1)),
        nbytes=rows * (ctx + 1) * DK * 2.0)
    # ---- the recurrences: prefill (FLOPs of the state update and read-out), decode (state bytes in and out)
    NS = max(seqs, rows) + 1
    p0, sl, sld = torch.zeros(seqs, **i32), torch.arange(seqs, **i32), torch.arange(rows, **i32)
    for name, (hh, hk, dd, dv), delta in (("delta", size["d"], True), ("gla", (size["g"][0], size["g"][0], *size["g"][1:]), False)):
        Cq = 2 * hk * dd + hh * dv
        S = torch.zeros(NS, hh, dd, dv, device=dev)

        def scan(proj, qs_, p0_, sl_, n):
            if delta:
                qsc, ksc = torch.rand(n, hk, device=dev), torch.rand(n, hk, device=dev)
                dec, beta = torch.rand(n, hh, device=dev), torch.rand(n, hh, device=dev)
                return lambda: hops.linear_scan(proj, 0, hk * dd, 2 * hk * dd, qsc, ksc, 1.0, dec, beta, qs_, p0_, sl_, S, hk, hh, dd, dv)
            dec = torch.rand(n, hh, dd, device=dev)
            return lambda: hops.linear_scan(proj, 0, hk * dd, 2 * hk * dd, None, None, dd ** -0.5, dec, None, qs_, p0_, sl_, S, hk, hh, dd, dv)

        proj = rnd(seqs * ctx, Cq, sc=0.5)
        rec(f"linear_scan.{name}.prefill", _time(scan(proj, qs, p0, sl, seqs * ctx), iters=3, warm=1),
            nbytes=seqs * ctx * Cq * 2.0, flops=seqs * ctx * hh * dd * dv * (6.0 if delta else 4.0))
        projd = rnd(rows, Cq, sc=0.5)
        rec(f"linear_scan.{name}.decode", _time(scan(projd, qsd, posd, sld, rows)), nbytes=rows * hh * dd * dv * 4 * 2.0)
    dh, dk, dd, dv = size["d"]
    Cc = 2 * dk * dd + dh * dv
    xc, taps = rnd(seqs * ctx, Cc + dh * dv), rnd(Cc, 4, dt=torch.float32)
    hist = torch.zeros(NS, 3, Cc, device=dev, dtype=bf)
    rec("short_conv.prefill", _time(lambda: hops.short_conv(xc, taps, tseq, qs, p0, sl, hist, True)), nbytes=seqs * ctx * Cc * 4.0)
    mh, md, mv = zsize["m"]
    Cm = 2 * mh * md + 2 * mh * mv
    mproj, gp = rnd(seqs * ctx, Cm, sc=0.5), rnd(seqs * ctx, 2 * mh, dt=torch.float32)
    mS, mn, mm = (torch.zeros(NS, mh, md, mv, device=dev), torch.zeros(NS, mh, md, device=dev), torch.zeros(NS, mh, device=dev))
    rec("zokunex.mlstm_scan.prefill", _time(lambda: hops.mlstm_scan(mproj, gp, qs, p0, sl, mS, mn, mm, mh, md, mv, 10.0, ctx), iters=3, warm=1),
        nbytes=seqs * ctx * Cm * 2.0, flops=seqs * ctx * mh * md * mv * 6.0)
    mprojd, gpd = rnd(rows, Cm, sc=0.5), rnd(rows, 2 * mh, dt=torch.float32)
    rec("zokunex.mlstm_scan.decode", _time(lambda: hops.mlstm_scan(mprojd, gpd, qsd, posd, sld, mS, mn, mm, mh, md, mv, 10.0, 1)),
        nbytes=rows * mh * md * mv * 4 * 2.0)
    # ---- feed-forwards: gated experts beside Zokunex's experts and Llama's dense SwiGLU; the gated unit's activation
    ne, top, eff = size["moe"]
    wr, br = rnd(ne, d, sc=0.05), rnd(ne, dt=torch.float32, sc=0.01)
    wgu = rnd(ne, 2 * eff, d, sc=d ** -0.5)[:, hops.moe_glu_row_order(eff).to(dev)].contiguous()
    wd = rnd(ne, d, eff, sc=eff ** -0.5)
    ze, zi, ztop, zeff = zsize["moe"]
    zwr, zcorr = rnd(ze + zi, d, sc=0.05), rnd(ze + zi, dt=torch.float32, sc=0.01)
    zwu, zwd = rnd(ze, zeff, d, sc=d ** -0.5), rnd(ze, d, zeff, sc=zeff ** -0.5)
    for name, tk in (("prefill", T), ("decode", rows)):
        h = rnd(tk, d)
        idx, wt = hops.moe_route_topk(h, wr, br, top)
        rec(f"moe_route_topk.{name}", _time(lambda: hops.moe_route_topk(h, wr, br, top)), nbytes=tk * d * 2.0 + ne * d * 2.0)
        used = min(ne, tk * top) * 3 * eff * d * 2.0
        rec(f"moe_glu_ffn.{name}", _time(lambda: hops.moe_glu_ffn(h, idx, wt, wgu, wd, 7.0, 1.702, 1.0, bf, True), iters=3, warm=1),
            nbytes=used + tk * d * 4.0, flops=tk * top * 6.0 * eff * d)
        zidx, zwt = hops.moe_route(h, zwr, zcorr, ztop)
        real = float((zidx < ze).sum())
        rec(f"zokunex.moe_ffn.{name}", _time(lambda: hops.moe_ffn(h, zidx, zwt, zwu, zwd, 1, bf), iters=3, warm=1),
            nbytes=min(ze, real) * 2 * zeff * d * 2.0 + tk * d * 4.0, flops=real * 4.0 * zeff * d)
        f = size["ff"]
        gu = rnd(tk, 2 * f)
        rec(f"glu.{name}", _time(lambda: hops.glu(gu, 7.0, 1.702, 1.0, bf)), nbytes=tk * f * 6.0)
        lf = int(3.5 * d)
        wgl, wdn = rnd(2 * lf, d, sc=d ** -0.5), rnd(d, lf, sc=lf ** -0.5)
        rec(f"llama.mlp.{name}", _time(lambda: ops.linear(ops.gate_up_silu(h, wgl), wdn), iters=3, warm=1),
            nbytes=3 * lf * d * 2.0 + tk * d * 4.0, flops=tk * 6.0 * lf * d)
    return out


def _kernels_tugovik(size: dict, ksize: dict, dev, T: int, ctx: int, rows: int) -> dict:
    """Tugovik's kernels and their closest existing kernels at this size: seconds, and the fraction of the roofline
    reached.  ``ksize``: the Kalesun sizes of the same width (for the kernels it stands beside)."""
    from chronos import ops
    from chronos.ops import hybrid as hops

    out = {}
    bf = torch.bfloat16
    d = size["width"]
    g = torch.Generator(device=dev).manual_seed(1)
    rnd = lambda *s, dt=bf, sc=1.0: (torch.randn(*s, device=dev, generator=g) * sc).to(dt)  # noqa: E731
    i32 = dict(dtype=torch.int32, device=dev)

    def rec(name, secs, nbytes=0.0, flops=0.0):
        roof = max(nbytes / HBM_BPS, flops / BF16_FLOPS)
        _say(f"  {name}: {secs * 1e6:.1f} us, roofline {roof * 1e6:.2f} us")
        out[name] = dict(us=round(secs * 1e6, 1), roofline_us=round(roof * 1e6, 2), of_roofline=round(roof / secs, 4))

    bs = 16
    seqs = max(1, T // ctx)
    per = ctx // bs + 1
    nb = max(seqs, rows) * per + 1
    bt = torch.arange(1, 1 + seqs * per, **i32).view(seqs, per)
    qs = torch.arange(0, (seqs + 1) * ctx, ctx, **i32)
    pos = torch.arange(ctx, **i32).repeat(seqs)
    tseq = torch.arange(seqs, **i32).repeat_interleave(ctx)
    btd = torch.arange(1, 1 + rows * per, **i32).view(rows, per)
    qsd = torch.arange(rows + 1, **i32)
    posd = torch.full((rows,), ctx, **i32)
    tseqd = torch.arange(rows, **i32)
    NS = max(seqs, rows) + 1
    p0, sl, sld = torch.zeros(seqs, **i32), torch.arange(seqs, **i32), torch.arange(rows, **i32)
    # ---- the stream's joins
    y, y2, x32, w32 = rnd(T, d), rnd(T, d), rnd(T, d, dt=torch.float32), rnd(d, dt=torch.float32)
    g2 = rnd(T, 1, dt=torch.float32)
    rec("add_rms_norm", _time(lambda: hops.add_rms_norm(y, x32, w32, 1e-6, bf)), T * d * (2 + 4 + 4 + 2))
    rec("add_rms_norm.gated_pair", _time(lambda: hops.add_rms_norm(y, x32, None, 1e-6, bf, y2, g2)), T * d * (2 + 2 + 4 + 4 + 2))
    rec("add_rms_norm.normed_addend", _time(lambda: hops.add_rms_norm(y, x32, w32, 1e-6, bf, w_y=w32)), T * d * (2 + 4 + 4 + 2))
    rec("kalesun.scale_add_rms_norm", _time(lambda: hops.scale_add_rms_norm(y, x32, w32, 1.0, 1e-6, bf)), T * d * (2 + 4 + 4 + 2))
    xb, wb = rnd(T, d), rnd(d)
    rec("llama.add_rmsnorm", _time(lambda: ops.add_rmsnorm(y, xb, wb, 1e-5)), T * d * (2 + 2 + 2 + 2))
    sd = size["side"]
    a_, table, ids = rnd(T, sd), rnd(VOCAB, 4 * sd), torch.randint(0, VOCAB, (T,), device=dev, generator=g).int()
    rec("token_gate", _time(lambda: hops.token_gate(a_, ids, table, sd, bf)), T * sd * 6.0)
    # ---- attention: the chunk mask beside Kalesun's window of the same span (with sink and gate) and Llama's
    H, G, D, Dv, chunk = size["a"]
    kc, vc = rnd(nb, bs, G, D, sc=0.3), rnd(nb, bs, G, Dv, sc=0.3)
    C = (H + G) * D + G * Dv
    qkv = rnd(seqs * ctx, C, sc=0.3)
    vis = sum(i % chunk + 1 for i in range(ctx))
    rec("chunk_attention.prefill", _time(lambda: hops.window_attention(qkv, kc, vc, bt, qs, pos, None, None, D ** -0.5, 0, 0, H, bf, ctx, chunk), iters=3, warm=1),
        flops=2.0 * seqs * vis * H * (D + Dv))
    rec("window_prep.plain.prefill", _time(lambda: hops.window_prep(qkv, H, G, D, Dv, None, None, pos, tseq, bt, None, None, 1e-6, None, 0, kc, vc, False)),
        nbytes=seqs * ctx * 2 * G * (D + Dv) * 2.0)
    qkvd = rnd(rows, C, sc=0.3)
    rec("chunk_attention.decode", _time(lambda: hops.window_attention(qkvd, kc, vc, btd, qsd, posd, None, None, D ** -0.5, 0, 0, H, bf, 1, chunk)),
        nbytes=rows * (ctx % chunk + 1) * G * (D + Dv) * 2.0)
    posm = torch.full((rows,), ctx // chunk * chunk + chunk - 1, **i32)   # the last position of a chunk: every key of it
    btm = torch.arange(1, 1 + rows * (per + chunk // bs), **i32).view(rows, -1) % (nb - 1) + 1
    rec("chunk_attention.decode_full_chunk", _time(lambda: hops.window_attention(qkvd, kc, vc, btm, qsd, posm, None, None, D ** -0.5, 0, 0, H, bf, 1, chunk)),
        nbytes=rows * chunk * G * (D + Dv) * 2.0)
    kH, kG, kD, kDv, win, keep = ksize["a"]
    kkc, kvc = rnd(nb, bs, kG, kD, sc=0.3), rnd(nb, bs, kG, kDv, sc=0.3)
    kqkv = rnd(seqs * ctx, (kH + kG) * kD + kG * kDv, sc=0.3)
    kgate, ksink = rnd(seqs * ctx, kH, dt=torch.float32), rnd(kH, dt=torch.float32)
    kvis = sum(min(i + 1, win) + max(0, min(keep, i + 1 - win)) for i in range(ctx))
    rec("kalesun.window_attention.prefill", _time(lambda: hops.window_attention(kqkv, kkc, kvc, bt, qs, pos, ksink, kgate, kD ** -0.5, win, keep, kH, bf, ctx), iters=3, warm=1),
        flops=2.0 * seqs * kvis * kH * (kD + kDv))
    kqkvd, kgated = rnd(rows, (kH + kG) * kD + kG * kDv, sc=0.3), rnd(rows, kH, dt=torch.float32)
    rec("kalesun.window_attention.decode", _time(lambda: hops.window_attention(kqkvd, kkc, kvc, btd, qsd, posd, ksink, kgated, kD ** -0.5, win, keep, kH, bf, 1)),
        nbytes=rows * (min(ctx + 1, win) + keep) * kG * (kD + kDv) * 2.0)
    hq = d // 128
    hkv = max(1, hq // 4)
    lkc, lvc = rnd(nb, hkv, bs, 128, sc=0.3), rnd(nb, hkv, 128, bs, sc=0.3)
    q = rnd(seqs * ctx, hq, 128, sc=0.3)
    ctxl = torch.full((seqs,), ctx, **i32)
    tiles = torch.tensor(ops.attention_tiles([ctx] * seqs, hq, hkv, 8), **i32).view(-1, 2)
    rec("llama.attention.prefill", _time(lambda: ops.paged_attention(q, lkc, lvc, bt, qs, ctxl, tiles, tiles.shape[0], 8, 1), iters=3, warm=1),
        flops=4.0 * seqs * ctx * (ctx + 1) / 2 * hq * 128)
    qd = rnd(rows, hq, 128, sc=0.3)
    ctxd = torch.full((rows,), ctx + 1, **i32)
    ns = ops.pick_nsplit(rows * hkv, ctx + 1)
    rec("llama.attention.decode", _time(lambda: ops.paged_attention(qd, lkc, lvc, btd, qsd, ctxd, None, rows, 1, ns)),
        nbytes=rows * (ctx + 1) * hkv * 128 * 2 * 2.0)
    # ---- the state-space layer: convolution, per-token scalars, scan, gated group norm
    mh, mv, mn, mg = size["m"]
    inner, Cc = mh * mv, mh * mv + 2 * mg * mn
    proj, taps, cb = rnd(seqs * ctx, inner + Cc, sc=0.5), rnd(Cc, 4, dt=torch.float32), rnd(Cc, dt=torch.float32)
    hist = torch.zeros(NS, 3, Cc, device=dev, dtype=bf)
    rec("short_conv.bias.prefill", _time(lambda: hops.short_conv(proj, taps, tseq, qs, p0, sl, hist, True, cb, inner)),
        nbytes=seqs * ctx * Cc * 4.0)
    xbc = hops.short_conv(proj, taps, tseq, qs, p0, sl, hist, True, cb, inner)
    dtp, alog = rnd(seqs * ctx, mh, dt=torch.float32), rnd(mh, dt=torch.float32, sc=0.3)
    rec("ssm_prep.prefill", _time(lambda: hops.ssm_prep(dtp, alog)), nbytes=seqs * ctx * mh * 12.0)
    decay, dts = hops.ssm_prep(dtp, alog)
    S = torch.zeros(NS, mh, mn, mv, device=dev)
    rec("linear_scan.ssm.prefill", _time(lambda: hops.linear_scan(xbc, inner + mg * mn, inner, 0, None, None, 1.0, decay, None, qs, p0, sl, S, mg, mh, mn, mv, dts), iters=3, warm=1),
        nbytes=seqs * ctx * Cc * 2.0, flops=seqs * ctx * mh * mn * mv * 4.0)
    xbcd = rnd(rows, Cc, sc=0.5)
    decd, dtd = torch.rand(rows, mh, device=dev), torch.rand(rows, mh, device=dev)
    rec("linear_scan.ssm.decode", _time(lambda: hops.linear_scan(xbcd, inner + mg * mn, inner, 0, None, None, 1.0, decd, None, qsd, posd, sld, S, mg, mh, mn, mv, dtd)),
        nbytes=rows * mh * mn * mv * 4 * 2.0)
    o = torch.randn(seqs * ctx, mh, mv, device=dev)
    skip, nw = rnd(mh, dt=torch.float32), rnd(inner, dt=torch.float32)
    rec("gated_group_norm.prefill", _time(lambda: hops.gated_group_norm(o, xbc, 0, skip, proj, 0, nw, mg, 1e-6, bf)),
        nbytes=seqs * ctx * inner * (4 + 2 + 2 + 2.0))
    rec("kalesun.head_norm_gate.prefill", _time(lambda: hops.head_norm_gate(o, proj, 0, nw, 1e-6, True, bf)),
        nbytes=seqs * ctx * inner * (4 + 2 + 2.0))
    for name, (hh, hk, dd, dv), delta in (("delta", ksize["d"], True), ("gla", (ksize["g"][0], ksize["g"][0], *ksize["g"][1:]), False)):
        Cq = 2 * hk * dd + hh * dv
        kS = torch.zeros(NS, hh, dd, dv, device=dev)

        def scan(pr, qs_, p0_, sl_, n):
            if delta:
                qsc, ksc = torch.rand(n, hk, device=dev), torch.rand(n, hk, device=dev)
                dec, beta = torch.rand(n, hh, device=dev), torch.rand(n, hh, device=dev)
                return lambda: hops.linear_scan(pr, 0, hk * dd, 2 * hk * dd, qsc, ksc, 1.0, dec, beta, qs_, p0_, sl_, kS, hk, hh, dd, dv)
            dec = torch.rand(n, hh, dd, device=dev)
            return lambda: hops.linear_scan(pr, 0, hk * dd, 2 * hk * dd, None, None, dd ** -0.5, dec, None, qs_, p0_, sl_, kS, hk, hh, dd, dv)

        kp = rnd(seqs * ctx, Cq, sc=0.5)
        rec(f"kalesun.linear_scan.{name}.prefill", _time(scan(kp, qs, p0, sl, seqs * ctx), iters=3, warm=1),
            nbytes=seqs * ctx * Cq * 2.0, flops=seqs * ctx * hh * dd * dv * (6.0 if delta else 4.0))
        kpd = rnd(rows, Cq, sc=0.5)
        rec(f"kalesun.linear_scan.{name}.decode", _time(scan(kpd, qsd, posd, sld, rows)), nbytes=rows * hh * dd * dv * 4 * 2.0)
    # ---- the gated linear recurrence: block-diagonal gate projections (float32 library product) and the scan
    rw, rb = size["r"]
    bw = rw // rb
    yx = rnd(seqs * ctx, 2 * rw, sc=0.5)
    u = rnd(seqs * ctx, rw, sc=0.5)
    wg, bg = rnd(rb, bw, 2 * bw, sc=bw ** -0.5), rnd(rb, 1, 2 * bw, dt=torch.float32)   # bfloat16 weights, float32 out
    rec("block_gates.prefill", _time(lambda: hops.block_gates(u, wg, bg), iters=3, warm=1),
        nbytes=seqs * ctx * rw * (2 + 8.0), flops=seqs * ctx * rw * bw * 4.0)
    gates = hops.block_gates(u, wg, bg)
    sp = torch.rand(rw, device=dev)
    Sr = torch.zeros(NS, rw, device=dev)
    rec("rglru_scan.prefill", _time(lambda: hops.rglru_scan(u, gates, sp, 8.0, yx, 0, qs, p0, sl, Sr, bf, ctx), iters=3, warm=1),
        nbytes=seqs * ctx * rw * (8 + 2 + 2 + 2.0))
    ud, yxd = rnd(rows, rw, sc=0.5), rnd(rows, 2 * rw, sc=0.5)
    rec("block_gates.decode", _time(lambda: hops.block_gates(ud, wg, bg)), nbytes=rb * bw * 2 * bw * 4.0)
    gd = hops.block_gates(ud, wg, bg)
    rec("rglru_scan.decode", _time(lambda: hops.rglru_scan(ud, gd, sp, 8.0, yxd, 0, qsd, posd, sld, Sr, bf, 1)),
        nbytes=rows * rw * (8 + 2 + 2 + 2 + 8.0))
    # ---- feed-forwards: the grouped sigmoid router beside the top-k softmax router; the experts are Kalesun's kernel
    ne, top, ng, keep, eff, sff = size["moe"]
    wr, br = rnd(ne, d, sc=0.05), rnd(ne, dt=torch.float32, sc=0.01)
    wgu = rnd(ne, 2 * eff, d, sc=d ** -0.5)[:, hops.moe_glu_row_order(eff).to(dev)].contiguous()
    wd = rnd(ne, d, eff, sc=eff ** -0.5)
    inf = float("inf")
    for name, tk in (("prefill", T), ("decode", rows)):
        h = rnd(tk, d)
        rec(f"moe_route_group.{name}", _time(lambda: hops.moe_route_group(h, wr, top, ng, keep, 2.5)), nbytes=tk * d * 2.0 + ne * d * 2.0)
        rec(f"kalesun.moe_route_topk.{name}", _time(lambda: hops.moe_route_topk(h, wr, br, top)), nbytes=tk * d * 2.0 + ne * d * 2.0)
        idx, wt = hops.moe_route_group(h, wr, top, ng, keep, 2.5)
        used = min(ne, tk * top) * 3 * eff * d * 2.0
        rec(f"moe_glu_ffn.silu.{name}", _time(lambda: hops.moe_glu_ffn(h, idx, wt, wgu, wd, inf, 1.0, 0.0, bf, True), iters=3, warm=1),
            nbytes=used + tk * d * 4.0, flops=tk * top * 6.0 * eff * d)
        rec(f"kalesun.moe_glu_ffn.{name}", _time(lambda: hops.moe_glu_ffn(h, idx, wt, wgu, wd, 7.0, 1.702, 1.0, bf, True), iters=3, warm=1),
            nbytes=used + tk * d * 4.0, flops=tk * top * 6.0 * eff * d)
        lf = int(3.5 * d)
        wgl, wdn = rnd(2 * lf, d, sc=d ** -0.5), rnd(d, lf, sc=lf ** -0.5)
        rec(f"llama.mlp.{name}", _time(lambda: ops.linear(ops.gate_up_silu(h, wgl), wdn), iters=3, warm=1),
            nbytes=3 * lf * d * 2.0 + tk * d * 4.0, flops=tk * 6.0 * lf * d)
    return out


def run_tugovik(sizes: list, seqs: int = 4, plen: int = 2048, rows: int = 64, ctx: int = 2048, device: str = "cuda") -> dict:
    from chronos import ops
    from chronos.models import kalesun, llama, tugovik
    from chronos.models.hybrid import HybridDecoder

    dev = torch.device(device if ":" in device else device + ":0")
    torch.cuda.set_device(dev)
    ops.load()
    ops.device_init()
    res = {}
    P = ctx + plen + 16
    for name in sizes:
        size, ksize = TUGOVIK_SIZES[name], KALESUN_SIZES[name]
        t0 = time.time()
        cfg = tugovik.config_from_dict(tugovik_config(size), name=f"tugovik-{name}", max_position=P)
        tm = HybridDecoder(cfg, tugovik.pack_weights(cfg, tugovik.random_tensors(cfg, 0), dev, torch.bfloat16), dev, P,
                           torch.bfloat16)
        entry = dict(tugovik=dict(params=cfg.param_count(), **_model_steps(tm, dev, seqs, plen, rows, ctx)))
        _say(f"size {name}: tugovik {entry['tugovik']}")
        del tm
        kcfg = kalesun.config_from_dict(kalesun_config(ksize), name=f"kalesun-{name}", max_position=P)
        km = HybridDecoder(kcfg, kalesun.pack_weights(kcfg, kalesun.random_tensors(kcfg, 0), dev, torch.bfloat16), dev, P,
                           torch.bfloat16)
        entry["kalesun"] = dict(params=kcfg.param_count(), **_model_steps(km, dev, seqs, plen, rows, ctx))
        _say(f"  kalesun {entry['kalesun']}")
        del km
        d = size["width"]
        lc = llama.LlamaConfig(name=f"llama-{name}", vocab_size=VOCAB, hidden_size=d, intermediate_size=int(3.5 * d),
                               num_layers=LAYERS, num_heads=d // 128, num_kv_heads=max(1, d // 512), max_position=P)
        lm = llama.LlamaModel(lc, llama.random_weights(lc, None, dev, 0), None, dev, P)
        entry["llama"] = dict(params=lc.param_count(), **_model_steps(lm, dev, seqs, plen, rows, ctx))
        _say(f"  llama {entry['llama']}")
        del lm
        torch.cuda.empty_cache()
        entry["kernels"] = _kernels_tugovik(size, ksize, dev, seqs * plen, ctx, rows)
        entry["seconds"] = round(time.time() - t0, 1)
        res[name] = entry
        torch.cuda.empty_cache()
    return dict(metric="design_compare", design="tugovik", beside="kalesun and llama (equal width and depth)",
                layers=LAYERS, workload=dict(prefill=f"{seqs} x {plen} tokens in one step",
                                             decode=f"{rows} rows at context {ctx}"),
                dtype="bf16", data="synthetic", sizes=res)


def _kernels_vogerax(size: dict, ksize: dict, dev, T: int, ctx: int, rows: int) -> dict:
    """Vogerax's kernels and their closest existing kernels at this size: seconds, and the fraction of the roofline
    reached.  ``ksize``: the Kalesun sizes of the same width (for the kernels it stands beside)."""
    from chronos import ops
    from chronos.models.hybrid import rope_cos_sin
    from chronos.ops import hybrid as hops

    out = {}
    bf = torch.bfloat16
    d, ng = size["width"], size["groups"]
    g = torch.Generator(device=dev).manual_seed(1)
    rnd = lambda *s, dt=bf, sc=1.0: (torch.randn(*s, device=dev, generator=g) * sc).to(dt)  # noqa: E731
    i32 = dict(dtype=torch.int32, device=dev)

    def rec(name, secs, nbytes=0.0, flops=0.0):
        roof = max(nbytes / HBM_BPS, flops / BF16_FLOPS)
        _say(f"  {name}: {secs * 1e6:.1f} us, roofline {roof * 1e6:.2f} us")
        out[name] = dict(us=round(secs * 1e6, 1), roofline_us=round(roof * 1e6, 2), of_roofline=round(roof / secs, 4))

    bs = 16
    seqs = max(1, T // ctx)
    per = ctx // bs + 1
    nb = max(seqs, rows) * per + 1
    bt = torch.arange(1, 1 + seqs * per, **i32).view(seqs, per)
    qs = torch.arange(0, (seqs + 1) * ctx, ctx, **i32)
    pos = torch.arange(ctx, **i32).repeat(seqs)
    tseq = torch.arange(seqs, **i32).repeat_interleave(ctx)
    btd = torch.arange(1, 1 + rows * per, **i32).view(rows, per)
    qsd = torch.arange(rows + 1, **i32)
    posd = torch.full((rows,), ctx, **i32)
    NS = max(seqs, rows) + 1
    p0, sl, sld = torch.zeros(seqs, **i32), torch.arange(seqs, **i32), torch.arange(rows, **i32)
    # ---- the stream's joins: norm of the addend, add, norm for the next sublayer, in one kernel
    y, y2, x32 = rnd(T, d), rnd(T, d), rnd(T, d, dt=torch.float32)
    w1, w2, w3, w4 = (rnd(d, dt=torch.float32) for _ in range(4))
    rec("sandwich_join", _time(lambda: hops.sandwich_join(y, x32, w1, w2, ng, 1e-5, bf)), T * d * (2 + 4 + 4 + 2))
    rec("sandwich_join.two_addends", _time(lambda: hops.sandwich_join(y, x32, w1, w2, ng, 1e-5, bf, y2)), T * d * (2 + 2 + 4 + 4 + 2))
    rec("sandwich_join.pair", _time(lambda: hops.sandwich_join(y, x32, w1, w2, ng, 1e-5, bf, y2, (w3, w4))), T * d * (2 + 2 + 4 + 4 + 2))
    yd, y2d, xd = rnd(rows, d), rnd(rows, d), rnd(rows, d, dt=torch.float32)
    rec("sandwich_join.pair.decode", _time(lambda: hops.sandwich_join(yd, xd, w1, w2, ng, 1e-5, bf, y2d, (w3, w4))), rows * d * 14.0)
    rec("kalesun.scale_add_rms_norm", _time(lambda: hops.scale_add_rms_norm(y, x32, w1, 1.0, 1e-6, bf)), T * d * (2 + 4 + 4 + 2))
    rec("tugovik.add_rms_norm.normed_addend", _time(lambda: hops.add_rms_norm(y, x32, w1, 1e-6, bf, w_y=w2)), T * d * (2 + 4 + 4 + 2))
    xb, wb = rnd(T, d), rnd(d)
    rec("llama.add_rmsnorm", _time(lambda: ops.add_rmsnorm(y, xb, wb, 1e-5)), T * d * (2 + 2 + 2 + 2))
    # ---- pooled-window attention beside Kalesun's window of the same span (with sink and gate) and Llama's
    H, G, D, win, pool = size["a"]
    ep = (bs + pool - 1) // pool
    kc, vc = rnd(nb, bs, G, D, sc=0.3), rnd(nb, bs, G, D, sc=0.3)
    kp, vp = rnd(nb, ep, G, D, sc=0.3), rnd(nb, ep, G, D, sc=0.3)
    C = (H + G) * D
    qk = rnd(seqs * ctx, C, sc=0.3)
    tab = rope_cos_sin(5e5, D // 2, ctx + 2, dev, ("linear", 4.0))
    vis = sum(min(i + 1, win) + max(0, i - win + 1) // pool for i in range(ctx))
    rec("pooled_attention.prefill", _time(lambda: hops.window_attention(qk, kc, vc, bt, qs, pos, None, None, D ** -0.5, win, 0, H, bf, ctx, 0, pool, kp, vp), iters=3, warm=1),
        flops=4.0 * seqs * vis * H * D)
    rec("window_prep.values_are_keys.prefill", _time(lambda: hops.window_prep(qk, H, G, D, D, None, None, pos, tseq, bt, None, None, 1e-5, tab, D // 2, kc, vc, False, H * D)),
        nbytes=seqs * ctx * (2 * (H + G) * D + 2 * G * D) * 2.0)
    rec("pool_blocks.prefill", _time(lambda: hops.pool_blocks(kc, vc, kp, vp, bt, qs, p0, pool, ctx)),
        nbytes=seqs * ctx * 2 * G * D * 2.0 * (1 + 1.0 / pool))
    qkd = rnd(rows, C, sc=0.3)
    rec("pooled_attention.decode", _time(lambda: hops.window_attention(qkd, kc, vc, btd, qsd, posd, None, None, D ** -0.5, win, 0, H, bf, 1, 0, pool, kp, vp)),
        nbytes=rows * (min(ctx + 1, win) + max(0, ctx - win + 1) // pool) * G * 2 * D * 2.0)
    rec("pool_blocks.decode", _time(lambda: hops.pool_blocks(kc, vc, kp, vp, btd, qsd, posd, pool, 1)), nbytes=1.0)
    kH, kG, kD, kDv, kwin, keep = ksize["a"]
    kkc, kvc = rnd(nb, bs, kG, kD, sc=0.3), rnd(nb, bs, kG, kDv, sc=0.3)
    kqkv = rnd(seqs * ctx, (kH + kG) * kD + kG * kDv, sc=0.3)
    kgate, ksink = rnd(seqs * ctx, kH, dt=torch.float32), rnd(kH, dt=torch.float32)
    kvis = sum(min(i + 1, kwin) + max(0, min(keep, i + 1 - kwin)) for i in range(ctx))
    rec("kalesun.window_attention.prefill", _time(lambda: hops.window_attention(kqkv, kkc, kvc, bt, qs, pos, ksink, kgate, kD ** -0.5, kwin, keep, kH, bf, ctx), iters=3, warm=1),
        flops=2.0 * seqs * kvis * kH * (kD + kDv))
    kqkvd, kgated = rnd(rows, (kH + kG) * kD + kG * kDv, sc=0.3), rnd(rows, kH, dt=torch.float32)
    rec("kalesun.window_attention.decode", _time(lambda: hops.window_attention(kqkvd, kkc, kvc, btd, qsd, posd, ksink, kgated, kD ** -0.5, kwin, keep, kH, bf, 1)),
        nbytes=rows * (min(ctx + 1, kwin) + keep) * kG * (kD + kDv) * 2.0)
    # ---- causal sink attention with rotated values and a gate per column, beside Llama's causal attention
    lH, lG, lD, lDv = size["l"]
    lkc, lvc = rnd(nb, bs, lG, lD, sc=0.3), rnd(nb, bs, lG, lDv, sc=0.3)
    Cl = (lH + lG) * lD + lG * lDv + lH * lDv
    lq = rnd(seqs * ctx, Cl, sc=0.3)
    lsink = rnd(lH, dt=torch.float32)
    vtab = rope_cos_sin(1e5, lDv, ctx + 2, dev)
    ltab = rope_cos_sin(1e5, lD // 2, ctx + 2, dev, ("ramp", 8.0, 4096.0, 16.0, 2.0))
    qn, kn = rnd(lD, dt=torch.float32), rnd(lD, dt=torch.float32)
    full_pairs = seqs * ctx * (ctx + 1) / 2
    lg_off = (lH + lG) * lD + lG * lDv   # outputs turned back and gated per column in the attention's epilogue
    rec("sink_attention.prefill", _time(lambda: hops.window_attention(lq, lkc, lvc, bt, qs, pos, lsink, None, lD ** -0.5, 0, 0, lH, bf, ctx, 0, 0, None, None, vtab, lg_off), iters=3, warm=1),
        flops=2.0 * full_pairs * lH * (lD + lDv))
    rec("window_prep.rotated_values.prefill", _time(lambda: hops.window_prep(lq, lH, lG, lD, lDv, None, None, pos, tseq, bt, qn, kn, 1e-5, ltab, lD // 2, lkc, lvc, False, -1, vtab)),
        nbytes=seqs * ctx * (2 * (lH + lG) * lD + 2 * lG * lDv) * 2.0)
    lo = rnd(seqs * ctx, lH * lDv)
    rec("unrotate_gate.prefill", _time(lambda: hops.unrotate_gate(lo, pos, vtab, lq, (lH + lG) * lD + lG * lDv, lH, lDv, bf)),
        nbytes=seqs * ctx * lH * lDv * 6.0)
    lqd = rnd(rows, Cl, sc=0.3)
    rec("sink_attention.decode", _time(lambda: hops.window_attention(lqd, lkc, lvc, btd, qsd, posd, lsink, None, lD ** -0.5, 0, 0, lH, bf, 1, 0, 0, None, None, vtab, lg_off)),
        nbytes=rows * (ctx + 1) * lG * (lD + lDv) * 2.0)
    hq = d // 128
    hkv = max(1, hq // 4)
    akc, avc = rnd(nb, hkv, bs, 128, sc=0.3), rnd(nb, hkv, 128, bs, sc=0.3)
    q = rnd(seqs * ctx, hq, 128, sc=0.3)
    ctxl = torch.full((seqs,), ctx, **i32)
    tiles = torch.tensor(ops.attention_tiles([ctx] * seqs, hq, hkv, 8), **i32).view(-1, 2)
    rec("llama.attention.prefill", _time(lambda: ops.paged_attention(q, akc, avc, bt, qs, ctxl, tiles, tiles.shape[0], 8, 1), iters=3, warm=1),
        flops=4.0 * full_pairs * hq * 128)
    qd = rnd(rows, hq, 128, sc=0.3)
    ctxd = torch.full((rows,), ctx + 1, **i32)
    ns = ops.pick_nsplit(rows * hkv, ctx + 1)
    rec("llama.attention.decode", _time(lambda: ops.paged_attention(qd, akc, avc, btd, qsd, ctxd, None, rows, 1, ns)),
        nbytes=rows * (ctx + 1) * hkv * 128 * 2 * 2.0)
    # ---- retention: the linear-state scan with fixed decays beside Kalesun's gated linear attention on the same kernel
    rh, rd, rv = size["r"]
    Cr = 2 * rh * rd + 2 * rh * rv
    S = torch.zeros(NS, rh, rd, rv, device=dev)
    dec = torch.tensor([math.exp(-1.0 / (16.0 * 128.0 ** (h / max(1, rh - 1)))) for h in range(rh)], device=dev)
    rtab = rope_cos_sin(1e4, rd, ctx + 2, dev)
    ones = torch.ones(rh * rv, device=dev)
    proj, projd = rnd(seqs * ctx, Cr, sc=0.5), rnd(rows, Cr, sc=0.5)
    rec("rotate_qk.prefill", _time(lambda: hops.rotate_qk(proj, 0, rh * rd, rh, rh, rd, rd, rtab, pos, 1.0, 1.0)), nbytes=seqs * ctx * 2 * rh * rd * 4.0)
    rec("retention_scan.prefill", _time(lambda: hops.linear_scan(proj, 0, rh * rd, 2 * rh * rd, None, None, 1.0, dec, None, qs, p0, sl, S, rh, rh, rd, rv), iters=3, warm=1),
        nbytes=seqs * ctx * Cr * 2.0, flops=seqs * ctx * rh * rd * rv * 4.0)
    rec("retention_scan.decode", _time(lambda: hops.linear_scan(projd, 0, rh * rd, 2 * rh * rd, None, None, 1.0, dec, None, qsd, posd, sld, S, rh, rh, rd, rv)),
        nbytes=rows * rh * rd * rv * 4 * 2.0)
    o32 = rnd(seqs * ctx, rh, rv, dt=torch.float32)
    rec("head_norm_gate.prefill", _time(lambda: hops.head_norm_gate(o32, proj, 2 * rh * rd + rh * rv, ones, 1e-5, True, bf)), nbytes=seqs * ctx * rh * rv * 8.0)
    gh, gd, gv = ksize["g"]
    gS = torch.zeros(NS, gh, gd, gv, device=dev)
    gproj, gprojd = rnd(seqs * ctx, 2 * gh * gd + gh * gv, sc=0.5), rnd(rows, 2 * gh * gd + gh * gv, sc=0.5)
    gdec, gdecd = torch.rand(seqs * ctx, gh, gd, device=dev), torch.rand(rows, gh, gd, device=dev)
    rec("kalesun.linear_scan.gla.prefill", _time(lambda: hops.linear_scan(gproj, 0, gh * gd, 2 * gh * gd, None, None, gd ** -0.5, gdec, None, qs, p0, sl, gS, gh, gh, gd, gv), iters=3, warm=1),
        nbytes=seqs * ctx * (2 * gh * gd + gh * gv) * 2.0, flops=seqs * ctx * gh * gd * gv * 4.0)
    rec("kalesun.linear_scan.gla.decode", _time(lambda: hops.linear_scan(gprojd, 0, gh * gd, 2 * gh * gd, None, None, gd ** -0.5, gdecd, None, qsd, posd, sld, gS, gh, gh, gd, gv)),
        nbytes=rows * gh * gd * gv * 4 * 2.0)
    # ---- feed-forwards: squared-ReLU experts behind a softmax router beside Kalesun's gated experts and Llama's MLP
    ne, top, eff, sff = size["moe"]
    wr, corr = rnd(ne, d, sc=0.05), torch.zeros(ne, device=dev)
    wu, wd = rnd(ne, eff, d, sc=d ** -0.5), rnd(ne, d, eff, sc=eff ** -0.5)
    kne, ktop, keff = ksize["moe"]
    kwr, kbr = rnd(kne, d, sc=0.05), rnd(kne, dt=torch.float32, sc=0.01)
    kwgu = rnd(kne, 2 * keff, d, sc=d ** -0.5)[:, hops.moe_glu_row_order(keff).to(dev)].contiguous()
    kwd = rnd(kne, d, keff, sc=keff ** -0.5)
    for name, tk in (("prefill", T), ("decode", rows)):
        h = rnd(tk, d)
        idx, wt = hops.moe_route(h, wr, corr, top)
        rec(f"moe_route.{name}", _time(lambda: hops.moe_route(h, wr, corr, top)), nbytes=tk * d * 2.0 + ne * d * 2.0)
        rec(f"moe_ffn.relu2.{name}", _time(lambda: hops.moe_ffn(h, idx, wt, wu, wd, hops.ACT_RELU2, bf), iters=3, warm=1),
            nbytes=min(ne, tk * top) * 2 * eff * d * 2.0 + tk * d * 4.0, flops=tk * top * 4.0 * eff * d)
        kidx, kwt = hops.moe_route_topk(h, kwr, kbr, ktop)
        rec(f"kalesun.moe_route_topk.{name}", _time(lambda: hops.moe_route_topk(h, kwr, kbr, ktop)), nbytes=tk * d * 2.0 + kne * d * 2.0)
        rec(f"kalesun.moe_glu_ffn.{name}", _time(lambda: hops.moe_glu_ffn(h, kidx, kwt, kwgu, kwd, 7.0, 1.702, 1.0, bf, True), iters=3, warm=1),
            nbytes=min(kne, tk * ktop) * 3 * keff * d * 2.0 + tk * d * 4.0, flops=tk * ktop * 6.0 * keff * d)
        lf = int(3.5 * d)
        wgl, wdn = rnd(2 * lf, d, sc=d ** -0.5), rnd(d, lf, sc=lf ** -0.5)
        rec(f"llama.mlp.{name}", _time(lambda: ops.linear(ops.gate_up_silu(h, wgl), wdn), iters=3, warm=1),
            nbytes=3 * lf * d * 2.0 + tk * d * 4.0, flops=tk * 6.0 * lf * d)
    return out


def run_vogerax(sizes: list, seqs: int = 4, plen: int = 2048, rows: int = 64, ctx: int = 2048, device: str = "cuda") -> dict:
    from chronos import ops
    from chronos.models import kalesun, llama, vogerax
    from chronos.models.hybrid import HybridDecoder

    dev = torch.device(device if ":" in device else device + ":0")
    torch.cuda.set_device(dev)
    ops.load()
    ops.device_init()
    res = {}
    P = ctx + plen + 16
    for name in sizes:
        size, ksize = VOGERAX_SIZES[name], KALESUN_SIZES[name]
        t0 = time.time()
        cfg = vogerax.config_from_dict(vogerax_config(size), name=f"vogerax-{name}", max_position=P)
        vm = HybridDecoder(cfg, vogerax.pack_weights(cfg, vogerax.random_tensors(cfg, 0), dev, torch.bfloat16), dev, P,
                           torch.bfloat16)
        entry = dict(vogerax=dict(params=cfg.param_count(), **_model_steps(vm, dev, seqs, plen, rows, ctx)))
        _say(f"size {name}: vogerax {entry['vogerax']}")
        del vm
        kcfg = kalesun.config_from_dict(kalesun_config(ksize), name=f"kalesun-{name}", max_position=P)
        km = HybridDecoder(kcfg, kalesun.pack_weights(kcfg, kalesun.random_tensors(kcfg, 0), dev, torch.bfloat16), dev, P,
                           torch.bfloat16)
        entry["kalesun"] = dict(params=kcfg.param_count(), **_model_steps(km, dev, seqs, plen, rows, ctx))
        _say(f"  kalesun {entry['kalesun']}")
        del km
        d = size["width"]
        lc = llama.LlamaConfig(name=f"llama-{name}", vocab_size=VOCAB, hidden_size=d, intermediate_size=int(3.5 * d),
                               num_layers=LAYERS, num_heads=d // 128, num_kv_heads=max(1, d // 512), max_position=P)
        lm = llama.LlamaModel(lc, llama.random_weights(lc, None, dev, 0), None, dev, P)
        entry["llama"] = dict(params=lc.param_count(), **_model_steps(lm, dev, seqs, plen, rows, ctx))
        _say(f"  llama {entry['llama']}")
        del lm
        torch.cuda.empty_cache()
        entry["kernels"] = _kernels_vogerax(size, ksize, dev, seqs * plen, ctx, rows)
        entry["seconds"] = round(time.time() - t0, 1)
        res[name] = entry
        torch.cuda.empty_cache()
    return dict(metric="design_compare", design="vogerax", beside="kalesun and llama (equal width and depth)",
                layers=LAYERS, workload=dict(prefill=f"{seqs} x {plen} tokens in one step",
                                             decode=f"{rows} rows at context {ctx}"),
                dtype="bf16", data="synthetic", sizes=res)


def run_kalesun(sizes: list, seqs: int = 4, plen: int = 2048, rows: int = 64, ctx: int = 2048, device: str = "cuda") -> dict:
    from chronos import ops
    from chronos.models import kalesun, llama, zokunex
    from chronos.models.hybrid import HybridDecoder

    dev = torch.device(device if ":" in device else device + ":0")
    torch.cuda.set_device(dev)
    ops.load()
    ops.device_init()
    res = {}
    P = ctx + plen + 16
    for name in sizes:
        size, zsize = KALESUN_SIZES[name], SIZES[name]
        t0 = time.time()
        cfg = kalesun.config_from_dict(kalesun_config(size), name=f"kalesun-{name}", max_position=P)
        km = HybridDecoder(cfg, kalesun.pack_weights(cfg, kalesun.random_tensors(cfg, 0), dev, torch.bfloat16), dev, P,
                           torch.bfloat16)
        entry = dict(kalesun=dict(params=cfg.param_count(), **_model_steps(km, dev, seqs, plen, rows, ctx)))
        _say(f"size {name}: kalesun {entry['kalesun']}")
        del km
        zcfg = zokunex.config_from_dict(zokunex_config(zsize), name=f"zokunex-{name}", max_position=P)
        zk = HybridDecoder(zcfg, zokunex.pack_weights(zcfg, zokunex.random_tensors(zcfg, 0), dev, torch.bfloat16), dev, P,
                           torch.bfloat16)
        entry["zokunex"] = dict(params=zcfg.param_count(), **_model_steps(zk, dev, seqs, plen, rows, ctx))
        _say(f"  zokunex {entry['zokunex']}")
        del zk
        d = size["width"]
        lc = llama.LlamaConfig(name=f"llama-{name}", vocab_size=VOCAB, hidden_size=d, intermediate_size=int(3.5 * d),
                               num_layers=LAYERS, num_heads=d // 128, num_kv_heads=max(1, d // 512), max_position=P)
        lm = llama.LlamaModel(lc, llama.random_weights(lc, None, dev, 0), None, dev, P)
        entry["llama"] = dict(params=lc.param_count(), **_model_steps(lm, dev, seqs, plen, rows, ctx))
        _say(f"  llama {entry['llama']}")
        del lm
        torch.cuda.empty_cache()
        entry["kernels"] = _kernels_kalesun(size, zsize, dev, seqs * plen, ctx, rows)
        entry["seconds"] = round(time.time() - t0, 1)
        res[name] = entry
        torch.cuda.empty_cache()
    return dict(metric="design_compare", design="kalesun", beside="zokunex and llama (equal width and depth)",
                layers=LAYERS, workload=dict(prefill=f"{seqs} x {plen} tokens in one step",
                                             decode=f"{rows} rows at context {ctx}"),
                dtype="bf16", data="synthetic", sizes=res)


def run(sizes: list, seqs: int = 4, plen: int = 2048, rows: int = 64, ctx: int = 2048, device: str = "cuda") -> dict:
    from chronos import ops
    from chronos.models import llama, zokunex
    from chronos.models.hybrid import HybridDecoder

    dev = torch.device(device if ":" in device else device + ":0")
    torch.cuda.set_device(dev)
    ops.load()
    ops.device_init()
    res = {}
    for name in sizes:
        size = SIZES[name]
        t0 = time.time()
        cfg = zokunex.config_from_dict(zokunex_config(size), name=f"zokunex-{name}", max_position=ctx + plen + 16)
        zk = HybridDecoder(cfg, zokunex.pack_weights(cfg, zokunex.random_tensors(cfg, 0), dev, torch.bfloat16), dev,
                           ctx + plen + 16, torch.bfloat16)
        d = size["width"]
        lc = llama.LlamaConfig(name=f"llama-{name}", vocab_size=VOCAB, hidden_size=d, intermediate_size=int(3.5 * d),
                               num_layers=LAYERS, num_heads=d // 128, num_kv_heads=max(1, d // 512),
                               max_position=ctx + plen + 16)
        lm = llama.LlamaModel(lc, llama.random_weights(lc, None, dev, 0), None, dev, ctx + plen + 16)
        _say(f"size {name}: models built")
        entry = dict(zokunex=dict(params=cfg.param_count(), **_model_steps(zk, dev, seqs, plen, rows, ctx)))
        _say(f"  zokunex {entry['zokunex']}")
        entry["llama"] = dict(params=lc.param_count(), **_model_steps(lm, dev, seqs, plen, rows, ctx))
        _say(f"  llama {entry['llama']}")
        entry["kernels"] = _kernels(size, dev, seqs * plen, ctx, rows)
        entry["seconds"] = round(time.time() - t0, 1)
        res[name] = entry
        del zk, lm
        torch.cuda.empty_cache()
    return dict(metric="design_compare", design="zokunex", beside="llama (equal width and depth)", layers=LAYERS,
                workload=dict(prefill=f"{seqs} x {plen} tokens in one step", decode=f"{rows} rows at context {ctx}"),
                dtype="bf16", data="synthetic", sizes=res)


def main(a) -> int:
    sizes = [s for s in a.design_sizes.split(",") if s]
    fn = {"kalesun": run_kalesun, "tugovik": run_tugovik, "vogerax": run_vogerax}.get(getattr(a, "design", "zokunex"), run)
    out = fn(sizes, device=a.device)
    print(json.dumps(out), flush=True)
    return 0
