"""Vogerax: a hybrid decoder on a sandwich residual stream (x <- x + N_b(sublayer(N_a(x))), every N an RMS norm over
equal parts of the row) whose layers mix tokens either with grouped-query attention whose values are the unrotated
keys, seen through a sliding window plus one pooled key and value per block of positions before the window, or with
two mixers side by side — causal attention with query/key norm, ramp-scaled rotation, rotated values, a softmax sink
and a sigmoid gate per output column, beside retention (linear attention with a fixed decay per head) — whose normed
outputs are averaged; and feed forward through a squared-ReLU unit, dense or as a mixture of experts behind a softmax
router (plain scores as weights) plus a shared expert.  A layer may run on another layer's weights.

This module is the design's reader: ``config.json`` -> :class:`chronos.models.hybrid.HybridConfig`, the checkpoint's
tensor names -> the packed weights the hybrid kernels take, and random weights of the same shapes for benchmarks and
tests.  Everything computed lives in :mod:`chronos.models.hybrid` and :mod:`chronos.ops.hybrid`.

config.json:  architecture "Vogerax"; vocab, width, norm{eps, groups}, embedding{scale};
              layers[i] = {type, mixer{...}, mlp|null, weights_of?}
  type "attention":  mixer {heads, kv_heads, dim, vdim, scale, mask{size, pool}, rot{base, dims, scaling{factor}}}
  type "parallel":   mixer {left {heads, kv_heads, dim, vdim, scale,
                                  rot{base, dims, scaling{factor, original, fast, slow}}},
                            right {heads, dim, vdim, decay[heads], rot{base, dims}}}
  mlp {kind "dense", ff} | {kind "moe", expert{ff}, router{experts, top}, shared{ff}}
tensors (bfloat16, [out, in]):  embed, head, final.norm, l<i>.norm1 / norm1b / norm2 / norm2b, l<i>.mix.*, l<i>.mlp.*
"""
from __future__ import annotations

import json
import os

import torch

from ..ops import hybrid as hops
from .hybrid import (FEED_FORWARDS, MIXERS, DenseFFSpec, HybridConfig, HybridDecoder, HybridLayerWeights, HybridWeights,
                     LayerSpec, MoEFFSpec, ParallelSpec, RetentionSpec, WindowAttentionSpec)
from .zokunex import _SafetensorsDir

ARCHITECTURE = "Vogerax"


def _rot(rot: dict | None, width: int, where: str):
    """(base, dims, scaling tuple) of a mixer's ``rot`` entry; a scaling with ``original`` is the ramp form."""
    if not rot or not int(rot.get("dims", 0)):
        return 10000.0, 0, None
    dims = int(rot["dims"])
    if dims % 2 or dims > width:
        raise ValueError(f"{where}: rot.dims must be even and at most dim")
    sc = rot.get("scaling")
    if sc and "original" in sc:
        scaling = ("ramp", float(sc["factor"]), float(sc["original"]), float(sc["fast"]), float(sc["slow"]))
    elif sc:
        scaling = ("linear", float(sc["factor"]))
    else:
        scaling = None
    return float(rot["base"]), dims, scaling


def _pooled_attention(mx: dict, where: str) -> WindowAttentionSpec:
    heads = int(mx["heads"])
    base, dims, scaling = _rot(mx.get("rot"), int(mx["dim"]), where)
    mask = mx.get("mask") or {}
    spec = WindowAttentionSpec(heads, int(mx.get("kv_heads", heads)), int(mx["dim"]), int(mx.get("vdim", mx["dim"])),
                               float(mx["scale"]), window=int(mask.get("size", 0)), rope_base=base, rope_dims=dims,
                               rope_scaling=scaling, qk_norm=False, sink=False, gate=False,
                               pool=int(mask.get("pool", 0)), v_from_k=True)
    if spec.heads % spec.kv_heads:
        raise ValueError(f"{where}: heads must be a multiple of kv_heads")
    if spec.vdim != spec.dim:
        raise ValueError(f"{where}: the values are the keys, so vdim must equal dim")
    return spec


def _sink_attention(mx: dict, where: str) -> WindowAttentionSpec:
    heads = int(mx["heads"])
    base, dims, scaling = _rot(mx.get("rot"), int(mx["dim"]), where)
    spec = WindowAttentionSpec(heads, int(mx.get("kv_heads", heads)), int(mx["dim"]), int(mx["vdim"]),
                               float(mx["scale"]), rope_base=base, rope_dims=dims, rope_scaling=scaling, qk_norm=True,
                               sink=True, gate=True, gate_wide=True, v_rot=True)
    if spec.heads % spec.kv_heads:
        raise ValueError(f"{where}: heads must be a multiple of kv_heads")
    if spec.vdim % 2:
        raise ValueError(f"{where}: rotated values need an even vdim")
    return spec


def _retention(mx: dict, where: str) -> RetentionSpec:
    base, dims, scaling = _rot(mx.get("rot"), int(mx["dim"]), where)
    spec = RetentionSpec(int(mx["heads"]), int(mx["dim"]), int(mx["vdim"]), tuple(float(v) for v in mx["decay"]),
                         base, dims, scaling)
    if len(spec.decay) != spec.heads:
        raise ValueError(f"{where}: one decay per head")
    return spec


def config_from_dict(c: dict, name: str = "vogerax", max_position: int = 8192) -> HybridConfig:
    layers, share = [], []
    for i, l in enumerate(c["layers"]):
        mx = l["mixer"]
        if l["type"] == "attention":
            mixer = _pooled_attention(mx, f"layer {i}")
        elif l["type"] == "parallel":
            mixer = ParallelSpec(_sink_attention(mx["left"], f"layer {i} left"), _retention(mx["right"], f"layer {i} right"))
        else:
            raise ValueError(f"layer {i}: unknown mixer type {l['type']!r}")
        mlp = l.get("mlp")
        if mlp is None:
            ff = None
        elif mlp.get("kind", "dense") == "dense":
            ff = DenseFFSpec(int(mlp["ff"]), hops.ACT_RELU2)
        elif mlp["kind"] == "moe":
            r = mlp["router"]
            ff = MoEFFSpec(int(r["experts"]), 0, int(r["top"]), int(mlp["expert"]["ff"]), hops.ACT_RELU2,
                           int((mlp.get("shared") or {}).get("ff", 0)), correction=False)
            if not 1 <= ff.top <= ff.experts:
                raise ValueError(f"layer {i}: router picks more experts than it has")
        else:
            raise ValueError(f"layer {i}: unknown feed-forward kind {mlp['kind']!r}")
        layers.append(LayerSpec(mixer, ff))
        j = int(l.get("weights_of", i))
        if not 0 <= j <= i or (j < i and share[j] != j):
            raise ValueError(f"layer {i}: weights_of must name an earlier layer with weights of its own")
        share.append(j)
    groups = int(c["norm"].get("groups", 1))
    if int(c["width"]) % groups:
        raise ValueError("width must be a multiple of norm.groups")
    return HybridConfig(name=name, vocab_size=int(c["vocab"]), hidden_size=int(c["width"]), layers=layers,
                        norm_eps=float(c["norm"]["eps"]), max_position=max_position, architecture=ARCHITECTURE,
                        residual="sandwich", norm_groups=groups,
                        embed_scale=float((c.get("embedding") or {}).get("scale", 1.0)),
                        share=share if any(j != i for i, j in enumerate(share)) else None)


def _rot_dict(m) -> dict | None:
    if not m.rope_dims:
        return None
    out = dict(base=m.rope_base, dims=m.rope_dims)
    if m.rope_scaling and m.rope_scaling[0] == "ramp":
        out["scaling"] = dict(zip(("factor", "original", "fast", "slow"), m.rope_scaling[1:]))
    elif m.rope_scaling:
        out["scaling"] = dict(factor=m.rope_scaling[1])
    return out


def config_to_dict(cfg: HybridConfig) -> dict:
    """The config.json form of a configuration (what :func:`config_from_dict` reads)."""
    layers = []
    for i, l in enumerate(cfg.layers):
        m = l.mixer
        if m.kind == "window_attention":
            mixer = dict(heads=m.heads, kv_heads=m.kv_heads, dim=m.dim, vdim=m.vdim, scale=m.scale)
            if m.window:
                mixer["mask"] = dict(size=m.window, pool=m.pool)
            if m.rope_dims:
                mixer["rot"] = _rot_dict(m)
            typ = "attention"
        else:
            a, r = m.left, m.right
            left = dict(heads=a.heads, kv_heads=a.kv_heads, dim=a.dim, vdim=a.vdim, scale=a.scale, rot=_rot_dict(a))
            right = dict(heads=r.heads, dim=r.dim, vdim=r.vdim, decay=list(r.decay))
            if r.rope_dims:
                right["rot"] = _rot_dict(r)
            mixer, typ = dict(left=left, right=right), "parallel"
        f = l.ff
        if f is None:
            mlp = None
        elif f.kind == "dense":
            mlp = dict(kind="dense", ff=f.ff)
        else:
            mlp = dict(kind="moe", expert=dict(ff=f.ff), router=dict(experts=f.experts, top=f.top))
            if f.shared_ff:
                mlp["shared"] = dict(ff=f.shared_ff)
        entry = dict(type=typ, mixer=mixer, mlp=mlp)
        if cfg.share is not None and cfg.share[i] != i:
            entry["weights_of"] = cfg.share[i]
        layers.append(entry)
    return dict(architecture=ARCHITECTURE, vocab=cfg.vocab_size, width=cfg.hidden_size,
                norm=dict(eps=cfg.norm_eps, groups=cfg.norm_groups), embedding=dict(scale=cfg.embed_scale),
                layers=layers)


def tensor_shapes(cfg: HybridConfig) -> dict:
    """Checkpoint tensor name -> shape (layers that run on another layer's weights have none)."""
    d, V = cfg.hidden_size, cfg.vocab_size
    out = {"embed": (V, d)}
    own = set(cfg.runs)
    for i, l in enumerate(cfg.layers):
        if i not in own:
            continue
        m, p = l.mixer, f"l{i}."
        out.update({p + "norm1": (d,), p + "norm1b": (d,)})
        if l.ff is not None:
            out.update({p + "norm2": (d,), p + "norm2b": (d,)})
        if m.kind == "window_attention":
            out.update({p + "mix.q": (m.heads * m.dim, d), p + "mix.k": (m.kv_heads * m.dim, d),
                        p + "mix.o": (d, m.heads * m.vdim)})
        else:
            a, r = m.left, m.right
            q = p + "mix.left."
            out.update({q + "q": (a.heads * a.dim, d), q + "k": (a.kv_heads * a.dim, d), q + "v": (a.kv_heads * a.vdim, d),
                        q + "q.norm": (a.dim,), q + "k.norm": (a.dim,), q + "sink": (a.heads,),
                        q + "g": (a.heads * a.vdim, d), q + "o": (d, a.heads * a.vdim)})
            q = p + "mix.right."
            out.update({q + "q": (r.heads * r.dim, d), q + "k": (r.heads * r.dim, d), q + "v": (r.heads * r.vdim, d),
                        q + "g": (r.heads * r.vdim, d), q + "o": (d, r.heads * r.vdim)})
            out.update({p + "mix.left.out": (d,), p + "mix.right.out": (d,)})
        f = l.ff
        if f is not None and f.kind == "dense":
            out.update({p + "mlp.up": (f.ff, d), p + "mlp.down": (d, f.ff)})
        elif f is not None:
            for e in range(f.experts):
                out.update({p + f"mlp.e{e}.up": (f.ff, d), p + f"mlp.e{e}.down": (d, f.ff)})
            out[p + "mlp.router"] = (f.experts, d)
            if f.shared_ff:
                out.update({p + "mlp.shared.up": (f.shared_ff, d), p + "mlp.shared.down": (d, f.shared_ff)})
    out["final.norm"] = (d,)
    out["head"] = (V, d)
    return out


def random_tensors(cfg: HybridConfig, seed: int = 0, device="cpu", std: float | None = None) -> dict:
    """Checkpoint-named random bfloat16 tensors: norm weights around one (those on the sublayers' outputs smaller, so
    that the stream grows slowly), sinks around zero, matrices at 1/sqrt(fan-in)."""
    gen = torch.Generator(device="cpu")
    gen.manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.rsplit(".", 1)[-1]
        rn = lambda s=1.0: torch.randn(shape, generator=gen) * s  # noqa: E731
        if leaf in ("norm1b", "norm2b"):
            t = rn(0.1) + 0.5
        elif leaf == "sink":
            t = rn(1.0)
        elif len(shape) == 1:
            t = rn(0.1) + 1.0
        else:
            t = rn(std if std is not None else shape[1] ** -0.5)
        out[name] = t.to(torch.bfloat16).to(device)
    return out


def pack_weights(cfg: HybridConfig, tensors, device, act_dtype) -> HybridWeights:
    """``tensors``: a mapping (or any object with ``__getitem__``) from checkpoint names to tensors.  Norm weights are
    served as float32.  A layer that runs on another layer's weights gets that layer's packed weights (one copy)."""
    a = lambda x: x.to(device=device, dtype=act_dtype).contiguous()  # noqa: E731
    f = lambda x: x.to(device=device, dtype=torch.float32).contiguous()  # noqa: E731
    shapes = tensor_shapes(cfg)

    def get(name):
        t = tensors[name]
        if tuple(t.shape) != tuple(shapes[name]):
            raise ValueError(f"tensor {name}: shape {tuple(t.shape)}, the configuration says {tuple(shapes[name])}")
        return t

    layers: list = []
    for i, (l, j) in enumerate(zip(cfg.layers, cfg.runs)):
        if j != i:
            layers.append(layers[j])
            continue
        p = f"l{i}.mix."
        names = [n[len(p):] for n in shapes if n.startswith(p)]
        mix = MIXERS[l.mixer.kind][1](l.mixer, {n: get(p + n) for n in names}, device, act_dtype)
        lw = HybridLayerWeights(f(get(f"l{i}.norm1")), mix, norm1b=f(get(f"l{i}.norm1b")))
        if l.ff is not None:
            p = f"l{i}.mlp."
            names = [n[len(p):] for n in shapes if n.startswith(p)]
            lw.norm2, lw.norm2b = f(get(f"l{i}.norm2")), f(get(f"l{i}.norm2b"))
            lw.ff = FEED_FORWARDS[l.ff.kind][1](l.ff, {n: get(p + n) for n in names}, device, act_dtype)
        layers.append(lw)
    return HybridWeights(a(get("embed")), layers, f(get("final.norm")), a(get("head")))


def is_checkpoint(path: str) -> bool:
    cj = os.path.join(path, "config.json")
    if not os.path.exists(cj):
        return False
    with open(cj) as fh:
        return json.load(fh).get("architecture") == ARCHITECTURE


def load(path: str, device="cpu", act_dtype=torch.bfloat16, max_position: int | None = None) -> HybridDecoder:
    with open(os.path.join(path, "config.json")) as fh:
        cfg = config_from_dict(json.load(fh), name=os.path.basename(path.rstrip("/")) or "vogerax",
                               max_position=max_position or 8192)
    return HybridDecoder(cfg, pack_weights(cfg, _SafetensorsDir(path), device, act_dtype), device, max_position,
                         act_dtype)


def save(cfg: HybridConfig, tensors: dict, path: str) -> None:
    """Write config.json + model.safetensors (bfloat16) — the layout :func:`load` reads."""
    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as fh:
        json.dump(config_to_dict(cfg), fh, indent=1)
    save_file({k: v.to(torch.bfloat16).cpu().contiguous() for k, v in tensors.items()},
              os.path.join(path, "model.safetensors"))


def _preset(width, vocab, pattern, heads, kv_heads, dim, window, pool, rheads, rdim, rvdim, ff, experts, top, eff, sff,
            groups=4, share=None) -> dict:
    """pattern: one letter per layer — a = pooled-window attention, p = parallel (sink attention beside retention);
    upper case = dense feed-forward, lower = mixture of experts.  share: {layer: layer whose weights it uses}."""
    import math

    layers = []
    for i, ch in enumerate(pattern):
        if ch.lower() == "a":
            mixer, typ = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=dim ** -0.5,
                              mask=dict(size=window, pool=pool),
                              rot=dict(base=5e5, dims=dim // 2, scaling=dict(factor=4.0))), "attention"
        else:
            left = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=dim ** -0.5,
                        rot=dict(base=1e5, dims=dim // 2, scaling=dict(factor=8.0, original=4096, fast=16.0, slow=2.0)))
            # memory spans of 16 to 2048 tokens, spread geometrically over the heads
            right = dict(heads=rheads, dim=rdim, vdim=rvdim, rot=dict(base=1e4, dims=rdim),
                         decay=[math.exp(-1.0 / (16.0 * 128.0 ** (h / max(1, rheads - 1)))) for h in range(rheads)])
            mixer, typ = dict(left=left, right=right), "parallel"
        mlp = dict(kind="dense", ff=ff) if ch.isupper() else dict(
            kind="moe", expert=dict(ff=eff), shared=dict(ff=sff), router=dict(experts=experts, top=top))
        entry = dict(type=typ, mixer=mixer, mlp=mlp)
        if share and i in share:
            entry["weights_of"] = share[i]
        layers.append(entry)
    return dict(architecture=ARCHITECTURE, vocab=vocab, width=width, norm=dict(eps=1e-6, groups=groups),
                embedding=dict(scale=8.0), layers=layers)


# random-init presets (benchmarks, smoke runs); sizes in the range of real models' layers
PRESETS = {
    "vogerax-tiny": _preset(128, 512, "ApAp", 4, 2, 32, 24, 8, 2, 32, 16, 256, 6, 2, 64, 64, share={2: 0}),
    "vogerax-1b": _preset(2048, 32768, "ApapaPap", 16, 4, 128, 1024, 64, 16, 128, 128, 8192, 16, 4, 1024, 2048),
    "vogerax-8b-layers": _preset(4096, 128256, "Apap", 32, 8, 128, 2048, 64, 32, 128, 128, 14336, 32, 4, 2048, 4096),
}


def build(name_or_path: str, device="cpu", seed: int = 0, act_dtype=torch.bfloat16,
          max_position: int | None = None) -> HybridDecoder:
    if os.path.isdir(name_or_path):
        return load(name_or_path, device, act_dtype, max_position)
    cfg = config_from_dict(PRESETS[name_or_path], name=name_or_path, max_position=max_position or 8192)
    w = pack_weights(cfg, random_tensors(cfg, seed), device, act_dtype)
    return HybridDecoder(cfg, w, device, max_position, act_dtype)
