"""Tugovik: a hybrid decoder on a pre-norm residual stream (x <- x + sublayer(rms_norm(x) (1 + w))) whose layers mix
tokens with chunked grouped-query attention (biased projections, no rotation, keys visible only inside the query's
own chunk of positions), with a state-space-duality layer (Mamba-2) or with a real-gated linear recurrent unit, feed
forward through a mixture of gated experts behind a sigmoid router whose choice is limited to the best groups of
experts, plus a shared expert with its own sigmoid gate, and add after every layer a gated projection of the token's
row in a second embedding table.  A range of layers may repeat, back to back, on shared weights.

This module is the design's reader: ``config.json`` -> :class:`chronos.models.hybrid.HybridConfig`, the checkpoint's
tensor names -> the packed weights the hybrid kernels take, and random weights of the same shapes for benchmarks and
tests.  Everything computed lives in :mod:`chronos.models.hybrid` and :mod:`chronos.ops.hybrid`.

config.json:  architecture "Tugovik"; vocab, width, norm.eps; token_side{dim}; loop{start, stop, times};
              layers[i] = {type, mixer{...}, mlp|null}
  type "attention":  mixer {heads, kv_heads, dim, vdim, scale, mask{size}}
  type "mamba2":     mixer {heads, vdim, state, groups, conv, norm_groups}
  type "rglru":      mixer {width, blocks, conv}
  mlp {kind "moe", expert{ff}, router{experts, top, scale, groups{count, keep}}, shared{ff}}
tensors (bfloat16, [out, in]):  embed, head, final.norm, side.embed, l<i>.norm1, l<i>.norm2, l<i>.mix.*, l<i>.mlp.*,
                                l<i>.side.gate / .proj / .norm
"""
from __future__ import annotations

import json
import os

import torch

from .hybrid import (FEED_FORWARDS, MIXERS, HybridConfig, HybridDecoder, HybridLayerWeights, HybridWeights, LayerSpec,
                     Mamba2Spec, MoEGroupGluSpec, RGLRUSpec, WindowAttentionSpec)
from .zokunex import _SafetensorsDir

ARCHITECTURE = "Tugovik"
RGLRU_C = 8.0   # log a = -8 r softplus(lam): fixed by the design


def config_from_dict(c: dict, name: str = "tugovik", max_position: int = 8192) -> HybridConfig:
    layers = []
    for i, l in enumerate(c["layers"]):
        mx = l["mixer"]
        if l["type"] == "attention":
            heads = int(mx["heads"])
            mixer = WindowAttentionSpec(heads, int(mx.get("kv_heads", heads)), int(mx["dim"]), int(mx["vdim"]),
                                        float(mx["scale"]), chunk=int((mx.get("mask") or {}).get("size", 0)),
                                        qk_norm=False, sink=False, gate=False, bias=True)
            if mixer.heads % mixer.kv_heads:
                raise ValueError(f"layer {i}: heads must be a multiple of kv_heads")
        elif l["type"] == "mamba2":
            mixer = Mamba2Spec(int(mx["heads"]), int(mx["vdim"]), int(mx["state"]), int(mx.get("groups", 1)),
                               int(mx["conv"]), int(mx.get("norm_groups", 1)))
            if mixer.heads % mixer.groups or mixer.inner % mixer.norm_groups or mixer.conv < 1:
                raise ValueError(f"layer {i}: heads must be a multiple of groups, heads * vdim of norm_groups")
        elif l["type"] == "rglru":
            mixer = RGLRUSpec(int(mx["width"]), int(mx.get("blocks", 1)), int(mx["conv"]), RGLRU_C)
            if mixer.width % mixer.blocks or mixer.conv < 1:
                raise ValueError(f"layer {i}: width must be a multiple of blocks")
        else:
            raise ValueError(f"layer {i}: unknown mixer type {l['type']!r}")
        mlp = l.get("mlp")
        if mlp is None:
            ff = None
        elif mlp.get("kind", "moe") == "moe":
            r = mlp["router"]
            grp = r.get("groups") or {}
            ff = MoEGroupGluSpec(int(r["experts"]), int(r["top"]), int(mlp["expert"]["ff"]), int(grp.get("count", 1)),
                                 int(grp.get("keep", grp.get("count", 1))), float(r.get("scale", 1.0)),
                                 int((mlp.get("shared") or {}).get("ff", 0)))
            if ff.experts % ff.groups or not 1 <= ff.keep <= ff.groups:
                raise ValueError(f"layer {i}: experts must split into equal groups, of which 1..count are kept")
            if not 1 <= ff.top <= ff.keep * (ff.experts // ff.groups):
                raise ValueError(f"layer {i}: router picks more experts than the kept groups hold")
        else:
            raise ValueError(f"layer {i}: unknown feed-forward kind {mlp['kind']!r}")
        layers.append(LayerSpec(mixer, ff))
    loop = c.get("loop")
    if loop:
        loop = (int(loop["start"]), int(loop["stop"]), int(loop.get("times", 1)))
        if not 0 <= loop[0] <= loop[1] <= len(layers) or loop[2] < 1:
            raise ValueError("loop: 0 <= start <= stop <= number of layers, times >= 1")
    return HybridConfig(name=name, vocab_size=int(c["vocab"]), hidden_size=int(c["width"]), layers=layers,
                        norm_eps=float(c["norm"]["eps"]), max_position=max_position, architecture=ARCHITECTURE,
                        residual="pre_norm", loop=loop, token_side=int((c.get("token_side") or {}).get("dim", 0)))


def config_to_dict(cfg: HybridConfig) -> dict:
    """The config.json form of a configuration (what :func:`config_from_dict` reads)."""
    layers = []
    for l in cfg.layers:
        m = l.mixer
        if m.kind == "window_attention":
            mixer = dict(heads=m.heads, kv_heads=m.kv_heads, dim=m.dim, vdim=m.vdim, scale=m.scale)
            if m.chunk:
                mixer["mask"] = dict(size=m.chunk)
            typ = "attention"
        elif m.kind == "mamba2":
            mixer, typ = dict(heads=m.heads, vdim=m.vdim, state=m.state, groups=m.groups, conv=m.conv,
                              norm_groups=m.norm_groups), "mamba2"
        else:
            mixer, typ = dict(width=m.width, blocks=m.blocks, conv=m.conv), "rglru"
        f = l.ff
        mlp = None
        if f is not None:
            mlp = dict(kind="moe", expert=dict(ff=f.ff), router=dict(experts=f.experts, top=f.top, scale=f.scale,
                                                                    groups=dict(count=f.groups, keep=f.keep)))
            if f.shared_ff:
                mlp["shared"] = dict(ff=f.shared_ff)
        layers.append(dict(type=typ, mixer=mixer, mlp=mlp))
    out = dict(architecture=ARCHITECTURE, vocab=cfg.vocab_size, width=cfg.hidden_size, norm=dict(eps=cfg.norm_eps),
               layers=layers)
    if cfg.loop:
        out["loop"] = dict(zip(("start", "stop", "times"), cfg.loop))
    if cfg.token_side:
        out["token_side"] = dict(dim=cfg.token_side)
    return out


def tensor_shapes(cfg: HybridConfig) -> dict:
    """Checkpoint tensor name -> shape."""
    d, V, sd = cfg.hidden_size, cfg.vocab_size, cfg.token_side
    out = {"embed": (V, d)}
    if sd:
        out["side.embed"] = (V, sd * len(cfg.layers))
    for i, l in enumerate(cfg.layers):
        m, p = l.mixer, f"l{i}."
        out[p + "norm1"] = (d,)
        if l.ff is not None:
            out[p + "norm2"] = (d,)
        if m.kind == "window_attention":
            out.update({p + "mix.q": (m.heads * m.dim, d), p + "mix.q.b": (m.heads * m.dim,),
                        p + "mix.k": (m.kv_heads * m.dim, d), p + "mix.k.b": (m.kv_heads * m.dim,),
                        p + "mix.v": (m.kv_heads * m.vdim, d), p + "mix.v.b": (m.kv_heads * m.vdim,),
                        p + "mix.o": (d, m.heads * m.vdim)})
        elif m.kind == "mamba2":
            out.update({p + "mix.in": (2 * m.inner + 2 * m.groups * m.state + m.heads, d),
                        p + "mix.conv": (m.conv_channels, m.conv), p + "mix.conv.b": (m.conv_channels,),
                        p + "mix.dt_bias": (m.heads,), p + "mix.A_log": (m.heads,), p + "mix.D": (m.heads,),
                        p + "mix.norm": (m.inner,), p + "mix.o": (d, m.inner)})
        else:
            bw = m.width // m.blocks
            out.update({p + "mix.y": (m.width, d), p + "mix.y.b": (m.width,), p + "mix.x": (m.width, d),
                        p + "mix.x.b": (m.width,), p + "mix.conv": (m.width, m.conv), p + "mix.conv.b": (m.width,),
                        p + "mix.ra": (m.blocks, bw, bw), p + "mix.ra.b": (m.blocks, bw),
                        p + "mix.ri": (m.blocks, bw, bw), p + "mix.ri.b": (m.blocks, bw), p + "mix.lam": (m.width,),
                        p + "mix.o": (d, m.width)})
        f = l.ff
        if f is not None:
            for e in range(f.experts):
                out.update({p + f"mlp.e{e}.gate": (f.ff, d), p + f"mlp.e{e}.up": (f.ff, d),
                            p + f"mlp.e{e}.down": (d, f.ff)})
            out[p + "mlp.router"] = (f.experts, d)
            if f.shared_ff:
                out.update({p + "mlp.shared.gate": (f.shared_ff, d), p + "mlp.shared.up": (f.shared_ff, d),
                            p + "mlp.shared.down": (d, f.shared_ff), p + "mlp.shared.sg": (1, d)})
        if sd:
            out.update({p + "side.gate": (sd, d), p + "side.proj": (d, sd), p + "side.norm": (d,)})
    out["final.norm"] = (d,)
    out["head"] = (V, d)
    return out


def random_tensors(cfg: HybridConfig, seed: int = 0, device="cpu", std: float | None = None) -> dict:
    """Checkpoint-named random bfloat16 tensors: the stream's norm weights around zero, the token input's norm around
    one, step biases and decay parameters in the range where the recurrent states neither vanish nor stand still."""
    gen = torch.Generator(device="cpu")
    gen.manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.split(".", 1)[1] if name.startswith("l") and "." in name else name
        rn = lambda s=1.0: torch.randn(shape, generator=gen) * s  # noqa: E731
        if leaf in ("mix.conv",):
            t = rn(0.5)
        elif leaf == "mix.A_log":
            t = torch.log(torch.rand(shape, generator=gen) * 3.0 + 0.5)
        elif leaf == "mix.dt_bias":
            t = rn(0.5) - 1.0
        elif leaf == "mix.D":
            t = rn(0.2) + 1.0
        elif leaf == "mix.lam":
            t = rn(0.7) - 1.5
        elif leaf in ("side.norm", "mix.norm"):
            t = rn(0.1) + 1.0
        elif len(shape) == 1 or leaf in ("mix.ra.b", "mix.ri.b"):
            t = rn(0.1)
        elif len(shape) == 3:
            t = rn(shape[2] ** -0.5)
        elif name == "side.embed":
            t = rn(1.0)
        else:
            t = rn(std if std is not None else shape[1] ** -0.5)
        out[name] = t.to(torch.bfloat16).to(device)
    return out


def pack_weights(cfg: HybridConfig, tensors, device, act_dtype) -> HybridWeights:
    """``tensors``: a mapping (or any object with ``__getitem__``) from checkpoint names to tensors.  The stream's
    norm weights are stored around zero and served as float32 1 + w."""
    a = lambda x: x.to(device=device, dtype=act_dtype).contiguous()  # noqa: E731
    f = lambda x: x.to(device=device, dtype=torch.float32).contiguous()  # noqa: E731
    one_plus = lambda x: (1.0 + x.to(device=device, dtype=torch.float32)).contiguous()  # noqa: E731
    shapes = tensor_shapes(cfg)

    def get(name):
        t = tensors[name]
        if tuple(t.shape) != tuple(shapes[name]):
            raise ValueError(f"tensor {name}: shape {tuple(t.shape)}, the configuration says {tuple(shapes[name])}")
        return t

    layers = []
    for i, l in enumerate(cfg.layers):
        p = f"l{i}.mix."
        names = [n[len(p):] for n in shapes if n.startswith(p)]
        mix = MIXERS[l.mixer.kind][1](l.mixer, {n: get(p + n) for n in names}, device, act_dtype)
        lw = HybridLayerWeights(one_plus(get(f"l{i}.norm1")), mix)
        if l.ff is not None:
            p = f"l{i}.mlp."
            names = [n[len(p):] for n in shapes if n.startswith(p)]
            lw.norm2 = one_plus(get(f"l{i}.norm2"))
            lw.ff = FEED_FORWARDS[l.ff.kind][1](l.ff, {n: get(p + n) for n in names}, device, act_dtype)
        if cfg.token_side:
            lw.side = dict(w_gate=a(get(f"l{i}.side.gate")), w_proj=a(get(f"l{i}.side.proj")),
                           norm=f(get(f"l{i}.side.norm")), col0=i * cfg.token_side)
        layers.append(lw)
    return HybridWeights(a(get("embed")), layers, one_plus(get("final.norm")), a(get("head")),
                         a(get("side.embed")) if cfg.token_side else None)


def is_checkpoint(path: str) -> bool:
    cj = os.path.join(path, "config.json")
    if not os.path.exists(cj):
        return False
    with open(cj) as fh:
        return json.load(fh).get("architecture") == ARCHITECTURE


def load(path: str, device="cpu", act_dtype=torch.bfloat16, max_position: int | None = None) -> HybridDecoder:
    with open(os.path.join(path, "config.json")) as fh:
        cfg = config_from_dict(json.load(fh), name=os.path.basename(path.rstrip("/")) or "tugovik",
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


def _preset(width, vocab, pattern, heads, kv_heads, dim, chunk, state, ssm_groups, rwidth, rblocks, experts, top,
            groups, keep, eff, sff, side, loop=None) -> dict:
    """pattern: one letter per layer — a = chunked attention, m = state-space layer, r = gated linear recurrence;
    upper case = no feed-forward, lower = mixture of experts."""
    layers = []
    for ch in pattern:
        k = ch.lower()
        if k == "a":
            mixer, typ = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=dim ** -0.5,
                              mask=dict(size=chunk)), "attention"
        elif k == "m":
            mixer, typ = dict(heads=2 * width // 64, vdim=64, state=state, groups=ssm_groups, conv=4,
                              norm_groups=ssm_groups), "mamba2"
        else:
            mixer, typ = dict(width=rwidth, blocks=rblocks, conv=4), "rglru"
        mlp = None if ch.isupper() else dict(
            kind="moe", expert=dict(ff=eff), shared=dict(ff=sff),
            router=dict(experts=experts, top=top, scale=2.5, groups=dict(count=groups, keep=keep)))
        layers.append(dict(type=typ, mixer=mixer, mlp=mlp))
    out = dict(architecture=ARCHITECTURE, vocab=vocab, width=width, norm=dict(eps=1e-6), layers=layers,
               token_side=dict(dim=side))
    if loop:
        out["loop"] = dict(zip(("start", "stop", "times"), loop))
    return out


# random-init presets (benchmarks, smoke runs); sizes in the range of real models' layers
PRESETS = {
    "tugovik-tiny": _preset(128, 512, "mar", 2, 1, 32, 24, 16, 1, 128, 2, 8, 2, 4, 2, 64, 64, 16, loop=(0, 2, 2)),
    "tugovik-1b": _preset(2048, 32768, "marAmara", 16, 4, 128, 1024, 128, 4, 2048, 8, 16, 4, 4, 2, 1024, 2048, 256),
    "tugovik-8b-layers": _preset(4096, 128256, "mara", 32, 8, 128, 4096, 128, 8, 4096, 16, 32, 4, 8, 4, 2048, 4096,
                                 256),
}


def build(name_or_path: str, device="cpu", seed: int = 0, act_dtype=torch.bfloat16,
          max_position: int | None = None) -> HybridDecoder:
    if os.path.isdir(name_or_path):
        return load(name_or_path, device, act_dtype, max_position)
    cfg = config_from_dict(PRESETS[name_or_path], name=name_or_path, max_position=max_position or 8192)
    w = pack_weights(cfg, random_tensors(cfg, seed), device, act_dtype)
    return HybridDecoder(cfg, w, device, max_position, act_dtype)

