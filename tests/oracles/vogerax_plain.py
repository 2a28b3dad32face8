"""A plain, slow Vogerax forward: one function per mechanism, written token by token from the design's equations.

It is the oracle the framework's Vogerax path is tested against and shares no code with it.  Everything is computed
in float64 from whatever weights it is given (a dict name -> tensor with the checkpoint's tensor names, and the parsed
config.json dict).  Sequences are processed one token at a time; caches and states are plain Python lists and tensors.
"""
from __future__ import annotations

import math

import torch

F = torch.float64


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + torch.exp(-z))


def silu(z):
    return z * sigmoid(z)


def group_norm(x, w, groups, eps):
    """x split into ``groups`` equal consecutive parts, each divided by its own root mean square; times w."""
    n = x.numel() // groups
    parts = [rms_unit(x[g * n:(g + 1) * n], eps) for g in range(groups)]
    return torch.cat(parts) * w


def frequencies(rot, dims=None):
    """Angle per position of every pair of a rotation, and the factor on cos and sin."""
    dims = dims or rot["dims"]
    base = float(rot["base"])
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    sc = rot.get("scaling")
    mag = 1.0
    if sc and "original" in sc:        # interpolation between scaled and unscaled frequencies along a ramp
        factor, orig = float(sc["factor"]), float(sc["original"])

        def where(turns):
            return dims * math.log(orig / (2 * math.pi * turns)) / (2 * math.log(base))

        lo = max(math.floor(where(float(sc["fast"]))), 0)
        hi = min(math.ceil(where(float(sc["slow"]))), dims - 1)
        out = []
        for i, fi in enumerate(f):
            ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
            out.append(fi / factor * ramp + fi * (1.0 - ramp))
        f = out
        mag = 0.1 * math.log(factor) + 1.0
    elif sc:                           # every frequency divided by the factor
        f = [fi / float(sc["factor"]) for fi in f]
    return f, mag


def rotate(x, pos, f, mag=1.0):
    """x [..., n]: the first 2 len(f) entries turn, entry i with entry i + len(f), by pos * f[i]."""
    half = len(f)
    c = torch.tensor([math.cos(pos * fi) * mag for fi in f], dtype=F)
    s = torch.tensor([math.sin(pos * fi) * mag for fi in f], dtype=F)
    u, v = x[..., :half], x[..., half:2 * half]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., 2 * half:]], -1)


def pooled_window_sets(i, size, pool):
    """(token positions, block indices) the query at position i sees: the window's tokens, and every block of
    ``pool`` positions that ends at or before i - size."""
    toks = [j for j in range(i + 1) if i - j < size]
    blocks = []
    if pool:
        b = 0
        while b * pool + pool - 1 <= i - size:
            blocks.append(b)
            b += 1
    return toks, blocks


def attention_token(h, W, p, mx, pos, state):
    """Grouped-query attention whose values are the unrotated keys, through a sliding window with pooled blocks.
    state["kv"]: list of (rotated k [G, D], v [G, D]) of all earlier tokens, this token's pair is appended;
    state["pooled"]: the means of the blocks seen so far (a block's mean never changes once all its tokens exist)."""
    H, G, D = mx["heads"], mx.get("kv_heads", mx["heads"]), mx["dim"]
    cache, pooled = state.setdefault("kv", []), state.setdefault("pooled", [])
    q = (W[p + "q"] @ h).view(H, D)
    k = (W[p + "k"] @ h).view(G, D)
    v = k.clone()
    rot = mx.get("rot")
    if rot:
        f, mag = frequencies(rot)
        q, k = rotate(q, pos, f, mag), rotate(k, pos, f, mag)
    cache.append((k, v))
    mask = mx.get("mask") or {}
    size, pool = mask.get("size", 0), mask.get("pool", 0)
    if size:
        toks, blocks = pooled_window_sets(pos, size, pool)
    else:
        toks, blocks = list(range(pos + 1)), []
    for b in blocks[len(pooled):]:
        pooled.append((torch.stack([cache[b * pool + r][0] for r in range(pool)]).mean(0),
                       torch.stack([cache[b * pool + r][1] for r in range(pool)]).mean(0)))
    keys = torch.stack([pooled[b][0] for b in blocks] + [cache[j][0] for j in toks])
    vals = torch.stack([pooled[b][1] for b in blocks] + [cache[j][1] for j in toks])
    out = torch.zeros(H, D, dtype=F)
    for hd in range(H):
        g = hd // (H // G)
        s = (keys[:, g] @ q[hd]) * mx["scale"]
        a = torch.softmax(s, 0)
        out[hd] = a @ vals[:, g]
    return W[p + "o"] @ out.reshape(-1)


def sink_attention_token(h, W, p, mx, eps, pos, cache):
    """Causal attention with per-head query/key norm, rotated keys AND values, a sink in the softmax and an
    element-wise sigmoid gate.  cache: list of (k [G, D], rotated v [G, Dv])."""
    H, G, D, Dv = mx["heads"], mx.get("kv_heads", mx["heads"]), mx["dim"], mx["vdim"]
    q = (W[p + "q"] @ h).view(H, D)
    k = (W[p + "k"] @ h).view(G, D)
    v = (W[p + "v"] @ h).view(G, Dv)
    q = rms_unit(q, eps) * W[p + "q.norm"]
    k = rms_unit(k, eps) * W[p + "k.norm"]
    f, mag = frequencies(mx["rot"])
    q, k = rotate(q, pos, f, mag), rotate(k, pos, f, mag)
    fv, _ = frequencies(dict(base=mx["rot"]["base"]), Dv)
    cache.append((k, rotate(v, pos, fv)))
    keys = torch.stack([c[0] for c in cache])
    vals = torch.stack([c[1] for c in cache])
    out = torch.zeros(H, Dv, dtype=F)
    for hd in range(H):
        g = hd // (H // G)
        s = (keys[:, g] @ q[hd]) * mx["scale"]
        m = max(float(s.max()), float(W[p + "sink"][hd]))
        e = torch.exp(s - m)
        den = e.sum() + math.exp(float(W[p + "sink"][hd]) - m)
        out[hd] = rotate((e / den) @ vals[:, g], -pos, fv)
    out = out.reshape(-1) * sigmoid(W[p + "g"] @ h)
    return W[p + "o"] @ out


def retention_token(h, W, p, mx, eps, pos, state):
    """Linear attention with one fixed decay per head.  state: dict with "S" [H, D, Dv]."""
    H, D, Dv = mx["heads"], mx["dim"], mx["vdim"]
    q = (W[p + "q"] @ h).view(H, D)
    k = (W[p + "k"] @ h).view(H, D)
    v = (W[p + "v"] @ h).view(H, Dv)
    if mx.get("rot"):
        f, mag = frequencies(mx["rot"])
        q, k = rotate(q, pos, f, mag), rotate(k, pos, f, mag)
    k = k * D ** -0.5
    if "S" not in state:
        state["S"] = torch.zeros(H, D, Dv, dtype=F)
    decay = torch.tensor(mx["decay"], dtype=F)
    S = decay[:, None, None] * state["S"] + k[:, :, None] * v[:, None, :]
    state["S"] = S
    o = torch.einsum("hdv,hd->hv", S, q)
    o = rms_unit(o, eps).reshape(-1) * silu(W[p + "g"] @ h)
    return W[p + "o"] @ o


def parallel_token(h, W, p, mx, eps, pos, state):
    """Two mixers on the same input; each output RMS-normed over the width with its own weight, then averaged."""
    left = sink_attention_token(h, W, p + "left.", mx["left"], eps, pos, state.setdefault("left", []))
    right = retention_token(h, W, p + "right.", mx["right"], eps, pos, state.setdefault("right", {}))
    return 0.5 * (rms_unit(left, eps) * W[p + "left.out"] + rms_unit(right, eps) * W[p + "right.out"])


def expert(h, W, p):
    return W[p + "down"] @ (torch.relu(W[p + "up"] @ h) ** 2)


def moe_token(h, W, p, mlp):
    r = mlp["router"]
    s = torch.softmax(W[p + "router"] @ h, 0)
    order = sorted(range(r["experts"]), key=lambda e: (-float(s[e]), e))[:r["top"]]
    y = torch.zeros_like(h)
    for e in order:
        y = y + s[e] * expert(h, W, p + f"e{e}.")
    if mlp.get("shared"):
        y = y + expert(h, W, p + "shared.")
    return y


def ff_token(h, W, p, mlp):
    if mlp.get("kind", "dense") == "dense":
        return expert(h, W, p)
    return moe_token(h, W, p, mlp)


class PlainVogerax:
    """One sequence, fed token by token; keeps every layer's cache and state."""

    def __init__(self, cfg: dict, tensors: dict):
        self.cfg = cfg
        self.W = {k: v.to(F) for k, v in tensors.items() if v.dtype.is_floating_point}
        self.states = [dict() for _ in cfg["layers"]]
        self.pos = 0

    def step(self, tok: int):
        """(logits [vocab], the residual stream after every layer run [runs][width]) of the next token."""
        cfg, W = self.cfg, self.W
        eps, groups = float(cfg["norm"]["eps"]), int(cfg["norm"].get("groups", 1))
        pos = self.pos
        per_layer = []
        x = W["embed"][tok] * float((cfg.get("embedding") or {}).get("scale", 1.0))
        for i, l in enumerate(cfg["layers"]):
            p = f"l{l.get('weights_of', i)}."
            st = self.states[i]
            h = group_norm(x, W[p + "norm1"], groups, eps)
            if l["type"] == "attention":
                y = attention_token(h, W, p + "mix.", l["mixer"], pos, st)
            elif l["type"] == "parallel":
                y = parallel_token(h, W, p + "mix.", l["mixer"], eps, pos, st)
            else:
                raise ValueError(l["type"])
            x = x + group_norm(y, W[p + "norm1b"], groups, eps)
            if l.get("mlp"):
                h = group_norm(x, W[p + "norm2"], groups, eps)
                x = x + group_norm(ff_token(h, W, p + "mlp.", l["mlp"]), W[p + "norm2b"], groups, eps)
            per_layer.append(x.clone())
        self.pos += 1
        return W["head"] @ group_norm(x, W["final.norm"], groups, eps), per_layer


def run(cfg: dict, tensors: dict, tokens, taps=None):
    """Logits [len(tokens), vocab] (float64) of one sequence.  ``taps``: a list that receives the residual stream after
    every layer run, [runs] of [tokens, width]."""
    m = PlainVogerax(cfg, tensors)
    out, per_layer = [], [[] for _ in cfg["layers"]]
    for tok in tokens:
        logits, xs = m.step(int(tok))
        out.append(logits)
        for i, x in enumerate(xs):
            per_layer[i].append(x)
    if taps is not None:
        taps.extend(torch.stack(r) for r in per_layer)
    return torch.stack(out)
