"""A plain, slow Tugovik forward: one function per mechanism, written token by token from the design's equations.

It is the oracle the framework's Tugovik path is tested against and shares no code with it.  Everything is computed
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


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def offset_norm(x, w, eps):
    """RMS norm whose weight is stored around zero."""
    return rms_unit(x, eps) * (1.0 + w)


def chunk_visible(i, j, size):
    """May the query at position i see the key at position j?  Only inside its own chunk of ``size`` positions."""
    return j <= i and (not size or i // size == j // size)


def attention_token(h, W, p, mx, pos, cache):
    """One token of the chunked attention mixer.  cache: list of (k [G, D], v [G, Dv]) of ALL earlier tokens; this
    token's pair is appended."""
    H, G, D, Dv = mx["heads"], mx.get("kv_heads", mx["heads"]), mx["dim"], mx["vdim"]
    q = (W[p + "q"] @ h + W[p + "q.b"]).view(H, D)
    k = (W[p + "k"] @ h + W[p + "k.b"]).view(G, D)
    v = (W[p + "v"] @ h + W[p + "v.b"]).view(G, Dv)
    cache.append((k, v))
    size = (mx.get("mask") or {}).get("size", 0)
    out = torch.zeros(H, Dv, dtype=F)
    js = [j for j in range(pos + 1) if chunk_visible(pos, j, size)]
    keys = torch.stack([cache[j][0] for j in js])    # [n, G, D]
    vals = torch.stack([cache[j][1] for j in js])    # [n, G, Dv]
    for hd in range(H):
        g = hd // (H // G)
        sc = (keys[:, g] @ q[hd]) * mx["scale"]
        a = torch.exp(sc - sc.max())
        a = a / a.sum()
        out[hd] = a @ vals[:, g]
    return W[p + "o"] @ out.reshape(-1)


def conv_token(u, taps, bias, hist):
    """Causal per-channel convolution: hist holds the last taps - 1 inputs (oldest first; zeros before the start) and
    is updated; the last tap weighs the current input."""
    K = taps.shape[1]
    ext = hist + [u]
    y = bias.clone()
    for i in range(K):
        y = y + taps[:, i] * ext[i]
    hist[:] = ext[1:] if K > 1 else []
    return y


def mamba2_token(h, W, p, mx, eps, state):
    """One token of the state-space mixer.  state: dict with 'S' [heads, N, P] and 'hist' (list of conv inputs)."""
    Hn, P, N, G = mx["heads"], mx["vdim"], mx["state"], mx.get("groups", 1)
    inner = Hn * P
    zx = W[p + "in"] @ h
    z, xbc, dt = zx[:inner], zx[inner:2 * inner + 2 * G * N], zx[2 * inner + 2 * G * N:]
    xbc = silu(conv_token(xbc, W[p + "conv"], W[p + "conv.b"], state["hist"]))
    x = xbc[:inner].view(Hn, P)
    Bm = xbc[inner:inner + G * N].view(G, N)
    Cm = xbc[inner + G * N:].view(G, N)
    dt = softplus(dt + W[p + "dt_bias"])
    y = torch.zeros(Hn, P, dtype=F)
    for hd in range(Hn):
        g = hd // (Hn // G)
        decay = torch.exp(-torch.exp(W[p + "A_log"][hd]) * dt[hd])
        state["S"][hd] = decay * state["S"][hd] + dt[hd] * torch.outer(Bm[g], x[hd])
        y[hd] = state["S"][hd].t() @ Cm[g] + W[p + "D"][hd] * x[hd]
    y = y.reshape(-1) * silu(z)
    ng = mx.get("norm_groups", 1)
    y = rms_unit(y.view(ng, inner // ng), eps).reshape(-1) * W[p + "norm"]
    return W[p + "o"] @ y


def rglru_token(h, W, p, mx, state):
    """One token of the gated linear recurrent mixer.  state: dict with 'S' [width] and 'hist'."""
    Wd, nb = mx["width"], mx.get("blocks", 1)
    y = gelu_tanh(W[p + "y"] @ h + W[p + "y.b"])
    u = conv_token(W[p + "x"] @ h + W[p + "x.b"], W[p + "conv"], W[p + "conv.b"], state["hist"])
    ub = u.view(nb, Wd // nb)
    r = sigmoid(torch.einsum("boi,bi->bo", W[p + "ra"], ub) + W[p + "ra.b"]).reshape(-1)
    i = sigmoid(torch.einsum("boi,bi->bo", W[p + "ri"], ub) + W[p + "ri.b"]).reshape(-1)
    log_a = -8.0 * r * softplus(W[p + "lam"])
    a = torch.exp(log_a)
    state["S"] = a * state["S"] + torch.sqrt(1.0 - a * a) * i * u
    return W[p + "o"] @ (state["S"] * y)


def gated_expert(h, W, p):
    return W[p + "down"] @ (silu(W[p + "gate"] @ h) * (W[p + "up"] @ h))


def route(h, W, p, r):
    """Chosen experts and their weights: sigmoid scores, groups ranked by their top two scores added up, the
    largest scores among those groups, normalised and scaled."""
    E, top = r["experts"], r["top"]
    s = sigmoid(W[p + "router"] @ h)
    allowed = torch.ones(E, dtype=torch.bool)
    grp = r.get("groups")
    if grp:
        n, keep = grp["count"], grp.get("keep", grp["count"])
        per = E // n
        gs = [float(torch.sort(s[g * per:(g + 1) * per], descending=True).values[:2].sum()) for g in range(n)]
        best = sorted(range(n), key=lambda g: (-gs[g], g))[:keep]
        allowed[:] = False
        for g in best:
            allowed[g * per:(g + 1) * per] = True
    order = sorted([e for e in range(E) if allowed[e]], key=lambda e: (-float(s[e]), e))[:top]
    wsum = sum(float(s[e]) for e in order) + 1e-20
    return [(e, float(s[e]) / wsum * r.get("scale", 1.0)) for e in order]


def moe_token(h, W, p, mlp):
    out = torch.zeros_like(h)
    for e, wgt in route(h, W, p, mlp["router"]):
        out = out + wgt * gated_expert(h, W, p + f"e{e}.")
    if mlp.get("shared"):
        out = out + sigmoid(W[p + "shared.sg"] @ h) * gated_expert(h, W, p + "shared.")
    return out


def side_token(x, W, li, token, dim, eps):
    """The per-layer token input: what is added to the stream after layer li's feed-forward."""
    e = W["side.embed"][token, li * dim:(li + 1) * dim]
    g = gelu_tanh(W[f"l{li}.side.gate"] @ x) * e
    y = W[f"l{li}.side.proj"] @ g
    return rms_unit(y, eps) * W[f"l{li}.side.norm"]


def layer_runs(cfg):
    """Layer index of every layer run, with the looped range repeated."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop or loop.get("times", 1) <= 1:
        return list(range(n))
    a, b, t = loop["start"], loop["stop"], loop["times"]
    return list(range(a)) + list(range(a, b)) * t + list(range(b, n))


class PlainTugovik:
    """Token-by-token forward of one sequence.  ``step(token)`` returns (logits, [stream after every layer run])."""

    def __init__(self, cfg: dict, tensors: dict):
        self.cfg = cfg
        self.W = {k: v.to(F) for k, v in tensors.items() if v.is_floating_point()}
        self.runs = layer_runs(cfg)
        self.pos = 0
        self.state = []
        for li in self.runs:
            l = cfg["layers"][li]
            mx = l["mixer"]
            if l["type"] == "attention":
                self.state.append([])
            elif l["type"] == "mamba2":
                ch = mx["heads"] * mx["vdim"] + 2 * mx.get("groups", 1) * mx["state"]
                self.state.append({"S": torch.zeros(mx["heads"], mx["state"], mx["vdim"], dtype=F),
                                   "hist": [torch.zeros(ch, dtype=F) for _ in range(mx["conv"] - 1)]})
            elif l["type"] == "rglru":
                self.state.append({"S": torch.zeros(mx["width"], dtype=F),
                                   "hist": [torch.zeros(mx["width"], dtype=F) for _ in range(mx["conv"] - 1)]})
            else:
                raise ValueError(l["type"])

    def step(self, token: int):
        cfg, W = self.cfg, self.W
        eps = cfg["norm"]["eps"]
        x = W["embed"][token].clone()
        streams = []
        for ri, li in enumerate(self.runs):
            l = cfg["layers"][li]
            p = f"l{li}."
            h = offset_norm(x, W[p + "norm1"], eps)
            if l["type"] == "attention":
                y = attention_token(h, W, p + "mix.", l["mixer"], self.pos, self.state[ri])
            elif l["type"] == "mamba2":
                y = mamba2_token(h, W, p + "mix.", l["mixer"], eps, self.state[ri])
            else:
                y = rglru_token(h, W, p + "mix.", l["mixer"], self.state[ri])
            x = x + y
            if l.get("mlp"):
                x = x + moe_token(offset_norm(x, W[p + "norm2"], eps), W, p + "mlp.", l["mlp"])
            if cfg.get("token_side"):
                x = x + side_token(x, W, li, token, cfg["token_side"]["dim"], eps)
            streams.append(x.clone())
        logits = W["head"] @ offset_norm(x, W["final.norm"], eps)
        self.pos += 1
        return logits, streams


def run(cfg: dict, tensors: dict, tokens):
    """Logits of every token [n, vocab] and the stream after every layer run [runs][n, width]."""
    m = PlainTugovik(cfg, tensors)
    logits, per_run = [], [[] for _ in m.runs]
    for t in tokens:
        lg, streams = m.step(int(t))
        logits.append(lg)
        for r, x in enumerate(streams):
            per_run[r].append(x)
    return torch.stack(logits), [torch.stack(v) for v in per_run]
