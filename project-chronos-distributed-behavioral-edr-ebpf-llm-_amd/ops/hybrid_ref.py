"""PyTorch references of the hybrid-decoder kernels (csrc/kernels/hybrid*.hip): the CPU execution path and the
numerics oracle of the GPU tests.  Same interfaces as the kernels (layouts, in-place arguments); everything the
kernels keep in 32-bit floats is computed in float32 here too, whatever the activation dtype.

Activation dtype ``AT`` is bfloat16 or float32; the residual stream is always float32.
"""
from __future__ import annotations

import math

import torch

ACT_RELU2, ACT_GELU = 0, 1


def embed_rows(ids, table, act_dtype, scale=1.0, emit=True):
    x = table[ids.long()].float()
    if scale != 1.0:
        x = x * scale
    return x, ((x if act_dtype == torch.float32 else x.to(act_dtype)) if emit else None)


def layer_norm(x, w, eps, act_dtype):
    xf = x.float()
    mu = xf.mean(-1, keepdim=True)
    d = xf - mu
    y = d * torch.rsqrt(d.pow(2).mean(-1, keepdim=True) + eps) * w.float()
    return y.to(act_dtype)


def add_layer_norm(y, x, w, eps, act_dtype):
    """x (float32, in place) <- x + layer_norm(y) * w; returns x in the activation dtype (x itself for float32)."""
    x.add_(layer_norm(y, w, eps, torch.float32))
    return x if act_dtype == torch.float32 else x.to(act_dtype)


def rowdot(h, w, bias=None):
    """float32 [T, N] = h @ w.T (+ bias) with float32 accumulation: the few-row projections whose outputs feed
    32-bit math (recurrence gates, router logits, head gates)."""
    z = h.float() @ w.float().t()
    return z if bias is None else z + bias.float()


def act_inplace(x, kind):
    xf = x.float()
    if kind == ACT_RELU2:
        r = torch.relu(xf) ** 2
    else:
        r = 0.5 * xf * (1.0 + torch.erf(xf * (1.0 / math.sqrt(2.0))))
    x.copy_(r.to(x.dtype))
    return x


def mlstm_scan(proj, gate_pre, q_start, pos0, slots, S, n, m, H, D, Dv, cap):
    """Stabilised matrix-memory recurrence over a flattened token stream.

    proj [T, >= 2 H D + H Dv]: per token q (H x D), k (H x D), v (H x Dv) side by side; gate_pre f32 [T, 2 H]: the
    input- and forget-gate pre-activations; q_start [B + 1]: token range of each sequence; pos0 [B]: position of the
    range's first token (0: the state starts at zero, with the running maximum at 0); slots [B]: row of the state
    tensors S [NS, H, D, Dv], n [NS, H, D], m [NS, H] (float32, updated in place).  Returns the normalised read-out
    f32 [T, H, Dv]."""
    T = proj.shape[0]
    out = torch.zeros(T, H, Dv, dtype=torch.float32, device=proj.device)
    qs = q_start.tolist()
    p0 = pos0.tolist()
    sl = slots.tolist()
    pf = proj.float()
    ig_all = cap * torch.tanh(gate_pre[:, :H].float() / cap)
    fg_all = torch.nn.functional.logsigmoid(cap * torch.tanh(gate_pre[:, H:2 * H].float() / cap))
    for b in range(len(sl)):
        s = sl[b]
        if p0[b] == 0:
            Sb = torch.zeros_like(S[s])
            nb = torch.zeros_like(n[s])
            mb = torch.zeros_like(m[s])
        else:
            Sb, nb, mb = S[s].clone(), n[s].clone(), m[s].clone()
        for t in range(qs[b], qs[b + 1]):
            q = pf[t, :H * D].view(H, D) * D ** -0.5
            k = pf[t, H * D:2 * H * D].view(H, D)
            v = pf[t, 2 * H * D:2 * H * D + H * Dv].view(H, Dv)
            ig, fg = ig_all[t], fg_all[t]
            mn = torch.maximum(fg + mb, ig)
            a, bb = torch.exp(fg + mb - mn), torch.exp(ig - mn)
            Sb = a[:, None, None] * Sb + bb[:, None, None] * (k[:, :, None] * v[:, None, :])
            nb = a[:, None] * nb + bb[:, None] * k
            mb = mn
            den = torch.maximum((nb * q).sum(-1).abs(), torch.exp(-mb)) + 1e-6
            out[t] = torch.einsum("hdv,hd->hv", Sb, q) / den[:, None]
        if qs[b + 1] > qs[b]:
            S[s], n[s], m[s] = Sb, nb, mb
    return out


def mlstm_out(o, proj, g_off, norm_w, eps, act_dtype):
    """Per-head unit RMS of the read-out, times the head-concatenated weight, times sigmoid of the gate columns
    proj[:, g_off : g_off + H Dv]."""
    T, H, Dv = o.shape
    y = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps)
    y = y.reshape(T, H * Dv) * norm_w.float() * torch.sigmoid(proj[:, g_off:g_off + H * Dv].float())
    return y.to(act_dtype)


def rotate_half_rows(x, cos_sin, pos, dims):
    """Rotary position on the first ``dims`` entries of the last axis (entry i pairs with i + dims/2); cos_sin
    [P, dims]: cos | sin of position x frequency, float32."""
    half = dims // 2
    cs = cos_sin[pos.long()]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    c, s = cs[:, :half].view(shape), cs[:, half:].view(shape)
    u, v = x[..., :half].float(), x[..., half:dims].float()
    out = x.float().clone()
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


def latent_prep(q, dkv, pos, tok_seq, block_table, w_norm, eps, cos_sin, dims, rank, cache):
    """Latent-attention cache write and query rotation.  dkv [T, rank + R]: the first rank columns are RMS-normed
    (times w_norm) into the latent, the last R rotated; both are written to cache [NB, BS, rank + R] at the token's
    page and slot.  q [T, H, D + R]: the last R columns of every head are rotated in place."""
    T = q.shape[0]
    R = dkv.shape[1] - rank
    D = q.shape[2] - R
    c = dkv[:, :rank].float()
    c = c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + eps) * w_norm.float()
    kr = rotate_half_rows(dkv[:, rank:], cos_sin, pos, dims)
    row = torch.cat([c, kr], 1).to(cache.dtype)
    bs = cache.shape[1]
    blk = block_table[tok_seq.long(), (pos // bs).long()].long()
    cache[blk, (pos % bs).long()] = row
    q[:, :, D:] = rotate_half_rows(q[:, :, D:], cos_sin, pos, dims).to(q.dtype)


def latent_attention(qa, cache, block_table, q_start, pos, gate, scale, rank, act_dtype):
    """Causal softmax attention of H query heads over ONE shared key row per token: key = the cached row (rank + R
    columns), value = its first rank columns.  qa [T, H, rank + R]; token t of sequence b sits at pos[t] and sees the
    cached rows 0..pos[t] of its sequence; gate f32 [T, H] or None: the output of head h is multiplied by
    sigmoid(gate).  Returns [T, H, rank]."""
    T, H, DK = qa.shape
    out = torch.zeros(T, H, rank, dtype=torch.float32, device=qa.device)
    bs = cache.shape[1]
    qs = q_start.tolist()
    for b in range(len(qs) - 1):
        t0, t1 = qs[b], qs[b + 1]
        if t1 <= t0:
            continue
        p = pos[t0:t1].long()
        ctx = int(p.max()) + 1
        nblk = (ctx + bs - 1) // bs
        keys = cache[block_table[b, :nblk].long()].reshape(nblk * bs, DK)[:ctx].float()
        sc = torch.einsum("thk,jk->thj", qa[t0:t1].float(), keys) * scale
        mask = torch.arange(ctx, device=qa.device)[None, :] > p[:, None]
        sc = sc.masked_fill(mask[:, None, :], float("-inf"))
        a = torch.softmax(sc, -1)
        out[t0:t1] = torch.einsum("thj,jr->thr", a, keys[:, :rank])
    if gate is not None:
        out = out * torch.sigmoid(gate.float())[:, :, None]
    return out.to(act_dtype)


def moe_route(h, w_router, correction, top):
    """Router of a mixture of experts: float32 logits, softmax over all outputs, the ``top`` largest of
    score + correction are chosen (ties: the lower index), weighted by their plain scores (not renormalised).
    Returns (idx int32 [T, top], weight f32 [T, top])."""
    s = torch.softmax(rowdot(h, w_router), -1)
    choice = s + correction.float()
    idx = torch.topk(choice, top, dim=-1).indices
    return idx.to(torch.int32), torch.gather(s, 1, idx)


def moe_ffn(h, idx, wt, w_up, w_down, act, act_dtype):
    """Weighted sum of each token's chosen experts.  w_up [E, F, d], w_down [E, d, F]; an index >= E is an identity
    expert (its output is the token itself)."""
    E = w_up.shape[0]
    hf = h.float()
    out = torch.zeros_like(hf)
    idl = idx.long()
    for e in range(E):
        tok, kk = torch.nonzero(idl == e, as_tuple=True)
        if tok.numel() == 0:
            continue
        z = (hf[tok].to(act_dtype) @ w_up[e].t().to(act_dtype))
        z = act_inplace(z, act)
        y = (z @ w_down[e].t().to(act_dtype)).float()
        out.index_add_(0, tok, y * wt[tok, kk][:, None])
    ident = (idl >= E).float() * wt
    out = out + ident.sum(-1, keepdim=True) * hf
    return out.to(act_dtype)


# ---- post-norm residual stream, clamped GLU, windowed attention with sinks, linear-state recurrences ---------------

ACT_GLU = 2  # gated unit: min(g, limit) * sigmoid(slope * g) * (clamp(u, +-limit) + shift)


def rms_norm(x, w, eps, act_dtype, groups=1):
    """``groups`` > 1: the row is split into that many equal consecutive parts, each divided by its own root mean
    square; the whole row is multiplied by w."""
    xf = x.float()
    if groups > 1:
        xg = xf.view(*xf.shape[:-1], groups, xf.shape[-1] // groups)
        xf = (xg * torch.rsqrt(xg.pow(2).mean(-1, keepdim=True) + eps)).view(xf.shape)
        return (xf * w.float()).to(act_dtype)
    return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * w.float()).to(act_dtype)


def scale_add_rms_norm(y, x, w, alpha, eps, act_dtype):
    """x (float32, in place) <- rms_norm(alpha * x + y) * w; returns x in the activation dtype (x itself for
    float32): the norm sits AFTER the residual sum and the stream itself is what the next sublayer reads."""
    x.copy_(rms_norm(alpha * x + y.float(), w, eps, torch.float32))
    return x if act_dtype == torch.float32 else x.to(act_dtype)


def glu(gu, limit, slope, shift, act_dtype):
    """gu [T, 2F]: gate columns then up columns -> [T, F]."""
    F = gu.shape[1] // 2
    g = gu[:, :F].float().clamp(max=limit)
    u = gu[:, F:].float().clamp(-limit, limit)
    return (g * torch.sigmoid(slope * g) * (u + shift)).to(act_dtype)


def window_prep(qkv, H, G, D, Dv, v_first, lam, pos, tok_seq, block_table, q_norm, k_norm, eps, cos_sin, dims, kc, vc,
                emit_v, v_off=-1, v_cos_sin=None):
    """qkv [T, H D + G D + G Dv]: per-head RMS norm (weights q_norm / k_norm [D], float32 math; both None: no
    norm) and rotation of the query and key heads, queries in place; values mixed with ``v_first`` [T, G Dv] as (1 - lam) v + lam v_first when
    given; keys and (mixed) values written to the paged caches kc [NB, BS, G, D], vc [NB, BS, G, Dv].  Returns the
    values as read from the projection [T, G Dv] when ``emit_v`` (the source of later layers' mixing), else None.
    ``v_off`` >= 0: the values start at that column of qkv instead of after the keys (at H D they are the keys as
    projected).  ``v_cos_sin`` [P, Dv]: the values are rotated by their position over all Dv columns before the
    write."""
    T = qkv.shape[0]
    q = qkv[:, :H * D].view(T, H, D)
    k = qkv[:, H * D:(H + G) * D].view(T, G, D)
    v0 = (H + G) * D if v_off < 0 else v_off
    v = qkv[:, v0:v0 + G * Dv].view(T, G, Dv)
    out_v = v.reshape(T, G * Dv).clone() if emit_v else None

    def norm_rot(x, w):
        xf = x.float()
        if w is not None:
            xf = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * w.float()
        return rotate_half_rows(xf, cos_sin, pos, dims) if dims else xf

    qn = norm_rot(q, q_norm)
    kn = norm_rot(k, k_norm)
    vf = v.float()
    if v_first is not None:
        l = lam.float().reshape(())
        vf = (1.0 - l) * vf + l * v_first.view(T, G, Dv).float()
    if v_cos_sin is not None:
        vf = rotate_half_rows(vf, v_cos_sin, pos, Dv)
    bs = kc.shape[1]
    blk = block_table[tok_seq.long(), (pos // bs).long()].long()
    kc[blk, (pos % bs).long()] = kn.to(kc.dtype)
    vc[blk, (pos % bs).long()] = vf.to(vc.dtype)
    q.copy_(qn.to(q.dtype))
    return out_v


def pool_blocks(kc, vc, kp, vp, block_table, q_start, pos0, pool):
    """Means of the cached keys and values of every block of ``pool`` positions whose last position is among this
    step's tokens (sequence b brings positions pos0[b] .. pos0[b] + n_b - 1), in float32, written in the cache dtype
    to kp / vp [NB, EP, G, .]: block e of a sequence sits in row e % EP of the sequence's page e // EP."""
    bs, ep = kc.shape[1], kp.shape[1]
    qs, p0 = q_start.tolist(), pos0.tolist()
    for b in range(len(qs) - 1):
        n = qs[b + 1] - qs[b]
        if n <= 0:
            continue
        for e in range(p0[b] // pool, (p0[b] + n) // pool):
            j = torch.arange(e * pool, (e + 1) * pool, device=kc.device)
            pages = block_table[b, (j // bs).long()].long()
            page = int(block_table[b, e // ep])
            kp[page, e % ep] = kc[pages, (j % bs).long()].float().mean(0).to(kp.dtype)
            vp[page, e % ep] = vc[pages, (j % bs).long()].float().mean(0).to(vp.dtype)


def window_attention(qkv, kc, vc, block_table, q_start, pos, sink, gate, scale, window, keep_first, H, act_dtype,
                     chunk=0, pool=0, kp=None, vp=None):
    """Causal softmax attention over a paged cache through a sliding window that also keeps a sequence's first
    tokens: the query at position i sees key j <= i when i - j < window or j < keep_first (window 0: every j <= i).
    ``chunk`` > 0 further hides every key outside the query's own chunk of that many positions (the chunk grid
    is anchored at the sequence's first position): j is visible only when j // chunk == i // chunk.
    ``sink`` f32 [H] or None: exp(sink_h) joins the softmax denominator (no key, no value).  ``gate`` f32 [T, H] or
    None: head h's output times sigmoid(gate).  Queries are the first H D columns of qkv; query head h reads
    key/value head h // (H / G).  ``pool`` > 0 (with a window): the query at i also sees the pooled pair of every
    block e with e pool + pool - 1 <= i - window (kp / vp as :func:`pool_blocks` leaves them), in the same softmax.
    Returns [T, H Dv]."""
    T = qkv.shape[0]
    G, D, Dv = kc.shape[2], kc.shape[3], vc.shape[3]
    q = qkv[:, :H * D].view(T, H, D).float()
    out = torch.zeros(T, H, Dv, dtype=torch.float32, device=qkv.device)
    bs = kc.shape[1]
    qs = q_start.tolist()
    rep = H // G
    for b in range(len(qs) - 1):
        t0, t1 = qs[b], qs[b + 1]
        if t1 <= t0:
            continue
        p = pos[t0:t1].long()
        ctx = int(p.max()) + 1
        nblk = (ctx + bs - 1) // bs
        pages = block_table[b, :nblk].long()
        keys = kc[pages].reshape(nblk * bs, G, D)[:ctx].float().repeat_interleave(rep, 1)
        vals = vc[pages].reshape(nblk * bs, G, Dv)[:ctx].float().repeat_interleave(rep, 1)
        sc = torch.einsum("thd,jhd->thj", q[t0:t1], keys) * scale
        j = torch.arange(ctx, device=qkv.device)[None, :]
        hidden = j > p[:, None]
        if window:
            hidden = hidden | ((p[:, None] - j >= window) & (j >= keep_first))
        if chunk:
            hidden = hidden | (j < (p[:, None] // chunk) * chunk)
        sc = sc.masked_fill(hidden[:, None, :], float("-inf"))
        nblocks = max(0, (int(p.max()) - window + 1) // pool) if pool and window else 0
        if nblocks:
            ep = kp.shape[1]
            e = torch.arange(nblocks, device=qkv.device)
            pg = block_table[b, (e // ep).long()].long()
            pk = kp[pg, (e % ep).long()].float().repeat_interleave(rep, 1)
            pv = vp[pg, (e % ep).long()].float().repeat_interleave(rep, 1)
            psc = torch.einsum("thd,jhd->thj", q[t0:t1], pk) * scale
            psc = psc.masked_fill(((e[None, :] + 1) * pool - 1 + window > p[:, None])[:, None, :], float("-inf"))
            sc = torch.cat([sc, psc], -1)
            vals = torch.cat([vals, pv], 0)
        if sink is not None:
            sc = torch.cat([sc, sink.float()[None, :, None].expand(t1 - t0, H, 1)], -1)
        a = torch.softmax(sc, -1)[:, :, :ctx + nblocks]
        out[t0:t1] = torch.einsum("thj,jhv->thv", a, vals)
    if gate is not None:
        out = out * torch.sigmoid(gate.float())[:, :, None]
    return out.reshape(T, H * Dv).to(act_dtype)


def short_conv(x, w, q_start, pos0, slots, hist, silu, bias=None, x_off=0):
    """Causal per-channel convolution over time on a flattened token stream, on the C columns of x [T, >= x_off + C]
    from column x_off on; w f32 [C, K] (the last column weighs the current token), bias f32 [C] or None; hist
    [NS, K - 1, C]: every sequence's last K - 1 inputs (oldest first), read when its range starts past position 0
    (zeros otherwise) and updated in place.  Returns [T, C] in x's dtype."""
    C, K = w.shape
    x = x[:, x_off:x_off + C]
    y = torch.empty_like(x)
    qs, p0, sl = q_start.tolist(), pos0.tolist(), slots.tolist()
    for b in range(len(sl)):
        t0, t1 = qs[b], qs[b + 1]
        if t1 <= t0:
            continue
        past = hist[sl[b]].clone() if p0[b] > 0 else torch.zeros(K - 1, C, dtype=x.dtype, device=x.device)
        ext = torch.cat([past, x[t0:t1]], 0).float()
        acc = torch.zeros(t1 - t0, C, dtype=torch.float32, device=x.device)
        for i in range(K):
            acc += ext[i:i + t1 - t0] * w[:, i].float()
        if bias is not None:
            acc += bias.float()
        if silu:
            acc = acc * torch.sigmoid(acc)
        y[t0:t1] = acc.to(x.dtype)
        if K > 1:
            hist[sl[b]] = ext[-(K - 1):].to(hist.dtype)
    return y


def delta_prep(y, ab, a_log, HK, H, D, q_mul):
    """Per-token scalars of the gated delta rule.  y [T, >= 2 HK D]: q heads then k heads (after convolution and
    activation); ab f32 [T, 2 H]: decay pre-activations (bias included) then write-strength pre-activations.
    Returns float32 (qscale [T, HK] = q_mul / sqrt(|q|^2 + 1e-6), kscale [T, HK] = 1 / sqrt(|k|^2 + 1e-6),
    decay [T, H] = exp(-exp(a_log) softplus(a)), beta [T, H] = sigmoid(b))."""
    T = y.shape[0]
    q = y[:, :HK * D].float().view(T, HK, D)
    k = y[:, HK * D:2 * HK * D].float().view(T, HK, D)
    qs = q_mul * torch.rsqrt(q.pow(2).sum(-1) + 1e-6)
    ks = torch.rsqrt(k.pow(2).sum(-1) + 1e-6)
    decay = torch.exp(-torch.exp(a_log.float()) * torch.nn.functional.softplus(ab[:, :H].float()))
    return qs, ks, decay, torch.sigmoid(ab[:, H:2 * H].float())


def decay_pow(z, inv_tau):
    """z f32 (in place) <- sigmoid(z) ** inv_tau, through the logarithm."""
    z.copy_(torch.exp(torch.nn.functional.logsigmoid(z) * inv_tau))
    return z


def linear_scan(proj, q_off, k_off, v_off, qscale, kscale, q_mul, decay, beta, q_start, pos0, slots, S, HK, H, D, Dv,
                vscale=None):
    """Linear-state recurrence over a flattened token stream, per value head h (reading q/k head h // (H / HK)):

        S <- decay * S                      decay f32 [T, H] (one per head), [T, H, D] (one per key channel / row)
                                            or [H] (one per head, the same for every token)
        u  = v - S^T k, times beta          only when beta f32 [T, H] is given (the delta rule); else u = v
        S <- S + k u^T;   o = S^T q

    q, k, v are columns of proj [T, C] at q_off / k_off / v_off; q is multiplied by qscale [T, HK] (or by q_mul when
    None), k by kscale [T, HK] (when given) and v by vscale [T, H] (when given; not with beta), in float32.  S f32
    [NS, H, D, Dv] by slot, in place; a range whose first token sits at position 0 starts from zero.  Returns o f32
    [T, H, Dv]."""
    T = proj.shape[0]
    out = torch.zeros(T, H, Dv, dtype=torch.float32, device=proj.device)
    qs, p0, sl = q_start.tolist(), pos0.tolist(), slots.tolist()
    pf = proj.float()
    q = pf[:, q_off:q_off + HK * D].view(T, HK, D)
    k = pf[:, k_off:k_off + HK * D].view(T, HK, D)
    v = pf[:, v_off:v_off + H * Dv].view(T, H, Dv)
    q = q * (qscale[:, :, None] if qscale is not None else q_mul)
    if kscale is not None:
        k = k * kscale[:, :, None]
    if vscale is not None:
        v = v * vscale[:, :, None]
    rep = H // HK
    q, k = q.repeat_interleave(rep, 1), k.repeat_interleave(rep, 1)
    if decay.dim() == 1:           # one fixed number per head
        decay = decay[None, :].expand(T, H)
    dec = decay.reshape(T, H, -1, 1)  # [T, H, 1 | D, 1]
    for b in range(len(sl)):
        if qs[b + 1] <= qs[b]:
            continue
        Sb = torch.zeros_like(S[sl[b]]) if p0[b] == 0 else S[sl[b]].clone()
        for t in range(qs[b], qs[b + 1]):
            Sb = dec[t] * Sb
            u = v[t]
            if beta is not None:
                u = beta[t][:, None] * (u - torch.einsum("hdv,hd->hv", Sb, k[t]))
            Sb = Sb + k[t][:, :, None] * u[:, None, :]
            out[t] = torch.einsum("hdv,hd->hv", Sb, q[t])
        S[sl[b]] = Sb
    return out


def head_norm_gate(o, src, g_off, w, eps, silu_gate, act_dtype):
    """Per-head unit RMS of o f32 [T, H, Dv], times w [H Dv], times sigmoid (or silu) of the gate columns
    src[:, g_off : g_off + H Dv]."""
    T, H, Dv = o.shape
    y = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps)
    g = src[:, g_off:g_off + H * Dv].float()
    g = g * torch.sigmoid(g) if silu_gate else torch.sigmoid(g)
    return (y.reshape(T, H * Dv) * w.float() * g).to(act_dtype)


def moe_route_topk(h, w_router, bias, top):
    """Router that picks the ``top`` largest logits (h W^T + bias, float32; ties: the lower index) and weighs them by
    the softmax over the chosen logits only.  Returns (idx int32 [T, top], weight f32 [T, top])."""
    z = rowdot(h, w_router, bias)
    val, idx = torch.topk(z, top, dim=-1)
    return idx.to(torch.int32), torch.softmax(val, -1)


def moe_glu_ffn(h, idx, wt, w_gu, w_down, limit, slope, shift, act_dtype):
    """Weighted sum of each token's chosen gated experts.  w_gu [E, 2F, d]: gate rows then up rows; w_down
    [E, d, F]."""
    E = w_gu.shape[0]
    hf = h.float()
    out = torch.zeros_like(hf)
    idl = idx.long()
    for e in range(E):
        tok, kk = torch.nonzero(idl == e, as_tuple=True)
        if tok.numel() == 0:
            continue
        gu = hf[tok].to(act_dtype) @ w_gu[e].t().to(act_dtype)
        y = (glu(gu, limit, slope, shift, act_dtype) @ w_down[e].t().to(act_dtype)).float()
        out.index_add_(0, tok, y * wt[tok, kk][:, None])
    return out.to(act_dtype)


# ---- pre-norm residual stream, per-layer token input, state-space and gated linear recurrences, grouped router ---


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z * z * z)))


def add_rms_norm(y, x, w_out, eps, act_dtype, y2=None, gate2=None, w_y=None, emit=True):
    """The pre-norm stream's join.  v = y (+ sigmoid(gate2) * y2, gate2 f32 [T, 1]); when w_y is given v is first
    scaled to unit RMS and multiplied by w_y; x (float32, in place) <- x + v.  Returns, in the
    activation dtype, rms_norm(x) * w_out when w_out is given, else x itself (None when ``emit`` is off)."""
    v = y.float()
    if y2 is not None:
        v = v + torch.sigmoid(gate2.float().reshape(-1, 1)) * y2.float()
    if w_y is not None:
        v = v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps) * w_y.float()
    x.add_(v)
    if not emit:
        return None
    if w_out is None:
        return x if act_dtype == torch.float32 else x.to(act_dtype)
    return rms_norm(x, w_out, eps, act_dtype)


def token_gate(a, ids, table, col0, act_dtype):
    """gelu_tanh(a) * table[ids, col0 : col0 + a.shape[1]]: a projection gated by each token's own row of a table."""
    e = table[ids.long(), col0:col0 + a.shape[1]].float()
    return (gelu_tanh(a.float()) * e).to(act_dtype)


def ssm_prep(dt_pre, a_log):
    """Per token and head of a state-space layer: step dt = softplus(dt_pre) (bias already added, no clamp) and
    decay = exp(-exp(a_log) dt).  dt_pre f32 [T, H].  Returns float32 (decay, dt)."""
    dt = torch.nn.functional.softplus(dt_pre.float(), threshold=30.0)
    return torch.exp(-torch.exp(a_log.float()) * dt), dt


def gated_group_norm(o, skip_src, skip_off, skip_w, gate_src, g_off, w, groups, eps, act_dtype):
    """Read-out of a state-space layer: y = (o + skip_w[h] * x) * silu(z) with x = skip_src[:, skip_off:...] and
    z = gate_src[:, g_off:...] (both [T, H Dv] column ranges), then RMS norm over ``groups`` equal column ranges of the
    H Dv columns (every range with its own statistic), times w [H Dv].  o f32 [T, H, Dv]."""
    T, H, Dv = o.shape
    n = H * Dv
    y = o + skip_w.float()[None, :, None] * skip_src[:, skip_off:skip_off + n].float().view(T, H, Dv)
    z = gate_src[:, g_off:g_off + n].float()
    y = y.reshape(T, n) * (z * torch.sigmoid(z))
    y = y.view(T, groups, n // groups)
    y = y * torch.rsqrt(y.pow(2).mean(-1, keepdim=True) + eps)
    return (y.reshape(T, n) * w.float()).to(act_dtype)


def rglru_scan(u, gates, sp, c, ysrc, y_off, q_start, pos0, slots, S, act_dtype):
    """Real-gated linear recurrent unit over a flattened token stream, per channel:

        r = sigmoid(gates[.., 0, :]),  i = sigmoid(gates[.., 1, :]),  log a = -c r sp,  a = exp(log a)
        S <- a S + sqrt(1 - a^2) i u;     out = S * gelu_tanh(y)

    u [T, W] (the convolved branch); gates f32 [NB, T, 2 W / NB]: per block of channels the pre-activations of r,
    then of i;
    sp f32 [W] = softplus of the decay parameter; y = ysrc[:, y_off : y_off + W]; S f32 [NS, W] by slot, in place; a
    range whose first token sits at position 0 starts from zero.  Returns [T, W] in the activation dtype."""
    T, W = u.shape
    NB = gates.shape[0]
    g = gates.float().reshape(NB, T, 2, W // NB).permute(1, 2, 0, 3).reshape(T, 2, W)
    r, i = torch.sigmoid(g[:, 0]), torch.sigmoid(g[:, 1])
    log_a = -c * r * sp.float()
    a = torch.exp(log_a)
    b = torch.sqrt(-torch.expm1(2.0 * log_a)) * i * u.float()
    out = torch.empty(T, W, dtype=torch.float32, device=u.device)
    qs, p0, sl = q_start.tolist(), pos0.tolist(), slots.tolist()
    for bb in range(len(sl)):
        if qs[bb + 1] <= qs[bb]:
            continue
        s = torch.zeros_like(S[sl[bb]]) if p0[bb] == 0 else S[sl[bb]].clone()
        for t in range(qs[bb], qs[bb + 1]):
            s = a[t] * s + b[t]
            out[t] = s
        S[sl[bb]] = s
    return (out * gelu_tanh(ysrc[:, y_off:y_off + W].float())).to(act_dtype)


def moe_route_group(h, w_router, top, n_groups, keep, scale):
    """Router with sigmoid scores and a choice limited to the best groups: the N outputs form n_groups equal groups
    of neighbours, a group scores its top two scores added up, the ``keep`` best groups stay, and the ``top``
    largest scores among them are chosen (ties: the lower index) and weighted by score / (sum of the chosen + 1e-20)
    * scale.  Returns (idx int32 [T, top], weight f32 [T, top])."""
    s = torch.sigmoid(rowdot(h, w_router))
    T, N = s.shape
    cand = s
    if n_groups > 1 and keep < n_groups:
        per = N // n_groups
        gs = s.view(T, n_groups, per).topk(min(2, per), dim=-1).values.sum(-1)
        # stable choice of the best groups: by score, then by the lower index
        order = torch.sort(gs, dim=-1, descending=True, stable=True).indices[:, :keep]
        ok = torch.zeros(T, n_groups, dtype=torch.bool, device=s.device).scatter_(1, order, True)
        cand = s.masked_fill(~ok[:, :, None].expand(T, n_groups, per).reshape(T, N), float("-inf"))
    idx = torch.sort(cand, dim=-1, descending=True, stable=True).indices[:, :top]
    val = torch.gather(s, 1, idx)
    return idx.to(torch.int32), val / (val.sum(-1, keepdim=True) + 1e-20) * scale


# ---- sandwich residual stream, pooled windows, rotated values, retention --------------------------------------------


def sandwich_join(y, x, w_y, w_out, groups, eps, act_dtype, y2=None, pair=None, emit=True):
    """The sandwich stream's join.  v = y (+ y2), or with ``pair`` = (w_a, w_b): v = (rms_norm(y) w_a +
    rms_norm(y2) w_b) / 2, both norms over the whole row.  Then v <- group_rms_norm(v) * w_y and x (float32, in
    place) <- x + v.  Returns group_rms_norm(x) * w_out in the activation dtype (None when ``emit`` is off)."""
    v = y.float()
    if pair is not None:
        v = 0.5 * (rms_norm(v, pair[0], eps, torch.float32) + rms_norm(y2.float(), pair[1], eps, torch.float32))
    elif y2 is not None:
        v = v + y2.float()
    x.add_(rms_norm(v, w_y, eps, torch.float32, groups))
    return rms_norm(x, w_out, eps, act_dtype, groups) if emit else None


def unrotate_gate(o, pos, v_cos_sin, gate_src, g_off, H, Dv, act_dtype):
    """o [T, H Dv]: every head's row is turned back by the token's position (the inverse of the rotation
    :func:`window_prep` applies to values; skipped without a table), then multiplied element by element with sigmoid
    of gate_src[:, g_off : g_off + H Dv] (skipped without a gate source)."""
    T = o.shape[0]
    of = o.float().view(T, H, Dv)
    if v_cos_sin is not None:
        half = Dv // 2
        cs = v_cos_sin[pos.long()]
        c, s = cs[:, None, :half], cs[:, None, half:]
        u, v = of[..., :half], of[..., half:]
        of = torch.cat([u * c + v * s, v * c - u * s], -1)
    of = of.reshape(T, H * Dv)
    if gate_src is not None:
        of = of * torch.sigmoid(gate_src[:, g_off:g_off + H * Dv].float())
    return of.to(act_dtype)


def rotate_qk(proj, q_off, k_off, HQ, HK, D, dims, cos_sin, pos, q_mul, k_mul):
    """In place on proj [T, C]: the HQ heads of D columns from q_off and the HK heads from k_off are rotated on their
    first ``dims`` columns (skipped without a table) and multiplied by q_mul / k_mul, in float32."""
    T = proj.shape[0]
    for off, n, mul in ((q_off, HQ, q_mul), (k_off, HK, k_mul)):
        x = proj[:, off:off + n * D].view(T, n, D)
        xf = rotate_half_rows(x, cos_sin, pos, dims) if (cos_sin is not None and dims) else x.float()
        x.copy_((xf * mul).to(x.dtype))
