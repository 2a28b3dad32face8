"""Hybrid decoders: a list of layers, each with a token mixer of some kind (recurrent matrix memory, latent
attention, windowed or chunked attention, gated delta rule, gated linear attention, state-space duality, real-gated
linear recurrence, retention, two mixers side by side) and an optional feed-forward (dense, gated, mixture of
experts), on a float32 residual stream.
The stream's rule is a parameter of the configuration: the norm on the sublayer's OUTPUT (``out_norm``:
x <- x + layer_norm(sublayer(x))), AFTER the sum (``post_norm``: x <- rms_norm(alpha x + sublayer(x))), on the
sublayer's INPUT (``pre_norm``: x <- x + sublayer(rms_norm(x))) or on both sides (``sandwich``:
x <- x + norm_b(sublayer(norm_a(x))), RMS norms over ``norm_groups`` equal parts of the row).  A range of layers may
repeat, back to back, on shared weights (``loop``), or single layers may name another layer whose weights they use
(``share``); every run has its own pages and state.

This module is the design-independent part: the mixer and feed-forward kinds with their sizes and constants as
parameters, the cache that holds pages for the attention layers and state slots for the recurrent ones, and the
forward over the engine's flattened step batch (:class:`chronos.models.llama.StepBatch`: prefill chunks, decode rows
or both in one step).  A design (``zokunex.py``) reads its configuration file and tensor names into these.

New mixer / feed-forward kinds register in ``MIXERS`` / ``FEED_FORWARDS``.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional

import torch

from ..ops import hybrid as hops
from ..parallel.tp import TPContext
from .llama import StepBatch, h2d


# -----------------------------------------------------------------------------------------------------------------
# configuration
# -----------------------------------------------------------------------------------------------------------------


@dataclass
class MLSTMSpec:
    """Matrix-memory recurrent mixer: per head a D x Dv state, exponential input gate and sigmoid forget gate in
    log space, both soft-capped (cap * tanh(z / cap)) and stabilised by a running maximum."""
    heads: int
    dim: int
    vdim: int
    gate_cap: float
    kind: str = "mlstm"


@dataclass
class LatentAttentionSpec:
    """Attention whose keys and values are up-projections of one cached low-rank latent per token, plus a rotated key
    part shared by all heads; sigmoid output gate per head."""
    heads: int
    dim: int        # unrotated query / key columns per head
    rot_dim: int    # rotated columns per head (the shared rotated key has as many)
    vdim: int
    kv_rank: int
    scale: float
    rope_base: float
    rope_dims: int  # leading columns of the rotated part that are actually rotated
    kind: str = "latent_attention"


@dataclass
class DenseFFSpec:
    ff: int
    act: int = hops.ACT_RELU2
    kind: str = "dense"


@dataclass
class MoEFFSpec:
    experts: int     # experts with weights
    identity: int    # further router outputs whose expert returns its input
    top: int
    ff: int
    act: int = hops.ACT_GELU
    shared_ff: int = 0   # > 0: a shared expert of this size (same form, no router weight) runs for every token
    correction: bool = True   # the checkpoint holds a per-output term that steers the router's choice
    kind: str = "moe"


@dataclass
class WindowAttentionSpec:
    """Grouped-query softmax attention through a sliding window that also keeps each sequence's first tokens, with
    per-head RMS norm of queries and keys, rotation of the leading ``rope_dims`` columns (``rope_scaling``: see
    :func:`rope_cos_sin`), a learned softmax sink per head, an optional mix of every token's values with those of the
    first such layer, and a sigmoid output gate (one number per head, or with ``gate_wide`` one per output column).
    ``pool`` > 0 (with a window): beside the window's tokens a query sees one key and value per block of ``pool``
    positions that lies wholly before its window — the means of the block's cached keys and values.  ``v_from_k``:
    there is no value projection, the values are the keys as projected (before norm and rotation).  ``v_rot``: values
    are cached rotated by their position over all ``vdim`` columns (frequencies rope_base^(-2m/vdim), unscaled) and
    every head's output is turned back by the query's position."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int = 0          # 0: every earlier token is visible
    keep_first: int = 0      # tokens at positions below this stay visible past the window
    rope_base: float = 10000.0
    rope_dims: int = 0       # 0: no rotation
    rope_scaling: Optional[tuple] = None
    v_mix: bool = False
    v_mix_first: bool = False  # this layer is the source of the mixed-in values (and does not mix itself)
    chunk: int = 0           # > 0: a query sees only the keys of its own chunk of this many positions
    qk_norm: bool = True     # per-head RMS norm of queries and keys
    sink: bool = True        # a learned softmax sink per head
    gate: bool = True        # a sigmoid output gate per head
    bias: bool = False       # the q, k, v projections add a bias
    pool: int = 0            # > 0: pooled blocks of this many positions stay visible before the window
    v_from_k: bool = False   # values = the keys as projected
    v_rot: bool = False      # values rotated by their position, outputs turned back
    gate_wide: bool = False  # the sigmoid output gate has heads * vdim rows instead of heads
    kind: str = "window_attention"

    def params(self, d: int) -> int:
        qkv = self.heads * self.dim + self.kv_heads * (self.dim + (0 if self.v_from_k else self.vdim))
        gate = self.heads * (self.vdim if self.gate_wide else 1) * self.gate
        return d * (qkv + gate) + 2 * self.dim * self.qk_norm + self.heads * self.sink + \
            (1 if self.v_mix and not self.v_mix_first else 0) + \
            self.heads * self.vdim * d + qkv * self.bias


@dataclass
class RetentionSpec:
    """Linear attention with one fixed decay per head and no softmax or denominator: per head a dim x vdim state
    S <- decay_h S + k v^T, o = S^T q, with q and k rotated (``rope_dims`` leading columns) and k times dim^(-1/2);
    each head's read-out is scaled to unit RMS and multiplied by silu of a gate projection."""
    heads: int
    dim: int
    vdim: int
    decay: tuple
    rope_base: float = 10000.0
    rope_dims: int = 0
    rope_scaling: Optional[tuple] = None
    kind: str = "retention"

    def params(self, d: int) -> int:
        return d * (2 * self.heads * self.dim + 2 * self.heads * self.vdim) + self.heads * self.vdim * d


@dataclass
class ParallelSpec:
    """Two mixers side by side on the same input; the result is half the sum of their outputs, each first scaled to
    unit RMS over the model width and multiplied by a weight of its own."""
    left: object
    right: object
    kind: str = "parallel"

    def params(self, d: int) -> int:
        return self.left.params(d) + self.right.params(d) + 2 * d


@dataclass
class DeltaRuleSpec:
    """Gated delta rule: per value head a dim x vdim state that decays, is corrected towards the current value along
    the current (unit) key, and is read by the (unit) query; q, k, v pass a short causal convolution and SiLU."""
    heads: int
    kv_heads: int   # query / key heads (value head h reads head h // (heads / kv_heads))
    dim: int
    vdim: int
    conv: int
    kind: str = "delta_rule"

    def params(self, d: int) -> int:
        c = 2 * self.kv_heads * self.dim + self.heads * self.vdim
        return c * (d + self.conv) + self.heads * (2 * d + 2) + self.vdim + 2 * self.heads * self.vdim * d


@dataclass
class GLASpec:
    """Gated linear attention: per head a dim x vdim state whose rows decay by sigmoid(z)^(1/tau), z a low-rank
    projection of the input with a bias."""
    heads: int
    dim: int
    vdim: int
    tau: float
    rank: int
    kind: str = "gla"

    def params(self, d: int) -> int:
        hd, hv = self.heads * self.dim, self.heads * self.vdim
        return d * (2 * hd + 2 * hv) + self.rank * (d + hd) + hd + self.vdim + hv * d


@dataclass
class Mamba2Spec:
    """State-space duality: per head a state x vdim matrix S <- exp(-exp(A) dt) S + dt B x^T, read by C, with B and C
    shared by the heads of a group; x, B and C pass a short causal convolution (with bias) and SiLU; the read-out
    plus D x is gated by silu(z) first and RMS-normed afterwards, over ``norm_groups`` column ranges of equal size."""
    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int = 1
    kind: str = "mamba2"

    @property
    def inner(self) -> int:
        return self.heads * self.vdim

    @property
    def conv_channels(self) -> int:
        return self.inner + 2 * self.groups * self.state

    def params(self, d: int) -> int:
        n_in = 2 * self.inner + 2 * self.groups * self.state + self.heads
        return d * n_in + self.conv_channels * (self.conv + 1) + 3 * self.heads + self.inner + self.inner * d


@dataclass
class RGLRUSpec:
    """Real-gated linear recurrent unit: per channel S <- a S + sqrt(1 - a^2) i u with a = exp(-c r softplus(lam)),
    the gates r and i sigmoids of block-diagonal projections of u, u a short causal convolution (with bias) of one
    input branch; the other branch, through gelu, multiplies the state on the way out."""
    width: int
    blocks: int
    conv: int
    c: float = 8.0
    kind: str = "rglru"

    def params(self, d: int) -> int:
        bw = self.width // self.blocks
        gates = 2 * self.blocks * bw * (bw + 1)
        return 2 * self.width * (d + 1) + self.width * (self.conv + 1) + gates + self.width + self.width * d


@dataclass
class GluFFSpec:
    """Gated feed-forward: y = g sigmoid(slope g) (u + shift) with g = min(W_gate h, limit) and
    u = clamp(W_up h, -limit, limit)."""
    ff: int
    limit: float
    slope: float = 1.702
    shift: float = 1.0
    kind: str = "glu"


@dataclass
class MoEGluSpec:
    """Mixture of gated experts; the router adds a bias to its logits, takes the ``top`` largest and weighs them by
    the softmax over the chosen logits only."""
    experts: int
    top: int
    ff: int
    limit: float
    slope: float = 1.702
    shift: float = 1.0
    kind: str = "moe_glu"


@dataclass
class MoEGroupGluSpec:
    """Mixture of gated experts behind a sigmoid router whose choice is limited to the best groups of neighbouring
    experts (a group scores its top two scores added up); weights = chosen scores / their sum * scale.  With
    ``shared_ff`` > 0 a shared gated expert of that size runs for every token, times sigmoid of one more projection."""
    experts: int
    top: int
    ff: int
    groups: int = 1
    keep: int = 1
    scale: float = 1.0
    shared_ff: int = 0
    limit: float = float("inf")   # the gated unit without clamp: silu(g) u
    slope: float = 1.0
    shift: float = 0.0
    kind: str = "moe_group_glu"


@dataclass
class LayerSpec:
    mixer: object
    ff: Optional[object]


@dataclass
class HybridConfig:
    name: str
    vocab_size: int
    hidden_size: int
    layers: list
    norm_eps: float
    logit_scale: float = 1.0
    max_position: int = 8192
    architecture: str = "hybrid"
    residual: str = "out_norm"     # "out_norm": x <- x + layer_norm(y);  "post_norm": x <- rms_norm(alpha x + y);
    #                                "pre_norm": x <- x + sublayer(rms_norm(x));
    #                                "sandwich": x <- x + norm_b(sublayer(norm_a(x)))
    norm_groups: int = 1           # sandwich: the stream's RMS norms work on this many equal parts of a row
    embed_scale: float = 1.0       # the embedding rows are multiplied by this
    share: Optional[list] = None   # share[i] = j: layer i runs on layer j's weights (j itself has its own)
    residual_alpha: float = 1.0
    tied_head: bool = False        # the logits come from the embedding table
    loop: Optional[tuple] = None   # (start, stop, times): layers [start, stop) run ``times`` times, back to back
    token_side: int = 0            # > 0: after every layer's feed-forward a gated, RMS-normed projection of this many
    #                                columns of a second embedding table (layer i owns columns [i dim, (i+1) dim))

    @property
    def num_layers(self) -> int:
        return len(self.runs)

    @property
    def runs(self) -> list:
        """Layer index of every layer run, in order (the looped range repeated); pages and state are per run."""
        n = len(self.layers)
        if self.share is not None:
            return [int(j) for j in self.share]
        if not self.loop or self.loop[2] <= 1:
            return list(range(n))
        a, b, t = self.loop
        return list(range(a)) + list(range(a, b)) * t + list(range(b, n))

    def param_count(self) -> int:
        d = self.hidden_size
        n = (1 if self.tied_head else 2) * self.vocab_size * d + d
        own = set(self.runs)
        for i, l in enumerate(self.layers):
            if i not in own:
                continue
            m = l.mixer
            if hasattr(m, "params"):
                n += m.params(d)
            elif m.kind == "mlstm":
                n += d * (2 * m.heads * m.dim + 2 * m.heads * m.vdim) + 2 * m.heads * (d + 1) + m.heads * m.vdim * (d + 1)
            else:
                n += d * (m.heads * (m.dim + m.rot_dim) + m.kv_rank + m.rot_dim + m.heads) + m.kv_rank
                n += m.kv_rank * m.heads * (m.dim + m.vdim) + m.heads * m.vdim * d
            n += d * (2 if self.residual == "sandwich" else 1)
            if l.ff is not None:
                f = l.ff
                n += d * (2 if self.residual == "sandwich" else 1)
                n += {"dense": lambda: 2 * d * f.ff, "glu": lambda: 3 * d * f.ff,
                      "moe": lambda: (f.experts * f.ff + f.shared_ff) * 2 * d + (f.experts + f.identity) * (d + f.correction),
                      "moe_glu": lambda: f.experts * (3 * d * f.ff + d + 1),
                      "moe_group_glu": lambda: f.experts * (3 * d * f.ff + d) + (
                          3 * d * f.shared_ff + d if f.shared_ff else 0)}[f.kind]()
            if self.token_side:
                n += self.token_side * (2 * d + self.vocab_size) + d
        return n


# -----------------------------------------------------------------------------------------------------------------
# cache: pages for the attention layers, state slots for the recurrent layers
# -----------------------------------------------------------------------------------------------------------------


class HybridCache:
    """Per latent-attention layer run a paged latent cache [NB, BS, kv_rank + rot_dim], per windowed-attention run
    paged keys [NB, BS, G, D] and values [NB, BS, G, Dv] (with pooled blocks also their means, ``kp`` / ``vp``
    [NB, ceil(BS / pool), G, .]: block e of a sequence sits in row e % EP of the sequence's page e // EP), all in the
    activation dtype (block 0 is the engine's scratch block); per recurrent run float32 state rows S [NS, H, D, Dv]
    (the matrix-memory layers also n [NS, H, D] and m [NS, H]; the gated linear recurrence keeps S [NS, width];
    layers with a short convolution also its last conv - 1 inputs, ``hist`` [NS, conv - 1, C] in the activation
    dtype), one row per engine slot plus a scratch row (``scratch_slot``) for the decode rows of slots that hold no
    running sequence.  Tensors are keyed by the index of the layer RUN: a layer inside a loop has one set per pass;
    the two halves of a parallel mixer are keyed (run, 0) and (run, 1).

    A sequence's state needs no reset: a step whose first token sits at position 0 starts from zero."""

    def __init__(self, cfg: HybridConfig, num_blocks: int, block_size: int, device, act_dtype, slots: int):
        self.num_blocks, self.block_size = num_blocks, block_size
        self.slots = slots
        self.scratch_slot = slots
        self.lat: dict = {}
        self.S: dict = {}
        self.n: dict = {}
        self.m: dict = {}
        self.kc: dict = {}
        self.vc: dict = {}
        self.kp: dict = {}
        self.vp: dict = {}
        self.hist: dict = {}
        self._dev, self._at = device, act_dtype
        for li, l in enumerate(cfg.layers[i] for i in cfg.runs):
            self._alloc(li, l.mixer)

    def _alloc(self, li, mx) -> None:
        num_blocks, block_size, slots, device, act_dtype = self.num_blocks, self.block_size, self.slots, self._dev, self._at
        if mx.kind == "parallel":
            self._alloc((li, 0), mx.left)
            self._alloc((li, 1), mx.right)
        elif mx.kind == "latent_attention":
            self.lat[li] = torch.zeros(num_blocks, block_size, mx.kv_rank + mx.rot_dim, device=device, dtype=act_dtype)
        elif mx.kind == "mlstm":
            f32 = dict(device=device, dtype=torch.float32)
            self.S[li] = torch.zeros(slots + 1, mx.heads, mx.dim, mx.vdim, **f32)
            self.n[li] = torch.zeros(slots + 1, mx.heads, mx.dim, **f32)
            self.m[li] = torch.zeros(slots + 1, mx.heads, **f32)
        elif mx.kind == "window_attention":
            pg = dict(device=device, dtype=act_dtype)
            self.kc[li] = torch.zeros(num_blocks, block_size, mx.kv_heads, mx.dim, **pg)
            self.vc[li] = torch.zeros(num_blocks, block_size, mx.kv_heads, mx.vdim, **pg)
            if mx.pool:
                ep = (block_size + mx.pool - 1) // mx.pool
                self.kp[li] = torch.zeros(num_blocks, ep, mx.kv_heads, mx.dim, **pg)
                self.vp[li] = torch.zeros(num_blocks, ep, mx.kv_heads, mx.vdim, **pg)
        elif mx.kind in ("delta_rule", "gla", "retention"):
            self.S[li] = torch.zeros(slots + 1, mx.heads, mx.dim, mx.vdim, device=device, dtype=torch.float32)
            if mx.kind == "delta_rule":
                ch = 2 * mx.kv_heads * mx.dim + mx.heads * mx.vdim
                self.hist[li] = torch.zeros(slots + 1, max(0, mx.conv - 1), ch, device=device, dtype=act_dtype)
        elif mx.kind == "mamba2":
            self.S[li] = torch.zeros(slots + 1, mx.heads, mx.state, mx.vdim, device=device, dtype=torch.float32)
            self.hist[li] = torch.zeros(slots + 1, max(0, mx.conv - 1), mx.conv_channels, device=device, dtype=act_dtype)
        elif mx.kind == "rglru":
            self.S[li] = torch.zeros(slots + 1, mx.width, device=device, dtype=torch.float32)
            self.hist[li] = torch.zeros(slots + 1, max(0, mx.conv - 1), mx.width, device=device, dtype=act_dtype)

    @staticmethod
    def bytes_per_block(cfg: HybridConfig, block_size: int, act_dtype) -> int:
        eb = 4 if act_dtype == torch.float32 else 2

        def per_page(m) -> int:   # elements one page of this mixer holds
            if m.kind == "parallel":
                return per_page(m.left) + per_page(m.right)
            if m.kind == "latent_attention":
                return block_size * (m.kv_rank + m.rot_dim)
            if m.kind == "window_attention":
                rows = block_size + ((block_size + m.pool - 1) // m.pool if m.pool else 0)
                return rows * m.kv_heads * (m.dim + m.vdim)
            return 0

        return max(1, sum(per_page(cfg.layers[i].mixer) for i in cfg.runs) * eb)

    def move_slots(self, src: torch.Tensor, dst: torch.Tensor) -> None:
        """Slot compaction: the recurrent state rows follow their sequences."""
        for t in (*self.S.values(), *self.n.values(), *self.m.values(), *self.hist.values()):
            t.index_copy_(0, dst, t.index_select(0, src))


# -----------------------------------------------------------------------------------------------------------------
# weights
# -----------------------------------------------------------------------------------------------------------------


@dataclass
class HybridLayerWeights:
    norm1: torch.Tensor
    mix: dict
    norm2: Optional[torch.Tensor] = None
    ff: dict = field(default_factory=dict)
    side: dict = field(default_factory=dict)   # the per-layer token input: w_gate, w_proj, norm, col0
    norm1b: Optional[torch.Tensor] = None      # sandwich stream: the norms on the sublayers' outputs
    norm2b: Optional[torch.Tensor] = None


@dataclass
class HybridWeights:
    embed: torch.Tensor
    layers: list
    final_norm: torch.Tensor
    head: torch.Tensor
    side_embed: Optional[torch.Tensor] = None

    def nbytes(self) -> int:
        n = 0
        for t in (self.embed, self.final_norm, self.head, self.side_embed):
            if t is not None:
                n += t.numel() * t.element_size()
        for l in {id(l): l for l in self.layers}.values():   # a layer that runs on another's weights counts once
            for t in (l.norm1, l.norm2, l.norm1b, l.norm2b, *l.mix.values(), *l.ff.values(), *l.side.values()):
                if isinstance(t, torch.Tensor):
                    n += t.numel() * t.element_size()
                elif isinstance(t, dict):
                    n += sum(v.numel() * v.element_size() for v in t.values() if isinstance(v, torch.Tensor))
        return n


def pack_mlstm(spec: MLSTMSpec, t: dict, device, act_dtype) -> dict:
    """t: q, k, v, g, o, norm, i, i.b, f, f.b (checkpoint layout, [out, in]).  q | k | v | g become one projection,
    the two gate rows one few-row float32-output projection."""
    a = lambda x: x.to(device=device, dtype=act_dtype).contiguous()  # noqa: E731
    f = lambda x: x.to(device=device, dtype=torch.float32).contiguous()  # noqa: E731
    return dict(w_proj=a(torch.cat([t["q"], t["k"], t["v"], t["g"]], 0)), w_if=a(torch.cat([t["i"], t["f"]], 0)),
                b_if=f(torch.cat([t["i.b"], t["f.b"]], 0)), norm=f(t["norm"]), w_o=a(t["o"]))


def pack_latent(spec: LatentAttentionSpec, t: dict, device, act_dtype) -> dict:
    """t: q, dkv, dkv.norm, uk, uv, g, o.  The per-head up-projections are kept as [H, D, rank] and [H, Dv, rank]:
    keys are never materialised (the query is carried into the latent space instead) and the value up-projection
    is applied to the attention's latent-space output."""
    a = lambda x: x.to(device=device, dtype=act_dtype).contiguous()  # noqa: E731
    f = lambda x: x.to(device=device, dtype=torch.float32).contiguous()  # noqa: E731
    return dict(w_q=a(t["q"]), w_dkv=a(t["dkv"]), dkv_norm=f(t["dkv.norm"]), w_g=a(t["g"]), w_o=a(t["o"]),
                w_uk=a(t["uk"].view(spec.heads, spec.dim, spec.kv_rank)),
                w_uv=a(t["uv"].view(spec.heads, spec.vdim, spec.kv_rank)))


def pack_dense(spec: DenseFFSpec, t: dict, device, act_dtype) -> dict:
    a = lambda x: x.to(device=device, dtype=act_dtype).contiguous()  # noqa: E731
    return dict(w_up=a(t["up"]), w_down=a(t["down"]))


def pack_moe(spec: MoEFFSpec, t: dict, device, act_dtype) -> dict:
    """t: router, correction (zeros when the design has none), e<k>.up, e<k>.down and, with a shared expert, shared.up, shared.down.
    Expert weights are stacked [E, ...] for the grouped kernels."""
    a = lambda x: x.to(device=device, dtype=act_dtype).contiguous()  # noqa: E731
    corr = t["correction"] if spec.correction else torch.zeros(spec.experts + spec.identity)
    out = dict(w_router=a(t["router"]), correction=corr.to(device=device, dtype=torch.float32).contiguous(),
               w_up=a(torch.stack([t[f"e{e}.up"] for e in range(spec.experts)])),
               w_down=a(torch.stack([t[f"e{e}.down"] for e in range(spec.experts)])))
    if spec.shared_ff:
        out.update(ws_up=a(t["shared.up"]), ws_down=a(t["shared.down"]))
    return out


def pack_window_attention(spec: WindowAttentionSpec, t: dict, device, act_dtype) -> dict:
    """t: q, k, v, q.norm, k.norm, sink, g, o and, in value-mixing layers, vmix.  q | k | v become one projection
    (q | k when the values are the keys; q | k | v | g with a gate per output column); per-head gate rows are a
    few-row float32-output projection."""
    a = lambda x: x.to(device=device, dtype=act_dtype).contiguous()  # noqa: E731
    f = lambda x: x.to(device=device, dtype=torch.float32).contiguous()  # noqa: E731
    rows = [t["q"], t["k"]] + ([] if spec.v_from_k else [t["v"]]) + ([t["g"]] if spec.gate and spec.gate_wide else [])
    out = dict(w_qkv=a(torch.cat(rows, 0)), w_o=a(t["o"]))
    if spec.qk_norm:
        out.update(q_norm=f(t["q.norm"]), k_norm=f(t["k.norm"]))
    if spec.sink:
        out["sink"] = f(t["sink"])
    if spec.gate and not spec.gate_wide:
        out["w_g"] = a(t["g"])
    if spec.bias:
        out["b_qkv"] = a(torch.cat([t["q.b"], t["k.b"], t["v.b"]], 0))
    if spec.v_mix and not spec.v_mix_first:
        out["vmix"] = f(t["vmix"]).reshape(1)
    return out


def pack_mamba2(spec: Mamba2Spec, t: dict, device, act_dtype) -> dict:
    """t: in ([z | x | B | C | dt] rows), conv, conv.b, dt_bias, A_log, D, norm, o.  The dt rows leave the big
    projection for a few-row float32-output projection whose bias is dt_bias."""
    a = lambda x: x.to(device=device, dtype=act_dtype).contiguous()  # noqa: E731
    f = lambda x: x.to(device=device, dtype=torch.float32).contiguous()  # noqa: E731
    n = 2 * spec.inner + 2 * spec.groups * spec.state
    return dict(w_in=a(t["in"][:n]), w_dt=a(t["in"][n:]), b_dt=f(t["dt_bias"]), taps=f(t["conv"]),
                b_conv=f(t["conv.b"]), a_log=f(t["A_log"]), skip=f(t["D"]), norm=f(t["norm"]), w_o=a(t["o"]))


def pack_rglru(spec: RGLRUSpec, t: dict, device, act_dtype) -> dict:
    """t: y, y.b, x, x.b, conv, conv.b, ra, ra.b, ri, ri.b, lam, o.  y | x are one biased projection; the two gate
    matrices of a block become one [blocks, in, 2 out] operand (its product accumulates and lands in float32);
    softplus(lam) is formed once, in float32."""
    a = lambda x: x.to(device=device, dtype=act_dtype).contiguous()  # noqa: E731
    f = lambda x: x.to(device=device, dtype=torch.float32).contiguous()  # noqa: E731
    wg = torch.cat([t["ra"].float().transpose(1, 2), t["ri"].float().transpose(1, 2)], 2)
    bg = torch.cat([t["ra.b"].float(), t["ri.b"].float()], 1)[:, None, :]
    return dict(w_yx=a(torch.cat([t["y"], t["x"]], 0)), b_yx=a(torch.cat([t["y.b"], t["x.b"]], 0)), taps=f(t["conv"]),
                b_conv=f(t["conv.b"]), w_gates=a(wg), b_gates=f(bg),
                sp=f(torch.nn.functional.softplus(t["lam"].float(), threshold=30.0)), w_o=a(t["o"]))


def pack_delta_rule(spec: DeltaRuleSpec, t: dict, device, act_dtype) -> dict:
    """t: q, k, v (+ .conv each), b, a, dt_bias, A_log, g, norm, o.  q | k | v | g are one projection, the
    convolution taps of q | k | v one [C, conv] float32 table, decay and write-strength rows one few-row
    float32-output projection (bias: dt_bias for the decay rows, zero for the others)."""
    a = lambda x: x.to(device=device, dtype=act_dtype).contiguous()  # noqa: E731
    f = lambda x: x.to(device=device, dtype=torch.float32).contiguous()  # noqa: E731
    return dict(w_proj=a(torch.cat([t["q"], t["k"], t["v"], t["g"]], 0)),
                taps=f(torch.cat([t["q.conv"], t["k.conv"], t["v.conv"]], 0)),
                w_ab=a(torch.cat([t["a"], t["b"]], 0)),
                b_ab=f(torch.cat([t["dt_bias"].float(), torch.zeros(spec.heads)], 0)), a_log=f(t["A_log"]),
                norm=f(t["norm"].float().repeat(spec.heads)), w_o=a(t["o"]))


def pack_gla(spec: GLASpec, t: dict, device, act_dtype) -> dict:
    """t: q, k, v, g, a1, a2, a2.b, norm, o.  q | k | v | g are one projection; the decay's low-rank projection keeps
    float32 outputs (a1 through the few-row projection, a2 as a float32 matrix)."""
    a = lambda x: x.to(device=device, dtype=act_dtype).contiguous()  # noqa: E731
    f = lambda x: x.to(device=device, dtype=torch.float32).contiguous()  # noqa: E731
    return dict(w_proj=a(torch.cat([t["q"], t["k"], t["v"], t["g"]], 0)), w_a1=a(t["a1"]), w_a2t=f(t["a2"].float().t()),
                b_a2=f(t["a2.b"]), norm=f(t["norm"].float().repeat(spec.heads)), w_o=a(t["o"]))


def pack_retention(spec: RetentionSpec, t: dict, device, act_dtype) -> dict:
    """t: q, k, v, g, o.  q | k | v | g are one projection; the decays are a float32 row, one number per head."""
    a = lambda x: x.to(device=device, dtype=act_dtype).contiguous()  # noqa: E731
    return dict(w_proj=a(torch.cat([t["q"], t["k"], t["v"], t["g"]], 0)), w_o=a(t["o"]),
                decay=torch.tensor(list(spec.decay), dtype=torch.float64).to(device=device, dtype=torch.float32),
                ones=torch.ones(spec.heads * spec.vdim, device=device, dtype=torch.float32))


def pack_parallel(spec: ParallelSpec, t: dict, device, act_dtype) -> dict:
    """t: left.* and right.* (each side's own tensors) plus left.out and right.out, the weights of the two outputs'
    norms over the model width."""
    f = lambda x: x.to(device=device, dtype=torch.float32).contiguous()  # noqa: E731
    side = lambda p: {k[len(p):]: v for k, v in t.items() if k.startswith(p) and k != p + "out"}  # noqa: E731
    return dict(left=MIXERS[spec.left.kind][1](spec.left, side("left."), device, act_dtype),
                right=MIXERS[spec.right.kind][1](spec.right, side("right."), device, act_dtype),
                out_l=f(t["left.out"]), out_r=f(t["right.out"]))


def pack_glu(spec: GluFFSpec, t: dict, device, act_dtype) -> dict:
    a = lambda x: x.to(device=device, dtype=act_dtype).contiguous()  # noqa: E731
    return dict(w_gu=a(torch.cat([t["gate"], t["up"]], 0)), w_down=a(t["down"]))


def pack_moe_glu(spec: MoEGluSpec, t: dict, device, act_dtype) -> dict:
    """t: router, router.b, e<k>.gate, e<k>.up, e<k>.down.  Per expert gate rows then up rows, stacked [E, 2F, d]."""
    a = lambda x: x.to(device=device, dtype=act_dtype).contiguous()  # noqa: E731
    out = dict(w_router=a(t["router"]), b_router=t["router.b"].to(device=device, dtype=torch.float32).contiguous(),
               w_gu=a(torch.stack([torch.cat([t[f"e{e}.gate"], t[f"e{e}.up"]], 0) for e in range(spec.experts)])),
               w_down=a(torch.stack([t[f"e{e}.down"] for e in range(spec.experts)])))
    d = out["w_gu"].shape[2]
    if act_dtype == torch.bfloat16 and torch.device(device).type == "cuda" and d % 128 == 0 and spec.ff % 128 == 0:
        # prompt portions take the grouped matrix-core path, which wants gate and up rows interleaved per tile
        out["w_gu"] = out["w_gu"][:, hops.moe_glu_row_order(spec.ff).to(out["w_gu"].device)].contiguous()
        out["gu_tiled"] = True
    return out


def pack_moe_group_glu(spec: MoEGroupGluSpec, t: dict, device, act_dtype) -> dict:
    """t: router, e<k>.gate / .up / .down and, with a shared expert, shared.gate / .up / .down / .sg."""
    a = lambda x: x.to(device=device, dtype=act_dtype).contiguous()  # noqa: E731
    out = pack_moe_glu(spec, {**t, "router.b": torch.zeros(spec.experts)}, device, act_dtype)
    del out["b_router"]
    if spec.shared_ff:
        out.update(ws_gu=a(torch.cat([t["shared.gate"], t["shared.up"]], 0)), ws_down=a(t["shared.down"]),
                   ws_gate=a(t["shared.sg"].reshape(1, -1)))
    return out


def rope_cos_sin(base: float, dims: int, max_pos: int, device, scaling: Optional[tuple] = None) -> torch.Tensor:
    """[max_pos, dims] float32: cos(p f_i) for i < dims/2, then sin(p f_i), f_i = base^(-2i/dims); angles in float64
    before the rounding to float32.  ``scaling``:

    (factor, low, high, original): frequencies whose wavelength is shorter than original/high stay, those longer than
        original/low are divided by factor, and between the two the frequency is interpolated linearly in
        original/wavelength;
    ("linear", factor): every frequency is divided by factor;
    ("ramp", factor, original, fast, slow): with n(t) = dims ln(original / (2 pi t)) / (2 ln base) the pair index at
        which ``original`` positions make t turns, lo = max(floor(n(fast)), 0), hi = min(ceil(n(slow)), dims - 1) and
        r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1), the frequency is f_i / factor r_i + f_i (1 - r_i), and
        cos and sin are multiplied by 0.1 ln(factor) + 1."""
    import math

    inv = base ** (-torch.arange(0, dims, 2, dtype=torch.float64) / dims)
    mag = 1.0
    if scaling is not None and scaling[0] == "linear":
        inv = inv / float(scaling[1])
    elif scaling is not None and scaling[0] == "ramp":
        factor, orig, fast, slow = (float(v) for v in scaling[1:])
        where = lambda t: dims * math.log(orig / (2 * math.pi * t)) / (2 * math.log(base))  # noqa: E731
        lo, hi = max(math.floor(where(fast)), 0), min(math.ceil(where(slow)), dims - 1)
        r = ((torch.arange(dims // 2, dtype=torch.float64) - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        inv = inv / factor * r + inv * (1 - r)
        mag = 0.1 * math.log(factor) + 1.0
    elif scaling is not None:
        factor, low, high, orig = (float(v) for v in scaling)
        wl = 2 * math.pi / inv
        s = ((orig / wl - low) / (high - low)).clamp(0.0, 1.0) if high != low else torch.ones_like(inv)
        mid = (1 - s) * inv / factor + s * inv
        inv = torch.where(wl < orig / high, inv, torch.where(wl > orig / low, inv / factor, mid))
    fr = torch.outer(torch.arange(max_pos, dtype=torch.float64), inv)
    return (torch.cat([fr.cos(), fr.sin()], 1) * mag).float().to(device)


# -----------------------------------------------------------------------------------------------------------------
# mixers and feed-forwards (one function per kind: h [T, d] in the activation dtype -> [T, d])
# -----------------------------------------------------------------------------------------------------------------


@dataclass
class StepMeta:
    """One step's flattened token stream, prefill chunks and decode rows alike: sequence b owns tokens
    q_start[b]:q_start[b+1], the first of them at position pos0[b], its pages in block_table[b], its state in row
    slots[b] of the recurrent-state tensors."""
    ids: torch.Tensor
    pos: torch.Tensor
    tok_seq: torch.Tensor
    block_table: torch.Tensor
    q_start: torch.Tensor
    pos0: torch.Tensor
    slots: torch.Tensor
    last_idx: torch.Tensor
    max_q: int
    shared: dict = field(default_factory=dict)  # what one layer of a step leaves for later layers of the same step


def mix_mlstm(model, li: int, spec: MLSTMSpec, w: dict, h, meta: StepMeta, cache: HybridCache):
    H, D, Dv = spec.heads, spec.dim, spec.vdim
    proj = hops.matmul(h, w["w_proj"])
    gate_pre = hops.rowdot(h, w["w_if"], w["b_if"])
    o = hops.mlstm_scan(proj, gate_pre, meta.q_start, meta.pos0, meta.slots, cache.S[li], cache.n[li], cache.m[li],
                        H, D, Dv, spec.gate_cap, meta.max_q)
    y = hops.mlstm_out(o, proj, 2 * H * D + H * Dv, w["norm"], model.cfg.norm_eps, model.act_dtype)
    return hops.matmul(y, w["w_o"])


def mix_latent_attention(model, li: int, spec: LatentAttentionSpec, w: dict, h, meta: StepMeta, cache: HybridCache):
    T = h.shape[0]
    H, D, R, rank = spec.heads, spec.dim, spec.rot_dim, spec.kv_rank
    q = hops.matmul(h, w["w_q"]).view(T, H, D + R)
    dkv = hops.matmul(h, w["w_dkv"])
    gate = hops.rowdot(h, w["w_g"])
    hops.latent_prep(q, dkv, meta.pos, meta.tok_seq, meta.block_table, w["dkv_norm"], model.cfg.norm_eps,
                     model.rope[li], spec.rope_dims, rank, cache.lat[li])
    # the query goes into the latent space (q_u W_uk per head), so a key is the cached row itself; the output
    # comes back through W_uv per head
    qa = torch.empty(T, H, rank + R, device=h.device, dtype=h.dtype)
    qa[:, :, :rank] = torch.bmm(q[:, :, :D].transpose(0, 1), w["w_uk"]).transpose(0, 1)
    qa[:, :, rank:] = q[:, :, D:]
    oa = hops.latent_attention(qa, cache.lat[li], meta.block_table, meta.q_start, meta.pos, gate, spec.scale, rank,
                               model.act_dtype, meta.max_q)
    ov = torch.bmm(oa.transpose(0, 1), w["w_uv"].transpose(1, 2)).transpose(0, 1).reshape(T, H * spec.vdim)
    return hops.matmul(ov, w["w_o"])


def mix_window_attention(model, li, spec: WindowAttentionSpec, w: dict, h, meta: StepMeta, cache: HybridCache):
    H, G, D, Dv = spec.heads, spec.kv_heads, spec.dim, spec.vdim
    qkv = hops.matmul(h, w["w_qkv"], w.get("b_qkv"))
    gate = hops.rowdot(h, w["w_g"]) if spec.gate and not spec.gate_wide else None
    mixes = spec.v_mix and not spec.v_mix_first
    v_tab = model.rope_v.get(li)
    v = hops.window_prep(qkv, H, G, D, Dv, meta.shared["v_first"] if mixes else None, w.get("vmix"), meta.pos,
                         meta.tok_seq, meta.block_table, w.get("q_norm"), w.get("k_norm"), model.cfg.norm_eps,
                         model.rope.get(li), spec.rope_dims, cache.kc[li], cache.vc[li], spec.v_mix_first,
                         H * D if spec.v_from_k else -1, v_tab)
    if spec.v_mix_first:
        meta.shared["v_first"] = v
    pooled = spec.pool > 0 and spec.window > 0
    if pooled:   # the blocks this step's tokens complete get their means before any query of the step looks
        hops.pool_blocks(cache.kc[li], cache.vc[li], cache.kp[li], cache.vp[li], meta.block_table, meta.q_start,
                         meta.pos0, spec.pool, meta.max_q)
    o = hops.window_attention(qkv, cache.kc[li], cache.vc[li], meta.block_table, meta.q_start, meta.pos, w.get("sink"),
                              gate, spec.scale, spec.window, spec.keep_first, H, model.act_dtype, meta.max_q,
                              spec.chunk, spec.pool if pooled else 0, cache.kp.get(li), cache.vp.get(li), v_tab,
                              (H + G) * D + G * Dv if spec.gate and spec.gate_wide else -1)
    return hops.matmul(o, w["w_o"])


def mix_retention(model, li, spec: RetentionSpec, w: dict, h, meta: StepMeta, cache: HybridCache):
    H, D, Dv = spec.heads, spec.dim, spec.vdim
    proj = hops.matmul(h, w["w_proj"])          # q | k | v | g
    hops.rotate_qk(proj, 0, H * D, H, H, D, spec.rope_dims, model.rope.get(li), meta.pos, 1.0, D ** -0.5)
    o = hops.linear_scan(proj, 0, H * D, 2 * H * D, None, None, 1.0, w["decay"], None, meta.q_start, meta.pos0,
                         meta.slots, cache.S[li], H, H, D, Dv)
    return hops.matmul(hops.head_norm_gate(o, proj, 2 * H * D + H * Dv, w["ones"], model.cfg.norm_eps, True,
                                           model.act_dtype), w["w_o"])


@dataclass
class PairOut:
    """What a parallel mixer hands to the stream's join: the two outputs and the weights of their norms."""
    y: torch.Tensor
    y2: torch.Tensor
    w: torch.Tensor
    w2: torch.Tensor


def mix_parallel(model, li, spec: ParallelSpec, w: dict, h, meta: StepMeta, cache: HybridCache):
    yl = MIXERS[spec.left.kind][0](model, (li, 0), spec.left, w["left"], h, meta, cache)
    yr = MIXERS[spec.right.kind][0](model, (li, 1), spec.right, w["right"], h, meta, cache)
    return PairOut(yl, yr, w["out_l"], w["out_r"])


def mix_mamba2(model, li: int, spec: Mamba2Spec, w: dict, h, meta: StepMeta, cache: HybridCache):
    H, P, N, G = spec.heads, spec.vdim, spec.state, spec.groups
    inner, GN = spec.inner, spec.groups * spec.state
    proj = hops.matmul(h, w["w_in"])                 # z | x | B | C
    dt_pre = hops.rowdot(h, w["w_dt"], w["b_dt"])    # float32 step pre-activations, bias included
    xbc = hops.short_conv(proj, w["taps"], meta.tok_seq, meta.q_start, meta.pos0, meta.slots, cache.hist[li], True,
                          w["b_conv"], inner)        # x | B | C after convolution and SiLU
    decay, dt = hops.ssm_prep(dt_pre, w["a_log"])
    # state rows = B, read by C, written with dt x: S <- decay S + B (dt x)^T, o = S^T C
    o = hops.linear_scan(xbc, inner + GN, inner, 0, None, None, 1.0, decay, None, meta.q_start, meta.pos0, meta.slots,
                         cache.S[li], G, H, N, P, dt)
    y = hops.gated_group_norm(o, xbc, 0, w["skip"], proj, 0, w["norm"], spec.norm_groups, model.cfg.norm_eps,
                              model.act_dtype)
    return hops.matmul(y, w["w_o"])


def mix_rglru(model, li: int, spec: RGLRUSpec, w: dict, h, meta: StepMeta, cache: HybridCache):
    W = spec.width
    proj = hops.matmul(h, w["w_yx"], w["b_yx"])      # y branch | x branch
    u = hops.short_conv(proj, w["taps"], meta.tok_seq, meta.q_start, meta.pos0, meta.slots, cache.hist[li], False,
                        w["b_conv"], W)
    gates = hops.block_gates(u, w["w_gates"], w["b_gates"])   # float32 [blocks, T, 2 W / blocks]
    o = hops.rglru_scan(u, gates, w["sp"], spec.c, proj, 0, meta.q_start, meta.pos0, meta.slots, cache.S[li],
                        model.act_dtype, meta.max_q)
    return hops.matmul(o, w["w_o"])


def mix_delta_rule(model, li: int, spec: DeltaRuleSpec, w: dict, h, meta: StepMeta, cache: HybridCache):
    H, HK, D, Dv = spec.heads, spec.kv_heads, spec.dim, spec.vdim
    C = 2 * HK * D + H * Dv
    proj = hops.matmul(h, w["w_proj"])          # q | k | v | g
    ab = hops.rowdot(h, w["w_ab"], w["b_ab"])   # decay and write-strength pre-activations, float32
    y = hops.short_conv(proj, w["taps"], meta.tok_seq, meta.q_start, meta.pos0, meta.slots, cache.hist[li], True)
    qscale, kscale, decay, beta = hops.delta_prep(y, ab, w["a_log"], HK, H, D, D ** -0.5)
    o = hops.linear_scan(y, 0, HK * D, 2 * HK * D, qscale, kscale, 1.0, decay, beta, meta.q_start, meta.pos0,
                         meta.slots, cache.S[li], HK, H, D, Dv)
    return hops.matmul(hops.head_norm_gate(o, proj, C, w["norm"], model.cfg.norm_eps, True, model.act_dtype), w["w_o"])


def mix_gla(model, li: int, spec: GLASpec, w: dict, h, meta: StepMeta, cache: HybridCache):
    H, D, Dv = spec.heads, spec.dim, spec.vdim
    proj = hops.matmul(h, w["w_proj"])          # q | k | v | g
    z = torch.addmm(w["b_a2"], hops.rowdot(h, w["w_a1"]), w["w_a2t"])  # float32 decay logits [T, H D]
    decay = hops.decay_pow(z, 1.0 / spec.tau)
    o = hops.linear_scan(proj, 0, H * D, 2 * H * D, None, None, D ** -0.5, decay, None, meta.q_start, meta.pos0,
                         meta.slots, cache.S[li], H, H, D, Dv)
    return hops.matmul(hops.head_norm_gate(o, proj, 2 * H * D + H * Dv, w["norm"], model.cfg.norm_eps, True,
                                           model.act_dtype), w["w_o"])


def ff_glu(model, spec: GluFFSpec, w: dict, h):
    return hops.matmul(hops.glu(hops.matmul(h, w["w_gu"]), spec.limit, spec.slope, spec.shift, model.act_dtype),
                       w["w_down"])


def ff_moe_glu(model, spec: MoEGluSpec, w: dict, h):
    idx, wt = hops.moe_route_topk(h, w["w_router"], w["b_router"], spec.top)
    return hops.moe_glu_ffn(h, idx, wt, w["w_gu"], w["w_down"], spec.limit, spec.slope, spec.shift, model.act_dtype,
                            bool(w.get("gu_tiled", False)))


def ff_moe_group_glu(model, spec: MoEGroupGluSpec, w: dict, h):
    """Returns the routed experts' sum and, with a shared expert, (sum, shared output, float32 gate logits [T, 1]):
    the stream's join adds sigmoid(gate) * shared."""
    idx, wt = hops.moe_route_group(h, w["w_router"], spec.top, spec.groups, spec.keep, spec.scale)
    y = hops.moe_glu_ffn(h, idx, wt, w["w_gu"], w["w_down"], spec.limit, spec.slope, spec.shift, model.act_dtype,
                         bool(w.get("gu_tiled", False)))
    if not spec.shared_ff:
        return y
    ys = hops.matmul(hops.glu(hops.matmul(h, w["ws_gu"]), spec.limit, spec.slope, spec.shift, model.act_dtype),
                     w["ws_down"])
    return y, ys, hops.rowdot(h, w["ws_gate"])


def ff_dense(model, spec: DenseFFSpec, w: dict, h):
    return hops.matmul(hops.act_inplace(hops.matmul(h, w["w_up"]), spec.act), w["w_down"])


def ff_moe(model, spec: MoEFFSpec, w: dict, h):
    """Returns the routed experts' sum and, with a shared expert, (sum, shared output): the stream's join adds both."""
    idx, wt = hops.moe_route(h, w["w_router"], w["correction"], spec.top)
    y = hops.moe_ffn(h, idx, wt, w["w_up"], w["w_down"], spec.act, model.act_dtype)
    if not spec.shared_ff:
        return y
    return y, hops.matmul(hops.act_inplace(hops.matmul(h, w["ws_up"]), spec.act), w["ws_down"])


MIXERS = {"mlstm": (mix_mlstm, pack_mlstm), "latent_attention": (mix_latent_attention, pack_latent),
          "window_attention": (mix_window_attention, pack_window_attention),
          "delta_rule": (mix_delta_rule, pack_delta_rule), "gla": (mix_gla, pack_gla),
          "mamba2": (mix_mamba2, pack_mamba2), "rglru": (mix_rglru, pack_rglru),
          "retention": (mix_retention, pack_retention), "parallel": (mix_parallel, pack_parallel)}
FEED_FORWARDS = {"dense": (ff_dense, pack_dense), "moe": (ff_moe, pack_moe), "glu": (ff_glu, pack_glu),
                 "moe_glu": (ff_moe_glu, pack_moe_glu), "moe_group_glu": (ff_moe_group_glu, pack_moe_group_glu)}
RECURRENT_MIXERS = ("mlstm", "delta_rule", "gla", "mamba2", "rglru", "retention")


def _is_recurrent(mx) -> bool:
    """Does a sequence hold something beyond the tokens of its own pages?  A recurrent state; or pooled blocks, whose
    pair sits in the page e // EP while its tokens may lie on later pages (blocks off the page grid), so that a page
    shared between sequences as a common prefix could be written with one sequence's continuation."""
    if mx.kind == "parallel":
        return _is_recurrent(mx.left) or _is_recurrent(mx.right)
    return mx.kind in RECURRENT_MIXERS or (mx.kind == "window_attention" and mx.pool > 0 and mx.window > 0)


# -----------------------------------------------------------------------------------------------------------------
# model
# -----------------------------------------------------------------------------------------------------------------


class HybridDecoder:
    """Serves through the same engine as the Llama models (same step batches, block manager, sampler).  What the
    engine needs from a model: ``cfg.vocab_size``, ``make_cache``, ``cache_bytes_per_block``, ``prefill_batch``,
    ``forward``, ``recurrent`` (state slots: no prefix sharing between sequences) and ``hq`` / ``hkv`` for its
    decode-split heuristics."""
    recurrent = True
    hq = hkv = 1

    def __init__(self, cfg: HybridConfig, weights: HybridWeights, device="cpu", max_position: int | None = None,
                 act_dtype=torch.bfloat16, tp: TPContext | None = None):
        self.cfg, self.w = cfg, weights
        self.tp = tp or TPContext.single()
        if self.tp.world > 1:
            raise NotImplementedError("the hybrid decoders run on full-weight ranks (data-parallel replicas only)")
        self.device = torch.device(device)
        self.act_dtype = act_dtype
        self.sequence_parallel = False
        self.decode_overlap_rows = 0
        P = max_position or cfg.max_position
        # rotation tables by run (the halves of a parallel mixer: (run, 0) and (run, 1)); equal tables are one tensor
        self.rope, self.rope_v, made = {}, {}, {}

        def table(base, dims, scaling):
            key = (float(base), int(dims), tuple(scaling) if scaling else None)
            if key not in made:
                made[key] = rope_cos_sin(base, dims, P, self.device, scaling)
            return made[key]

        def tables(key, mx):
            if mx.kind == "parallel":
                tables((key, 0), mx.left)
                tables((key, 1), mx.right)
            elif mx.kind in ("latent_attention", "window_attention", "retention"):
                if mx.rope_dims:
                    self.rope[key] = table(mx.rope_base, mx.rope_dims, getattr(mx, "rope_scaling", None))
                if getattr(mx, "v_rot", False):
                    self.rope_v[key] = table(mx.rope_base, mx.vdim, None)

        for ri, l in enumerate(cfg.layers[i] for i in cfg.runs):
            tables(ri, l.mixer)
        self.recurrent = any(_is_recurrent(l.mixer) for l in cfg.layers)
        if cfg.residual not in ("out_norm", "post_norm", "pre_norm", "sandwich"):
            raise ValueError(f"unknown residual rule {cfg.residual!r}")
        if cfg.token_side and cfg.residual != "pre_norm":
            raise ValueError("the per-layer token input is part of the pre-norm stream's join")

    # ---- what the engine calls --------------------------------------------------------------------------------
    def make_cache(self, num_blocks: int, block_size: int, slots: int, kv_dtype: str = "bf16", k_scale: float = 1.0,
                   v_scale: float = 1.0) -> HybridCache:
        if kv_dtype != "bf16":
            raise ValueError("the hybrid decoders cache in their activation dtype (kv_dtype must stay 'bf16')")
        return HybridCache(self.cfg, num_blocks, block_size, self.device, self.act_dtype, slots)

    def cache_bytes_per_block(self, block_size: int, kv_dtype: str = "bf16") -> int:
        return HybridCache.bytes_per_block(self.cfg, block_size, self.act_dtype)

    def prefill_batch(self, chunks, starts, block_tables, slots, max_blocks=None, nqt: int = 2, split: int = 1,
                      want=None) -> StepBatch:
        """Host builder of a prefill step: chunks[b] are sequence b's next tokens, the first at position starts[b];
        slots[b] its state slot.  ``want``: token indices (into the flattened stream) whose logits are asked for
        (default: every sequence's last token)."""
        ids, pos, tok_seq, qs = [], [], [], [0]
        for b, (toks, s0) in enumerate(zip(chunks, starts)):
            ids += toks
            pos += list(range(s0, s0 + len(toks)))
            tok_seq += [b] * len(toks)
            qs.append(qs[-1] + len(toks))
        mb = max_blocks or max(len(x) for x in block_tables)
        bt = torch.zeros(len(chunks), mb, dtype=torch.int32)
        for b, blks in enumerate(block_tables):
            bt[b, :len(blks)] = torch.tensor(blks, dtype=torch.int32)
        it = lambda x: torch.tensor(x, dtype=torch.int32)  # noqa: E731
        last = torch.tensor([q - 1 for q in qs[1:]] if want is None else list(want), dtype=torch.int64)
        dv = lambda t: h2d(t, self.device)  # noqa: E731
        mq = max((len(c) for c in chunks), default=0)
        return StepBatch(dv(it(ids)), dv(it(pos)), dv(it(tok_seq)), dv(bt), dv(it(qs)),
                         dv(it([s0 + len(t) for t, s0 in zip(chunks, starts)])), dv(last),
                         dv(torch.zeros(max(1, len(chunks)), 2, dtype=torch.int32)), len(chunks), nqt, 1,
                         slots=dv(it(list(slots))), max_q=mq)

    def _meta(self, sb: StepBatch) -> StepMeta:
        def one(p: StepBatch) -> StepMeta:
            if p.slots is None:
                raise ValueError("a hybrid decoder's step batch needs the sequences' state slots")
            if p.tiles is None:  # decode rows: token i is sequence i
                return StepMeta(p.ids, p.pos, p.tok_seq, p.block_table, p.q_start, p.pos, p.slots, p.last_idx, 1)
            pos0 = p.pos.index_select(0, p.q_start[:-1].long().clamp(max=max(0, p.pos.numel() - 1)))
            return StepMeta(p.ids, p.pos, p.tok_seq, p.block_table, p.q_start, pos0, p.slots, p.last_idx,
                            p.max_q or p.ids.numel())

        m = one(sb)
        if sb.dec is None:
            return m
        d = one(sb.dec)
        T, B = m.ids.numel(), m.block_table.shape[0]
        return StepMeta(torch.cat([m.ids, d.ids]), torch.cat([m.pos, d.pos]), torch.cat([m.tok_seq, d.tok_seq + B]),
                        torch.cat([m.block_table, d.block_table]), torch.cat([m.q_start, d.q_start[1:] + T]),
                        torch.cat([m.pos0, d.pos0]), torch.cat([m.slots, d.slots]), sb.last_idx, max(m.max_q, 1))

    def forward(self, sb: StepBatch, cache: HybridCache, logits_dtype=torch.float32) -> torch.Tensor:
        """Logits [len(sb.last_idx), V] of the tokens at sb.last_idx (with ``sb.dec``: indices into prefill tokens
        followed by decode rows)."""
        cfg, w, at = self.cfg, self.w, self.act_dtype
        meta = self._meta(sb)
        x, h = hops.embed_rows(meta.ids, w.embed, at, cfg.embed_scale, cfg.residual not in ("pre_norm", "sandwich"))
        if cfg.residual == "pre_norm":
            self._forward_pre_norm(x, meta, cache)
        elif cfg.residual == "sandwich":
            self._forward_sandwich(x, meta, cache)
        else:
            for ri, li in enumerate(cfg.runs):   # the cache is keyed by run, the weights by layer
                spec, lw = cfg.layers[li], w.layers[li]
                y = MIXERS[spec.mixer.kind][0](self, ri, spec.mixer, lw.mix, h, meta, cache)
                h = self._join(y, x, lw.norm1)
                if spec.ff is not None:
                    y = FEED_FORWARDS[spec.ff.kind][0](self, spec.ff, lw.ff, h)
                    h = self._join(y, x, lw.norm2)
                if self.layer_tap is not None:
                    self.layer_tap(ri, x)
        xs = x.index_select(0, meta.last_idx)
        if cfg.residual == "out_norm":
            xn = hops.layer_norm(xs, w.final_norm, cfg.norm_eps, at)
        else:
            xn = hops.rms_norm(xs, w.final_norm, cfg.norm_eps, at, cfg.norm_groups if cfg.residual == "sandwich" else 1)
        logits = hops.matmul(xn, w.head).float()
        if cfg.logit_scale != 1.0:
            logits = logits * cfg.logit_scale
        return logits if logits.dtype == logits_dtype else logits.to(logits_dtype)

    def _forward_pre_norm(self, x, meta: StepMeta, cache: HybridCache) -> None:
        """x <- x + mixer(norm1(x)); x <- x + ff(norm2(x)); with a per-layer token input
        x <- x + rms_unit(W_proj (gelu(W_gate x) * e)) * w, e the layer's columns of each token's row of a second
        embedding table.  Every join kernel adds to the float32 stream in place and emits what the next sublayer
        reads: the next norm's output, or the stream's copy in the activation dtype for the token input's gate."""
        cfg, w, at, eps = self.cfg, self.w, self.act_dtype, self.cfg.norm_eps
        runs = cfg.runs
        h = hops.rms_norm(x, w.layers[runs[0]].norm1, eps, at) if runs else None
        for ri, li in enumerate(runs):
            spec, lw = cfg.layers[li], w.layers[li]
            nxt = w.layers[runs[ri + 1]].norm1 if ri + 1 < len(runs) else None   # the last run emits nothing:
            last = ri + 1 == len(runs)                                           # the final norm reads chosen rows
            y = MIXERS[spec.mixer.kind][0](self, ri, spec.mixer, lw.mix, h, meta, cache)
            y2 = g2 = None
            if spec.ff is not None:
                h = hops.add_rms_norm(y, x, lw.norm2, eps, at)
                y = FEED_FORWARDS[spec.ff.kind][0](self, spec.ff, lw.ff, h)
                if isinstance(y, tuple):
                    y, y2, g2 = y
            if cfg.token_side:
                xa = hops.add_rms_norm(y, x, None, eps, at, y2, g2)
                g = hops.token_gate(hops.matmul(xa, lw.side["w_gate"]), meta.ids, w.side_embed, lw.side["col0"], at)
                h = hops.add_rms_norm(hops.matmul(g, lw.side["w_proj"]), x, nxt, eps, at, w_y=lw.side["norm"],
                                      emit=not last)
            else:
                h = hops.add_rms_norm(y, x, nxt, eps, at, y2, g2, emit=not last)
            if self.layer_tap is not None:
                self.layer_tap(ri, x)

    def _forward_sandwich(self, x, meta: StepMeta, cache: HybridCache) -> None:
        """x <- x + norm1b(mixer(norm1(x))); x <- x + norm2b(ff(norm2(x))), every norm an RMS norm over
        ``norm_groups`` equal parts of the row.  One join kernel per sublayer: it norms the sublayer's output (a
        parallel mixer's two outputs are normed over the width and averaged first, a shared expert's output is added
        first), adds it to the float32 stream in place and emits the norm the next sublayer reads."""
        cfg, w, at, eps, ng = self.cfg, self.w, self.act_dtype, self.cfg.norm_eps, self.cfg.norm_groups
        runs = cfg.runs
        h = hops.rms_norm(x, w.layers[runs[0]].norm1, eps, at, ng) if runs else None
        for ri, li in enumerate(runs):
            spec, lw = cfg.layers[li], w.layers[li]
            last = ri + 1 == len(runs)    # the last run emits nothing: the final norm reads the wanted rows only
            nxt = None if last else w.layers[runs[ri + 1]].norm1
            y = MIXERS[spec.mixer.kind][0](self, ri, spec.mixer, lw.mix, h, meta, cache)
            y2 = pair = None
            if isinstance(y, PairOut):
                y, y2, pair = y.y, y.y2, (y.w, y.w2)
            if spec.ff is None:
                h = hops.sandwich_join(y, x, lw.norm1b, nxt, ng, eps, at, y2, pair, emit=not last)
            else:
                h = hops.sandwich_join(y, x, lw.norm1b, lw.norm2, ng, eps, at, y2, pair)
                y = FEED_FORWARDS[spec.ff.kind][0](self, spec.ff, lw.ff, h)
                y, y2 = y if isinstance(y, tuple) else (y, None)
                h = hops.sandwich_join(y, x, lw.norm2b, nxt, ng, eps, at, y2, None, emit=not last)
            if self.layer_tap is not None:
                self.layer_tap(ri, x)

    def _join(self, y, x, w):
        """The residual rule: folds the sublayer output y into the float32 stream x (in place) and returns the
        stream in the activation dtype for the next sublayer."""
        cfg = self.cfg
        if isinstance(y, (tuple, PairOut)):
            raise NotImplementedError("a feed-forward with a separate part needs the pre-norm or the sandwich stream, "
                                      "a parallel mixer the sandwich stream")
        if cfg.residual == "post_norm":
            return hops.scale_add_rms_norm(y, x, w, cfg.residual_alpha, cfg.norm_eps, self.act_dtype)
        return hops.add_layer_norm(y, x, w, cfg.norm_eps, self.act_dtype)

    layer_tap = None  # debugging hook: called with (layer index, residual stream) after every layer
