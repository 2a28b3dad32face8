"""Ops of the hybrid decoders (recurrent matrix-memory layers, linear-state recurrences, latent and windowed
attention, mixtures of experts, layer and RMS norms on a float32 residual stream): gfx950 HIP kernels on the GPU
(csrc/hybrid/*.hip), the PyTorch references of :mod:`.hybrid_ref` on the CPU.

As everywhere in :mod:`chronos.ops` a GPU tensor never falls back silently: it goes to ``torch.ops.chronos.hy_*`` or
raises.  ``CHRONOS_HYBRID_REF=1`` is a bring-up switch that runs the PyTorch references on GPU tensors (it syncs with
the host and cannot be captured into a graph).

Activations are bfloat16 or float32 (one build serves both: the kernels are instantiated for the two); the residual
stream, norms, recurrent state, gates, router and attention scores are float32 in either mode.
"""
from __future__ import annotations

import os

import torch

from . import hybrid_ref as ref
from .hybrid_ref import ACT_GELU, ACT_GLU, ACT_RELU2  # noqa: F401

_REF_ON_GPU = os.environ.get("CHRONOS_HYBRID_REF", "0") not in ("", "0")


def _gpu(t: torch.Tensor) -> bool:
    return t.is_cuda and not _REF_ON_GPU


_lib_loaded = False


def load() -> None:
    """Load (building in-tree if stale) the hybrid kernel library; raises on failure."""
    global _lib_loaded
    if not _lib_loaded:
        from ..native import hybrid_lib

        hybrid_lib()
        _lib_loaded = True


def _k():
    load()
    return torch.ops.chronos


def _f32(act_dtype) -> bool:
    return act_dtype == torch.float32


def matmul(x: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
    """x @ w.T (+ bias): the framework's routed projection GEMMs for bfloat16, the library's float32 GEMM otherwise.
    A biased projection is one library GEMM whose epilogue adds the bias (in the activation dtype, like w) to the
    float accumulator before the rounding."""
    if bias is not None:
        return torch.addmm(bias, x, w.t())
    if x.dtype == torch.bfloat16:
        from . import linear

        return linear(x, w)
    return torch.matmul(x, w.t())


def embed_rows(ids, table, act_dtype, scale: float = 1.0, emit: bool = True):
    """(float32 residual rows times ``scale``, the same rows in the activation dtype or None when ``emit`` is off)."""
    if _gpu(table):
        x = _k().hy_embed(ids, table, scale)
        return x, ((x if _f32(act_dtype) else _k().hy_cast_bf16(x)) if emit else None)
    return ref.embed_rows(ids, table, act_dtype, scale, emit)


def layer_norm(x, w, eps: float, act_dtype):
    if _gpu(x):
        return _k().hy_layer_norm(x, w, eps, _f32(act_dtype))
    return ref.layer_norm(x, w, eps, act_dtype)


def add_layer_norm(y, x, w, eps: float, act_dtype):
    """x (float32 residual, in place) <- x + layer_norm(y) * w; returns the updated rows in the activation dtype
    (x itself when that is float32)."""
    if _gpu(x):
        h = _k().hy_add_layer_norm(y, x, w, eps, _f32(act_dtype))
        return x if _f32(act_dtype) else h
    return ref.add_layer_norm(y, x, w, eps, act_dtype)


def rowdot(h, w, bias=None):
    if _gpu(h):
        return _k().hy_rowdot(h, w, bias)
    return ref.rowdot(h, w, bias)


def act_inplace(x, kind: int):
    if _gpu(x):
        _k().hy_act(x, kind)
        return x
    return ref.act_inplace(x, kind)


def mlstm_scan(proj, gate_pre, q_start, pos0, slots, S, n, m, H: int, D: int, Dv: int, cap: float, max_q: int = 0):
    """``max_q``: the most tokens any sequence brings in this step (a launch-shape hint; 0 = unknown)."""
    if _gpu(proj):
        return _k().hy_mlstm_scan(proj, gate_pre, q_start, pos0, slots, S, n, m, H, D, Dv, cap)
    return ref.mlstm_scan(proj, gate_pre, q_start, pos0, slots, S, n, m, H, D, Dv, cap)


def mlstm_out(o, proj, g_off: int, norm_w, eps: float, act_dtype):
    if _gpu(o):
        return _k().hy_mlstm_out(o, proj, g_off, norm_w, eps, _f32(act_dtype))
    return ref.mlstm_out(o, proj, g_off, norm_w, eps, act_dtype)


def latent_prep(q, dkv, pos, tok_seq, block_table, w_norm, eps: float, cos_sin, dims: int, rank: int, cache) -> None:
    if _gpu(q):
        _k().hy_latent_prep(q, dkv, pos, tok_seq, block_table, w_norm, eps, cos_sin, dims, rank, cache)
    else:
        ref.latent_prep(q, dkv, pos, tok_seq, block_table, w_norm, eps, cos_sin, dims, rank, cache)


def latent_attention(qa, cache, block_table, q_start, pos, gate, scale: float, rank: int, act_dtype, max_q: int):
    """``max_q``: the most tokens any sequence brings in this step (sizes the launch grid)."""
    if _gpu(qa):
        return _k().hy_latent_attention(qa, cache, block_table, q_start, pos, gate, scale, rank, max_q)
    return ref.latent_attention(qa, cache, block_table, q_start, pos, gate, scale, rank, act_dtype)


def moe_route(h, w_router, correction, top: int):
    if _gpu(h):
        return _k().hy_moe_route(h, w_router, correction, top)
    return ref.moe_route(h, w_router, correction, top)


def moe_ffn(h, idx, wt, w_up, w_down, act: int, act_dtype):
    if _gpu(h):
        return _k().hy_moe_ffn(h, idx, wt, w_up, w_down, act)
    return ref.moe_ffn(h, idx, wt, w_up, w_down, act, act_dtype)


# ---- post-norm residual stream, clamped GLU, windowed attention with sinks, linear-state recurrences ---------------


def rms_norm(x, w, eps: float, act_dtype, groups: int = 1):
    """``groups`` > 1: every one of that many equal parts of a row is divided by its own root mean square."""
    if _gpu(x):
        if groups > 1:
            return _k().hy_sandwich_join(None, None, x, None, w, None, None, groups, eps, _f32(act_dtype), False, True)
        return _k().hy_rms_norm(x, w, eps, _f32(act_dtype))
    return ref.rms_norm(x, w, eps, act_dtype, groups)


def scale_add_rms_norm(y, x, w, alpha: float, eps: float, act_dtype):
    """x (float32 residual, in place) <- rms_norm(alpha * x + y) * w; returns the updated rows in the activation
    dtype (x itself when that is float32)."""
    if _gpu(x):
        h = _k().hy_scale_add_rms_norm(y, x, w, alpha, eps, _f32(act_dtype))
        return x if _f32(act_dtype) else h
    return ref.scale_add_rms_norm(y, x, w, alpha, eps, act_dtype)


def glu(gu, limit: float, slope: float, shift: float, act_dtype):
    if _gpu(gu):
        return _k().hy_glu(gu, limit, slope, shift)
    return ref.glu(gu, limit, slope, shift, act_dtype)


def window_prep(qkv, H: int, G: int, D: int, Dv: int, v_first, lam, pos, tok_seq, block_table, q_norm, k_norm,
                eps: float, cos_sin, dims: int, kc, vc, emit_v: bool, v_off: int = -1, v_cos_sin=None):
    """``v_off`` >= 0: the column of qkv where the values start (default: after the keys); ``v_cos_sin``: a rotation
    table over all Dv columns that the values pass before they are cached."""
    if _gpu(qkv):
        v = _k().hy_window_prep(qkv, H, G, D, Dv, v_first, lam, pos, tok_seq, block_table, q_norm, k_norm, eps, cos_sin,
                                dims, kc, vc, emit_v, v_off, v_cos_sin)
        return v if emit_v else None
    return ref.window_prep(qkv, H, G, D, Dv, v_first, lam, pos, tok_seq, block_table, q_norm, k_norm, eps, cos_sin,
                           dims, kc, vc, emit_v, v_off, v_cos_sin)


def pool_blocks(kc, vc, kp, vp, block_table, q_start, pos0, pool: int, max_q: int) -> None:
    """Means of the keys and values of the blocks of ``pool`` positions that this step's tokens complete, into the
    pooled caches.  ``max_q``: the most tokens any sequence brings in this step (sizes the launch grid)."""
    if _gpu(kc):
        _k().hy_pool_blocks(kc, vc, kp, vp, block_table, q_start, pos0, pool, max_q)
    else:
        ref.pool_blocks(kc, vc, kp, vp, block_table, q_start, pos0, pool)


def window_attention(qkv, kc, vc, block_table, q_start, pos, sink, gate, scale: float, window: int, keep_first: int,
                     H: int, act_dtype, max_q: int, chunk: int = 0, pool: int = 0, kp=None, vp=None, v_cos_sin=None,
                     g_off: int = -1):
    """``max_q``: the most tokens any sequence brings in this step (sizes the launch grid).  ``chunk`` > 0: keys
    outside the query's own chunk of that many positions are hidden.  ``pool`` > 0: the pooled pairs of the blocks
    that lie wholly before a query's window join its softmax.  ``v_cos_sin`` [P, Dv]: every head's output is turned
    back by the query's position (the values were cached rotated); ``g_off`` >= 0: the output is multiplied element by
    element with sigmoid of qkv[:, g_off : g_off + H Dv].  The matrix-core kernel does both in its epilogue."""
    if _gpu(qkv):
        return _k().hy_window_attention(qkv, kc, vc, block_table, q_start, pos, sink, gate, scale, window, keep_first,
                                        chunk, H, max_q, pool, kp if pool else None, vp if pool else None, v_cos_sin,
                                        g_off)
    o = ref.window_attention(qkv, kc, vc, block_table, q_start, pos, sink, gate, scale, window, keep_first, H,
                             act_dtype, chunk, pool, kp, vp)
    if v_cos_sin is not None or g_off >= 0:
        o = ref.unrotate_gate(o, pos, v_cos_sin, qkv if g_off >= 0 else None, g_off, H, vc.shape[3], act_dtype)
    return o


def short_conv(x, w, tok_seq, q_start, pos0, slots, hist, silu: bool = True, bias=None, x_off: int = 0):
    if _gpu(x):
        return _k().hy_short_conv(x, w, tok_seq, q_start, pos0, slots, hist, silu, bias, x_off)
    return ref.short_conv(x, w, q_start, pos0, slots, hist, silu, bias, x_off)


def delta_prep(y, ab, a_log, HK: int, H: int, D: int, q_mul: float):
    if _gpu(y):
        return _k().hy_delta_prep(y, ab, a_log, HK, H, D, q_mul)
    return ref.delta_prep(y, ab, a_log, HK, H, D, q_mul)


def decay_pow(z, inv_tau: float):
    if _gpu(z):
        _k().hy_decay_pow(z, inv_tau)
        return z
    return ref.decay_pow(z, inv_tau)


def linear_scan(proj, q_off: int, k_off: int, v_off: int, qscale, kscale, q_mul: float, decay, beta, q_start, pos0,
                slots, S, HK: int, H: int, D: int, Dv: int, vscale=None):
    if _gpu(proj):
        return _k().hy_linear_scan(proj, q_off, k_off, v_off, qscale, kscale, q_mul, decay, beta, q_start, pos0, slots,
                                   S, HK, H, D, Dv, vscale)
    return ref.linear_scan(proj, q_off, k_off, v_off, qscale, kscale, q_mul, decay, beta, q_start, pos0, slots, S, HK,
                           H, D, Dv, vscale)


def head_norm_gate(o, src, g_off: int, w, eps: float, silu_gate: bool, act_dtype):
    if _gpu(o):
        return _k().hy_head_norm_gate(o, src, g_off, w, eps, silu_gate, _f32(act_dtype))
    return ref.head_norm_gate(o, src, g_off, w, eps, silu_gate, act_dtype)


def moe_route_topk(h, w_router, bias, top: int):
    if _gpu(h):
        return _k().hy_moe_route_topk(h, w_router, bias, top)
    return ref.moe_route_topk(h, w_router, bias, top)


def moe_glu_row_order(F: int) -> torch.Tensor:
    """Row order of a gated expert's [2F, d] gate-then-up matrix for the grouped MFMA path (F % 128 == 0): every
    128-row tile holds, for each of its two 64-row halves, 32 gate rows followed by the 32 up rows of the same
    outputs, so that a lane's accumulators hold a gate value and its up value."""
    n = torch.arange(2 * F)
    tile, local = n // 128, n % 128
    half, s, j = local // 64, (local % 64) // 16, local % 16
    out_col = tile * 64 + half * 32 + (s % 2) * 16 + j
    return out_col + (s >= 2) * F


def moe_glu_ffn(h, idx, wt, w_gu, w_down, limit: float, slope: float, shift: float, act_dtype, tiled: bool = False):
    """``tiled``: every expert's rows of w_gu are in :func:`moe_glu_row_order` (bfloat16 on the GPU, d and F on the
    128 grid): prompt-sized batches then run as grouped matrix-core GEMMs."""
    if _gpu(h):
        return _k().hy_moe_glu_ffn(h, idx, wt, w_gu, w_down, limit, slope, shift, tiled)
    if tiled:
        w_gu = w_gu[:, torch.argsort(moe_glu_row_order(w_gu.shape[1] // 2)).to(w_gu.device)]
    return ref.moe_glu_ffn(h, idx, wt, w_gu, w_down, limit, slope, shift, act_dtype)


# ---- pre-norm residual stream, per-layer token input, state-space and gated linear recurrences, grouped router ---


def add_rms_norm(y, x, w_out, eps: float, act_dtype, y2=None, gate2=None, w_y=None, emit: bool = True):
    """x (float32 residual, in place) <- x + v, v = y (+ sigmoid(gate2) y2), scaled to unit RMS and
    times w_y when that is given.  Returns in the activation dtype rms_norm(x) * w_out, or the updated rows
    themselves when w_out is None (x itself for float32), or None when ``emit`` is off."""
    if _gpu(x):
        h = _k().hy_add_rms_norm(y, x, w_out, eps, _f32(act_dtype), y2, gate2, w_y, emit)
        if not emit:
            return None
        return x if (w_out is None and _f32(act_dtype)) else h
    return ref.add_rms_norm(y, x, w_out, eps, act_dtype, y2, gate2, w_y, emit)


def token_gate(a, ids, table, col0: int, act_dtype):
    if _gpu(a):
        return _k().hy_token_gate(a, ids, table, col0)
    return ref.token_gate(a, ids, table, col0, act_dtype)


def ssm_prep(dt_pre, a_log):
    if _gpu(dt_pre):
        return _k().hy_ssm_prep(dt_pre, a_log)
    return ref.ssm_prep(dt_pre, a_log)


def gated_group_norm(o, skip_src, skip_off: int, skip_w, gate_src, g_off: int, w, groups: int, eps: float, act_dtype):
    if _gpu(o):
        return _k().hy_gated_group_norm(o, skip_src, skip_off, skip_w, gate_src, g_off, w, groups, eps, _f32(act_dtype))
    return ref.gated_group_norm(o, skip_src, skip_off, skip_w, gate_src, g_off, w, groups, eps, act_dtype)


def block_gates(u, w_gates, b_gates):
    """Gate pre-activations of a block-diagonal projection, float32: u [T, W] split into NB blocks of channels, block b
    times w_gates[b] ([W / NB, n]) plus b_gates[b] ([1, n], float32).  Returns [NB, T, n].  A library product with
    float32 accumulation and float32 output (its results are gates of a recurrence): bfloat16 operands go to the
    matrix cores as they are (their products are exact in float32), float32 operands to the float32 GEMM."""
    NB = w_gates.shape[0]
    T, W = u.shape
    ub = u.view(T, NB, W // NB).transpose(0, 1)
    if u.is_cuda and u.dtype == torch.bfloat16 and w_gates.dtype == torch.bfloat16:
        return torch.baddbmm(b_gates, ub, w_gates, out_dtype=torch.float32)
    return torch.baddbmm(b_gates, ub.float(), w_gates.float())


def rglru_scan(u, gates, sp, c: float, ysrc, y_off: int, q_start, pos0, slots, S, act_dtype, max_q: int = 0):
    """``max_q``: the most tokens any sequence brings in this step (sizes the launch grid; 0 = unknown)."""
    if _gpu(u):
        return _k().hy_rglru_scan(u, gates.contiguous(), sp, c, ysrc, y_off, q_start, pos0, slots, S, max_q)
    return ref.rglru_scan(u, gates, sp, c, ysrc, y_off, q_start, pos0, slots, S, act_dtype)


def moe_route_group(h, w_router, top: int, n_groups: int, keep: int, scale: float):
    if _gpu(h):
        return _k().hy_moe_route_group(h, w_router, top, n_groups, keep, scale)
    return ref.moe_route_group(h, w_router, top, n_groups, keep, scale)


# ---- sandwich residual stream, rotated values, retention -----------------------------------------------------------


def sandwich_join(y, x, w_y, w_out, groups: int, eps: float, act_dtype, y2=None, pair=None, emit: bool = True):
    """x (float32 residual, in place) <- x + group_rms_norm(v) * w_y with v = y (+ y2), or with ``pair`` = (w_a, w_b)
    v = (rms_norm(y) w_a + rms_norm(y2) w_b) / 2.  Returns group_rms_norm(x) * w_out in the activation dtype, or None
    when ``emit`` is off."""
    if _gpu(x):
        h = _k().hy_sandwich_join(y, y2, x, w_y, w_out if emit else None, pair[0] if pair else None,
                                  pair[1] if pair else None, groups, eps, _f32(act_dtype), True, emit)
        return h if emit else None
    return ref.sandwich_join(y, x, w_y, w_out, groups, eps, act_dtype, y2, pair, emit)


def unrotate_gate(o, pos, v_cos_sin, gate_src, g_off: int, H: int, Dv: int, act_dtype):
    if _gpu(o):
        return _k().hy_unrotate_gate(o, pos, v_cos_sin, gate_src, g_off, H, Dv)
    return ref.unrotate_gate(o, pos, v_cos_sin, gate_src, g_off, H, Dv, act_dtype)


def rotate_qk(proj, q_off: int, k_off: int, HQ: int, HK: int, D: int, dims: int, cos_sin, pos, q_mul: float,
              k_mul: float) -> None:
    if _gpu(proj):
        _k().hy_rotate_qk(proj, q_off, k_off, HQ, HK, D, dims if cos_sin is not None else 0, cos_sin, pos, q_mul, k_mul)
    else:
        ref.rotate_qk(proj, q_off, k_off, HQ, HK, D, dims, cos_sin, pos, q_mul, k_mul)
