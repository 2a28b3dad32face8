"""The HIP kernels of the pre-norm hybrid mechanisms (csrc/hybrid/pre_norm.hip, the chunk mask of the attention
kernels, the convolution's bias, the scan's value scale, the grouped sigmoid router of moe.hip) against their PyTorch
references (chronos.ops.hybrid_ref), in both activation dtypes, at sizes off the kernels' tiles, with prompt portions
and decode rows in one launch."""
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda"
DTYPES = [torch.bfloat16, torch.float32]


@pytest.fixture(scope="module", autouse=True)
def _lib():
    from chronos.ops import hybrid as hops

    hops.load()
    import chronos.native as n

    assert "_H" in n._loaded, "the hybrid HIP library must be the one running"


def _gen(seed):
    return torch.Generator(device=DEV).manual_seed(seed)


def _rand(g, *shape, dtype=torch.float32, scale=1.0):
    return (torch.randn(*shape, device=DEV, generator=g) * scale).to(dtype)


def _close(a, b, tol):
    a, b = a.float(), b.float()
    err = float((a - b).abs().max())
    ref = float(b.abs().max()) + 1e-6
    assert err <= tol * ref, f"max err {err:.4g} vs magnitude {ref:.4g}"


def _tol(dt, f32=2e-5, bf16=1.5e-2):
    return f32 if dt == torch.float32 else bf16


def _i32(x):
    return torch.tensor(x, dtype=torch.int32, device=DEV)


def _stream(lens, starts, bs, nblocks):
    perm = (torch.randperm(nblocks - 1, generator=torch.Generator().manual_seed(7)) + 1).tolist()
    mb = max((s + n + bs - 1) // bs for s, n in zip(starts, lens))
    bt = torch.zeros(len(lens), mb, dtype=torch.int32)
    for b, (s, n) in enumerate(zip(starts, lens)):
        need = (s + n + bs - 1) // bs
        bt[b, :need] = torch.tensor([perm.pop() for _ in range(need)], dtype=torch.int32)
    pos = [p for s, n in zip(starts, lens) for p in range(s, s + n)]
    seq = [b for b, n in enumerate(lens) for _ in range(n)]
    qs = [0]
    for n in lens:
        qs.append(qs[-1] + n)
    return _i32(pos), _i32(seq), bt.to(DEV), _i32(qs)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("rows,d", [(1, 96), (7, 254), (33, 1000), (3, 4096), (2, 5000), (4, 4100)])
def test_add_rms_norm(dt, rows, d):
    from chronos.ops import hybrid as hops, hybrid_ref as ref

    g = _gen(rows * d)
    y = _rand(g, rows, d, dtype=dt, scale=3.0) + 0.7
    y2 = _rand(g, rows, d, dtype=dt, scale=2.0)
    g2 = _rand(g, rows, 1, scale=2.0)
    w_out = _rand(g, d) * 0.2 + 1.0
    w_y = _rand(g, d) * 0.2 + 1.0
    for kw in (dict(), dict(y2=y2, gate2=g2), dict(w_y=w_y), dict(y2=y2, gate2=g2, w_y=w_y)):
        for wo, emit in ((w_out, True), (None, True), (None, False)):
            x = _rand(g, rows, d)
            x2 = x.clone()
            h = hops.add_rms_norm(y, x, wo, 1e-6, dt, emit=emit, **kw)
            h2 = ref.add_rms_norm(y, x2, wo, 1e-6, dt, emit=emit, **kw)
            _close(x, x2, 1e-5)
            if emit:
                _close(h, h2, _tol(dt, 1e-5, 8e-3))
            else:
                assert h is None and h2 is None


@pytest.mark.parametrize("dt", DTYPES)
def test_token_gate_and_ssm_prep(dt):
    from chronos.ops import hybrid as hops, hybrid_ref as ref

    g = _gen(5)
    T, n, V = 19, 24, 50
    a = _rand(g, T, n, dtype=dt, scale=2.0)
    table = _rand(g, V, 5 * n + 3, dtype=dt)
    ids = torch.randint(0, V, (T,), device=DEV, generator=g).int()
    for col0 in (0, 2 * n, 4 * n + 3):
        _close(hops.token_gate(a, ids, table, col0, dt), ref.token_gate(a, ids, table, col0, dt), _tol(dt, 1e-5, 8e-3))
    dtp = _rand(g, T, 6, scale=8.0)
    dtp[0, 0], dtp[1, 1] = 45.0, -60.0
    al = _rand(g, 6)
    for x, y in zip(hops.ssm_prep(dtp, al), ref.ssm_prep(dtp, al)):
        _close(x, y, 1e-5)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H,Dv,groups", [(6, 24, 2), (4, 64, 1), (3, 40, 3), (16, 64, 1), (5, 24, 5)])
def test_gated_group_norm(dt, H, Dv, groups):
    from chronos.ops import hybrid as hops, hybrid_ref as ref

    g = _gen(H * Dv)
    T, n = 13, H * Dv
    o = _rand(g, T, H, Dv)
    xs = _rand(g, T, n + 11, dtype=dt)
    zs = _rand(g, T, 2 * n + 5, dtype=dt, scale=2.0)
    skip = _rand(g, H) + 1.0
    w = _rand(g, n) * 0.2 + 1.0
    _close(hops.gated_group_norm(o, xs, 7, skip, zs, 3, w, groups, 1e-6, dt),
           ref.gated_group_norm(o, xs, 7, skip, zs, 3, w, groups, 1e-6, dt), _tol(dt, 1e-5, 8e-3))


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("W,NB,lens,starts", [(176, 2, [21, 1, 40, 1, 2], [0, 9, 16, 0, 33]),
                                              (300, 3, [200, 1, 65, 64, 1], [0, 5, 7, 0, 0]),
                                              (64, 1, [1, 1, 1, 1, 1], [3, 0, 9, 1, 2]),
                                              (520, 4, [130, 300, 1, 2, 129], [64, 0, 1, 0, 100])])
def test_rglru_scan(dt, W, NB, lens, starts):
    """Prompt portions longer than a chunk of the two-launch form, beside decode rows and fresh sequences."""
    from chronos.ops import hybrid as hops, hybrid_ref as ref

    g = _gen(W + NB)
    slots = [2, 0, 4, 1, 3]
    pos, seq, bt, qs = _stream(lens, starts, 16, 64)
    T = int(qs[-1])
    u = _rand(g, T, W, dtype=dt)
    ysrc = _rand(g, T, W + 9, dtype=dt)
    wg = _rand(g, NB, W // NB, 2 * (W // NB), scale=(W // NB) ** -0.5)
    bg = _rand(g, NB, 1, 2 * (W // NB))
    gates = hops.block_gates(u, wg, bg)
    want = torch.einsum("tbi,bio->bto", u.float().view(T, NB, W // NB), wg) + bg
    _close(gates, want, 1e-5)
    sp = torch.nn.functional.softplus(_rand(g, W) - 1.0)
    S = _rand(g, 6, W)
    S2 = S.clone()
    p0, sl = _i32(starts), _i32(slots)
    o = hops.rglru_scan(u, gates, sp, 8.0, ysrc, 9, qs, p0, sl, S, dt, max(lens))
    o2 = ref.rglru_scan(u, gates, sp, 8.0, ysrc, 9, qs, p0, sl, S2, dt)
    _close(o, o2, _tol(dt, 2e-5, 8e-3))
    _close(S, S2, 2e-5)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("HK,H,D,Dv", [(2, 6, 48, 24), (1, 4, 128, 64), (3, 3, 16, 40), (2, 8, 64, 64)])
def test_linear_scan_value_scale(dt, HK, H, D, Dv):
    """The state-space form of the scan: one decay per head, rows shared by the heads of a group, the written value
    scaled per token and head, no delta correction."""
    from chronos.ops import hybrid as hops, hybrid_ref as ref

    g = _gen(H * D + Dv)
    lens, starts, slots = [21, 1, 40, 1, 2], [0, 9, 16, 0, 33], [2, 0, 4, 1, 3]
    pos, seq, bt, qs = _stream(lens, starts, 16, 16)
    T = int(qs[-1])
    C = H * Dv + 2 * HK * D
    xbc = _rand(g, T, C, dtype=dt, scale=0.6)
    decay, dt_ = ref.ssm_prep(_rand(g, T, H), _rand(g, H) * 0.3)
    S = _rand(g, 6, H, D, Dv, scale=0.3)
    S2 = S.clone()
    p0, sl = _i32(starts), _i32(slots)
    args = (H * Dv + HK * D, H * Dv, 0, None, None, 1.0, decay, None, qs, p0, sl)
    o = hops.linear_scan(xbc, *args, S, HK, H, D, Dv, dt_)
    o2 = ref.linear_scan(xbc, *args, S2, HK, H, D, Dv, dt_)
    _close(o, o2, 2e-4)
    _close(S, S2, 2e-4)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("C,K,off", [(70, 4, 9), (328, 3, 200), (17, 1, 0), (64, 2, 64)])
def test_short_conv_bias_and_offset(dt, C, K, off):
    from chronos.ops import hybrid as hops, hybrid_ref as ref

    g = _gen(C * K)
    lens, starts, slots = [5, 1, 1, 9, 2], [0, 4, 0, 7, 3], [2, 0, 4, 1, 3]
    pos, seq, bt, qs = _stream(lens, starts, 16, 16)
    T = int(qs[-1])
    x = _rand(g, T, off + C + 6, dtype=dt)
    w = _rand(g, C, K, scale=0.5)
    bias = _rand(g, C)
    hist = _rand(g, 6, K - 1, C, dtype=dt)
    hist2 = hist.clone()
    p0, sl = _i32(starts), _i32(slots)
    for silu in (True, False):
        y = hops.short_conv(x, w, seq, qs, p0, sl, hist.clone(), silu, bias, off)
        y2 = ref.short_conv(x, w, qs, p0, sl, hist2.clone(), silu, bias, off)
        _close(y, y2, _tol(dt, 1e-5, 8e-3))
    hops.short_conv(x, w, seq, qs, p0, sl, hist, False, bias, off)
    ref.short_conv(x, w, qs, p0, sl, hist2, False, bias, off)
    assert torch.equal(hist, hist2)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H,G,D,Dv,chunk,window", [(6, 2, 80, 48, 50, 0), (4, 2, 24, 40, 9, 0), (2, 2, 128, 128, 64, 0),
                                                  (8, 2, 64, 64, 100, 0), (3, 1, 32, 16, 1, 0), (4, 4, 64, 48, 70, 30),
                                                  (2, 1, 128, 64, 200, 0)])
def test_chunked_attention(dt, H, G, D, Dv, chunk, window):
    """The chunk mask on both attention kernels, without query/key norm, sink or gate; prompt portions that start and
    end inside chunks, beside decode rows at chunk borders."""
    from chronos.ops import hybrid as hops, hybrid_ref as ref

    g = _gen(H * D + chunk)
    bs, nb = 16, 256
    lens, starts = [37, 1, 150, 1, 2, 1, 70], [0, 2 * chunk, 60, 0, 3 * chunk - 1, 4 * chunk - 1, 130]
    pos, seq, bt, qs = _stream(lens, starts, bs, nb)
    T = int(qs[-1])
    kc = _rand(g, nb, bs, G, D, dtype=dt)
    vc = _rand(g, nb, bs, G, Dv, dtype=dt)
    kc2, vc2 = kc.clone(), vc.clone()
    qkv = _rand(g, T, (H + G) * D + G * Dv, dtype=dt)
    qkv2 = qkv.clone()
    hops.window_prep(qkv, H, G, D, Dv, None, None, pos, seq, bt, None, None, 1e-6, None, 0, kc, vc, False)
    ref.window_prep(qkv2, H, G, D, Dv, None, None, pos, seq, bt, None, None, 1e-6, None, 0, kc2, vc2, False)
    assert torch.equal(qkv, qkv2) and torch.equal(kc, kc2) and torch.equal(vc, vc2)
    o = hops.window_attention(qkv, kc, vc, bt, qs, pos, None, None, 0.3, window, 0, H, dt, max(lens), chunk)
    o2 = ref.window_attention(qkv2, kc2, vc2, bt, qs, pos, None, None, 0.3, window, 0, H, dt, chunk)
    _close(o, o2, _tol(dt, 2e-5, 1e-2))


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("T,d,N,top,ng,keep", [(9, 72, 12, 3, 3, 2), (70, 64, 16, 4, 4, 2), (5, 100, 6, 3, 1, 1),
                                               (33, 48, 64, 6, 8, 3), (4, 32, 8, 2, 8, 2), (3, 40, 9, 3, 3, 3),
                                               (11, 64, 256, 8, 64, 5)])
def test_moe_route_group(dt, T, d, N, top, ng, keep):
    from chronos.ops import hybrid as hops, hybrid_ref as ref

    g = _gen(T * d + N)
    h = _rand(g, T, d, dtype=dt)
    wr = _rand(g, N, d, dtype=dt, scale=0.5)
    idx, wt = hops.moe_route_group(h, wr, top, ng, keep, 2.5)
    idx2, wt2 = ref.moe_route_group(h, wr, top, ng, keep, 2.5)
    assert torch.equal(idx, idx2)
    _close(wt, wt2, 1e-5)
    assert torch.allclose(wt.sum(-1), torch.full((T,), 2.5, device=DEV), atol=1e-4)


def test_group_router_choice_is_limited_to_the_best_groups():
    """One-hot inputs make the router logits the rows' first column: the largest single score sits in a group whose
    second score is small, so that group loses against groups with two good scores and its expert must not be chosen."""
    from chronos.ops import hybrid as hops

    z = torch.tensor([4.0, -9.0, 2.0, 2.5, 1.0, 1.5, -3.0, -3.0])   # groups of 2: sums of sigmoids
    wr = torch.zeros(8, 4, device=DEV)
    wr[:, 0] = z.to(DEV)
    h = torch.zeros(3, 4, device=DEV)
    h[:, 0] = 1.0
    idx, wt = hops.moe_route_group(h, wr, 2, 4, 2, 1.0)
    # group scores: g0 = s(4) + s(-9) ~ 0.98, g1 = s(2) + s(2.5) ~ 1.80, g2 = s(1) + s(1.5) ~ 1.55 -> g1, g2 kept
    assert idx.tolist() == [[3, 2]] * 3
    s = torch.sigmoid(torch.tensor([2.5, 2.0]))
    assert torch.allclose(wt[0].cpu(), s / s.sum(), atol=1e-6)
    idx, _ = hops.moe_route_group(h, wr, 2, 4, 4, 1.0)     # every group kept: the single best score wins
    assert idx.tolist() == [[0, 3]] * 3
    idx, _ = hops.moe_route_group(torch.zeros(2, 4, device=DEV), wr, 3, 4, 2, 1.0)   # all ties: the lower indices
    assert idx.tolist() == [[0, 1, 2]] * 2
