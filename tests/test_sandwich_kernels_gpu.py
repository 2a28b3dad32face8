"""The HIP kernels of the sandwich-stream hybrid mechanisms (csrc/hybrid/sandwich.hip, the pooled tiles of the two
attention kernels, the block pooling and the value offset / rotation of window_prep, the scan's fixed decays, the
embedding's scale) against their PyTorch references (chronos.ops.hybrid_ref), in both activation dtypes, at sizes
off the kernels' tiles, with prompt portions and decode rows in one launch."""
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
@pytest.mark.parametrize("rows,d,groups", [(1, 96, 2), (7, 252, 3), (33, 1000, 5), (3, 4096, 1), (3, 4096, 16), (2, 5000, 4),
                                           (4, 4100, 2), (5, 30, 3), (9, 320, 2), (6, 70, 7), (3, 2048, 2), (4, 1088, 17),
                                           (5, 1024, 8), (2, 3072, 32)])
def test_sandwich_join(dt, rows, d, groups):
    """Register path (groups of whole 4-column chunks, up to 4096 columns) and the per-wave path (everything else);
    plain add, two addends, the pair form, emit on and off; the plain grouped norm."""
    from chronos.ops import hybrid as hops, hybrid_ref as ref

    g = _gen(rows * d + groups)
    y = _rand(g, rows, d, dtype=dt, scale=3.0) + 0.7
    y2 = _rand(g, rows, d, dtype=dt, scale=0.5)
    w_y, w_out, w_a, w_b = (_rand(g, d) * 0.2 + 1.0 for _ in range(4))
    for kw in (dict(), dict(y2=y2), dict(y2=y2, pair=(w_a, w_b))):
        for emit in (True, False):
            x = _rand(g, rows, d)
            xr = x.clone()
            h = hops.sandwich_join(y, x, w_y, w_out, groups, 1e-5, dt, emit=emit, **kw)
            hr = ref.sandwich_join(y, xr, w_y, w_out, groups, 1e-5, dt, emit=emit, **kw)
            _close(x, xr, 2e-5)
            assert (h is None) == (hr is None) == (not emit)
            if emit:
                assert h.dtype == dt
                _close(h, hr, _tol(dt))
    x = _rand(g, rows, d, scale=4.0)
    keep = x.clone()
    _close(hops.rms_norm(x, w_out, 1e-5, dt, groups), ref.rms_norm(keep, w_out, 1e-5, dt, groups), _tol(dt))
    assert torch.equal(x, keep)


@pytest.mark.parametrize("dt", DTYPES)
def test_embed_scale(dt):
    from chronos.ops import hybrid as hops, hybrid_ref as ref

    g = _gen(1)
    table = _rand(g, 50, 72, dtype=dt)
    ids = _i32([3, 49, 0, 3])
    for scale, emit in ((1.0, True), (7.25, False), (0.3, True)):
        x, h = hops.embed_rows(ids, table, dt, scale, emit)
        xr, hr = ref.embed_rows(ids, table, dt, scale, emit)
        _close(x, xr, 1e-6)
        assert (h is None) == (hr is None)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("HQ,HK,D,dims", [(3, 3, 8, 8), (4, 2, 12, 6), (1, 5, 64, 0), (2, 2, 6, 2), (16, 16, 128, 128)])
def test_rotate_qk(dt, HQ, HK, D, dims):
    from chronos.models.hybrid import rope_cos_sin
    from chronos.ops import hybrid as hops, hybrid_ref as ref

    g = _gen(HQ * D + dims)
    T = 21
    proj = _rand(g, T, 5 + HQ * D + 3 + HK * D + 9, dtype=dt)
    pos = _i32([(7 * t) % 60 for t in range(T)])
    tab = rope_cos_sin(1e4, dims, 64, DEV, ("linear", 2.0)) if dims else None
    a, b = proj.clone(), proj.clone()
    hops.rotate_qk(a, 5, 5 + HQ * D + 3, HQ, HK, D, dims, tab, pos, 1.0, D ** -0.5)
    ref.rotate_qk(b, 5, 5 + HQ * D + 3, HQ, HK, D, dims, tab, pos, 1.0, D ** -0.5)
    _close(a, b, _tol(dt, 2e-6, 8e-3))
    assert torch.equal(a[:, :5], proj[:, :5]) and torch.equal(a[:, -9:], proj[:, -9:])


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H,Dv,rot,gate", [(3, 8, True, True), (4, 70, True, False), (2, 6, False, True), (16, 128, True, True)])
def test_unrotate_gate(dt, H, Dv, rot, gate):
    from chronos.models.hybrid import rope_cos_sin
    from chronos.ops import hybrid as hops, hybrid_ref as ref

    g = _gen(H * Dv)
    T = 19
    o = _rand(g, T, H * Dv, dtype=dt)
    src = _rand(g, T, 11 + H * Dv, dtype=dt, scale=2.0) if gate else None
    pos = _i32([(5 * t) % 40 for t in range(T)])
    tab = rope_cos_sin(2.5e5, Dv, 48, DEV) if rot else None
    _close(hops.unrotate_gate(o, pos, tab, src, 11, H, Dv, dt), ref.unrotate_gate(o, pos, tab, src, 11, H, Dv, dt),
           _tol(dt, 2e-6, 8e-3))


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H,G,D,Dv,v_from_k,v_rot,norm", [(4, 2, 12, 12, True, False, False), (3, 3, 8, 20, False, True, True),
                                                           (8, 2, 64, 64, True, False, False), (4, 4, 64, 32, False, True, True)])
def test_window_prep_value_source_and_rotation(dt, H, G, D, Dv, v_from_k, v_rot, norm):
    from chronos.models.hybrid import rope_cos_sin
    from chronos.ops import hybrid as hops, hybrid_ref as ref

    g = _gen(H * D + Dv)
    bs, nb = 16, 12
    pos, seq, bt, _ = _stream([37, 1, 9], [0, 50, 15], bs, nb)
    T = pos.numel()
    width = (H + G) * D + (0 if v_from_k else G * Dv) + 24
    qkv = _rand(g, T, width, dtype=dt)
    tab = rope_cos_sin(1e4, D // 2 * 2 - 2, 128, DEV, ("ramp", 4.0, 64.0, 8.0, 1.0))
    vtab = rope_cos_sin(1e4, Dv, 128, DEV) if v_rot else None
    qn = (_rand(g, D) * 0.1 + 1.0) if norm else None
    kn = (_rand(g, D) * 0.1 + 1.0) if norm else None
    res = []
    for fn in (hops.window_prep, ref.window_prep):
        q = qkv.clone()
        kc = torch.zeros(nb, bs, G, D, dtype=dt, device=DEV)
        vc = torch.zeros(nb, bs, G, Dv, dtype=dt, device=DEV)
        fn(q, H, G, D, Dv, None, None, pos, seq, bt, qn, kn, 1e-5, tab, tab.shape[1], kc, vc, False,
           H * D if v_from_k else -1, vtab)
        res.append((q, kc, vc))
    for a, b in zip(*res):
        _close(a, b, _tol(dt, 2e-6, 8e-3))


def _pooled_case(dt, H, G, D, Dv, lens, starts, window, pool, bs=16, seed=0):
    """Caches filled for every sequence up to the end of its range, pooled by the framework's own kernel."""
    from chronos.ops import hybrid as hops

    g = _gen(seed + H * D + window + pool)
    nb = sum((s + n + bs - 1) // bs for s, n in zip(starts, lens)) + 2
    pos, seq, bt, qs = _stream(lens, starts, bs, nb)
    kc = _rand(g, nb, bs, G, D, dtype=dt)
    vc = _rand(g, nb, bs, G, Dv, dtype=dt)
    ep = (bs + pool - 1) // pool
    kp = torch.full((nb, ep, G, D), float("nan"), dtype=dt, device=DEV)
    vp = torch.full((nb, ep, G, Dv), float("nan"), dtype=dt, device=DEV)
    ends = [s + n for s, n in zip(starts, lens)]
    hops.pool_blocks(kc, vc, kp, vp, bt, _i32([0] + torch.tensor(ends).cumsum(0).tolist()), _i32([0] * len(lens)), pool,
                     max(ends))
    qkv = _rand(g, pos.numel(), H * D + 5, dtype=dt)
    return qkv, kc, vc, kp, vp, bt, qs, pos


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("pool", [1, 3, 16, 23])
@pytest.mark.parametrize("G,D,Dv", [(2, 12, 20), (1, 9, 5), (8, 128, 72)])
def test_pool_blocks(dt, pool, G, D, Dv):
    """Steps that end inside blocks, at their ends and several blocks later, for sequences at different offsets; blocks
    that straddle pages; a block larger than a page.  Widths on the 8-column grid take the kernel with wide loads
    (one and several 512-column slabs), the others the column-per-thread kernel."""
    from chronos.ops import hybrid as hops, hybrid_ref as ref

    g = _gen(pool)
    bs = 16
    lens, starts = [40, 1, 9, 3], [0, pool * 3 - 1 if pool > 1 else 7, 15, 30]
    nb = 16
    _, _, bt, qs = _stream(lens, starts, bs, nb)
    kc = _rand(g, nb, bs, G, D, dtype=dt)
    vc = _rand(g, nb, bs, G, Dv, dtype=dt)
    ep = (bs + pool - 1) // pool
    out = []
    for fn in (lambda *a: hops.pool_blocks(*a, max(lens)), ref.pool_blocks):
        kp = torch.zeros(nb, ep, G, D, dtype=dt, device=DEV)
        vp = torch.zeros(nb, ep, G, Dv, dtype=dt, device=DEV)
        fn(kc, vc, kp, vp, bt, qs, _i32(starts), pool)
        out.append((kp, vp))
    assert float(out[1][0].abs().sum()) > 0
    for a, b in zip(*out):
        _close(a, b, _tol(dt, 2e-6, 8e-3))
        assert torch.equal(a == 0, b == 0)   # only the blocks that end in this step are written


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H,G,D,Dv", [(4, 2, 12, 20), (8, 2, 64, 64), (6, 1, 32, 16), (3, 3, 128, 128)])
@pytest.mark.parametrize("window,pool", [(9, 4), (40, 16), (24, 7), (100, 3)])
def test_pooled_window_attention(dt, H, G, D, Dv, window, pool):
    """Prompt portions beside decode rows: a long portion from position 0, a decode row deep in a sequence, a short
    portion in the middle, a two-token portion; with and without a sink.  bfloat16 at the larger sizes runs the
    matrix-core kernel (the decode-heavy launch with its key tiles split over workgroups)."""
    from chronos.ops import hybrid as hops, hybrid_ref as ref

    for lens, starts in (([150, 1, 9, 2], [0, 333, 75, 140]), ([1, 1, 1], [200, 64, 17])):
        qkv, kc, vc, kp, vp, bt, qs, pos = _pooled_case(dt, H, G, D, Dv, lens, starts, window, pool)
        for sink in (None, _rand(_gen(3), H)):
            a = hops.window_attention(qkv, kc, vc, bt, qs, pos, sink, None, D ** -0.5, window, 0, H, dt, max(lens), 0, pool,
                                      kp, vp)
            b = ref.window_attention(qkv, kc, vc, bt, qs, pos, sink, None, D ** -0.5, window, 0, H, dt, 0, pool, kp, vp)
            assert torch.isfinite(a.float()).all()
            _close(a, b, _tol(dt, 2e-5, 1.5e-2))


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H,D,Dv", [(3, 8, 10), (4, 64, 32), (2, 128, 128), (5, 20, 6)])
def test_linear_scan_with_fixed_decays(dt, H, D, Dv):
    from chronos.ops import hybrid as hops, hybrid_ref as ref

    g = _gen(H * D + Dv)
    lens, starts = [70, 1, 5], [0, 9, 3]
    qs = [0, 70, 71, 76]
    T = 76
    proj = _rand(g, T, 2 * H * D + H * Dv + 7, dtype=dt, scale=0.5)
    decay = torch.tensor([1.0 - 2.0 ** (-1 - 2 * h) for h in range(H)], device=DEV)
    S0 = _rand(g, 5, H, D, Dv)
    out = []
    for fn in (hops.linear_scan, ref.linear_scan):
        S = S0.clone()
        o = fn(proj, 0, H * D, 2 * H * D, None, None, 1.0, decay, None, _i32(qs), _i32(starts), _i32([2, 0, 4]), S, H, H, D, Dv)
        out.append((o, S))
    for a, b in zip(*out):
        _close(a, b, 2e-5)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H,G,D,Dv", [(4, 2, 64, 64), (8, 8, 32, 32), (2, 1, 128, 128), (6, 2, 64, 48), (4, 4, 32, 16),
                                      (3, 1, 12, 20), (2, 2, 256, 256)])
@pytest.mark.parametrize("rot,wide", [(True, True), (True, False), (False, True)])
def test_attention_turns_outputs_back_and_gates(dt, H, G, D, Dv, rot, wide):
    """The attention's last steps — every head's output turned back by the query's position, times sigmoid of a gate
    per output column read from the query's projection row — against the reference chain.  bfloat16 with value widths
    on the 32 grid does them in the matrix-core kernel's epilogue (long portions) or in the merge of split key tiles
    (few rows over long contexts), other widths and float32 in a pass of their own."""
    from chronos.models.hybrid import rope_cos_sin
    from chronos.ops import hybrid as hops, hybrid_ref as ref

    bs = 16
    for lens, starts in (([150, 1, 9, 2], [0, 333, 75, 140]), ([1, 1, 1], [700, 64, 17])):
        g = _gen(H * D + Dv + len(lens))
        nb = sum((s + n + bs - 1) // bs for s, n in zip(starts, lens)) + 2
        pos, seq, bt, qs = _stream(lens, starts, bs, nb)
        kc, vc = _rand(g, nb, bs, G, D, dtype=dt), _rand(g, nb, bs, G, Dv, dtype=dt)
        g_off = (H + G) * D + G * Dv
        qkv = _rand(g, pos.numel(), g_off + H * Dv + 8, dtype=dt)
        sink = _rand(g, H)
        tab = rope_cos_sin(1e4, Dv, 800, DEV) if rot else None
        a = hops.window_attention(qkv, kc, vc, bt, qs, pos, sink, None, D ** -0.5, 0, 0, H, dt, max(lens), 0, 0, None, None,
                                  tab, g_off if wide else -1)
        b = ref.window_attention(qkv, kc, vc, bt, qs, pos, sink, None, D ** -0.5, 0, 0, H, dt)
        b = ref.unrotate_gate(b, pos, tab, qkv if wide else None, g_off, H, Dv, dt)
        _close(a, b, _tol(dt, 2e-5, 1.5e-2))
