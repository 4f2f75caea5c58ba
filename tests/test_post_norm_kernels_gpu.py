"""The HIP kernels of the post-norm hybrid mechanisms (csrc/hybrid/post_norm.hip, window_attention.hip, linear_scan.hip,
the top-k router and gated experts of moe.hip) against their PyTorch references (chronos.ops.hybrid_ref), in both
activation dtypes, at sizes off the kernels' tiles, with mixed prompt portions and decode rows in one launch."""
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


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("rows,d", [(1, 96), (7, 254), (33, 1000), (3, 4096), (2, 5000)])
def test_rms_norms(dt, rows, d):
    from chronos.ops import hybrid as hops, hybrid_ref as ref

    g = _gen(rows * d)
    y = _rand(g, rows, d, dtype=dt, scale=3.0) + 0.7
    x = _rand(g, rows, d)
    w = _rand(g, d) * 0.2 + 1.0
    x2 = x.clone()
    h = hops.scale_add_rms_norm(y, x, w, 1.7, 1e-6, dt)
    h2 = ref.scale_add_rms_norm(y, x2, w, 1.7, 1e-6, dt)
    _close(x, x2, 1e-5)
    _close(h, h2, _tol(dt, 1e-5, 8e-3))
    _close(hops.rms_norm(x, w, 1e-5, dt), ref.rms_norm(x2, w, 1e-5, dt), _tol(dt, 1e-5, 8e-3))


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("rows,F", [(5, 40), (9, 333)])
def test_glu_and_decay(dt, rows, F):
    from chronos.ops import hybrid as hops, hybrid_ref as ref

    g = _gen(F)
    gu = _rand(g, rows, 2 * F, dtype=dt, scale=2.0)
    _close(hops.glu(gu, 1.5, 1.702, 1.0, dt), ref.glu(gu, 1.5, 1.702, 1.0, dt), _tol(dt, 1e-5, 8e-3))
    z = _rand(g, rows, F, scale=4.0)
    _close(hops.decay_pow(z.clone(), 1 / 16.0), ref.decay_pow(z.clone(), 1 / 16.0), 1e-6)


def _stream(lens, starts, bs, nblocks, gen):
    """A flattened step of sequences with ``lens`` new tokens starting at positions ``starts``; pages dealt at
    random from the pool."""
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
@pytest.mark.parametrize("H,G,D,Dv,dims,window,keep", [(4, 2, 24, 40, 8, 9, 3), (3, 3, 64, 16, 64, 0, 0),
                                                       (6, 1, 16, 72, 0, 70, 5), (2, 2, 128, 128, 32, 130, 66),
                                                       (6, 2, 64, 48, 16, 20, 70), (12, 1, 32, 16, 32, 0, 0),
                                                       (4, 4, 256, 256, 64, 64, 1), (5, 1, 96, 80, 0, 3, 0)])
def test_window_attention(dt, H, G, D, Dv, dims, window, keep):
    from chronos.models.hybrid import rope_cos_sin
    from chronos.ops import hybrid as hops, hybrid_ref as ref

    g = _gen(H * D + window)
    bs, nb = 16, 64
    lens, starts = [37, 1, 150, 1, 2], [0, 95, 60, 0, 200]
    pos, seq, bt, qs = _stream(lens, starts, bs, nb, g)
    T = int(qs[-1])
    kc = _rand(g, nb, bs, G, D, dtype=dt)
    vc = _rand(g, nb, bs, G, Dv, dtype=dt)
    kc2, vc2 = kc.clone(), vc.clone()
    qkv = _rand(g, T, (H + G) * D + G * Dv, dtype=dt)
    qkv2 = qkv.clone()
    vf = _rand(g, T, G * Dv, dtype=dt)
    lam = torch.tensor([0.3], device=DEV)
    qn, kn = _rand(g, D) * 0.2 + 1, _rand(g, D) * 0.2 + 1
    cs = rope_cos_sin(1000.0, dims, 512, DEV, (8.0, 1.0, 4.0, 64.0)) if dims else None
    v = hops.window_prep(qkv, H, G, D, Dv, vf, lam, pos, seq, bt, qn, kn, 1e-6, cs, dims, kc, vc, True)
    v2 = ref.window_prep(qkv2, H, G, D, Dv, vf, lam, pos, seq, bt, qn, kn, 1e-6, cs, dims, kc2, vc2, True)
    assert torch.equal(v, v2)
    _close(qkv, qkv2, _tol(dt, 1e-5, 8e-3))
    _close(kc, kc2, _tol(dt, 1e-5, 8e-3))
    _close(vc, vc2, _tol(dt, 1e-5, 8e-3))
    kc.copy_(kc2); vc.copy_(vc2); qkv.copy_(qkv2)
    sink = _rand(g, H)
    gate = _rand(g, T, H)
    for sk, gt in ((sink, gate), (None, None)):
        o = hops.window_attention(qkv, kc, vc, bt, qs, pos, sk, gt, 0.3, window, keep, H, dt, max(lens))
        o2 = ref.window_attention(qkv2, kc2, vc2, bt, qs, pos, sk, gt, 0.3, window, keep, H, dt)
        _close(o, o2, _tol(dt, 2e-5, 1e-2))


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("C,K", [(70, 4), (300, 2), (17, 1), (64, 7), (1024 + 16, 4), (8, 3)])
def test_short_conv(dt, C, K):
    from chronos.ops import hybrid as hops, hybrid_ref as ref

    g = _gen(C * K)
    lens, starts, slots = [5, 1, 1, 9, 2], [0, 4, 0, 7, 3], [2, 0, 4, 1, 3]
    pos, seq, bt, qs = _stream(lens, starts, 16, 16, g)
    T = int(qs[-1])
    x = _rand(g, T, C + (13 if C % 8 else 24), dtype=dt)
    w = _rand(g, C, K, scale=0.5)
    hist = _rand(g, 6, K - 1, C, dtype=dt)
    hist2 = hist.clone()
    p0, sl = _i32(starts), _i32(slots)
    y = hops.short_conv(x, w, seq, qs, p0, sl, hist, True)
    y2 = ref.short_conv(x, w, qs, p0, sl, hist2, True)
    _close(y, y2, _tol(dt, 1e-5, 8e-3))
    assert torch.equal(hist, hist2)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("HK,H,D,Dv,mode", [(1, 2, 24, 40, "delta"), (3, 3, 64, 100, "delta"), (2, 4, 128, 64, "delta"),
                                            (2, 2, 20, 200, "gla"), (1, 1, 256, 70, "gla"), (2, 2, 33, 17, "both"),
                                            (2, 2, 33, 17, "plain")])
def test_linear_scan(dt, HK, H, D, Dv, mode):
    from chronos.ops import hybrid as hops, hybrid_ref as ref

    g = _gen(H * D + Dv)
    lens, starts, slots = [21, 1, 40, 1, 2], [0, 9, 16, 0, 33], [2, 0, 4, 1, 3]
    pos, seq, bt, qs = _stream(lens, starts, 16, 16, g)
    T = int(qs[-1])
    C = 2 * HK * D + H * Dv
    proj = _rand(g, T, C + 5, dtype=dt, scale=0.6)
    ab = _rand(g, T, 2 * H)
    qscale, kscale, decay, beta = hops.delta_prep(proj, ab, _rand(g, H) * 0.3, HK, H, D, D ** -0.5)
    r = ref.delta_prep(proj, ab, _rand(_gen(H * D + Dv + 1), H) * 0.3, HK, H, D, D ** -0.5)
    _close(qscale, r[0], 1e-5)
    _close(kscale, r[1], 1e-5)
    if mode in ("gla", "both"):
        decay = torch.sigmoid(_rand(g, T, H, D) + 2)
    if mode in ("gla", "plain"):
        beta, qscale, kscale = None, None, None
    S = _rand(g, 6, H, D, Dv, scale=0.3)
    S2 = S.clone()
    p0, sl = _i32(starts), _i32(slots)
    args = (5, 5 + HK * D, 5 + 2 * HK * D, qscale, kscale, 0.25, decay, beta, qs, p0, sl)
    o = hops.linear_scan(proj, *args, S, HK, H, D, Dv)
    o2 = ref.linear_scan(proj, *args, S2, HK, H, D, Dv)
    _close(o, o2, 2e-4)
    _close(S, S2, 2e-4)
    gsrc = _rand(g, T, H * Dv + 3, dtype=dt)
    w = _rand(g, H * Dv) * 0.2 + 1
    for silu in (True, False):
        _close(hops.head_norm_gate(o, gsrc, 3, w, 1e-6, silu, dt), ref.head_norm_gate(o2, gsrc, 3, w, 1e-6, silu, dt),
               _tol(dt, 1e-3, 1e-2))


def test_delta_prep_values():
    from chronos.ops import hybrid as hops, hybrid_ref as ref

    g = _gen(3)
    y = _rand(g, 11, 2 * 3 * 20 + 7, dtype=torch.bfloat16)
    ab = _rand(g, 11, 8, scale=5.0)
    al = _rand(g, 4)
    for a, b in zip(hops.delta_prep(y, ab, al, 3, 4, 20, 0.5), ref.delta_prep(y, ab, al, 3, 4, 20, 0.5)):
        _close(a, b, 1e-5)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("T,d,F,E,top", [(9, 72, 40, 5, 2), (3, 256, 64, 16, 3), (6, 100, 24, 1, 1), (70, 64, 16, 7, 7)])
def test_moe_glu(dt, T, d, F, E, top):
    from chronos.ops import hybrid as hops, hybrid_ref as ref

    g = _gen(T * d + E)
    h = _rand(g, T, d, dtype=dt)
    wr = _rand(g, E, d, dtype=dt, scale=0.5)
    br = _rand(g, E)
    idx, wt = hops.moe_route_topk(h, wr, br, top)
    idx2, wt2 = ref.moe_route_topk(h, wr, br, top)
    assert torch.equal(idx, idx2)
    _close(wt, wt2, 1e-5)
    wgu = _rand(g, E, 2 * F, d, dtype=dt, scale=d ** -0.5)
    wd = _rand(g, E, d, F, dtype=dt, scale=F ** -0.5)
    _close(hops.moe_glu_ffn(h, idx, wt, wgu, wd, 1.5, 1.702, 1.0, dt),
           ref.moe_glu_ffn(h, idx2, wt2, wgu, wd, 1.5, 1.702, 1.0, dt), _tol(dt, 2e-5, 1.5e-2))


@pytest.mark.parametrize("T,d,F,E,top", [(200, 256, 128, 4, 2), (90, 128, 384, 3, 3)])
def test_moe_glu_tile_order(T, d, F, E, top):
    """bfloat16 experts in the grouped path's row order: prompt-sized batches on the grouped matrix-core GEMMs and a
    few rows on the token kernel, both against the reference on the natural row order."""
    from chronos.ops import hybrid as hops, hybrid_ref as ref

    dt = torch.bfloat16
    g = _gen(T + F)
    h = _rand(g, T, d, dtype=dt)
    idx, wt = hops.moe_route_topk(h, _rand(g, E, d, dtype=dt, scale=0.5), _rand(g, E), top)
    wgu = _rand(g, E, 2 * F, d, dtype=dt, scale=d ** -0.5)
    wd = _rand(g, E, d, F, dtype=dt, scale=F ** -0.5)
    tiled = wgu[:, hops.moe_glu_row_order(F).to(DEV)].contiguous()
    want = ref.moe_glu_ffn(h, idx, wt, wgu, wd, 2.0, 1.702, 1.0, dt)
    _close(hops.moe_glu_ffn(h, idx, wt, tiled, wd, 2.0, 1.702, 1.0, dt, True), want, 1.5e-2)
    _close(hops.moe_glu_ffn(h[:3], idx[:3], wt[:3], tiled, wd, 2.0, 1.702, 1.0, dt, True), want[:3], 1.5e-2)


def test_router_ties_go_to_the_lower_index():
    from chronos.ops import hybrid as hops

    h = torch.zeros(2, 8, device=DEV)
    wr = torch.zeros(6, 8, device=DEV)
    bias = torch.tensor([0.0, 1.0, 1.0, -1.0, 1.0, 0.0], device=DEV)
    idx, wt = hops.moe_route_topk(h, wr, bias, 2)
    assert idx.tolist() == [[1, 2], [1, 2]]
    assert torch.allclose(wt, torch.full_like(wt, 0.5))
