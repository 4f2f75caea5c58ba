"""Every hybrid-decoder HIP kernel (csrc/hybrid) against its PyTorch reference (chronos.ops.hybrid_ref), in both
activation dtypes, at sizes that are not multiples of the kernels' tiles."""
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


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("rows,d", [(1, 96), (7, 256), (33, 1000), (4, 4096)])
def test_layer_norms(dt, rows, d):
    from chronos.ops import hybrid as hops, hybrid_ref as ref

    g = _gen(rows * d)
    y = _rand(g, rows, d, dtype=dt, scale=3.0) + 0.7
    x = _rand(g, rows, d)
    w = _rand(g, d) * 0.2 + 1.0
    x2 = x.clone()
    h = hops.add_layer_norm(y, x, w, 1e-6, dt)
    h2 = ref.add_layer_norm(y, x2, w, 1e-6, dt)
    _close(x, x2, 1e-5)
    _close(h, h2, _tol(dt, 1e-5, 8e-3))
    _close(hops.layer_norm(x, w, 1e-5, dt), ref.layer_norm(x2, w, 1e-5, dt), _tol(dt, 1e-5, 8e-3))


@pytest.mark.parametrize("dt", DTYPES)
def test_embed_rowdot_act(dt):
    from chronos.ops import hybrid as hops, hybrid_ref as ref

    g = _gen(5)
    table = _rand(g, 50, 72, dtype=dt)
    ids = torch.tensor([3, 49, 0, 3, 17], dtype=torch.int32, device=DEV)
    x, h = hops.embed_rows(ids, table, dt)
    x2, h2 = ref.embed_rows(ids, table, dt)
    assert torch.equal(x, x2) and torch.equal(h, h2)
    hh = _rand(g, 9, 200, dtype=dt)
    w = _rand(g, 5, 200, dtype=dt)
    b = _rand(g, 5)
    _close(hops.rowdot(hh, w, b), ref.rowdot(hh, w, b), 1e-5)
    _close(hops.rowdot(hh, w), ref.rowdot(hh, w), 1e-5)
    for kind in (0, 1):
        z = _rand(g, 13, 77, dtype=dt, scale=2.0)
        z2 = z.clone()
        _close(hops.act_inplace(z, kind), ref.act_inplace(z2, kind), _tol(dt, 1e-6, 8e-3))


def _stream(lens, starts):
    qs = [0]
    for n in lens:
        qs.append(qs[-1] + n)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)  # noqa: E731
    pos = [s + i for n, s in zip(lens, starts) for i in range(n)]
    seq = [b for b, n in enumerate(lens) for _ in range(n)]
    return i32(qs), i32(starts), i32(pos), i32(seq)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H,D,Dv", [(2, 40, 72), (3, 20, 40), (1, 130, 72), (2, 260, 200), (4, 256, 128)])
def test_mlstm_scan(dt, H, D, Dv):
    """Fresh sequences, continued sequences (state from the slot), an empty one, one token, a tile-straddling one."""
    from chronos.ops import hybrid as hops, hybrid_ref as ref

    g = _gen(H * D + Dv)
    lens, starts = [11, 1, 0, 19, 8], [0, 5, 3, 7, 0]
    slots = torch.tensor([2, 0, 4, 1, 3], dtype=torch.int32, device=DEV)
    q_start, pos0, _, _ = _stream(lens, starts)
    T, C = sum(lens), 2 * H * D + 2 * H * Dv
    proj = _rand(g, T, C, dtype=dt)
    gate_pre = _rand(g, T, 2 * H, scale=4.0)
    gate_pre[:, H:] += 3.0
    S = _rand(g, 6, H, D, Dv)
    n = _rand(g, 6, H, D)
    m = _rand(g, 6, H)
    S2, n2, m2 = S.clone(), n.clone(), m.clone()
    o = hops.mlstm_scan(proj, gate_pre, q_start, pos0, slots, S, n, m, H, D, Dv, 12.0, max(lens))
    o2 = ref.mlstm_scan(proj, gate_pre, q_start, pos0, slots, S2, n2, m2, H, D, Dv, 12.0)
    _close(o, o2, 3e-5)
    _close(S, S2, 3e-5)
    _close(n, n2, 3e-5)
    _close(m, m2, 1e-6)
    assert torch.equal(S[4], S2[4]) and torch.equal(S[5], S2[5]), "slots without tokens must stay untouched"
    w = _rand(g, H * Dv) * 0.1 + 1
    _close(hops.mlstm_out(o2, proj, 2 * H * D + H * Dv, w, 1e-6, dt),
           ref.mlstm_out(o2, proj, 2 * H * D + H * Dv, w, 1e-6, dt), _tol(dt, 1e-5, 8e-3))


def _paged(g, lens, starts, BS, DK, dt, shuffle=True):
    nblk = [(s + n + BS - 1) // BS for n, s in zip(lens, starts)]
    NB = sum(nblk) + 3
    perm = torch.randperm(NB - 1, generator=torch.Generator().manual_seed(1)).add(1).tolist() if shuffle else list(range(1, NB))
    bt = torch.zeros(len(lens), max(nblk) + 1, dtype=torch.int32)
    k = 0
    for b, nb in enumerate(nblk):
        for j in range(nb):
            bt[b, j] = perm[k]
            k += 1
    cache = _rand(g, NB, BS, DK, dtype=dt)
    return cache, bt.to(DEV)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H,D,R,rank,dims", [(2, 24, 32, 32, 16), (3, 24, 16, 40, 8), (1, 8, 4, 130, 4), (8, 16, 64, 512, 64),
                                             (5, 16, 32, 160, 32), (1, 8, 16, 16, 16), (70, 8, 32, 96, 32)])
def test_latent_prep_and_attention(dt, H, D, R, rank, dims):
    """Prefill portions over a cached prefix, decode rows, a first token; pages in shuffled order, partial last
    pages, query tiles that straddle key tiles."""
    from chronos.models.hybrid import rope_cos_sin
    from chronos.ops import hybrid as hops, hybrid_ref as ref

    g = _gen(H + D + rank)
    BS = 16
    lens, starts = [70, 1, 1, 5, 130], [0, 200, 0, 63, 17]
    q_start, _, pos, seq = _stream(lens, starts)
    T, DK = sum(lens), rank + R
    cache, bt = _paged(g, lens, starts, BS, DK, dt)
    cache2 = cache.clone()
    q = _rand(g, T, H, D + R, dtype=dt)
    q2 = q.clone()
    dkv = _rand(g, T, DK, dtype=dt)
    wn = _rand(g, rank) * 0.1 + 1
    cs = rope_cos_sin(10000.0, dims, 512, DEV)
    hops.latent_prep(q, dkv, pos, seq, bt, wn, 1e-6, cs, dims, rank, cache)
    ref.latent_prep(q2, dkv, pos, seq, bt, wn, 1e-6, cs, dims, rank, cache2)
    _close(q, q2, _tol(dt, 1e-6, 8e-3))
    _close(cache, cache2, _tol(dt, 1e-6, 8e-3))
    qa = _rand(g, T, H, DK, dtype=dt, scale=0.3)
    gate = _rand(g, T, H)
    for gt in (gate, None):
        o = hops.latent_attention(qa, cache2, bt, q_start, pos, gt, 0.17, rank, dt, max(lens))
        o2 = ref.latent_attention(qa, cache2, bt, q_start, pos, gt, 0.17, rank, dt)
        _close(o, o2, _tol(dt, 2e-5, 1e-2))


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("R", [8, 32])
def test_latent_attention_sees_exactly_its_prefix(dt, R):
    """One key far back carries a huge score and a marker value: a query at or after it must return the marker, the
    query just before it must not (causal edge, inside a prompt portion and for a decode row)."""
    from chronos.ops import hybrid as hops

    g = _gen(9)
    H, rank, BS = 2, 32, 16     # (R = 32 in bfloat16: the matrix-core kernel; otherwise the general one)
    DK = rank + R
    lens, starts = [40, 1, 1], [100, 120, 119]
    q_start, _, pos, seq = _stream(lens, starts)
    cache, bt = _paged(g, lens, starts, BS, DK, dt)
    cache.mul_(0.01)
    far = 120
    for b in range(3):
        row = cache[bt[b, far // BS].item(), far % BS]
        row.zero_()
        row[rank:] = 8.0
        row[0] = 5.0
    qa = torch.zeros(sum(lens), H, DK, device=DEV, dtype=dt)
    qa[:, :, rank:] = 8.0
    o = hops.latent_attention(qa, cache, bt, q_start, pos, None, 1.0, rank, dt, max(lens)).float()
    first = o[:, 0, 0]
    assert float(first[21:40].min()) > 4.9 and float(first[:20].abs().max()) < 0.5    # prompt portion: positions 100..139
    assert float(first[40]) > 4.9 and abs(float(first[41])) < 0.5                      # decode rows at 120 and 119


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("d,F,E,I,top,T", [(192, 48, 6, 3, 2, 21), (96, 40, 3, 0, 1, 21), (128, 200, 5, 2, 7, 21),
                                            (256, 128, 6, 2, 3, 1), (128, 384, 3, 1, 2, 300), (384, 256, 9, 0, 4, 77)])
def test_moe(dt, d, F, E, I, top, T):
    """Widths on the 128 grid take the grouped MFMA GEMMs in bfloat16 (experts with no token, with one, with more
    than a tile of them), every other case the token-parallel kernel."""
    from chronos.ops import hybrid as hops, hybrid_ref as ref

    g = _gen(d + F)
    h = _rand(g, T, d, dtype=dt)
    wr = _rand(g, E + I, d, dtype=dt, scale=0.3)
    corr = _rand(g, E + I, scale=0.2)
    idx, wt = hops.moe_route(h, wr, corr, top)
    idx2, wt2 = ref.moe_route(h, wr, corr, top)
    assert torch.equal(idx.sort(-1).values, idx2.sort(-1).values)
    _close(wt.sum(-1), wt2.sum(-1), 1e-5)
    wu = _rand(g, E, F, d, dtype=dt, scale=d ** -0.5)
    wd = _rand(g, E, d, F, dtype=dt, scale=F ** -0.5)
    for act in (0, 1):
        y = hops.moe_ffn(h, idx2, wt2, wu, wd, act, dt)
        y2 = ref.moe_ffn(h, idx2, wt2, wu, wd, act, dt)
        _close(y, y2, _tol(dt, 2e-5, 1.5e-2))


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H,R,rank", [(4, 32, 96), (16, 64, 512), (3, 8, 40)])
def test_latent_attention_long_context_few_rows(dt, H, R, rank):
    """Decode rows and a two-token portion over contexts of very different lengths (3 to 1500 keys) behind a wide
    block table: the bfloat16 matrix-core kernel splits the key range over several workgroups and merges the
    partials; splits that get no key tile must not disturb the result."""
    from chronos.ops import hybrid as hops, hybrid_ref as ref

    g = _gen(H + rank)
    BS, DK = 16, rank + R
    lens, starts = [1, 1, 2, 1], [1499, 700, 2, 255]
    q_start, _, pos, _ = _stream(lens, starts)
    cache, bt = _paged(g, lens, starts, BS, DK, dt)
    wide = torch.zeros(len(lens), 128, dtype=torch.int32, device=DEV)
    wide[:, :bt.shape[1]] = bt
    qa = _rand(g, sum(lens), H, DK, dtype=dt, scale=0.3)
    gate = _rand(g, sum(lens), H)
    o = hops.latent_attention(qa, cache, wide, q_start, pos, gate, 0.2, rank, dt, max(lens))
    o2 = ref.latent_attention(qa, cache, wide, q_start, pos, gate, 0.2, rank, dt)
    _close(o, o2, _tol(dt, 2e-5, 1e-2))
