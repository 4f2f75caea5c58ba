"""Throughput of a hybrid design (Zokunex) beside the Llama family at equal width and depth: whole-model prefill and
decode steps, and each new kernel beside its closest Llama kernel with the fraction of its roofline it reaches.

``python bench.py --design-compare [--design-sizes 1k,2k,4k]`` prints one JSON line (the default benchmark and its
output line are untouched).  Weights are random; every number is measured on the GPU this process runs on.

Rooflines: HBM 8 TB/s for kernels bound by the bytes they must move, 2.5 PFLOP/s dense bf16 for the matrix-shaped
ones (the attention kernels over a long context are priced by their FLOPs in prefill and by their cache bytes in
decode, like the Llama kernels they stand beside).
"""
from __future__ import annotations

import json
import sys
import time

import torch

HBM_BPS = 8.0e12
BF16_FLOPS = 2.5e15

# width -> (mlstm heads, dim, vdim | latent heads, dim, rot, vdim, rank | dense ff | experts, identity, top, expert ff)
SIZES = {
    "1k": dict(width=1024, m=(4, 128, 256), a=(8, 64, 32, 64, 256), ff=4096, moe=(8, 2, 2, 512)),
    "2k": dict(width=2048, m=(4, 256, 512), a=(16, 128, 64, 128, 512), ff=8192, moe=(16, 2, 4, 1408)),
    "4k": dict(width=4096, m=(8, 256, 512), a=(32, 128, 64, 128, 512), ff=14336, moe=(32, 2, 4, 2048)),
}
LAYERS = 4
VOCAB = 32768


def zokunex_config(size: dict) -> dict:
    mh, md, mv = size["m"]
    ah, ad, ar, av, rank = size["a"]
    ne, ni, top, eff = size["moe"]
    mix_m = dict(type="mlstm", mixer=dict(heads=mh, dim=md, vdim=mv, gate_cap=10.0))
    mix_a = dict(type="latent_attention", mixer=dict(heads=ah, dim=ad, rot_dim=ar, vdim=av, kv_rank=rank,
                                                     scale=(ad + ar) ** -0.5, rot=dict(base=10000.0, dims=ar)))
    dense = dict(kind="dense", ff=size["ff"])
    moe = dict(kind="moe", expert=dict(ff=eff), router=dict(experts=ne, identity=ni, top=top))
    layers = [dict(mix_m, mlp=dense), dict(mix_a, mlp=moe), dict(mix_m, mlp=moe), dict(mix_a, mlp=dense)][:LAYERS]
    return dict(architecture="Zokunex", vocab=VOCAB, width=size["width"], logit_scale=1.0, norm=dict(eps=1e-5),
                layers=layers)


def _say(msg: str) -> None:
    print(f"[design-compare] {time.strftime('%H:%M:%S')} {msg}", file=sys.stderr, flush=True)


def _time(fn, iters: int = 10, warm: int = 2) -> float:
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(iters):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / iters * 1e-3


def _graph(fn):
    fn()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        fn()
    return g.replay


def _model_steps(model, dev, seqs: int, plen: int, rows: int, ctx: int) -> dict:
    """Prefill of ``seqs`` prompts of ``plen`` tokens in one step; then decode steps of ``rows`` rows at context
    ``ctx`` (captured into a graph, as the engine runs them)."""
    from chronos.models.llama import StepBatch

    bs = 16
    need = max(seqs * plen, rows * (ctx + 1))
    nb = need // bs + rows + seqs + 2
    cache = model.make_cache(nb, bs, max(rows, seqs))
    vocab = model.cfg.vocab_size
    g = torch.Generator().manual_seed(0)
    per = (plen + bs - 1) // bs
    chunks = [torch.randint(0, vocab, (plen,), generator=g).tolist() for _ in range(seqs)]
    bts = [list(range(1 + b * per, 1 + (b + 1) * per)) for b in range(seqs)]
    sb = model.prefill_batch(chunks, [0] * seqs, bts, list(range(seqs)), max_blocks=per, nqt=8)
    t_pre = _time(lambda: model.forward(sb, cache), iters=3, warm=1)
    per = (ctx + 1 + bs - 1) // bs
    i32 = dict(dtype=torch.int32, device=dev)
    bt = torch.arange(1, 1 + rows * per, **i32).view(rows, per)
    ar = torch.arange(rows + 1, **i32)
    from chronos import ops

    dsb = StepBatch(torch.randint(0, vocab, (rows,), generator=g).to(dev).int(), torch.full((rows,), ctx, **i32),
                    ar[:rows], bt, ar, torch.full((rows,), ctx + 1, **i32), torch.arange(rows, device=dev), None, rows, 1,
                    ops.pick_nsplit(rows * model.hkv, ctx + 1), slots=ar[:rows].clone(), max_q=1)
    t_dec = _time(_graph(lambda: model.forward(dsb, cache)), iters=20)
    return dict(prefill_tokens_s=seqs * plen / t_pre, prefill_ms=t_pre * 1e3, decode_tokens_s=rows / t_dec,
                decode_ms=t_dec * 1e3)


def _kernels(size: dict, dev, T: int, ctx: int, rows: int) -> dict:
    """Each new kernel and its Llama counterpart at this size: seconds, and the fraction of the roofline reached."""
    from chronos import ops
    from chronos.models.hybrid import rope_cos_sin
    from chronos.ops import hybrid as hops

    out = {}
    bf = torch.bfloat16
    d = size["width"]
    g = torch.Generator(device=dev).manual_seed(1)
    rnd = lambda *s, dt=bf, sc=1.0: (torch.randn(*s, device=dev, generator=g) * sc).to(dt)  # noqa: E731
    i32 = dict(dtype=torch.int32, device=dev)

    def rec(name, secs, nbytes=0.0, flops=0.0):
        roof = max(nbytes / HBM_BPS, flops / BF16_FLOPS)
        _say(f"  {name}: {secs * 1e6:.1f} us, roofline {roof * 1e6:.2f} us")
        out[name] = dict(us=round(secs * 1e6, 1), roofline_us=round(roof * 1e6, 2), of_roofline=round(roof / secs, 4))

    # ---- norms on the residual stream
    y, x32, w32 = rnd(T, d), rnd(T, d, dt=torch.float32), rnd(d, dt=torch.float32)
    rec("add_layer_norm", _time(lambda: hops.add_layer_norm(y, x32, w32, 1e-5, bf)), T * d * (2 + 4 + 4 + 2))
    xb, wb = rnd(T, d), rnd(d)
    rec("llama.add_rmsnorm", _time(lambda: ops.add_rmsnorm(y, xb, wb, 1e-5)), T * d * (2 + 2 + 2 + 2))
    # ---- attention: prefill of T tokens (seqs of `ctx`), decode of `rows` rows at context ctx
    H, D, R, Dv, rank = size["a"]
    DK, bs = rank + R, 16
    seqs = max(1, T // ctx)
    per = ctx // bs + 1
    nb = max(seqs, rows) * per + 1
    cache = rnd(nb, bs, DK, sc=0.3)
    qa = rnd(seqs * ctx, H, DK, sc=0.3)
    gate = rnd(seqs * ctx, H, dt=torch.float32)
    bt = torch.arange(1, 1 + seqs * per, **i32).view(seqs, per)
    qs = torch.arange(0, (seqs + 1) * ctx, ctx, **i32)
    pos = torch.arange(ctx, **i32).repeat(seqs)
    pairs = seqs * ctx * (ctx + 1) / 2
    rec("latent_attention.prefill", _time(lambda: hops.latent_attention(qa, cache, bt, qs, pos, gate, 0.1, rank, bf, ctx), iters=3, warm=1),
        flops=2.0 * pairs * H * (DK + rank))
    btd = torch.arange(1, 1 + rows * per, **i32).view(rows, per)
    qsd = torch.arange(rows + 1, **i32)
    posd = torch.full((rows,), ctx, **i32)
    qad, gated = rnd(rows, H, DK, sc=0.3), rnd(rows, H, dt=torch.float32)
    rec("latent_attention.decode", _time(lambda: hops.latent_attention(qad, cache, btd, qsd, posd, gated, 0.1, rank, bf, 1)),
        nbytes=rows * (ctx + 1) * DK * 2.0)
    hq = d // 128
    hkv = max(1, hq // 4)
    kc, vc = rnd(nb, hkv, bs, 128, sc=0.3), rnd(nb, hkv, 128, bs, sc=0.3)
    q = rnd(seqs * ctx, hq, 128, sc=0.3)
    ctxl = torch.full((seqs,), ctx, **i32)
    tiles = torch.tensor(ops.attention_tiles([ctx] * seqs, hq, hkv, 8), **i32).view(-1, 2)
    rec("llama.attention.prefill", _time(lambda: ops.paged_attention(q, kc, vc, bt, qs, ctxl, tiles, tiles.shape[0], 8, 1), iters=3, warm=1),
        flops=4.0 * pairs * hq * 128)
    qd = rnd(rows, hq, 128, sc=0.3)
    ctxd = torch.full((rows,), ctx + 1, **i32)
    ns = ops.pick_nsplit(rows * hkv, ctx + 1)
    rec("llama.attention.decode", _time(lambda: ops.paged_attention(qd, kc, vc, btd, qsd, ctxd, None, rows, 1, ns)),
        nbytes=rows * (ctx + 1) * hkv * 128 * 2 * 2.0)
    # ---- the recurrence: prefill (FLOPs of the state update and read-out), decode (state bytes in and out)
    mh, md, mv = size["m"]
    C = 2 * mh * md + 2 * mh * mv
    proj = rnd(seqs * ctx, C, sc=0.5)
    gp = rnd(seqs * ctx, 2 * mh, dt=torch.float32)
    NS = max(seqs, rows) + 1
    S, n, m = (torch.zeros(NS, mh, md, mv, device=dev), torch.zeros(NS, mh, md, device=dev), torch.zeros(NS, mh, device=dev))
    p0 = torch.zeros(seqs, **i32)
    sl = torch.arange(seqs, **i32)
    rec("mlstm_scan.prefill", _time(lambda: hops.mlstm_scan(proj, gp, qs, p0, sl, S, n, m, mh, md, mv, 10.0, ctx), iters=3, warm=1),
        nbytes=seqs * ctx * C * 2.0, flops=seqs * ctx * mh * md * mv * 6.0)
    projd, gpd = rnd(rows, C, sc=0.5), rnd(rows, 2 * mh, dt=torch.float32)
    sld = torch.arange(rows, **i32)
    rec("mlstm_scan.decode", _time(lambda: hops.mlstm_scan(projd, gpd, qsd, posd, sld, S, n, m, mh, md, mv, 10.0, 1)),
        nbytes=rows * mh * md * mv * 4 * 2.0)
    # ---- feed-forwards: the mixture of experts beside a dense SwiGLU of the Llama model at this width
    ne, ni, top, eff = size["moe"]
    wr, corr = rnd(ne + ni, d, sc=0.05), rnd(ne + ni, dt=torch.float32, sc=0.01)
    wu, wd = rnd(ne, eff, d, sc=d ** -0.5), rnd(ne, d, eff, sc=eff ** -0.5)
    for name, tk in (("prefill", T), ("decode", rows)):
        h = rnd(tk, d)
        idx, wt = hops.moe_route(h, wr, corr, top)
        rec(f"moe_route.{name}", _time(lambda: hops.moe_route(h, wr, corr, top)), nbytes=tk * d * 2.0 + (ne + ni) * d * 2.0)
        real = float((idx < ne).sum())
        used = min(ne, real) * 2 * eff * d * 2.0
        rec(f"moe_ffn.{name}", _time(lambda: hops.moe_ffn(h, idx, wt, wu, wd, 1, bf), iters=3, warm=1),
            nbytes=used + tk * d * 4.0, flops=real * 4.0 * eff * d)
        f = int(3.5 * d)
        wgu, wdn = rnd(2 * f, d, sc=d ** -0.5), rnd(d, f, sc=f ** -0.5)
        rec(f"llama.mlp.{name}", _time(lambda: ops.linear(ops.gate_up_silu(h, wgu), wdn), iters=3, warm=1),
            nbytes=3 * f * d * 2.0 + tk * d * 4.0, flops=tk * 6.0 * f * d)
    return out


def run(sizes: list, seqs: int = 4, plen: int = 2048, rows: int = 64, ctx: int = 2048, device: str = "cuda") -> dict:
    from chronos import ops
    from chronos.models import llama, zokunex
    from chronos.models.hybrid import HybridDecoder

    dev = torch.device(device if ":" in device else device + ":0")
    torch.cuda.set_device(dev)
    ops.load()
    ops.device_init()
    res = {}
    for name in sizes:
        size = SIZES[name]
        t0 = time.time()
        cfg = zokunex.config_from_dict(zokunex_config(size), name=f"zokunex-{name}", max_position=ctx + plen + 16)
        zk = HybridDecoder(cfg, zokunex.pack_weights(cfg, zokunex.random_tensors(cfg, 0), dev, torch.bfloat16), dev,
                           ctx + plen + 16, torch.bfloat16)
        d = size["width"]
        lc = llama.LlamaConfig(name=f"llama-{name}", vocab_size=VOCAB, hidden_size=d, intermediate_size=int(3.5 * d),
                               num_layers=LAYERS, num_heads=d // 128, num_kv_heads=max(1, d // 512),
                               max_position=ctx + plen + 16)
        lm = llama.LlamaModel(lc, llama.random_weights(lc, None, dev, 0), None, dev, ctx + plen + 16)
        _say(f"size {name}: models built")
        entry = dict(zokunex=dict(params=cfg.param_count(), **_model_steps(zk, dev, seqs, plen, rows, ctx)))
        _say(f"  zokunex {entry['zokunex']}")
        entry["llama"] = dict(params=lc.param_count(), **_model_steps(lm, dev, seqs, plen, rows, ctx))
        _say(f"  llama {entry['llama']}")
        entry["kernels"] = _kernels(size, dev, seqs * plen, ctx, rows)
        entry["seconds"] = round(time.time() - t0, 1)
        res[name] = entry
        del zk, lm
        torch.cuda.empty_cache()
    return dict(metric="design_compare", design="zokunex", beside="llama (equal width and depth)", layers=LAYERS,
                workload=dict(prefill=f"{seqs} x {plen} tokens in one step", decode=f"{rows} rows at context {ctx}"),
                dtype="bf16", data="synthetic", sizes=res)


def main(a) -> int:
    out = run([s for s in a.design_sizes.split(",") if s], device=a.device)
    print(json.dumps(out), flush=True)
    return 0
