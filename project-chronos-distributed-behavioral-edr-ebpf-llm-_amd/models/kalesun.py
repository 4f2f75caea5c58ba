"""Kalesun: a hybrid decoder on a post-norm residual stream (x <- rms_norm(alpha x + sublayer(x))) whose layers mix
tokens with windowed grouped-query attention (query/key norm, partial rotation with wavelength-dependent frequency
scaling, a softmax sink per head, kept first tokens, value mixing across layers, per-head output gates), with the
gated delta rule, or with gated linear attention, and feed forward through a clamped gated unit, dense or as a mixture
of experts whose weights are the softmax over the chosen logits.  The logits come from the embedding table.

This module is the design's reader: ``config.json`` -> :class:`chronos.models.hybrid.HybridConfig`, the checkpoint's
tensor names -> the packed weights the hybrid kernels take, and random weights of the same shapes for benchmarks and
tests.  Everything computed lives in :mod:`chronos.models.hybrid` and :mod:`chronos.ops.hybrid`.

config.json:  architecture "Kalesun"; vocab, width, postln_alpha, norm.eps; layers[i] = {type, mixer{...}, mlp|null}
  type "attention":  mixer {heads, kv_heads, dim, vdim, scale, mask{size, keep_first}, v_mix,
                            rot{base, dims, scaling{factor, low, high, original}}}
  type "delta":      mixer {heads, kv_heads, dim, vdim, conv}
  type "gla":        mixer {heads, dim, vdim, tau}          (the decay projection's rank is the shape of mix.a1)
  mlp {kind "dense", ff, limit} | {kind "moe", expert{ff, limit}, router{experts, top}}
tensors (bfloat16, [out, in]):  embed, final.norm, l<i>.norm1, l<i>.norm2, l<i>.mix.*, l<i>.mlp.*
"""
from __future__ import annotations

import json
import os

import torch

from .hybrid import (FEED_FORWARDS, MIXERS, DeltaRuleSpec, GLASpec, GluFFSpec, HybridConfig, HybridDecoder,
                     HybridLayerWeights, HybridWeights, LayerSpec, MoEGluSpec, WindowAttentionSpec)
from .zokunex import _SafetensorsDir

ARCHITECTURE = "Kalesun"
GLU_SLOPE, GLU_SHIFT = 1.702, 1.0   # y = g sigmoid(1.702 g) (u + 1): fixed by the design
DEFAULT_GLA_RANK = 16


def config_from_dict(c: dict, name: str = "kalesun", max_position: int = 8192, gla_ranks: dict | None = None) -> HybridConfig:
    """``gla_ranks``: layer index -> rank of that layer's decay projection (a checkpoint's ``mix.a1`` has that many
    rows; config.json may also carry it as mixer.rank)."""
    layers, seen_vmix = [], False
    for i, l in enumerate(c["layers"]):
        mx = l["mixer"]
        if l["type"] == "attention":
            rot, mask = mx.get("rot") or {}, mx.get("mask") or {}
            sc = rot.get("scaling")
            mixer = WindowAttentionSpec(
                int(mx["heads"]), int(mx.get("kv_heads", mx["heads"])), int(mx["dim"]), int(mx["vdim"]),
                float(mx["scale"]), int(mask.get("size", 0)), int(mask.get("keep_first", 0)),
                float(rot.get("base", 10000.0)), int(rot.get("dims", 0)),
                (float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"])) if sc else None,
                bool(mx.get("v_mix", False)))
            if mixer.v_mix and not seen_vmix:
                mixer.v_mix_first, seen_vmix = True, True
            if mixer.heads % mixer.kv_heads:
                raise ValueError(f"layer {i}: heads must be a multiple of kv_heads")
            if mixer.rope_dims % 2 or mixer.rope_dims > mixer.dim:
                raise ValueError(f"layer {i}: rot.dims must be even and at most dim")
        elif l["type"] == "delta":
            mixer = DeltaRuleSpec(int(mx["heads"]), int(mx.get("kv_heads", mx["heads"])), int(mx["dim"]),
                                  int(mx["vdim"]), int(mx["conv"]))
            if mixer.heads % mixer.kv_heads or mixer.conv < 1:
                raise ValueError(f"layer {i}: heads must be a multiple of kv_heads and conv at least 1")
        elif l["type"] == "gla":
            rank = int((gla_ranks or {}).get(i, mx.get("rank", DEFAULT_GLA_RANK)))
            mixer = GLASpec(int(mx["heads"]), int(mx["dim"]), int(mx["vdim"]), float(mx["tau"]), rank)
        else:
            raise ValueError(f"layer {i}: unknown mixer type {l['type']!r}")
        mlp = l.get("mlp")
        if mlp is None:
            ff = None
        elif mlp["kind"] == "dense":
            ff = GluFFSpec(int(mlp["ff"]), float(mlp["limit"]), GLU_SLOPE, GLU_SHIFT)
        elif mlp["kind"] == "moe":
            r = mlp["router"]
            ff = MoEGluSpec(int(r["experts"]), int(r["top"]), int(mlp["expert"]["ff"]), float(mlp["expert"]["limit"]),
                            GLU_SLOPE, GLU_SHIFT)
            if not 1 <= ff.top <= ff.experts:
                raise ValueError(f"layer {i}: router picks more experts than it has")
        else:
            raise ValueError(f"layer {i}: unknown feed-forward kind {mlp['kind']!r}")
        layers.append(LayerSpec(mixer, ff))
    vm = [l.mixer for l in layers if l.mixer.kind == "window_attention" and l.mixer.v_mix]
    if any((m.kv_heads, m.vdim) != (vm[0].kv_heads, vm[0].vdim) for m in vm):
        raise ValueError("value-mixing layers must agree in kv_heads and vdim")
    return HybridConfig(name=name, vocab_size=int(c["vocab"]), hidden_size=int(c["width"]), layers=layers,
                        norm_eps=float(c["norm"]["eps"]), max_position=max_position, architecture=ARCHITECTURE,
                        residual="post_norm", residual_alpha=float(c["postln_alpha"]), tied_head=True)


def config_to_dict(cfg: HybridConfig) -> dict:
    """The config.json form of a configuration (what :func:`config_from_dict` reads)."""
    layers = []
    for l in cfg.layers:
        m = l.mixer
        if m.kind == "window_attention":
            mixer = dict(heads=m.heads, kv_heads=m.kv_heads, dim=m.dim, vdim=m.vdim, scale=m.scale, v_mix=m.v_mix)
            if m.window:
                mixer["mask"] = dict(size=m.window, keep_first=m.keep_first)
            if m.rope_dims:
                mixer["rot"] = dict(base=m.rope_base, dims=m.rope_dims)
                if m.rope_scaling:
                    mixer["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), m.rope_scaling))
            typ = "attention"
        elif m.kind == "delta_rule":
            mixer, typ = dict(heads=m.heads, kv_heads=m.kv_heads, dim=m.dim, vdim=m.vdim, conv=m.conv), "delta"
        else:
            mixer, typ = dict(heads=m.heads, dim=m.dim, vdim=m.vdim, tau=m.tau, rank=m.rank), "gla"
        if l.ff is None:
            mlp = None
        elif l.ff.kind == "glu":
            mlp = dict(kind="dense", ff=l.ff.ff, limit=l.ff.limit)
        else:
            mlp = dict(kind="moe", expert=dict(ff=l.ff.ff, limit=l.ff.limit),
                       router=dict(experts=l.ff.experts, top=l.ff.top))
        layers.append(dict(type=typ, mixer=mixer, mlp=mlp))
    return dict(architecture=ARCHITECTURE, vocab=cfg.vocab_size, width=cfg.hidden_size,
                postln_alpha=cfg.residual_alpha, norm=dict(eps=cfg.norm_eps), layers=layers)


def tensor_shapes(cfg: HybridConfig) -> dict:
    """Checkpoint tensor name -> shape."""
    d, out = cfg.hidden_size, {"embed": (cfg.vocab_size, cfg.hidden_size), "final.norm": (cfg.hidden_size,)}
    for i, l in enumerate(cfg.layers):
        m, p = l.mixer, f"l{i}."
        out[p + "norm1"] = (d,)
        if m.kind == "window_attention":
            out.update({p + "mix.q": (m.heads * m.dim, d), p + "mix.k": (m.kv_heads * m.dim, d),
                        p + "mix.v": (m.kv_heads * m.vdim, d), p + "mix.q.norm": (m.dim,), p + "mix.k.norm": (m.dim,),
                        p + "mix.sink": (m.heads,), p + "mix.g": (m.heads, d), p + "mix.o": (d, m.heads * m.vdim)})
            if m.v_mix:
                out[p + "mix.vmix"] = ()
        elif m.kind == "delta_rule":
            qk, hv = m.kv_heads * m.dim, m.heads * m.vdim
            out.update({p + "mix.q": (qk, d), p + "mix.q.conv": (qk, m.conv), p + "mix.k": (qk, d),
                        p + "mix.k.conv": (qk, m.conv), p + "mix.v": (hv, d), p + "mix.v.conv": (hv, m.conv),
                        p + "mix.b": (m.heads, d), p + "mix.a": (m.heads, d), p + "mix.A_log": (m.heads,),
                        p + "mix.dt_bias": (m.heads,), p + "mix.norm": (m.vdim,), p + "mix.g": (hv, d),
                        p + "mix.o": (d, hv)})
        else:
            hd, hv = m.heads * m.dim, m.heads * m.vdim
            out.update({p + "mix.q": (hd, d), p + "mix.k": (hd, d), p + "mix.v": (hv, d), p + "mix.g": (hv, d),
                        p + "mix.o": (d, hv), p + "mix.norm": (m.vdim,), p + "mix.a1": (m.rank, d),
                        p + "mix.a2": (hd, m.rank), p + "mix.a2.b": (hd,)})
        f = l.ff
        if f is not None:
            out[p + "norm2"] = (d,)
            if f.kind == "glu":
                out.update({p + "mlp.gate": (f.ff, d), p + "mlp.up": (f.ff, d), p + "mlp.down": (d, f.ff)})
            else:
                for e in range(f.experts):
                    out.update({p + f"mlp.e{e}.gate": (f.ff, d), p + f"mlp.e{e}.up": (f.ff, d),
                                p + f"mlp.e{e}.down": (d, f.ff)})
                out.update({p + "mlp.router": (f.experts, d), p + "mlp.router.b": (f.experts,)})
    return out


def random_tensors(cfg: HybridConfig, seed: int = 0, device="cpu", std: float | None = None) -> dict:
    """Checkpoint-named random bfloat16 tensors (norm weights near one; biases, sinks and decay parameters small;
    decay-logit biases positive, so the linear-attention state mostly persists)."""
    gen = torch.Generator(device="cpu")
    gen.manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        if len(shape) == 0:
            t = torch.rand((), generator=gen) * 0.5 + 0.2
        elif len(shape) == 1:
            t = torch.randn(shape, generator=gen) * 0.1
            if "norm" in name:
                t = t + 1.0
            if name.endswith("a2.b"):
                t = t + 2.0
        elif name.endswith(".conv"):
            t = torch.randn(shape, generator=gen) * 0.5
        else:
            t = torch.randn(shape, generator=gen) * (std if std is not None else shape[1] ** -0.5)
        out[name] = t.to(torch.bfloat16).to(device)
    return out


def pack_weights(cfg: HybridConfig, tensors, device, act_dtype) -> HybridWeights:
    """``tensors``: a mapping (or any object with ``__getitem__``) from checkpoint names to tensors."""
    a = lambda x: x.to(device=device, dtype=act_dtype).contiguous()  # noqa: E731
    f = lambda x: x.to(device=device, dtype=torch.float32).contiguous()  # noqa: E731
    shapes = tensor_shapes(cfg)

    def get(name):
        t = tensors[name]
        if tuple(t.shape) != tuple(shapes[name]):
            raise ValueError(f"tensor {name}: shape {tuple(t.shape)}, the configuration says {tuple(shapes[name])}")
        return t

    layers = []
    for i, l in enumerate(cfg.layers):
        p = f"l{i}.mix."
        names = [n[len(p):] for n in shapes if n.startswith(p)]
        if l.mixer.kind == "window_attention" and l.mixer.v_mix_first:
            names.remove("vmix")   # the source layer of the mixed-in values has the tensor but does not use it
        mix = MIXERS[l.mixer.kind][1](l.mixer, {n: get(p + n) for n in names}, device, act_dtype)
        lw = HybridLayerWeights(f(get(f"l{i}.norm1")), mix)
        if l.ff is not None:
            p = f"l{i}.mlp."
            names = [n[len(p):] for n in shapes if n.startswith(p)]
            lw.norm2 = f(get(f"l{i}.norm2"))
            lw.ff = FEED_FORWARDS[l.ff.kind][1](l.ff, {n: get(p + n) for n in names}, device, act_dtype)
        layers.append(lw)
    embed = a(get("embed"))
    return HybridWeights(embed, layers, f(get("final.norm")), embed)


def is_checkpoint(path: str) -> bool:
    cj = os.path.join(path, "config.json")
    if not os.path.exists(cj):
        return False
    with open(cj) as fh:
        return json.load(fh).get("architecture") == ARCHITECTURE


def load(path: str, device="cpu", act_dtype=torch.bfloat16, max_position: int | None = None) -> HybridDecoder:
    with open(os.path.join(path, "config.json")) as fh:
        c = json.load(fh)
    tensors = _SafetensorsDir(path)
    ranks = {i: int(tensors.shape(f"l{i}.mix.a1")[0]) for i, l in enumerate(c["layers"]) if l["type"] == "gla"}
    cfg = config_from_dict(c, name=os.path.basename(path.rstrip("/")) or "kalesun",
                           max_position=max_position or 8192, gla_ranks=ranks)
    return HybridDecoder(cfg, pack_weights(cfg, tensors, device, act_dtype), device, max_position, act_dtype)


def save(cfg: HybridConfig, tensors: dict, path: str) -> None:
    """Write config.json + model.safetensors (bfloat16) — the layout :func:`load` reads."""
    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as fh:
        json.dump(config_to_dict(cfg), fh, indent=1)
    save_file({k: v.to(torch.bfloat16).cpu().contiguous() for k, v in tensors.items()},
              os.path.join(path, "model.safetensors"))


def _preset(width, vocab, pattern, heads, kv_heads, dim, vdim, window, keep, ff, experts, top, eff) -> dict:
    """pattern: one letter per layer — a = windowed attention, d = delta rule, g = gated linear attention; upper case
    = dense feed-forward, lower = mixture of experts."""
    layers = []
    for ch in pattern:
        k = ch.lower()
        if k == "a":
            mixer, typ = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=dim ** -0.5, v_mix=True,
                              mask=dict(size=window, keep_first=keep),
                              rot=dict(base=500000.0, dims=dim // 2,
                                       scaling=dict(factor=8.0, low=1.0, high=4.0, original=8192))), "attention"
        elif k == "d":
            mixer, typ = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, conv=4), "delta"
        else:
            mixer, typ = dict(heads=heads, dim=dim, vdim=vdim, tau=16.0, rank=16), "gla"
        mlp = dict(kind="dense", ff=ff, limit=7.0) if ch.isupper() else dict(
            kind="moe", expert=dict(ff=eff, limit=7.0), router=dict(experts=experts, top=top))
        layers.append(dict(type=typ, mixer=mixer, mlp=mlp))
    return dict(architecture=ARCHITECTURE, vocab=vocab, width=width, postln_alpha=2.0, norm=dict(eps=1e-6),
                layers=layers)


# random-init presets (benchmarks, smoke runs); sizes in the range of real models' layers
PRESETS = {
    "kalesun-tiny": _preset(128, 512, "DgA", 2, 1, 32, 32, 24, 4, 256, 4, 2, 64),
    "kalesun-1b": _preset(2048, 32768, "DgAdDgAd", 16, 4, 128, 128, 1024, 16, 8192, 16, 4, 1024),
    "kalesun-8b-layers": _preset(4096, 128256, "DgAd", 32, 8, 128, 128, 4096, 64, 14336, 32, 4, 2048),
}


def build(name_or_path: str, device="cpu", seed: int = 0, act_dtype=torch.bfloat16,
          max_position: int | None = None) -> HybridDecoder:
    if os.path.isdir(name_or_path):
        return load(name_or_path, device, act_dtype, max_position)
    cfg = config_from_dict(PRESETS[name_or_path], name=name_or_path, max_position=max_position or 8192)
    w = pack_weights(cfg, random_tensors(cfg, seed), device, act_dtype)
    return HybridDecoder(cfg, w, device, max_position, act_dtype)
