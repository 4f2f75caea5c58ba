"""Zokunex: a hybrid decoder whose layers mix tokens either with a matrix-memory recurrence (mLSTM) or with latent
attention, and feed forward through a dense squared-ReLU layer or a mixture of experts with identity experts and a
selection-only router correction.

This module is the design's reader: ``config.json`` -> :class:`chronos.models.hybrid.HybridConfig`, the checkpoint's
tensor names -> the packed weights the hybrid kernels take, and random weights of the same shapes for benchmarks and
tests.  Everything computed lives in :mod:`chronos.models.hybrid` and :mod:`chronos.ops.hybrid`.

config.json:  architecture "Zokunex"; vocab, width, logit_scale, norm.eps; layers[i] = {type, mixer{...}, mlp|null}
  type "mlstm":             mixer {heads, dim, vdim, gate_cap}
  type "latent_attention":  mixer {heads, dim, rot_dim, vdim, kv_rank, scale, rot{base, dims}}
  mlp {kind "dense", ff} | {kind "moe", expert{ff}, router{experts, identity, top}}
tensors (bfloat16, [out, in]):  embed, head, final.norm, l<i>.norm1, l<i>.norm2, l<i>.mix.*, l<i>.mlp.*
"""
from __future__ import annotations

import json
import os

import torch

from ..ops import hybrid as hops
from .hybrid import (FEED_FORWARDS, MIXERS, DenseFFSpec, HybridConfig, HybridDecoder, HybridLayerWeights,
                     HybridWeights, LatentAttentionSpec, LayerSpec, MLSTMSpec, MoEFFSpec)

ARCHITECTURE = "Zokunex"


def config_from_dict(c: dict, name: str = "zokunex", max_position: int = 8192) -> HybridConfig:
    layers = []
    for i, l in enumerate(c["layers"]):
        mx = l["mixer"]
        if l["type"] == "mlstm":
            mixer = MLSTMSpec(int(mx["heads"]), int(mx["dim"]), int(mx["vdim"]), float(mx["gate_cap"]))
        elif l["type"] == "latent_attention":
            rot = mx.get("rot") or {}
            mixer = LatentAttentionSpec(int(mx["heads"]), int(mx["dim"]), int(mx["rot_dim"]), int(mx["vdim"]),
                                        int(mx["kv_rank"]), float(mx["scale"]), float(rot["base"]),
                                        int(rot.get("dims", mx["rot_dim"])))
            if mixer.rope_dims % 2 or mixer.rope_dims > mixer.rot_dim:
                raise ValueError(f"layer {i}: rot.dims must be even and at most rot_dim")
        else:
            raise ValueError(f"layer {i}: unknown mixer type {l['type']!r}")
        mlp = l.get("mlp")
        if mlp is None:
            ff = None
        elif mlp["kind"] == "dense":
            ff = DenseFFSpec(int(mlp["ff"]), hops.ACT_RELU2)
        elif mlp["kind"] == "moe":
            r = mlp["router"]
            ff = MoEFFSpec(int(r["experts"]), int(r.get("identity", 0)), int(r["top"]), int(mlp["expert"]["ff"]),
                           hops.ACT_GELU)
            if ff.top > ff.experts + ff.identity:
                raise ValueError(f"layer {i}: router picks more experts than it has")
        else:
            raise ValueError(f"layer {i}: unknown feed-forward kind {mlp['kind']!r}")
        layers.append(LayerSpec(mixer, ff))
    return HybridConfig(name=name, vocab_size=int(c["vocab"]), hidden_size=int(c["width"]), layers=layers,
                        norm_eps=float(c["norm"]["eps"]), logit_scale=float(c.get("logit_scale", 1.0)),
                        max_position=max_position, architecture=ARCHITECTURE)


def config_to_dict(cfg: HybridConfig) -> dict:
    """The config.json form of a configuration (what :func:`config_from_dict` reads)."""
    layers = []
    for l in cfg.layers:
        m = l.mixer
        if m.kind == "mlstm":
            mixer = dict(heads=m.heads, dim=m.dim, vdim=m.vdim, gate_cap=m.gate_cap)
        else:
            mixer = dict(heads=m.heads, dim=m.dim, rot_dim=m.rot_dim, vdim=m.vdim, kv_rank=m.kv_rank, scale=m.scale,
                         rot=dict(base=m.rope_base, dims=m.rope_dims))
        if l.ff is None:
            mlp = None
        elif l.ff.kind == "dense":
            mlp = dict(kind="dense", ff=l.ff.ff)
        else:
            mlp = dict(kind="moe", expert=dict(ff=l.ff.ff),
                       router=dict(experts=l.ff.experts, identity=l.ff.identity, top=l.ff.top))
        layers.append(dict(type=m.kind, mixer=mixer, mlp=mlp))
    return dict(architecture=ARCHITECTURE, vocab=cfg.vocab_size, width=cfg.hidden_size, logit_scale=cfg.logit_scale,
                norm=dict(eps=cfg.norm_eps), layers=layers)


def tensor_shapes(cfg: HybridConfig) -> dict:
    """Checkpoint tensor name -> shape."""
    d, out = cfg.hidden_size, {"embed": (cfg.vocab_size, cfg.hidden_size), "final.norm": (cfg.hidden_size,),
                               "head": (cfg.vocab_size, cfg.hidden_size)}
    for i, l in enumerate(cfg.layers):
        m, p = l.mixer, f"l{i}."
        out[p + "norm1"] = (d,)
        if m.kind == "mlstm":
            out.update({p + "mix.q": (m.heads * m.dim, d), p + "mix.k": (m.heads * m.dim, d),
                        p + "mix.v": (m.heads * m.vdim, d), p + "mix.g": (m.heads * m.vdim, d),
                        p + "mix.o": (d, m.heads * m.vdim), p + "mix.norm": (m.heads * m.vdim,),
                        p + "mix.i": (m.heads, d), p + "mix.i.b": (m.heads,), p + "mix.f": (m.heads, d),
                        p + "mix.f.b": (m.heads,)})
        else:
            out.update({p + "mix.q": (m.heads * (m.dim + m.rot_dim), d), p + "mix.dkv": (m.kv_rank + m.rot_dim, d),
                        p + "mix.dkv.norm": (m.kv_rank,), p + "mix.uk": (m.heads * m.dim, m.kv_rank),
                        p + "mix.uv": (m.heads * m.vdim, m.kv_rank), p + "mix.g": (m.heads, d),
                        p + "mix.o": (d, m.heads * m.vdim)})
        f = l.ff
        if f is not None:
            out[p + "norm2"] = (d,)
            if f.kind == "dense":
                out.update({p + "mlp.up": (f.ff, d), p + "mlp.down": (d, f.ff)})
            else:
                for e in range(f.experts):
                    out.update({p + f"mlp.e{e}.up": (f.ff, d), p + f"mlp.e{e}.down": (d, f.ff)})
                out.update({p + "mlp.router": (f.experts + f.identity, d),
                            p + "mlp.correction": (f.experts + f.identity,)})
    return out


def random_tensors(cfg: HybridConfig, seed: int = 0, device="cpu", std: float | None = None) -> dict:
    """Checkpoint-named random bfloat16 tensors (norm weights near one, biases and corrections small)."""
    gen = torch.Generator(device="cpu")
    gen.manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        if len(shape) == 1:
            t = torch.randn(shape, generator=gen) * 0.1
            if "norm" in name:
                t = t + 1.0
            if name.endswith("f.b"):
                t = t + 2.0   # forget gates that mostly keep the state
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
        mix = MIXERS[l.mixer.kind][1](l.mixer, {n: get(p + n) for n in names}, device, act_dtype)
        lw = HybridLayerWeights(f(get(f"l{i}.norm1")), mix)
        if l.ff is not None:
            p = f"l{i}.mlp."
            names = [n[len(p):] for n in shapes if n.startswith(p)]
            lw.norm2 = f(get(f"l{i}.norm2"))
            lw.ff = FEED_FORWARDS[l.ff.kind][1](l.ff, {n: get(p + n) for n in names}, device, act_dtype)
        layers.append(lw)
    return HybridWeights(a(get("embed")), layers, f(get("final.norm")), a(get("head")))


class _SafetensorsDir:
    def __init__(self, path: str):
        import glob

        from safetensors import safe_open

        files = sorted(glob.glob(os.path.join(path, "*.safetensors")))
        if not files:
            raise FileNotFoundError(f"no *.safetensors in {path}")
        self._h = [safe_open(f, framework="pt") for f in files]
        self._where = {k: h for h in self._h for k in h.keys()}

    def __getitem__(self, name):
        if name not in self._where:
            raise KeyError(f"checkpoint has no tensor {name!r}")
        return self._where[name].get_tensor(name)

    def shape(self, name) -> tuple:
        if name not in self._where:
            raise KeyError(f"checkpoint has no tensor {name!r}")
        return tuple(self._where[name].get_slice(name).get_shape())


def is_checkpoint(path: str) -> bool:
    cj = os.path.join(path, "config.json")
    if not os.path.exists(cj):
        return False
    with open(cj) as fh:
        return json.load(fh).get("architecture") == ARCHITECTURE


def load(path: str, device="cpu", act_dtype=torch.bfloat16, max_position: int | None = None) -> HybridDecoder:
    with open(os.path.join(path, "config.json")) as fh:
        cfg = config_from_dict(json.load(fh), name=os.path.basename(path.rstrip("/")) or "zokunex",
                               max_position=max_position or 8192)
    w = pack_weights(cfg, _SafetensorsDir(path), device, act_dtype)
    return HybridDecoder(cfg, w, device, max_position, act_dtype)


def save(cfg: HybridConfig, tensors: dict, path: str) -> None:
    """Write config.json + model.safetensors (bfloat16) — the layout :func:`load` reads."""
    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as fh:
        json.dump(config_to_dict(cfg), fh, indent=1)
    save_file({k: v.to(torch.bfloat16).cpu().contiguous() for k, v in tensors.items()},
              os.path.join(path, "model.safetensors"))


def _preset(width, vocab, pattern, heads, dim, vdim, kv_rank, rot_dim, ff, experts, identity, top, eff) -> dict:
    """pattern: one letter per layer — m = mlstm, a = latent attention; upper case = dense feed-forward, lower = moe."""
    layers = []
    for ch in pattern:
        if ch.lower() == "m":
            mixer, typ = dict(heads=heads, dim=dim, vdim=vdim, gate_cap=10.0), "mlstm"
        else:
            mixer, typ = dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank,
                              scale=(dim + rot_dim) ** -0.5, rot=dict(base=10000.0, dims=rot_dim)), "latent_attention"
        mlp = dict(kind="dense", ff=ff) if ch.isupper() else dict(
            kind="moe", expert=dict(ff=eff), router=dict(experts=experts, identity=identity, top=top))
        layers.append(dict(type=typ, mixer=mixer, mlp=mlp))
    return dict(architecture=ARCHITECTURE, vocab=vocab, width=width, logit_scale=1.0, norm=dict(eps=1e-5),
                layers=layers)


# random-init presets (benchmarks, smoke runs); sizes in the range of real models' layers
PRESETS = {
    "zokunex-tiny": _preset(128, 512, "Mam", 2, 32, 32, 32, 16, 256, 4, 2, 2, 64),
    "zokunex-1b": _preset(2048, 32768, "MamaMamaMamaMama", 8, 128, 256, 256, 64, 8192, 16, 2, 4, 1024),
    "zokunex-8b-layers": _preset(4096, 128256, "MaMa", 16, 128, 256, 512, 64, 14336, 32, 2, 4, 2048),
}


def build(name_or_path: str, device="cpu", seed: int = 0, act_dtype=torch.bfloat16,
          max_position: int | None = None) -> HybridDecoder:
    if os.path.isdir(name_or_path):
        return load(name_or_path, device, act_dtype, max_position)
    cfg = config_from_dict(PRESETS[name_or_path], name=name_or_path, max_position=max_position or 8192)
    w = pack_weights(cfg, random_tensors(cfg, seed), device, act_dtype)
    return HybridDecoder(cfg, w, device, max_position, act_dtype)
