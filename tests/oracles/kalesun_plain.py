"""A plain, slow Kalesun forward: one function per mechanism, written token by token from the design's equations.

It is the oracle the framework's Kalesun path is tested against and shares no code with it.  Everything is computed
in float64 from whatever weights it is given (a dict name -> tensor with the checkpoint's tensor names, and the parsed
config.json dict).  Sequences are processed one token at a time; caches and states are plain Python lists.
"""
from __future__ import annotations

import math

import torch

F = torch.float64


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + torch.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def rope_frequency(i, dims, base, scaling):
    """Frequency of rotated pair i, with the wavelength-dependent slowdown of long wavelengths."""
    f = base ** (-2.0 * i / dims)
    if not scaling:
        return f
    factor, low, high, orig = scaling["factor"], scaling["low"], scaling["high"], scaling["original"]
    wl = 2 * math.pi / f
    if wl < orig / high:
        return f
    if wl > orig / low:
        return f / factor
    s = (orig / wl - low) / (high - low)
    return (1 - s) * f / factor + s * f


def rotate_half(vec, pos, rot):
    """Rotary position on the first rot['dims'] entries of the last axis: entry i pairs with i + dims/2."""
    if not rot:
        return vec
    dims = rot["dims"]
    half = dims // 2
    out = vec.clone()
    for i in range(half):
        a = pos * rope_frequency(i, dims, rot["base"], rot.get("scaling"))
        u, v = vec[..., i].clone(), vec[..., i + half].clone()
        out[..., i] = u * math.cos(a) - v * math.sin(a)
        out[..., i + half] = v * math.cos(a) + u * math.sin(a)
    return out


def visible(i, j, mask):
    """May the query at position i see the key at position j?"""
    if j > i:
        return False
    if not mask:
        return True
    return i - j < mask["size"] or j < mask.get("keep_first", 0)


def attention_token(h, W, p, mx, eps, pos, cache, v_first, is_first_vmix):
    """One token of the windowed attention mixer.  cache: list of (k [G, D], v [G, Dv]) of the earlier tokens, this
    token's pair is appended.  v_first: this token's values in the first value-mixing layer (None in that layer and
    in layers that do not mix).  Returns (output, this token's unmixed-or-mixed cached v)."""
    H, G, D, Dv = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
    q = (W[p + "q"] @ h).view(H, D)
    k = (W[p + "k"] @ h).view(G, D)
    v = (W[p + "v"] @ h).view(G, Dv)
    q = rms_unit(q, eps) * W[p + "q.norm"]
    k = rms_unit(k, eps) * W[p + "k.norm"]
    q = rotate_half(q, pos, mx.get("rot"))
    k = rotate_half(k, pos, mx.get("rot"))
    if mx.get("v_mix") and not is_first_vmix:
        lam = W[p + "vmix"]
        v = (1 - lam) * v + lam * v_first
    cache.append((k, v))
    gate = sigmoid(W[p + "g"] @ h)
    out = torch.zeros(H, Dv, dtype=F)
    for hh in range(H):
        g = hh // (H // G)
        js = [j for j in range(pos + 1) if visible(pos, j, mx.get("mask"))]
        sc = torch.stack([(q[hh] * cache[j][0][g]).sum() * mx["scale"] for j in js])
        sink = W[p + "sink"][hh]
        m = torch.maximum(sc.max(), sink)
        e = torch.exp(sc - m)
        den = e.sum() + torch.exp(sink - m)
        for w_, j in zip(e / den, js):
            out[hh] += w_ * cache[j][1][g]
        out[hh] *= gate[hh]
    return W[p + "o"] @ out.reshape(-1), v


def short_conv_token(x, taps_w, hist):
    """Causal per-channel convolution: hist holds the last taps-1 inputs (oldest first, zeros before the start);
    the last column of taps_w weighs the current input.  Returns (output, new history)."""
    K = taps_w.shape[1]
    window = hist + [x]
    y = sum(taps_w[:, i] * window[i] for i in range(K))
    return y, window[1:] if K > 1 else []


def delta_token(h, W, p, mx, eps, state):
    """One token of the gated delta rule.  state = dict(S [heads, dim, vdim], q/k/v convolution histories)."""
    H, G, D, Dv, K = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"], mx["conv"]
    if not state:
        state.update(S=torch.zeros(H, D, Dv, dtype=F),
                     q=[torch.zeros(G * D, dtype=F)] * (K - 1), k=[torch.zeros(G * D, dtype=F)] * (K - 1),
                     v=[torch.zeros(H * Dv, dtype=F)] * (K - 1))
    q, state["q"] = short_conv_token(W[p + "q"] @ h, W[p + "q.conv"], state["q"])
    k, state["k"] = short_conv_token(W[p + "k"] @ h, W[p + "k.conv"], state["k"])
    v, state["v"] = short_conv_token(W[p + "v"] @ h, W[p + "v.conv"], state["v"])
    q, k, v = silu(q).view(G, D), silu(k).view(G, D), silu(v).view(H, Dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = sigmoid(W[p + "b"] @ h)
    decay = torch.exp(-torch.exp(W[p + "A_log"]) * softplus(W[p + "a"] @ h + W[p + "dt_bias"]))
    gate = silu(W[p + "g"] @ h).view(H, Dv)
    S = state["S"]
    out = torch.zeros(H, Dv, dtype=F)
    for hh in range(H):
        g = hh // (H // G)
        Sh = decay[hh] * S[hh]
        u = beta[hh] * (v[hh] - Sh.t() @ k[g])
        Sh = Sh + torch.outer(k[g], u)
        S[hh] = Sh
        out[hh] = rms_unit(Sh.t() @ q[g], eps) * W[p + "norm"] * gate[hh]
    return W[p + "o"] @ out.reshape(-1)


def gla_token(h, W, p, mx, eps, state):
    """One token of gated linear attention with a decay per key channel.  state = dict(S [heads, dim, vdim])."""
    H, D, Dv = mx["heads"], mx["dim"], mx["vdim"]
    if not state:
        state.update(S=torch.zeros(H, D, Dv, dtype=F))
    q = (W[p + "q"] @ h).view(H, D) * D ** -0.5
    k = (W[p + "k"] @ h).view(H, D)
    v = (W[p + "v"] @ h).view(H, Dv)
    z = W[p + "a2"] @ (W[p + "a1"] @ h) + W[p + "a2.b"]
    alpha = (sigmoid(z) ** (1.0 / mx["tau"])).view(H, D)
    gate = silu(W[p + "g"] @ h).view(H, Dv)
    S = state["S"]
    out = torch.zeros(H, Dv, dtype=F)
    for hh in range(H):
        S[hh] = alpha[hh][:, None] * S[hh] + torch.outer(k[hh], v[hh])
        out[hh] = rms_unit(S[hh].t() @ q[hh], eps) * W[p + "norm"] * gate[hh]
    return W[p + "o"] @ out.reshape(-1)


def glu_clamped(h, w_gate, w_up, w_down, limit):
    g = torch.clamp(w_gate @ h, max=limit)
    u = torch.clamp(w_up @ h, -limit, limit)
    return w_down @ (g * sigmoid(1.702 * g) * (u + 1))


def dense_ff(h, W, p, mlp):
    return glu_clamped(h, W[p + "gate"], W[p + "up"], W[p + "down"], mlp["limit"])


def moe_ff(h, W, p, mlp):
    """Returns (output, chosen experts, margin between the last chosen and the first rejected logit)."""
    r = mlp["router"]
    z = W[p + "router"] @ h + W[p + "router.b"]
    order = sorted(range(r["experts"]), key=lambda e: (-float(z[e]), e))
    chosen = order[:r["top"]]
    margin = float(z[order[r["top"] - 1]] - z[order[r["top"]]]) if r["top"] < r["experts"] else float("inf")
    wts = torch.softmax(torch.stack([z[e] for e in chosen]), 0)
    out = torch.zeros_like(h)
    for w_, e in zip(wts, chosen):
        out = out + w_ * glu_clamped(h, W[p + f"e{e}.gate"], W[p + f"e{e}.up"], W[p + f"e{e}.down"],
                                     mlp["expert"]["limit"])
    return out, chosen, margin


class Plain:
    """The whole model for one sequence: ``step(token)`` returns the logits of the next token and records the residual
    stream after every layer in ``self.layers`` (list over tokens of [layers, width])."""

    def __init__(self, config: dict, tensors: dict):
        self.c = config
        self.W = {k: v.to(F) for k, v in tensors.items()}
        self.pos = 0
        self.state = [dict() for _ in config["layers"]]
        self.kv = [[] for _ in config["layers"]]
        self.layers = []
        self.min_margin = float("inf")
        vm = [i for i, l in enumerate(config["layers"]) if l["type"] == "attention" and l["mixer"].get("v_mix")]
        self.first_vmix = vm[0] if vm else None

    def step(self, token: int) -> torch.Tensor:
        c, W = self.c, self.W
        eps, alpha = c["norm"]["eps"], c["postln_alpha"]
        x = W["embed"][token].clone()
        taps = []
        v_first = None
        for i, l in enumerate(c["layers"]):
            p, mx = f"l{i}.mix.", l["mixer"]
            if l["type"] == "attention":
                y, v = attention_token(x, W, p, mx, eps, self.pos, self.kv[i], v_first, i == self.first_vmix)
                if i == self.first_vmix:
                    v_first = v
            elif l["type"] == "delta":
                y = delta_token(x, W, p, mx, eps, self.state[i])
            elif l["type"] == "gla":
                y = gla_token(x, W, p, mx, eps, self.state[i])
            else:
                raise ValueError(l["type"])
            x = rms_unit(alpha * x + y, eps) * W[f"l{i}.norm1"]
            mlp = l.get("mlp")
            if mlp is not None:
                if mlp["kind"] == "dense":
                    y = dense_ff(x, W, f"l{i}.mlp.", mlp)
                else:
                    y, _, margin = moe_ff(x, W, f"l{i}.mlp.", mlp)
                    self.min_margin = min(self.min_margin, margin)
                x = rms_unit(alpha * x + y, eps) * W[f"l{i}.norm2"]
            taps.append(x.clone())
        self.layers.append(torch.stack(taps))
        self.pos += 1
        return W["embed"] @ (rms_unit(x, eps) * W["final.norm"])


def run(config: dict, tensors: dict, tokens) -> tuple:
    """(logits [T, vocab], residual stream [layers, T, width]) of one sequence."""
    m = Plain(config, tensors)
    logits = torch.stack([m.step(int(t)) for t in tokens])
    return logits, torch.stack(m.layers, 1)
