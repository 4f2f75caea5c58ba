"""A plain, slow Zokunex forward: one function per mechanism, written token by token from the design's equations.

It is the oracle the framework's Zokunex path is tested against and shares no code with it.  Everything is computed
in float64 from whatever weights it is given (a dict name -> tensor with the checkpoint's tensor names, and the parsed
config.json dict).  Sequences are processed one token at a time; the caches are plain Python lists.
"""
from __future__ import annotations

import math

import torch

F = torch.float64


def layer_norm(x, w, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def soft_cap(z, cap):
    return cap * torch.tanh(z / cap)


def rotate_half(vec, pos, base, dims):
    """Rotary position on the first ``dims`` entries of the last axis: entry i pairs with i + dims/2."""
    half = dims // 2
    out = vec.clone()
    for i in range(half):
        a = pos * base ** (-2.0 * i / dims)
        u, v = vec[..., i].clone(), vec[..., i + half].clone()
        out[..., i] = u * math.cos(a) - v * math.sin(a)
        out[..., i + half] = v * math.cos(a) + u * math.sin(a)
    return out


def mlstm_token(h, W, p, mx, eps, state):
    """One token of the matrix-memory mixer.  state = [S (heads, dim, vdim), n (heads, dim), m (heads)] or None."""
    H, D, Dv, cap = mx["heads"], mx["dim"], mx["vdim"], mx["gate_cap"]
    if state is None:
        state = [torch.zeros(H, D, Dv, dtype=F), torch.zeros(H, D, dtype=F), torch.zeros(H, dtype=F)]
    S, n, m = state
    q = (W[p + "q"] @ h).view(H, D) * D ** -0.5
    k = (W[p + "k"] @ h).view(H, D)
    v = (W[p + "v"] @ h).view(H, Dv)
    ig = soft_cap(W[p + "i"] @ h + W[p + "i.b"], cap)
    fg = torch.nn.functional.logsigmoid(soft_cap(W[p + "f"] @ h + W[p + "f.b"], cap))
    m_new = torch.maximum(fg + m, ig)
    a = torch.exp(fg + m - m_new)
    b = torch.exp(ig - m_new)
    S = a[:, None, None] * S + b[:, None, None] * (k[:, :, None] * v[:, None, :])
    n = a[:, None] * n + b[:, None] * k
    num = torch.einsum("hdv,hd->hv", S, q)
    den = torch.maximum((n * q).sum(-1).abs(), torch.exp(-m_new)) + 1e-6
    o = num / den[:, None]
    o = rms_unit(o, eps).reshape(-1) * W[p + "norm"]
    o = o * torch.sigmoid(W[p + "g"] @ h)
    return W[p + "o"] @ o, [S, n, m_new]


def latent_attention_token(h, W, p, mx, eps, pos, cache):
    """One token of the latent-attention mixer.  cache: list of (latent c, rotated shared key) of earlier tokens."""
    H, D, R, Dv, rank = mx["heads"], mx["dim"], mx["rot_dim"], mx["vdim"], mx["kv_rank"]
    base, dims = mx["rot"]["base"], mx["rot"]["dims"]
    q = (W[p + "q"] @ h).view(H, D + R)
    qu, qr = q[:, :D], rotate_half(q[:, D:], pos, base, dims)
    dkv = W[p + "dkv"] @ h
    c = rms_unit(dkv[:rank], eps) * W[p + "dkv.norm"]
    kr = rotate_half(dkv[rank:], pos, base, dims)
    cache.append((c, kr))
    scores = []
    vals = []
    for cj, krj in cache:
        ku = (W[p + "uk"] @ cj).view(H, D)
        vals.append((W[p + "uv"] @ cj).view(H, Dv))
        scores.append(((qu * ku).sum(-1) + qr @ krj) * mx["scale"])
    a = torch.softmax(torch.stack(scores, 0), 0)            # [keys, H]
    o = (a[:, :, None] * torch.stack(vals, 0)).sum(0)       # [H, Dv]
    o = o * torch.sigmoid(W[p + "g"] @ h)[:, None]
    return W[p + "o"] @ o.reshape(-1)


def dense_ff(h, W, p):
    return W[p + "down"] @ torch.relu(W[p + "up"] @ h) ** 2


def moe_ff(h, W, p, mlp):
    r = mlp["router"]
    E, I, top = r["experts"], r.get("identity", 0), r["top"]
    s = torch.softmax(W[p + "router"] @ h, -1)
    pick = torch.topk(s + W[p + "correction"], top).indices.tolist()
    out = torch.zeros_like(h)
    for e in pick:
        if e >= E:                                            # the last I router outputs are identity experts
            assert e < E + I
            out = out + s[e] * h
        else:
            z = W[p + f"e{e}.up"] @ h
            out = out + s[e] * (W[p + f"e{e}.down"] @ (0.5 * z * (1 + torch.erf(z / math.sqrt(2)))))
    return out


def forward(cfg, weights, tokens, want=None, layers_out=None):
    """Logits [len(want) or len(tokens), vocab] (float64) of one sequence; ``layers_out``: a list that receives the
    residual stream after every layer, [layers][tokens] -> width."""
    W = {k: v.to(F) for k, v in weights.items()}
    eps = cfg["norm"]["eps"]
    states = [None if l["type"] == "mlstm" else [] for l in cfg["layers"]]
    rows, per_layer = [], [[] for _ in cfg["layers"]]
    for pos, tok in enumerate(tokens):
        x = W["embed"][tok].clone()
        for li, l in enumerate(cfg["layers"]):
            p = f"l{li}.mix."
            if l["type"] == "mlstm":
                y, states[li] = mlstm_token(x, W, p, l["mixer"], eps, states[li])
            elif l["type"] == "latent_attention":
                y = latent_attention_token(x, W, p, l["mixer"], eps, pos, states[li])
            else:
                raise ValueError(l["type"])
            x = x + layer_norm(y, W[f"l{li}.norm1"], eps)
            if l.get("mlp"):
                p = f"l{li}.mlp."
                y = dense_ff(x, W, p) if l["mlp"]["kind"] == "dense" else moe_ff(x, W, p, l["mlp"])
                x = x + layer_norm(y, W[f"l{li}.norm2"], eps)
            per_layer[li].append(x.clone())
        rows.append(W["head"] @ layer_norm(x, W["final.norm"], eps) * cfg["logit_scale"])
    if layers_out is not None:
        layers_out.extend(torch.stack(r) for r in per_layer)
    out = torch.stack(rows)
    return out if want is None else out[list(want)]
