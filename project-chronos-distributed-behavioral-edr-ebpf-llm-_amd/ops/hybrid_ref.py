"""PyTorch references of the hybrid-decoder kernels (csrc/kernels/hybrid*.hip): the CPU execution path and the
numerics oracle of the GPU tests.  Same interfaces as the kernels (layouts, in-place arguments); everything the
kernels keep in 32-bit floats is computed in float32 here too, whatever the activation dtype.

Activation dtype ``AT`` is bfloat16 or float32; the residual stream is always float32.
"""
from __future__ import annotations

import math

import torch

ACT_RELU2, ACT_GELU = 0, 1


def embed_rows(ids, table, act_dtype):
    x = table[ids.long()].float()
    return x, (x if act_dtype == torch.float32 else x.to(act_dtype))


def layer_norm(x, w, eps, act_dtype):
    xf = x.float()
    mu = xf.mean(-1, keepdim=True)
    d = xf - mu
    y = d * torch.rsqrt(d.pow(2).mean(-1, keepdim=True) + eps) * w.float()
    return y.to(act_dtype)


def add_layer_norm(y, x, w, eps, act_dtype):
    """x (float32, in place) <- x + layer_norm(y) * w; returns x in the activation dtype (x itself for float32)."""
    x.add_(layer_norm(y, w, eps, torch.float32))
    return x if act_dtype == torch.float32 else x.to(act_dtype)


def rowdot(h, w, bias=None):
    """float32 [T, N] = h @ w.T (+ bias) with float32 accumulation: the few-row projections whose outputs feed
    32-bit math (recurrence gates, router logits, head gates)."""
    z = h.float() @ w.float().t()
    return z if bias is None else z + bias.float()


def act_inplace(x, kind):
    xf = x.float()
    if kind == ACT_RELU2:
        r = torch.relu(xf) ** 2
    else:
        r = 0.5 * xf * (1.0 + torch.erf(xf * (1.0 / math.sqrt(2.0))))
    x.copy_(r.to(x.dtype))
    return x


def mlstm_scan(proj, gate_pre, q_start, pos0, slots, S, n, m, H, D, Dv, cap):
    """Stabilised matrix-memory recurrence over a flattened token stream.

    proj [T, >= 2 H D + H Dv]: per token q (H x D), k (H x D), v (H x Dv) side by side; gate_pre f32 [T, 2 H]: the
    input- and forget-gate pre-activations; q_start [B + 1]: token range of each sequence; pos0 [B]: position of the
    range's first token (0: the state starts at zero, with the running maximum at 0); slots [B]: row of the state
    tensors S [NS, H, D, Dv], n [NS, H, D], m [NS, H] (float32, updated in place).  Returns the normalised read-out
    f32 [T, H, Dv]."""
    T = proj.shape[0]
    out = torch.zeros(T, H, Dv, dtype=torch.float32, device=proj.device)
    qs = q_start.tolist()
    p0 = pos0.tolist()
    sl = slots.tolist()
    pf = proj.float()
    ig_all = cap * torch.tanh(gate_pre[:, :H].float() / cap)
    fg_all = torch.nn.functional.logsigmoid(cap * torch.tanh(gate_pre[:, H:2 * H].float() / cap))
    for b in range(len(sl)):
        s = sl[b]
        if p0[b] == 0:
            Sb = torch.zeros_like(S[s])
            nb = torch.zeros_like(n[s])
            mb = torch.zeros_like(m[s])
        else:
            Sb, nb, mb = S[s].clone(), n[s].clone(), m[s].clone()
        for t in range(qs[b], qs[b + 1]):
            q = pf[t, :H * D].view(H, D) * D ** -0.5
            k = pf[t, H * D:2 * H * D].view(H, D)
            v = pf[t, 2 * H * D:2 * H * D + H * Dv].view(H, Dv)
            ig, fg = ig_all[t], fg_all[t]
            mn = torch.maximum(fg + mb, ig)
            a, bb = torch.exp(fg + mb - mn), torch.exp(ig - mn)
            Sb = a[:, None, None] * Sb + bb[:, None, None] * (k[:, :, None] * v[:, None, :])
            nb = a[:, None] * nb + bb[:, None] * k
            mb = mn
            den = torch.maximum((nb * q).sum(-1).abs(), torch.exp(-mb)) + 1e-6
            out[t] = torch.einsum("hdv,hd->hv", Sb, q) / den[:, None]
        if qs[b + 1] > qs[b]:
            S[s], n[s], m[s] = Sb, nb, mb
    return out


def mlstm_out(o, proj, g_off, norm_w, eps, act_dtype):
    """Per-head unit RMS of the read-out, times the head-concatenated weight, times sigmoid of the gate columns
    proj[:, g_off : g_off + H Dv]."""
    T, H, Dv = o.shape
    y = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps)
    y = y.reshape(T, H * Dv) * norm_w.float() * torch.sigmoid(proj[:, g_off:g_off + H * Dv].float())
    return y.to(act_dtype)


def rotate_half_rows(x, cos_sin, pos, dims):
    """Rotary position on the first ``dims`` entries of the last axis (entry i pairs with i + dims/2); cos_sin
    [P, dims]: cos | sin of position x frequency, float32."""
    half = dims // 2
    cs = cos_sin[pos.long()]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    c, s = cs[:, :half].view(shape), cs[:, half:].view(shape)
    u, v = x[..., :half].float(), x[..., half:dims].float()
    out = x.float().clone()
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


def latent_prep(q, dkv, pos, tok_seq, block_table, w_norm, eps, cos_sin, dims, rank, cache):
    """Latent-attention cache write and query rotation.  dkv [T, rank + R]: the first rank columns are RMS-normed
    (times w_norm) into the latent, the last R rotated; both are written to cache [NB, BS, rank + R] at the token's
    page and slot.  q [T, H, D + R]: the last R columns of every head are rotated in place."""
    T = q.shape[0]
    R = dkv.shape[1] - rank
    D = q.shape[2] - R
    c = dkv[:, :rank].float()
    c = c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + eps) * w_norm.float()
    kr = rotate_half_rows(dkv[:, rank:], cos_sin, pos, dims)
    row = torch.cat([c, kr], 1).to(cache.dtype)
    bs = cache.shape[1]
    blk = block_table[tok_seq.long(), (pos // bs).long()].long()
    cache[blk, (pos % bs).long()] = row
    q[:, :, D:] = rotate_half_rows(q[:, :, D:], cos_sin, pos, dims).to(q.dtype)


def latent_attention(qa, cache, block_table, q_start, pos, gate, scale, rank, act_dtype):
    """Causal softmax attention of H query heads over ONE shared key row per token: key = the cached row (rank + R
    columns), value = its first rank columns.  qa [T, H, rank + R]; token t of sequence b sits at pos[t] and sees the
    cached rows 0..pos[t] of its sequence; gate f32 [T, H] or None: the output of head h is multiplied by
    sigmoid(gate).  Returns [T, H, rank]."""
    T, H, DK = qa.shape
    out = torch.zeros(T, H, rank, dtype=torch.float32, device=qa.device)
    bs = cache.shape[1]
    qs = q_start.tolist()
    for b in range(len(qs) - 1):
        t0, t1 = qs[b], qs[b + 1]
        if t1 <= t0:
            continue
        p = pos[t0:t1].long()
        ctx = int(p.max()) + 1
        nblk = (ctx + bs - 1) // bs
        keys = cache[block_table[b, :nblk].long()].reshape(nblk * bs, DK)[:ctx].float()
        sc = torch.einsum("thk,jk->thj", qa[t0:t1].float(), keys) * scale
        mask = torch.arange(ctx, device=qa.device)[None, :] > p[:, None]
        sc = sc.masked_fill(mask[:, None, :], float("-inf"))
        a = torch.softmax(sc, -1)
        out[t0:t1] = torch.einsum("thj,jr->thr", a, keys[:, :rank])
    if gate is not None:
        out = out * torch.sigmoid(gate.float())[:, :, None]
    return out.to(act_dtype)


def moe_route(h, w_router, correction, top):
    """Router of a mixture of experts: float32 logits, softmax over all outputs, the ``top`` largest of
    score + correction are chosen (ties: the lower index), weighted by their plain scores (not renormalised).
    Returns (idx int32 [T, top], weight f32 [T, top])."""
    s = torch.softmax(rowdot(h, w_router), -1)
    choice = s + correction.float()
    idx = torch.topk(choice, top, dim=-1).indices
    return idx.to(torch.int32), torch.gather(s, 1, idx)


def moe_ffn(h, idx, wt, w_up, w_down, act, act_dtype):
    """Weighted sum of each token's chosen experts.  w_up [E, F, d], w_down [E, d, F]; an index >= E is an identity
    expert (its output is the token itself)."""
    E = w_up.shape[0]
    hf = h.float()
    out = torch.zeros_like(hf)
    idl = idx.long()
    for e in range(E):
        tok, kk = torch.nonzero(idl == e, as_tuple=True)
        if tok.numel() == 0:
            continue
        z = (hf[tok].to(act_dtype) @ w_up[e].t().to(act_dtype))
        z = act_inplace(z, act)
        y = (z @ w_down[e].t().to(act_dtype)).float()
        out.index_add_(0, tok, y * wt[tok, kk][:, None])
    ident = (idl >= E).float() * wt
    out = out + ident.sum(-1, keepdim=True) * hf
    return out.to(act_dtype)
