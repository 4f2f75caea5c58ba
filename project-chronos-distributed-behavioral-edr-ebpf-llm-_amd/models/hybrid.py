"""Hybrid decoders: a list of layers, each with a token mixer of some kind (recurrent matrix memory, latent
attention) and an optional feed-forward (dense, mixture of experts), on a float32 residual stream with the norm on the
sublayer's OUTPUT (x <- x + norm(sublayer(x))).

This module is the design-independent part: the mixer and feed-forward kinds with their sizes and constants as
parameters, the cache that holds pages for the attention layers and state slots for the recurrent ones, and the
forward over the engine's flattened step batch (:class:`chronos.models.llama.StepBatch`: prefill chunks, decode rows
or both in one step).  A design (``zokunex.py``) reads its configuration file and tensor names into these.

New mixer / feed-forward kinds register in ``MIXERS`` / ``FEED_FORWARDS``.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional

import torch

from ..ops import hybrid as hops
from ..parallel.tp import TPContext
from .llama import StepBatch, h2d


# -----------------------------------------------------------------------------------------------------------------
# configuration
# -----------------------------------------------------------------------------------------------------------------


@dataclass
class MLSTMSpec:
    """Matrix-memory recurrent mixer: per head a D x Dv state, exponential input gate and sigmoid forget gate in
    log space, both soft-capped (cap * tanh(z / cap)) and stabilised by a running maximum."""
    heads: int
    dim: int
    vdim: int
    gate_cap: float
    kind: str = "mlstm"


@dataclass
class LatentAttentionSpec:
    """Attention whose keys and values are up-projections of one cached low-rank latent per token, plus a rotated key
    part shared by all heads; sigmoid output gate per head."""
    heads: int
    dim: int        # unrotated query / key columns per head
    rot_dim: int    # rotated columns per head (the shared rotated key has as many)
    vdim: int
    kv_rank: int
    scale: float
    rope_base: float
    rope_dims: int  # leading columns of the rotated part that are actually rotated
    kind: str = "latent_attention"


@dataclass
class DenseFFSpec:
    ff: int
    act: int = hops.ACT_RELU2
    kind: str = "dense"


@dataclass
class MoEFFSpec:
    experts: int     # experts with weights
    identity: int    # further router outputs whose expert returns its input
    top: int
    ff: int
    act: int = hops.ACT_GELU
    kind: str = "moe"


@dataclass
class LayerSpec:
    mixer: object
    ff: Optional[object]


@dataclass
class HybridConfig:
    name: str
    vocab_size: int
    hidden_size: int
    layers: list
    norm_eps: float
    logit_scale: float = 1.0
    max_position: int = 8192
    architecture: str = "hybrid"

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    def param_count(self) -> int:
        d, n = self.hidden_size, 2 * self.vocab_size * self.hidden_size + self.hidden_size
        for l in self.layers:
            m = l.mixer
            if m.kind == "mlstm":
                n += d * (2 * m.heads * m.dim + 2 * m.heads * m.vdim) + 2 * m.heads * (d + 1) + m.heads * m.vdim * (d + 1)
            else:
                n += d * (m.heads * (m.dim + m.rot_dim) + m.kv_rank + m.rot_dim + m.heads) + m.kv_rank
                n += m.kv_rank * m.heads * (m.dim + m.vdim) + m.heads * m.vdim * d
            n += d
            if l.ff is not None:
                n += d + (2 * d * l.ff.ff if l.ff.kind == "dense" else
                          l.ff.experts * 2 * d * l.ff.ff + (l.ff.experts + l.ff.identity) * (d + 1))
        return n


# -----------------------------------------------------------------------------------------------------------------
# cache: pages for the attention layers, state slots for the recurrent layers
# -----------------------------------------------------------------------------------------------------------------


class HybridCache:
    """Per attention layer a paged latent cache [NB, BS, kv_rank + rot_dim] in the activation dtype (block 0 is the
    engine's scratch block); per recurrent layer float32 state rows S [NS, H, D, Dv], n [NS, H, D], m [NS, H], one row
    per engine slot plus a scratch row (``scratch_slot``) for the decode rows of slots that hold no running sequence.

    A sequence's state needs no reset: a step whose first token sits at position 0 starts from zero."""

    def __init__(self, cfg: HybridConfig, num_blocks: int, block_size: int, device, act_dtype, slots: int):
        self.num_blocks, self.block_size = num_blocks, block_size
        self.slots = slots
        self.scratch_slot = slots
        self.lat: dict[int, torch.Tensor] = {}
        self.S: dict[int, torch.Tensor] = {}
        self.n: dict[int, torch.Tensor] = {}
        self.m: dict[int, torch.Tensor] = {}
        for li, l in enumerate(cfg.layers):
            mx = l.mixer
            if mx.kind == "latent_attention":
                self.lat[li] = torch.zeros(num_blocks, block_size, mx.kv_rank + mx.rot_dim, device=device,
                                           dtype=act_dtype)
            elif mx.kind == "mlstm":
                f32 = dict(device=device, dtype=torch.float32)
                self.S[li] = torch.zeros(slots + 1, mx.heads, mx.dim, mx.vdim, **f32)
                self.n[li] = torch.zeros(slots + 1, mx.heads, mx.dim, **f32)
                self.m[li] = torch.zeros(slots + 1, mx.heads, **f32)

    @staticmethod
    def bytes_per_block(cfg: HybridConfig, block_size: int, act_dtype) -> int:
        eb = 4 if act_dtype == torch.float32 else 2
        return max(1, sum(block_size * (l.mixer.kv_rank + l.mixer.rot_dim) * eb for l in cfg.layers
                          if l.mixer.kind == "latent_attention"))

    def move_slots(self, src: torch.Tensor, dst: torch.Tensor) -> None:
        """Slot compaction: the recurrent state rows follow their sequences."""
        for t in (*self.S.values(), *self.n.values(), *self.m.values()):
            t.index_copy_(0, dst, t.index_select(0, src))


# -----------------------------------------------------------------------------------------------------------------
# weights
# -----------------------------------------------------------------------------------------------------------------


@dataclass
class HybridLayerWeights:
    norm1: torch.Tensor
    mix: dict
    norm2: Optional[torch.Tensor] = None
    ff: dict = field(default_factory=dict)


@dataclass
class HybridWeights:
    embed: torch.Tensor
    layers: list
    final_norm: torch.Tensor
    head: torch.Tensor

    def nbytes(self) -> int:
        n = 0
        for t in (self.embed, self.final_norm, self.head):
            n += t.numel() * t.element_size()
        for l in self.layers:
            for t in (l.norm1, l.norm2, *l.mix.values(), *l.ff.values()):
                if isinstance(t, torch.Tensor):
                    n += t.numel() * t.element_size()
        return n


def pack_mlstm(spec: MLSTMSpec, t: dict, device, act_dtype) -> dict:
    """t: q, k, v, g, o, norm, i, i.b, f, f.b (checkpoint layout, [out, in]).  q | k | v | g become one projection,
    the two gate rows one few-row float32-output projection."""
    a = lambda x: x.to(device=device, dtype=act_dtype).contiguous()  # noqa: E731
    f = lambda x: x.to(device=device, dtype=torch.float32).contiguous()  # noqa: E731
    return dict(w_proj=a(torch.cat([t["q"], t["k"], t["v"], t["g"]], 0)), w_if=a(torch.cat([t["i"], t["f"]], 0)),
                b_if=f(torch.cat([t["i.b"], t["f.b"]], 0)), norm=f(t["norm"]), w_o=a(t["o"]))


def pack_latent(spec: LatentAttentionSpec, t: dict, device, act_dtype) -> dict:
    """t: q, dkv, dkv.norm, uk, uv, g, o.  The per-head up-projections are kept as [H, D, rank] and [H, Dv, rank]:
    keys are never materialised (the query is carried into the latent space instead) and the value up-projection
    is applied to the attention's latent-space output."""
    a = lambda x: x.to(device=device, dtype=act_dtype).contiguous()  # noqa: E731
    f = lambda x: x.to(device=device, dtype=torch.float32).contiguous()  # noqa: E731
    return dict(w_q=a(t["q"]), w_dkv=a(t["dkv"]), dkv_norm=f(t["dkv.norm"]), w_g=a(t["g"]), w_o=a(t["o"]),
                w_uk=a(t["uk"].view(spec.heads, spec.dim, spec.kv_rank)),
                w_uv=a(t["uv"].view(spec.heads, spec.vdim, spec.kv_rank)))


def pack_dense(spec: DenseFFSpec, t: dict, device, act_dtype) -> dict:
    a = lambda x: x.to(device=device, dtype=act_dtype).contiguous()  # noqa: E731
    return dict(w_up=a(t["up"]), w_down=a(t["down"]))


def pack_moe(spec: MoEFFSpec, t: dict, device, act_dtype) -> dict:
    """t: router, correction, e<k>.up, e<k>.down.  Expert weights are stacked [E, ...] for the grouped kernels."""
    a = lambda x: x.to(device=device, dtype=act_dtype).contiguous()  # noqa: E731
    return dict(w_router=a(t["router"]), correction=t["correction"].to(device=device, dtype=torch.float32).contiguous(),
                w_up=a(torch.stack([t[f"e{e}.up"] for e in range(spec.experts)])),
                w_down=a(torch.stack([t[f"e{e}.down"] for e in range(spec.experts)])))


def rope_cos_sin(base: float, dims: int, max_pos: int, device) -> torch.Tensor:
    """[max_pos, dims] float32: cos(p f_i) for i < dims/2, then sin(p f_i), f_i = base^(-2i/dims); angles in float64
    before the rounding to float32."""
    inv = base ** (-torch.arange(0, dims, 2, dtype=torch.float64) / dims)
    fr = torch.outer(torch.arange(max_pos, dtype=torch.float64), inv)
    return torch.cat([fr.cos(), fr.sin()], 1).float().to(device)


# -----------------------------------------------------------------------------------------------------------------
# mixers and feed-forwards (one function per kind: h [T, d] in the activation dtype -> [T, d])
# -----------------------------------------------------------------------------------------------------------------


@dataclass
class StepMeta:
    """One step's flattened token stream, prefill chunks and decode rows alike: sequence b owns tokens
    q_start[b]:q_start[b+1], the first of them at position pos0[b], its pages in block_table[b], its state in row
    slots[b] of the recurrent-state tensors."""
    ids: torch.Tensor
    pos: torch.Tensor
    tok_seq: torch.Tensor
    block_table: torch.Tensor
    q_start: torch.Tensor
    pos0: torch.Tensor
    slots: torch.Tensor
    last_idx: torch.Tensor
    max_q: int


def mix_mlstm(model, li: int, spec: MLSTMSpec, w: dict, h, meta: StepMeta, cache: HybridCache):
    H, D, Dv = spec.heads, spec.dim, spec.vdim
    proj = hops.matmul(h, w["w_proj"])
    gate_pre = hops.rowdot(h, w["w_if"], w["b_if"])
    o = hops.mlstm_scan(proj, gate_pre, meta.q_start, meta.pos0, meta.slots, cache.S[li], cache.n[li], cache.m[li],
                        H, D, Dv, spec.gate_cap, meta.max_q)
    y = hops.mlstm_out(o, proj, 2 * H * D + H * Dv, w["norm"], model.cfg.norm_eps, model.act_dtype)
    return hops.matmul(y, w["w_o"])


def mix_latent_attention(model, li: int, spec: LatentAttentionSpec, w: dict, h, meta: StepMeta, cache: HybridCache):
    T = h.shape[0]
    H, D, R, rank = spec.heads, spec.dim, spec.rot_dim, spec.kv_rank
    q = hops.matmul(h, w["w_q"]).view(T, H, D + R)
    dkv = hops.matmul(h, w["w_dkv"])
    gate = hops.rowdot(h, w["w_g"])
    hops.latent_prep(q, dkv, meta.pos, meta.tok_seq, meta.block_table, w["dkv_norm"], model.cfg.norm_eps,
                     model.rope[li], spec.rope_dims, rank, cache.lat[li])
    # the query goes into the latent space (q_u W_uk per head), so a key is the cached row itself; the output
    # comes back through W_uv per head
    qa = torch.empty(T, H, rank + R, device=h.device, dtype=h.dtype)
    qa[:, :, :rank] = torch.bmm(q[:, :, :D].transpose(0, 1), w["w_uk"]).transpose(0, 1)
    qa[:, :, rank:] = q[:, :, D:]
    oa = hops.latent_attention(qa, cache.lat[li], meta.block_table, meta.q_start, meta.pos, gate, spec.scale, rank,
                               model.act_dtype, meta.max_q)
    ov = torch.bmm(oa.transpose(0, 1), w["w_uv"].transpose(1, 2)).transpose(0, 1).reshape(T, H * spec.vdim)
    return hops.matmul(ov, w["w_o"])


def ff_dense(model, spec: DenseFFSpec, w: dict, h):
    return hops.matmul(hops.act_inplace(hops.matmul(h, w["w_up"]), spec.act), w["w_down"])


def ff_moe(model, spec: MoEFFSpec, w: dict, h):
    idx, wt = hops.moe_route(h, w["w_router"], w["correction"], spec.top)
    return hops.moe_ffn(h, idx, wt, w["w_up"], w["w_down"], spec.act, model.act_dtype)


MIXERS = {"mlstm": (mix_mlstm, pack_mlstm), "latent_attention": (mix_latent_attention, pack_latent)}
FEED_FORWARDS = {"dense": (ff_dense, pack_dense), "moe": (ff_moe, pack_moe)}


# -----------------------------------------------------------------------------------------------------------------
# model
# -----------------------------------------------------------------------------------------------------------------


class HybridDecoder:
    """Serves through the same engine as the Llama models (same step batches, block manager, sampler).  What the
    engine needs from a model: ``cfg.vocab_size``, ``make_cache``, ``cache_bytes_per_block``, ``prefill_batch``,
    ``forward``, ``recurrent`` (state slots: no prefix sharing between sequences) and ``hq`` / ``hkv`` for its
    decode-split heuristics."""
    recurrent = True
    hq = hkv = 1

    def __init__(self, cfg: HybridConfig, weights: HybridWeights, device="cpu", max_position: int | None = None,
                 act_dtype=torch.bfloat16, tp: TPContext | None = None):
        self.cfg, self.w = cfg, weights
        self.tp = tp or TPContext.single()
        if self.tp.world > 1:
            raise NotImplementedError("the hybrid decoders run on full-weight ranks (data-parallel replicas only)")
        self.device = torch.device(device)
        self.act_dtype = act_dtype
        self.sequence_parallel = False
        self.decode_overlap_rows = 0
        P = max_position or cfg.max_position
        self.rope = {li: rope_cos_sin(l.mixer.rope_base, l.mixer.rope_dims, P, self.device)
                     for li, l in enumerate(cfg.layers) if l.mixer.kind == "latent_attention"}
        self.recurrent = any(l.mixer.kind == "mlstm" for l in cfg.layers)

    # ---- what the engine calls --------------------------------------------------------------------------------
    def make_cache(self, num_blocks: int, block_size: int, slots: int, kv_dtype: str = "bf16", k_scale: float = 1.0,
                   v_scale: float = 1.0) -> HybridCache:
        if kv_dtype != "bf16":
            raise ValueError("the hybrid decoders cache in their activation dtype (kv_dtype must stay 'bf16')")
        return HybridCache(self.cfg, num_blocks, block_size, self.device, self.act_dtype, slots)

    def cache_bytes_per_block(self, block_size: int, kv_dtype: str = "bf16") -> int:
        return HybridCache.bytes_per_block(self.cfg, block_size, self.act_dtype)

    def prefill_batch(self, chunks, starts, block_tables, slots, max_blocks=None, nqt: int = 2, split: int = 1,
                      want=None) -> StepBatch:
        """Host builder of a prefill step: chunks[b] are sequence b's next tokens, the first at position starts[b];
        slots[b] its state slot.  ``want``: token indices (into the flattened stream) whose logits are asked for
        (default: every sequence's last token)."""
        ids, pos, tok_seq, qs = [], [], [], [0]
        for b, (toks, s0) in enumerate(zip(chunks, starts)):
            ids += toks
            pos += list(range(s0, s0 + len(toks)))
            tok_seq += [b] * len(toks)
            qs.append(qs[-1] + len(toks))
        mb = max_blocks or max(len(x) for x in block_tables)
        bt = torch.zeros(len(chunks), mb, dtype=torch.int32)
        for b, blks in enumerate(block_tables):
            bt[b, :len(blks)] = torch.tensor(blks, dtype=torch.int32)
        it = lambda x: torch.tensor(x, dtype=torch.int32)  # noqa: E731
        last = torch.tensor([q - 1 for q in qs[1:]] if want is None else list(want), dtype=torch.int64)
        dv = lambda t: h2d(t, self.device)  # noqa: E731
        mq = max((len(c) for c in chunks), default=0)
        return StepBatch(dv(it(ids)), dv(it(pos)), dv(it(tok_seq)), dv(bt), dv(it(qs)),
                         dv(it([s0 + len(t) for t, s0 in zip(chunks, starts)])), dv(last),
                         dv(torch.zeros(max(1, len(chunks)), 2, dtype=torch.int32)), len(chunks), nqt, 1,
                         slots=dv(it(list(slots))), max_q=mq)

    def _meta(self, sb: StepBatch) -> StepMeta:
        def one(p: StepBatch) -> StepMeta:
            if p.slots is None:
                raise ValueError("a hybrid decoder's step batch needs the sequences' state slots")
            if p.tiles is None:  # decode rows: token i is sequence i
                return StepMeta(p.ids, p.pos, p.tok_seq, p.block_table, p.q_start, p.pos, p.slots, p.last_idx, 1)
            pos0 = p.pos.index_select(0, p.q_start[:-1].long().clamp(max=max(0, p.pos.numel() - 1)))
            return StepMeta(p.ids, p.pos, p.tok_seq, p.block_table, p.q_start, pos0, p.slots, p.last_idx,
                            p.max_q or p.ids.numel())

        m = one(sb)
        if sb.dec is None:
            return m
        d = one(sb.dec)
        T, B = m.ids.numel(), m.block_table.shape[0]
        return StepMeta(torch.cat([m.ids, d.ids]), torch.cat([m.pos, d.pos]), torch.cat([m.tok_seq, d.tok_seq + B]),
                        torch.cat([m.block_table, d.block_table]), torch.cat([m.q_start, d.q_start[1:] + T]),
                        torch.cat([m.pos0, d.pos0]), torch.cat([m.slots, d.slots]), sb.last_idx, max(m.max_q, 1))

    def forward(self, sb: StepBatch, cache: HybridCache, logits_dtype=torch.float32) -> torch.Tensor:
        """Logits [len(sb.last_idx), V] of the tokens at sb.last_idx (with ``sb.dec``: indices into prefill tokens
        followed by decode rows)."""
        cfg, w, at = self.cfg, self.w, self.act_dtype
        meta = self._meta(sb)
        x, h = hops.embed_rows(meta.ids, w.embed, at)
        for li, (spec, lw) in enumerate(zip(cfg.layers, w.layers)):
            y = MIXERS[spec.mixer.kind][0](self, li, spec.mixer, lw.mix, h, meta, cache)
            h = hops.add_layer_norm(y, x, lw.norm1, cfg.norm_eps, at)
            if spec.ff is not None:
                y = FEED_FORWARDS[spec.ff.kind][0](self, spec.ff, lw.ff, h)
                h = hops.add_layer_norm(y, x, lw.norm2, cfg.norm_eps, at)
            if self.layer_tap is not None:
                self.layer_tap(li, x)
        xs = x.index_select(0, meta.last_idx)
        logits = hops.matmul(hops.layer_norm(xs, w.final_norm, cfg.norm_eps, at), w.head).float()
        if cfg.logit_scale != 1.0:
            logits = logits * cfg.logit_scale
        return logits if logits.dtype == logits_dtype else logits.to(logits_dtype)

    layer_tap = None  # debugging hook: called with (layer index, residual stream) after every layer
