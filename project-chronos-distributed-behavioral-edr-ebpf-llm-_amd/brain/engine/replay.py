"""Trace replay: feed GIVEN token ids through an engine's model step by step and return logits, sampling nothing.

A trace step names, per request, the next tokens and the places among them whose logits are wanted; all of a step's
requests run as ONE batch — prompt portions through the prefill path, single follow-up tokens through the decode path,
side by side in a mixed step — on the engine's own block manager, state slots, cache and model.  Requests that end
give their pages and slot back, so a pool smaller than the sum of all requests is reused.

Used by ``bin/trace_run`` to replay recorded schedules (for instance to compare logits between builds or dtypes).
"""
from __future__ import annotations

from dataclasses import dataclass, field

import torch

from ...models.llama import StepBatch, h2d
from .engine import Engine


@dataclass
class _Live:
    slot: int
    blocks: list = field(default_factory=list)
    pos: int = 0


class TraceSession:
    def __init__(self, engine: Engine):
        if engine.has_work():
            raise RuntimeError("trace replay needs an idle engine")
        self.eng = engine
        self.live: dict[str, _Live] = {}

    def step(self, entries: list, end: list) -> torch.Tensor:
        """entries: [{"id", "tokens", "want"}]; end: ids finished after this step.  Returns float32 logits
        [sum(len(want)), vocab] on the host, in the order of the entries and of their ``want`` lists."""
        eng = self.eng
        pre, dec = [], []
        for e in entries:
            toks = list(e["tokens"])
            if not toks:
                continue
            r = self.live.get(e["id"])
            if r is None:
                if not eng.free_slots:
                    raise RuntimeError("no free state slot: too many live requests")
                r = self.live[e["id"]] = _Live(eng.free_slots.pop())
            if r.pos + len(toks) > eng.cfg.max_model_len:
                raise RuntimeError(f"request {e['id']} exceeds max_model_len {eng.cfg.max_model_len}")
            need = eng.blocks.blocks_for(r.pos + len(toks)) - len(r.blocks)
            if need > 0:
                r.blocks += eng.blocks.alloc(need)
            (dec if len(toks) == 1 and r.pos > 0 else pre).append((e, r, toks))
        out = None
        if pre or dec:
            out = self._forward(pre, dec, entries)
        for _, r, toks in pre + dec:
            r.pos += len(toks)
        for i in end:
            r = self.live.pop(i, None)
            if r is not None:
                eng.blocks.release(r.blocks)
                eng.free_slots.append(r.slot)
                eng.free_slots.sort(reverse=True)
        vocab = eng.model.cfg.vocab_size
        return out if out is not None else torch.zeros(0, vocab)

    def _decode_batch(self, dec) -> StepBatch:
        eng, n = self.eng, len(dec)
        i32 = lambda x: h2d(torch.tensor(x, dtype=torch.int32), eng.device)  # noqa: E731
        bt = torch.zeros(n, eng.max_blocks_per_seq, dtype=torch.int32)
        for i, (_, r, _) in enumerate(dec):
            bt[i, :len(r.blocks)] = torch.tensor(r.blocks, dtype=torch.int32)
        ctx = [r.pos + 1 for _, r, _ in dec]
        return StepBatch(i32([t[0] for *_, t in dec]), i32([r.pos for _, r, _ in dec]), i32(list(range(n))),
                         h2d(bt, eng.device), i32(list(range(n + 1))), i32(ctx),
                         h2d(torch.arange(n, dtype=torch.int64), eng.device), None, n, 1,
                         eng._nsplit(n, max(ctx)), slots=i32([r.slot for _, r, _ in dec]), max_q=1)

    def _forward(self, pre, dec, entries) -> torch.Tensor:
        eng = self.eng
        # flattened token order: the prefill portions, then the decode rows; the wanted rows in the entries' order
        at, off = {}, 0
        for e, _, toks in pre:
            at[id(e)] = off
            off += len(toks)
        for e, _, _ in dec:
            at[id(e)] = off
            off += 1
        want = [at[id(e)] + int(k) for e in entries if id(e) in at for k in e.get("want", ())]
        dsb = self._decode_batch(dec) if dec else None
        if pre:
            sb = eng.model.prefill_batch([t for *_, t in pre], [r.pos for _, r, _ in pre],
                                         [r.blocks for _, r, _ in pre], [r.slot for _, r, _ in pre],
                                         max_blocks=eng.max_blocks_per_seq, nqt=eng.cfg.prefill_nqt, want=want)
            sb.dec = dsb
        else:
            sb = dsb
            sb.last_idx = h2d(torch.tensor(want, dtype=torch.int64), eng.device)
        if not want:  # nothing asked for: still run the step (it fills the cache and advances the state)
            sb.last_idx = h2d(torch.zeros(1, dtype=torch.int64), eng.device)
        logits = eng.model.forward(sb, eng.kv, torch.float32)
        eng.stats["replay_steps"] += 1
        eng.stats["replay_tokens"] += off
        return logits.float().cpu() if want else torch.zeros(0, logits.shape[-1])
