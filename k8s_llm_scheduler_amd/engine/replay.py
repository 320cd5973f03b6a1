"""Replay of given token ids through the engine, step by step, returning logits instead of sampling.

A replay step is one engine iteration whose tokens are dictated: every entry brings the next tokens of one request (a
portion of its prompt, or one token after an earlier portion) and all entries of a step form one batch.  The step
uses what generation uses: a slot per live request, blocks from the allocator (taken as the request grows and given
back when it ends, so pages and slots are reused), the varlen ``forward_prefill`` for steps that hold prompt portions
(single tokens of other requests ride along as 1-token sequences, as running decodes do in a mixed step) and
``forward_decode`` over the slot rows for steps that hold only single tokens.  Mixed into :class:`~.engine.LLMEngine`.
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from .common import Request
from .sampling import SamplingParams


class ReplayMixin:
    _replay: Optional[Dict[str, Request]] = None

    def _replay_request(self, key: str) -> Request:
        if self._replay is None:
            self._replay = {}
        r = self._replay.get(key)
        if r is None:
            if not self.free_slots:
                raise RuntimeError(f"no free slot for request {key!r}: {self.max_batch} are live")
            r = Request(next(self._ids), [], SamplingParams(), 0)
            r.slot = self.free_slots.pop()
            self.requests[r.rid] = r
            self.prefilling.append(r)
            self._replay[key] = r
        return r

    def _replay_grow(self, r: Request, n: int) -> None:
        """Blocks for ``n`` more tokens of ``r``."""
        total = r.computed + n
        if total > self.max_model_len:
            raise ValueError(f"request of {total} tokens exceeds max_model_len {self.max_model_len}")
        need = math.ceil(total / self.block_size) - len(r.blocks)
        if need > 0:
            r.blocks += list(self.allocator.allocate([], need * self.block_size).blocks)

    def replay_step(self, entries: Sequence[Tuple[str, List[int], List[int]]], end: Sequence[str] = ()) -> torch.Tensor:
        """``entries``: (request key, its next tokens, indices among them whose logits are wanted).  Returns the wanted
        rows' fp32 logits [rows, vocab] in entry order (CPU).  ``end``: requests whose slot and blocks are released
        after the step."""
        with self.lock:
            chunk = []
            for key, tokens, _ in entries:
                if not tokens:
                    raise ValueError(f"request {key!r}: empty portion")
                r = self._replay_request(key)
                self._replay_grow(r, len(tokens))
                r.prompt_ids += list(tokens)
                chunk.append((r, r.computed, r.computed + len(tokens)))
            rows = None
            if chunk:
                if all(e - s == 1 and s > 0 for _, s, e in chunk):
                    logits, row_of = self._replay_decode(chunk)
                else:
                    logits, row_of = self._replay_varlen(chunk, [w for _, _, w in entries])
                pick = []
                for i, (_, _, want) in enumerate(entries):
                    pick += [row_of(i, w) for w in want]
                for r, _, e in chunk:
                    r.computed = e
                if pick:
                    rows = logits[0].index_select(0, self._dev(pick, torch.long)).float().cpu()
                elif self.gpu:
                    self._wait_device("replay")
            for key in end:
                r = (self._replay or {}).pop(key, None)
                if r is not None:
                    self._finish(r, "replay")
                    self.requests.pop(r.rid, None)
            V = self.model.cfg.vocab
            return rows if rows is not None else torch.zeros(0, V)

    def _replay_varlen(self, chunk, wants):
        ids, pos, slots, cu, ctx, _, bt = self._chunk_inputs(chunk)
        last, base = [], []
        for i, w in enumerate(wants):
            base.append(len(last))
            last += [cu[i] + k for k in w]
        t = self._dev
        logits = self.model.forward_prefill(t(ids), t(pos), t(slots), t(cu), t(ctx), self._dev(bt),
                                            max(e - s for _, s, e in chunk), t(last or [0]),
                                            **self._state_kw([r.slot for r, _, _ in chunk]))
        self.stats["prefill_tokens"] += len(ids)
        return logits, lambda i, w: base[i] + wants[i].index(w)

    def _replay_decode(self, chunk):
        """Single tokens only: the decode forward over the slot rows (idle rows have context length 0)."""
        B = self._bucket(max(r.slot for r, _, _ in chunk) + 1)
        tok = torch.zeros(B, dtype=torch.int32)
        ctx = torch.zeros(B, dtype=torch.int32)
        bt = torch.zeros(B, self.max_blocks_per_seq, dtype=torch.int32)
        for r, s, e in chunk:
            tok[r.slot] = r.prompt_ids[s]
            ctx[r.slot] = e
            bt[r.slot, :len(r.blocks)] = torch.tensor(r.blocks, dtype=torch.int32)
        self.s_tokens[:B].copy_(self._dev(tok))
        self.s_ctx[:B].copy_(self._dev(ctx))
        self.s_bt[:B].copy_(self._dev(bt))
        mc = next(c for c in self._ctx_classes() if max(e for _, _, e in chunk) <= c)
        logits = self.model.forward_decode(self.s_tokens[:B], self.s_ctx[:B], self.s_bt[:B], mc)
        self.s_ctx[:B].zero_()
        self.stats["decode_steps"] += 1
        slot_of = [r.slot for r, _, _ in chunk]
        return logits, lambda i, w: slot_of[i]
