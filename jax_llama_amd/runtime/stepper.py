"""Request stepper: feeds GIVEN tokens of named requests through a model, portion by portion.

The counterpart of the generation engine for replaying a trace (or scoring text): each request owns one row of cache
(keys / values of the attention layers, the recurrent layers' state) from its first portion until it ends; a portion
runs only its own tokens on top of what the earlier portions left, through the model's step function
(``forward_tokens``) -- the same one the engine's prefill and decode steps call. Rows are pooled: an ended request's row
goes back to the pool and is reset when the next request takes it.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

import torch


class SequenceStepper:
    def __init__(self, model, max_tokens: int):
        """``max_tokens``: the most tokens a request may hold (the length of a cache row)."""
        self.model = model
        self.max_tokens = int(max_tokens)
        self._free: List = []               # pooled single-row caches
        self._live: Dict[str, Tuple] = {}   # request id -> cache

    # ---------------------------------------------------------------- rows
    def _row(self, rid: str):
        cache = self._live.get(rid)
        if cache is None:
            cache = self._free.pop() if self._free else self.model.init_cache(1, self.max_tokens)
            cache.reset()
            self._live[rid] = cache
        return cache

    def live(self) -> List[str]:
        return sorted(self._live)

    def held(self, rid: str) -> int:
        return self._live[rid].index if rid in self._live else 0

    def end(self, rid: str) -> None:
        cache = self._live.pop(rid, None)
        if cache is not None:
            self._free.append(cache)

    # ---------------------------------------------------------------- steps
    def feed(self, rid: str, tokens: Sequence[int], want: Sequence[int] = ()) -> Optional[torch.Tensor]:
        """Run the next ``tokens`` of request ``rid``; returns fp32 logits ``[len(want), vocab]`` at the places ``want``
        (indices into ``tokens``), or None when nothing is wanted."""
        n = len(tokens)
        if n == 0:
            return None
        cache = self._row(rid)
        s0 = cache.index
        if s0 + n > cache.max_length:
            raise ValueError(f"request {rid!r} would hold {s0 + n} tokens, more than {cache.max_length}")
        if any(w < 0 or w >= n for w in want):
            raise ValueError(f"request {rid!r}: wanted place outside the portion")
        dev = self.model.device
        ids = torch.tensor([list(tokens)], dtype=torch.int32, device=dev)
        pos = torch.arange(s0, s0 + n, dtype=torch.int32, device=dev).reshape(1, n)
        if len(want):
            rows = torch.tensor(list(want), dtype=torch.long, device=dev)
            logits, *_ = self.model.forward_tokens(ids, pos, cache, cache.index_t, logits_mode="rows", logit_rows=rows)
        else:
            logits = None
            self.model.forward_tokens(ids, pos, cache, cache.index_t, logits_mode="none")
        cache.advance(n)
        return logits

    def step(self, entries: Sequence[dict], end: Sequence[str] = ()) -> Optional[torch.Tensor]:
        """One trace step: ``entries`` of ``{"id", "tokens", "want"}`` run in order, then the requests in ``end`` give
        their rows back. Returns the wanted logits of all entries stacked (None if none)."""
        outs = []
        for e in entries:
            lg = self.feed(e["id"], e["tokens"], e.get("want", ()))
            if lg is not None:
                outs.append(lg)
        for rid in end:
            self.end(rid)
        return torch.cat(outs, 0) if outs else None
