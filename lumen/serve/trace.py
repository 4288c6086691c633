"""Replay of a token trace through the serving engine: given token ids in, logits out.

A trace is a list of steps; each step names, per request, the next tokens to feed and the places
among them whose logits are wanted.  Nothing is sampled: the tokens are forced.  Every step is
ONE engine batch built by the engine's own input builder (``LLMEngine._build_input``) and run
by its model runner on its block manager / state slots: entries with several tokens (or a
request's first entry) are prefill chunks, single tokens of requests already in the cache are
decode rows (a step of decode rows only takes the hipGraph decode path, as in generation).
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .engine import LLMEngine
from .scheduler import Batch
from .sequence import SamplingParams, Sequence, Status


class TraceReplay:
    def __init__(self, engine: LLMEngine):
        if engine.tp > 1:
            raise ValueError("trace replay runs at tensor-parallel size 1")
        self.engine = engine
        self.live: Dict[str, Sequence] = {}

    def _admit(self, rid: str) -> Sequence:
        eng = self.engine
        if len(self.live) >= eng.cfg.max_num_seqs:
            raise RuntimeError(f"more than {eng.cfg.max_num_seqs} live requests")
        s = Sequence([], SamplingParams(max_tokens=1, temperature=0.0, ignore_eos=True), rid)
        s.status = Status.RUNNING
        if eng.states is not None:
            eng.states.alloc(s.seq_id)
        self.live[rid] = s
        return s

    def _retire(self, rid: str) -> None:
        s = self.live.pop(rid, None)
        if s is None:
            return
        eng = self.engine
        eng.blocks.free_seq(s.seq_id)
        if eng.states is not None:
            eng.states.release(s.seq_id)
        s.status = Status.FINISHED

    @torch.no_grad()
    def step(self, entries: List[dict], end: Optional[List[str]] = None) -> torch.Tensor:
        """Feed each entry's ``tokens`` to its request ``id``; returns the logits [n, V] (fp32, on
        the host) at every entry's ``want`` places, in entry order.  Requests in ``end`` give
        their blocks and state slot back after the step."""
        eng = self.engine
        pre, dec = [], []
        for k, e in enumerate(entries):
            toks = [int(t) for t in e["tokens"]]
            if not toks:
                continue
            s = self.live.get(e["id"]) or self._admit(e["id"])
            if any(t < 0 or t >= eng.model_config.vocab_size for t in toks):
                raise ValueError(f"request {e['id']}: token id out of range")
            s.prompt_ids.extend(toks)
            if s.length > eng.cfg.max_model_len:
                raise ValueError(f"request {e['id']}: {s.length} tokens exceed max_model_len")
            eng.blocks.ensure(s.seq_id, s.length)
            (dec if len(toks) == 1 and s.num_cached > 0 else pre).append((k, s, len(toks)))
        if not pre and not dec:
            for rid in end or []:
                self._retire(rid)
            return torch.empty(0, eng.model_config.vocab_size)
        batch = Batch("mixed" if pre else "decode", [(s, c) for _, s, c in pre],
                      [s for _, s, _ in dec])
        # row of each entry's first token in the step: prefill chunks first, then decode rows
        first, r = {}, 0
        for k, s, c in pre + dec:
            first[k] = r
            r += c
        rows = [first[k] + int(w) for k, e in enumerate(entries) if k in first
                for w in e.get("want", [])]
        inp = eng._build_input(batch)
        want = torch.tensor(rows, dtype=torch.long, device=eng.device)
        if batch.kind == "decode":
            logits = eng.runner.decode(inp)[want]
        else:
            inp.sample_rows = want
            inp.extra_rows = None
            logits = eng.runner.execute(inp)
        for _, s, c in pre + dec:
            s.num_cached += c
        eng.stats["steps"] += 1
        eng.stats["prefill_tokens"] += inp.num_prefill_rows
        eng.stats["decode_tokens"] += len(dec)
        out = logits.float().cpu()
        for rid in end or []:
            self._retire(rid)
        return out
