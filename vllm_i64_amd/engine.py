"""Engine: requests, slots, pages, step batching and sampling on top of any registered runner.

A step is one batch: portions of prompts beside single decoded tokens, rows in request order.  `Engine.step` runs exactly the
tokens it is given from the cache that earlier steps left (replay of a recorded schedule, tests); `Engine.generate` makes the
steps itself: requests are admitted while a slot is free and their pages fit, prompts are cut into portions under a token budget,
running sequences decode in the same steps, finished ones give slot and pages back at once (continuous batching).  Both go
through the same `_run`, i.e. the same runner.forward, cache and kernels."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Iterable, List, Optional, Sequence, Tuple

import torch


@dataclass
class SamplingParams:
    max_new_tokens: int = 16
    temperature: float = 0.0       # 0: greedy
    top_k: int = 0                 # 0: no limit
    top_p: float = 1.0
    seed: Optional[int] = None
    stop_token: Optional[int] = None


@dataclass
class _Seq:
    rid: str
    slot: int
    cached: int = 0                                      # tokens whose state is in the cache
    pending: List[int] = field(default_factory=list)     # prompt tokens not yet run (generation API)
    out: List[int] = field(default_factory=list)
    params: Optional[SamplingParams] = None
    gen: Optional[torch.Generator] = None
    next_token: Optional[int] = None                     # sampled, to be run by the next step


class Engine:
    def __init__(self, model, max_batch_tokens: int = 512):
        self.model, self.kv, self.device = model, model.kv, model.device
        self.max_batch_tokens = int(max_batch_tokens)
        self.seqs: Dict[str, _Seq] = {}
        self._free_slots = list(range(self.kv.max_seqs - 1, -1, -1))
        self._waiting: List[Tuple[str, List[int], SamplingParams]] = []
        self._finished: Dict[str, List[int]] = {}
        self._auto = 0

    # ---- requests, slots, pages -----------------------------------------------------------------------------------------------
    def admit(self, rid: str) -> _Seq:
        if rid in self.seqs:
            raise ValueError(f"request '{rid}' is live already")
        if not self._free_slots:
            raise RuntimeError(f"no free slot: {len(self.seqs)} requests are live, the cache has {self.kv.max_seqs} slots")
        s = _Seq(rid=rid, slot=self._free_slots.pop())
        self.seqs[rid] = s
        return s

    def release(self, rid: str) -> None:
        s = self.seqs.pop(rid)
        self.kv.free(s.slot)
        self._free_slots.append(s.slot)

    # ---- one step ---------------------------------------------------------------------------------------------------------------
    def _run(self, batch: Sequence[Tuple[_Seq, Sequence[int], Sequence[int]]]) -> torch.Tensor:
        """batch: (sequence, its next tokens, the places among them whose logits are wanted).  Returns fp32 [wanted, V]."""
        ids: List[int] = []
        pos: List[int] = []
        slots: List[int] = []
        rows: List[int] = []
        tps: List[int] = []
        for s, toks, want in batch:
            k = len(toks)
            if k == 0:
                continue
            self.kv.reserve(s.slot, s.cached + k)
            base = len(ids)
            for w in want:
                if not 0 <= int(w) < k:
                    raise ValueError(f"request '{s.rid}': place {w} outside its {k} tokens")
                rows.append(base + int(w))
            ids.extend(int(t) for t in toks)
            pos.extend(range(s.cached, s.cached + k))
            slots.extend([s.slot] * k)
            tps.append(k)
        V = self.model.cfg.vocab_size
        if not ids:
            return torch.empty(0, V, dtype=torch.float32, device=self.device)
        if min(ids) < 0 or max(ids) >= V:
            raise ValueError(f"token id outside [0, {V})")
        dev = self.device
        t_ids = torch.tensor(ids, dtype=torch.int64).to(dev)
        t_pos = torch.tensor(pos, dtype=torch.int32).to(dev)
        t_slots = torch.tensor(slots, dtype=torch.int32).to(dev)
        t_rows = torch.tensor(rows, dtype=torch.int32).to(dev)
        if not rows:   # nothing asked for: the step still runs (it fills the cache); one row keeps the shapes non-empty
            t_rows = torch.zeros(1, dtype=torch.int32, device=dev)
        logits = self.model.forward(t_ids, t_pos, t_slots, (t_pos + 1).contiguous(), logit_rows=t_rows, max_ctx_hint=max(pos) + 1,
                                    tokens_per_seq=tps)
        self.model.check_sync(force=False)
        for s, toks, _ in batch:
            s.cached += len(toks)
        return logits[: len(rows)]

    def step(self, entries: Iterable[Tuple[str, Sequence[int], Sequence[int]]], end: Iterable[str] = ()) -> torch.Tensor:
        """Run one given step: entries = (request id, its next tokens, wanted places).  A request is admitted at its first entry; the
        requests in `end` give back slot and pages after the step.  Returns the wanted logits in entry order."""
        batch = []
        for rid, toks, want in entries:
            s = self.seqs.get(rid) or self.admit(rid)
            batch.append((s, list(toks), list(want)))
        try:
            return self._run(batch)
        finally:
            for rid in end:
                if rid in self.seqs:
                    self.release(rid)

    # ---- generation -------------------------------------------------------------------------------------------------------------
    def add_request(self, prompt: Sequence[int], params: Optional[SamplingParams] = None, rid: Optional[str] = None) -> str:
        if not len(prompt):
            raise ValueError("empty prompt")
        if rid is None:
            rid = f"req{self._auto}"
            self._auto += 1
        self._waiting.append((rid, [int(t) for t in prompt], params or SamplingParams()))
        return rid

    def _admit_waiting(self) -> None:
        """First come, first served: a request starts when a slot is free and the pages of its prompt and its answer fit beside
        what the live requests may still grow to."""
        while self._waiting and self._free_slots:
            rid, prompt, params = self._waiting[0]
            committed = sum(self.kv.blocks_for(s.cached + len(s.pending) + s.params.max_new_tokens - len(s.out)) - len(self.kv.blocks_of(s.slot))
                            for s in self.seqs.values() if s.params is not None)
            if self.kv.blocks_for(len(prompt) + params.max_new_tokens) > self.kv.free_blocks - max(committed, 0):
                if not self.seqs:
                    raise RuntimeError(f"request '{rid}' needs more pages than the pool has")
                break
            self._waiting.pop(0)
            s = self.admit(rid)
            s.pending, s.params = prompt, params
            if params.temperature > 0:
                s.gen = torch.Generator().manual_seed(params.seed if params.seed is not None else 0)

    def schedule(self) -> List[Tuple[_Seq, List[int], List[int]]]:
        """The next step: one token of every decoding sequence, then prompt portions in arrival order while the budget lasts."""
        self._admit_waiting()
        batch, budget = [], self.max_batch_tokens
        live = [s for s in self.seqs.values() if s.params is not None]
        for s in live:
            if not s.pending and s.next_token is not None and budget > 0:
                batch.append((s, [s.next_token], [0]))
                budget -= 1
        for s in live:
            if s.pending and budget > 0:
                k = min(budget, len(s.pending))
                batch.append((s, s.pending[:k], [k - 1] if k == len(s.pending) else []))
                budget -= k
        return batch

    def _sample(self, logits: torch.Tensor, seqs: List[_Seq]) -> List[int]:
        from . import ops_dense
        if all(s.params.temperature <= 0 for s in seqs):
            return ops_dense.sample_rows(logits.contiguous()).tolist()
        dev = self.device
        temp = torch.tensor([max(s.params.temperature, 0.0) for s in seqs], dtype=torch.float32).to(dev)
        top_k = torch.tensor([s.params.top_k for s in seqs], dtype=torch.int32).to(dev)
        top_p = torch.tensor([s.params.top_p for s in seqs], dtype=torch.float32).to(dev)
        u = torch.tensor([float(torch.rand(1, generator=s.gen)) if s.gen is not None else 0.0 for s in seqs], dtype=torch.float32).to(dev)
        return ops_dense.sample_rows(logits.contiguous(), temperature=temp, top_k=top_k, top_p=top_p, u=u).tolist()

    def run_step(self) -> List[Tuple[str, int]]:
        """Schedule, run and sample one step of the generation API; returns the (request, token) pairs it produced."""
        batch = self.schedule()
        if not batch:
            return []
        logits = self._run(batch)
        asked = [s for s, toks, want in batch if want]
        for s, toks, _ in batch:
            if s.pending:
                del s.pending[: len(toks)]
        produced = []
        if asked:
            for s, tok in zip(asked, self._sample(logits, asked)):
                s.out.append(int(tok))
                s.next_token = int(tok)
                produced.append((s.rid, int(tok)))
                if len(s.out) >= s.params.max_new_tokens or (s.params.stop_token is not None and tok == s.params.stop_token):
                    self._finished[s.rid] = s.out
                    self.release(s.rid)
        return produced

    def generate(self, prompts: Sequence[Sequence[int]], params: Optional[SamplingParams] = None) -> List[List[int]]:
        """Run the prompts to completion (more prompts than slots: the later ones wait their turn); the new tokens per prompt."""
        rids = [self.add_request(p, params) for p in prompts]
        while self._waiting or any(s.params is not None for s in self.seqs.values()):
            if not self.run_step() and not self._waiting and not any(s.params is not None for s in self.seqs.values()):
                break
        return [self._finished.pop(r) for r in rids]
