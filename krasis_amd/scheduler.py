"""BatchEngine and Scheduler: requests in, batched steps of the serving store out.

`BatchEngine` owns a `ServeStore`, maps request ids to cache slots and runs one step for a list of (request, tokens, wanted places) -- the step
function every caller shares: the scheduler below for generation, and the trace replay of `python -m krasis_amd trace`.
`Scheduler` is continuous batching over it: up to `max_slots` live requests, decoding requests put one token into every step, prompts are fed in
portions within a token budget per step, a request is admitted when a slot is free and the pool can hold its prompt and its new tokens."""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

from . import serve_store as S

_DTYPES = {"bfloat16": S.BF16, "bf16": S.BF16, "float32": S.F32, "f32": S.F32}


def _named(get, name: str):
    """a checkpoint tensor, or with `tensor@row` one row of it (a table that holds one vector per pass of a repeated block)"""
    if "@" in name:
        base, row = name.rsplit("@", 1)
        return get(base)[int(row)]
    return get(name)


class BatchEngine:
    def __init__(self, spec, dtype: str = "bfloat16", max_tokens: int = 4096, max_slots: int = 4, device: int = 0, build: bool = False):
        if dtype not in _DTYPES:
            raise ValueError(f"dtype {dtype!r}: bfloat16 | float32")
        self.spec = spec
        self.store = S.ServeStore(spec.vocab, spec.width, spec.layers, dtype=_DTYPES[dtype], norm_kind=spec.norm_kind, norm_eps=spec.norm_eps,
                                  max_slots=max_slots, pool_tokens=max_tokens, device=device, build=build, block_kind=spec.block_kind, pre_norm=spec.pre_norm,
                                  post_norm=spec.post_norm, norm_bias=spec.norm_bias, residual_mult=spec.residual_mult, norm_groups=spec.norm_groups,
                                  embed_scale=spec.embed_scale, canon_taps=spec.canon_taps, res_gate=spec.res_gate, norm_weight_offset=spec.norm_weight_offset,
                                  embed_norm=spec.embed_norm, bigram=spec.bigram, logit_scale=spec.logit_scale)
        self.vocab = spec.vocab
        self._slot: Dict[object, int] = {}

    # ---- weights
    def load_safetensors(self, path: str) -> None:
        from .model_registry import SafetensorsFile
        f = SafetensorsFile(path)
        extra = getattr(self.spec, "extra", None) or {}
        for layer, role, index, name in self.spec.tensors(self.spec):
            self.store.set_tensor(layer, role, extra[name] if name in extra else _named(f.get, name), index)
        self.store.finalize()

    def load_arrays(self, arrays: Dict[str, np.ndarray]) -> None:
        """tensors by checkpoint name: float32, or uint16 bf16 bit patterns"""
        extra = getattr(self.spec, "extra", None) or {}
        for layer, role, index, name in self.spec.tensors(self.spec):
            self.store.set_tensor(layer, role, extra[name] if name in extra else _named(arrays.__getitem__, name), index)
        self.store.finalize()

    def load_synthetic(self, seed: int = 1, amp: float = 1.0) -> None:
        self.store.fill_synthetic(seed, amp)
        self.store.finalize()

    # ---- requests
    def live(self) -> List[object]:
        return list(self._slot)

    def admit(self, rid) -> int:
        if rid in self._slot:
            raise ValueError(f"request {rid!r} is already live")
        self._slot[rid] = self.store.admit()
        return self._slot[rid]

    def finish(self, rid) -> None:
        self.store.release(self._slot.pop(rid))

    def length(self, rid) -> int:
        return self.store.slot_len(self._slot[rid])

    def step(self, entries: Sequence[Tuple[object, Sequence[int], Sequence[int]]], logits: bool = True):
        """entries: (request id, its next tokens, places among them whose logits are wanted).  A request is admitted at its first entry.
        Returns (logits [wanted, vocab] or None, argmax [wanted]) in the order of the entries and of their wanted places."""
        batch, want, base = [], [], 0
        for rid, toks, places in entries:
            if rid not in self._slot:
                self.admit(rid)
            n = len(toks)
            for p in places:
                if not 0 <= p < n:
                    raise ValueError(f"request {rid!r}: wanted place {p} of {n} tokens")
                want.append(base + p)
            batch.append((self._slot[rid], toks))
            base += n
        return self.store.step(batch, want, logits=logits)

    # ---- generation through the scheduler
    def generate(self, prompts: Sequence[Sequence[int]], max_new_tokens: int, temperature: float = 0.0, top_k: int = 0, top_p: float = 1.0,
                 stop_ids: Sequence[int] = (), seed: int = 0, token_budget: int = 2048) -> List[List[int]]:
        sch = Scheduler(self, token_budget=token_budget)
        ids = [sch.submit(p, max_new_tokens, temperature, top_k, top_p, stop_ids, seed + i if seed else 0) for i, p in enumerate(prompts)]
        sch.run()
        return [sch.result(i) for i in ids]


@dataclass
class _Request:
    rid: int
    prompt: List[int]
    max_new: int
    temperature: float
    top_k: int
    top_p: float
    stop: frozenset
    seed: int
    fed: int = 0                         # prompt tokens already in the cache
    out: List[int] = field(default_factory=list)
    pending: Optional[int] = None        # sampled token not yet in the cache
    done: bool = False


class Scheduler:
    def __init__(self, engine: BatchEngine, token_budget: int = 2048):
        self.engine, self.token_budget = engine, max(1, token_budget)
        self._wait: deque = deque()
        self._live: List[_Request] = []
        self._all: Dict[int, _Request] = {}
        self._reserved = 0               # pages promised to live requests
        self.steps = 0

    def _pages(self, r: _Request) -> int:
        pt = self.engine.store.page_tokens
        return (len(r.prompt) + r.max_new + pt - 1) // pt

    def submit(self, prompt: Sequence[int], max_new_tokens: int, temperature: float = 0.0, top_k: int = 0, top_p: float = 1.0, stop_ids: Sequence[int] = (),
               seed: int = 0) -> int:
        if len(prompt) < 1:
            raise ValueError("empty prompt")
        r = _Request(len(self._all), list(prompt), max_new_tokens, temperature, top_k, top_p, frozenset(stop_ids), seed)
        if self._pages(r) * self.engine.store.page_tokens > self.engine.store.pool_tokens:
            raise ValueError(f"request needs {self._pages(r)} pages; the pool holds {self.engine.store.pool_tokens // self.engine.store.page_tokens}")
        self._all[r.rid] = r
        self._wait.append(r)
        return r.rid

    def result(self, rid: int) -> List[int]:
        return list(self._all[rid].out)

    def _admit(self) -> None:
        total = self.engine.store.pool_tokens // self.engine.store.page_tokens
        while self._wait and len(self._live) < self.engine.store.max_slots and self._reserved + self._pages(self._wait[0]) <= total:
            r = self._wait.popleft()
            self.engine.admit(("sched", r.rid))
            self._reserved += self._pages(r)
            self._live.append(r)

    def step(self) -> bool:
        """One batched step; False when nothing is left to do."""
        self._admit()
        if not self._live:
            return False
        budget = self.token_budget
        entries, owners = [], []
        for r in self._live:             # decoding requests first: one token each
            if r.pending is not None:
                entries.append((("sched", r.rid), [r.pending], [0])); owners.append(r); budget -= 1
        for r in self._live:             # then prompt portions while the budget lasts
            if r.pending is None and r.fed < len(r.prompt) and budget > 0:
                n = min(budget, len(r.prompt) - r.fed)
                last = r.fed + n == len(r.prompt)
                entries.append((("sched", r.rid), r.prompt[r.fed:r.fed + n], [n - 1] if last else [])); owners.append(r); budget -= n
        if not entries:
            return False
        _, amax = self.engine.step(entries, logits=False)
        self.steps += 1
        row = 0
        for (rid, toks, places), r in zip(entries, owners):
            if r.pending is not None:
                r.pending = None
            else:
                r.fed += len(toks)
            if not places:
                continue
            if r.temperature > 0.0:
                tok = self.engine.store.sample(row, r.temperature, r.top_k, r.top_p, (r.seed + len(r.out)) if r.seed else 0)
            else:
                tok = int(amax[row])
            row += 1
            r.out.append(tok)
            if tok in r.stop or len(r.out) >= r.max_new:
                r.done = True
            else:
                r.pending = tok
        for r in [q for q in self._live if q.done]:
            self.engine.finish(("sched", r.rid))
            self._reserved -= self._pages(r)
            self._live.remove(r)
        return True

    def run(self) -> None:
        while self.step():
            pass
