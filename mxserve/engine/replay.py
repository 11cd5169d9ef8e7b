"""Trace replay: feed given token ids through the engine step by step and return logits instead of
sampled tokens.  A trace dictates every step -- which requests run, how many of their next tokens,
which rows' logits are wanted, which requests end -- so the scheduler's policy is bypassed
(Scheduler.schedule_forced), while block allocation, the runner's batch preparation, its
block-table rows and state slots, the decode graphs and the kernels are those of generation.

One step is one JSON object:
    {"step": n, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}, ...], "end": ["a"]}
A request is admitted at its first entry, may skip steps, and gives back its blocks and its slot
when a step lists it under "end".
"""
from __future__ import annotations

from typing import Optional

import torch

from .engine import LLMEngine
from .request import Request, SamplingParams


class TraceReplayer:
    def __init__(self, engine: LLMEngine):
        self.engine = engine
        self.live: dict[str, Request] = {}

    def step(self, entries: list, end: list) -> Optional[torch.Tensor]:
        """Run one step; returns the wanted rows' logits [n, vocab] (fp32, on the host) in the order of
        the entries and of each entry's `want`, or None when nothing is wanted."""
        eng = self.engine
        sched = eng.scheduler
        plan = []
        for e in entries:
            rid, toks = str(e["id"]), [int(t) for t in e["tokens"]]
            req = self.live.get(rid)
            if req is None:
                req = Request(rid, [], SamplingParams(max_tokens=1, temperature=0.0))
                sched.admit_forced(req)
                eng.requests[rid] = req
                self.live[rid] = req
            req.prompt_token_ids.extend(toks)
            want = sorted(int(k) for k in e.get("want") or ())
            if want and not (0 <= want[0] and want[-1] < len(toks)):
                raise ValueError(f"{rid}: wanted rows {want} outside its {len(toks)} tokens")
            plan.append((req, len(toks), want))
        logits = None
        if plan:
            so = sched.schedule_forced(plan)
            handle = eng.runner.launch(so)
            eng.num_steps += 1
            lg = handle.get("logits")
            if lg is not None and lg.shape[0]:
                # rows come back in batch order (single tokens first, then chunks): restore the entries' order
                order = {id(s.req): k for k, s in enumerate(so.all())}
                counts = [len(s.logit_offsets or ()) for s in so.all()]
                starts = [sum(counts[:k]) for k in range(len(counts))]
                pick = [starts[order[id(req)]] + j for req, _, want in plan for j in range(len(want))]
                lg = lg.float()
                if pick != list(range(lg.shape[0])):
                    lg = lg.index_select(0, torch.tensor(pick, dtype=torch.int64, device=lg.device))
                logits = lg.cpu()
        for rid in end:
            req = self.live.pop(str(rid), None)
            if req is not None:
                sched.finish_forced(req)
                eng.requests.pop(req.request_id, None)
                eng.runner.release(req.request_id)
        return logits
