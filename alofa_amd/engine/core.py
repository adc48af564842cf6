"""The engine loop above the step function: prepare -> forward -> choose ->
settle, one scheduler action per tick (src/alofa/engine/core.mojo:382-694).

  prepare  reports last tick's news to the scheduler (arrivals, cancels,
           completions, pages given back), takes its action, drops cancelled and
           preempted requests from the cache, and turns prefill slices and
           decodes into the entries of one step;
  forward  runs the step function once;
  choose   picks a token for every entry that owes one (greedy or sampled);
  settle   records the tokens, queues each as its request's next row, and ends
           requests that have produced ``max_new`` tokens: their pages go back
           at once and the scheduler hears of it on the next tick.

Preemption is recompute: the victim loses its pages, its generated tokens and
its generator state, and is fed again from its first prompt token. There is no
end-of-sequence check: a request ends by count or by cancel (core.mojo:659-665)."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional

import numpy as np
import torch

from .. import ops
from ..errors import AlofaError
from ..sampling.sampler import SampleParams, Sampler, SplitMix64
from .scheduler import Action, SchedConfig, SchedInput, Scheduler, blocks_for
from .step import StepEntry, StepFunction
from .trace import config_line, trace_line

QUEUED, RESIDENT, DONE = "queued", "resident", "done"


@dataclass
class Request:
    id: int
    prompt: list
    max_new: int
    params: SampleParams
    seed: int
    state: str = QUEUED
    fed: int = 0                     # prompt tokens delivered to the cache
    out: list = field(default_factory=list)
    rng: Optional[SplitMix64] = None
    reported: bool = False
    preemptions: int = 0
    shared: int = 0                  # prompt tokens taken over from another request's pages


class EngineCore:
    def __init__(self, step_fn: StepFunction, sched_cfg: SchedConfig, trace_path=None, share_prefixes: bool = False):
        self.fn = step_fn
        # a new request starts on the whole pages of a resident request with the same first tokens
        # (by reference count) instead of computing them again; off unless asked for
        self.share_prefixes = bool(share_prefixes)
        self.shared_tokens = 0
        self.cache = step_fn.cache
        pool_blocks = min((g.pool.n_blocks for g in self.cache.groups), default=sched_cfg.capacity_blocks)
        if sched_cfg.capacity_blocks > pool_blocks:
            raise AlofaError("invalid_argument", "the scheduler counts more blocks than the pool has", f"scheduler={sched_cfg.capacity_blocks} pool={pool_blocks}")
        if sched_cfg.block_size != self.cache.block_size:
            raise AlofaError("invalid_argument", "scheduler and cache disagree on the block size", f"scheduler={sched_cfg.block_size} cache={self.cache.block_size}")
        self.sched = Scheduler(sched_cfg)
        self.requests: dict = {}
        self._arrivals: list = []
        self._cancels: list = []
        self._to_report: list = []
        self._freed_blocks = 0
        # blocks the scheduler charges a request with when it finishes (prompt + max_new), kept from
        # submission until the scheduler has let go of the id: a finished request may be released
        # before the tick that reports its completion
        self._charge: dict = {}
        self.sampler = Sampler()
        self.ticks = 0
        self.last_rows = 0
        self.last_action: Optional[Action] = None
        self._trace = open(trace_path, "w") if trace_path else None
        if self._trace:
            self._trace.write(config_line(sched_cfg) + "\n")

    # ------------------------------------------------------------ requests
    def submit(self, req: int, prompt: list, max_new: int, params: Optional[SampleParams] = None, seed: int = 1234) -> None:
        if req in self.requests or req in self._charge:
            raise AlofaError("invalid_argument", "duplicate request id", f"request={req}")
        if len(prompt) == 0 or max_new <= 0:
            raise AlofaError("invalid_argument", "a request needs a prompt and a positive max_new", f"request={req}")
        if len(prompt) + max_new > self.fn.n_positions:
            raise AlofaError("out_of_range", "prompt plus max_new passes the context bound", f"request={req} need={len(prompt) + max_new} bound={self.fn.n_positions}")
        vocab = self.fn.model.spec.vocab_size
        if min(prompt) < 0 or max(prompt) >= vocab:
            raise AlofaError("out_of_range", "token id outside the vocabulary", f"request={req} vocab={vocab}")
        self.requests[req] = Request(req, [int(t) for t in prompt], int(max_new), params or SampleParams(temperature=0.0), int(seed),
                                     rng=SplitMix64(seed))
        self._charge[req] = blocks_for(len(prompt) + int(max_new), self.sched.cfg.block_size)
        self._arrivals.append(req)

    def can_admit(self, prompt_len: int, max_new: int) -> bool:
        """Whether the scheduler would take such a request on the next tick."""
        pending = tuple((len(self.requests[a].prompt), self.requests[a].max_new) for a in self._arrivals)
        return self.sched.would_admit(prompt_len, max_new, pending)

    def cancel(self, req: int) -> None:
        if req in self.requests and self.requests[req].state != DONE:
            self._cancels.append(req)

    def is_done(self, req: int) -> bool:
        return self.requests[req].state == DONE

    def output(self, req: int) -> list:
        return list(self.requests[req].out)

    def release(self, req: int) -> None:
        if self.requests[req].state != DONE:
            raise AlofaError("invalid_argument", "only a finished request can be released", f"request={req}")
        del self.requests[req]

    def has_work(self) -> bool:
        return (bool(self._arrivals) or bool(self._cancels) or bool(self._to_report) or self._freed_blocks > 0
                or any(r.state != DONE for r in self.requests.values()))

    def _scheduler_let_go(self, cancelled: list, finished: list) -> None:
        """What follows from the scheduler's phases 1 and 2: a cancelled request loses its pages here
        too (the scheduler subtracted its blocks itself), and the blocks the scheduler moved to its
        "cached" count for a finished one are owed back on the next tick, since this engine keeps
        no prefix cache. The request itself may already have been released."""
        for c in cancelled:
            self._charge.pop(c, None)
            r = self.requests.get(c)
            if r is not None and r.state != DONE:
                self._drop(r)
                r.state = DONE
        for f in finished:
            self._freed_blocks += self._charge.pop(f, 0)

    # ---------------------------------------------------------------- tick
    def _drop(self, r: Request) -> None:
        if self.cache.has(r.id):
            self.cache.free(r.id)

    def prepare(self) -> list:
        """One scheduler tick; returns the entries of the step and who owes a token."""
        inp = SchedInput(
            arrivals=[(a, len(self.requests[a].prompt), self.requests[a].max_new) for a in self._arrivals],
            cancelled=list(self._cancels), finished=list(self._to_report), freed_blocks=self._freed_blocks)
        arrivals, self._arrivals = self._arrivals, []
        self._cancels, self._to_report, self._freed_blocks = [], [], 0
        try:
            act = self.sched.step(inp)
        except AlofaError:
            # a refused admission: the scheduler applied last tick's news (phases 0 to 2 stand) and
            # took none of this tick's arrivals; they are retired so that nothing asks for them again
            self._scheduler_let_go(inp.cancelled, inp.finished)
            for a in arrivals:
                self._charge.pop(a, None)
                if a in self.requests:
                    self.requests[a].state = DONE
            raise
        if self._trace:
            self._trace.write(trace_line(inp, act) + "\n")
            self._trace.flush()
        self.last_action = act
        self._scheduler_let_go(inp.cancelled, act.finished)
        for p in act.preempted:
            r = self.requests[p]
            self._drop(r)
            r.out, r.fed, r.state, r.rng = [], 0, QUEUED, SplitMix64(r.seed)
            r.preemptions += 1
        entries, owes = [], []
        for req, start, end in act.prefill:
            r = self.requests[req]
            skip = 0
            if start == 0 and not self.cache.has(req):
                self.cache.admit(req)
                if self.share_prefixes:
                    skip = r.shared = self._take_shared_prefix(r, end)
            elif r.fed != start:
                raise AlofaError("invalid_argument", "prefill slice does not continue the request", f"request={req} fed={r.fed} start={start}")
            last = end == len(r.prompt)
            entries.append(StepEntry(req, r.prompt[start + skip:end], [end - start - skip - 1] if last else []))
            owes.append(req if last else None)
            r.fed, r.state = end, RESIDENT
        for req in act.decode:
            r = self.requests[req]
            if req in act.preempted or r.state == DONE:
                continue
            if r.state != RESIDENT or not r.out:
                raise AlofaError("invalid_argument", "decode for a request that is not resident", f"request={req}")
            entries.append(StepEntry(req, [r.out[-1]], [0]))
            owes.append(req)
        return entries, owes

    def _take_shared_prefix(self, r: Request, end: int) -> int:
        """Let the freshly admitted ``r`` hold the whole pages that a resident request has already
        written for the same first tokens; returns how many tokens of the slice ``[0, end)`` are
        history from now on. The slice's last token is always computed
        (src/alofa/engine/executor.mojo:459-479)."""
        bs = self.cache.block_size
        best, donor = 0, None
        for o in self.requests.values():
            if o is r or o.state != RESIDENT or not self.cache.has(o.id):
                continue
            known = (o.prompt + o.out)[:self.cache.length(o.id)]
            n = 0
            for a, b in zip(known, r.prompt[:end - 1]):
                if a != b:
                    break
                n += 1
            if n // bs > best // bs:
                best, donor = n, o
        if donor is None:
            return 0
        got = self.cache.share_prefix(donor.id, r.id, best)
        self.shared_tokens += got
        return got

    def choose(self, logits: torch.Tensor, owes: list) -> list:
        """One token per row of ``logits``, for the requests in ``owes`` (in order)."""
        reqs = [self.requests[o] for o in owes]
        chosen = [None] * len(reqs)
        dev = [i for i, r in enumerate(reqs) if r.params.plain]
        if dev:
            greedy = [i for i in dev if r_is_greedy(reqs[i])]
            drawn = [i for i in dev if not r_is_greedy(reqs[i])]
            if greedy:
                rows = logits if len(greedy) == len(reqs) else logits[torch.tensor(greedy, device=logits.device)]
                out = torch.empty(len(greedy), dtype=torch.int32, device=logits.device)
                ops.argmax(out, rows)
                for i, t in zip(greedy, out.tolist()):
                    chosen[i] = int(t)
            if drawn:
                rows = logits[torch.tensor(drawn, device=logits.device)].contiguous()
                temp = torch.tensor([reqs[i].params.temperature for i in drawn], dtype=torch.float64, device=logits.device)
                u = torch.tensor([reqs[i].rng.next_uniform() for i in drawn], dtype=torch.float64, device=logits.device)
                out = torch.empty(len(drawn), dtype=torch.int32, device=logits.device)
                ops.sample(out, rows, temp, u)
                for i, t in zip(drawn, out.tolist()):
                    chosen[i] = int(t)
        host = [i for i in range(len(reqs)) if chosen[i] is None]
        if host:
            rows = logits[torch.tensor(host, device=logits.device)].cpu().numpy()
            for k, i in enumerate(host):
                r = reqs[i]
                self.sampler.build(rows[k], r.params, r.prompt + r.out)
                chosen[i] = self.sampler.pick(r.rng.next_uniform()) if not r.params.greedy else int(np.argmax(self.sampler.weights))
        return chosen

    def settle(self, owes: list, chosen: list) -> None:
        it = iter(chosen)
        for o in owes:
            if o is None:
                continue
            r = self.requests[o]
            r.out.append(next(it))
            if len(r.out) >= r.max_new:
                self._drop(r)
                r.state = DONE
                if self.sched.find(r.id) >= 0 and r.id not in self.last_action.finished:
                    self._to_report.append(r.id)
        for f in self.last_action.finished:
            r = self.requests.get(f)
            if r is not None and r.state != DONE:
                self._drop(r)
                r.state = DONE

    def tick(self) -> int:
        """One whole tick; returns the rows that ran."""
        entries, owes = self.prepare()
        self.ticks += 1
        self.last_rows = sum(len(e.tokens) for e in entries)
        if entries:
            logits = self.fn.run(entries)
            wanted = [o for o in owes if o is not None]
            chosen = self.choose(logits, wanted) if wanted else []
            self.settle(owes, chosen)
        else:
            self.settle([], [])
        return self.last_rows

    def run(self, max_ticks: int = 1 << 30) -> None:
        n = 0
        while self.has_work():
            if n >= max_ticks:
                raise AlofaError("capacity", "the engine did not finish within the tick limit", f"max_ticks={max_ticks}")
            self.tick()
            n += 1


def r_is_greedy(r: Request) -> bool:
    return r.params.greedy
