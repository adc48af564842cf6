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

A token chosen on the device stays there: the choice writes it to the step
function's token store, where the next step's embedding finds it. What the host
needs of it is only its value for the output, and nothing the scheduler decides
depends on values (requests end by count). So the engine runs ahead: a tick
lays out and launches its step, launches the choice and an asynchronous copy
of the chosen tokens, and only then reads back the tokens of the tick before;
the GPU never waits for the host between steps. Outputs lag the ticks by one
until ``flush`` (``run`` and ``is_done`` see to that). Requests whose sampling
needs the host (filters, penalties) make their tick synchronous.

Preemption is recompute: the victim loses its pages, its generated tokens and
its generator state, and is fed again from its first prompt token. There is no
end-of-sequence check: a request ends by count or by cancel (core.mojo:659-665)."""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Optional

import numpy as np
import torch

from .. import ops
from ..errors import AlofaError
from ..sampling.sampler import SampleParams, Sampler, SplitMix64
from .scheduler import Action, SchedConfig, SchedInput, Scheduler
from .step import TOKEN_ON_DEVICE, StepEntry, StepFunction
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
    pending: int = 0                 # tokens chosen on the device whose values have not been read back yet
    on_device: bool = False          # the last chosen token lies in the step function's token store


class EngineCore:
    def __init__(self, step_fn: StepFunction, sched_cfg: SchedConfig, trace_path=None, share_prefixes: bool = False,
                 run_ahead: bool = True):
        self.fn = step_fn
        # read the tokens of a tick back only after the next tick's step has been launched
        self.run_ahead = bool(run_ahead)
        self._inflight: deque = deque()      # (owed [(request id, preemptions)], pinned tokens, count, event), oldest first
        self._staging = None
        # a new request starts on the whole pages of a resident request with the same first tokens
        # (by reference count) instead of computing them again; off unless asked for
        self.share_prefixes = bool(share_prefixes)
        self.shared_tokens = 0
        self.cache = step_fn.cache
        # the scheduler counts the pages of every group of layers: one rule per group (a scheduler with a single
        # rule over several groups counts for all of them with it, so every pool must hold what it counts)
        rules, pools = sched_cfg.groups, [g.pool.n_blocks for g in self.cache.groups]
        if len(rules) not in (1, len(pools)):
            raise AlofaError("invalid_argument", "the scheduler's groups are not the cache's", f"scheduler={len(rules)} cache={len(pools)}")
        for g, n in enumerate(pools):
            capacity = rules[g if len(rules) > 1 else 0][0]
            if capacity > n:
                raise AlofaError("invalid_argument", "the scheduler counts more blocks than the pool has", f"group={g} scheduler={capacity} pool={n}")
        if sched_cfg.block_size != self.cache.block_size:
            raise AlofaError("invalid_argument", "scheduler and cache disagree on the block size", f"scheduler={sched_cfg.block_size} cache={self.cache.block_size}")
        self.sched = Scheduler(sched_cfg)
        self.requests: dict = {}
        self._arrivals: list = []
        self._cancels: list = []
        self._to_report: list = []
        self._freed_blocks = [0] * len(rules)     # per group of the scheduler
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
        cfg = self.sched.cfg
        self._charge[req] = [cfg.blocks(len(prompt) + int(max_new), g) for g in range(len(cfg.groups))]
        self._arrivals.append(req)

    def can_admit(self, prompt_len: int, max_new: int) -> bool:
        """Whether the scheduler would take such a request on the next tick."""
        pending = tuple((len(self.requests[a].prompt), self.requests[a].max_new) for a in self._arrivals)
        return self.sched.would_admit(prompt_len, max_new, pending)

    def cancel(self, req: int) -> None:
        if req in self.requests and self.requests[req].state != DONE:
            self._cancels.append(req)

    def is_done(self, req: int) -> bool:
        """Finished, and every token's value has arrived."""
        r = self.requests[req]
        return r.state == DONE and r.pending == 0

    def output(self, req: int) -> list:
        return list(self.requests[req].out)

    def release(self, req: int) -> None:
        if not self.is_done(req):
            raise AlofaError("invalid_argument", "only a finished request can be released", f"request={req}")
        del self.requests[req]

    def has_work(self) -> bool:
        return (bool(self._arrivals) or bool(self._cancels) or bool(self._to_report) or any(self._freed_blocks)
                or bool(self._inflight) or any(r.state != DONE for r in self.requests.values()))

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
            for g, n in enumerate(self._charge.pop(f, ())):
                self._freed_blocks[g] += n

    # ---------------------------------------------------------------- tick
    def _drop(self, r: Request) -> None:
        if self.cache.has(r.id):
            self.cache.free(r.id)

    def prepare(self) -> list:
        """One scheduler tick; returns the entries of the step and who owes a token."""
        inp = SchedInput(
            arrivals=[(a, len(self.requests[a].prompt), self.requests[a].max_new) for a in self._arrivals],
            cancelled=list(self._cancels), finished=list(self._to_report), freed_blocks=list(self._freed_blocks))
        arrivals, self._arrivals = self._arrivals, []
        self._cancels, self._to_report, self._freed_blocks = [], [], [0] * len(self._freed_blocks)
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
            r.pending, r.on_device = 0, False          # a token of its still on its way is dropped when it arrives
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
            if r.state != RESIDENT or not (r.out or r.pending):
                raise AlofaError("invalid_argument", "decode for a request that is not resident", f"request={req}")
            entries.append(StepEntry(req, [TOKEN_ON_DEVICE if r.on_device else r.out[-1]], [0]))
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

    # ------------------------------------------------------------------ choice
    def _stage(self):
        """Small pinned blocks (taking turns, as a block's copy runs only when the GPU gets there)
        and their mirror on the device: request slots of the rows that choose on the device,
        temperatures and uniform numbers going up, chosen tokens coming down."""
        if self._staging is None:
            cap, dev = self.cache.max_requests, self.fn.device
            up_bytes = 4 * cap + 16 * cap                       # int32 slots, float64 temperatures, float64 uniforms

            def views(block, host):
                v = {"slots": block[:4 * cap].view(torch.int32), "temperature": block[4 * cap:12 * cap].view(torch.float64),
                     "uniform": block[12 * cap:].view(torch.float64)}
                return {k: t.numpy() for k, t in v.items()} if host else v
            mirror = torch.empty(up_bytes, dtype=torch.uint8, device=dev)
            turns = []
            for _ in range(3):
                up = torch.empty(up_bytes, dtype=torch.uint8, pin_memory=True)
                down = torch.empty(cap, dtype=torch.int32, pin_memory=True)
                turns.append({"up": up, "down": down, "tokens": down.numpy(), "event": torch.cuda.Event(), **views(up, True)})
            self._staging = {"turns": turns, "turn": 0, "mirror": mirror, "chosen": torch.empty(cap, dtype=torch.int32, device=dev),
                             **views(mirror, False)}
        return self._staging

    def choose(self, logits: Optional[torch.Tensor], owes: list, by_step: Optional[torch.Tensor] = None) -> Optional[list]:
        """One token per row of ``logits``, for the requests in ``owes`` (in order); or, with
        ``by_step`` (int32 on the device, what a step that chose greedily by itself returned, the
        token store already written), only their way to the host. Requests that
        sample plainly (greedy, or temperature alone) choose on the device; the tokens go to the
        token store and set out for the host, and None is returned: ``collect`` reads them later.
        With a request that needs the host's chain the whole tick is synchronous and the tokens
        are returned."""
        reqs = [self.requests[o] for o in owes]
        n = len(reqs)
        if by_step is not None:
            st = self._stage()
            turn = st["turns"][st["turn"]]
            st["turn"] = (st["turn"] + 1) % len(st["turns"])
            turn["event"].synchronize()                          # this block's last use (three ticks ago) is over
            turn["down"][:n].copy_(by_step[:n], non_blocking=True)
            turn["event"].record()
            for r in reqs:
                r.on_device = True
            self._inflight.append(([(r.id, r.preemptions) for r in reqs], turn["tokens"], n, turn["event"]))
            return None
        host = [i for i, r in enumerate(reqs) if not r.params.plain]
        greedy = [i for i, r in enumerate(reqs) if r.params.plain and r_is_greedy(r)]
        drawn = [i for i, r in enumerate(reqs) if r.params.plain and not r_is_greedy(r)]
        order = greedy + drawn
        if order:
            st = self._stage()
            turn = st["turns"][st["turn"]]
            st["turn"] = (st["turn"] + 1) % len(st["turns"])
            turn["event"].synchronize()                          # this block's last use (three ticks ago) is over
            ctx = self.fn.last_context
            ng, nd = len(greedy), len(drawn)
            slots = [self.cache.slot(reqs[i].id) for i in order]
            if ng == n and ctx.request_slots is not None and ctx.request_slots.shape[0] == n:
                slots_dev = ctx.request_slots                    # a decode step keeps its requests' slots on the device
            else:
                turn["slots"][:ng + nd] = slots
                for k, i in enumerate(drawn):
                    turn["temperature"][k] = reqs[i].params.temperature
                    turn["uniform"][k] = reqs[i].rng.next_uniform()
                st["mirror"].copy_(turn["up"], non_blocking=True)
                slots_dev = st["slots"][:ng + nd]
            chosen = st["chosen"]
            if ng:
                rows = logits if ng == n else logits[torch.tensor(greedy, device=logits.device)]
                ops.argmax(chosen[:ng], rows, store=self.fn.token_store, store_index=slots_dev[:ng])
            if nd:
                rows = logits[torch.tensor(drawn, device=logits.device)].contiguous()
                ops.sample(chosen[ng:ng + nd], rows, st["temperature"][:nd], st["uniform"][:nd],
                           store=self.fn.token_store, store_index=slots_dev[ng:ng + nd])
            turn["down"][:ng + nd].copy_(chosen[:ng + nd], non_blocking=True)
            turn["event"].record()
            for i in order:
                reqs[i].on_device = True
            sent = ([(reqs[i].id, reqs[i].preemptions) for i in order], turn["tokens"], ng + nd, turn["event"])
            if not host:
                self._inflight.append(sent)
                return None
        if not host:
            return None
        # the host's chain needs the logits now: this tick is synchronous, every value is returned
        self.collect()
        values = [None] * n
        if order:
            sent[3].synchronize()
            for i, tok in zip(order, sent[1][:sent[2]].tolist()):
                values[i] = int(tok)
        rows = logits[torch.tensor(host, device=logits.device)].cpu().numpy()
        for k, i in enumerate(host):
            r = reqs[i]
            self.sampler.build(rows[k], r.params, r.prompt + r.out)
            values[i] = self.sampler.pick(r.rng.next_uniform()) if not r.params.greedy else int(np.argmax(self.sampler.weights))
            r.on_device = False
        return values

    def collect(self, keep: int = 0) -> None:
        """Read back the tokens that earlier choices sent on their way, oldest first, all but the
        newest ``keep`` sets. A request that was preempted since, or released, no longer takes its token."""
        while len(self._inflight) > keep:
            owed, tokens, n, event = self._inflight.popleft()
            event.synchronize()
            for (rid, life), tok in zip(owed, tokens[:n].tolist()):
                r = self.requests.get(rid)
                if r is not None and r.preemptions == life and r.pending > 0:
                    r.out.append(int(tok))
                    r.pending -= 1

    def flush(self) -> None:
        """Every token chosen so far is in its request's output afterwards."""
        self.collect()

    def settle(self, owes: list, chosen: Optional[list]) -> None:
        """``chosen``: the tokens (one per owing request, None where the value is still on its way) or
        None when all are on their way. Ends requests by count; a token's value is not needed for that."""
        it = iter(chosen) if chosen is not None else None
        for o in owes:
            if o is None:
                continue
            r = self.requests[o]
            tok = next(it) if it is not None else None
            if tok is None:
                r.pending += 1
            else:
                r.out.append(tok)
            if len(r.out) + r.pending >= r.max_new:
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
        """One whole tick; returns the rows that ran. When it returns, the tokens of the tick
        before are in the outputs (all of them with ``run_ahead`` off)."""
        entries, owes = self.prepare()
        self.ticks += 1
        self.last_rows = sum(len(e.tokens) for e in entries)
        if entries:
            wanted = [o for o in owes if o is not None]
            # where every request that is owed a token takes the first maximum, the step chooses by itself
            # (the vocabulary product leaves no logits then)
            by_step = bool(wanted) and all(self.requests[o].params.plain and r_is_greedy(self.requests[o]) for o in wanted)
            result = self.fn.run(entries, greedy=by_step)
            chosen = (self.choose(None, wanted, result) if by_step else self.choose(result, wanted)) if wanted else []
            self.settle(owes, chosen)
            self.collect(keep=1 if self.run_ahead else 0)
        else:
            self.settle([], [])
            self.collect()
        return self.last_rows

    def run(self, max_ticks: int = 1 << 30) -> None:
        n = 0
        while self.has_work():
            if n >= max_ticks:
                raise AlofaError("capacity", "the engine did not finish within the tick limit", f"max_ticks={max_ticks}")
            self.tick()
            n += 1
        self.flush()


def r_is_greedy(r: Request) -> bool:
    return r.params.greedy
