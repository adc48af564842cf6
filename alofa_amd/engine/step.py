"""The step function: one batch of (request, its next tokens) — portions of
prompts beside single decoded tokens, cut anywhere — run as one packed matrix
from the cache that earlier steps left; logits come back at the wanted places
only. Rows of one request are contiguous and in position order; requests lie in
the order given (src/alofa/engine/executor.mojo:555-609 for the row layout,
:665-859 for the pass)."""
from __future__ import annotations

import gc
import os
from dataclasses import dataclass, field
from typing import Optional

import numpy as np
import torch

from .. import ops
from ..cache.manager import CacheManager
from ..errors import AlofaError


def _pow2_ceil(n: int) -> int:
    return max(64, 1 << (int(n) - 1).bit_length())


TOKEN_ON_DEVICE = -1     # as a StepEntry's only token: the token the last choice for this request left on the device


@dataclass
class StepEntry:
    """Next tokens of one request. ``want``: places among these tokens whose
    logits are asked for (may be empty). ``tokens == [TOKEN_ON_DEVICE]``: the one
    token that the last choice for this request wrote to the step function's
    ``token_store`` (``ops.argmax(..., store=)``); it never visits the host."""
    request: object
    tokens: list
    want: list = field(default_factory=list)


@dataclass(frozen=True)
class Span:
    """Where one request's rows lie in the step."""
    request: object
    slot: int        # its request slot (index into per-request state)
    row0: int        # first row in the packed matrix
    n: int           # rows
    pos0: int        # absolute position of the first row


@dataclass
class CacheView:
    """What a mixer sees of its cache in one step."""
    tensors: dict                  # name -> [blocks, *page shape], as the mixer's CacheNeed named them
    block_table: torch.Tensor      # int32 [requests, max_blocks], -1 where no page
    slots: Optional[torch.Tensor]  # int64 [T] cache slot per row (page * page size + place); None for a reader
    owner: bool                    # False: reads another entry's cache, writes nothing
    group: int

    @property
    def k(self) -> torch.Tensor:
        return self.tensors["k"]

    @property
    def v(self) -> torch.Tensor:
        return self.tensors["v"]


KVView = CacheView


class StepContext:
    """Everything the parts need to know about one step."""

    def __init__(self, fn: "StepFunction", spans: list, positions_host: np.ndarray):
        self.fn = fn
        self.spans = spans
        self.positions_host = positions_host
        self.tokens = int(positions_host.shape[0])
        self.max_q_len = max(s.n for s in spans)            # most rows of one request
        # longest context after this step, rounded up to a power of two: it only shapes
        # launches, and a coarse value lets captured decode graphs be used again
        self.max_context = _pow2_ceil(max(s.pos0 + s.n for s in spans))
        self.n_positions = fn.n_positions
        self.entry_slots = self.entry_tokens = None   # request slot and token count per entry, as arrays
        self.positions: torch.Tensor = None
        self.req_of_token: torch.Tensor = None
        self._tables: list = []
        self._slots: list = []
        self._memo: dict = {}
        self.token_store = fn.token_store
        self.request_slots: Optional[torch.Tensor] = None   # int32 [entries] on the device, where the step keeps them there (decode graphs)
        self.want_slots: Optional[torch.Tensor] = None      # int32 [wanted rows] on the device: the request slot behind every wanted row

    @property
    def device(self):
        return self.fn.device

    def scratch(self, name: str, shape: tuple, dtype: torch.dtype) -> torch.Tensor:
        return self.fn.scratch(name, shape, dtype)

    def memo(self, key, build):
        """What a kind of part derives from this step's layout once and uses in every layer
        (how its kernels share the rows out, index tensors): ``build()`` runs at the first call."""
        if key not in self._memo:
            self._memo[key] = build()
        return self._memo[key]

    def kv(self, where) -> CacheView:
        """The cache of the mixer at ``where`` (a run entry, or (entry, k) for the k-th mixer of its block)."""
        where = where if isinstance(where, tuple) else (where, 0)
        owner = self.fn.cache_owner.get(where)
        if owner is None:
            raise AlofaError("invalid_argument", "this mixer keeps no cache", f"where={where}")
        g = self.fn.cache.group_of_entry[owner]
        owns = owner == where
        return CacheView(self.fn.cache.tensors[owner], self._tables[g], self._slots[g] if owns else None, owns, g)

    def state(self, where) -> torch.Tensor:
        """Per-request state of the mixer at ``where``: [max_requests, *shape]; row = Span.slot."""
        where = where if isinstance(where, tuple) else (where, 0)
        return self.fn.cache.state[where]

    def identity_rotation(self, head_dim: int):
        return self.fn.identity_rotation(head_dim)

    def digest(self) -> int:
        """One number for the layout of this step as the kernels will see it (read back from the
        device): which request slot brings which rows at which positions, and per cache group the
        pages behind every request and the slot every row is written to. Equal steps on equal
        caches give equal digests; it is the scheduler digest's arithmetic
        (src/alofa/engine/executor.mojo:980-999 for the step's, scheduler.mojo:463-479 for the folding)."""
        h = 0

        def fold(values):
            nonlocal h
            for x in values:
                h = (h * 1000003 + int(x) + 1) % 2147483647       # + 1: "no page" is -1

        bs = self.fn.cache.block_size
        for s in self.spans:
            fold((s.slot, s.row0, s.n, s.pos0))
        fold(self.positions.cpu().tolist())
        fold(self.req_of_token.cpu().tolist())
        for table, slots in zip(self._tables, self._slots):
            t = table.cpu()
            for i, s in enumerate(self.spans):
                fold(t[i, :(s.pos0 + s.n + bs - 1) // bs].tolist())
            fold(slots.cpu().tolist())
        return h


class StepFunction:
    def __init__(self, model, cache: CacheManager, n_positions: int):
        self.model = model
        self.cache = cache
        self.n_positions = int(n_positions)
        self.device = model.rt.device
        self._scratch: dict = {}
        self._views: dict = {}                   # per set of buffers: (name, dtype, shape) -> (buffer, its view of that shape)
        self._eager_scratch = self._scratch      # buffers of steps that run kernel by kernel
        self._retired: list = []                 # outgrown buffers that captured graphs may still use
        self._eager_hosts: list = []             # pinned blocks the eager steps are laid out in, taking turns
        self._eager_turn = 0
        self._identity: dict = {}
        # the last token chosen for the request in each slot, for choices that stay on the device
        self.token_store = torch.zeros(cache.max_requests, dtype=torch.int32, device=self.device)
        self._chosen = torch.empty(cache.max_requests, dtype=torch.int32, device=self.device)   # what a step that chooses greedily returns
        self.cache_owner = model.cache_owners()      # (entry, k) -> the key of the cache that mixer uses
        self.steps_run = 0
        self.rows_run = 0
        self.last_context: Optional[StepContext] = None
        # decode steps (one token per request) replay a captured HIP graph when every
        # part runs native kernels only; ALOFA_GRAPHS=0 switches that off
        self.use_graphs = os.environ.get("ALOFA_GRAPHS", "1") != "0" and model.capturable
        self._graphs: dict = {}
        self._graph_buffers: dict = {}
        self.graph_replays = 0
        # what must not move once steps run (position tables up to the context bound) is built now
        model.prepare(self.n_positions)

    # ------------------------------------------------------------- scratch
    def scratch(self, name: str, shape: tuple, dtype: torch.dtype) -> torch.Tensor:
        """A named buffer re-used from step to step and layer to layer; it grows
        (outside the steady state) when a step is larger than any before."""
        key = (name, dtype)
        buf = self._scratch.get(key)
        # (every layer asks for the same shapes: a buffer's views are kept beside it, and go when it is replaced)
        views = self._views.setdefault(id(self._scratch), {})
        shape = tuple(shape)
        known = views.get(key)
        if known is not None and known[0] is buf:
            view = known[1].get(shape)
            if view is not None:
                return view
        n = 1
        for s in shape:
            n *= int(s)
        if buf is None or buf.numel() < n:
            if buf is not None and self._scratch is not self._eager_scratch:
                # a captured graph may hold this buffer's address (graphs of one batch size share
                # buffers, and a longer context needs more room for attention's partial results):
                # it is kept for good, so that replays of the older graph write where nothing else lives
                self._retired.append(buf)
            buf = torch.empty(max(n, 1), dtype=dtype, device=self.device)
            self._scratch[key] = buf
        if known is None or known[0] is not buf or len(known[1]) >= 64:
            known = views[key] = (buf, {})
        view = known[1][shape] = buf[:n].view(shape)
        return view

    def scratch_bytes(self) -> int:
        """Bytes of the named buffers (eager steps' and the captured graphs'), retired ones included."""
        bufs = list(self._eager_scratch.values()) + list(self._retired)
        for b in self._graph_buffers.values():
            bufs += list(b["scratch"].values()) + [b["dev"]]
        return sum(t.numel() * t.element_size() for t in bufs)

    def identity_rotation(self, head_dim: int):
        key = head_dim
        if key not in self._identity:
            self._identity[key] = (torch.ones(self.n_positions, head_dim // 2, dtype=torch.float32, device=self.device),
                                   torch.zeros(self.n_positions, head_dim // 2, dtype=torch.float32, device=self.device))
        return self._identity[key]

    # ----------------------------------------------------------------- run
    def plan(self, entries: list):
        """Check a batch (host only, nothing is changed). Returns (request slots, tokens per
        entry, all token ids) as arrays."""
        if not entries:
            raise AlofaError("invalid_argument", "a step needs at least one entry")
        vocab = self.model.spec.vocab_size
        n_tokens = np.fromiter((len(e.tokens) for e in entries), dtype=np.int32, count=len(entries))
        if n_tokens.min() <= 0:
            raise AlofaError("invalid_argument", "an entry brings no tokens", f"request={entries[int(n_tokens.argmin())].request}")
        slots = np.fromiter((self.cache.slot(e.request) for e in entries), dtype=np.int32, count=len(entries))
        ids = np.fromiter((t for e in entries for t in e.tokens), dtype=np.int64, count=int(n_tokens.sum()))
        if ids.min() < 0:
            # a token left on the device: the embedding is told the request's slot, as -(slot + 1)
            starts = np.cumsum(n_tokens) - n_tokens
            carried = ids[starts] == TOKEN_ON_DEVICE
            if (ids < 0).sum() != carried.sum() or (n_tokens[carried] != 1).any():
                raise AlofaError("out_of_range", "token id outside the vocabulary (a token left on the device is an entry's only token)", f"min={ids.min()}")
            ids[starts[carried]] = -(slots[carried].astype(np.int64) + 1)
        if ids.max() >= vocab:
            raise AlofaError("out_of_range", "token id outside the vocabulary", f"vocab={vocab} min={ids.min()} max={ids.max()}")
        for e, n in zip(entries, n_tokens):
            for w in e.want:
                if not 0 <= int(w) < n:
                    raise AlofaError("out_of_range", "wanted place outside the entry's tokens", f"request={e.request} want={w} tokens={n}")
        return slots, n_tokens, ids.astype(np.int32)

    @staticmethod
    def _spans(entries: list, slots, n_tokens, pos0) -> list:
        spans, row = [], 0
        for e, slot, n, p in zip(entries, slots.tolist(), n_tokens.tolist(), pos0.tolist()):
            spans.append(Span(e.request, slot, row, n, p))
            row += n
        return spans

    def begin(self, entries: list):
        """Take the pages the entries need and lay the step out on the device.
        Returns (context, token ids [T] int32, wanted rows or None). Either every
        entry gets its pages or nothing is changed (capacity error)."""
        slots, n_tokens, ids = self.plan(entries)
        cache = self.cache
        n, T, G = len(entries), int(n_tokens.sum()), len(cache.groups)
        want = [(i, int(w)) for i, e in enumerate(entries) for w in e.want]
        width = cache.step_width(slots, n_tokens)
        # one pinned block, laid out in place, and one copy that the host does not wait for:
        # ids, positions, request of every token, wanted rows and their requests' slots, block tables (int32); cache slots (int64)
        n32 = 3 * T + 2 * len(want) + G * n * width
        n32 += n32 % 2
        nbytes = 4 * n32 + 8 * G * T
        host = self._eager_host(nbytes)
        h32, h64 = host["block"][:4 * n32].view(torch.int32).numpy(), host["block"][4 * n32:nbytes].view(torch.int64).numpy()
        at_rows, at_tables = 3 * T, 3 * T + 2 * len(want)
        pos0 = np.empty(n, dtype=np.int64)
        cache.plan_step_into(slots, n_tokens, self.n_positions, pos0, h32[T:2 * T], h32[2 * T:3 * T],
                             h32[at_tables:at_tables + G * n * width].reshape(G, n, width), h64.reshape(G, T))
        h32[:T] = ids
        spans = self._spans(entries, slots, n_tokens, pos0)
        if want:
            h32[at_rows:at_rows + len(want)] = [spans[i].row0 + w for i, w in want]
            h32[at_rows + len(want):at_tables] = [slots[i] for i, _ in want]      # the requests' places in the token store
        ctx = StepContext(self, spans, h32[T:2 * T].copy())
        ctx.entry_slots, ctx.entry_tokens = slots, n_tokens
        block = torch.empty(nbytes, dtype=torch.uint8, device=self.device)
        block.copy_(host["block"][:nbytes], non_blocking=True)
        host["copied"].record()
        d32, d64 = block[:4 * n32].view(torch.int32), block[4 * n32:].view(torch.int64)
        ids_d, ctx.positions, ctx.req_of_token = d32[:T], d32[T:2 * T], d32[2 * T:3 * T]
        tables_d, slots_d = d32[at_tables:at_tables + G * n * width].view(G, n, width), d64.view(G, T)
        ctx._tables = [tables_d[g] for g in range(G)]
        ctx._slots = [slots_d[g] for g in range(G)]
        rows = d32[at_rows:at_rows + len(want)] if want else None
        ctx.want_slots = d32[at_rows + len(want):at_tables] if want else None
        return ctx, ids_d, rows

    def _eager_host(self, nbytes: int) -> dict:
        """The pinned block an eager step is laid out in: three take turns (a block is written again
        only when its last copy has run), and one that is too small is replaced by a bigger one."""
        ring = self._eager_hosts
        if len(ring) < 3:
            ring.append({"block": torch.empty(max(nbytes, 1 << 16), dtype=torch.uint8, pin_memory=True), "copied": torch.cuda.Event()})
            return ring[-1]
        host = ring[self._eager_turn]
        self._eager_turn = (self._eager_turn + 1) % len(ring)
        host["copied"].synchronize()
        if host["block"].numel() < nbytes:
            host["block"] = torch.empty(2 * nbytes, dtype=torch.uint8, pin_memory=True)
        return host

    def finish(self, ctx: StepContext) -> None:
        """The step's tokens are written: lengths advance and pages that a window
        has passed go back to the pool."""
        self.cache.commit_step(ctx.entry_slots, ctx.entry_tokens)
        self.steps_run += 1
        self.rows_run += ctx.tokens

    # ---------------------------------------------------------- decode graphs
    def _decode_buffers(self, B: int) -> dict:
        """Static device buffers of the decode graphs for batch B, and the pinned host blocks that
        are copied over them in one piece before a replay. The host blocks take turns: a step may
        be laid out while the copy of the step before has not run yet (it runs when the GPU gets
        there), so that the host never has to wait for the GPU in order to prepare the next step."""
        if B not in self._graph_buffers:
            W = max(1, (self.n_positions + self.cache.block_size - 1) // self.cache.block_size)
            G = len(self.cache.groups)
            n32 = 4 * B + G * B * W                      # ids, positions, req_of_token, request slots, tables
            n32 += n32 % 2                               # keep the int64 part 8-byte aligned
            nbytes = 4 * n32 + 8 * G * B                 # + cache slots

            def views(block, host):
                b32, b64 = block[:4 * n32].view(torch.int32), block[4 * n32:].view(torch.int64)
                v = {"ids": b32[:B], "positions": b32[B:2 * B], "req_of_token": b32[2 * B:3 * B], "request_slots": b32[3 * B:4 * B],
                     "tables": b32[4 * B:4 * B + G * B * W].view(G, B, W), "slots": b64.view(G, B)}
                return {k: t.numpy() for k, t in v.items()} if host else v
            devb = torch.empty(nbytes, dtype=torch.uint8, device=self.device)
            buf = {"dev": devb, "W": W, "scratch": {}, "turn": 0, "hosts": [], **views(devb, False),
                   "rows": torch.arange(B, dtype=torch.int32, device=self.device)}
            for _ in range(3):
                host = torch.empty(nbytes, dtype=torch.uint8, pin_memory=True)
                buf["hosts"].append({"block": host, "copied": torch.cuda.Event(), **views(host, True)})
                buf["hosts"][-1]["req_of_token"][:] = np.arange(B, dtype=np.int32)
            self._graph_buffers[B] = buf
        return self._graph_buffers[B]

    def _run_decode_graph(self, entries: list, greedy: bool = False) -> torch.Tensor:
        slots, n_tokens, ids = self.plan(entries)
        cache = self.cache
        B = len(entries)
        buf = self._decode_buffers(B)
        host = buf["hosts"][buf["turn"]]
        buf["turn"] = (buf["turn"] + 1) % len(buf["hosts"])
        host["copied"].synchronize()                     # this block's last copy (three steps ago) is done
        pos0 = np.empty(B, dtype=np.int64)
        # the layout goes straight into the pinned block that is copied to the device in one piece
        cache.plan_step_into(slots, n_tokens, self.n_positions, pos0, host["positions"], host["req_of_token"], host["tables"], host["slots"])
        host["ids"][:] = ids
        host["request_slots"][:] = slots
        spans = self._spans(entries, slots, n_tokens, pos0)
        ctx = StepContext(self, spans, host["positions"].copy())
        ctx.entry_slots, ctx.entry_tokens = slots, n_tokens
        ctx.positions, ctx.req_of_token = buf["positions"], buf["req_of_token"]
        ctx.request_slots = buf["request_slots"]
        ctx._tables = [buf["tables"][g] for g in range(len(cache.groups))]
        ctx._slots = [buf["slots"][g] for g in range(len(cache.groups))]
        buf["dev"].copy_(host["block"], non_blocking=True)
        host["copied"].record()
        ctx.want_slots = buf["request_slots"]
        key = (B, ctx.max_context, greedy)
        saved, self._scratch = self._scratch, buf["scratch"]   # graphs of one batch size share their own buffers
        chosen = self._chosen[:B]

        def outcome(hidden):      # logits of every row, or (greedy) only each row's first maximum, which also goes to the token store
            if greedy:
                self.model.greedy(ctx, hidden, buf["rows"], chosen, self.token_store, buf["request_slots"])
                return chosen
            return self.model.logits(ctx, hidden, buf["rows"])
        try:
            if key not in self._graphs:
                # once eagerly, so that every buffer exists before the capture and the
                # step's result does not depend on the capture itself
                hidden = self.model.forward(ctx, buf["ids"])
                logits = outcome(hidden)
                torch.cuda.current_stream().synchronize()
                graph = torch.cuda.CUDAGraph()
                # No garbage collection while the stream is capturing: a collected object that owns device
                # or pinned memory, an event or an older graph (a step function that went out of use, for
                # one: it and its last context refer to each other) frees it with calls that a capturing
                # stream forbids, and an error in a destructor ends the process. What is garbage already
                # goes before the capture begins.
                collecting = gc.isenabled()
                gc.collect()
                gc.disable()
                try:
                    with torch.cuda.graph(graph), ops.stream_scope():
                        hidden = self.model.forward(ctx, buf["ids"])
                        captured = outcome(hidden)
                finally:
                    if collecting:
                        gc.enable()
                if captured.data_ptr() != logits.data_ptr():
                    raise AlofaError("invalid_argument", "a buffer moved between the eager run and the capture")
                self._graphs[key] = (graph, captured)
                # the capture itself ran nothing: the eager results stand
            else:
                graph, logits = self._graphs[key]
                graph.replay()
                self.graph_replays += 1
        finally:
            self._scratch = saved
        self.finish(ctx)
        self.last_context = ctx
        return logits

    def run(self, entries: list, greedy: bool = False) -> Optional[torch.Tensor]:
        """Run the step. Returns float32 logits [wanted, vocab] on the device in
        the order of the entries and of their ``want`` lists, or None when nothing
        is wanted. With ``greedy`` the step chooses by itself: it returns, instead of
        the logits, int32 [wanted] with the first index of every wanted row's highest
        logit, and leaves the same in the token store at the row's request's slot.
        The buffer is re-used by the next step."""
        with ops.stream_scope():
            if self.use_graphs and all(len(e.tokens) == 1 and list(e.want) == [0] for e in entries):
                return self._run_decode_graph(entries, greedy)
            ctx, ids, rows = self.begin(entries)
            hidden = self.model.forward(ctx, ids)
            out = None
            if rows is not None and greedy:
                out = self._chosen[:rows.shape[0]]
                self.model.greedy(ctx, hidden, rows, out, self.token_store, ctx.want_slots)
            elif rows is not None:
                out = self.model.logits(ctx, hidden, rows)
            self.finish(ctx)
            self.last_context = ctx
            return out
