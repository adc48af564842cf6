"""Trace replay: feeds given token ids through a model step by step and writes
logits; it samples nothing. It drives the engine's own model, step function,
cache and kernels — the ones generation uses.

    bin/trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N [--blocks N] [--window-blocks N]

Steps come on standard input, one JSON object a line:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

For a step in which something is wanted, ``DIR/<step>.f32`` receives the logits
at the wanted places ([wanted, vocab] little-endian float32, in the order of the
entries and of ``want``), and ``DIR/<step>.tsv`` one line ``request<TAB>position``
per row of them (the position counts from the request's first token), so that
outputs of different cuttings can be compared position by position without the
input. After every step a line ``done <step>`` is printed.

The cache pool is made for ``--max-tokens`` tokens, or, with ``--blocks``, of so
many pages; ``--window-blocks`` gives the pools of layers that see only a window
of keys a size of their own.

A request's first entry may start on pages another live request has filled:

    {"id": "b", "share": {"from": "a", "tokens": 32}, "tokens": [...from position 0...], "want": [40]}

``tokens`` then holds b's tokens from its first one, of which up to 32 must equal
a's. The whole pages among them that a has written are held by both requests from
then on (by reference count) and their arithmetic is skipped: they are b's
history. At least b's last token of the entry is always computed
(src/alofa/engine/executor.mojo:459-479), b writes its own tokens to fresh pages
only (src/alofa/runtime/kv/__init__.mojo:24-30), and a may end before b. Places
in ``want`` count from the entry's first token and must lie beyond what was
shared. A model whose layers see only a window of keys, or that carries state,
shares nothing and computes everything."""
from __future__ import annotations

import argparse
import json
import sys
from pathlib import Path
from typing import Optional

from .errors import AlofaError


class Replayer:
    """The replay loop as an object: one ``step`` per input line."""

    def __init__(self, model_dir, dtype: str, max_tokens: int, block_size: int = 16, device: str = "cuda:0",
                 blocks: Optional[int] = None, window_blocks: Optional[int] = None):
        """``blocks``: pages of every pool (default: what ``max_tokens`` tokens take); ``window_blocks``: pages of
        the pools of groups of layers that see a window only, when they are to differ."""
        from .csrc.build import load
        load()  # compile at the first call if nothing is built; fail loudly if it cannot
        from .cache.manager import CacheManager
        from .engine.step import StepFunction
        from .model import load_model

        self.config, self.model = load_model(model_dir, dtype, device)
        n_blocks = int(blocks) if blocks is not None else max(1, (int(max_tokens) + block_size - 1) // block_size)
        needs = self.model.cache_needs()
        if window_blocks is not None:
            n_blocks = {w: n_blocks if w is None else int(window_blocks) for w in CacheManager.windows_of(needs)}
        self.cache = CacheManager(needs, self.model.state_needs(), n_blocks, block_size,
                                  max_requests=8, device=self.model.rt.device, dtype=self.model.rt.dtype)
        # the position table is as long as a request can get here, not the checkpoint's
        # max_position_embeddings, which the reference does not read (qwen.mojo:849)
        self.fn = StepFunction(self.model, self.cache, n_positions=max(int(max_tokens), 64))
        self.tokens: dict = {}       # request -> the tokens it has been given so far
        self.shared: dict = {}       # request -> tokens it took over from another request's pages
        self.last_index: list = []   # (request, position) of every row of the last step's logits

    def step(self, rec: dict):
        """Run one step record; returns float32 logits [wanted, vocab] as a NumPy
        array, or None when nothing is wanted."""
        from .engine.step import StepEntry
        entries = []
        for e in rec.get("entries", []):
            tokens, want = [int(t) for t in e["tokens"]], [int(w) for w in e.get("want", [])]
            if "share" in e:
                skipped = self._share(e["id"], e["share"], tokens)
                if any(w < skipped for w in want):
                    self.cache.free(e["id"])
                    del self.tokens[e["id"]]
                    raise AlofaError("out_of_range", "a wanted place lies in the shared prefix, which is not computed",
                                     f"request={e['id']} shared={skipped} want={min(want)}")
                tokens, want = tokens[skipped:], [w - skipped for w in want]
            elif not self.cache.has(e["id"]):
                self.cache.admit(e["id"])
                self.tokens[e["id"]] = []
            entries.append(StepEntry(e["id"], tokens, want))
        out = None
        self.last_index = [(e.request, len(self.tokens[e.request]) + w) for e in entries for w in e.want]
        if entries:
            logits = self.fn.run(entries)
            for e in entries:
                self.tokens[e.request].extend(e.tokens)
            if logits is not None:
                out = logits.detach().cpu().numpy().astype("<f4")
        for r in rec.get("end", []):
            if self.cache.has(r):
                self.cache.free(r)
                del self.tokens[r]
        return out

    def _share(self, req, share: dict, tokens: list) -> int:
        """Start ``req`` on the pages of ``share["from"]``; returns how many of ``tokens`` are
        its history from now on."""
        src, n = share["from"], int(share["tokens"])
        if self.cache.has(req):
            raise AlofaError("invalid_argument", "only a request's first entry can share a prefix", f"request={req}")
        if not self.cache.has(src):
            raise AlofaError("invalid_argument", "the request to share with is not live", f"request={req} from={src}")
        if n < 0 or n > len(tokens) or tokens[:n] != self.tokens[src][:n]:
            raise AlofaError("invalid_argument", "the tokens to share are not the other request's first tokens", f"request={req} from={src} tokens={n}")
        self.cache.admit(req)
        # the entry's last token is always computed: its logits are what the request speaks from
        skipped = self.cache.share_prefix(src, req, min(n, len(tokens) - 1))
        self.tokens[req] = tokens[:skipped]
        self.shared[req] = skipped
        return skipped


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time (each request rounded up to a multiple of 64)")
    ap.add_argument("--block-size", type=int, default=16, help="tokens per cache page")
    ap.add_argument("--blocks", type=int, default=None, help="pages of the cache pool, instead of what --max-tokens tokens take")
    ap.add_argument("--window-blocks", type=int, default=None, help="pages of the pools of layers that see a window only (default: as the others)")
    args = ap.parse_args(argv)
    out = Path(args.out)
    out.mkdir(parents=True, exist_ok=True)
    replayer = Replayer(args.model, args.dtype, args.max_tokens, args.block_size, blocks=args.blocks, window_blocks=args.window_blocks)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        logits = replayer.step(rec)
        if logits is not None:
            logits.tofile(out / f"{rec['step']}.f32")
            (out / f"{rec['step']}.tsv").write_text("".join(f"{r}\t{p}\n" for r, p in replayer.last_index))
        print(f"done {rec['step']}", flush=True)
    return 0


if __name__ == "__main__":
    try:
        sys.exit(main())
    except AlofaError as e:
        print(f"trace_run: {e}", file=sys.stderr)
        sys.exit(1)
