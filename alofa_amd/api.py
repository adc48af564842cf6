"""Python entry point: an engine over a model folder that generates tokens for
batches of prompts (token ids; the tokenizer is outside this engine)."""
from __future__ import annotations

import os
import sys
from pathlib import Path
from typing import Optional

from .cache.manager import CacheManager
from .engine.core import EngineCore
from .engine.scheduler import SchedConfig
from .engine.step import StepFunction
from .errors import AlofaError
from .model import load_model
from .sampling.sampler import SampleParams


class Engine:
    """``max_tokens`` is the context window of one request (prompt + generated),
    as the reference's ALOFA_MAX_TOKENS (src/alofa/srv/config.mojo:94-97).
    ``kv_blocks`` pages of ``block_size`` tokens make the pool of a group of layers that
    keeps every key, by default enough for ``max_batch`` requests of ``max_tokens``; a group
    whose layers see a window only gets what ``max_batch`` requests can hold of it (the
    window, a step's tokens and two pages each), never more than ``kv_blocks``. A dict
    from a group's window (None: every key) to its pages sets every pool by hand. With
    ``share_prefixes`` a new request starts on the whole pages a resident request has
    written for the same first tokens (src/alofa/runtime/kv/space.mojo:166-243, block by block)."""

    def __init__(self, model_dir, dtype: str = "bfloat16", max_tokens: int = 256, max_batch: int = 8,
                 kv_blocks: Optional[int] = None, block_size: int = 16, token_budget: int = 2048, max_chunk: Optional[int] = None,
                 watermark_permille: int = 900, max_wait_ticks: int = 8, seed: int = 1234, device: str = "cuda:0",
                 trace_path=None, share_prefixes: bool = False, model=None, report=None, run_ahead: bool = True,
                 memory_fraction: Optional[float] = None):
        """``model``: a (config, Model) pair already on the device, instead of a folder to load.
        ``report``: a callable that receives one line about device memory at start (default:
        standard error when ALOFA_REPORT_MEMORY is set). ``run_ahead``: a tick reads the tokens of the
        tick before only after its own step is launched (``EngineCore``); off, every tick is synchronous.
        ``memory_fraction`` (with no ``kv_blocks``): the pool of the layers that keep every key takes this share
        of the device memory that is free once the weights are loaded (less what the windowed layers' pools take),
        instead of what ``max_batch`` requests of ``max_tokens`` need.
        ``max_chunk``: the most prompt tokens of one request in a tick; by default the whole ``token_budget``,
        so that a lone long prompt takes one step (requests are served in order of arrival either way, and the
        budget alone bounds a tick's length)."""
        max_chunk = token_budget if max_chunk is None else max_chunk
        from .csrc.build import load
        load()
        self.config, self.model = model if model is not None else load_model(Path(model_dir), dtype, device)
        if max_tokens > self.model.spec.max_positions:
            raise AlofaError("out_of_range", "max_tokens passes the model's position bound", f"max_tokens={max_tokens} max_position_embeddings={self.model.spec.max_positions}")
        needs = self.model.cache_needs()
        if not isinstance(kv_blocks, dict):
            def under_watermark(pages):      # enough for max_batch such requests below the scheduler's watermark
                return (pages * 1000 + watermark_permille - 1) // watermark_permille + 1
            own = {w: under_watermark(CacheManager.pages_for(w, max_batch, max_tokens, max_chunk, block_size))
                   for w in CacheManager.windows_of(needs)}
            if kv_blocks is None and memory_fraction is not None:
                kv_blocks = self._pages_that_fit(needs, own, memory_fraction, block_size)
            kv_blocks = {w: n if kv_blocks is None else (int(kv_blocks) if w is None else min(int(kv_blocks), n)) for w, n in own.items()}
        self.cache = CacheManager(needs, self.model.state_needs(), kv_blocks, block_size,
                                  max_requests=max(32, max_batch), device=self.model.rt.device, dtype=self.model.rt.dtype)
        self.step_fn = StepFunction(self.model, self.cache, n_positions=max_tokens)
        # (the scheduler counts a request's pages in every group of layers by what that group holds of it:
        # everything, or a window and a step's tokens; the group that binds decides)
        self.sched_cfg = SchedConfig.for_groups(self.cache.group_rules(max_chunk), token_budget=token_budget, max_chunk=max_chunk,
                                                block_size=block_size, watermark_permille=watermark_permille,
                                                max_wait_ticks=max_wait_ticks, n_slots=max(32, max_batch))
        self.core = EngineCore(self.step_fn, self.sched_cfg, trace_path, share_prefixes=share_prefixes, run_ahead=run_ahead)
        self.seed = seed
        self._next_id = 1
        if report is None and os.environ.get("ALOFA_REPORT_MEMORY"):
            report = lambda line: print(line, file=sys.stderr, flush=True)   # noqa: E731
        if report is not None:
            m = self.memory()
            report(f"[alofa_amd] device memory: weights {m['weights'] / 2**20:.1f} MiB + cache pool {m['cache_pool'] / 2**20:.1f} MiB "
                   f"({' + '.join(str(g.pool.n_blocks) for g in self.cache.groups) or 0} pages of {block_size} tokens in {len(self.cache.groups)} group(s)) + scratch {m['scratch'] / 2**20:.1f} MiB "
                   f"(grows to the largest step, then stays) = {m['total'] / 2**20:.1f} MiB")

    def _pages_that_fit(self, needs, own: dict, fraction: float, block_size: int) -> int:
        """Pages for the pool of the layers that keep every key: what ``fraction`` of the free device memory holds
        beside the windowed layers' pools (sized by their windows: ``own``)."""
        import torch
        if not 0.0 < fraction <= 1.0:
            raise AlofaError("invalid_argument", "memory_fraction lies in (0, 1]", f"memory_fraction={fraction}")
        per_page = CacheManager.page_bytes(needs, block_size, self.model.rt.dtype)
        free = torch.cuda.mem_get_info(self.model.rt.device)[0]
        left = int(free * fraction) - sum(own[w] * b for w, b in per_page.items() if w is not None)
        pages = left // per_page[None] if None in per_page else 1
        if pages <= 0:
            raise AlofaError("capacity", "the cache pool does not fit the device memory that is free", f"free={free} fraction={fraction}")
        return int(min(pages, (1 << 31) - 1))

    def memory(self) -> dict:
        """Bytes of device memory by use: the rule is weights + cache pool + scratch, nothing else
        (the reference's gate is resident memory <= 1.15 x weights, tests/unit/test_memory_gate.mojo:49-50)."""
        weights, pool, scratch = self.model.weight_bytes(), self.cache.device_bytes(), self.step_fn.scratch_bytes()
        return {"weights": weights, "cache_pool": pool, "scratch": scratch, "total": weights + pool + scratch}

    def generate(self, prompts: list, max_new: int = 16, temperature: float = 0.0, top_k: int = 0, top_p: float = 1.0,
                 min_p: float = 0.0, repetition_penalty: float = 1.0, frequency_penalty: float = 0.0,
                 presence_penalty: float = 0.0, seed: Optional[int] = None, max_ticks: int = 1 << 30) -> list:
        """Greedy (temperature 0) or sampled continuation of every prompt; every
        request draws from its own generator seeded with ``seed``."""
        params = SampleParams(temperature=temperature, top_k=top_k, top_p=top_p, min_p=min_p,
                              repetition_penalty=repetition_penalty, frequency_penalty=frequency_penalty,
                              presence_penalty=presence_penalty)
        use_seed = self.seed if seed is None else seed
        ids, waiting = [], []
        for p in prompts:
            ids.append(self._next_id)
            waiting.append((self._next_id, list(p)))
            self._next_id += 1
        ticks = 0
        while waiting or self.core.has_work():
            # requests the watermark cannot hold yet wait here until earlier ones end
            while waiting and self.core.can_admit(len(waiting[0][1]), max_new):
                rid, p = waiting.pop(0)
                self.core.submit(rid, p, max_new, params, use_seed)
            if not self.core.has_work():
                raise AlofaError("capacity", "a request can never be admitted: it does not fit under the kv watermark",
                                 f"prompt={len(waiting[0][1])} max_new={max_new}")
            self.core.tick()
            ticks += 1
            if ticks > max_ticks:
                raise AlofaError("capacity", "generation did not finish within the tick limit", f"max_ticks={max_ticks}")
        self.core.flush()
        outs = {}
        for rid in ids:
            outs[rid] = self.core.output(rid)
            self.core.release(rid)
        return [outs[rid] for rid in ids]
