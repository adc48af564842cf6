"""The plain path: the whole model on the host in formula order (float32 storage,
float64 accumulation, contiguous keys and values), the oracle inside the library
that the engine's exact path is held against; it needs no GPU. The arithmetic is
C++ (csrc/host/plain.cpp, after src/alofa/kernels/cpu/scalar.mojo and the forward
pass src/alofa/model/arch/qwen.mojo:1362-1525 of the reference); this class loads
the tensors by name, widens bfloat16 exactly, and hands them over.

It serves the one architecture whose formulas it transcribes (Qwen2ForCausalLM);
any other configuration is refused by name."""
from __future__ import annotations

import ctypes
from pathlib import Path

import numpy as np
import torch

from .config.registry import load_config
from .csrc import hostlib
from .errors import AlofaError
from .model import expected_tensors
from .models.qwen2 import Qwen2Config
from .weights.loader import load_weights


class PlainModel:
    """``run(ids)`` extends the stored history by ``ids`` and returns the logits of every new
    position (float32 [len(ids), vocab]); ``reset()`` forgets the history."""

    def __init__(self, model_dir, max_tokens: int = 512):
        cfg = load_config(Path(model_dir))
        if not isinstance(cfg, Qwen2Config):
            raise AlofaError("unsupported", "the plain path transcribes the Qwen2 formulas only", f"architecture={type(cfg).__name__}")
        self.config, self.max_tokens = cfg, int(max_tokens)
        weights = load_weights(Path(model_dir), expected_tensors(cfg.spec()))
        self._lib = hostlib.lib()
        self._lib.alofa_plain_new.restype = ctypes.c_void_p
        self._lib.alofa_plain_last_error.restype = ctypes.c_char_p
        sizes = hostlib.long_array([cfg.num_hidden_layers, cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim,
                                    cfg.intermediate_size, cfg.vocab_size, int(cfg.tie_word_embeddings), self.max_tokens])
        windows = hostlib.long_array([cfg.window_of(i) or 0 for i in range(cfg.num_hidden_layers)])
        self._h = ctypes.c_void_p(self._lib.alofa_plain_new(sizes, ctypes.c_double(cfg.rms_norm_eps), ctypes.c_double(cfg.rope_theta), windows))
        if not self._h:
            raise AlofaError("invalid_argument", "the plain model refused its sizes", self._lib.alofa_plain_last_error().decode())
        # float32 copies that live as long as the model (bfloat16 widens exactly)
        self._kept = {n: t.to(torch.float32).contiguous().numpy() for n, t in weights.items()}
        for name, a in self._kept.items():
            self._lib.alofa_plain_set_tensor(self._h, name.encode(), a.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), ctypes.c_int64(a.size))

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.alofa_plain_free(self._h)
            self._h = None

    def reset(self) -> None:
        self._lib.alofa_plain_reset(self._h)

    def __len__(self) -> int:
        return self._lib.alofa_plain_length(self._h)

    def run(self, ids, all_rows: bool = True) -> np.ndarray:
        ids = np.ascontiguousarray(ids, dtype=np.int32)
        rows = len(ids) if all_rows else 1
        out = np.empty((rows, self.config.vocab_size), dtype=np.float32)
        rc = self._lib.alofa_plain_run(self._h, ids.ctypes.data_as(ctypes.POINTER(ctypes.c_int)), len(ids), int(all_rows),
                                       out.ctypes.data_as(ctypes.POINTER(ctypes.c_float)))
        if rc < 0:
            text = self._lib.alofa_plain_last_error().decode()
            name = "out_of_range" if "outside" in text or "exceed" in text else "invalid_argument"
            raise AlofaError(name, *text.partition(" [")[::2])
        return out

    def greedy(self, prompt, n_new: int) -> list:
        """Greedy continuation from a fresh history: the prompt whole, then token by token
        (the first maximum, lowest index on ties: src/alofa/model/arch/qwen.mojo:1527-1541)."""
        self.reset()
        out, feed = [], list(prompt)
        for _ in range(n_new):
            row = self.run(feed, all_rows=False)[0]
            tok = int(self._lib.alofa_plain_argmax(row.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), row.shape[0]))
            out.append(tok)
            feed = [tok]
        return out
