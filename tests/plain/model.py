"""Plain Qwen2 decoder: whole sequences, no cache, float32 storage with
float64 accumulation and one rounding where the reference rounds.

Paths cited are relative to the reference checkout.
"""
from __future__ import annotations

import json
import math
from pathlib import Path

import numpy as np

F32 = np.float32
F64 = np.float64
LOWEST_FP32 = F32(-3.4028234663852886e38)  # src/alofa/kernels/cpu/scalar.mojo:32-35


def read_config(model_dir) -> dict:
    """The keys the reference reads and their rules
    (src/alofa/model/arch/qwen.mojo:939-954, :977-994), plus the window keys
    that the engine adds (absent in the reference, which ignores them)."""
    raw = json.loads((Path(model_dir) / "config.json").read_text())
    cfg = {
        "L": int(raw["num_hidden_layers"]),
        "h": int(raw["hidden_size"]),
        "H": int(raw["num_attention_heads"]),
        "Hkv": int(raw["num_key_value_heads"]),
        "I": int(raw["intermediate_size"]),
        "V": int(raw["vocab_size"]),
        "eps": float(raw["rms_norm_eps"]),
        "theta": float(raw["rope_theta"]),
        "tied": bool(raw["tie_word_embeddings"]),
    }
    cfg["d"] = int(raw["head_dim"]) if "head_dim" in raw else cfg["h"] // cfg["H"]
    cfg["windows"] = [None] * cfg["L"]
    if raw.get("use_sliding_window", False):
        first = int(raw.get("max_window_layers", cfg["L"]))
        for i in range(first, cfg["L"]):
            cfg["windows"][i] = int(raw["sliding_window"])
    return cfg


def read_weights(model_dir) -> dict:
    """name -> float32 array. bfloat16 widens exactly
    (src/alofa/model/safetensors.mojo:123-137). Read with the safetensors
    library, which the engine's own reader does not use."""
    import torch
    from safetensors.torch import load_file

    out = {}
    for name, t in load_file(str(Path(model_dir) / "model.safetensors")).items():
        out[name] = t.to(torch.float32).numpy()
    return out


# --------------------------------------------------------------------- parts

def embed(table: np.ndarray, ids) -> np.ndarray:
    """hidden[r] = E[id_r], no scaling (src/alofa/model/arch/qwen.mojo:1391-1413)."""
    ids = np.asarray(ids, dtype=np.int64)
    if ids.min() < 0 or ids.max() >= table.shape[0]:
        raise IndexError("token id outside the vocabulary")
    return table[ids].astype(F32)


def rmsnorm(x: np.ndarray, w: np.ndarray, eps: float) -> np.ndarray:
    """y = x * 1/sqrt(mean(x^2) + eps) * w, float64 inside, eps as float32
    inside the root, weight after the scale, no 1+w
    (src/alofa/kernels/cpu/scalar.mojo:93-129)."""
    x64 = x.astype(F64)
    ss = (x64 * x64).sum(axis=-1, keepdims=True)
    scale = 1.0 / np.sqrt(ss / x.shape[-1] + F64(F32(eps)))
    return (x64 * scale * w.astype(F64)).astype(F32)


def linear(x: np.ndarray, w: np.ndarray, b: np.ndarray | None = None) -> np.ndarray:
    """y = x @ w.T (+ b), w stored [out, in], float64 accumulator that starts
    at the bias (src/alofa/kernels/cpu/scalar.mojo:132-193)."""
    acc = x.astype(F64) @ w.astype(F64).T
    if b is not None:
        acc = b.astype(F64) + acc
    return acc.astype(F32)


def rope_table(n_pos: int, d: int, theta: float):
    """cos/sin [n_pos, d]: inv = f32(1)/f32(pow(theta, 2i/d)); angle = f32(pos)*inv
    in float32; cos and sin taken in float64, rounded once; both halves equal
    (src/alofa/model/arch/qwen.mojo:830-880)."""
    half = d // 2
    inv = np.empty(half, dtype=F32)
    for i in range(half):
        inv[i] = F32(1.0) / F32(math.pow(theta, (2.0 * i) / d))
    pos = np.arange(n_pos, dtype=F32)[:, None]
    ang = (pos * inv[None, :]).astype(F32)
    c = np.cos(ang.astype(F64)).astype(F32)
    s = np.sin(ang.astype(F64)).astype(F32)
    return np.concatenate([c, c], axis=1), np.concatenate([s, s], axis=1)


def rope_apply(x: np.ndarray, cos: np.ndarray, sin: np.ndarray, positions, d: int) -> np.ndarray:
    """Half-split rotation of every head of x [T, heads*d] in float32:
    out[j] = x[j]*cos[p,j] - x[j+d/2]*sin[p,j];
    out[j+d/2] = x[j+d/2]*cos[p,j+d/2] + x[j]*sin[p,j+d/2]
    (src/alofa/kernels/cpu/scalar.mojo:283-344; position per row
    src/alofa/kernels/cpu/segments.mojo:48-130)."""
    T = x.shape[0]
    heads = x.shape[1] // d
    half = d // 2
    xs = x.reshape(T, heads, d).astype(F32)
    p = np.asarray(positions, dtype=np.int64)
    c = cos[p][:, None, :].astype(F32)
    s = sin[p][:, None, :].astype(F32)
    a = xs[:, :, :half]
    b = xs[:, :, half:]
    lo = (a * c[:, :, :half]).astype(F32) - (b * s[:, :, :half]).astype(F32)
    hi = (b * c[:, :, half:]).astype(F32) + (a * s[:, :, half:]).astype(F32)
    return np.concatenate([lo, hi], axis=2).astype(F32).reshape(T, heads * d)


def attention(q, k, v, H: int, Hkv: int, d: int, window: int | None = None) -> np.ndarray:
    """Causal grouped-query attention of q [n, H*d] over k, v [L, Hkv*d]; query
    row t stands at position L-n+t and sees keys 0..position. Key head =
    query head // (H/Hkv). Dot in float64 rounded to float32, then times
    float32 1/sqrt(d); max and exp in float32; the sum of the weights and the
    weighted sum of v in float64; one division per channel at the end
    (src/alofa/kernels/cpu/scalar.mojo:392-470, same body in
    src/alofa/kernels/cpu/paged.mojo:249-336).
    ``window`` (not in the reference): only the last ``window`` keys up to and
    including the query's own position are seen."""
    n, L = q.shape[0], k.shape[0]
    assert n <= L
    g = H // Hkv
    scale = F32(1.0) / np.sqrt(F32(d))
    out = np.zeros((n, H * d), dtype=F32)
    k64 = k.astype(F64)
    v64 = v.astype(F64)
    for head in range(H):
        kh = head // g
        kk = k64[:, kh * d:(kh + 1) * d]
        vv = v64[:, kh * d:(kh + 1) * d]
        for t in range(n):
            pos = L - n + t
            lo = 0 if window is None else max(0, pos - window + 1)
            qv = q[t, head * d:(head + 1) * d].astype(F64)
            s = ((kk[lo:pos + 1] @ qv).astype(F32) * scale).astype(F32)
            m = max(LOWEST_FP32, s.max())
            e = np.exp((s - m).astype(F32)).astype(F32)
            z = e.astype(F64).sum()
            out[t, head * d:(head + 1) * d] = ((e.astype(F64) @ vv[lo:pos + 1]) / z).astype(F32)
    return out


def silu(x: np.ndarray) -> np.ndarray:
    """x / (1 + exp(-x)) in float64 (src/alofa/kernels/cpu/scalar.mojo:208-216)."""
    v = x.astype(F64)
    with np.errstate(over="ignore"):
        return (v / (1.0 + np.exp(-v))).astype(F32)


def swiglu(gate: np.ndarray, up: np.ndarray) -> np.ndarray:
    """silu(gate) * up with the product in float64
    (src/alofa/kernels/cpu/scalar.mojo:219-231)."""
    v = gate.astype(F64)
    with np.errstate(over="ignore"):
        return (v / (1.0 + np.exp(-v)) * up.astype(F64)).astype(F32)


def add(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """Residual sum in float32 (src/alofa/kernels/cpu/scalar.mojo:196-205)."""
    return (a.astype(F32) + b.astype(F32)).astype(F32)


# --------------------------------------------------------------- whole model
# ``store`` (not in the reference, whose activations are all float32): a function applied to every
# activation that an engine with narrower activations keeps in memory between two operators (the
# normed stream, q, k and v, rotated q and k, the attention output, the activated feed-forward
# product); the residual stream and all sums stay as they are. With it the plain model shows how
# far rounding the activations alone moves the logits, which is what a tolerance for such an
# engine has to be measured against.

def _keep(x):
    return x


def attention_block(w, cfg, i, x, cos, sin, positions, store=_keep):
    """q, k, v with bias; rotate q and k, not v; attend; output projection
    without bias (src/alofa/model/arch/qwen.mojo:1429-1480)."""
    p = f"model.layers.{i}.self_attn."
    q = store(linear(x, w[p + "q_proj.weight"], w[p + "q_proj.bias"]))
    k = store(linear(x, w[p + "k_proj.weight"], w[p + "k_proj.bias"]))
    v = store(linear(x, w[p + "v_proj.weight"], w[p + "v_proj.bias"]))
    q = store(rope_apply(q, cos, sin, positions, cfg["d"]))
    k = store(rope_apply(k, cos, sin, positions, cfg["d"]))
    a = store(attention(q, k, v, cfg["H"], cfg["Hkv"], cfg["d"], cfg["windows"][i]))
    return linear(a, w[p + "o_proj.weight"])


def feed_forward(w, cfg, i, x, store=_keep):
    """down(silu(gate(x)) * up(x)), no biases
    (src/alofa/engine/executor.mojo:806-837)."""
    p = f"model.layers.{i}.mlp."
    g = linear(x, w[p + "gate_proj.weight"])
    u = linear(x, w[p + "up_proj.weight"])
    return linear(store(swiglu(g, u)), w[p + "down_proj.weight"])


def decoder_block(w, cfg, i, hidden, cos, sin, positions, store=_keep):
    """Pre-norm block with two residual sums
    (src/alofa/model/arch/qwen.mojo:1418-1510)."""
    p = f"model.layers.{i}."
    n1 = store(rmsnorm(hidden, w[p + "input_layernorm.weight"], cfg["eps"]))
    hidden = add(hidden, attention_block(w, cfg, i, n1, cos, sin, positions, store))
    n2 = store(rmsnorm(hidden, w[p + "post_attention_layernorm.weight"], cfg["eps"]))
    return add(hidden, feed_forward(w, cfg, i, n2, store))


def output_matrix(w, cfg):
    """lm_head.weight if the file has it, else the embedding when tied, else an
    error (src/alofa/model/arch/qwen.mojo:1080-1089)."""
    if "lm_head.weight" in w:
        return w["lm_head.weight"]
    if cfg["tied"]:
        return w["model.embed_tokens.weight"]
    raise KeyError("no output matrix: lm_head.weight is absent and the embedding is not tied")


def to_bfloat16(x: np.ndarray) -> np.ndarray:
    """x rounded to the nearest bfloat16 (ties to even), as float32: a ``store`` for the plain model."""
    bits = np.ascontiguousarray(x, dtype=F32).view(np.uint32).astype(np.uint64)
    rounded = ((bits + 0x7FFF + ((bits >> 16) & 1)) >> 16) << 16
    return rounded.astype(np.uint32).view(F32).reshape(np.shape(x))


def forward_logits(w, cfg, ids, first_position: int = 0, store=_keep) -> np.ndarray:
    """Logits [len(ids), V] at every position of one sequence whose first token
    stands at ``first_position`` (0 in the reference; another value only shifts
    the rotary angles) (src/alofa/model/arch/qwen.mojo:1362-1525)."""
    T = len(ids)
    positions = np.arange(first_position, first_position + T)
    cos, sin = rope_table(first_position + T, cfg["d"], cfg["theta"])
    hidden = embed(w["model.embed_tokens.weight"], ids)
    for i in range(cfg["L"]):
        hidden = decoder_block(w, cfg, i, hidden, cos, sin, positions, store)
    y = store(rmsnorm(hidden, w["model.norm.weight"], cfg["eps"]))
    return linear(y, output_matrix(w, cfg))


def argmax(row: np.ndarray) -> int:
    """First maximum: strict >, lowest index wins ties
    (src/alofa/model/arch/qwen.mojo:1527-1541)."""
    best, at = LOWEST_FP32, 0
    for i, v in enumerate(np.asarray(row, dtype=F32)):
        if v > best:
            best, at = v, i
    return at


def greedy(w, cfg, prompt, n_new: int) -> list:
    """Greedy continuation by recomputing the whole sequence each time."""
    ids = list(prompt)
    out = []
    for _ in range(n_new):
        tok = int(np.argmax(forward_logits(w, cfg, ids)[-1]))
        out.append(tok)
        ids.append(tok)
    return out
