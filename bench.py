"""Decode and prefill throughput of the engine at Qwen2.5-0.5B layer sizes with
random weights, on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch B] [--layers L] [--dtype bfloat16]

A step is one decode step of the whole engine loop (scheduler tick, the step
function over the paged cache, greedy choice, settle) with every request of the
batch decoding one token. Prints one JSON line; ``value`` is decoded tokens per
second at the default batch. Peaks are the published MI355X figures."""
import argparse
import json
import sys
import tempfile
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

PEAK_HBM_GBS = 8000.0
PEAK_FLOPS = {"bfloat16": 2.5e15, "float32": 157.3e12}

# Qwen2.5-0.5B layer sizes (the benchmark configuration)
QWEN25_05B = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "num_hidden_layers": 24, "hidden_size": 896,
    "num_attention_heads": 14, "num_key_value_heads": 2, "intermediate_size": 4864, "vocab_size": 151936,
    "rope_theta": 1000000.0, "rms_norm_eps": 1e-6, "tie_word_embeddings": True, "use_sliding_window": False,
    "max_position_embeddings": 32768,
}
CONTEXT, PROMPT, BLOCK = 4096, 512, 16


def linear_params_per_layer(c):
    h, d = c["hidden_size"], c["hidden_size"] // c["num_attention_heads"]
    qd, kvd, i = c["num_attention_heads"] * d, c["num_key_value_heads"] * d, c["intermediate_size"]
    return h * (qd + 2 * kvd) + qd * h + 3 * h * i


def decode_bytes(c, ctx_lens, dtype_bytes=2):
    """Bytes one decode step has to read: every weight it uses once (layer
    matrices, biases, norms, the output matrix) and the cache of the live requests."""
    h, d, L = c["hidden_size"], c["hidden_size"] // c["num_attention_heads"], c["num_hidden_layers"]
    qd, kvd = c["num_attention_heads"] * d, c["num_key_value_heads"] * d
    per_layer = linear_params_per_layer(c) * dtype_bytes + (qd + 2 * kvd) * 4 + 2 * h * 4
    weights = L * per_layer + h * 4 + c["vocab_size"] * h * dtype_bytes
    cache = sum(ctx_lens) * 2 * kvd * dtype_bytes * L
    return weights + cache


def prefill_flops(c, T, wanted=1):
    h, d, L = c["hidden_size"], c["hidden_size"] // c["num_attention_heads"], c["num_hidden_layers"]
    linear = 2 * T * linear_params_per_layer(c) * L
    attention = L * 2 * d * c["num_attention_heads"] * T * (T + 1)   # QK^T and PV over the causal half
    return linear + attention + 2 * wanted * h * c["vocab_size"]


def sync():
    import torch
    torch.cuda.synchronize()


def measure_decode(model_dir, cfg, dtype, batch, steps, warmup, seed=0, prompt=None):
    import numpy as np
    from alofa_amd import Engine
    rng = np.random.default_rng(seed)
    per_req = (CONTEXT + BLOCK - 1) // BLOCK
    eng = Engine(model_dir, dtype=dtype, max_tokens=CONTEXT, max_batch=batch, kv_blocks=per_req * batch + 64,
                 block_size=BLOCK, token_budget=max(2048, batch), max_chunk=512, watermark_permille=1000)
    core = eng.core
    prompt = PROMPT if prompt is None else prompt
    for r in range(batch):
        core.submit(r + 1, [int(t) for t in rng.integers(0, cfg["vocab_size"], prompt)], CONTEXT - prompt)
    while not (core.last_action and len(core.last_action.decode) == batch and not core.last_action.prefill):
        core.tick()
    for _ in range(warmup):
        core.tick()
    sync()
    t0 = time.perf_counter()
    for _ in range(steps):
        rows = core.tick()
        assert rows == batch, f"a timed step ran {rows} rows, not {batch}"
    sync()
    dt = time.perf_counter() - t0
    ctx_lens = [eng.cache.length(r + 1) for r in range(batch)]
    for r in range(batch):
        core.cancel(r + 1)
    core.tick()
    del eng
    import torch
    torch.cuda.empty_cache()
    return dt / steps, ctx_lens


def measure_prefill(model_dir, cfg, dtype, T=2048, reps=3, seed=1):
    import numpy as np
    from alofa_amd.replay import Replayer
    rng = np.random.default_rng(seed)
    r = Replayer(model_dir, dtype, max_tokens=CONTEXT, block_size=BLOCK)
    best = None
    for i in range(reps + 1):
        ids = [int(t) for t in rng.integers(0, cfg["vocab_size"], T)]
        from alofa_amd.engine.step import StepEntry
        r.cache.admit(i)
        sync()
        t0 = time.perf_counter()
        r.fn.run([StepEntry(i, ids, [T - 1])])
        sync()
        dt = time.perf_counter() - t0
        r.cache.free(i)
        if i > 0:
            best = dt if best is None else min(best, dt)
    return best


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt", type=int, default=PROMPT, help="prompt length of the timed decode steps' requests (context = prompt + steps so far)")
    ap.add_argument("--layers", type=int, default=QWEN25_05B["num_hidden_layers"], help="fewer layers than the configuration has, where memory or time needs it")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 / 64 points and the prefill")
    ap.add_argument("--only-prefill", action="store_true", help="run the 2,048-token prefill alone (for profiling) and print its line")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU only: this engine has no multi-GPU path (--gpus must be 1)")
        return 2

    from alofa_amd.csrc.build import load
    load()
    from alofa_amd.weights import write_random_model
    cfg = dict(QWEN25_05B, num_hidden_layers=args.layers)
    with tempfile.TemporaryDirectory() as d:
        write_random_model(cfg, d, seed=20260918)
        if args.only_prefill:
            pt = measure_prefill(d, cfg, args.dtype, 2048)
            print(json.dumps({"prefill": {"value": round(2048 / pt, 1), "tokens": 2048, "ms": round(pt * 1e3, 3),
                                          "frac": round(prefill_flops(cfg, 2048) / pt / PEAK_FLOPS[args.dtype], 4)}}))
            return 0
        if not 1 <= args.prompt <= CONTEXT - args.steps - args.warmup - 1:
            print(f"--prompt must leave room for the decode steps within the context of {CONTEXT}")
            return 2
        ms, ctx_lens = measure_decode(d, cfg, args.dtype, args.batch, args.steps, args.warmup, prompt=args.prompt)
        value = args.batch / ms
        dbytes = 2 if args.dtype == "bfloat16" else 4
        achieved = decode_bytes(cfg, ctx_lens, dbytes) / ms / 1e9
        out = {
            "metric": "decode tok/s @ batch 8 (Qwen2.5-0.5B sizes); prefill tok/s @ 2,048 tok; decode @ batch 1/64 under points",
            "value": round(value, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": round(ms * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic (random weights N(0, 0.02), uniform random token ids)",
            "config": {"model": "Qwen2.5-0.5B sizes, random weights", "layers": args.layers, "layers_full": QWEN25_05B["num_hidden_layers"],
                       "hidden": 896, "heads": 14, "kv_heads": 2, "head_dim": 64, "intermediate": 4864, "vocab": 151936,
                       "global_batch": args.batch, "seq_len": CONTEXT, "prompt_len": args.prompt, "decode_context": int(sum(ctx_lens) / len(ctx_lens)),
                       "kv_block": BLOCK, "tied_embeddings": True, "parallelism": "single GPU"},
            "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                         "frac": round(achieved / PEAK_HBM_GBS, 4)},
        }
        if not args.no_points:
            T = 2048
            pt = measure_prefill(d, cfg, args.dtype, T)
            out["prefill"] = {"value": round(T / pt, 1), "tokens": T, "ms": round(pt * 1e3, 3),
                              "frac": round(prefill_flops(cfg, T) / pt / PEAK_FLOPS[args.dtype], 4)}
            points = {}
            for b in (1, 64):
                pms, _ = measure_decode(d, cfg, args.dtype, b, max(16, args.steps // 2), max(4, args.warmup // 2))
                points[f"decode_b{b}"] = round(b / pms, 1)
            # the same near the end of the context window (prompts of 3,840 tokens)
            for b in (8, 64):
                pms, _ = measure_decode(d, cfg, args.dtype, b, max(16, args.steps // 4), max(4, args.warmup // 4), prompt=CONTEXT - 256)
                points[f"decode_b{b}_ctx{CONTEXT - 256}"] = round(b / pms, 1)
            out["points"] = points
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
