"""The ``generate`` command. As in the reference, it is configured by
environment variables, not flags (src/alofa/srv/config.mojo:1-107): an unset
variable takes its default; a malformed or out-of-range value is a named error,
never a silent fallback. Names the reference has keep their meaning:

  ALOFA_WEIGHTS            model folder (config.json + model.safetensors)
  ALOFA_MAX_TOKENS         context window, prompt + generated   (256; 1..32768)
  ALOFA_MAX_PROMPT_TOKENS  longest prompt taken                 (128; 1..32768)
  ALOFA_SEED               seed of every request's generator    (1234)
  ALOFA_BATCH              most requests running together       (8; 1..1024)

and the engine's own:

  ALOFA_DTYPE              bfloat16 | float32                   (bfloat16)
  ALOFA_PROMPT_IDS         prompts as token ids, "5,17,3;9,2"   (or the first argument)
  ALOFA_PROMPT_FILE        a file of such prompts, one a line   (when neither of the two is given)
  ALOFA_MAX_NEW            tokens to generate per prompt        (16)
  ALOFA_TEMPERATURE ALOFA_TOP_K ALOFA_TOP_P ALOFA_MIN_P ALOFA_REPETITION_PENALTY
  ALOFA_FREQUENCY_PENALTY ALOFA_PRESENCE_PENALTY   sampling; temperature 0 = greedy (0)
  ALOFA_KV_FRACTION        permille of the free device memory for the cache pool, when
                           ALOFA_KV_BLOCKS is not set                  (0: by ALOFA_BATCH x ALOFA_MAX_TOKENS)
  ALOFA_BLOCK_SIZE ALOFA_KV_BLOCKS ALOFA_TOKEN_BUDGET ALOFA_MAX_CHUNK
  ALOFA_WATERMARK_PERMILLE ALOFA_MAX_WAIT_TICKS   cache and scheduler
  ALOFA_TRACE              file that receives the scheduler trace
  ALOFA_SHARE_PREFIX       1: a new request starts on the pages a running one wrote
                           for the same first tokens                 (0)
  ALOFA_RANDOM_CONFIG      config.json to make random weights from (with ALOFA_SEED)
                           into ALOFA_WEIGHTS when that folder has no model yet

There is no tokenizer here: prompts and outputs are token ids, one line of
comma-separated ids per prompt."""
from __future__ import annotations

import json
import os
import sys
from pathlib import Path

from .errors import AlofaError


def env_str(name: str, default: str) -> str:
    raw = os.environ.get(name, "")
    return raw if raw else default


def env_int(name: str, default: int, lo: int, hi: int) -> int:
    raw = os.environ.get(name, "")
    value = default
    if raw:
        try:
            value = int(raw)
        except ValueError:
            raise AlofaError("invalid_argument", "environment variable is not an integer", f"{name}={raw}") from None
    if not lo <= value <= hi:
        raise AlofaError("invalid_argument", "environment variable is out of range", f"{name}={value} not in [{lo}, {hi}]")
    return value


def env_float(name: str, default: float, lo: float, hi: float) -> float:
    raw = os.environ.get(name, "")
    value = default
    if raw:
        try:
            value = float(raw)
        except ValueError:
            raise AlofaError("invalid_argument", "environment variable is not a number", f"{name}={raw}") from None
    if not lo <= value <= hi:
        raise AlofaError("invalid_argument", "environment variable is out of range", f"{name}={value} not in [{lo}, {hi}]")
    return value


def parse_prompts(text: str) -> list:
    prompts = []
    for part in text.replace("\n", ";").split(";"):
        part = part.strip()
        if not part:
            continue
        try:
            prompts.append([int(t) for t in part.replace(" ", ",").split(",") if t])
        except ValueError:
            raise AlofaError("parse", "prompts are comma-separated token ids, one prompt per ';'", f"prompt={part[:40]}") from None
    if not prompts:
        raise AlofaError("invalid_argument", "no prompt given: set ALOFA_PROMPT_IDS or pass the ids as the first argument")
    return prompts


def main(argv=None) -> int:
    argv = sys.argv[1:] if argv is None else argv
    weights = env_str("ALOFA_WEIGHTS", "")
    if not weights:
        raise AlofaError("invalid_argument", "ALOFA_WEIGHTS is not set: it names the model folder")
    max_tokens = env_int("ALOFA_MAX_TOKENS", 256, 1, 32768)
    max_prompt = env_int("ALOFA_MAX_PROMPT_TOKENS", 128, 1, 32768)
    seed = env_int("ALOFA_SEED", 1234, 0, 2_147_483_647)
    batch = env_int("ALOFA_BATCH", 8, 1, 1024)
    dtype = env_str("ALOFA_DTYPE", "bfloat16")
    if dtype not in ("bfloat16", "float32"):
        raise AlofaError("invalid_argument", "ALOFA_DTYPE is bfloat16 or float32", f"ALOFA_DTYPE={dtype}")
    max_new = env_int("ALOFA_MAX_NEW", 16, 1, 32768)
    text = argv[0] if argv else env_str("ALOFA_PROMPT_IDS", "")
    prompt_file = env_str("ALOFA_PROMPT_FILE", "")
    if not text and prompt_file:
        try:
            text = Path(prompt_file).read_text()
        except OSError as e:
            raise AlofaError("io", "cannot read ALOFA_PROMPT_FILE", f"path={prompt_file} reason={e}") from None
    prompts = parse_prompts(text)
    for p in prompts:
        if len(p) > max_prompt:
            raise AlofaError("out_of_range", "prompt is longer than ALOFA_MAX_PROMPT_TOKENS", f"tokens={len(p)} limit={max_prompt}")
        if len(p) + max_new > max_tokens:
            raise AlofaError("out_of_range", "prompt plus ALOFA_MAX_NEW passes ALOFA_MAX_TOKENS", f"need={len(p) + max_new} window={max_tokens}")
    random_config = env_str("ALOFA_RANDOM_CONFIG", "")
    if random_config and not (Path(weights) / "model.safetensors").exists():
        from .weights import write_random_model
        write_random_model(json.loads(Path(random_config).read_text()), weights, seed)
    block = env_int("ALOFA_BLOCK_SIZE", 16, 1, 1024)
    kv_blocks = env_int("ALOFA_KV_BLOCKS", 0, 0, 1 << 30)
    kv_permille = env_int("ALOFA_KV_FRACTION", 0, 0, 1000)

    budget = env_int("ALOFA_TOKEN_BUDGET", 2048, 1, 1 << 20)
    from .api import Engine
    engine = Engine(weights, dtype=dtype, max_tokens=max_tokens, max_batch=batch, kv_blocks=kv_blocks or None,
                    block_size=block, token_budget=budget,
                    max_chunk=env_int("ALOFA_MAX_CHUNK", budget, 1, 1 << 20),
                    watermark_permille=env_int("ALOFA_WATERMARK_PERMILLE", 900, 1, 1000),
                    max_wait_ticks=env_int("ALOFA_MAX_WAIT_TICKS", 8, 0, 1 << 20), seed=seed,
                    trace_path=env_str("ALOFA_TRACE", "") or None,
                    share_prefixes=bool(env_int("ALOFA_SHARE_PREFIX", 0, 0, 1)),
                    memory_fraction=kv_permille / 1000.0 if kv_permille and not kv_blocks else None,
                    report=lambda line: print(line, file=sys.stderr, flush=True))
    outs = engine.generate(prompts, max_new=max_new,
                           temperature=env_float("ALOFA_TEMPERATURE", 0.0, 0.0, 1e6),
                           top_k=env_int("ALOFA_TOP_K", 0, 0, 1 << 30), top_p=env_float("ALOFA_TOP_P", 1.0, 1e-9, 1.0),
                           min_p=env_float("ALOFA_MIN_P", 0.0, 0.0, 1.0),
                           repetition_penalty=env_float("ALOFA_REPETITION_PENALTY", 1.0, 1e-9, 1e6),
                           frequency_penalty=env_float("ALOFA_FREQUENCY_PENALTY", 0.0, -1e6, 1e6),
                           presence_penalty=env_float("ALOFA_PRESENCE_PENALTY", 0.0, -1e6, 1e6))
    for out in outs:
        print(",".join(str(t) for t in out), flush=True)
    return 0


def run() -> int:
    try:
        return main()
    except AlofaError as e:
        print(f"generate: {e}", file=sys.stderr)
        return 1


if __name__ == "__main__":
    sys.exit(run())
