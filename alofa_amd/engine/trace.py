"""Text form of scheduler ticks, one line each, so that a run can be recorded
and replayed (src/alofa/engine/trace.mojo:63-238):

  CFG b=<budget> c=<max_chunk> s=<block_size> k=<capacity_blocks> w=<permille> t=<max_wait>
  IN=A=<id:prompt:max_new,...|->|C=<ids|->|F=<ids|->|R=<n> OUT=t=<tick> P=<id:start:end,...|-> D=<ids|-> X=<ids|-> F=<ids|-> C=<preempt_total> K=<digest>
"""
from __future__ import annotations

from ..errors import AlofaError
from .scheduler import Action, SchedConfig, SchedInput


def _ints(items) -> str:
    return ",".join(str(i) for i in items) if items else "-"


def config_line(cfg: SchedConfig) -> str:
    return f"CFG b={cfg.token_budget} c={cfg.max_chunk} s={cfg.block_size} k={cfg.capacity_blocks} w={cfg.watermark_permille} t={cfg.max_wait_ticks}"


def parse_config(line: str) -> SchedConfig:
    f = line.split(" ")
    if len(f) != 7 or f[0] != "CFG":
        raise AlofaError("parse", "config line must be CFG plus six fields", line)
    try:
        vals = {kv.split("=")[0]: int(kv.split("=")[1]) for kv in f[1:]}
        return SchedConfig(vals["b"], vals["c"], vals["s"], vals["k"], vals["w"], vals["t"])
    except (KeyError, ValueError, IndexError):
        raise AlofaError("parse", "malformed config line", line) from None


def input_line(inp: SchedInput) -> str:
    arrivals = ",".join(f"{a}:{p}:{m}" for a, p, m in inp.arrivals) if inp.arrivals else "-"
    # (R: the blocks given back in the first group of layers, the one the reference's single count stands for)
    freed = inp.freed_blocks[0] if isinstance(inp.freed_blocks, (list, tuple)) else inp.freed_blocks
    return f"IN=A={arrivals}|C={_ints(inp.cancelled)}|F={_ints(inp.finished)}|R={freed}"


def action_line(act: Action) -> str:
    prefill = ",".join(f"{r}:{s}:{e}" for r, s, e in act.prefill) if act.prefill else "-"
    return (f"OUT=t={act.tick_seq} P={prefill} D={_ints(act.decode)} X={_ints(act.preempted)} "
            f"F={_ints(act.finished)} C={act.preempt_total} K={act.state_digest}")


def trace_line(inp: SchedInput, act: Action) -> str:
    return input_line(inp) + " " + action_line(act)


def parse_input(text: str) -> SchedInput:
    if not text.startswith("IN="):
        raise AlofaError("parse", "input line must start with IN=", text)
    groups = text[3:].split("|")
    if len(groups) != 4:
        raise AlofaError("parse", "input line must have four groups", text)
    inp = SchedInput()
    try:
        for g, key in zip(groups, "ACFR"):
            if not g.startswith(key + "="):
                raise ValueError(g)
            items = g[2:]
            if items == "-":
                continue
            if key == "A":
                for item in items.split(","):
                    a, p, m = item.split(":")
                    inp.arrivals.append((int(a), int(p), int(m)))
            elif key == "R":
                inp.freed_blocks = int(items)
            else:
                (inp.cancelled if key == "C" else inp.finished).extend(int(i) for i in items.split(","))
    except ValueError:
        raise AlofaError("parse", "malformed input line", text) from None
    return inp
