"""Helpers of the GPU tests: traces in the replay program's step format, cut in
different ways, and the comparison with the plain implementation."""
import functools

import numpy as np

from plain import model as pm


def round64(n):
    return (n + 63) // 64 * 64


@functools.lru_cache(maxsize=None)
def plain_model(model_dir):
    return pm.read_config(model_dir), pm.read_weights(model_dir)


class Reference(np.ndarray):
    """Logits of the plain model [positions, vocab] that also know how far rounding the activations
    to bfloat16 alone moves them (``rounded()``: the plain model with its ``store`` hook); rows cut
    out of it keep that knowledge."""
    _rounded = None

    def __array_finalize__(self, obj):
        self._rounded = None

    def __getitem__(self, index):
        out = super().__getitem__(index)
        if isinstance(out, Reference) and self._rounded is not None:
            parent = self._rounded
            out._rounded = lambda: parent()[index]
        return out

    def rounded(self):
        return None if self._rounded is None else self._rounded()


@functools.lru_cache(maxsize=64)
def _plain_logits(model_dir, ids, rounded):
    cfg, w = plain_model(model_dir)
    return pm.forward_logits(w, cfg, list(ids), store=pm.to_bfloat16 if rounded else (lambda x: x))


def plain_logits(model_dir, ids):
    ref = _plain_logits(str(model_dir), tuple(ids), False).view(Reference)
    ref._rounded = lambda: _plain_logits(str(model_dir), tuple(ids), True)
    return ref


def random_ids(seed, n, vocab):
    return [int(t) for t in np.random.default_rng(seed).integers(0, vocab, n)]


def bound(dtype, ref):
    """float32: the reference's criterion 1e-5 * max(1, max|ref|)
    (tests/unit/test_layer0_parity.mojo:46 there). bfloat16 without a measure of the rounding: 1e-2
    of the same scale."""
    return (1e-5 if dtype == "float32" else 1e-2) * max(1.0, float(np.abs(ref).max()))


RATIOS = []      # (what, largest error / rounding's largest, rms error / rounding's rms) of the bfloat16 comparisons


def assert_close(got, ref, dtype, what=""):
    """float32: within the reference's criterion. bfloat16: measured against what rounding alone
    does. The engine keeps its activations in bfloat16 between kernels; the plain model with the
    same activations rounded (and nothing else changed) differs from the exact one by some largest
    and some root-mean-square error, and the engine, whose sums run in another order and whose
    softmax weights are rounded too, may differ from the exact logits by at most twice the one and
    one and a half times the other. A fault (a key too many or too few, a stale page, a wrong
    row) moves logits by far more than the rounding does."""
    noise = ref.rounded() if isinstance(ref, Reference) and dtype == "bfloat16" else None
    got, ref = np.asarray(got, dtype=np.float64), np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape, f"{what}: shape {got.shape} vs {ref.shape}"
    assert np.isfinite(got).all(), f"{what}: not finite"
    err = np.abs(got - ref)
    if noise is not None:
        n = np.abs(np.asarray(noise, dtype=np.float64) - ref)
        b, rms, n_rms = 2.0 * n.max(), float(np.sqrt((err ** 2).mean())), float(np.sqrt((n ** 2).mean()))
        RATIOS.append((what, err.max() / max(n.max(), 1e-30), rms / max(n_rms, 1e-30)))
        assert rms <= 1.5 * n_rms, f"{what}: rms error {rms:.3e} > 1.5 x {n_rms:.3e}, the rms error of rounding alone"
    else:
        b = bound(dtype, ref)
    if err.max() > b:
        at = np.unravel_index(np.argmax(err), err.shape)
        first = int(np.argmax(err.reshape(err.shape[0], -1).max(axis=1) > b))
        raise AssertionError(f"{what}: max abs diff {err.max():.3e} > {b:.3e} at {at}; first wrong row {first}")
    if got.ndim == 2 and got.shape[1] > 8:
        def lowest_cosine(x):
            return float(((x * ref).sum(1) / (np.linalg.norm(x, axis=1) * np.linalg.norm(ref, axis=1) + 1e-30)).min())
        if noise is not None:
            # 1 - cosine goes with the square of the relative error: 1.5 times rounding's error is 2.25 times its 1 - cosine
            allowed = 1.0 - 3.0 * (1.0 - lowest_cosine(np.asarray(noise, dtype=np.float64)))
            assert lowest_cosine(got) >= min(allowed, 0.999), f"{what}: cosine {lowest_cosine(got)} < {allowed}"
        else:
            assert lowest_cosine(got) >= (0.999999 if dtype == "float32" else 0.999), f"{what}: cosine {lowest_cosine(got)}"


# ------------------------------------------------------------------ cuttings

def whole(req, ids, step0=0):
    return [{"step": step0, "entries": [{"id": req, "tokens": list(ids), "want": list(range(len(ids)))}], "end": [req]}]


def bulk_and_tail(req, ids, tail=32, step0=0):
    """Most of it in one step, the last ``tail`` tokens one by one."""
    n = len(ids) - tail
    steps = [{"step": step0, "entries": [{"id": req, "tokens": list(ids[:n]), "want": list(range(n))}], "end": []}]
    for i in range(n, len(ids)):
        steps.append({"step": step0 + len(steps), "entries": [{"id": req, "tokens": [ids[i]], "want": [0]}],
                      "end": [req] if i == len(ids) - 1 else []})
    return steps


def portions(req, ids, sizes=(7, 2, 16, 3, 2, 31, 5, 2, 17), step0=0):
    steps, pos, k = [], 0, 0
    while pos < len(ids):
        n = min(sizes[k % len(sizes)], len(ids) - pos)
        if len(ids) - pos - n == 1:      # never leave a single token: portions go down to two, not one
            n += 1
        k += 1
        steps.append({"step": step0 + len(steps), "entries": [{"id": req, "tokens": list(ids[pos:pos + n]), "want": list(range(n))}],
                      "end": [req] if pos + n == len(ids) else []})
        pos += n
    return steps


def mixed(requests, seed, tail=32, max_live=4, step0=0):
    """Up to ``max_live`` live requests: portions of some beside single decoded
    tokens of others, a request left out of a step now and then; a finished
    request ends and the next one starts, so its pages are used again.
    Returns (steps, peak of the live requests' token counts rounded up to 64)."""
    rnd = np.random.default_rng(seed)
    waiting = list(requests.items())
    live, pos, steps, peak = [], {}, [], 0
    while waiting or live:
        while waiting and len(live) < max_live:
            r, ids = waiting.pop(0)
            live.append(r)
            pos[r] = 0
        entries, ended = [], []
        for r in list(live):
            ids = requests[r]
            if len(live) > 1 and rnd.random() < 0.2:
                continue                                       # left out of this step
            left = len(ids) - pos[r]
            if left <= tail:
                n = 1                                          # decoding: one token
            else:
                n = int(min(rnd.integers(2, 24), left - tail))
                if left - tail - n == 1:
                    n += 1
            entries.append({"id": r, "tokens": list(ids[pos[r]:pos[r] + n]), "want": list(range(n))})
            pos[r] += n
            if pos[r] == len(ids):
                ended.append(r)
        peak = max(peak, sum(round64(len(requests[r])) for r in live))
        for r in ended:
            live.remove(r)
        if entries:
            steps.append({"step": step0 + len(steps), "entries": entries, "end": ended})
    return steps, peak


def collect(replayer, steps):
    """Run steps through a Replayer; returns {request: [logits row per position]}."""
    out, at = {}, {}
    for rec in steps:
        logits = replayer.step(rec)
        k = 0
        for e in rec["entries"]:
            base = at.get(e["id"], 0)
            for w in e["want"]:
                out.setdefault(e["id"], {})[base + w] = logits[k].copy()
                k += 1
            at[e["id"]] = base + len(e["tokens"])
        assert (logits is None and k == 0) or logits.shape[0] == k
    return {r: np.stack([rows[p] for p in sorted(rows)]) for r, rows in out.items()}
