"""Helpers of the GPU tests: traces in the replay tool's format, an in-process replayer that
drives the engine's own step function, and the comparison with the plain implementation."""
from __future__ import annotations

import random
from typing import Dict, List, Sequence, Tuple

import torch

# Tolerances, as a fraction of the largest reference logit of the compared rows.  float32:
# both sides compute in 32 bits and differ only in the order of sums.  bfloat16: weights
# are the same bfloat16 values on both sides; activations between kernels are rounded to
# 8 mantissa bits (relative 2^-9 each), a handful of times per layer.
# The worst errors the tests print on an MI355X: float32 5.9e-6 (tiny and real sizes, every way
# of cutting); bfloat16 1.1e-2 at real layer sizes and 1.4e-2 on the long-context model, whose
# sharpened scores make the rounding of q and k show more.  The bounds are about three times
# the float32 figure and one and a half times the bfloat16 one.
TOL = {"float32": 2e-5, "bfloat16": 2e-2}


def random_prompt(rng: random.Random, n: int, vocab: int) -> List[int]:
    return [rng.randrange(vocab) for _ in range(n)]


# ---- traces -----------------------------------------------------------------------------
def trace_whole(reqs: Dict[str, List[int]]) -> List[dict]:
    """Each request alone and whole, every position wanted."""
    steps = []
    for i, (rid, toks) in enumerate(reqs.items()):
        steps.append({"step": i, "entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}],
                      "end": [rid]})
    return steps


def trace_tail_one_by_one(reqs: Dict[str, List[int]], tail: int = 32) -> List[dict]:
    """Most of a request in one step, then its last `tail` tokens one by one."""
    steps, s = [], 0
    for rid, toks in reqs.items():
        head = max(1, len(toks) - tail)
        steps.append({"step": s, "entries": [{"id": rid, "tokens": toks[:head], "want": list(range(head))}], "end": []})
        s += 1
        for p in range(head, len(toks)):
            steps.append({"step": s, "entries": [{"id": rid, "tokens": [toks[p]], "want": [0]}],
                          "end": [rid] if p == len(toks) - 1 else []})
            s += 1
        if head == len(toks):
            steps[-1]["end"] = [rid]
    return steps


def trace_portions(reqs: Dict[str, List[int]], sizes: Sequence[int] = (7, 2, 19, 3, 2, 31, 5, 2, 64, 11)) -> List[dict]:
    """Portions of changing size, down to two tokens (a single last token may remain)."""
    steps, s = [], 0
    for rid, toks in reqs.items():
        p, k = 0, 0
        while p < len(toks):
            n = min(sizes[k % len(sizes)], len(toks) - p)
            k += 1
            last = p + n == len(toks)
            steps.append({"step": s, "entries": [{"id": rid, "tokens": toks[p:p + n], "want": list(range(n))}],
                          "end": [rid] if last else []})
            p += n
            s += 1
    return steps


def trace_mixed(reqs: Dict[str, List[int]], seed: int, max_live: int = 4, tail: int = 6,
                sizes: Sequence[int] = (9, 2, 17, 4, 2, 23, 3)) -> List[dict]:
    """Up to `max_live` requests at a time: portions of some beside single tokens of others,
    a request now and then left out of a step; a request that ends makes room for the next,
    whose pages are then pages used before."""
    rng = random.Random(seed)
    waiting = list(reqs.items())
    live: List[dict] = []
    steps, s = [], 0
    while waiting or live:
        while waiting and len(live) < max_live:
            rid, toks = waiting.pop(0)
            live.append({"id": rid, "toks": toks, "pos": 0, "k": rng.randrange(len(sizes))})
        entries, end = [], []
        for r in live:
            if len(live) > 1 and rng.random() < 0.2:
                continue                                   # left out of this step
            remaining = len(r["toks"]) - r["pos"]
            if remaining <= tail:
                n = 1                                        # decode-like single token
            else:
                n = min(sizes[r["k"] % len(sizes)], remaining - tail)
                r["k"] += 1
            entries.append({"id": r["id"], "tokens": r["toks"][r["pos"]:r["pos"] + n], "want": list(range(n))})
            r["pos"] += n
            if r["pos"] == len(r["toks"]):
                end.append(r["id"])
        if not entries:
            continue
        live = [r for r in live if r["id"] not in end]
        steps.append({"step": s, "entries": entries, "end": end})
        s += 1
    return steps


def trace_batch_decode(reqs: Dict[str, List[int]], tail: int = 4) -> List[dict]:
    """All requests live together: their heads as portions of one step, then `tail` steps that
    bring one token of every request (a wide decode batch), every position wanted."""
    steps = [{"step": 0, "end": [], "entries": [
        {"id": rid, "tokens": toks[:len(toks) - tail], "want": list(range(len(toks) - tail))} for rid, toks in reqs.items()]}]
    for k in range(tail):
        steps.append({"step": 1 + k, "end": list(reqs) if k == tail - 1 else [], "entries": [
            {"id": rid, "tokens": [toks[len(toks) - tail + k]], "want": [0]} for rid, toks in reqs.items()]})
    return steps


def tokens_needed(steps: List[dict], page: int) -> int:
    """The most tokens live requests hold at any time, each rounded up to a page."""
    held: Dict[str, int] = {}
    worst = 0
    for st in steps:
        for e in st["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        worst = max(worst, sum(-(-n // page) * page for n in held.values()))
        for rid in st["end"]:
            held.pop(rid, None)
    return worst


# ---- replay in process ----------------------------------------------------------------------
def replay(runner, steps: List[dict]) -> Dict[Tuple[str, int], torch.Tensor]:
    """Drives `runner.step` with a trace; returns logits by (request, position)."""
    from xinfer_amd.engine import StepEntry
    ids: Dict[str, int] = {}
    fed: Dict[str, int] = {}
    nxt = [1000]
    out: Dict[Tuple[str, int], torch.Tensor] = {}
    for st in steps:
        entries = []
        for e in st["entries"]:
            if e["id"] not in ids:
                ids[e["id"]] = nxt[0]
                nxt[0] += 1
                fed[e["id"]] = 0
                runner.add_request(ids[e["id"]])
            entries.append(StepEntry(ids[e["id"]], e["tokens"], e["want"]))
        logits = runner.step(entries).cpu()
        row = 0
        for e in st["entries"]:
            for w in e["want"]:
                out[(e["id"], fed[e["id"]] + w)] = logits[row]
                row += 1
            fed[e["id"]] += len(e["tokens"])
        assert row == logits.shape[0]
        for rid in st["end"]:
            runner.release(ids.pop(rid))
            fed.pop(rid)
        runner.cache.check()
    return out


def compare(got: Dict[Tuple[str, int], torch.Tensor], ref: Dict[str, torch.Tensor], tol: float, what: str):
    """Every (request, position) of `got` against the plain logits `ref[request][position]`.
    Reports the first wrong position of the worst request."""
    assert got, f"{what}: nothing was compared"
    scale = max(float(r.abs().max()) for r in ref.values())
    worst, first_bad = 0.0, None
    for (rid, pos) in sorted(got):
        err = float((got[(rid, pos)].double() - ref[rid][pos].double()).abs().max())
        if not (err == err):
            raise AssertionError(f"{what}: NaN in the logits of request {rid} position {pos}")
        if err > worst:
            worst = err
        if err > tol * scale and first_bad is None:
            first_bad = (rid, pos, err)
    if first_bad is not None:
        rid, pos, err = first_bad
        raise AssertionError(
            f"{what}: first wrong logits at request {rid} position {pos}: |diff| {err:.3e} > "
            f"{tol:g} * {scale:.3e} (worst over all {worst:.3e})")
    return worst / scale
