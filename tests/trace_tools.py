"""Builds replay traces for a set of requests and collects the logits a runner returns.

A trace is a list of step objects in the format of bin/trace_run. The four ways of cutting
the same requests: whole, most of it in one step and the last tokens one by one, portions of
changing size, and mixed with other requests on a pool so small that pages are used again.
"""
from __future__ import annotations

from typing import Callable, Dict, List, Optional, Sequence, Tuple

import numpy as np


def whole(reqs: Dict[str, List[int]]) -> List[dict]:
    steps = []
    for i, (rid, toks) in enumerate(reqs.items()):
        steps.append({"step": i, "entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}],
                      "end": [rid]})
    return steps


def tail_decode(reqs: Dict[str, List[int]], tail: int = 32) -> List[dict]:
    steps = []
    for rid, toks in reqs.items():
        head = max(1, len(toks) - tail)
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks[:head], "want": [head - 1]}],
                      "end": []})
        for p in range(head, len(toks)):
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": [toks[p]], "want": [0]}],
                          "end": [rid] if p == len(toks) - 1 else []})
        if head == len(toks):
            steps[-1]["end"] = [rid]
    return steps


def portions(reqs: Dict[str, List[int]], sizes: Sequence[int] = (7, 5, 3, 2, 11, 2, 17, 2, 4)) -> List[dict]:
    steps = []
    k = 0
    for rid, toks in reqs.items():
        p = 0
        while p < len(toks):
            n = min(sizes[k % len(sizes)], len(toks) - p)
            if len(toks) - p - n == 1:          # never leave a lone last token: portions go down to two
                n += 1
            k += 1
            chunk = toks[p:p + n]
            p += n
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": chunk, "want": list(range(len(chunk)))}],
                          "end": [rid] if p == len(toks) else []})
    return steps


def mixed(reqs: Dict[str, List[int]], prompt_lens: Dict[str, int], max_live: int = 4, seed: int = 0,
          max_portion: int = 9) -> List[dict]:
    """Up to ``max_live`` requests at a time. A request first feeds its prompt in portions of
    random size (2..max_portion), then its remaining tokens one by one; some live requests sit a
    step out. A finished request is ended at once and the next one starts, so its pages go to
    the newcomers."""
    rng = np.random.default_rng(seed)
    waiting = list(reqs.keys())
    live: List[str] = []
    done_upto = {rid: 0 for rid in reqs}
    steps = []
    while waiting or live:
        while waiting and len(live) < max_live:
            live.append(waiting.pop(0))
        entries, ended = [], []
        for rid in list(live):
            if len(live) > 1 and rng.random() < 0.25:
                continue                                     # left out of this step
            toks, p = reqs[rid], done_upto[rid]
            if p < prompt_lens[rid]:
                n = int(rng.integers(2, max_portion + 1))
                n = min(n, prompt_lens[rid] - p)
                if prompt_lens[rid] - p - n == 1:
                    n += 1
            else:
                n = 1
            chunk = toks[p:p + n]
            done_upto[rid] = p + n
            entries.append({"id": rid, "tokens": chunk, "want": list(range(len(chunk)))})
            if done_upto[rid] == len(toks):
                ended.append(rid)
                live.remove(rid)
        if entries:
            steps.append({"step": len(steps), "entries": entries, "end": ended})
    return steps


def max_live_tokens(steps: List[dict], rounding: int = 64) -> int:
    """The --max-tokens a trace needs: the most tokens live requests hold at any time, each
    request's count rounded up to ``rounding``."""
    held: Dict[str, int] = {}
    worst = 0
    for st in steps:
        for e in st["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        worst = max(worst, sum(-(-n // rounding) * rounding for n in held.values()))
        for rid in st["end"]:
            held.pop(rid, None)
    return worst


def collect(steps: List[dict], run_step: Callable[[dict], Optional[np.ndarray]]) -> Dict[Tuple[str, int], np.ndarray]:
    """Runs the steps and returns {(request, position): logits row}."""
    pos: Dict[str, int] = {}
    out: Dict[Tuple[str, int], np.ndarray] = {}
    for st in steps:
        logits = run_step(st)
        row = 0
        for e in st["entries"]:
            base = pos.get(e["id"], 0)
            for w in e.get("want", []):
                assert logits is not None and row < logits.shape[0], "fewer logits rows than wanted"
                out[(e["id"], base + w)] = np.array(logits[row], dtype=np.float32)
                row += 1
            pos[e["id"]] = base + len(e["tokens"])
        assert logits is None or row == logits.shape[0], "more logits rows than wanted"
        for rid in st["end"]:
            pos.pop(rid, None)
    return out



def crowd(reqs: Dict[str, List[int]], prompt_lens: Dict[str, int], seed: int = 0, max_portion: int = 9,
          sit_out: float = 0.0) -> List[dict]:
    """Every request is live from the first step on. Prompts go in portions of random size
    (2..max_portion); a request whose prompt is in decodes one token a step until its tokens run out.
    With requests of different lengths the steps go from many prompt portions side by side, through
    portions beside decoded tokens, to decode-only steps whose number of sequences falls from all
    requests to one. ``sit_out``: chance that a live request is left out of a step."""
    rng = np.random.default_rng(seed)
    live = list(reqs.keys())
    done_upto = {rid: 0 for rid in reqs}
    steps = []
    while live:
        entries, ended = [], []
        for rid in list(live):
            if sit_out and len(live) > 1 and rng.random() < sit_out:
                continue
            toks, p = reqs[rid], done_upto[rid]
            if p < prompt_lens[rid]:
                n = min(int(rng.integers(2, max_portion + 1)), prompt_lens[rid] - p)
                if prompt_lens[rid] - p - n == 1:
                    n += 1
            else:
                n = 1
            chunk = toks[p:p + n]
            done_upto[rid] = p + n
            entries.append({"id": rid, "tokens": chunk, "want": list(range(len(chunk)))})
            if done_upto[rid] == len(toks):
                ended.append(rid)
                live.remove(rid)
        if entries:
            steps.append({"step": len(steps), "entries": entries, "end": ended})
    return steps


def prompts_then_subsets(reqs: Dict[str, List[int]], prompt_lens: Dict[str, int], subsets: Sequence[Sequence[str]],
                         seed: int = 0, max_portion: int = 2048, want_prompt_rows: bool = True) -> List[dict]:
    """All requests live at once: first their prompts in portions of random size (2..max_portion), side
    by side; then decode-only steps whose participants follow ``subsets`` in turn (a request that has
    no token left is dropped from a subset), until every request has brought all its tokens. Which
    requests share a decode step decides the longest context of the step, so the subsets take the
    step through every launch plan the context lengths select."""
    rng = np.random.default_rng(seed)
    done_upto = {rid: 0 for rid in reqs}
    steps: List[dict] = []
    while any(done_upto[r] < prompt_lens[r] for r in reqs):
        entries = []
        for rid, toks in reqs.items():
            p = done_upto[rid]
            if p >= prompt_lens[rid]:
                continue
            n = min(int(rng.integers(2, max_portion + 1)), prompt_lens[rid] - p)
            if prompt_lens[rid] - p - n == 1:
                n += 1
            chunk = toks[p:p + n]
            done_upto[rid] = p + n
            want = list(range(len(chunk))) if want_prompt_rows else []
            entries.append({"id": rid, "tokens": chunk, "want": want})
        steps.append({"step": len(steps), "entries": entries, "end": []})
    k = 0
    while any(done_upto[r] < len(reqs[r]) for r in reqs):
        subset = [r for r in subsets[k % len(subsets)] if done_upto[r] < len(reqs[r])]
        k += 1
        if not subset:
            continue
        entries, ended = [], []
        for rid in subset:
            p = done_upto[rid]
            entries.append({"id": rid, "tokens": [reqs[rid][p]], "want": [0]})
            done_upto[rid] = p + 1
            if p + 1 == len(reqs[rid]):
                ended.append(rid)
        steps.append({"step": len(steps), "entries": entries, "end": ended})
    return steps


def only_last_rows(steps: List[dict]) -> List[dict]:
    """The same steps, each entry wanting the logits of its last token only (what generation asks for)."""
    return [dict(st, entries=[dict(e, want=[len(e["tokens"]) - 1]) for e in st["entries"]]) for st in steps]
