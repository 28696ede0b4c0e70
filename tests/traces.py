"""Traces for replay: ways of cutting the same requests into steps.  A trace is a list of
steps ``{"step", "entries": [{"id", "tokens", "want"}], "end"}`` as ``bin/trace_run`` reads
them; every token's logits are wanted, so that each mode can be compared with the plain
implementation position by position."""
from __future__ import annotations

import random
from typing import Dict, List, Sequence


def _entry(rid, tokens, lo, hi):
    # "start" is optional for the replay program; the traces give it, so that every replay
    # also checks that the engine holds exactly the tokens the trace thinks it holds
    return {"id": rid, "tokens": list(tokens[lo:hi]), "want": list(range(hi - lo)), "start": lo}


def whole(requests: Dict[str, Sequence[int]]) -> List[dict]:
    """Each request alone, whole, in one step."""
    steps = []
    for rid, toks in requests.items():
        steps.append({"step": len(steps), "entries": [_entry(rid, toks, 0, len(toks))],
                      "end": [rid]})
    return steps


def prefill_then_single(requests: Dict[str, Sequence[int]], tail: int = 32) -> List[dict]:
    """Most of a request in one step, its last ``tail`` tokens one by one."""
    steps = []
    for rid, toks in requests.items():
        n = len(toks)
        head = max(n - tail, 1)
        steps.append({"step": len(steps), "entries": [_entry(rid, toks, 0, head)], "end": []})
        for p in range(head, n):
            steps.append({"step": len(steps), "entries": [_entry(rid, toks, p, p + 1)], "end": []})
        steps[-1]["end"] = [rid]
    return steps


PORTIONS = (7, 24, 2, 13, 2, 5, 3, 40, 1, 2, 17, 2, 9, 31)


def changing_portions(requests: Dict[str, Sequence[int]], sizes=PORTIONS) -> List[dict]:
    """Portions of changing size, down to two tokens (and one), at unaligned offsets."""
    steps = []
    for rid, toks in requests.items():
        p, i = 0, 0
        while p < len(toks):
            n = min(sizes[i % len(sizes)], len(toks) - p)
            steps.append({"step": len(steps), "entries": [_entry(rid, toks, p, p + n)],
                          "end": []})
            p += n
            i += 1
        steps[-1]["end"] = [rid]
    return steps


def token_by_token(requests: Dict[str, Sequence[int]]) -> List[dict]:
    steps = []
    for rid, toks in requests.items():
        for p in range(len(toks)):
            steps.append({"step": len(steps), "entries": [_entry(rid, toks, p, p + 1)], "end": []})
        steps[-1]["end"] = [rid]
    return steps


def mixed(requests: Dict[str, Sequence[int]], max_live: int = 4, seed: int = 0,
          decode_tail: int = 12) -> List[dict]:
    """Up to ``max_live`` requests live at a time: portions of some beside single tokens of
    others; a request may sit a step out; finished requests end and later ones reuse their
    pages.  The last ``decode_tail`` tokens of each request come one per step."""
    rnd = random.Random(seed)
    waiting = list(requests.items())
    live: List[list] = []          # [rid, tokens, position]
    steps = []
    while waiting or live:
        while waiting and len(live) < max_live:
            rid, toks = waiting.pop(0)
            live.append([rid, toks, 0])
        entries, end = [], []
        for item in live:
            rid, toks, p = item
            if len(live) > 1 and rnd.random() < 0.2:
                continue                       # left out of this step, goes on later
            left = len(toks) - p
            if left <= decode_tail:
                n = 1
            else:
                n = min(rnd.choice((2, 3, 5, 8, 16, 17, 30)), left - decode_tail)
            entries.append(_entry(rid, toks, p, p + n))
            item[2] = p + n
            if item[2] == len(toks):
                end.append(rid)
        if not entries:
            continue
        steps.append({"step": len(steps), "entries": entries, "end": end})
        live = [it for it in live if it[2] < len(it[1])]
    return steps


def peak_tokens(steps: List[dict], unit: int = 64) -> int:
    """The most tokens live requests hold at any time, each rounded up to ``unit``."""
    held: Dict[str, int] = {}
    peak = 0
    for st in steps:
        for e in st["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        peak = max(peak, sum((v + unit - 1) // unit * unit for v in held.values()))
        for rid in st["end"]:
            held.pop(rid, None)
    return peak


def collect(steps: List[dict], outputs: Dict[int, "object"], vocab: int):
    """Puts the logits rows of every step back in request order: {id: [rows...]}."""
    import numpy as np
    rows: Dict[str, list] = {}
    for st in steps:
        if st["step"] not in outputs:
            assert all(not e["want"] for e in st["entries"])
            continue
        out = np.asarray(outputs[st["step"]]).reshape(-1, vocab)
        r = 0
        for e in st["entries"]:
            for _ in e["want"]:
                rows.setdefault(e["id"], []).append(out[r])
                r += 1
        assert r == out.shape[0]
    return {rid: np.stack(v) for rid, v in rows.items()}
