"""Ways of cutting the same requests into steps; each yields trace records and, for every
request, where its logits end up.  Used with the engine directly and with bin/trace_run."""
from __future__ import annotations

from typing import Dict, List, Tuple


def whole(requests: Dict[str, List[int]]):
    """Each request alone and whole, all logits wanted."""
    steps = []
    for i, (rid, toks) in enumerate(requests.items()):
        steps.append({"step": i, "entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}], "end": [rid]})
    return steps


def tail_decoded(requests: Dict[str, List[int]], tail: int = 32):
    """Most of a request in one step, its last `tail` tokens one by one."""
    steps, n = [], 0
    for rid, toks in requests.items():
        head = max(1, len(toks) - tail)
        steps.append({"step": n, "entries": [{"id": rid, "tokens": toks[:head], "want": list(range(head))}], "end": []})
        n += 1
        for i in range(head, len(toks)):
            end = [rid] if i == len(toks) - 1 else []
            steps.append({"step": n, "entries": [{"id": rid, "tokens": [toks[i]], "want": [0]}], "end": end})
            n += 1
        if head == len(toks):
            steps[-1]["end"] = [rid]
    return steps


def portions(requests: Dict[str, List[int]], sizes=(2, 3, 5, 8, 13, 21, 34, 2, 7)):
    """Portions of changing size, down to two tokens."""
    steps, n = [], 0
    for rid, toks in requests.items():
        at, k = 0, 0
        while at < len(toks):
            size = min(sizes[k % len(sizes)], len(toks) - at)
            k += 1
            chunk = toks[at:at + size]
            at += size
            steps.append({"step": n, "entries": [{"id": rid, "tokens": chunk, "want": list(range(len(chunk)))}],
                          "end": [rid] if at == len(toks) else []})
            n += 1
    return steps


def mixed(requests: Dict[str, List[int]], max_live: int = 4, prompt_fraction: float = 0.6,
          sizes=(5, 2, 9, 17, 3, 30)):
    """Up to `max_live` requests at a time: each is fed its first part in portions, the rest token by
    token, portions of some beside single tokens of others; a finished request's place is taken
    by the next one, so its pages are used again."""
    waiting = list(requests.items())
    live: List[dict] = []
    steps, n, k = [], 0, 0
    while waiting or live:
        while waiting and len(live) < max_live:
            rid, toks = waiting.pop(0)
            live.append({"id": rid, "toks": toks, "at": 0, "prompt": max(1, int(len(toks) * prompt_fraction))})
        entries, end = [], []
        for i, r in enumerate(live):
            if (n + i) % 5 == 4 and len(live) > 1:
                continue  # now and then a request sits a step out
            if r["at"] < r["prompt"]:
                size = min(sizes[k % len(sizes)], r["prompt"] - r["at"])
                k += 1
            else:
                size = 1
            chunk = r["toks"][r["at"]:r["at"] + size]
            r["at"] += size
            entries.append({"id": r["id"], "tokens": chunk, "want": list(range(len(chunk)))})
            if r["at"] == len(r["toks"]):
                end.append(r["id"])
        live = [r for r in live if r["id"] not in end]
        if entries:
            steps.append({"step": n, "entries": entries, "end": end})
        n += 1
    return steps


def max_live_tokens(steps, round_to: int = 64) -> int:
    """The largest number of tokens live requests hold after any step, each rounded up."""
    held: Dict[str, int] = {}
    worst = 0
    for s in steps:
        for e in s["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        worst = max(worst, sum((v + round_to - 1) // round_to * round_to for v in held.values()))
        for rid in s["end"]:
            held.pop(rid, None)
    return worst


def collect(steps, outputs: Dict[int, "object"]) -> Dict[str, list]:
    """Reassembles, per request, the logits rows in position order.  `outputs[step]` is [wanted, vocab]."""
    rows: Dict[str, list] = {}
    for s in steps:
        if not any(e["want"] for e in s["entries"]):
            continue
        block = outputs[s["step"]]
        at = 0
        for e in s["entries"]:
            for _ in e["want"]:
                rows.setdefault(e["id"], []).append(block[at])
                at += 1
    return rows
