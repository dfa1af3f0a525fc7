"""Traces for the replay tests: the same requests whole, with the last tokens
decoded one by one, in portions of changing size, and mixed with other requests
under a pool so small that pages are used again."""
from __future__ import annotations

from typing import Dict, List

import torch


def random_tokens(vocab: int, n: int, seed: int) -> List[int]:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def whole(requests: Dict[str, List[int]]):
    """Each request alone, all of it in one step, every position wanted."""
    steps = []
    for i, (rid, toks) in enumerate(requests.items()):
        steps.append({"step": i, "entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}], "end": [rid]})
    return steps


def tail_decoded(requests: Dict[str, List[int]], tail: int = 32):
    """Most of a request in one step, its last `tail` tokens one by one."""
    steps, n = [], 0
    for rid, toks in requests.items():
        head = max(len(toks) - tail, 1)
        steps.append({"step": n, "entries": [{"id": rid, "tokens": toks[:head], "want": list(range(head))}], "end": []})
        n += 1
        for i in range(head, len(toks)):
            steps.append({"step": n, "entries": [{"id": rid, "tokens": [toks[i]], "want": [0]}],
                          "end": [rid] if i == len(toks) - 1 else []})
            n += 1
        if head == len(toks):
            steps[-1]["end"] = [rid]
    return steps


def portions(requests: Dict[str, List[int]], sizes=(7, 2, 16, 3, 2, 33, 5, 2, 64, 2, 19)):
    """Portions of changing size, down to two tokens."""
    steps, n = [], 0
    for rid, toks in requests.items():
        pos, k = 0, 0
        while pos < len(toks):
            c = min(sizes[k % len(sizes)], len(toks) - pos)
            k += 1
            steps.append({"step": n, "entries": [{"id": rid, "tokens": toks[pos:pos + c], "want": list(range(c))}],
                          "end": [rid] if pos + c == len(toks) else []})
            pos += c
            n += 1
    return steps


def mixed(requests: Dict[str, List[int]], live: int = 4, prefill_sizes=(5, 2, 11, 3, 17), decode_after: float = 0.5):
    """Up to `live` requests at a time: each is fed in portions up to a part of its
    length and then token by token, portions of some beside single tokens of others;
    a request that ends makes room (and pages) for the next."""
    order = list(requests)
    pos = {rid: 0 for rid in order}
    active: List[str] = []
    steps, n, k = [], 0, 0
    waiting = list(order)
    while waiting or active:
        while waiting and len(active) < live:
            active.append(waiting.pop(0))
        entries, ended = [], []
        for j, rid in enumerate(list(active)):
            toks = requests[rid]
            if (n + j) % 5 == 4 and len(active) > 1:
                continue            # left out of this step; it goes on later
            if pos[rid] < int(len(toks) * decode_after):
                c = min(prefill_sizes[k % len(prefill_sizes)], len(toks) - pos[rid])
                k += 1
            else:
                c = 1
            entries.append({"id": rid, "tokens": toks[pos[rid]:pos[rid] + c], "want": list(range(c))})
            pos[rid] += c
            if pos[rid] == len(toks):
                ended.append(rid)
                active.remove(rid)
        if entries:
            steps.append({"step": n, "entries": entries, "end": ended})
            n += 1
    return steps


def collect(steps, outputs):
    """{request: {position: logits row}} from a replay's per-step outputs."""
    rows: Dict[str, Dict[int, object]] = {}
    pos: Dict[str, int] = {}
    for step, out in zip(steps, outputs):
        r = 0
        for e in step["entries"]:
            start = pos.get(e["id"], 0)
            for w in e["want"]:
                rows.setdefault(e["id"], {})[start + w] = out[r]
                r += 1
            pos[e["id"]] = start + len(e["tokens"])
        for rid in step["end"]:
            pos.pop(rid, None)
    return rows


def live_token_need(steps, round_to: int = 64) -> int:
    """The most tokens live requests hold at any time, each rounded up to `round_to`."""
    held: Dict[str, int] = {}
    worst = 0
    for step in steps:
        for e in step["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        worst = max(worst, sum(-(-v // round_to) * round_to for v in held.values()))
        for rid in step["end"]:
            held.pop(rid, None)
    return worst
