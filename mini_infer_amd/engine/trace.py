"""Schedules for trace replay: ways of cutting the same requests into steps.

Token ids are given, so the logits at a position must be the same (beyond rounding)
under every schedule.  A schedule is a list of steps `{"feed": {request id: number of its
next tokens}, "end": [request ids]}`; `to_trace_lines` turns one into the JSON lines that
the replay program reads (`bin/trace_run`, `python -m mini_infer_amd replay`), asking for
the logits of every fed token.

Four families: each request alone and whole; most of it in one step and the last tokens
one by one; portions of changing size down to two tokens; and mixed, up to four live
requests, portions of some beside single tokens of others, a finished request's pages
handed on to the next.
"""

from __future__ import annotations

import json

import numpy as np


def schedule_whole(requests: dict[str, list[int]]) -> list[dict]:
    return [{"feed": {rid: len(tokens)}, "end": [rid]} for rid, tokens in requests.items()]


def schedule_prefill_then_decode(requests: dict[str, list[int]], tail: int = 32) -> list[dict]:
    steps = []
    for rid, tokens in requests.items():
        head = max(1, len(tokens) - tail)
        steps.append({"feed": {rid: head}})
        for _ in range(len(tokens) - head):
            steps.append({"feed": {rid: 1}})
        steps[-1]["end"] = [rid]
    return steps


def schedule_portions(requests: dict[str, list[int]], seed: int) -> list[dict]:
    """Each request alone, in portions of changing size, many of them two tokens."""
    rng = np.random.default_rng(seed)
    sizes = [2, 7, 2, 13, 3, 2, 5, 29, 2, 1, 17, 4]
    steps = []
    for rid, tokens in requests.items():
        left = len(tokens)
        k = int(rng.integers(0, len(sizes)))
        while left > 0:
            count = min(sizes[k % len(sizes)], left)
            steps.append({"feed": {rid: count}})
            left -= count
            k += 1
        steps[-1]["end"] = [rid]
    return steps


def schedule_mixed(requests: dict[str, list[int]], seed: int, max_live: int = 4, tail: int = 32) -> list[dict]:
    """Up to `max_live` requests at a time: portions of some beside single tokens of others.

    A request feeds portions until `tail` tokens are left, then one token a step;
    now and then a request sits a step out.  A finished request ends at once and
    the next one starts in the following step, so pages are handed on.
    """
    rng = np.random.default_rng(seed)
    waiting = list(requests)
    live: list[str] = []
    left = {rid: len(tokens) for rid, tokens in requests.items()}
    steps = []
    while waiting or live:
        while waiting and len(live) < max_live:
            live.append(waiting.pop(0))
        feed: dict[str, int] = {}
        for rid in live:
            if len(live) > 1 and rng.random() < 0.15:
                continue  # sits this step out
            if left[rid] > tail:
                count = int(min(left[rid] - tail, rng.choice([2, 2, 3, 5, 8, 16, 31])))
            else:
                count = 1
            feed[rid] = count
        if not feed:
            feed[live[0]] = 1 if left[live[0]] <= tail else 2
        ended = []
        for rid, count in feed.items():
            left[rid] -= count
            if left[rid] == 0:
                ended.append(rid)
        for rid in ended:
            live.remove(rid)
        steps.append({"feed": feed, "end": ended})
    return steps


def peak_pages(requests: dict[str, list[int]], schedule: list[dict], page_size: int) -> int:
    """Most pages held at once under `schedule` (requests hold ceil(len/page) pages)."""
    fed = {rid: 0 for rid in requests}
    live: set[str] = set()
    peak = 0
    for step in schedule:
        for rid, count in step["feed"].items():
            fed[rid] += count
            live.add(rid)
        peak = max(peak, sum(-(-fed[rid] // page_size) for rid in live))
        for rid in step.get("end", []):
            live.discard(rid)
    return peak


FAMILIES = ("whole", "decode", "portions", "mixed")


def make_schedule(family: str, requests: dict[str, list[int]], seed: int = 0, tail: int = 32) -> list[dict]:
    if family == "whole":
        return schedule_whole(requests)
    if family == "decode":
        return schedule_prefill_then_decode(requests, tail=tail)
    if family == "portions":
        return schedule_portions(requests, seed)
    if family == "mixed":
        return schedule_mixed(requests, seed, tail=tail)
    raise ValueError(f"no schedule family {family!r}; there are {FAMILIES}")


def to_trace_lines(requests: dict[str, list[int]], schedule: list[dict]) -> list[str]:
    """The schedule as the replay program's input, logits wanted at every fed token."""
    fed = {rid: 0 for rid in requests}
    lines = []
    for number, step in enumerate(schedule):
        entries = []
        for rid, count in step["feed"].items():
            tokens = requests[rid][fed[rid] : fed[rid] + count]
            if len(tokens) != count:
                raise ValueError(f"the schedule feeds past the end of request {rid!r}")
            entries.append({"id": rid, "tokens": tokens, "want": list(range(count))})
            fed[rid] += count
        lines.append(json.dumps({"step": number, "entries": entries, "end": list(step.get("end", []))}))
    return lines
