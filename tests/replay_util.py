"""Helpers of the GPU replay tests: schedules, running them, comparing with the plain model."""

from __future__ import annotations

import numpy as np

FP32_TOL = 1e-4  # max-abs on logits, float32 engine against the float64 plain model
BF16_REL_TOL = 0.04  # max-abs error allowed as a fraction of the largest |logit|


def assert_close(got: np.ndarray, expected: np.ndarray, dtype: str, what: str = "") -> None:
    assert got.shape == expected.shape, f"{what}: shape {got.shape} != {expected.shape}"
    err = np.abs(got.astype(np.float64) - expected)
    worst = np.unravel_index(np.argmax(err), err.shape)
    limit = FP32_TOL if dtype == "float32" else BF16_REL_TOL * max(1.0, float(np.abs(expected).max()))
    assert err.max() < limit, (
        f"{what} [{dtype}]: max error {err.max():.3e} at row {worst[0]} (limit {limit:.3e}); "
        f"first row over the limit: {int(np.argmax(err.max(axis=1) >= limit))}"
    )


def run_schedule(runner, requests: dict[str, list[int]], schedule: list[dict]) -> dict[str, np.ndarray]:
    """Feed `schedule` (steps of {"feed": {id: n_tokens}, "end": [ids]}) and collect the
    logits of every fed position per request."""
    from mini_infer_amd.engine import StepEntry

    fed = {rid: 0 for rid in requests}
    rows: dict[str, list[np.ndarray]] = {rid: [] for rid in requests}
    for step in schedule:
        entries = []
        for rid, count in step["feed"].items():
            tokens = requests[rid][fed[rid] : fed[rid] + count]
            assert len(tokens) == count, f"schedule feeds past the end of {rid}"
            entries.append(StepEntry(rid, tokens, list(range(count))))
            fed[rid] += count
        logits = runner.step(entries).cpu().numpy()
        at = 0
        for entry in entries:
            rows[entry.request_id].append(logits[at : at + len(entry.tokens)])
            at += len(entry.tokens)
        assert at == logits.shape[0]
        for rid in step.get("end", []):
            runner.free_request(rid)
    return {rid: np.concatenate(parts, axis=0) for rid, parts in rows.items() if parts}


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
