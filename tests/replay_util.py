"""Helpers of the GPU replay tests: schedules, running them, comparing with the plain model."""

from __future__ import annotations

import numpy as np

from mini_infer_amd.engine.trace import (  # noqa: F401  (the schedule families live with the replay tool)
    peak_pages,
    schedule_mixed,
    schedule_portions,
    schedule_prefill_then_decode,
    schedule_whole,
)

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
