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
# bfloat16 against a yardstick: the plain model with every stored tensor rounded to bfloat16
# and all arithmetic exact shows how far bfloat16 storage alone moves the logits of this very
# input.  The engine (which adds float32 summation and, on the matrix cores, probabilities in
# bfloat16) may err at most twice as far at its worst logit and one and a half times as far at
# the 99th percentile.  Measured: 0.9-1.6 times at the worst logit, 1.0-1.2 times at the 99th
# percentile, on all tiny configurations under all schedules.
BF16_MAX_FACTOR = 2.0
BF16_P99_FACTOR = 1.5
BF16_REL_TOL = 0.04  # for parts defined in tests, which have no yardstick: share of the largest |logit|


class Oracle:
    """Logits of the plain model for one request: `exact`, and `rounded` (bfloat16 storage, exact
    arithmetic).  Indexing gives the rows asked for; the yardstick's statistics stay those of
    the whole request, so that a comparison of few rows is not at the mercy of those rows."""

    def __init__(self, exact: np.ndarray, rounded: np.ndarray, yard: tuple[float, float] | None = None) -> None:
        self.exact, self.rounded = exact, rounded
        if yard is None:
            moved = np.abs(rounded - exact)
            yard = (float(moved.max()), float(np.percentile(moved, 99)))
        self.yard_max, self.yard_p99 = yard

    @property
    def shape(self):
        return self.exact.shape

    def __getitem__(self, rows) -> "Oracle":
        return Oracle(self.exact[rows], self.rounded[rows], (self.yard_max, self.yard_p99))


def oracle(cfg: dict, weights: dict, tokens, **kwargs) -> Oracle:
    """Exact and bfloat16-storage logits of the plain NumPy model for one request."""
    import plain_llama

    ids = np.asarray(tokens)
    return Oracle(
        plain_llama.llama_logits(cfg, weights, ids, **kwargs),
        plain_llama.llama_logits(cfg, weights, ids, store=plain_llama.bf16_round, **kwargs),
    )


def assert_close(got: np.ndarray, expected, dtype: str, what: str = "") -> None:
    """`expected`: an `Oracle`, or an array (then bfloat16 falls back to a share of the largest logit)."""
    yardstick = expected if isinstance(expected, Oracle) else None
    exact = expected.exact if yardstick is not None else expected
    assert got.shape == exact.shape, f"{what}: shape {got.shape} != {exact.shape}"
    err = np.abs(got.astype(np.float64) - exact)
    worst = np.unravel_index(np.argmax(err), err.shape)
    if dtype == "float32":
        limit = FP32_TOL
    elif yardstick is not None:
        limit = BF16_MAX_FACTOR * yardstick.yard_max
        if err.size >= 2000:
            p99, p99_limit = float(np.percentile(err, 99)), BF16_P99_FACTOR * yardstick.yard_p99
            assert p99 < p99_limit, f"{what} [{dtype}]: 99th percentile of the error {p99:.3e} (limit {p99_limit:.3e})"
    else:
        limit = BF16_REL_TOL * max(1.0, float(np.abs(exact).max()))
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
