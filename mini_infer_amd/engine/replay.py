"""Trace replay: feed given token ids through the model step by step and write logits.

It samples nothing.  It drives the same runner, step function, cache manager and
kernels that generation uses.  Steps come from standard input, one JSON object a
line:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

For a step with wanted places, `OUT/<step>.f32` holds the logits [wanted, vocab]
as little-endian float32, in the order of the entries and of `want`.  After each
step `done <step>` is printed and flushed.  When the input ends, requests still live are
ended, and the program checks that every page of the pool is free again (exit code 1 if
one is lost, else 0).
"""

from __future__ import annotations

import argparse
import json
import sys
from pathlib import Path

DEFAULT_REPLAY_BLOCK_SIZE = 16


def build_parser() -> argparse.ArgumentParser:
    parser = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    parser.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    parser.add_argument("--dtype", choices=("bfloat16", "float32"), default="bfloat16")
    parser.add_argument("--out", required=True, help="folder the logits files are written to")
    parser.add_argument(
        "--max-tokens",
        type=int,
        required=True,
        help="most tokens live requests hold at any time (each rounded up to a multiple of 64)",
    )
    parser.add_argument("--block-size", type=int, default=DEFAULT_REPLAY_BLOCK_SIZE)
    parser.add_argument("--max-concurrent", type=int, default=64)
    parser.add_argument("--device", default="cuda:0")
    return parser


def run(args: argparse.Namespace, lines=None, out=None) -> int:
    lines = sys.stdin if lines is None else lines
    out = sys.stdout if out is None else out

    # building the kernels (first call in a fresh checkout) reports on stderr
    from mini_infer_amd.ops import library

    library.load()

    import numpy as np

    from mini_infer_amd.engine.batch import StepEntry
    from mini_infer_amd.engine.model_runner import ModelRunner

    if args.block_size <= 0 or 64 % args.block_size != 0:
        raise SystemExit("--block-size must divide 64, so that --max-tokens counts whole pages")
    num_blocks = max(1, -(-args.max_tokens // args.block_size))
    runner = ModelRunner.from_pretrained(
        args.model,
        device=args.device,
        dtype=args.dtype,
        num_blocks=num_blocks,
        block_size=args.block_size,
        max_concurrent=args.max_concurrent,
    )
    out_dir = Path(args.out)
    out_dir.mkdir(parents=True, exist_ok=True)

    for line in lines:
        line = line.strip()
        if not line:
            continue
        record = json.loads(line)
        step = record["step"]
        entries = [
            StepEntry(e["id"], e["tokens"], e.get("want", ()))
            for e in record.get("entries", [])
        ]
        logits = runner.step(entries)
        if logits.shape[0] > 0:
            values = logits.detach().to("cpu").numpy().astype("<f4", copy=False)
            np.ascontiguousarray(values).tofile(str(out_dir / f"{step}.f32"))
        for request_id in record.get("end", []):
            if runner.has_request(request_id):
                runner.free_request(request_id)
        print(f"done {step}", file=out, flush=True)

    # The input has ended: what the trace left live is given back, and then every page
    # must be free again and none held twice: a page lost on the way is the engine's
    # fault, never the trace's, and the only reason to end with another code than 0.
    for request_id in runner.cache.live_requests():
        runner.free_request(request_id)
    try:
        runner.cache.check()
        lost = num_blocks - runner.num_free_blocks()
        if lost:
            raise AssertionError(f"{lost} of {num_blocks} pages are still held after every request ended")
    except AssertionError as err:
        print(f"trace_run: the cache is not whole at the end of the trace: {err}", file=sys.stderr, flush=True)
        return 1
    return 0


def main(argv: list[str] | None = None) -> int:
    return run(build_parser().parse_args(argv))


if __name__ == "__main__":
    sys.exit(main())
