"""Command line: `python -m mini_infer_amd <command>`.

  generate        tokens from a model folder (prompt as text or token ids)
  random-weights  write a model folder (config.json + model.safetensors) from a
                  config.json and a seed
  replay          the trace replay tool (same as bin/trace_run)
  make-trace      print a trace for it: random token ids cut into steps by one of the
                  schedule families (whole, decode, portions, mixed)

Engine options carry the reference's constructor names (engine/model_runner.py:84-100,
scheduler/continuous_scheduler.py:168-177): --num-blocks, --block-size,
--max-concurrent, --chunk-size, --decode-headroom-blocks; sampling options those of
its `SamplingParams` and completion request (engine/sampler.py:7-21,
api/schemas.py:23-30): --max-tokens, --temperature, --top-k, --top-p.
"""

from __future__ import annotations

import argparse
import json
import sys

from mini_infer_amd.config import EngineConfig


def _add_engine_options(parser: argparse.ArgumentParser) -> None:
    parser.add_argument("--dtype", choices=("bfloat16", "float32"), default="bfloat16")
    parser.add_argument("--device", default="cuda:0")
    defaults = EngineConfig()
    parser.add_argument("--num-blocks", type=int, default=defaults.num_blocks)
    parser.add_argument("--block-size", type=int, default=defaults.block_size)
    parser.add_argument("--max-concurrent", type=int, default=defaults.max_concurrent)
    parser.add_argument("--max-num-batched-tokens", type=int, default=defaults.max_num_batched_tokens)
    parser.add_argument("--chunk-size", type=int, default=defaults.chunk_size)
    parser.add_argument("--decode-headroom-blocks", type=int, default=defaults.decode_headroom_blocks)
    parser.add_argument("--trace-out", default=None, help="write a Chrome trace of the steps to this file")


def _generate(args: argparse.Namespace) -> int:
    from mini_infer_amd.engine.llm import LLM
    from mini_infer_amd.sampling.params import SamplingParams

    prompts: list = []
    for text in args.prompt or []:
        prompts.append(text)
    for ids in args.prompt_ids or []:
        prompts.append([int(t) for t in ids.replace(",", " ").split()])
    if not prompts:
        raise SystemExit("give --prompt TEXT or --prompt-ids '1 2 3' (either may repeat)")
    from mini_infer_amd.config import EngineConfig

    engine = EngineConfig(
        dtype=args.dtype,
        device=args.device,
        num_blocks=args.num_blocks,
        block_size=args.block_size,
        max_concurrent=args.max_concurrent,
        max_num_batched_tokens=args.max_num_batched_tokens,
        chunk_size=args.chunk_size,
        decode_headroom_blocks=args.decode_headroom_blocks,
        seed=args.seed,
        trace_out=args.trace_out,
    )
    llm = LLM(args.model, engine=engine)
    params = SamplingParams(
        temperature=args.temperature,
        top_k=args.top_k,
        top_p=args.top_p,
        seed=args.seed if args.temperature > 0 else None,
        ignore_eos=args.ignore_eos,
    )
    for prompt, result in zip(prompts, llm.generate(prompts, params, max_tokens=args.max_tokens)):
        print(
            json.dumps(
                {
                    "prompt": prompt,
                    "tokens": result.tokens,
                    "text": result.text,
                    "finish_reason": result.finish_reason,
                    "prompt_tokens": result.prompt_tokens,
                }
            ),
            flush=True,
        )
    return 0


def _random_weights(args: argparse.Namespace) -> int:
    from mini_infer_amd.config import read_config_json
    from mini_infer_amd.weights import write_random_model

    out = write_random_model(
        read_config_json(args.config),
        args.seed,
        args.out,
        std=args.std,
        norm_jitter=args.norm_jitter,
        dtype=args.dtype,
    )
    print(out)
    return 0


def _replay(args: argparse.Namespace) -> int:
    from mini_infer_amd.engine import replay

    return replay.run(args)


def _make_trace(args: argparse.Namespace) -> int:
    import numpy as np

    from mini_infer_amd.engine import trace

    rng = np.random.default_rng(args.seed)
    lengths = [int(n) for n in args.lengths.replace(",", " ").split()]
    requests = {f"r{i}": rng.integers(0, args.vocab_size, size=n).tolist() for i, n in enumerate(lengths)}
    schedule = trace.make_schedule(args.family, requests, seed=args.seed, tail=args.tail)
    for line in trace.to_trace_lines(requests, schedule):
        print(line)
    print(
        f"{len(schedule)} steps, at most {trace.peak_pages(requests, schedule, 64) * 64} tokens live "
        f"(each request rounded up to 64)",
        file=sys.stderr,
    )
    return 0


def main(argv: list[str] | None = None) -> int:
    parser = argparse.ArgumentParser(prog="python -m mini_infer_amd", description=__doc__.split("\n\n")[0])
    commands = parser.add_subparsers(dest="command", required=True)

    gen = commands.add_parser("generate", help="generate tokens from a model folder")
    gen.add_argument("--model", required=True, help="folder with config.json and safetensors")
    gen.add_argument("--prompt", action="append", help="text prompt (needs tokenizer.json in the folder)")
    gen.add_argument("--prompt-ids", action="append", help="token ids, separated by spaces or commas")
    gen.add_argument("--max-tokens", type=int, default=16)
    gen.add_argument("--temperature", type=float, default=0.0)
    gen.add_argument("--top-k", type=int, default=0)
    gen.add_argument("--top-p", type=float, default=1.0)
    gen.add_argument("--seed", type=int, default=0)
    gen.add_argument("--ignore-eos", action="store_true")
    _add_engine_options(gen)
    gen.set_defaults(run=_generate)

    rnd = commands.add_parser("random-weights", help="write a random-weight model folder")
    rnd.add_argument("--config", required=True, help="a config.json (or a folder holding one)")
    rnd.add_argument("--seed", type=int, default=0)
    rnd.add_argument("--out", required=True)
    rnd.add_argument("--dtype", choices=("bfloat16", "float32"), default="bfloat16")
    rnd.add_argument("--std", type=float, default=0.02)
    rnd.add_argument("--norm-jitter", type=float, default=0.1)
    rnd.set_defaults(run=_random_weights)

    from mini_infer_amd.engine.replay import build_parser as replay_parser

    rep = commands.add_parser("replay", parents=[replay_parser()], add_help=False, help="trace replay")
    rep.set_defaults(run=_replay)

    from mini_infer_amd.engine.trace import FAMILIES

    mk = commands.add_parser("make-trace", help="print a replay trace of random token ids")
    mk.add_argument("--family", choices=FAMILIES, default="mixed")
    mk.add_argument("--lengths", required=True, help="request lengths, e.g. '150,40,97,1'")
    mk.add_argument("--vocab-size", type=int, required=True)
    mk.add_argument("--seed", type=int, default=0)
    mk.add_argument("--tail", type=int, default=32, help="tokens at the end of a request fed one by one")
    mk.set_defaults(run=_make_trace)

    args = parser.parse_args(argv)
    return args.run(args)


if __name__ == "__main__":
    sys.exit(main())
