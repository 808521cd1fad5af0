"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--batch B] [--sizes 8b|3b|70b]
                    [--max-context N] [--serving] [--reference-workload]
                    [--long-context 8192,32768,131072] [--attention TOKENS]

Default workload: the layer sizes of Llama 3.1 8B with random bfloat16 weights
made on the device, a batch of 8 requests with 2,048-token uniform-random prompts,
decoded greedily from position 2,048 on; one "step" is one decode step of the whole
batch (step function + greedy choice on the device + ids back to the host, which reads
them one step late: the next step takes its tokens from the device).  The
line it prints also holds the prefill rate of one 2,048-token prompt, the decode
rates at batch 1 and 64, and the decode step's share of the HBM roofline.
"""

from __future__ import annotations

import argparse
import json
import sys
import time

PEAK_HBM_GBS = 8000.0  # MI355X HBM3E, GB/s
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

LLAMA_31_8B = {
    "architectures": ["LlamaForCausalLM"],
    "num_hidden_layers": 32,
    "hidden_size": 4096,
    "num_attention_heads": 32,
    "num_key_value_heads": 8,
    "head_dim": 128,
    "intermediate_size": 14336,
    "vocab_size": 128256,
    "rope_theta": 500000.0,
    "rope_scaling": {
        "rope_type": "llama3",
        "factor": 8.0,
        "low_freq_factor": 1.0,
        "high_freq_factor": 4.0,
        "original_max_position_embeddings": 8192,
    },
    "rms_norm_eps": 1e-5,
    "tie_word_embeddings": False,
    "max_position_embeddings": 131072,
}
# the serving workload's model (--serving): Llama 3.2 3B layer sizes
LLAMA_32_3B = {
    "architectures": ["LlamaForCausalLM"],
    "num_hidden_layers": 28,
    "hidden_size": 3072,
    "num_attention_heads": 24,
    "num_key_value_heads": 8,
    "head_dim": 128,
    "intermediate_size": 8192,
    "vocab_size": 128256,
    "rope_theta": 500000.0,
    "rope_scaling": {
        "rope_type": "llama3",
        "factor": 32.0,
        "low_freq_factor": 1.0,
        "high_freq_factor": 4.0,
        "original_max_position_embeddings": 8192,
    },
    "rms_norm_eps": 1e-5,
    "tie_word_embeddings": True,
    "max_position_embeddings": 131072,
}
LLAMA_31_70B = dict(
    LLAMA_31_8B, num_hidden_layers=80, hidden_size=8192, num_attention_heads=64, intermediate_size=28672
)
LLAMA_32_1B = dict(
    LLAMA_32_3B, num_hidden_layers=16, hidden_size=2048, num_attention_heads=32, head_dim=64, intermediate_size=8192
)
SIZES = {"8b": ("Llama-3.1-8B", LLAMA_31_8B), "3b": ("Llama-3.2-3B", LLAMA_32_3B), "70b": ("Llama-3.1-70B", LLAMA_31_70B),
         "1b": ("Llama-3.2-1B", LLAMA_32_1B)}
PROMPT_LEN = 2048
BLOCK_SIZE = 16


def weight_bytes(cfg: dict, elem: int) -> int:
    """Bytes of every weight a decode step reads once (the embedding table is only gathered)."""
    h, i, v = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    d = cfg["head_dim"]
    q, kv = cfg["num_attention_heads"] * d, cfg["num_key_value_heads"] * d
    per_layer = (q + 2 * kv) * h + h * q + 2 * i * h + h * i + 2 * h
    return (cfg["num_hidden_layers"] * per_layer + v * h + h) * elem


def kv_bytes_per_token(cfg: dict, elem: int) -> int:
    return 2 * cfg["num_hidden_layers"] * cfg["num_key_value_heads"] * cfg["head_dim"] * elem


def prefill_flops(cfg: dict, tokens: int) -> float:
    h, i, v = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    d = cfg["head_dim"]
    q, kv = cfg["num_attention_heads"] * d, cfg["num_key_value_heads"] * d
    per_layer_params = (q + 2 * kv) * h + h * q + 2 * i * h + h * i
    linear = 2.0 * tokens * cfg["num_hidden_layers"] * per_layer_params
    # causal attention: QK^T and PV over tokens*(tokens+1)/2 query-key pairs per head
    attention = 4.0 * (tokens * (tokens + 1) / 2) * d * cfg["num_attention_heads"] * cfg["num_hidden_layers"]
    head = 2.0 * v * h
    return linear + attention + head


def measure_serving(dtype: str, mixed_graphs: bool = True) -> dict:
    """Continuous batching through the scheduler: 32 concurrent requests, prompt lengths
    uniform in [128, 4096] of uniform-random ids, 256 greedy tokens each, a 2,048-token
    budget per step, at Llama-3.2-3B layer sizes with random weights."""
    import numpy as np
    import torch

    from mini_infer_amd import ContinuousScheduler, ModelRunner, Request, SamplingParams

    requests_n, new_tokens, longest = 32, 256, 4096
    pages = requests_n * (-(-(longest + new_tokens) // BLOCK_SIZE)) + 64
    runner = ModelRunner.from_random(
        LLAMA_32_3B, seed=0, dtype=dtype, num_blocks=pages, block_size=BLOCK_SIZE, max_concurrent=requests_n
    )
    import os

    runner.decode_graphs.mixed = mixed_graphs
    scheduler = ContinuousScheduler(
        runner, max_concurrent=requests_n, chunk_size=2048, max_num_batched_tokens=2048, trace_out=os.devnull
    )
    rng = np.random.default_rng(3)

    def workload() -> list:
        lengths = rng.integers(128, longest + 1, size=requests_n)
        return [
            Request(rng.integers(0, LLAMA_32_3B["vocab_size"], size=int(n)).tolist(), SamplingParams(ignore_eos=True), new_tokens)
            for n in lengths
        ]

    scheduler.run_all(workload()[:4])  # warm-up: kernels built, graphs of the first buckets recorded
    batch = workload()
    prompt_tokens = sum(len(r.prompt) for r in batch)
    steps_before = scheduler.stats["steps"]
    events_before = len(scheduler.trace_events())
    torch.cuda.synchronize()
    started = time.perf_counter()
    results = scheduler.run_all(batch)
    torch.cuda.synchronize()
    seconds = time.perf_counter() - started
    generated = sum(len(r.tokens) for r in results)
    # host time from one step to the next, by kind of step (with asynchronous sampling a
    # step's time shows in the step after it, so the kinds blur at their borders)
    step_ms: dict[str, list[float]] = {}
    for event in scheduler.trace_events()[events_before:]:
        step_ms.setdefault(event["args"]["phase"], []).append(event["dur"] / 1e3)
    histogram = {
        kind: {"steps": len(v), "p50_ms": round(float(np.percentile(v, 50)), 2), "p90_ms": round(float(np.percentile(v, 90)), 2),
               "max_ms": round(max(v), 2)}
        for kind, v in step_ms.items()
    }
    return {
        "step_ms": histogram,
        "model": "Llama-3.2-3B layer sizes",
        "requests": requests_n,
        "prompt_tokens": prompt_tokens,
        "generated_tokens": generated,
        "seconds": round(seconds, 3),
        "steps": scheduler.stats["steps"] - steps_before,
        "generated_tok_s": round(generated / seconds, 1),
        "total_tok_s": round((prompt_tokens + generated) / seconds, 1),
        "preemptions": scheduler.stats["preemptions"],
    }


def measure_reference_workload(dtype: str, mixed_graphs: bool = True, sizes: str = "8b") -> dict:
    """The workload the reference publishes numbers for (docs/benchmarks/
    2026-11-05-model-metrics.md:19-41; scripts/bench/modal_model_metrics.py:58-62, :239-252):
    1,024-token prompts, 128 greedy tokens, 2,048 pages of 16, 16 seats.  Time to the first
    token and decode speed of one request at a time (median of 5), then 16 requests that
    start together.  Here: Llama-3.1-8B layer sizes with random weights, prompts of random
    ids (no request stops early), and up to 4,096 tokens a step, which is what a step of the
    reference can carry in this setting (16 requests x its chunk of 256 each; it has no
    budget over all requests).  Then short prompts, where the host's share of a step shows:
    16 requests of 16 tokens each that start together, 64 tokens each."""
    import statistics

    import numpy as np
    import torch

    from mini_infer_amd import ContinuousScheduler, ModelRunner, Request, SamplingParams

    prompt_len, new_tokens, concurrency = 1024, 128, 16
    model_name, model = SIZES[sizes]
    runner = ModelRunner.from_random(
        model, seed=0, dtype=dtype, num_blocks=2048, block_size=BLOCK_SIZE, max_concurrent=concurrency
    )
    runner.decode_graphs.mixed = mixed_graphs
    scheduler = ContinuousScheduler(runner, max_concurrent=concurrency, chunk_size=4096, max_num_batched_tokens=4096)
    rng = np.random.default_rng(5)

    def request(length: int = prompt_len, tokens: int = new_tokens) -> Request:
        ids = rng.integers(0, model["vocab_size"], size=length).tolist()
        return Request(ids, SamplingParams(ignore_eos=True), tokens)

    def timed(requests: list) -> list[dict]:
        """Drive the engine from here; per request: submit, first token and last token times, tokens."""
        handles, marks = [], []
        for r in requests:
            marks.append({"submit": time.perf_counter(), "first": None, "last": None, "tokens": 0})
            handles.append(scheduler.submit(r))
        while not all(h.done() for h in handles):
            scheduler.step()
            now = time.perf_counter()
            for h, mark in zip(handles, marks):
                tokens = sum(1 for step in h.steps() if step.finish_reason is None)
                if tokens > mark["tokens"]:
                    mark["tokens"], mark["last"] = tokens, now
                    if mark["first"] is None:
                        mark["first"] = now
        return marks

    timed([request() for _ in range(2)])  # warm-up: graphs of the buckets recorded
    timed([request() for _ in range(concurrency)])
    single = [timed([request()])[0] for _ in range(5)]
    torch.cuda.synchronize()
    batch = timed([request() for _ in range(concurrency)])
    torch.cuda.synchronize()
    seconds = max(m["last"] for m in batch) - min(m["submit"] for m in batch)
    # short prompts: requests arrive one step apart (1, 2, 3, ... live), so that steps of a few
    # tokens with a prompt among single tokens are what runs, then all 16 at once
    def staggered() -> list[dict]:
        handles, marks = [], []
        while len(handles) < concurrency or not all(h.done() for h in handles):
            if len(handles) < concurrency:
                marks.append({"submit": time.perf_counter(), "first": None, "last": None, "tokens": 0})
                handles.append(scheduler.submit(request(16, 64)))
            scheduler.step()
            now = time.perf_counter()
            for h, mark in zip(handles, marks):
                tokens = sum(1 for step in h.steps() if step.finish_reason is None)
                if tokens > mark["tokens"]:
                    mark["tokens"], mark["last"] = tokens, now
                    if mark["first"] is None:
                        mark["first"] = now
        return marks

    staggered()  # warm-up
    timed([request(16, 64) for _ in range(concurrency)])
    torch.cuda.synchronize()
    short = timed([request(16, 64) for _ in range(concurrency)])
    short_seconds = max(m["last"] for m in short) - min(m["submit"] for m in short)
    torch.cuda.synchronize()
    arriving = staggered()
    arriving_seconds = max(m["last"] for m in arriving) - min(m["submit"] for m in arriving)
    return {
        "model": model_name + " layer sizes",
        "mixed_steps_recorded": mixed_graphs,
        "short_prompts_16x16_tok_s": round(sum(m["tokens"] for m in short) / short_seconds, 1),
        "short_prompts_16x16_ttft_ms": round(statistics.median((m["first"] - m["submit"]) * 1e3 for m in short), 2),
        "short_prompts_arriving_tok_s": round(sum(m["tokens"] for m in arriving) / arriving_seconds, 1),
        "short_prompts_arriving_ttft_ms": round(statistics.median((m["first"] - m["submit"]) * 1e3 for m in arriving), 2),
        "prompt_tokens": prompt_len,
        "new_tokens": new_tokens,
        "tokens_per_step": 4096,
        "ttft_ms": round(statistics.median((m["first"] - m["submit"]) * 1e3 for m in single), 2),
        "decode_tok_s": round(statistics.median((m["tokens"] - 1) / (m["last"] - m["first"]) for m in single), 1),
        "throughput_tok_s_16": round(sum(m["tokens"] for m in batch) / seconds, 1),
        "ttft_at_16_ms": round(statistics.median((m["first"] - m["submit"]) * 1e3 for m in batch), 1),
    }


def measure_attention(tokens: int, batch: int, repeats: int, sizes: dict) -> dict:
    """The attention kernel alone at the head sizes of `sizes`, on random keys, values and
    queries in shuffled pages (the workload of the hardware-counter runs under `profiles/`):
    with `batch` == 0 one whole prompt of `tokens` tokens (prefill shape, causal), else one
    token of each of `batch` requests over `tokens` keys (decode shape)."""
    import math

    import torch

    from mini_infer_amd import ops

    device = "cuda:0"
    q_heads, kv_heads, head_dim = sizes["num_attention_heads"], sizes["num_key_value_heads"], sizes["head_dim"]
    requests = max(1, batch)
    pages_each = -(-tokens // BLOCK_SIZE)
    pages = requests * pages_each
    keys = (torch.randn(pages, kv_heads, BLOCK_SIZE, head_dim, device=device) * 0.5).bfloat16()
    values = (torch.randn(pages, kv_heads, head_dim, BLOCK_SIZE, device=device) * 0.5).bfloat16()  # transposed pages
    table = torch.randperm(pages, device=device).int().view(requests, pages_each).contiguous()
    if batch == 0:
        rows, cu = tokens, [0, tokens]
        positions = torch.arange(tokens, dtype=torch.int32, device=device)
        token_request = torch.zeros(tokens, dtype=torch.int32, device=device)
        flops = 4.0 * head_dim * q_heads * tokens * (tokens + 1) / 2
        moved = 2.0 * tokens * kv_heads * head_dim * 2
    else:
        rows, cu = batch, list(range(batch + 1))
        positions = torch.full((batch,), tokens - 1, dtype=torch.int32, device=device)
        token_request = torch.arange(batch, dtype=torch.int32, device=device)
        flops = 4.0 * head_dim * q_heads * tokens * batch
        moved = 2.0 * tokens * kv_heads * head_dim * 2 * batch
    queries = torch.randn(rows, q_heads * head_dim, device=device).bfloat16()
    cu_device = torch.tensor(cu, dtype=torch.int32, device=device)

    def call() -> None:
        ops.paged_attention(
            queries, keys, values, table, token_request, positions, cu_device, cu, q_heads=q_heads,
            kv_heads=kv_heads, head_dim=head_dim, scale=1 / math.sqrt(head_dim), window=None,
            max_seq_len=tokens, v_transposed=True,
        )

    call()
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(repeats):
        call()
    end.record()
    torch.cuda.synchronize()
    seconds = start.elapsed_time(end) / 1e3 / repeats
    return {
        "kernel": "paged attention, " + ("one prompt (prefill shape)" if batch == 0 else f"{batch} single tokens (decode shape)"),
        "tokens": tokens, "q_heads": q_heads, "kv_heads": kv_heads, "head_dim": head_dim,
        "us": round(seconds * 1e6, 2), "tflops": round(flops / seconds / 1e12, 1),
        "frac_of_bf16_peak": round(flops / seconds / PEAK_FLOPS["bf16"], 4),
        "kv_gb_s": round(moved / seconds / 1e9, 1),
    }


LONG_DECODE_STEPS = 32
LONG_WARMUP_STEPS = 8
LONG_PORTION = 8192


def measure_long_context(contexts: list[int], batch: int, dtype: str, sizes: str, layers: int | None) -> dict:
    """Prefill and decode at long contexts: for each context length C, requests with prompts of
    C - 40 tokens are prefilled in portions of 8,192 tokens (the first one is timed: tokens a
    second over the whole prompt, share of the matrix peak) and then decoded 8 untimed and 32
    timed steps, ending at C positions, once alone and once `batch` together."""
    import numpy as np
    import torch

    from mini_infer_amd.engine import ModelRunner, StepEntry
    from mini_infer_amd.sampling import sample_from_slots

    model_name, full = SIZES[sizes]
    cfg = dict(full)
    cfg["num_hidden_layers"] = layers if layers is not None else full["num_hidden_layers"]
    elem = 2 if dtype == "bfloat16" else 4
    peak = PEAK_FLOPS["bf16" if dtype == "bfloat16" else "fp32"]
    longest = max(contexts)
    if longest > cfg["max_position_embeddings"]:
        raise SystemExit(f"bench.py: context {longest} is beyond max_position_embeddings {cfg['max_position_embeddings']}")
    runner = ModelRunner.from_random(
        cfg, seed=0, dtype=dtype, num_blocks=batch * (-(-longest // BLOCK_SIZE)) + 8, block_size=BLOCK_SIZE, max_concurrent=batch
    )
    print(f"bench.py: {model_name} layer sizes, {cfg['num_hidden_layers']} layers, weights are on the device", file=sys.stderr, flush=True)
    rng = np.random.default_rng(0)
    # untimed: the first call of every kernel and library routine at this portion size
    runner.step([StepEntry("warm", rng.integers(0, cfg["vocab_size"], size=LONG_PORTION).tolist(), [])])
    runner.free_request("warm")
    rows = []
    for context in contexts:
        prompt_len = context - LONG_WARMUP_STEPS - LONG_DECODE_STEPS
        prefill_seconds = None
        for live in sorted({1, batch}):
            ids = [f"c{context}_{live}_{i}" for i in range(live)]
            last = []
            for rid in ids:
                prompt = rng.integers(0, cfg["vocab_size"], size=prompt_len).tolist()
                torch.cuda.synchronize()
                started = time.perf_counter()
                for at in range(0, prompt_len, LONG_PORTION):
                    portion = prompt[at : at + LONG_PORTION]
                    final = at + LONG_PORTION >= prompt_len
                    logits = runner.step([StepEntry(rid, portion, [len(portion) - 1] if final else [])])
                torch.cuda.synchronize()
                seconds = time.perf_counter() - started
                prefill_seconds = seconds if prefill_seconds is None else min(prefill_seconds, seconds)
                last.append(int(sample_from_slots(logits, runner.last_row_slots, runner.cache.states.table).tolist()[0]))
                print(f"bench.py: context {context}: prompt of {rid} in {seconds:.2f} s", file=sys.stderr, flush=True)
            on_device = None
            for k in range(LONG_WARMUP_STEPS + LONG_DECODE_STEPS):
                if k == LONG_WARMUP_STEPS:
                    torch.cuda.synchronize()
                    started = time.perf_counter()
                if on_device is None:
                    entries = [StepEntry(rid, [tok], [0]) for rid, tok in zip(ids, last)]
                else:
                    entries = [StepEntry(rid, [0], [0], device_row=row) for row, rid in enumerate(ids)]
                logits = runner.step(entries, device_tokens=on_device)
                on_device = sample_from_slots(logits, runner.last_row_slots, runner.cache.states.table)
            torch.cuda.synchronize()
            step = (time.perf_counter() - started) / LONG_DECODE_STEPS
            mean_context = context - LONG_DECODE_STEPS / 2
            step_bytes = weight_bytes(cfg, elem) + live * mean_context * kv_bytes_per_token(cfg, elem)
            rows.append({
                "context": context,
                "batch": live,
                "decode_tok_s": round(live / step, 2),
                "ms_per_step": round(step * 1e3, 3),
                "hbm_frac": round(step_bytes / step / 1e9 / PEAK_HBM_GBS, 4),
                "prefill_tok_s": round(prompt_len / prefill_seconds, 1),
                "prefill_s": round(prefill_seconds, 3),
                "prefill_frac": round(prefill_flops(cfg, prompt_len) / prefill_seconds / peak, 4),
            })
            print(f"bench.py: {rows[-1]}", file=sys.stderr, flush=True)
            for rid in ids:
                runner.free_request(rid)
    return {
        "metric": f"long contexts, {model_name} layer sizes, prompts prefilled in portions of {LONG_PORTION}, {LONG_DECODE_STEPS} decode steps timed",
        "dtype": "bf16" if dtype == "bfloat16" else "fp32",
        "layers": cfg["num_hidden_layers"],
        "layers_full_model": full["num_hidden_layers"],
        "rows": rows,
    }


def main() -> int:
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    # defaults: 8 untimed steps, then every step up to 4,096 total positions
    parser.add_argument("--steps", type=int, default=PROMPT_LEN - 8)
    parser.add_argument("--warmup", type=int, default=8)
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--layers", type=int, default=None, help="fewer layers than the model has (both numbers are reported)")
    parser.add_argument("--dtype", choices=("bfloat16", "float32"), default="bfloat16")
    parser.add_argument("--sizes", choices=sorted(SIZES), default="8b", help="layer sizes of the model (default: Llama 3.1 8B)")
    parser.add_argument("--max-context", type=int, default=2 * PROMPT_LEN,
                        help="total positions a request may reach (default 4,096; 8,192 for the 70B workload)")
    parser.add_argument("--no-points", action="store_true", help="skip the batch 1 and 64 points")
    parser.add_argument("--no-prefill", action="store_true")
    parser.add_argument(
        "--serving", action="store_true",
        help="also run 32 concurrent requests through the scheduler at Llama-3.2-3B sizes (adds a 'serving' entry)",
    )
    parser.add_argument(
        "--reference-workload", action="store_true",
        help="also run the workload the reference publishes numbers for (1,024-token prompts, 128 tokens, "
        "1 request and 16 at once; adds a 'reference_workload' entry)",
    )
    parser.add_argument(
        "--attention", type=int, default=None, metavar="TOKENS",
        help="time the attention kernel alone instead: one prompt of TOKENS tokens, or with --attention-batch B one "
        "token of each of B requests over TOKENS keys; prints one JSON line and exits",
    )
    parser.add_argument(
        "--long-context", default=None, metavar="C1,C2,...",
        help="instead of the default run: for each context length C, prompts of C-40 tokens prefilled in portions "
        "of 8,192 and decoded to C positions, at batch 1 and at --batch; prints one JSON line and exits",
    )
    parser.add_argument("--no-mixed-graphs", action="store_true",
                        help="with --serving / --reference-workload: launch steps that have portions of prompts in them kernel "
                        "by kernel, however few their tokens (recorded steps of single tokens stay)")
    parser.add_argument("--attention-batch", type=int, default=0)
    parser.add_argument("--attention-repeats", type=int, default=20)
    args = parser.parse_args()
    if args.attention is not None:
        print(json.dumps(measure_attention(args.attention, args.attention_batch, args.attention_repeats, SIZES[args.sizes][1])), flush=True)
        return 0
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2
    if args.long_context is not None:
        contexts = [int(c) for c in args.long_context.split(",")]
        print(json.dumps(measure_long_context(contexts, args.batch, args.dtype, args.sizes, args.layers)), flush=True)
        return 0
    room = args.max_context - PROMPT_LEN
    if args.steps <= 0 or args.warmup < 0 or args.steps + args.warmup > room:
        print(f"bench.py: --warmup + --steps must be at most {room} (decoding runs from {PROMPT_LEN} to at most "
              f"{args.max_context} positions; see --max-context)")
        return 2

    import numpy as np
    import torch

    from mini_infer_amd.engine import ModelRunner, StepEntry
    from mini_infer_amd.sampling import sample_from_slots

    model_name, sizes = SIZES[args.sizes]
    full_layers = sizes["num_hidden_layers"]
    cfg = dict(sizes)
    cfg["num_hidden_layers"] = args.layers if args.layers is not None else full_layers
    elem = 2 if args.dtype == "bfloat16" else 4
    batches = [args.batch] if args.no_points else sorted({1, args.batch, 64})
    context_end = PROMPT_LEN + args.warmup + args.steps
    pages_per_request = -(-(context_end + 1) // BLOCK_SIZE)
    num_blocks = max(batches) * pages_per_request + 8
    print(f"bench.py: {model_name} layer sizes, {cfg['num_hidden_layers']} layers: making random weights on the device",
          file=sys.stderr, flush=True)
    runner = ModelRunner.from_random(
        cfg,
        seed=0,
        dtype=args.dtype,
        num_blocks=num_blocks,
        block_size=BLOCK_SIZE,
        max_concurrent=max(batches),
    )
    print("bench.py: weights are on the device", file=sys.stderr, flush=True)
    rng = np.random.default_rng(0)

    def sample(logits) -> torch.Tensor:
        """The greedy choice of every row on the device: each request's sampling state (greedy
        by default) is read from its state slot, as the scheduler's sampling does."""
        return sample_from_slots(logits, runner.last_row_slots, runner.cache.states.table)

    def sync() -> None:
        torch.cuda.synchronize()

    def prefill(request_id, tokens) -> torch.Tensor:
        return runner.step([StepEntry(request_id, tokens, [len(tokens) - 1])])

    def measure_decode(batch: int) -> tuple[float, float]:
        """(seconds per step, mean context length) over `--steps` decode steps."""
        ids = [f"b{batch}_{i}" for i in range(batch)]
        last = []
        for rid in ids:
            prompt = rng.integers(0, cfg["vocab_size"], size=PROMPT_LEN).tolist()
            logits = prefill(rid, prompt)
            last.append(int(sample(logits).tolist()[0]))
        host_ids = [torch.empty(batch, dtype=torch.int32, pin_memory=True) for _ in range(2)]
        copied = [torch.cuda.Event(), torch.cuda.Event()]

        # A step: the step function, the greedy choice on the device, the ids on their way to
        # the host.  The next step takes its tokens from the device (`device_row`), so it is
        # launched before the last one's ids have arrived; the host reads them one step late.
        def one_step(ids_on_device: torch.Tensor | None, tokens: list[int], draw: int) -> torch.Tensor:
            if ids_on_device is None:
                entries = [StepEntry(rid, [tok], [0]) for rid, tok in zip(ids, tokens)]
            else:
                entries = [StepEntry(rid, [0], [0], device_row=row) for row, rid in enumerate(ids)]
            logits = runner.step(entries, device_tokens=ids_on_device)
            sampled = sample(logits)
            host_ids[draw % 2].copy_(sampled, non_blocking=True)
            copied[draw % 2].record()
            return sampled

        def read_ids(draw: int) -> list[int]:
            copied[draw % 2].synchronize()
            return host_ids[draw % 2].tolist()

        on_device = None
        for w in range(args.warmup):
            on_device = one_step(on_device, last, w)
            if w > 0:
                read_ids(w - 1)
        if args.warmup > 0:
            last = read_ids(args.warmup - 1)
        sync()
        started = time.perf_counter()
        generated = 0
        for k in range(args.steps):
            draw = args.warmup + k
            on_device = one_step(on_device, last, draw)
            if k > 0:
                generated += len(read_ids(draw - 1))
            if k % 1024 == 1023:  # a long run shows that it is alive (a line on stderr every thousand steps)
                print(f"bench.py: batch {batch}: {k + 1} of {args.steps} steps, "
                      f"{(time.perf_counter() - started) / (k + 1) * 1e3:.3f} ms a step so far", file=sys.stderr, flush=True)
        generated += len(read_ids(args.warmup + args.steps - 1))
        sync()
        assert generated == batch * args.steps
        seconds = (time.perf_counter() - started) / args.steps
        for rid in ids:
            runner.free_request(rid)
        mean_context = PROMPT_LEN + args.warmup + (args.steps + 1) / 2
        return seconds, mean_context

    result_prefill = None
    if not args.no_prefill:
        times = []
        for rep in range(4):
            prompt = rng.integers(0, cfg["vocab_size"], size=PROMPT_LEN).tolist()
            sync()
            started = time.perf_counter()
            prefill(f"p{rep}", prompt)
            sync()
            times.append(time.perf_counter() - started)
            runner.free_request(f"p{rep}")
        seconds = min(times[1:])
        peak = PEAK_FLOPS["bf16" if args.dtype == "bfloat16" else "fp32"]
        result_prefill = {
            "value": round(PROMPT_LEN / seconds, 1),
            "tokens": PROMPT_LEN,
            "ms": round(seconds * 1e3, 3),
            "frac": round(prefill_flops(cfg, PROMPT_LEN) / seconds / peak, 4),
        }

    per_batch: dict[int, tuple[float, float]] = {}
    for batch in batches:
        per_batch[batch] = measure_decode(batch)

    seconds, mean_context = per_batch[args.batch]
    step_bytes = weight_bytes(cfg, elem) + args.batch * mean_context * kv_bytes_per_token(cfg, elem)
    achieved = step_bytes / seconds / 1e9
    line = {
        "metric": f"decode tok/s at batch {args.batch}, {model_name} layer sizes, 2048-token prompts",
        "value": round(args.batch / seconds, 2),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(seconds * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic: uniform-random token ids, random-init weights N(0, 0.02)",
        "config": {
            "model": f"{model_name} layer sizes",
            "layers": cfg["num_hidden_layers"],
            "layers_full_model": full_layers,
            "hidden_size": cfg["hidden_size"],
            "num_attention_heads": cfg["num_attention_heads"],
            "num_key_value_heads": cfg["num_key_value_heads"],
            "head_dim": cfg["head_dim"],
            "intermediate_size": cfg["intermediate_size"],
            "vocab_size": cfg["vocab_size"],
            "global_batch": args.batch,
            "seq_len": PROMPT_LEN,
            "context_start": PROMPT_LEN + args.warmup,
            "context_end": context_end,
            "kv_block_size": BLOCK_SIZE,
            "parallelism": "single GPU",
        },
        "roofline": {
            "bound": "hbm",
            "achieved": round(achieved, 1),
            "peak": PEAK_HBM_GBS,
            "unit": "GB/s",
            "frac": round(achieved / PEAK_HBM_GBS, 4),
        },
    }
    if result_prefill is not None:
        line["prefill"] = result_prefill
    points = {f"decode_b{b}": round(b / per_batch[b][0], 2) for b in batches if b != args.batch}
    if points:
        line["points"] = points
    if args.serving:
        del runner
        torch.cuda.empty_cache()
        line["serving"] = measure_serving(args.dtype, not args.no_mixed_graphs)
    if args.reference_workload:
        runner = None
        torch.cuda.empty_cache()
        line["reference_workload"] = measure_reference_workload(args.dtype, not args.no_mixed_graphs, args.sizes)
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
