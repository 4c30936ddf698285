"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--layers L]

A "step" is one decode step of the engine loop (schedule, the step function over
the paged cache, sampling) with ``--batch`` live requests, each after a prompt of
``--prompt-len`` random tokens.  The model has the layer sizes of Qwen3-0.6B (or
of ``--size``) with random weights.  One JSON line is printed: decoded tokens a second, the prefill
rate of one 2,048-token prompt with its fraction of the bf16 MFMA peak, the
fraction of the HBM peak that the decode step reaches, decode rates at batch 1 and
64, a mixed run (64 requests with prompts of 128 to 2,048 tokens, portions of 512
beside decode tokens under a budget of 2,048 tokens a step, through the scheduler), and what the card reaches on a plain
device copy and a large library product (the two fractions are given against these
measured rates as well as against the published peaks).
"""

from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# MI355X published peaks
HBM_GBPS = 8000.0
PEAK_TFLOPS = {"bfloat16": 2500.0, "float32": 157.3}

# layer sizes of the Qwen3 dense models; the default run is the first
_COMMON = dict(head_dim=128, vocab_size=151936, max_position_embeddings=40960, rms_norm_eps=1e-6, rope_theta=1e6)
SIZES = {
    "0.6B": dict(hidden_size=1024, intermediate_size=3072, num_hidden_layers=28, num_attention_heads=16,
                 num_key_value_heads=8, tie_word_embeddings=True, **_COMMON),
    "8B": dict(hidden_size=4096, intermediate_size=12288, num_hidden_layers=36, num_attention_heads=32,
               num_key_value_heads=8, tie_word_embeddings=False, **_COMMON),
    "32B": dict(hidden_size=5120, intermediate_size=25600, num_hidden_layers=64, num_attention_heads=64,
                num_key_value_heads=8, tie_word_embeddings=False, **_COMMON),
}


def parse_args():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=128)
    parser.add_argument("--warmup", type=int, default=8)
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--prompt-len", type=int, default=2048)
    parser.add_argument("--context", type=int, default=4096)
    parser.add_argument("--size", default="0.6B", choices=tuple(SIZES), help="layer sizes of this Qwen3 model")
    parser.add_argument("--layers", type=int, default=None, help="fewer layers than the model has (named in config)")
    parser.add_argument("--dtype", default="bfloat16", choices=("bfloat16", "float32"))
    parser.add_argument("--prefill-tokens", type=int, default=2048)
    parser.add_argument("--no-points", action="store_true", help="skip the batch 1 and 64 points and the mixed run")
    parser.add_argument("--mixed-requests", type=int, default=64, help="requests of the mixed continuous-batching run")
    parser.add_argument("--mixed-new-tokens", type=int, default=128, help="tokens each of them generates")
    parser.add_argument("--eager", action="store_true", help="no HIP graphs for decode steps")
    return parser.parse_args()


def weight_bytes(model, itemsize):
    """Bytes of every weight a decode step uses once (a tied head counts once; the
    embedding table is read by row, not whole, unless it is the head)."""

    total = 0
    tied = model.spec.head.params.get("tied_to")
    for spec in model.weight_specs():
        if spec.same_as is not None:
            continue
        if spec.name == model.spec.embedding.prefix + "weight" and not tied:
            continue
        count = 1
        for size in spec.shape:
            count *= size
        total += count * itemsize
    return total


def prefill_flops(config, tokens):
    """Matrix products of the layers and of the head on one row, plus causal attention
    (2 * heads * head_dim * T^2 per layer: two products over the lower triangle)."""

    h, i, layers = config.hidden_size, config.intermediate_size, config.num_hidden_layers
    q, kv = config.num_attention_heads * config.head_dim, config.num_key_value_heads * config.head_dim
    per_token = 2 * (h * (q + 2 * kv) + q * h + 3 * h * i)
    return layers * (per_token * tokens + 2 * config.num_attention_heads * config.head_dim * tokens * tokens) + \
        2 * h * config.vocab_size


def main() -> int:
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported (this engine does not span GPUs).")
        return 2
    import torch

    from miniserve_amd.config import EngineConfig, Qwen3Config
    from miniserve_amd.engine import Engine, ModelRunner, SamplingParams, StepEntry

    sizes = dict(SIZES[args.size])
    full_layers = sizes["num_hidden_layers"]
    if args.layers is not None:
        sizes["num_hidden_layers"] = args.layers
    config = Qwen3Config(**sizes)
    device = "cuda:0"
    itemsize = 2 if args.dtype == "bfloat16" else 4
    generator = torch.Generator().manual_seed(0)

    def random_prompts(count, length):
        return [torch.randint(0, config.vocab_size, (length,), generator=generator).tolist() for _ in range(count)]

    def make_runner(batch):
        pages = batch * (-(-args.context // 16)) + 16
        engine_config = EngineConfig(
            dtype=args.dtype, max_model_len=args.context, max_num_seqs=batch, max_num_batched_tokens=args.context,
            kv_block_size=16, num_kv_blocks=pages, enable_chunked_prefill=True, prefill_chunk_size=args.prompt_len,
            max_pending_requests=max(64, batch), decode_graphs=not args.eager,
        )
        return ModelRunner.from_random(config, engine_config, seed=0, device=device)

    def decode_rate(batch, steps, warmup):
        """(tokens a second, ms a step, mean context) of ``steps`` decode steps at ``batch``."""

        runner = make_runner(batch)
        engine = Engine(runner)
        params = SamplingParams(max_new_tokens=steps + warmup + batch + 8)   # nobody ends inside the timed steps
        for index, prompt in enumerate(random_prompts(batch, args.prompt_len)):
            engine.add_request(f"r{index}", prompt, params, arrival_ns=index)
        while engine.counters["decode_tokens"] == 0 or engine.last_plan.prefill_items:
            engine.step()                       # prompts, untimed
        for _ in range(warmup):
            engine.step()
        start_context = args.prompt_len + 1 + warmup + 1
        torch.cuda.synchronize()
        begin = time.perf_counter()
        for _ in range(steps):
            out = engine.step()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - begin
        assert len(out) == batch and engine.last_plan.prefill_items == ()
        del engine, runner
        torch.cuda.empty_cache()
        return batch * steps / elapsed, 1000 * elapsed / steps, start_context + steps / 2

    def mixed_rate(requests, new_tokens, chunk=512):
        """Continuous batching as a server sees it: ``requests`` prompts of 128 to
        ``prompt_len`` tokens (uniform, seeded) arrive at once, prompts go in portions of
        ``chunk`` beside the decode tokens of the others, each request generates
        ``new_tokens``.  All tokens, prompt and generated, over the wall time."""

        longest = min(args.prompt_len, args.context - new_tokens)
        rounds = []
        for _ in range(2):      # the first is untimed: the library's choices for these shapes, the recorded steps
            lengths = torch.randint(min(128, longest), longest + 1, (requests,), generator=generator).tolist()
            rounds.append([random_prompts(1, length)[0] for length in lengths])
        pages = max(sum(-(-(len(prompt) + new_tokens) // 16) for prompt in prompts) for prompts in rounds) + 16
        engine_config = EngineConfig(
            dtype=args.dtype, max_model_len=args.context, max_num_seqs=requests,
            max_num_batched_tokens=min(args.context, 4 * chunk), kv_block_size=16, num_kv_blocks=pages,
            enable_chunked_prefill=True, prefill_chunk_size=chunk, max_pending_requests=max(64, requests),
            decode_graphs=not args.eager,
        )
        runner = ModelRunner.from_random(config, engine_config, seed=0, device=device)
        params = SamplingParams(max_new_tokens=new_tokens)
        for prompts in rounds:
            engine = Engine(runner)
            for index, prompt in enumerate(prompts):
                engine.add_request(f"m{index}", prompt, params, arrival_ns=index)
            torch.cuda.synchronize()
            begin = time.perf_counter()
            mixed_steps = 0
            while engine.has_unfinished():
                engine.step()
                mixed_steps += bool(engine.last_plan.prefill_items and engine.last_plan.decode_items)
            torch.cuda.synchronize()
            elapsed = time.perf_counter() - begin
            counters = dict(engine.counters)
        del engine, runner
        torch.cuda.empty_cache()
        total = counters["prefill_tokens"] + counters["decode_tokens"]
        return {
            "value": round(total / elapsed, 1), "unit": "tokens/s, prompt and generated", "requests": requests,
            "prompt_tokens": counters["prefill_tokens"], "generated_tokens": counters["decode_tokens"] + requests,
            "steps": counters["steps"], "steps_with_both": mixed_steps, "chunk": chunk,
            "token_budget": engine_config.max_num_batched_tokens, "ms": round(1000 * elapsed, 1),
            "preemptions": counters.get("preemptions", 0),
        }

    value, ms_per_step, mean_context = decode_rate(args.batch, args.steps, args.warmup)

    # ---- roofline of the decode step --------------------------------------------------
    runner = make_runner(1)
    model_bytes = weight_bytes(runner.model, itemsize)
    kv_bytes_per_token = runner.cache.layout.bytes_per_token(itemsize)
    step_bytes = model_bytes + args.batch * mean_context * kv_bytes_per_token
    achieved = step_bytes / (ms_per_step / 1000) / 1e9

    # ---- prefill of one prompt -----------------------------------------------------------
    prompt = random_prompts(1, args.prefill_tokens)[0]
    times = []
    for repeat in range(4):
        runner.admit("p")
        torch.cuda.synchronize()
        begin = time.perf_counter()
        runner.step([StepEntry("p", tuple(prompt), (len(prompt) - 1,))])
        torch.cuda.synchronize()
        times.append(time.perf_counter() - begin)
        runner.release("p")
    prefill_s = statistics.median(times[1:])
    flops = prefill_flops(config, args.prefill_tokens)
    del runner
    torch.cuda.empty_cache()

    # ---- what this card reaches on plain work: a device copy and a large library product ----
    from miniserve_amd import ops

    def rate(function, repeats=5):
        function()
        torch.cuda.synchronize()
        begin = time.perf_counter()
        for _ in range(repeats):
            function()
        torch.cuda.synchronize()
        return (time.perf_counter() - begin) / repeats

    source = torch.empty(1 << 30, dtype=torch.uint8, device=device)
    target = torch.empty_like(source)
    copy_gbps = 2 * source.numel() / rate(lambda: target.copy_(source)) / 1e9       # bytes read and written
    del source, target
    a = torch.randn(8192, 8192, device=device, dtype=torch.bfloat16)
    b = torch.randn(8192, 8192, device=device, dtype=torch.bfloat16)
    gemm_tflops = 2 * 8192**3 / rate(lambda: ops.linear(a, b)) / 1e12
    del a, b
    torch.cuda.empty_cache()

    points = {}
    if not args.no_points:
        for batch in (1, 64):
            rate, _, _ = decode_rate(batch, max(16, args.steps // 4), min(args.warmup, 4))
            points[f"decode_b{batch}"] = round(rate, 1)
    mixed = None
    if not args.no_points:
        mixed = mixed_rate(args.mixed_requests, args.mixed_new_tokens)

    line = {
        "metric": f"decode tok/s at batch {args.batch} (Qwen3-{args.size} sizes, {args.prompt_len:,}-token prompts, "
                  "paged cache)",
        "value": round(value, 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic: random weights, uniform random token ids",
        "config": {
            "model": f"Qwen3-{args.size} sizes",
            "global_batch": args.batch,
            "seq_len": args.context,
            "prompt_len": args.prompt_len,
            "parallelism": "1 GPU",
            "layers": config.num_hidden_layers,
            "layers_of_model": full_layers,
            "hidden_size": config.hidden_size,
            "intermediate_size": config.intermediate_size,
            "q_heads": config.num_attention_heads,
            "kv_heads": config.num_key_value_heads,
            "head_dim": config.head_dim,
            "vocab_size": config.vocab_size,
            "tied_embeddings": config.tie_word_embeddings,
            "kv_block_size": 16,
            "decode_graphs": not args.eager,
        },
        "prefill": {
            "value": round(args.prefill_tokens / prefill_s, 1),
            "tokens": args.prefill_tokens,
            "ms": round(1000 * prefill_s, 3),
            "frac": round(flops / prefill_s / (PEAK_TFLOPS[args.dtype] * 1e12), 5),
            "frac_of_measured_gemm": round(flops / prefill_s / (gemm_tflops * 1e12), 5),
        },
        "roofline": {
            "bound": "hbm",
            "achieved": round(achieved, 1),
            "peak": HBM_GBPS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_GBPS, 5),
            "frac_of_measured_copy": round(achieved / copy_gbps, 5),
        },
        "points": points,
        "mixed": mixed,
        "measured": {"copy_GBps": round(copy_gbps, 1), "library_gemm_8192_TFLOPs": round(gemm_tflops, 1)},
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
