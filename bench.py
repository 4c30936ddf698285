"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--layers L] [--size 0.6B|8B|32B] [--parity]
                    [--also-sizes 8B,32B|none]

A "step" is one decode step of the engine loop (schedule, the step function over
the paged cache, sampling) with ``--batch`` live requests, each after a prompt of
``--prompt-len`` random tokens.  The model has the layer sizes of Qwen3-0.6B (or
of ``--size``) with random weights.  One JSON line is printed.

How the numbers are taken.  ``value`` and ``ms_per_step``: the wall clock around
exactly ``--steps`` steps, a device synchronisation on both sides.  Beside it the
same steps by device events (one recorded before every step): the median step and
sixteen of the samples are kept (``decode_device``).  The prefill of one
2,048-token prompt is timed by device events over five runs after one that is not
counted; the median counts and all five samples are kept.  ``roofline`` and
``points_frac``: the bytes a decode step has to read (every weight once, the cache of
the live requests at their mean length) over its time, as a fraction of the
published 8 TB/s.  ``mixed``: 64 requests with prompts of 128 to 2,048 tokens arrive
at once and generate 128 tokens each, portions of 512 beside decode tokens under a
budget of 2,048 tokens a step, through the scheduler; all tokens over the wall time,
and by device events per step the share of steps that only decode (as a fraction
of the HBM peak) and of steps that run prompt portions (as a fraction of the MFMA
peak).  ``measured``: what the card reaches on a plain device copy and a large
library product.  ``sizes``: with the default size, the same decode points and prefill at
the layer sizes of Qwen3-8B and Qwen3-32B (all their layers), and for 32B the mixed run.  ``--parity`` adds a 32-bit run of the same layer sizes (two layers
unless ``--layers`` says otherwise) against the plain float64 implementation of
``tests/plain_qwen3.py``: a prompt whole, then 32 tokens one by one.

``--account-trace FILE`` runs nothing on the GPU: it reads the kernel trace
(``*_kernel_trace.csv``) that ``rocprofv3 --kernel-trace --output-format csv`` wrote
for a run of this program and prints, kernel by kernel, the time of a decode step,
of the prefill step and of the mixed run's steps (medians over the steps).
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
SIZES = ("0.6B", "8B", "32B")       # layer sizes that ship as config presets (qwen3-<size>)


def parse_args():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=128)
    parser.add_argument("--warmup", type=int, default=8)
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--prompt-len", type=int, default=2048)
    parser.add_argument("--context", type=int, default=4096)
    parser.add_argument("--size", default="0.6B", choices=SIZES, help="layer sizes of this Qwen3 model")
    parser.add_argument("--layers", type=int, default=None, help="fewer layers than the model has (named in config)")
    parser.add_argument("--dtype", default="bfloat16", choices=("bfloat16", "float32"))
    parser.add_argument("--prefill-tokens", type=int, default=2048)
    parser.add_argument("--no-points", action="store_true", help="skip the batch 1 and 64 points and the mixed run")
    parser.add_argument("--no-mixed", action="store_true", help="skip the mixed run")
    parser.add_argument("--also-sizes", default="8B,32B",
                        help="with the default size: the sizes whose decode, prefill (and, for 32B, mixed) numbers are "
                             "added under \"sizes\" ('none': the headline alone)")
    parser.add_argument("--mixed-requests", type=int, default=64, help="requests of the mixed continuous-batching run")
    parser.add_argument("--mixed-new-tokens", type=int, default=128, help="tokens each of them generates")
    parser.add_argument("--eager", action="store_true", help="no HIP graphs for decode steps")
    parser.add_argument("--parity", action="store_true",
                        help="also run these layer sizes in 32-bit against the plain float64 implementation")
    parser.add_argument("--account-trace", metavar="KERNEL_TRACE_CSV", default=None,
                        help="no run: the per-step kernel times of a rocprofv3 kernel trace of this program")
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


def per_token_flops(config):
    """Matrix products of all layers on one row of the batch (without attention and head)."""

    h, i, layers = config.hidden_size, config.intermediate_size, config.num_hidden_layers
    q, kv = config.num_attention_heads * config.head_dim, config.num_key_value_heads * config.head_dim
    return layers * 2 * (h * (q + 2 * kv) + q * h + 3 * h * i)


def prefill_flops(config, tokens):
    """Matrix products of the layers and of the head on one row, plus causal attention
    (2 * heads * head_dim * T^2 per layer: two products over the lower triangle)."""

    h, i, layers = config.hidden_size, config.intermediate_size, config.num_hidden_layers
    q, kv = config.num_attention_heads * config.head_dim, config.num_key_value_heads * config.head_dim
    per_token = 2 * (h * (q + 2 * kv) + q * h + 3 * h * i)
    return layers * (per_token * tokens + 2 * config.num_attention_heads * config.head_dim * tokens * tokens) + \
        2 * h * config.vocab_size


def parity_run(sizes, layers, device, prompt_len=300, tail=32):
    """The same layer sizes in true 32-bit against the plain float64 implementation of
    the tests: a model folder with random weights, a prompt whole and ``tail`` tokens
    one by one; the largest difference of a logit, the largest logit, and whether the
    tokens decoded one by one gave the logits of the whole run to the bit."""

    import tempfile

    import torch

    tests = os.path.join(ROOT, "tests")
    if not os.path.isfile(os.path.join(tests, "plain_qwen3.py")):
        raise SystemExit(f"--parity compares with the plain implementation in {tests}/plain_qwen3.py, which this checkout lacks.")
    sys.path.insert(0, tests)
    import plain_qwen3

    from miniserve_amd.config import EngineConfig, config_from_dict
    from miniserve_amd.engine import ModelRunner, StepEntry
    from miniserve_amd.weights import write_random_model

    data = dict(sizes)
    data["num_hidden_layers"] = layers
    data["max_position_embeddings"] = 1024
    generator = torch.Generator().manual_seed(1)
    tokens = torch.randint(0, data["vocab_size"], (prompt_len + tail,), generator=generator).tolist()
    places = list(range(0, prompt_len, 25)) + list(range(prompt_len - 1, prompt_len + tail))
    with tempfile.TemporaryDirectory() as folder:
        write_random_model(config_from_dict(data), folder, seed=2, store_dtype="bfloat16")
        from safetensors.torch import load_file

        weights = {name: tensor.double() for name, tensor in load_file(os.path.join(folder, "model.safetensors")).items()}
        exact = plain_qwen3.forward_logits(weights, data, tokens, rows=places).float()
        del weights
        engine_config = EngineConfig(dtype="float32", kv_block_size=16, num_kv_blocks=2 * (len(tokens) // 16 + 2),
                                     max_num_seqs=2, enable_chunked_prefill=True, decode_graphs=False)
        runner = ModelRunner.from_folder(folder, engine_config, device=device)
        runner.admit("whole")
        whole = runner.step([StepEntry("whole", tuple(tokens), tuple(places))]).cpu()
        runner.release("whole")
        runner.admit("cut")
        head_places = [place for place in places if place < prompt_len]
        rows = [runner.step([StepEntry("cut", tuple(tokens[:prompt_len]), tuple(head_places))]).cpu()]
        for position in range(prompt_len, prompt_len + tail):
            rows.append(runner.step([StepEntry("cut", (tokens[position],), (0,))]).cpu())
        cut = torch.cat(rows)
        del runner
        torch.cuda.empty_cache()
    return {
        "dtype": "fp32", "layers": layers, "tokens": len(tokens), "compared_positions": len(places),
        "max_abs_diff": float((whole - exact).abs().max()), "max_abs_logit": float(exact.abs().max()),
        "decoded_equals_whole_bitwise": bool(torch.equal(whole, cut)),
    }


def account_trace(path: str) -> None:
    """Per-step kernel times from a rocprofv3 kernel trace of this program.  A step
    begins with the embedding kernel.  Decode steps are those of the most frequent
    kernel count (the first four are left out as warm-up), the prefill steps the last
    three that bring neither that count nor single-token attention, the mixed steps
    the later half (the timed run) of those that hold both attention kernels."""

    import collections
    import csv
    import re

    with open(path, newline="") as handle:
        rows = sorted(csv.DictReader(handle), key=lambda row: int(row["Start_Timestamp"]))

    def short(name: str) -> str:
        name = name.replace("void ", "").replace("(anonymous namespace)::", "")
        library = re.match(r"(Custom_)?Cijk_\w*?(MT\d+x\d+x\d+)", name)
        return "hipBLASLt " + library.group(2) if library else re.sub(r"\(.*", "", name)

    names = [short(row["Kernel_Name"]) for row in rows]
    begin = [int(row["Start_Timestamp"]) / 1e3 for row in rows]
    length = [(int(row["End_Timestamp"]) - int(row["Start_Timestamp"])) / 1e3 for row in rows]
    starts = [index for index, name in enumerate(names) if name.startswith("embedding_gather")] + [len(rows)]
    steps = list(zip(starts[:-1], starts[1:]))
    if not steps:
        print("no step (no embedding kernel) in this trace")
        return

    def table(chosen, title):
        if not chosen:
            return
        busy = [sum(length[a:b]) for a, b in chosen]
        span = [begin[b - 1] + length[b - 1] - begin[a] for a, b in chosen]
        print(f"\n{title}: {len(chosen)} steps, {statistics.median(b - a for a, b in chosen):.0f} kernels a step; "
              f"kernel time {statistics.median(busy):.1f} us, first start to last end {statistics.median(span):.1f} us (medians)")
        print(f"{'kernel':58s} {'calls':>5s} {'us/step':>8s} {'avg us':>7s} {'in steps':>8s}")
        per_kernel = collections.defaultdict(list)
        for a, b in chosen:
            inside = collections.defaultdict(list)
            for name, us in zip(names[a:b], length[a:b]):
                inside[name].append(us)
            for name, values in inside.items():
                per_kernel[name].append((len(values), sum(values)))
        for name, seen in sorted(per_kernel.items(), key=lambda item: -statistics.median(x[1] for x in item[1])):
            if len(seen) * 8 < len(chosen):
                continue                      # a library product of a row count that few steps had
            calls = statistics.median(x[0] for x in seen)
            us = statistics.median(x[1] for x in seen)
            print(f"{name[:58]:58s} {calls:5.0f} {us:8.1f} {us / calls:7.2f} {len(seen):8d}")

    def holds(step, prefix):
        return any(name.startswith(prefix) for name in names[step[0]:step[1]])

    count = collections.Counter(b - a for a, b in steps if not holds((a, b), "attention_prefill")).most_common(1)
    decode = [s for s in steps if count and s[1] - s[0] == count[0][0] and not holds(s, "attention_prefill")][4:]
    mixed = [s for s in steps if holds(s, "attention_prefill") and holds(s, "attention_decode")]
    prefill = [s for s in steps if holds(s, "attention_prefill") and not holds(s, "attention_decode")
               and not holds(s, "at::native")][-3:]
    table(decode, "decode step")
    table(prefill, "prefill step")
    if len(mixed) >= 8:                       # fewer: the prompts of the decode runs, not the mixed run
        table(mixed[len(mixed) // 2:], "step with prompt portions beside decode tokens")


def measure(args, *, with_measured: bool = True) -> dict:
    """Everything the line holds for the layer sizes ``args.size``."""

    import torch

    from miniserve_amd.config import EngineConfig, config_dict_from_preset_or_file, config_from_dict
    from miniserve_amd.engine import Engine, ModelRunner, SamplingParams, StepEntry

    sizes = config_dict_from_preset_or_file(f"qwen3-{args.size}")
    full_layers = sizes["num_hidden_layers"]
    if args.layers is not None:
        sizes["num_hidden_layers"] = args.layers
    config = config_from_dict(sizes)
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

    def thin(samples, keep=16):
        """At most ``keep`` of the samples, evenly spaced, in milliseconds."""

        stride = max(1, len(samples) // keep)
        return [round(value, 4) for value in samples[::stride][:keep]]

    def decode_rate(batch, steps, warmup):
        """``steps`` decode steps at ``batch``: tokens a second and ms a step by the wall
        clock around all of them, the mean context, and the single steps by device events."""

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
        marks = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
        torch.cuda.synchronize()
        begin = time.perf_counter()
        for index in range(steps):
            marks[index].record()
            out = engine.step()
        marks[steps].record()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - begin
        assert len(out) == batch and engine.last_plan.prefill_items == ()
        by_device = [marks[index].elapsed_time(marks[index + 1]) for index in range(steps)]
        del engine, runner
        torch.cuda.empty_cache()
        device = {"median_ms": round(statistics.median(by_device), 4), "samples_ms": thin(by_device), "steps": steps}
        return batch * steps / elapsed, 1000 * elapsed / steps, start_context + steps / 2, device

    def step_bytes_of(batch, context, model_bytes, kv_bytes_per_token):
        return model_bytes + batch * context * kv_bytes_per_token

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
        model_bytes = weight_bytes(runner.model, itemsize)
        kv_bytes_per_token = runner.cache.layout.bytes_per_token(itemsize)
        params = SamplingParams(max_new_tokens=new_tokens)
        for prompts in rounds:
            engine = Engine(runner)
            for index, prompt in enumerate(prompts):
                engine.add_request(f"m{index}", prompt, params, arrival_ns=index)
            marks, plans = [], []
            torch.cuda.synchronize()
            begin = time.perf_counter()
            while engine.has_unfinished():
                mark = torch.cuda.Event(enable_timing=True)
                mark.record()
                marks.append(mark)
                engine.step()
                plans.append(engine.last_plan)
            mark = torch.cuda.Event(enable_timing=True)
            mark.record()
            marks.append(mark)
            torch.cuda.synchronize()
            elapsed = time.perf_counter() - begin
            counters = dict(engine.counters)
        # the last round by phase: steps of single tokens only against the HBM peak (their weights once and
        # the cache they read), steps with prompt portions against the MFMA peak (their products and attention)
        decode_only = {"steps": 0, "ms": 0.0, "bytes": 0.0}
        with_prompts = {"steps": 0, "ms": 0.0, "flops": 0.0, "tokens": 0}
        per_token = per_token_flops(config)
        for index, plan in enumerate(plans):
            if plan.empty:
                continue
            ms = marks[index].elapsed_time(marks[index + 1])
            if plan.prefill_items:
                flops = per_token * plan.scheduled_tokens
                for item in plan.prefill_items:
                    keys = item.num_tokens * (item.token_start + (item.num_tokens + 1) / 2)
                    flops += config.num_hidden_layers * 4 * config.num_attention_heads * config.head_dim * keys
                for item in plan.decode_items:
                    flops += config.num_hidden_layers * 4 * config.num_attention_heads * config.head_dim * (item.position + 1)
                with_prompts["steps"] += 1
                with_prompts["ms"] += ms
                with_prompts["flops"] += flops
                with_prompts["tokens"] += plan.scheduled_tokens
            else:
                cache_tokens = sum(item.position + 1 for item in plan.decode_items)
                decode_only["steps"] += 1
                decode_only["ms"] += ms
                decode_only["bytes"] += model_bytes + cache_tokens * kv_bytes_per_token
        mixed_steps = sum(1 for plan in plans if plan.prefill_items and plan.decode_items)
        del engine, runner
        torch.cuda.empty_cache()
        total = counters["prefill_tokens"] + counters["decode_tokens"]
        phases = {}
        if decode_only["steps"]:
            phases["decode_only"] = {
                "steps": decode_only["steps"], "ms": round(decode_only["ms"], 1),
                "frac_hbm": round(decode_only["bytes"] / (decode_only["ms"] / 1000) / 1e9 / HBM_GBPS, 4),
            }
        if with_prompts["steps"]:
            phases["with_prompts"] = {
                "steps": with_prompts["steps"], "ms": round(with_prompts["ms"], 1), "tokens": with_prompts["tokens"],
                "frac_mfma": round(with_prompts["flops"] / (with_prompts["ms"] / 1000) / (PEAK_TFLOPS[args.dtype] * 1e12), 4),
            }
        return {
            "value": round(total / elapsed, 1), "unit": "tokens/s, prompt and generated", "requests": requests,
            "prompt_tokens": counters["prefill_tokens"], "generated_tokens": counters["decode_tokens"] + requests,
            "steps": counters["steps"], "steps_with_both": mixed_steps, "chunk": chunk,
            "token_budget": engine_config.max_num_batched_tokens, "ms": round(1000 * elapsed, 1),
            "preemptions": counters.get("preemptions", 0), "phases": phases,
        }

    value, ms_per_step, mean_context, decode_device = decode_rate(args.batch, args.steps, args.warmup)

    # ---- roofline of the decode step --------------------------------------------------
    runner = make_runner(1)
    model_bytes = weight_bytes(runner.model, itemsize)
    kv_bytes_per_token = runner.cache.layout.bytes_per_token(itemsize)
    step_bytes = step_bytes_of(args.batch, mean_context, model_bytes, kv_bytes_per_token)
    achieved = step_bytes / (ms_per_step / 1000) / 1e9

    # ---- prefill of one prompt: device events, the median of five runs after one uncounted ----
    prompt = random_prompts(1, args.prefill_tokens)[0]
    prefill_samples = []
    for repeat in range(6):
        runner.admit("p")
        before, after = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        before.record()
        runner.step([StepEntry("p", tuple(prompt), (len(prompt) - 1,))])
        after.record()
        torch.cuda.synchronize()
        prefill_samples.append(before.elapsed_time(after))
        runner.release("p")
    prefill_samples = prefill_samples[1:]
    prefill_s = statistics.median(prefill_samples) / 1000
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

    copy_gbps = gemm_tflops = None
    if with_measured:
        source = torch.empty(1 << 30, dtype=torch.uint8, device=device)
        target = torch.empty_like(source)
        copy_gbps = 2 * source.numel() / rate(lambda: target.copy_(source)) / 1e9       # bytes read and written
        del source, target
        a = torch.randn(8192, 8192, device=device, dtype=torch.bfloat16)
        b = torch.randn(8192, 8192, device=device, dtype=torch.bfloat16)
        gemm_tflops = 2 * 8192**3 / rate(lambda: ops.linear(a, b)) / 1e12
        del a, b
        torch.cuda.empty_cache()

    points, points_frac = {}, {}
    if not args.no_points:
        for batch in (1, 64):
            point_rate, point_ms, point_context, _ = decode_rate(batch, max(16, args.steps // 4), min(args.warmup, 4))
            points[f"decode_b{batch}"] = round(point_rate, 1)
            point_bytes = step_bytes_of(batch, point_context, model_bytes, kv_bytes_per_token)
            points_frac[f"decode_b{batch}"] = round(point_bytes / (point_ms / 1000) / 1e9 / HBM_GBPS, 4)
    mixed = None
    if not args.no_points and not args.no_mixed:
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
        "decode_device": decode_device,
        "prefill": {
            "value": round(args.prefill_tokens / prefill_s, 1),
            "tokens": args.prefill_tokens,
            "ms": round(1000 * prefill_s, 3),
            "samples_ms": [round(sample, 3) for sample in prefill_samples],
            "frac": round(flops / prefill_s / (PEAK_TFLOPS[args.dtype] * 1e12), 5),
        },
        "roofline": {
            "bound": "hbm",
            "achieved": round(achieved, 1),
            "peak": HBM_GBPS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_GBPS, 5),
        },
        "points": points,
        "points_frac": points_frac,
        "mixed": mixed,
    }
    if with_measured:
        line["prefill"]["frac_of_measured_gemm"] = round(flops / prefill_s / (gemm_tflops * 1e12), 5)
        line["roofline"]["frac_of_measured_copy"] = round(achieved / copy_gbps, 5)
        line["measured"] = {"copy_GBps": round(copy_gbps, 1), "library_gemm_8192_TFLOPs": round(gemm_tflops, 1)}
    if args.parity:
        line["parity"] = parity_run(sizes, args.layers if args.layers is not None else 2, device)
    return line


def summary_of(line: dict) -> dict:
    """What the line of another size adds to the headline's: decode at batch 1, 8 and 64 with the fractions of
    the HBM peak, the prefill with its fraction of the MFMA peak, the mixed run, and how many layers ran."""

    batch = line["config"]["global_batch"]
    short = {
        "layers": line["config"]["layers"], "layers_of_model": line["config"]["layers_of_model"],
        "decode": {f"decode_b{batch}": line["value"], **line["points"]},
        "decode_frac_hbm": {f"decode_b{batch}": line["roofline"]["frac"], **line["points_frac"]},
        "ms_per_step": line["ms_per_step"],
        "prefill": {key: line["prefill"][key] for key in ("value", "tokens", "ms", "frac")},
    }
    if line.get("mixed"):
        short["mixed"] = {key: line["mixed"][key] for key in ("value", "requests", "steps", "ms", "preemptions", "phases")}
    return short


def main() -> int:
    args = parse_args()
    if args.account_trace:
        account_trace(args.account_trace)
        return 0
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported (this engine does not span GPUs).")
        return 2
    line = measure(args)
    others = [size for size in args.also_sizes.split(",") if size and size != "none"]
    if others and (args.no_points or args.size != "0.6B"):
        others = []             # the other sizes go with the default run only
    for size in others:
        if size not in SIZES:
            raise SystemExit(f"--also-sizes knows {', '.join(SIZES)}; not {size!r}.")
        print(f"[bench] Qwen3-{size} sizes ...", file=sys.stderr, flush=True)
        other = argparse.Namespace(**vars(args))
        other.size, other.layers, other.parity = size, None, False
        other.steps, other.warmup = min(args.steps, 24), min(args.warmup, 4)
        other.no_mixed = size != "32B"          # the mixed continuous batch is the 32B sizes' configuration
        line.setdefault("sizes", {})[size] = summary_of(measure(other, with_measured=False))
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
