"""Trace replay: given token ids go through the model step by step and the logits
at the wanted places are written out.  Nothing is sampled.  The replay drives the
same ``ModelRunner.step`` (model, cache and kernels) that generation uses; it has
no forward pass, cache or loader of its own.

Input, one JSON object a line on standard input::

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

``entries``: for each request its next tokens and the places among them whose
logits are wanted; all entries of a step are one batch.  A request is admitted
at its first entry.  ``end``: requests that are finished after this step; what
they hold is given back.  For a step in which something is wanted the logits are
written to ``<out>/<step>.f32`` as little-endian float32 ``[wanted, vocab]``, in
the order of the entries and of ``want``.  After every step ``done <step>`` is
printed and flushed.
"""

from __future__ import annotations

import argparse
import json
import sys
from pathlib import Path
from typing import Iterable, TextIO

from ..config import EngineConfig, load_config
from .batch import StepEntry

MAX_LIVE_REQUESTS = 8


def replay(runner, lines: Iterable[str], out_dir: Path, *, report: TextIO = sys.stdout) -> int:
    """Feed the steps of ``lines`` through ``runner``; returns the number of steps."""

    import numpy as np

    out_dir.mkdir(parents=True, exist_ok=True)
    count = 0
    for line in lines:
        line = line.strip()
        if not line:
            continue
        record = json.loads(line)
        step = record["step"]
        entries = []
        for item in record.get("entries", ()):
            request_id = str(item["id"])
            if not runner.cache.is_live(request_id):
                runner.admit(request_id)
            entries.append(
                StepEntry(request_id, tuple(int(t) for t in item["tokens"]), tuple(int(w) for w in item.get("want", ())))
            )
        if entries:
            logits = runner.step(entries)
            if logits is not None:
                array = logits.detach().to("cpu").numpy().astype("<f4", copy=False)
                np.ascontiguousarray(array).tofile(out_dir / f"{step}.f32")
        for request_id in record.get("end", ()):
            if runner.cache.is_live(str(request_id)):
                runner.release(str(request_id))
        count += 1
        print(f"done {step}", file=report, flush=True)
    return count


def build_parser() -> argparse.ArgumentParser:
    parser = argparse.ArgumentParser(
        prog="trace_run", description="Feed given token ids through a model step by step and write logits."
    )
    parser.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    parser.add_argument("--dtype", required=True, choices=("bfloat16", "float32"))
    parser.add_argument("--out", required=True, help="folder for <step>.f32 files")
    parser.add_argument(
        "--max-tokens", type=int, required=True,
        help="most tokens that live requests hold at any time, each request rounded up to a multiple of 64",
    )
    parser.add_argument("--kv-block-size", type=int, default=16)
    return parser


def main(argv: list[str] | None = None) -> int:
    args = build_parser().parse_args(argv)
    if args.max_tokens <= 0:
        raise SystemExit("--max-tokens must be positive.")
    if args.kv_block_size <= 0 or 64 % args.kv_block_size:
        raise SystemExit("--kv-block-size must divide 64.")
    print(f"[trace_run] loading {args.model} as {args.dtype}", file=sys.stderr, flush=True)
    from .. import ops

    ops.load()      # compiles the kernels at the first call of a fresh checkout
    from .runner import ModelRunner

    config = load_config(args.model)
    max_positions = config.model_spec().max_positions
    engine_config = EngineConfig(
        dtype=args.dtype,
        max_model_len=max_positions,
        max_num_seqs=MAX_LIVE_REQUESTS,
        max_num_batched_tokens=max_positions,
        kv_block_size=args.kv_block_size,
        num_kv_blocks=-(-args.max_tokens // args.kv_block_size),
        enable_chunked_prefill=True,
        decode_graphs=False,
    )
    runner = ModelRunner.from_folder(args.model, engine_config)
    print("[trace_run] ready", file=sys.stderr, flush=True)
    replay(runner, sys.stdin, Path(args.out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
