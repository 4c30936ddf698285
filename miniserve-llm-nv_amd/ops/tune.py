"""Measures the table of pinned hipBLASLt solutions (``ops/library_products.json``).

    python -m miniserve_amd.ops.tune --presets qwen3-0.6b qwen3-8b qwen3-32b
    python -m miniserve_amd.ops.tune --config path/to/config.json --max-tokens 4096

For each model (one layer of it, random weights) it runs steps of every bucket of row
counts through the engine's own step function and notes which products the fixed rule
sends to hipBLASLt; each of those shapes is then timed, every candidate from flushed
caches, and the fastest solution is pinned for (matrix, output type, bucket).  A serving
process reads the table and times nothing, so its sums are the same in every run.
The table holds for the build of hipBLASLt that it names; pins measured under another
build are dropped when the table is written anew.
"""

from __future__ import annotations

import argparse
import json
import sys

import torch

from .. import ops

# the row counts that stand for their buckets: the largest of each bucket of few rows, the
# smallest of each bucket of 256
FEW_ROWS = (8, 16, 32, 64, 128, 255)


def shapes_of_model(config_dict: dict, max_tokens: int, device: str) -> set[tuple[int, int, int, int]]:
    """(m, n, k, out is float) of every product that hipBLASLt serves when one layer of
    the model runs steps of the buckets' row counts."""

    from ..config import EngineConfig, config_from_dict
    from ..engine import ModelRunner, StepEntry

    data = dict(config_dict)
    data["num_hidden_layers"] = 1
    config = config_from_dict(data)
    many = [rows for rows in range(256, max_tokens + 1, 256)]
    longest = max([1, *many])
    engine_config = EngineConfig(dtype="bfloat16", max_num_seqs=256, max_model_len=longest + 1,
                                 max_num_batched_tokens=longest + 1, kv_block_size=16,
                                 num_kv_blocks=256 + longest // 16 + 2, decode_graphs=False)
    runner = ModelRunner.from_random(config, engine_config, seed=0, device=device)
    seen: set[tuple[int, int, int, int]] = set()
    with ops.noting_library_products(seen):
        for rows in FEW_ROWS:
            names = [f"t{index}" for index in range(rows)]
            for name in names:
                runner.admit(name)
            runner.step([StepEntry(name, (index % 7,), (0,)) for index, name in enumerate(names)])
            for name in names:
                runner.release(name)
        for rows in many:
            runner.admit("p")
            runner.step([StepEntry("p", tuple(index % 7 for index in range(rows)), (rows - 1,))])
            runner.release("p")
    torch.cuda.synchronize()
    del runner
    torch.cuda.empty_cache()
    return seen


def main(argv=None) -> int:
    from ..config import config_dict_from_preset_or_file

    parser = argparse.ArgumentParser(prog="python -m miniserve_amd.ops.tune", description=__doc__.split("\n\n")[0])
    parser.add_argument("--presets", nargs="*", default=[], help="names of layer sizes that ship with the package")
    parser.add_argument("--config", action="append", default=[], help="a config.json (may be given more than once)")
    parser.add_argument("--max-tokens", type=int, default=2048, help="the most tokens a step brings")
    parser.add_argument("--out", default=str(ops.LIBRARY_PRODUCTS_TABLE))
    parser.add_argument("--device", default="cuda:0")
    args = parser.parse_args(argv)
    sources = [*args.presets, *args.config]
    if not sources:
        parser.error("name at least one preset or config.json.")
    build = ops.hipblaslt_build(ops.open_gemm_library())
    pins: dict[tuple[int, int, int, int], int] = {}
    try:
        with open(args.out) as handle:
            old = json.load(handle)
        if old.get("library") == build:
            pins = {tuple(entry[:4]): entry[4] for entry in old.get("pins", ())}
    except FileNotFoundError:
        pass
    flush = torch.empty(384 << 20, dtype=torch.uint8, device=args.device)      # more than the last-level cache holds
    for source in sources:
        shapes = shapes_of_model(config_dict_from_preset_or_file(source), args.max_tokens, args.device)
        for m, n, k, out_float in sorted(shapes):
            timed = [(ms, solution) for solution, ms in
                     ops.time_library_product(m, n, k, out_float32=bool(out_float), flush=flush, device=args.device)
                     if ms > 0]
            if not timed:
                continue
            first_ms = timed[0][0]
            best_ms, best = min(timed)
            pins[(n, k, out_float, ops.library_product_bucket(m))] = best
            print(f"{source}: {m} x {n} x {k}{' f32' if out_float else ''}: first choice {first_ms * 1e3:.1f} us, "
                  f"pinned {best} {best_ms * 1e3:.1f} us", flush=True)
    table = {"library": build, "device": torch.cuda.get_device_name(torch.device(args.device)),
             "pins": [[*key, solution] for key, solution in sorted(pins.items())]}
    with open(args.out, "w") as handle:        # one pin a line: [n, k, out is float32, bucket, solution]
        lines = ",\n  ".join(json.dumps(pin, separators=(",", ":")) for pin in table["pins"])
        handle.write(f'{{"library": {json.dumps(table["library"])}, "device": {json.dumps(table["device"])}, '
                     f'"pins": [\n  {lines}\n]}}\n')
    print(f"{len(pins)} pins -> {args.out}", file=sys.stderr)
    return 0


if __name__ == "__main__":
    sys.exit(main())
