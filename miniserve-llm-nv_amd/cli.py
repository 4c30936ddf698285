"""Command line: generate token ids from prompts of token ids.

    python -m miniserve_amd.cli --model DIR --prompt-ids 1,2,3 --max-new-tokens 8
    python -m miniserve_amd.cli --random-weights config.json --seed 0 --prompt-len 32
    python -m miniserve_amd.cli --random-weights qwen3-0.6b --layers 4 --prompt-len 32

Engine options carry the names of the reference's launcher
(miniserve/api/server.py:350-397); per-request options the names of its request
body (miniserve/api/schemas.py:21-42: temperature, top_p, top_k, seed) and of its
``SamplingParams`` (miniserve/engine/request.py:19-24).
"""

from __future__ import annotations

import argparse
import json
import sys


def build_cli_parser() -> argparse.ArgumentParser:
    parser = argparse.ArgumentParser(prog="miniserve-generate", description=__doc__.split("\n\n")[0])
    source = parser.add_mutually_exclusive_group(required=True)
    source.add_argument("--model", help="folder with config.json and safetensors")
    source.add_argument("--random-weights", metavar="PRESET|CONFIG_JSON",
                        help="layer sizes by name (qwen3-0.6b, qwen3-8b, qwen3-32b) or a config.json; weights are drawn from --seed")
    parser.add_argument("--layers", type=int, default=None,
                        help="with --random-weights: this many layers instead of the configuration's own number")
    parser.add_argument("--seed", type=int, default=0, help="seed of the random weights and of sampling")
    parser.add_argument("--dtype", choices=("bfloat16", "float32"), default="bfloat16")
    parser.add_argument("--max-model-len", type=int, default=None)
    parser.add_argument("--num-kv-blocks", type=int, default=None)
    parser.add_argument("--max-num-seqs", type=int, default=8)
    parser.add_argument("--max-pending-requests", type=int, default=64)
    parser.add_argument("--max-num-batched-tokens", type=int, default=None)
    parser.add_argument("--kv-block-size", type=int, default=16)
    chunk = parser.add_mutually_exclusive_group()
    chunk.add_argument("--chunked-prefill", dest="enable_chunked_prefill", action="store_true")
    chunk.add_argument("--no-chunked-prefill", dest="enable_chunked_prefill", action="store_false")
    parser.set_defaults(enable_chunked_prefill=False)
    parser.add_argument("--prefill-chunk-size", type=int, default=None)
    parser.add_argument("--decode-execution", choices=("hip_graph", "eager"), default="hip_graph")
    prompts = parser.add_mutually_exclusive_group(required=True)
    prompts.add_argument("--prompt-ids", action="append", help="comma-separated token ids; may repeat")
    prompts.add_argument("--prompt-len", type=int, action="append", help="a random prompt of this length; may repeat")
    parser.add_argument("--max-new-tokens", type=int, default=16)
    parser.add_argument("--temperature", type=float, default=0.0)
    parser.add_argument("--top-p", type=float, default=1.0)
    parser.add_argument("--top-k", type=int, default=0)
    parser.add_argument("--stop-token-ids", default="", help="comma-separated token ids")
    return parser


def main(argv: list[str] | None = None) -> int:
    parser = build_cli_parser()
    args = parser.parse_args(argv)
    import torch

    from .config import config_dict_from_preset_or_file, config_from_dict
    from .engine import SamplingParams
    from .entrypoint import LLM

    model_dir = args.model
    if args.random_weights:
        try:
            data = config_dict_from_preset_or_file(args.random_weights)
        except FileNotFoundError as exc:
            parser.error(str(exc))
        if args.layers is not None:
            data["num_hidden_layers"] = args.layers
        model_dir = config_from_dict(data)        # a configuration: the weights are drawn on the device
    try:
        llm = LLM(
            model_dir,
            seed=args.seed,
            dtype=args.dtype,
            max_model_len=args.max_model_len,
            num_kv_blocks=args.num_kv_blocks,
            max_num_seqs=args.max_num_seqs,
            max_pending_requests=args.max_pending_requests,
            max_num_batched_tokens=args.max_num_batched_tokens,
            kv_block_size=args.kv_block_size,
            enable_chunked_prefill=args.enable_chunked_prefill,
            prefill_chunk_size=args.prefill_chunk_size,
            decode_graphs=args.decode_execution == "hip_graph",
        )
    except ValueError as exc:
        parser.error(str(exc))
    vocab = llm.runner.spec.vocab_size
    if args.prompt_ids:
        prompts = [[int(t) for t in text.split(",") if t.strip()] for text in args.prompt_ids]
    else:
        generator = torch.Generator().manual_seed(args.seed)
        prompts = [torch.randint(0, vocab, (n,), generator=generator).tolist() for n in args.prompt_len]
    stops = tuple(int(t) for t in args.stop_token_ids.split(",") if t.strip())
    params = [
        SamplingParams(
            temperature=args.temperature,
            top_p=args.top_p,
            top_k=args.top_k,
            max_new_tokens=args.max_new_tokens,
            stop_token_ids=stops,
            seed=args.seed + index,
        )
        for index in range(len(prompts))
    ]
    for prompt, tokens in zip(prompts, llm.generate(prompts, params)):
        print(json.dumps({"prompt_token_ids": prompt, "token_ids": tokens}))
    return 0


if __name__ == "__main__":
    sys.exit(main())
