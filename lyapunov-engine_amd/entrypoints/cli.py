"""Command line: ``lyapunov generate``.

Options and defaults are the reference's (python/lyapunov_engine/entrypoints/
cli.py:82-98): ``--model`` and ``--prompt`` (required there), ``--max-tokens 64``,
``--temperature 0.7``, ``--top-p 1.0``, ``--block-size 16``, ``--num-blocks 512``,
``--max-num-seqs 16``, ``--max-batched-tokens 2048``; one request "req-0" is added
and ``step()`` is looped until nothing is unfinished (:34-46).  Added: ``--top-k``,
``--seed``, ``--dtype``, ``--prompt-ids`` (token ids instead of text, so that no
tokenizer is needed) and ``--random-weights SEED`` (write a random model of the
folder's config.json first).  The reference loads a tokenizer through
transformers (:4, 14); here ``tokenizer.json`` of the model folder is read with
the tokenizers library when there is one.  ``lyapunov serve`` (:101-115) starts
an HTTP server in the reference and is not part of this engine.
"""
from __future__ import annotations

import argparse
import os
import sys


def _load_tokenizer(model_dir: str):
    path = os.path.join(model_dir, "tokenizer.json")
    if not os.path.exists(path):
        return None
    from tokenizers import Tokenizer

    return Tokenizer.from_file(path)


def run_generate(args) -> int:
    from ..config.engine_config import EngineConfig
    from ..engine.llm_engine import LLMEngine
    from ..sampling.params import SamplingParams

    if args.random_weights is not None:
        import json

        from ..weights.random_init import write_random_model

        with open(os.path.join(args.model, "config.json"), "r", encoding="utf-8") as f:
            raw = json.load(f)
        print(f"Writing random weights (seed {args.random_weights}): {args.model}")
        write_random_model(raw, args.model, args.random_weights, raw.get("torch_dtype") or "bfloat16")

    tokenizer = _load_tokenizer(args.model)
    if args.prompt_ids is not None:
        prompt_tokens = [int(t) for t in args.prompt_ids.replace(",", " ").split()]
    elif args.prompt is not None:
        if tokenizer is None:
            print(f"{args.model} has no tokenizer.json: give the prompt as --prompt-ids", file=sys.stderr)
            return 2
        print(f"Loading tokenizer: {args.model}")
        prompt_tokens = tokenizer.encode(args.prompt).ids
    else:
        print("one of --prompt and --prompt-ids is required", file=sys.stderr)
        return 2

    print(f"Loading weights: {args.model}")
    config = EngineConfig(block_size=args.block_size, num_gpu_blocks=args.num_blocks, max_num_seqs=args.max_num_seqs,
                          max_num_batched_tokens=args.max_batched_tokens, dtype=args.dtype, seed=args.seed)
    engine = LLMEngine(args.model, config)
    sampling = SamplingParams(temperature=args.temperature, top_p=args.top_p, top_k=args.top_k,
                              max_tokens=args.max_tokens)
    engine.add_request("req-0", prompt_tokens, sampling)
    print("\n--- Output Generation ---")
    while engine.has_unfinished_requests():
        for out in engine.step():
            if out.is_finished:
                if tokenizer is not None:
                    print(tokenizer.decode(out.output_tokens, skip_special_tokens=True))
                else:
                    print(" ".join(str(t) for t in out.output_tokens))
    return 0


def build_parser() -> argparse.ArgumentParser:
    parser = argparse.ArgumentParser(prog="lyapunov",
                                     description="Lyapunov Engine for AMD MI355X: Llama inference on one GPU")
    sub = parser.add_subparsers(dest="subcommand", required=True)
    gen = sub.add_parser("generate", help="Run text generation from prompt")
    gen.add_argument("--model", type=str, required=True, help="local model directory (config.json, *.safetensors)")
    gen.add_argument("--prompt", type=str, default=None, help="Prompt text (needs tokenizer.json in the model folder)")
    gen.add_argument("--prompt-ids", type=str, default=None, help="Prompt as token ids, e.g. '1,15,27'")
    gen.add_argument("--max-tokens", type=int, default=64)
    gen.add_argument("--temperature", type=float, default=0.7)
    gen.add_argument("--top-p", type=float, default=1.0)
    gen.add_argument("--top-k", type=int, default=-1)
    gen.add_argument("--seed", type=int, default=0)
    gen.add_argument("--dtype", type=str, default="bfloat16", choices=["bfloat16", "float32"])
    gen.add_argument("--block-size", type=int, default=16)
    gen.add_argument("--num-blocks", type=int, default=512)
    gen.add_argument("--max-num-seqs", type=int, default=16)
    gen.add_argument("--max-batched-tokens", type=int, default=2048)
    gen.add_argument("--random-weights", type=int, default=None, metavar="SEED",
                     help="first write model.safetensors with random weights for the folder's config.json")
    serve = sub.add_parser("serve", help="(not part of this engine) the reference's HTTP server")
    serve.add_argument("--model", type=str, default=None)
    return parser


def main(argv=None) -> int:
    args = build_parser().parse_args(argv)
    if args.subcommand == "generate":
        return run_generate(args)
    print("lyapunov serve: this engine has no HTTP server; use `lyapunov generate` or the Python API",
          file=sys.stderr)
    return 2


if __name__ == "__main__":
    sys.exit(main())
