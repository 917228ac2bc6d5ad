"""Offline command line: token ids in, token ids out.

The reference's only command line is its HTTP server (``jllm/server.py:245-269``); the engine
options here keep its names, defaults and meanings: ``--model-path`` (env ``JLLM_MODEL_PATH``),
``--max-num-seqs 4``, ``--max-model-len 2048``, ``--max-prefill-len 512``,
``--dtype {bf16,fp32}``, ``--no-prewarm``.  Server options (host, port, model name) have no
counterpart: there is no server.  Added: the page geometry
(``--block-size``, ``--num-blocks``, the arguments of the reference's ``make_driver``), the
token budget of a step, sampling, and a random-weights mode.

    python -m jax_vllm_amd --model-path DIR --prompt-ids "1 2 3" --prompt-ids "4 5" --max-new-tokens 16
    python -m jax_vllm_amd --random-config config.json --random-seed 0 --write-model DIR   # writes a model folder
"""
from __future__ import annotations

import argparse
import json
import os
import sys


def build_parser() -> argparse.ArgumentParser:
    p = argparse.ArgumentParser(prog="jax_vllm_amd", description="Generate token ids with the MI355X Qwen3 engine.")
    p.add_argument("--model-path", default=os.environ.get("JLLM_MODEL_PATH"),
                   help="Path to HF model directory (config.json + *.safetensors). Env: JLLM_MODEL_PATH.")
    p.add_argument("--max-num-seqs", type=int, default=4)
    p.add_argument("--max-model-len", type=int, default=2048)
    p.add_argument("--max-prefill-len", type=int, default=512, help="longest prompt accepted")
    p.add_argument("--dtype", choices=["bf16", "fp32"], default="bf16")
    p.add_argument("--block-size", type=int, default=16, help="tokens per cache page")
    p.add_argument("--num-blocks", type=int, default=None, help="cache pages, the null page included (default: worst case)")
    p.add_argument("--max-num-batched-tokens", type=int, default=2048, help="token budget of one step")
    p.add_argument("--max-chunk", type=int, default=None, help="largest prompt portion of one request per step")
    p.add_argument("--no-prefix-cache", dest="prefix_cache", action="store_false")
    p.add_argument("--no-hip-graphs", dest="hip_graphs", action="store_false")
    p.add_argument("--no-decode-ahead", dest="decode_ahead", action="store_false",
                   help="Wait for a decode step's tokens before the next step is started.")
    p.add_argument("--no-prewarm", dest="prewarm", action="store_false",
                   help="Skip building the kernels and capturing the decode steps before the first prompt.")
    p.add_argument("--prompt-ids", action="append", default=[], metavar="'ID ID ...'",
                   help="one prompt as space- or comma-separated token ids (repeatable)")
    p.add_argument("--prompt-file", help="file with one prompt per line (token ids), or a JSON list of lists")
    p.add_argument("--max-new-tokens", type=int, default=64)
    p.add_argument("--eos-id", type=int, default=None)
    p.add_argument("--temperature", type=float, default=0.0, help="0: greedy")
    p.add_argument("--seed", type=int, default=0, help="sampling seed")
    p.add_argument("--random-config", help="config.json of a model to fill with random weights instead of --model-path")
    p.add_argument("--random-seed", type=int, default=0)
    p.add_argument("--random-std", type=float, default=0.02)
    p.add_argument("--write-model", help="with --random-config: write config.json and model.safetensors there and exit")
    p.add_argument("--stats", action="store_true", help="print the engine's counters to stderr")
    return p


def parse_ids(text: str) -> list:
    return [int(t) for t in text.replace(",", " ").split()]


def read_prompts(args) -> list:
    prompts = [parse_ids(t) for t in args.prompt_ids]
    if args.prompt_file:
        text = open(args.prompt_file).read()
        try:
            data = json.loads(text)
            prompts += [[int(t) for t in row] for row in data]
        except json.JSONDecodeError:
            prompts += [parse_ids(line) for line in text.splitlines() if line.strip()]
    return prompts


def main(argv=None) -> int:
    args = build_parser().parse_args(argv)
    if args.random_config and args.write_model:
        from ..weights import write_random_model

        cfg = json.loads(open(args.random_config).read())
        folder = write_random_model(args.write_model, cfg, args.random_seed, std=args.random_std, norm_std=args.random_std)
        print(f"wrote {folder}", file=sys.stderr)
        return 0
    prompts = read_prompts(args)
    if not prompts:
        print("no prompts given (--prompt-ids or --prompt-file)", file=sys.stderr)
        return 2
    if not args.model_path and not args.random_config:
        print("give --model-path (or JLLM_MODEL_PATH) or --random-config", file=sys.stderr)
        return 2
    from .llm import LLM
    from .request import SamplingParams

    model = json.loads(open(args.random_config).read()) if args.random_config else args.model_path
    print(f"loading {args.model_path or args.random_config} ({args.dtype})...", file=sys.stderr, flush=True)
    llm = LLM(model, random_seed=args.random_seed, dtype=args.dtype, block_size=args.block_size,
              num_blocks=args.num_blocks, max_num_seqs=args.max_num_seqs, max_model_len=args.max_model_len,
              max_prefill_len=min(args.max_prefill_len, args.max_model_len),
              max_num_batched_tokens=args.max_num_batched_tokens, max_chunk=args.max_chunk,
              enable_prefix_cache=args.prefix_cache, use_hip_graphs=args.hip_graphs, decode_ahead=args.decode_ahead,
              seed=args.seed)
    if args.prewarm:
        print(f"prewarmed in {llm.prewarm():.2f}s", file=sys.stderr, flush=True)
    sp = SamplingParams(max_new_tokens=args.max_new_tokens, eos_id=args.eos_id, temperature=args.temperature)
    for out in llm.generate(prompts, sp):
        print(" ".join(str(t) for t in out), flush=True)
    if args.stats:
        print(llm.stats, file=sys.stderr)
    return 0


if __name__ == "__main__":
    sys.exit(main())
