"""Command line for generation: ``python -m somi_inference_amd.entrypoints.cli``.

The reference has no generation command; its manner is ``python -m <module>``
with long dashed flags (benchmarks/bench_e2e.py:173-324): ``--model-name``,
``--device``, ``--dtype``, ``--block-size``, ``--num-blocks``,
``--max-concurrent``, ``--seed``, ``--temperature``, ``--top-k``, ``--top-p``,
``--repetition-penalty``, ``--output-file`` (JSONL, appended).  Those names and
meanings are kept; ``--prompt`` / ``--prompt-ids`` / ``--max-new-tokens`` and the
random-weights mode are added.
"""

from __future__ import annotations

import argparse
import json
import sys


def parse_args(argv: list[str] | None = None) -> argparse.Namespace:
    parser = argparse.ArgumentParser(description="Generate tokens with the MI355X engine.")
    parser.add_argument("--model-name", type=str, default=None,
                        help="Local model folder (config.json + model.safetensors).")
    parser.add_argument("--write-random-model", type=str, default=None, metavar="DIR",
                        help="Write a model folder of seeded random weights from --config-json and exit "
                             "(or go on to generate from it when prompts are given).")
    parser.add_argument("--config-json", type=str, default=None,
                        help="A config.json to make random weights for (with --write-random-model).")
    parser.add_argument("--random-seed", type=int, default=0, help="Seed of the random weights.")
    parser.add_argument("--num-blocks", type=int, default=256,
                        help="Total KV cache blocks. 0: as many as fit into --memory-fraction of the free memory.")
    parser.add_argument("--memory-fraction", type=float, default=0.9,
                        help="Share of the free device memory that --num-blocks 0 fills with cache blocks.")
    parser.add_argument("--block-size", type=int, default=16, help="KV cache block size.")
    parser.add_argument("--max-concurrent", type=int, default=16, help="Scheduler max concurrent sequences.")
    parser.add_argument("--max-num-batched-tokens", type=int, default=2048, help="Token budget of one step.")
    parser.add_argument("--max-chunk", type=int, default=None, help="Largest prompt portion in one step.")
    parser.add_argument("--device", type=str, default="cuda", choices=["cuda"], help="Execution device.")
    parser.add_argument("--dtype", type=str, default="bfloat16", choices=["float32", "bfloat16"],
                        help="Model and KV-cache dtype.")
    parser.add_argument("--seed", type=int, default=42, help="Random seed for sampling.")
    parser.add_argument("--prompt", type=str, action="append", default=[], help="Text prompt (repeatable).")
    parser.add_argument("--prompt-ids", type=str, action="append", default=[],
                        help="Prompt as comma-separated token ids (repeatable).")
    parser.add_argument("--max-new-tokens", type=int, default=16, help="Tokens to generate per prompt.")
    parser.add_argument("--temperature", type=float, default=0.0,
                        help="Sampling temperature. Use 0.0 for greedy decoding.")
    parser.add_argument("--top-k", type=int, default=-1, help="Top-k sampling cutoff. -1 disables top-k filtering.")
    parser.add_argument("--top-p", type=float, default=1.0, help="Top-p sampling cutoff.")
    parser.add_argument("--repetition-penalty", type=float, default=1.0,
                        help="Repetition penalty applied by the sampler.")
    parser.add_argument("--output-file", type=str, default=None, help="Append results to a JSONL file.")
    parser.add_argument("--warm-up", action="store_true",
                        help="Capture the decode steps as graphs before the prompt is served.")
    return parser.parse_args(argv)


def main(argv: list[str] | None = None) -> int:
    args = parse_args(argv)
    model_dir = args.model_name
    if args.write_random_model:
        if not args.config_json:
            print("--write-random-model needs --config-json", file=sys.stderr)
            return 2
        from ..config.registry import config_from_dict
        from ..weights.random_init import write_random_model
        with open(args.config_json, "r", encoding="utf-8") as handle:
            _, config = config_from_dict(json.load(handle))
        model_dir = write_random_model(args.write_random_model, config, args.random_seed)
        print(f"wrote {model_dir}", file=sys.stderr)
    prompts: list = list(args.prompt) + [[int(t) for t in ids.split(",") if t.strip()] for ids in args.prompt_ids]
    if not prompts:
        return 0 if args.write_random_model else _usage_error("give --prompt or --prompt-ids")
    if not model_dir:
        return _usage_error("give --model-name (or --write-random-model with --config-json)")
    from .llm import LLM
    llm = LLM(model_dir, num_blocks=args.num_blocks or None, memory_fraction=args.memory_fraction,
              block_size=args.block_size,
              max_concurrent=args.max_concurrent, device=args.device, dtype=args.dtype,
              max_num_batched_tokens=args.max_num_batched_tokens, max_chunk=args.max_chunk, seed=args.seed)
    if args.warm_up:
        llm.warm_up()
    outputs = llm.generate(prompts, max_new_tokens=args.max_new_tokens, temperature=args.temperature,
                           top_k=args.top_k, top_p=args.top_p, repetition_penalty=args.repetition_penalty,
                           seed=args.seed)
    for prompt, output in zip(prompts, outputs):
        record = {"prompt": prompt, "output": output}
        print(json.dumps(record))
        if args.output_file:
            with open(args.output_file, "a", encoding="utf-8") as handle:
                handle.write(json.dumps(record) + "\n")
    return 0


def _usage_error(text: str) -> int:
    print(f"error: {text}", file=sys.stderr)
    return 2


if __name__ == "__main__":
    sys.exit(main())
