"""Minimal usage (options as in the reference's examples/generate.py:10-15; --backend is parsed for that command
line's sake and takes "auto" or "hip", the one attention implementation there is):

    python examples/generate.py --model DIR --max-tokens 64 --temperature 0.0
    python examples/generate.py --model DIR --prompt "Once upon a time" --prompt "The capital of France is"
    python examples/generate.py --model DIR --random-weights 0 --prompt-ids 1,2,3 --prompt-ids 4,5

Without --prompt or --prompt-ids: with a tokenizer.json in the folder the three built-in text prompts are used (two
share a prefix, to show a cache hit); without one, token-id prompts.  Text prompts need the folder's tokenizer.json.
"""
import argparse
import logging
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

from paged_llm_amd import EngineConfig, SamplingParams  # noqa: E402
from paged_llm_amd.engine.llm_engine import LLMEngine  # noqa: E402


def main(argv=None) -> int:
    logging.basicConfig(level=logging.INFO, format="%(message)s")
    ap = argparse.ArgumentParser()
    ap.add_argument("--model", required=True, help="folder with config.json and *.safetensors")
    ap.add_argument("--backend", default="auto", choices=["auto", "hip"])
    ap.add_argument("--max-tokens", type=int, default=64)
    ap.add_argument("--temperature", type=float, default=0.0)
    ap.add_argument("--top-k", type=int, default=-1)
    ap.add_argument("--top-p", type=float, default=1.0)
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--dtype", default="auto", choices=["auto", "bfloat16", "float32"])
    ap.add_argument("--block-size", type=int, default=16)
    ap.add_argument("--num-gpu-blocks", type=int, default=None)
    ap.add_argument("--max-num-batched-tokens", type=int, default=2048)
    ap.add_argument("--max-model-len", type=int, default=4096)
    ap.add_argument("--random-weights", type=int, default=None, metavar="SEED",
                    help="ignore the folder's tensors and fill the model of its config.json with seeded random weights")
    ap.add_argument("--prompt", action="append", default=None, help="a text prompt (needs tokenizer.json in the folder); may be repeated")
    ap.add_argument("--prompt-ids", action="append", default=None, help="comma-separated token ids; may be repeated")
    ap.add_argument("--ignore-eos", action="store_true")
    args = ap.parse_args(argv)

    overrides = {}
    if args.random_weights is not None:
        overrides["random_weights"] = args.random_weights
    engine = LLMEngine(args.model, EngineConfig(
        block_size=args.block_size, num_gpu_blocks=args.num_gpu_blocks, max_num_batched_tokens=args.max_num_batched_tokens,
        max_model_len=args.max_model_len, dtype=args.dtype, seed=args.seed), **overrides)
    if args.prompt or args.prompt_ids:
        if args.prompt and engine.tokenizer is None:
            ap.error(f"--prompt needs a tokenizer.json in {args.model}; give token ids with --prompt-ids instead")
        prompts = list(args.prompt or []) + [[int(t) for t in p.split(",") if t.strip()] for p in args.prompt_ids or []]
    elif engine.tokenizer is not None:
        prompts = [
            "The three laws of robotics are",
            "Explain why paged attention reduces GPU memory fragmentation in one paragraph.",
            "Explain why paged attention reduces GPU memory fragmentation in two sentences.",
        ]
    else:
        shared = list(range(1, 41))
        prompts = [[5, 6, 7, 8, 9], shared + [50, 51], shared + [60, 61, 62]]
    sp = SamplingParams(temperature=args.temperature, top_k=args.top_k, top_p=args.top_p, max_tokens=args.max_tokens,
                        ignore_eos=args.ignore_eos)
    for out in engine.generate(prompts, sp):
        shown = out.text if engine.tokenizer is not None else " ".join(str(t) for t in out.token_ids)
        print(f"--- [{out.finish_reason}] cached_prefix_tokens={out.num_cached_tokens}\n{shown}\n")
    s = engine.stats
    print(f"steps={s.num_steps} prefill_tokens={s.num_prefill_tokens} decode_tokens={s.num_decode_tokens} "
          f"preemptions={s.num_preemptions} attention={engine.attention_backend} dtype={engine.dtype}")
    return 0


if __name__ == "__main__":
    sys.exit(main())
