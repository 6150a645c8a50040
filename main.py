"""Command line of the engine, in the manner of the reference's main.py: the options
carry the names of its constants (main.py:17-27) and mean the same.

    python main.py --model-name-or-path DIR --prompt "text" --max-new-tokens 64
    python main.py --model-name-or-path DIR --prompt-ids 5,17,3 --prompt-ids 9,9
    python main.py --random-weights CONFIG.json --seed 0 --model-name-or-path OUT_DIR ...
"""
import argparse
import json
import os
import sys

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

DEFAULT_PROMPTS = [   # the reference's three prompts (main.py:64-68); the third is a prefix of the second
    "介绍一下Qwen模型",
    "How can remote teams improve trust, focus, communication, and delivery speed without adding more "
    "meetings? Please include practical examples that small teams can apply immediately.",
    "How can remote teams improve trust, focus, communication, and delivery speed without adding",
]


def parse_args(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--model-name-or-path", "--model", required=True, dest="model_name_or_path",
                    help="folder with config.json and *.safetensors (and tokenizer.json for text prompts)")
    ap.add_argument("--random-weights", metavar="CONFIG_JSON", default=None,
                    help="write random weights for this config.json into --model-name-or-path first")
    ap.add_argument("--seed", type=int, default=0, help="seed of random weights and of sampling")
    ap.add_argument("--prompt", action="append", default=[], help="a text prompt (repeatable)")
    ap.add_argument("--prompt-ids", action="append", default=[],
                    help="a prompt as comma-separated token ids (repeatable)")
    ap.add_argument("--max-new-tokens", type=int, default=64)
    ap.add_argument("--max-num-seqs", type=int, default=4)
    ap.add_argument("--max-model-len", type=int, default=256)
    ap.add_argument("--block-size", type=int, default=16, help="tokens per cache page")
    ap.add_argument("--num-blocks", type=int, default=None,
                    help="cache pages; default max_num_seqs * ceil(max_model_len / block_size)")
    ap.add_argument("--gpu-memory-fraction", type=float, default=None,
                    help="without --num-blocks: size the cache from this fraction of the device memory that is "
                         "free once the weights are loaded")
    ap.add_argument("--model-dtype", "--dtype", dest="model_dtype", default="bfloat16",
                    choices=["bfloat16", "float32"])
    ap.add_argument("--temperature", type=float, default=0.0, help="0: greedy")
    ap.add_argument("--max-step-tokens", type=int, default=2048, help="token budget of one step")
    ap.add_argument("--prefill-chunk", type=int, default=512, help="largest portion of a prompt in a step in which some request decodes (else the whole budget)")
    ap.add_argument("--ignore-eos", action="store_true")
    ap.add_argument("--no-prefix-sharing", action="store_true")
    ap.add_argument("--debug-poison", action="store_true",
                    help="fill every cache page with NaN when it is handed out and when it goes back")
    ap.add_argument("--stats", action="store_true", help="print the engine's counters at the end")
    return ap.parse_args(argv)


def main(argv=None) -> int:
    args = parse_args(argv)
    import torch
    import qwen_engine_amd  # noqa: F401
    from qwen_engine_amd.config import EngineConfig, config_from_dict
    from qwen_engine_amd.engine import LLMEngine
    from qwen_engine_amd.weights import write_model_folder

    if args.random_weights:
        with open(args.random_weights) as f:
            config = config_from_dict(json.load(f))
        write_model_folder(args.model_name_or_path, config, args.seed, dtype=torch.bfloat16)

    engine_config = EngineConfig(
        dtype=args.model_dtype, block_size=args.block_size, num_blocks=args.num_blocks,
        max_num_seqs=args.max_num_seqs, max_model_len=args.max_model_len,
        max_step_tokens=args.max_step_tokens, prefill_chunk=args.prefill_chunk,
        enable_prefix_sharing=not args.no_prefix_sharing, seed=args.seed,
        debug_poison=args.debug_poison, gpu_memory_fraction=args.gpu_memory_fraction)
    engine = LLMEngine.from_folder(args.model_name_or_path, engine_config)

    prompts = list(args.prompt) + [[int(t) for t in p.split(",") if t.strip()] for p in args.prompt_ids]
    if not prompts:
        if engine.tokenizer is None:
            print("no prompt given and the model folder has no tokenizer.json: use --prompt-ids", file=sys.stderr)
            return 2
        prompts = DEFAULT_PROMPTS
    engine.submit(prompts, max_new_tokens=args.max_new_tokens, temperature=args.temperature,
                  ignore_eos=args.ignore_eos)

    def print_info(prompt_text, output_text):   # main.py:74-79
        print("=" * 88)
        print(f"Prompt: {prompt_text}")
        print("=" * 88)
        print(output_text)
        print("=" * 88)

    engine.serving(print_func=print_info)
    if args.stats:
        print(json.dumps(engine.stats()))
    return 0


if __name__ == "__main__":
    sys.exit(main())
