"""The command line: generate from a model folder or from seeded random weights.

In the manner of the reference's ``python generate.py`` (``generate.py:245-315``): it loads the
model, streams the generated tokens as they come, prints the run's metrics (time to first token,
time per output token, tokens a second, peak memory) and, if asked, writes them as JSON.  What the
reference fixes as constants in its ``__main__`` are options here, with the reference's values as
defaults where it has them (temperature 0.7, top-k 50, top-p 0.9, a context of 4096).
"""

from __future__ import annotations

import argparse
import json
import sys


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(prog="generate.py", description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    src = ap.add_mutually_exclusive_group(required=True)
    src.add_argument("--model", help="folder with config.json and model.safetensors")
    src.add_argument("--random", metavar="PRESET", help="random weights for a named shape (see --list-presets)")
    ap.add_argument("--seed", type=int, default=0, help="seed of the random weights")
    ap.add_argument("--write-model", metavar="DIR", help="with --random: write the model folder there and exit")
    prm = ap.add_mutually_exclusive_group()
    prm.add_argument("--prompt-ids", help="comma separated token ids")
    prm.add_argument("--prompt", help="text (the model folder must hold tokenizer.json)")
    prm.add_argument("--prompt-len", type=int, help="that many seeded random token ids")
    ap.add_argument("--max-new-tokens", type=int, default=256)
    ap.add_argument("--temperature", type=float, default=0.7, help="0 is greedy")
    ap.add_argument("--top-k", type=int, default=50, help="0 turns it off")
    ap.add_argument("--top-p", type=float, default=0.9, help="1 turns it off")
    ap.add_argument("--sample-seed", type=int, default=0)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--max-seq-len", type=int, default=4096)
    ap.add_argument("--max-running", type=int, default=8)
    ap.add_argument("--block-size", type=int, default=16, help="tokens per cache page")
    ap.add_argument("--num-kv-blocks", type=int, default=None, help="cache pages (default: max_running full contexts)")
    ap.add_argument("--chunk-tokens", type=int, default=512, help="most tokens one step runs")
    ap.add_argument("--no-graphs", action="store_true", help="do not replay decode steps from hipGraphs")
    ap.add_argument("--no-run-ahead", action="store_true",
                    help="do not launch a step before the tokens of the step before have been read")
    ap.add_argument("--use-prefix-cache", action="store_true")
    ap.add_argument("--profile-ranges", action="store_true",
                    help="named ranges around schedule / forward / sample / collect for a profiler's timeline")
    ap.add_argument("--stats-json", metavar="FILE", help="write the run's metrics there")
    ap.add_argument("--device", default="cuda:0")
    return ap


def main(argv=None) -> int:
    if argv is not None and "--list-presets" in argv or argv is None and "--list-presets" in sys.argv:
        from .config import PRESETS
        print("\n".join(sorted(PRESETS)))
        return 0
    args = build_parser().parse_args(argv)
    import torch

    from . import Engine, EngineConfig, preset
    from .weights import random_tensors, write_model_folder

    if args.write_model:
        if not args.random:
            print("--write-model needs --random", file=sys.stderr)
            return 2
        from .engine.build import build_model
        cfg = preset(args.random)
        model, model_cfg = build_model(cfg, EngineConfig(device="cpu", dtype="float32", max_seq_len=64), kernels=None)
        write_model_folder(args.write_model, model_cfg.to_dict(), random_tensors(model.expected_tensors(), args.seed))
        print(f"wrote {args.write_model}")
        return 0

    ecfg = EngineConfig(
        max_running=args.max_running, max_seq_len=args.max_seq_len, block_size=args.block_size,
        num_kv_blocks=args.num_kv_blocks, chunk_tokens=args.chunk_tokens, dtype=args.dtype,
        use_graphs=not args.no_graphs, run_ahead=not args.no_run_ahead, use_prefix_cache=args.use_prefix_cache, profile_ranges=args.profile_ranges,
        device=args.device)
    print("Loading model...", file=sys.stderr, flush=True)
    if args.model:
        engine = Engine.from_folder(args.model, ecfg)
    else:
        engine = Engine.from_random(preset(args.random), args.seed, ecfg, generate_on_device=True)
    vocab = engine.model.vocab_size
    print(engine.describe(), file=sys.stderr, flush=True)

    tokenizer = None
    if args.prompt is not None:
        from .tokenizer import Tokenizer
        tokenizer = Tokenizer.from_folder(args.model or ".", engine.model.plan.bos_token_id)
        prompt = tokenizer.encode(args.prompt, add_bos=True)
    elif args.prompt_ids is not None:
        prompt = [int(t) for t in args.prompt_ids.replace(" ", "").split(",") if t]
    else:
        g = torch.Generator().manual_seed(args.sample_seed)
        prompt = torch.randint(0, vocab, (args.prompt_len or 16,), generator=g).tolist()

    def show(token):
        print(tokenizer.decode([token]) if tokenizer else token, end="" if tokenizer else " ", flush=True)

    print(f"Prompt: {len(prompt)} tokens\nOutput: ", end="", flush=True)
    tokens, stats = engine.generate_with_stats(
        prompt, max_new_tokens=args.max_new_tokens, temperature=args.temperature, top_k=args.top_k,
        top_p=args.top_p, seed=args.sample_seed, on_token=show)
    print()
    print("=" * 52)
    for key in ("prompt_tokens", "new_tokens", "ttft_ms", "tpot_ms", "decode_tok_s", "total_tok_s", "total_wall_ms",
                "peak_vram_gb"):
        v = stats[key]
        print(f"  {key:<16}: {v:.3f}" if isinstance(v, float) else f"  {key:<16}: {v}")
    print("=" * 52)
    if args.stats_json:
        stats["tokens"] = tokens
        stats["sampling"] = {"temperature": args.temperature, "top_k": args.top_k, "top_p": args.top_p,
                             "seed": args.sample_seed}
        with open(args.stats_json, "w") as f:
            json.dump(stats, f, indent=2)
    return 0


if __name__ == "__main__":
    sys.exit(main())
