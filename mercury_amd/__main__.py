"""Command line: ``python -m mercury_amd generate ...`` and ``python -m mercury_amd random-weights ...``.

Token ids in, token ids out; no tokenizer is involved.  Engine options carry the names and
meanings of the reference's server command line where it has them
(reference: mercury/server.py:249-284).
"""

from __future__ import annotations

import argparse
import json
import sys


def build_parser() -> argparse.ArgumentParser:
    parser = argparse.ArgumentParser("mercury_amd")
    sub = parser.add_subparsers(dest="command", required=True)

    g = sub.add_parser("generate", help="generate tokens for prompts given as token ids")
    g.add_argument("--model", default=None, help="folder with config.json and safetensors weights")
    g.add_argument("--random-config", default=None, metavar="CONFIG_JSON",
                   help="instead of --model: a config.json (or a folder with one) whose model "
                        "gets random weights, drawn from --weight-seed")
    g.add_argument("--weight-seed", type=int, default=0)
    g.add_argument("--weight-std", type=float, default=0.02)
    g.add_argument("--prompt-ids", action="append", default=[],
                   help="one prompt as comma- or space-separated token ids; may be repeated")
    g.add_argument("--prompt-file", default=None,
                   help="file with one prompt per line (token ids, or a JSON list)")
    g.add_argument("--max-tokens", type=int, default=16)
    g.add_argument("--temperature", type=float, default=0.0)
    g.add_argument("--top-p", type=float, default=1.0)
    g.add_argument("--ignore-eos", action="store_true")
    g.add_argument("--device", default="cuda:0")
    g.add_argument("--dtype", default="bfloat16", help="bfloat16 or float32")
    g.add_argument("--policy", default="fcfs", choices=("fcfs", "lpm", "lpm_aging"))
    g.add_argument("--block-size", type=int, default=16)
    g.add_argument("--num-blocks", type=int, default=4096, help="-1 sizes to free memory")
    g.add_argument("--max-running", type=int, default=64)
    g.add_argument("--prefill-budget", type=int, default=8192)
    g.add_argument("--max-model-len", type=int, default=8192)
    g.add_argument("--aging-tokens-per-s", type=float, default=2000.0)
    g.add_argument("--max-wait-s", type=float, default=5.0)
    g.add_argument("--scan-limit", type=int, default=128)
    g.add_argument("--cryptographic-hashes", action="store_true")
    g.add_argument("--debug-invariants", action="store_true")
    g.add_argument("--no-graphs", action="store_true",
                   help="launch every decode step kernel by kernel instead of replaying a HIP graph")
    g.add_argument("--no-lookahead", action="store_true",
                   help="never start a decode step before the previous one's tokens are read")
    g.add_argument("--seed", type=int, default=0)
    g.add_argument("--stats", action="store_true", help="print the engine snapshot to stderr")

    r = sub.add_parser("random-weights", help="write a model folder with seeded random weights")
    r.add_argument("--config", required=True, help="a config.json naming the architecture and sizes")
    r.add_argument("--out", required=True, help="folder to write config.json and model.safetensors")
    r.add_argument("--seed", type=int, default=0)
    r.add_argument("--std", type=float, default=0.02)
    r.add_argument("--dtype", default="bfloat16", help="storage dtype: bfloat16 or float32")
    return parser


def parse_prompt(text: str) -> list:
    text = text.strip()
    if text.startswith("["):
        return [int(t) for t in json.loads(text)]
    return [int(t) for t in text.replace(",", " ").split()]


def run_generate(args) -> int:
    from .config.engine_config import EngineConfig
    from .engine.engine import Engine
    from .engine import SamplingParams

    prompts = [parse_prompt(p) for p in args.prompt_ids]
    if args.prompt_file:
        with open(args.prompt_file) as f:
            prompts += [parse_prompt(line) for line in f if line.strip()]
    if not prompts:
        print("no prompts: give --prompt-ids or --prompt-file", file=sys.stderr)
        return 2
    if (args.model is None) == (args.random_config is None):
        print("give exactly one of --model and --random-config", file=sys.stderr)
        return 2
    cfg = EngineConfig(
        model=args.model or args.random_config, random_weights=args.model is None,
        weight_seed=args.weight_seed, weight_std=args.weight_std, device=args.device, dtype=args.dtype, block_size=args.block_size,
        num_blocks=args.num_blocks, max_running=args.max_running,
        prefill_budget=args.prefill_budget, max_model_len=args.max_model_len, policy=args.policy,
        aging_tokens_per_s=args.aging_tokens_per_s, max_wait_s=args.max_wait_s,
        scan_limit=args.scan_limit, cryptographic_hashes=args.cryptographic_hashes,
        debug_invariants=args.debug_invariants, seed=args.seed,
        use_graphs=not args.no_graphs, lookahead=not args.no_lookahead)
    engine = Engine(cfg)
    params = SamplingParams(temperature=args.temperature, top_p=args.top_p,
                            ignore_eos=args.ignore_eos)
    outputs = engine.generate(prompts, params, args.max_tokens)
    for index, tokens in enumerate(outputs):
        print(json.dumps({"prompt_index": index, "tokens": tokens}), flush=True)
    if args.stats:
        print(json.dumps(engine.snapshot()), file=sys.stderr)
    return 0


def run_random_weights(args) -> int:
    import torch

    from .weights.random_init import write_random_model

    dtypes = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16,
              "float32": torch.float32, "fp32": torch.float32}
    if args.dtype not in dtypes:
        print(f"--dtype must be one of {sorted(dtypes)}", file=sys.stderr)
        return 2
    with open(args.config) as f:
        config = json.load(f)
    folder = write_random_model(args.out, config, args.seed, args.std, dtypes[args.dtype])
    print(folder)
    return 0


def main(argv=None) -> int:
    args = build_parser().parse_args(argv)
    if args.command == "generate":
        return run_generate(args)
    return run_random_weights(args)


if __name__ == "__main__":
    sys.exit(main())
