"""Command line of the engine.  The reference ships no generation program, only its
simulator (sim/simulate.cpp:231-301); ``sim`` keeps that program's option names and exit
codes (--traces, --seed, --trace, --verbose, --model; unknown option: 2; violations: 1), and
``generate`` takes the reference's EngineConfig and SamplingParams field names as options.

    python -m bitwise_amd generate --model DIR --prompt-tokens 5,17,3 --max-new-tokens 16
    python -m bitwise_amd sim --traces 50
    python -m bitwise_amd random --config config.json --seed 0 --out DIR
"""

from __future__ import annotations

import argparse
import json
import sys
from typing import List, Optional

TINY_SIM_CONFIG = {
    # the reference simulator's tiny model sizes (sim/simulate.cpp:64-79) as a Llama: no biases
    "architectures": ["LlamaForCausalLM"], "vocab_size": 97, "hidden_size": 64, "num_hidden_layers": 2,
    "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 16, "intermediate_size": 512,
    "rope_theta": 10000.0, "rms_norm_eps": 1e-6, "tie_word_embeddings": False, "max_position_embeddings": 256,
    "eos_token_id": 3,
}


class _Parser(argparse.ArgumentParser):
    def error(self, message):
        print(f"{self.prog}: {message} (see --help)", file=sys.stderr)
        raise SystemExit(2)


def _engine_options(p: argparse.ArgumentParser) -> None:
    p.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    p.add_argument("--num-blocks", type=int, default=512, help="pages in the cache pool")
    p.add_argument("--block-size", type=int, default=16, help="tokens in a page")
    p.add_argument("--max-batched-tokens", type=int, default=256, help="token budget of one step")
    p.add_argument("--max-num-seqs", type=int, default=32, help="running requests at a time")
    p.add_argument("--no-prefix-caching", action="store_true")
    p.add_argument("--no-graphs", action="store_true", help="launch decode steps kernel by kernel")


def _config(args, bw):
    return bw.EngineConfig(num_blocks=args.num_blocks, max_batched_tokens=args.max_batched_tokens,
                           max_num_seqs=args.max_num_seqs, prefix_caching=not args.no_prefix_caching,
                           block_size=args.block_size, dtype=args.dtype, use_graphs=not args.no_graphs)


def main(argv: Optional[List[str]] = None) -> int:
    ap = _Parser(prog="bitwise_amd", description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    sub = ap.add_subparsers(dest="command", parser_class=_Parser)

    g = sub.add_parser("generate", help="generate tokens for prompts given as token ids")
    g.add_argument("--model", required=True, help="folder with config.json and *.safetensors")
    g.add_argument("--prompt-tokens", action="append", required=True,
                   help="comma-separated token ids; repeat the option for several requests")
    g.add_argument("--max-new-tokens", type=int, default=32)
    g.add_argument("--temperature", type=float, default=0.0, help="0 means greedy")
    g.add_argument("--seed", type=int, default=0)
    g.add_argument("--ignore-eos", action="store_true")
    _engine_options(g)

    s = sub.add_parser("sim", help="randomized scheduling traces against solo runs")
    s.add_argument("--traces", type=int, default=50, help="randomized workloads to run")
    s.add_argument("--seed", type=int, default=1, help="base seed")
    s.add_argument("--trace", type=int, default=-1, help="run only trace N")
    s.add_argument("--verbose", action="store_true", help="print each violation")
    s.add_argument("--model", default="", help="model folder instead of the random tiny model")
    s.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    s.add_argument("--block-size", type=int, default=16)

    r = sub.add_parser("random", help="write a model folder with seeded random weights")
    r.add_argument("--config", required=True, help="a config.json")
    r.add_argument("--seed", type=int, default=0)
    r.add_argument("--sigma", type=float, default=0.02, help="standard deviation of linear and embedding weights")
    r.add_argument("--weight-dtype", choices=["bfloat16", "float32"], default="bfloat16")
    r.add_argument("--out", required=True)

    args = ap.parse_args(argv)
    if args.command is None:
        ap.print_help()
        return 2
    import bitwise_amd as bw

    if args.command == "random":
        cfg = json.loads(open(args.config).read())
        print(bw.write_random_model(args.out, cfg, args.seed, args.sigma, args.weight_dtype))
        return 0

    if args.command == "generate":
        model = bw.Model.load(args.model, args.dtype)
        prompts = [[int(t) for t in p.replace(" ", "").split(",") if t] for p in args.prompt_tokens]
        sp = bw.SamplingParams(temperature=args.temperature, seed=args.seed, max_new_tokens=args.max_new_tokens,
                               ignore_eos=args.ignore_eos)
        for i, res in enumerate(bw.generate(model, prompts, sp, _config(args, bw))):
            print(json.dumps({"request": i, "tokens": res.tokens, "logits_fingerprint": hex(res.logits_fingerprint),
                              "preemptions": res.preemptions, "prefix_cached_tokens": res.prefix_cached_tokens}))
        return 0

    from .sim import Simulator
    if args.model:
        model = bw.Model.load(args.model, args.dtype)
    else:
        model = bw.Model.random(TINY_SIM_CONFIG, 42, args.dtype, sigma=0.08)
    sim = Simulator(model, args.dtype, args.block_size, args.verbose)
    out = sim.run(args.traces, args.seed, args.trace)
    print(Simulator.report("invariant kernels", out, args.traces))
    if args.verbose:
        for note in out.notes:
            print("  " + note)
    return 1 if out.violations() else 0


if __name__ == "__main__":
    sys.exit(main())
