"""Command line of the engine.  The reference ships no generation program, only its
simulator (sim/simulate.cpp:231-301); ``sim`` keeps that program's option names and exit
codes (--traces, --seed, --trace, --fault, --sweep-faults, --verbose, --model; unknown option: 2;
violations: 1), and ``generate`` takes the reference's EngineConfig and SamplingParams field names as options.

    python -m bitwise_amd generate --model DIR --prompt-tokens 5,17,3 --max-new-tokens 16
    python -m bitwise_amd generate --random-config config.json --weights-seed 0 --prompt-tokens 5,17,3
    python -m bitwise_amd sim --traces 50 [--fault 4 | --sweep-faults]
    python -m bitwise_amd bench --model DIR --batch 8 --context 512
    python -m bitwise_amd random --config config.json --seed 0 --out DIR
"""

from __future__ import annotations

import argparse
import json
import sys
from typing import List, Optional


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


def _model_options(p: argparse.ArgumentParser) -> None:
    p.add_argument("--model", default="", help="folder with config.json and *.safetensors")
    p.add_argument("--random-config", default="", help="a config.json: run it with seeded random weights instead of a folder")
    p.add_argument("--weights-seed", type=int, default=0, help="seed of the random weights")
    p.add_argument("--sigma", type=float, default=0.02, help="standard deviation of random linear and embedding weights")


def _load_model(args, bw):
    if bool(args.model) == bool(args.random_config):
        print("bitwise_amd: give one of --model DIR and --random-config FILE (see --help)", file=sys.stderr)
        raise SystemExit(2)
    if args.model:
        return bw.Model.load(args.model, args.dtype)
    return bw.Model.random(json.loads(open(args.random_config).read()), args.weights_seed, args.dtype, sigma=args.sigma)


def _config(args, bw):
    return bw.EngineConfig(num_blocks=args.num_blocks, max_batched_tokens=args.max_batched_tokens,
                           max_num_seqs=args.max_num_seqs, prefix_caching=not args.no_prefix_caching,
                           block_size=args.block_size, dtype=args.dtype, use_graphs=not args.no_graphs)


def _sim(args, bw) -> int:
    from .config.engine import Fault
    from .registry import ARCHITECTURES
    from .sim import Simulator

    if args.fault and args.fault not in Fault.NAMES:
        print(f"bitwise_amd sim: --fault takes one of {sorted(Fault.NAMES)} (3 belongs to speculative decoding, which "
              f"this engine does not do)", file=sys.stderr)
        return 2
    if args.model:
        model = bw.Model.load(args.model, args.dtype)
    else:
        tiny = ARCHITECTURES[args.architecture].tiny_config
        if tiny is None:
            print(f"bitwise_amd sim: architecture {args.architecture} names no tiny configuration; give --model", file=sys.stderr)
            return 2
        model = bw.Model.random(tiny, 42, args.dtype, sigma=0.08)

    def run(fault: int, label: str):
        tally = Simulator(model, args.dtype, args.verbose, fault=fault).run(args.traces, args.seed, args.trace)
        print(tally.line(label), flush=True)
        if args.verbose:
            for note in tally.notes:
                print("  " + note.replace("\n", "\n  "))
        return tally

    if not args.sweep_faults:
        return 1 if run(args.fault, Fault.NAMES.get(args.fault, "no fault")).violations() else 0
    clean = run(0, "no fault")
    caught = sum(run(f, f"fault {f}, {name}").violations() > 0 for f, name in sorted(Fault.NAMES.items()))
    print(f"caught {caught} of {len(Fault.NAMES)} injected faults; violations of the run without a fault: {clean.violations()}")
    return 1 if clean.violations() or caught < len(Fault.NAMES) else 0


def _bench(args, bw) -> int:
    import torch
    from . import measure

    model = _load_model(args, bw)
    cfg = model.config.to_dict()
    out = {"model": args.model or args.random_config, "dtype": args.dtype, "batch": args.batch, "context": args.context}
    out["decode"] = measure.measure_decode(bw, torch, model, cfg, args.dtype, args.batch, args.steps, args.warmup, context=args.context)
    if args.prefill_tokens:
        out["prefill"] = measure.measure_prefill(bw, torch, model, cfg, args.dtype, measure.PEAK_FLOPS[args.dtype], args.prefill_tokens)
    print(json.dumps(out))
    return 0


def main(argv: Optional[List[str]] = None) -> int:
    ap = _Parser(prog="bitwise_amd", description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    sub = ap.add_subparsers(dest="command", parser_class=_Parser)

    g = sub.add_parser("generate", help="generate tokens for prompts given as token ids")
    _model_options(g)
    g.add_argument("--prompt-tokens", action="append", required=True,
                   help="comma-separated token ids; repeat the option for several requests")
    g.add_argument("--max-new-tokens", type=int, default=32)
    g.add_argument("--temperature", type=float, default=0.0, help="0 means greedy")
    g.add_argument("--seed", type=int, default=0)
    g.add_argument("--ignore-eos", action="store_true")
    _engine_options(g)

    s = sub.add_parser("sim", help="randomized scheduling scenarios against solo runs")
    s.add_argument("--traces", type=int, default=50, help="randomized scenarios to run")
    s.add_argument("--seed", type=int, default=1, help="base seed")
    s.add_argument("--trace", type=int, default=-1, help="run only scenario N")
    s.add_argument("--fault", type=int, default=0, help="switch on test-only bug F of the engine (1, 2, 4 or 5): the run must report violations")
    s.add_argument("--sweep-faults", action="store_true", help="run without a fault and with every fault; report which are caught")
    s.add_argument("--verbose", action="store_true", help="print each violation with its scenario")
    s.add_argument("--model", default="", help="model folder instead of the architecture's tiny random model")
    s.add_argument("--architecture", default="LlamaForCausalLM", help="whose tiny configuration to simulate without --model")
    s.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")

    b = sub.add_parser("bench", help="time decode steps and a prefill of a model with synthetic tokens")
    _model_options(b)
    b.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    b.add_argument("--batch", type=int, default=8, help="requests decoding at once")
    b.add_argument("--context", type=int, default=512, help="tokens each request holds when the timed steps begin")
    b.add_argument("--steps", type=int, default=32)
    b.add_argument("--warmup", type=int, default=4)
    b.add_argument("--prefill-tokens", type=int, default=512, help="length of the timed prompt (0: no prefill)")

    r = sub.add_parser("random", help="write a model folder with seeded random weights")
    r.add_argument("--config", required=True, help="a config.json")
    r.add_argument("--seed", type=int, default=0)
    r.add_argument("--sigma", type=float, default=0.02, help="standard deviation of linear and embedding weights")
    r.add_argument("--weight-dtype", choices=["bfloat16", "float32", "float16"], default="bfloat16")
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
    if args.command == "sim":
        return _sim(args, bw)
    if args.command == "bench":
        return _bench(args, bw)

    model = _load_model(args, bw)
    prompts = [[int(t) for t in p.replace(" ", "").split(",") if t] for p in args.prompt_tokens]
    sp = bw.SamplingParams(temperature=args.temperature, seed=args.seed, max_new_tokens=args.max_new_tokens,
                           ignore_eos=args.ignore_eos)
    for i, res in enumerate(bw.generate(model, prompts, sp, _config(args, bw))):
        print(json.dumps({"request": i, "tokens": res.tokens, "logits_fingerprint": hex(res.logits_fingerprint),
                          "preemptions": res.preemptions, "prefix_cached_tokens": res.prefix_cached_tokens}))
    return 0


if __name__ == "__main__":
    sys.exit(main())
