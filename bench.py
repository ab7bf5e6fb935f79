#!/usr/bin/env python3
"""Decode and prefill throughput of the engine on one MI355X, at the SmolLM2-1.7B shape with
random weights and uniform random token ids.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--dtype bf16|fp32] [--batch B] [--layers L]
                    [--prefill-tokens T] [--no-points] [--shape smollm2|llama3_8b] [--trace-only] [--decode-phases] [--portion-align A] [--mixed] [--sweep]

A step is one decode step of the whole engine (scheduler, graph replay of the model, sampling,
token hand-back) for a batch of B requests that each hold a 2,048-token context.  ``value`` is
decoded tokens per second.  One JSON line is printed; it also carries the 2,048-token prefill,
the decode step's HBM roofline, decode at batch 1 and 64 with their rooflines, the same model's true
32-bit path (decode and prefill) and, at Llama-3-8B's sizes, decode, prefill, a continuous-batching workload
of 64 requests and a trace of 128 requests with shared prefixes, cancellations and preemption whose sampled requests
are checked against solo runs.
"""

from __future__ import annotations

import argparse
import json
import sys
import time

PREFILL_TOKENS = 2048

# Layer sizes of the SmolLM2-1.7B shape: 24 layers, width 2048, 32 heads on 32 kv heads of size
# 64, feed-forward 8192, vocabulary 49152, rotary base 130000, eps 1e-5, tied embeddings.
SMOLLM2_1_7B = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama", "hidden_act": "silu",
    "vocab_size": 49152, "hidden_size": 2048, "num_hidden_layers": 24, "num_attention_heads": 32,
    "num_key_value_heads": 32, "head_dim": 64, "intermediate_size": 8192, "rope_theta": 130000.0,
    "rms_norm_eps": 1e-5, "tie_word_embeddings": True, "max_position_embeddings": 4096,
    "bos_token_id": 1, "eos_token_id": 2,
}
BASELINE_TOK_S = 7.26               # the reference's published SmolLM2-1.7B decode rate (one stream, 4-core CPU)


LLAMA3_8B = {
    # Llama-3-8B's sizes: 32 layers, width 4096, 32 heads on 8 kv heads of 128,
    # feed-forward 14336, vocabulary 128256, rotary base 500000 without scaling, eps 1e-5, untied head.
    "architectures": ["LlamaForCausalLM"], "model_type": "llama", "hidden_act": "silu",
    "vocab_size": 128256, "hidden_size": 4096, "num_hidden_layers": 32, "num_attention_heads": 32,
    "num_key_value_heads": 8, "head_dim": 128, "intermediate_size": 14336, "rope_theta": 500000.0,
    "rms_norm_eps": 1e-5, "tie_word_embeddings": False, "max_position_embeddings": 8192,
    "bos_token_id": 1, "eos_token_id": 2,
}


def sweep(bw, torch, steps: int, dtype: str) -> int:
    """Decode steps over batch and context, prefills over length: in bfloat16 at both shapes, in the 32-bit mode a
    coarser grid at the small one.  One JSON object a line."""
    from bitwise_amd.measure import PEAK_FLOPS, measure_decode, measure_prefill
    bf16 = dtype == "bfloat16"
    shapes = (("SmolLM2-1.7B", SMOLLM2_1_7B), ("Llama-3-8B", LLAMA3_8B)) if bf16 else (("SmolLM2-1.7B", SMOLLM2_1_7B),)
    for name, shape in shapes:
        cfg = dict(shape, max_position_embeddings=16384)
        model = bw.Model.random(cfg, seed=0, dtype=dtype, sigma=0.02, on_device=True)
        for tokens in ((128, 256, 512, 1024, 2048) if bf16 else (128, 512, 2048)):
            m = measure_prefill(bw, torch, model, cfg, dtype, PEAK_FLOPS[dtype], tokens)
            print(json.dumps({"shape": name, "dtype": dtype, "prefill_tokens": tokens, "ms": m["ms"], "tok_s": m["value"],
                              "frac_of_matrix_peak": m["frac"]}), flush=True)
        for context in ((512, 2048, 8192) if bf16 else (512, 2048)):
            for batch in ((1, 2, 4, 8, 16, 32, 64, 128) if bf16 else (1, 8, 64)):
                if batch * context > 512 * 1024:          # (a pool of at most half a million tokens)
                    continue
                m = measure_decode(bw, torch, model, cfg, dtype, batch, steps, 4, context=context)
                print(json.dumps({"shape": name, "dtype": dtype, "decode_batch": batch, "context": context,
                                  "ms_per_step": m["ms_per_step"], "tok_s": m["tok_s"], "frac_of_8_TBs": m["roofline"]["frac"]}),
                      flush=True)
        del model
        torch.cuda.empty_cache()
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--dtype", choices=["bf16", "fp32"], default="bf16")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=0, help="run fewer layers than the shape has (named in config)")
    ap.add_argument("--prefill-tokens", type=int, default=PREFILL_TOKENS,
                    help="the length of the headline prefill's prompt (for profiles of shorter prompts; up to 2048)")
    ap.add_argument("--shape", choices=["smollm2", "llama3_8b"], default="smollm2",
                    help="the layer sizes of the headline run (llama3_8b: for profiles of that shape; implies --no-points)")
    ap.add_argument("--trace-only", action="store_true",
                    help="run nothing but the 128-request shared-prefix trace at Llama-3-8B's sizes and print its figures (for profiles)")
    ap.add_argument("--decode-phases", action="store_true",
                    help="the headline decode with EngineConfig.decode_phases (its products as phases of a few launches; for profiles)")
    ap.add_argument("--portion-align", type=int, default=64,
                    help="EngineConfig.portion_align of the headline decode's engine (1: prompts cut exactly at the budget; for profiles)")
    ap.add_argument("--mixed", action="store_true",
                    help="only: an 8,192-token prompt beside 7 decoding requests, with portions cut at the budget and cut to whole blocks")
    ap.add_argument("--sweep", action="store_true",
                    help="print a table instead of the line: decode at batches 1 to 128 and contexts of 512 to 8,192 tokens, prefills "
                         "of 128 to 2,048 tokens, at both shapes (with --dtype fp32: a coarser grid at the small shape)")
    ap.add_argument("--no-points", action="store_true",
                    help="only the headline: skip decode at batch 1 and 64, the 32-bit path and the Llama-3-8B sizes")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported (use --gpus 1)")
        return 2

    import torch
    import bitwise_amd as bw
    from bitwise_amd.measure import (CONTEXT, PEAK_FLOPS, measure_chunked_prefill, measure_decode, measure_prefill, measure_serving,
                                     measure_trace)

    dtype = "bfloat16" if args.dtype == "bf16" else "float32"
    if args.sweep:
        return sweep(bw, torch, args.steps, dtype)
    if args.mixed:
        from bitwise_amd.measure import measure_prefill_beside_decodes, measure_qkv_row_orders
        cfg = dict(SMOLLM2_1_7B if args.shape == "smollm2" else LLAMA3_8B, max_position_embeddings=16384)
        model = bw.Model.random(cfg, seed=0, dtype=dtype, sigma=0.02, on_device=True)
        print(json.dumps({"shape": args.shape, "dtype": args.dtype,
                          "prompt_beside_decodes": [measure_prefill_beside_decodes(bw, torch, model, cfg, dtype, portion_align=a)
                                                    for a in (1, 64, 1, 64)],
                          "qkv_us_by_row_order": measure_qkv_row_orders(torch, cfg) if args.dtype == "bf16" else {}}))
        return 0
    if args.trace_only:
        big = dict(LLAMA3_8B, max_position_embeddings=16384)
        model8 = bw.Model.random(big, seed=1, dtype=dtype, sigma=0.02, on_device=True)
        print(json.dumps({"llama3_8b.trace8k": measure_trace(bw, torch, model8, big, dtype, check=8), "dtype": args.dtype}))
        return 0
    cfg = dict(SMOLLM2_1_7B if args.shape == "smollm2" else LLAMA3_8B)
    shape_name = "SmolLM2-1.7B" if args.shape == "smollm2" else "Llama-3-8B"
    if args.shape != "smollm2":
        args.no_points = True
    full_layers = cfg["num_hidden_layers"]
    if args.layers:
        cfg["num_hidden_layers"] = args.layers
    t_start = time.perf_counter()
    model = bw.Model.random(cfg, seed=0, dtype=dtype, sigma=0.02, on_device=True)
    vocab = cfg["vocab_size"]
    side_steps = max(16, args.steps // 2)

    if not 1 <= args.prefill_tokens <= PREFILL_TOKENS:
        print(f"bench.py: --prefill-tokens {args.prefill_tokens} is outside 1..{PREFILL_TOKENS}")
        return 2
    prefill = measure_prefill(bw, torch, model, cfg, dtype, PEAK_FLOPS[args.dtype], args.prefill_tokens)
    head = measure_decode(bw, torch, model, cfg, dtype, args.batch, args.steps, args.warmup, decode_phases=args.decode_phases,
                         portion_align=args.portion_align)
    points, point_rooflines = {}, {}
    extra = {}
    if not args.no_points:
        for b in (1, 64):
            m = measure_decode(bw, torch, model, cfg, dtype, b, side_steps, 4)
            points[f"decode_b{b}"] = m["tok_s"]
            point_rooflines[f"decode_b{b}"] = m["roofline"]
        for t in (128, 512):                          # shorter prompts, one step each: tokens a second
            points[f"prefill_t{t}"] = measure_prefill(bw, torch, model, cfg, dtype, PEAK_FLOPS[args.dtype], t)["value"]
        if args.dtype == "bf16":
            # the same layers with 8,192-token contexts (position tables of 16,384; batch 8)
            del model
            torch.cuda.empty_cache()
            long_cfg = dict(cfg, max_position_embeddings=16384)
            model_long = bw.Model.random(long_cfg, seed=0, dtype=dtype, sigma=0.02, on_device=True)
            m = measure_decode(bw, torch, model_long, long_cfg, dtype, 8, side_steps, 4, context=8192)
            points["decode_b8_ctx8192"] = m["tok_s"]
            point_rooflines["decode_b8_ctx8192"] = m["roofline"]
            del model_long
            model = None
            torch.cuda.empty_cache()
            # the true 32-bit path of the same model (the same bfloat16 weights, widened exactly; 32-bit caches)
            model32 = bw.Model.random(cfg, seed=0, dtype="float32", sigma=0.02, on_device=True)
            m = measure_decode(bw, torch, model32, cfg, "float32", args.batch, side_steps, 4)
            extra["fp32"] = {"decode_tok_s": m["tok_s"], "batch": args.batch, "ms_per_step": m["ms_per_step"],
                             "roofline": m["roofline"], "weights_stored_as": "bfloat16, widened exactly where they are used",
                             "prefill": measure_prefill(bw, torch, model32, cfg, "float32", PEAK_FLOPS["fp32"])}
            del model32
            torch.cuda.empty_cache()
            # Llama-3-8B's sizes, all 32 layers, bfloat16 (position tables of 16,384 for the 8,192-token contexts): decode at
            # batch 8, 1 and 64 with 2,048-token contexts and at batch 8 with 8,192-token contexts, a prefill of 2,048 tokens
            # in one step and one of 8,192 in portions of 2,048
            big = dict(LLAMA3_8B, max_position_embeddings=16384)
            model8 = bw.Model.random(big, seed=1, dtype="bfloat16", sigma=0.02, on_device=True)
            m = measure_decode(bw, torch, model8, big, "bfloat16", 8, side_steps, 4)
            points8, rooflines8 = {}, {}
            for name, b, ctx in (("decode_b1", 1, CONTEXT), ("decode_b64", 64, CONTEXT), ("decode_b8_ctx8192", 8, 8192)):
                mp = measure_decode(bw, torch, model8, big, "bfloat16", b, side_steps, 4, context=ctx)
                points8[name] = mp["tok_s"]
                rooflines8[name] = mp["roofline"]["frac"]
            extra["llama3_8b"] = {"layers": big["num_hidden_layers"], "hidden": big["hidden_size"], "heads": 32, "kv_heads": 8,
                                  "head_dim": 128, "ffn": big["intermediate_size"], "vocab": big["vocab_size"],
                                  "decode_tok_s": m["tok_s"], "batch": 8, "ms_per_step": m["ms_per_step"],
                                  "roofline": m["roofline"], "points": points8, "point_roofline_fracs": rooflines8,
                                  "prefill": measure_prefill(bw, torch, model8, big, "bfloat16", PEAK_FLOPS["bf16"]),
                                  "prefill_8192_in_portions": measure_chunked_prefill(bw, torch, model8, big, "bfloat16",
                                                                                      PEAK_FLOPS["bf16"]),
                                  "serving": measure_serving(bw, torch, model8, big, "bfloat16"),
                                  # 128 requests, four shared 1,024-token starts, contexts up to 6,144, a tenth cancelled, a pool
                                  # that forces preemption; 8 of them checked against solo runs
                                  "trace8k": measure_trace(bw, torch, model8, big, "bfloat16", check=8)}
            del model8
            model = None

    value = head["tok_s"]
    # The reference's figure is one stream on a CPU: like for like is this engine's rate at batch 1, where it is measured.
    one_stream = points.get("decode_b1", value if args.batch == 1 else None)
    line = {
        "metric": f"decode tok/s at batch {args.batch}, {shape_name} shape, 2048-token contexts",
        "value": value, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": head["ms_per_step"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": round(value / BASELINE_TOK_S, 1) if args.shape == "smollm2" else None,
        "vs_baseline_one_stream": round(one_stream / BASELINE_TOK_S, 1) if args.shape == "smollm2" and one_stream else None,
        "dtype": args.dtype,
        "data": "synthetic",
        "config": {
            "model": f"{shape_name} shape, random weights", "layers": cfg["num_hidden_layers"],
            "layers_full": full_layers, "hidden": cfg["hidden_size"], "heads": cfg["num_attention_heads"],
            "kv_heads": cfg["num_key_value_heads"], "head_dim": cfg["head_dim"], "ffn": cfg["intermediate_size"],
            "vocab": vocab, "tied": bool(cfg["tie_word_embeddings"]), "global_batch": args.batch, "seq_len": CONTEXT, "max_context": 4096,
            "page_size": 16, "parallelism": "single GPU", "weights": "bf16" if args.dtype == "bf16" else "bf16 widened",
            "baseline": f"reference CPU decode, one stream, 7.26 tok/s (vs_baseline: batch {args.batch} over it)",
        },
        "prefill": prefill,
        "roofline": head["roofline"],
        "points": points,
        "point_rooflines": point_rooflines,
    }
    line.update(extra)
    line["wall_s"] = round(time.perf_counter() - t_start, 1)
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
