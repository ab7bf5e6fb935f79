#!/usr/bin/env python3
"""Decode and prefill throughput of the engine on one MI355X, at the SmolLM2-1.7B shape with
random weights and uniform random token ids.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--dtype bf16|fp32] [--batch B] [--layers L]

A step is one decode step of the whole engine (scheduler, graph replay of the model, sampling,
token hand-back) for a batch of B requests that each hold a 2,048-token context.  ``value`` is
decoded tokens per second.  One JSON line is printed; it also carries the 2,048-token prefill,
the decode step's HBM roofline and decode at batch 1 and 64.
"""

from __future__ import annotations

import argparse
import json
import sys
import time

# Layer sizes of the SmolLM2-1.7B shape: 24 layers, width 2048, 32 heads on 32 kv heads of size
# 64, feed-forward 8192, vocabulary 49152, rotary base 130000, eps 1e-5, tied embeddings.
SMOLLM2_1_7B = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama", "hidden_act": "silu",
    "vocab_size": 49152, "hidden_size": 2048, "num_hidden_layers": 24, "num_attention_heads": 32,
    "num_key_value_heads": 32, "head_dim": 64, "intermediate_size": 8192, "rope_theta": 130000.0,
    "rms_norm_eps": 1e-5, "tie_word_embeddings": True, "max_position_embeddings": 4096,
    "bos_token_id": 1, "eos_token_id": 2,
}
CONTEXT = 2048                      # tokens each request holds when decoding starts
PREFILL_TOKENS = 2048
BASELINE_TOK_S = 7.26               # the reference's published SmolLM2-1.7B decode rate (one stream, 4-core CPU)
PEAK_HBM_GBS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}


def prefill_flops(cfg: dict, tokens: int) -> float:
    h, inter, v = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    qd = cfg["num_attention_heads"] * cfg["head_dim"]
    kvd = cfg["num_key_value_heads"] * cfg["head_dim"]
    per_token = 2 * (h * (qd + 2 * kvd) + qd * h + 2 * h * inter + inter * h)
    attn = 2 * 2 * cfg["num_attention_heads"] * cfg["head_dim"] * tokens * (tokens + 1) / 2
    return cfg["num_hidden_layers"] * (per_token * tokens + attn) + 2 * h * v      # the head runs for one row


def make_engine(bw, model, batch: int, steps_total: int, dtype: str):
    block = 16
    per_request = CONTEXT + steps_total + 2 * block
    cfg = bw.EngineConfig(num_blocks=batch * ((per_request + block - 1) // block) + 8, max_batched_tokens=2048,
                          max_num_seqs=max(batch, 1), prefix_caching=False, fingerprint_logits=False,
                          block_size=block, dtype=dtype, max_model_len=4096)
    return bw.Engine(model, None, cfg)


def fill(engine, bw, torch, batch: int, vocab: int, new_tokens: int, seed: int):
    """Admit ``batch`` requests with CONTEXT random tokens each and run their prompts."""
    g = torch.Generator().manual_seed(seed)
    for _ in range(batch):
        prompt = torch.randint(0, vocab, (CONTEXT,), generator=g).tolist()
        engine.add_request(prompt, bw.SamplingParams(temperature=0.0, max_new_tokens=new_tokens, ignore_eos=True))
    while engine.num_waiting or any(s.computed < s.prompt_len for s in engine.sched.running):
        engine.step()


def time_decode(engine, torch, steps: int, warmup: int):
    for _ in range(warmup):
        engine.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        engine.step()
    torch.cuda.synchronize()
    return time.perf_counter() - t0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--dtype", choices=["bf16", "fp32"], default="bf16")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=0, help="run fewer layers than the shape has (named in config)")
    ap.add_argument("--no-points", action="store_true", help="skip the batch-1 and batch-64 decode points")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported (use --gpus 1)")
        return 2

    import torch
    import bitwise_amd as bw

    dtype = "bfloat16" if args.dtype == "bf16" else "float32"
    cfg = dict(SMOLLM2_1_7B)
    full_layers = cfg["num_hidden_layers"]
    if args.layers:
        cfg["num_hidden_layers"] = args.layers
    t_start = time.perf_counter()
    model = bw.Model.random(cfg, seed=0, dtype=dtype, sigma=0.02, on_device=True)
    vocab = cfg["vocab_size"]
    total = args.steps + args.warmup

    # ---- prefill of one 2,048-token prompt (one step: model, head for the last row, sampling)
    engine = make_engine(bw, model, 1, 8, dtype)
    g = torch.Generator().manual_seed(99)
    prefill_ms = []
    for rep in range(3):
        prompt = torch.randint(0, vocab, (PREFILL_TOKENS,), generator=g).tolist()
        engine.add_request(prompt, bw.SamplingParams(max_new_tokens=1, ignore_eos=True))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        engine.step()
        torch.cuda.synchronize()
        prefill_ms.append((time.perf_counter() - t0) * 1e3)
        assert engine.idle()
    pf_ms = min(prefill_ms[1:])
    flops = prefill_flops(cfg, PREFILL_TOKENS)
    prefill = {"value": round(PREFILL_TOKENS / pf_ms * 1e3, 1), "tokens": PREFILL_TOKENS, "ms": round(pf_ms, 3),
               "frac": round(flops / (pf_ms * 1e-3) / PEAK_FLOPS[args.dtype], 4)}
    del engine

    def decode_point(batch: int, steps: int, warmup: int):
        torch.cuda.empty_cache()
        # Requests admitted early decode while the later ones are still being prefilled (one prompt a
        # step): every request gets enough new tokens to outlast the prefills, the warm-up and the
        # timed steps, so that each timed step has all ``batch`` rows.
        new_tokens = steps + warmup + batch + 8
        eng = make_engine(bw, model, batch, new_tokens, dtype)
        fill(eng, bw, torch, batch, vocab, new_tokens, seed=batch)
        assert len(eng.sched.running) == batch
        secs = time_decode(eng, torch, steps, warmup)
        assert len(eng.sched.running) == batch, "a request finished inside the timed steps"
        kv_token = eng.exec.storage.bytes_per_token()
        del eng
        return secs, kv_token

    secs, kv_token = decode_point(args.batch, args.steps, args.warmup)
    ms_step = secs / args.steps * 1e3
    value = args.batch * args.steps / secs
    # keys a decoded token reads, on average: the prompt, what the request decoded while later
    # prompts were prefilled, the warm-up, and half the timed steps
    avg_ctx = CONTEXT + (args.batch - 1) / 2 + args.warmup + (args.steps + 1) / 2
    step_bytes = model.weight_bytes + args.batch * avg_ctx * kv_token
    achieved = step_bytes / (ms_step * 1e-3) / 1e9
    points = {}
    if not args.no_points:
        for b in (1, 64):
            s, _ = decode_point(b, max(16, args.steps // 2), 4)
            points[f"decode_b{b}"] = round(b * max(16, args.steps // 2) / s, 1)

    line = {
        "metric": "decode tok/s at batch 8, SmolLM2-1.7B shape, 2048-token contexts",
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": round(value / BASELINE_TOK_S, 1), "dtype": args.dtype, "data": "synthetic",
        "config": {
            "model": "SmolLM2-1.7B shape, random weights", "layers": cfg["num_hidden_layers"],
            "layers_full": full_layers, "hidden": cfg["hidden_size"], "heads": cfg["num_attention_heads"],
            "kv_heads": cfg["num_key_value_heads"], "head_dim": cfg["head_dim"], "ffn": cfg["intermediate_size"],
            "vocab": vocab, "tied": True, "global_batch": args.batch, "seq_len": CONTEXT, "max_context": 4096,
            "page_size": 16, "parallelism": "single GPU", "weights": "bf16" if args.dtype == "bf16" else "bf16 widened",
            "baseline": "reference CPU decode, one stream, 7.26 tok/s",
        },
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM_GBS, 4)},
        "points": points,
        "wall_s": round(time.perf_counter() - t_start, 1),
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
