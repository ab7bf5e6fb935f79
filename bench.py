#!/usr/bin/env python3
"""Decode and prefill throughput of the engine on one MI355X, at the SmolLM2-1.7B shape with
random weights and uniform random token ids.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--dtype bf16|fp32] [--batch B] [--layers L]
                    [--prefill-tokens T] [--no-points] [--shape smollm2|llama3_8b]

A step is one decode step of the whole engine (scheduler, graph replay of the model, sampling,
token hand-back) for a batch of B requests that each hold a 2,048-token context.  ``value`` is
decoded tokens per second.  One JSON line is printed; it also carries the 2,048-token prefill,
the decode step's HBM roofline, decode at batch 1 and 64 with their rooflines, the same model's true
32-bit path (decode and prefill) and, at Llama-3-8B's sizes, decode, prefill and a continuous-batching workload
of 64 requests.
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


def make_engine(bw, model, batch: int, steps_total: int, dtype: str, context: int = CONTEXT):
    block = 16
    per_request = context + steps_total + 2 * block
    cfg = bw.EngineConfig(num_blocks=batch * ((per_request + block - 1) // block) + 8, max_batched_tokens=2048,
                          max_num_seqs=max(batch, 1), prefix_caching=False, fingerprint_logits=False,
                          block_size=block, dtype=dtype, max_model_len=max(4096, context + 1024))
    return bw.Engine(model, None, cfg)


def fill(engine, bw, torch, batch: int, vocab: int, new_tokens: int, seed: int, context: int = CONTEXT):
    """Admit ``batch`` requests with ``context`` random tokens each and run their prompts."""
    g = torch.Generator().manual_seed(seed)
    for _ in range(batch):
        prompt = torch.randint(0, vocab, (context,), generator=g).tolist()
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


LLAMA3_8B = {
    # Llama-3-8B's sizes (BASELINE.json configs[3]): 32 layers, width 4096, 32 heads on 8 kv heads of 128,
    # feed-forward 14336, vocabulary 128256, rotary base 500000 without scaling, eps 1e-5, untied head.
    "architectures": ["LlamaForCausalLM"], "model_type": "llama", "hidden_act": "silu",
    "vocab_size": 128256, "hidden_size": 4096, "num_hidden_layers": 32, "num_attention_heads": 32,
    "num_key_value_heads": 8, "head_dim": 128, "intermediate_size": 14336, "rope_theta": 500000.0,
    "rms_norm_eps": 1e-5, "tie_word_embeddings": False, "max_position_embeddings": 8192,
    "bos_token_id": 1, "eos_token_id": 2,
}


def measure_prefill(bw, torch, model, cfg: dict, dtype: str, peak_flops: float, tokens: int = PREFILL_TOKENS) -> dict:
    """One prompt of ``tokens`` tokens (2,048 unless said otherwise) in one step (model, head for the last row,
    sampling); the best of six after two untimed ones (the shader clock takes some milliseconds of load to rise
    from its idle 2.1 GHz to 2.4)."""
    engine = make_engine(bw, model, 1, 8, dtype)
    g = torch.Generator().manual_seed(99)
    times = []
    for _ in range(8):
        prompt = torch.randint(0, cfg["vocab_size"], (tokens,), generator=g).tolist()
        engine.add_request(prompt, bw.SamplingParams(max_new_tokens=1, ignore_eos=True))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        engine.step()
        torch.cuda.synchronize()
        times.append((time.perf_counter() - t0) * 1e3)
        assert engine.idle()
    ms = min(times[2:])
    flops = prefill_flops(cfg, tokens)
    return {"value": round(tokens / ms * 1e3, 1), "tokens": tokens, "ms": round(ms, 3),
            "frac": round(flops / (ms * 1e-3) / peak_flops, 4)}


def measure_decode(bw, torch, model, cfg: dict, dtype: str, batch: int, steps: int, warmup: int,
                   context: int = CONTEXT) -> dict:
    """``steps`` decode steps of ``batch`` requests that each hold a context of ``context`` tokens (2,048 unless
    said otherwise): tokens a second, and the bytes a step has to read (every weight once, the cache of the live
    requests) over its time."""
    torch.cuda.empty_cache()
    # Requests admitted early decode while the later ones are still being prefilled (2,048 prompt
    # tokens a step): every request gets enough new tokens to outlast the prefills, the warm-up and the
    # timed steps, so that each timed step has all ``batch`` rows.
    chunks = (context + 2047) // 2048                  # steps a prompt takes under the 2,048-token budget
    new_tokens = steps + warmup + batch * chunks + 8
    eng = make_engine(bw, model, batch, new_tokens, dtype, context)
    fill(eng, bw, torch, batch, cfg["vocab_size"], new_tokens, seed=batch, context=context)
    assert len(eng.sched.running) == batch
    secs = time_decode(eng, torch, steps, warmup)
    assert len(eng.sched.running) == batch, "a request finished inside the timed steps"
    kv_token = eng.exec.storage.bytes_per_token()
    del eng
    ms = secs / steps * 1e3
    # keys a decoded token reads, on average: the prompt, what the request decoded while later
    # prompts were prefilled, the warm-up, and half the timed steps
    avg_ctx = context + chunks * (batch - 1) / 2 + warmup + (steps + 1) / 2
    step_bytes = model.weight_bytes + batch * avg_ctx * kv_token
    achieved = step_bytes / (ms * 1e-3) / 1e9
    return {"tok_s": round(batch * steps / secs, 1), "ms_per_step": round(ms, 4),
            "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                         "frac": round(achieved / PEAK_HBM_GBS, 4)}}


def measure_serving(bw, torch, model, cfg: dict, dtype: str, requests: int = 64, seed: int = 5) -> dict:
    """The continuous-batching workload of the reference's load generator (bench/loadgen.py:170-207) with synthetic
    tokens: ``requests`` requests at once, prompt lengths uniform in [128, 2048], generation lengths uniform in
    [64, 512], greedy, prompts cut into portions under a budget of 2,048 tokens a step, decoded beside each other."""
    import random
    rng = random.Random(seed)
    g = torch.Generator().manual_seed(seed)
    work = []
    for _ in range(requests):
        n, new = rng.randint(128, 2048), rng.randint(64, 512)
        work.append((torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist(), new))
    block = 16
    pages = sum((len(p) + new + 2 * block) // block + 1 for p, new in work)
    ecfg = bw.EngineConfig(num_blocks=pages, max_batched_tokens=2048, max_num_seqs=requests, prefix_caching=False,
                           fingerprint_logits=False, block_size=block, dtype=dtype, max_model_len=4096)
    eng = bw.Engine(model, None, ecfg)
    for p, new in work:
        eng.add_request(p, bw.SamplingParams(max_new_tokens=new, ignore_eos=True))
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    steps = 0
    while not eng.idle():
        eng.step()
        steps += 1
    torch.cuda.synchronize()
    secs = time.perf_counter() - t0
    generated = eng.stats.generated_tokens
    prompt_tokens = sum(len(p) for p, _ in work)
    assert generated == sum(new for _, new in work)
    return {"requests": requests, "prompt_tokens": prompt_tokens, "generated_tokens": generated, "steps": steps,
            "seconds": round(secs, 3), "generated_tok_s": round(generated / secs, 1),
            "all_tok_s": round((generated + prompt_tokens) / secs, 1), "preemptions": eng.stats.preemptions}


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
    ap.add_argument("--no-points", action="store_true",
                    help="only the headline: skip decode at batch 1 and 64, the 32-bit path and the Llama-3-8B sizes")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported (use --gpus 1)")
        return 2

    import torch
    import bitwise_amd as bw

    dtype = "bfloat16" if args.dtype == "bf16" else "float32"
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
    head = measure_decode(bw, torch, model, cfg, dtype, args.batch, args.steps, args.warmup)
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
                             "roofline": m["roofline"],
                             "prefill": measure_prefill(bw, torch, model32, cfg, "float32", PEAK_FLOPS["fp32"])}
            del model32
            torch.cuda.empty_cache()
            # Llama-3-8B's sizes, all 32 layers, bfloat16: decode at batch 8 with 2,048-token contexts, one prefill
            big = dict(LLAMA3_8B)
            model8 = bw.Model.random(big, seed=1, dtype="bfloat16", sigma=0.02, on_device=True)
            m = measure_decode(bw, torch, model8, big, "bfloat16", 8, side_steps, 4)
            extra["llama3_8b"] = {"layers": big["num_hidden_layers"], "hidden": big["hidden_size"], "heads": 32, "kv_heads": 8,
                                  "head_dim": 128, "ffn": big["intermediate_size"], "vocab": big["vocab_size"],
                                  "decode_tok_s": m["tok_s"], "batch": 8, "ms_per_step": m["ms_per_step"],
                                  "roofline": m["roofline"],
                                  "prefill": measure_prefill(bw, torch, model8, big, "bfloat16", PEAK_FLOPS["bf16"]),
                                  "serving": measure_serving(bw, torch, model8, big, "bfloat16")}
            del model8
            model = None

    value = head["tok_s"]
    line = {
        "metric": f"decode tok/s at batch {args.batch}, {shape_name} shape, 2048-token contexts",
        "value": value, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": head["ms_per_step"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": round(value / BASELINE_TOK_S, 1) if args.shape == "smollm2" else None, "dtype": args.dtype,
        "data": "synthetic",
        "config": {
            "model": f"{shape_name} shape, random weights", "layers": cfg["num_hidden_layers"],
            "layers_full": full_layers, "hidden": cfg["hidden_size"], "heads": cfg["num_attention_heads"],
            "kv_heads": cfg["num_key_value_heads"], "head_dim": cfg["head_dim"], "ffn": cfg["intermediate_size"],
            "vocab": vocab, "tied": bool(cfg["tie_word_embeddings"]), "global_batch": args.batch, "seq_len": CONTEXT, "max_context": 4096,
            "page_size": 16, "parallelism": "single GPU", "weights": "bf16" if args.dtype == "bf16" else "bf16 widened",
            "baseline": "reference CPU decode, one stream, 7.26 tok/s",
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
