"""Measuring the engine: decode steps, prefills and serving workloads with seeded synthetic tokens, each with
the bytes or flops it has to move against the MI355X's published peaks (HBM 8 TB/s; dense matrix peaks 2.5 PFLOP/s
in bfloat16 and 157.3 TFLOP/s in 32-bit).  ``bench.py`` and ``python -m bitwise_amd bench`` both call these."""

from __future__ import annotations

import time

CONTEXT = 2048                      # tokens each request holds when decoding starts
PREFILL_TOKENS = 2048
PEAK_HBM_GBS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12, "bfloat16": 2.5e15, "float32": 157.3e12}


def prefill_flops(cfg: dict, tokens: int) -> float:
    h, inter, v = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    qd = cfg["num_attention_heads"] * cfg["head_dim"]
    kvd = cfg["num_key_value_heads"] * cfg["head_dim"]
    per_token = 2 * (h * (qd + 2 * kvd) + qd * h + 2 * h * inter + inter * h)
    attn = 2 * 2 * cfg["num_attention_heads"] * cfg["head_dim"] * tokens * (tokens + 1) / 2
    return cfg["num_hidden_layers"] * (per_token * tokens + attn) + 2 * h * v      # the head runs for one row


def make_engine(bw, model, batch: int, steps_total: int, dtype: str, context: int = CONTEXT, decode_phases: bool = False,
                portion_align: int = 64):
    block = 16
    per_request = context + steps_total + 2 * block
    cfg = bw.EngineConfig(num_blocks=batch * ((per_request + block - 1) // block) + 8, max_batched_tokens=2048,
                          max_num_seqs=max(batch, 1), prefix_caching=False, fingerprint_logits=False,
                          block_size=block, dtype=dtype, max_model_len=max(4096, context + 1024),
                          decode_phases=decode_phases, portion_align=portion_align)
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




def measure_prefill(bw, torch, model, cfg: dict, dtype: str, peak_flops: float, tokens: int = PREFILL_TOKENS) -> dict:
    """One prompt of ``tokens`` tokens (2,048 unless said otherwise) in one step (model, head for the last row,
    sampling): the median of six after two untimed ones (the shader clock takes some milliseconds of load to rise
    from its idle 2.1 GHz to 2.4); the best of the six is given beside it."""
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
    timed = sorted(times[2:])
    ms, best = (timed[2] + timed[3]) / 2, timed[0]
    flops = prefill_flops(cfg, tokens)
    return {"value": round(tokens / ms * 1e3, 1), "tokens": tokens, "ms": round(ms, 3),
            "frac": round(flops / (ms * 1e-3) / peak_flops, 4), "ms_best": round(best, 3),
            "ms_mean": round(sum(timed) / len(timed), 3), "runs": len(timed)}


def measure_chunked_prefill(bw, torch, model, cfg: dict, dtype: str, peak_flops: float, tokens: int = 8192,
                            budget: int = 2048) -> dict:
    """One prompt of ``tokens`` tokens cut into portions under a budget of ``budget`` tokens a step, each portion
    against the cache the earlier ones left: the median of three after an untimed one."""
    block = 16
    ecfg = bw.EngineConfig(num_blocks=(tokens + 4 * block) // block + 8, max_batched_tokens=budget, max_num_seqs=1,
                           prefix_caching=False, fingerprint_logits=False, block_size=block, dtype=dtype,
                           max_model_len=tokens + 1024)
    engine = bw.Engine(model, None, ecfg)
    g = torch.Generator().manual_seed(98)
    times, steps = [], 0
    for _ in range(4):
        prompt = torch.randint(0, cfg["vocab_size"], (tokens,), generator=g).tolist()
        engine.add_request(prompt, bw.SamplingParams(max_new_tokens=1, ignore_eos=True))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        steps = 0
        while not engine.idle():
            engine.step()
            steps += 1
        torch.cuda.synchronize()
        times.append((time.perf_counter() - t0) * 1e3)
    timed = sorted(times[1:])
    ms = timed[1]
    return {"value": round(tokens / ms * 1e3, 1), "tokens": tokens, "budget": budget, "steps": steps, "ms": round(ms, 3),
            "frac": round(prefill_flops(cfg, tokens) / (ms * 1e-3) / peak_flops, 4), "ms_best": round(timed[0], 3),
            "ms_mean": round(sum(timed) / len(timed), 3), "runs": len(timed)}


def measure_prefill_beside_decodes(bw, torch, model, cfg: dict, dtype: str, tokens: int = 8192, decoders: int = 7,
                                   portion_align: int = 64) -> dict:
    """One prompt of ``tokens`` tokens arriving while ``decoders`` requests decode (512-token contexts): every step
    holds the decoders' single tokens and a portion of the prompt under a budget of 2,048 tokens.  The time from the
    prompt's arrival to its first token: the median of three after an untimed one."""
    block = 16
    ecfg = bw.EngineConfig(num_blocks=(tokens + decoders * 1024) // block + 16, max_batched_tokens=2048,
                           max_num_seqs=decoders + 1, prefix_caching=False, fingerprint_logits=False, block_size=block,
                           dtype=dtype, max_model_len=tokens + 1024, portion_align=portion_align)
    engine = bw.Engine(model, None, ecfg)
    g = torch.Generator().manual_seed(97)
    for _ in range(decoders):
        prompt = torch.randint(0, cfg["vocab_size"], (512,), generator=g).tolist()
        engine.add_request(prompt, bw.SamplingParams(max_new_tokens=400, ignore_eos=True))
    while engine.num_waiting or any(s.computed < s.prompt_len for s in engine.sched.running):
        engine.step()
    times, steps = [], 0
    for _ in range(4):
        prompt = torch.randint(0, cfg["vocab_size"], (tokens,), generator=g).tolist()
        rid = engine.add_request(prompt, bw.SamplingParams(max_new_tokens=1, ignore_eos=True))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        steps = 0
        while not engine.result(rid).finished:
            engine.step()
            steps += 1
        torch.cuda.synchronize()
        times.append((time.perf_counter() - t0) * 1e3)
    assert len(engine.sched.running) == decoders, "a decoding request finished inside the measurement"
    timed = sorted(times[1:])
    return {"tokens": tokens, "decoders": decoders, "portion_align": portion_align, "steps": steps, "ms": round(timed[1], 3),
            "ms_best": round(timed[0], 3), "prompt_tok_s": round(tokens / timed[1] * 1e3, 1)}


def measure_qkv_row_orders(torch, cfg: dict, calls: int = 30) -> dict:
    """The q|k|v product with rotation and cache write in its epilogue, called alone on about 2,048 rows composed in
    different ways (one request; portions of two requests and decoded tokens of others, behind or in front): microseconds
    a call.  Heads of 64 only (other sizes rotate in a kernel of their own)."""
    from bitwise_amd.csrc import ops
    dev = torch.device("cuda:0")
    heads, kvh, hd, K, ps = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"], cfg["hidden_size"], 16
    if hd != 64:
        return {}
    N, pool = (heads + 2 * kvh) * hd, 1100
    g = torch.Generator().manual_seed(1)
    w = (torch.randn(N, K, generator=g) * 0.02).bfloat16().to(dev)
    kc = torch.zeros(pool, kvh, ps, hd, dtype=torch.bfloat16, device=dev)
    vc = torch.zeros(pool, kvh, hd, ps, dtype=torch.bfloat16, device=dev)
    ang = torch.arange(4096, dtype=torch.float64)[:, None] * (cfg["rope_theta"] ** (-torch.arange(0, hd, 2, dtype=torch.float64) / hd))[None, :]
    cos, sin = ang.cos().float().to(dev), ang.sin().float().to(dev)
    out = {}

    def case(name, segs):                       # segs: (request, first position, rows)
        M = sum(n for _, _, n in segs)
        nseq = max(s for s, _, _ in segs) + 1
        pos = torch.cat([torch.arange(p0, p0 + n, dtype=torch.int32) for _, p0, n in segs]).to(dev)
        rs = torch.cat([torch.full((n,), s, dtype=torch.int32) for s, _, n in segs]).to(dev)
        table = torch.zeros(nseq, 264, dtype=torch.int32)
        for s in range(nseq):
            table[s, :130] = torch.arange(130 * s, 130 * s + 130, dtype=torch.int32)
        table = table.to(dev)
        x = torch.randn(M, K, generator=g).bfloat16().to(dev)
        q = torch.zeros(M, heads * hd, dtype=torch.bfloat16, device=dev)
        for i in range(calls + 5):
            if i == 5:
                torch.cuda.synchronize()
                t0 = time.perf_counter()
            ops.gemm_qkv_rope_bf16(x, w, q, pos, rs, table, cos, sin, kc, vc, M, heads, kvh, hd, ps)
        torch.cuda.synchronize()
        out[name] = round((time.perf_counter() - t0) / calls * 1e6, 1)

    decoded = [(2 + i, 2048, 1) for i in range(5)]
    case("one request, positions 0..2047", [(0, 0, 2048)])
    case("64 rows of one request, 1920 of another, 5 decoded tokens", [(0, 1984, 64), (1, 0, 1920)] + decoded)
    case("the 5 decoded tokens in front", decoded + [(0, 1984, 64), (1, 0, 1920)])
    case("1 decoded token in front of 2047 rows of a request", [(1, 2048, 1), (0, 0, 2047)])
    case("2047 rows of a request, then 1 decoded token", [(0, 0, 2047), (1, 2048, 1)])
    return out


def measure_decode(bw, torch, model, cfg: dict, dtype: str, batch: int, steps: int, warmup: int,
                   context: int = CONTEXT, decode_phases: bool = False, portion_align: int = 64) -> dict:
    """``steps`` decode steps of ``batch`` requests that each hold a context of ``context`` tokens (2,048 unless
    said otherwise): tokens a second, and the bytes a step has to read (every weight once, the cache of the live
    requests) over its time."""
    torch.cuda.empty_cache()
    # Requests admitted early decode while the later ones are still being prefilled (2,048 prompt
    # tokens a step): every request gets enough new tokens to outlast the prefills, the warm-up and the
    # timed steps, so that each timed step has all ``batch`` rows.
    # (a step of the fill holds at least 2,048 tokens less the decoded ones and less what a cut gives up to end on
    # a whole block)
    fill_steps = -(-batch * context // (2048 - batch - 64)) + 1
    new_tokens = steps + warmup + fill_steps + 8
    eng = make_engine(bw, model, batch, new_tokens, dtype, context, decode_phases, portion_align)
    fill(eng, bw, torch, batch, cfg["vocab_size"], new_tokens, seed=batch, context=context)
    assert len(eng.sched.running) == batch
    secs = time_decode(eng, torch, steps, warmup)
    assert len(eng.sched.running) == batch, "a request finished inside the timed steps"
    kv_token = eng.exec.storage.bytes_per_token()
    del eng
    ms = secs / steps * 1e3
    # keys a decoded token reads, on average: the prompt, what the request decoded while later
    # prompts were prefilled, the warm-up, and half the timed steps
    avg_ctx = context + batch * context / 2048 * (batch - 1) / (2 * batch) + warmup + (steps + 1) / 2
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




def shared_prefix_trace(vocab: int, requests: int, seed: int, prefixes: int = 4, prefix_tokens: int = 1024,
                        suffix=(16, 4096), outputs=(32, 1024), rate: float = 40.0, cancel_share: float = 0.1):
    """The randomized trace of the hardest workload the reference's simulator and load generator describe
    (sim/simulate.cpp:120-210, bench/loadgen.py:170-207) at serving sizes, with synthetic tokens: ``requests``
    requests with exponential gaps between their arrivals (``rate`` a second); every prompt is one of ``prefixes``
    shared starts of ``prefix_tokens`` tokens and a suffix of its own, uniform in ``suffix``; new tokens uniform in
    ``outputs``; greedy or temperature 0.7 with a seed of its own; a share of them is given up by the client some
    time after it arrived.  Returns a list of dicts: prompt, params (temperature, seed, max_new_tokens), at (seconds),
    cancel_at (seconds or None)."""
    import random
    rng = random.Random(seed)
    stems = [[rng.randrange(vocab) for _ in range(prefix_tokens)] for _ in range(prefixes)]
    out, t = [], 0.0
    for i in range(requests):
        t += rng.expovariate(rate)
        prompt = list(rng.choice(stems)) + [rng.randrange(vocab) for _ in range(rng.randint(*suffix))]
        out.append({"prompt": prompt, "temperature": 0.0 if rng.random() < 0.5 else 0.7, "seed": rng.getrandbits(48),
                    "max_new_tokens": rng.randint(*outputs), "at": t,
                    "cancel_at": t + rng.uniform(0.0, 3.0) if rng.random() < cancel_share else None})
    return out


def measure_trace(bw, torch, model, cfg: dict, dtype: str, requests: int = 128, seed: int = 7, pool_tokens: int = 96 * 1024,
                  max_num_seqs: int = 64, check: int = 16, trace=None, clock=None) -> dict:
    """Run ``shared_prefix_trace`` through an engine whose page pool (``pool_tokens`` tokens) is smaller than what its
    running requests come to hold, so that some are preempted and recomputed, with the prefix cache on and logits
    fingerprints kept; then run a seeded sample of ``check`` requests that were not cancelled alone (no prefix cache, a
    pool of their own) and compare tokens and fingerprints.  Arrivals and cancellations follow the wall clock (or
    ``clock``, a function of the engine's step count, for a run that does not depend on the machine's speed)."""
    import random
    trace = trace if trace is not None else shared_prefix_trace(cfg["vocab_size"], requests, seed)
    block = 16
    longest = max(len(r["prompt"]) + r["max_new_tokens"] for r in trace)
    ecfg = bw.EngineConfig(num_blocks=pool_tokens // block, max_batched_tokens=2048, max_num_seqs=max_num_seqs, prefix_caching=True,
                           fingerprint_logits=True, block_size=block, dtype=dtype, max_model_len=longest + block)
    eng = bw.Engine(model, None, ecfg)
    params = [bw.SamplingParams(temperature=r["temperature"], seed=r["seed"], max_new_tokens=r["max_new_tokens"], ignore_eos=True)
              for r in trace]
    ids = [None] * len(trace)
    cancelled = set()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    steps, nxt = 0, 0
    while nxt < len(trace) or not eng.idle():
        now = clock(steps) if clock is not None else time.perf_counter() - t0
        while nxt < len(trace) and trace[nxt]["at"] <= now:
            ids[nxt] = eng.add_request(trace[nxt]["prompt"], params[nxt])
            nxt += 1
        for i, r in enumerate(trace[:nxt]):
            if r["cancel_at"] is not None and r["cancel_at"] <= now and i not in cancelled:
                cancelled.add(i)
                eng.cancel(ids[i])
        if eng.idle():
            if clock is None:
                time.sleep(min(0.001, max(0.0, trace[nxt]["at"] - now)))      # nothing to do before the next arrival
            steps += 1
            continue
        eng.step()
        steps += 1
    torch.cuda.synchronize()
    secs = time.perf_counter() - t0
    results = [eng.result(i) for i in ids]
    really_cancelled = [i for i in cancelled if results[i].cancelled]
    done = [i for i in range(len(trace)) if not results[i].cancelled]
    generated = eng.stats.generated_tokens
    stats = eng.stats
    leaked = not eng.manager.all_free()
    del eng
    torch.cuda.empty_cache()
    # a seeded sample of the finished requests, each alone on an engine of its own
    sample = random.Random(seed + 1).sample(done, min(check, len(done)))
    wrong = []
    for i in sample:
        need = len(trace[i]["prompt"]) + trace[i]["max_new_tokens"]
        solo_cfg = bw.EngineConfig(num_blocks=need // block + 2, max_batched_tokens=2048, max_num_seqs=1, prefix_caching=False,
                                   fingerprint_logits=True, block_size=block, dtype=dtype, max_model_len=need + block)
        (ref,) = bw.generate(model, [trace[i]["prompt"]], params[i], solo_cfg)
        if ref.tokens != results[i].tokens or ref.logits_fingerprint != results[i].logits_fingerprint:
            wrong.append(i)
    return {"requests": len(trace), "cancelled": len(really_cancelled), "prompt_tokens": sum(len(r["prompt"]) for r in trace),
            "generated_tokens": generated, "steps": stats.steps, "seconds": round(secs, 3),
            "generated_tok_s": round(generated / secs, 1), "preemptions": stats.preemptions,
            "prefix_hit_tokens": stats.prefix_hit_tokens, "evictions": stats.evictions, "pool_tokens": pool_tokens,
            "checked_against_solo": len(sample), "differ_from_solo": len(wrong), "pages_lost": bool(leaked),
            "longest_request": longest}
