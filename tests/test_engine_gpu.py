"""The engine on the GPU: greedy and sampled generation through the entry point against the
plain implementation, crowded batches against solo runs to the last bit, long decoding, and
randomized scheduling traces (the reference's engine test and simulator,
tests/test_main.cpp:241-302, sim/simulate.cpp)."""

import json
import os
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

import bitwise_amd as bw
import plain_llama as pl
import tiny
from bitwise_amd.sim import Simulator

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parents[1]


@pytest.fixture(scope="module")
def folders(tmp_path_factory, gpu):
    tmp = tmp_path_factory.mktemp("models")
    return {n: tiny.make_folder(tmp, n) for n in ("A", "B")}


def engine_config(name, dtype, **kw):
    base = dict(num_blocks=64, block_size=tiny.CONFIGS[name][3], dtype=dtype)
    base.update(kw)
    return bw.EngineConfig(**base)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_generation_equals_plain(folders, name, dtype):
    """Greedy and temperature sampling through bw.generate: the tokens of the plain
    implementation, which recomputes the whole sequence for every token."""
    cfg, w = tiny.read_config(folders[name]), tiny.read_weights(folders[name])
    model = bw.Model.load(folders[name], dtype)
    g = torch.Generator().manual_seed(4)
    prompts = [torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist() for n in (1, 7, 19, 33)]
    params = [bw.SamplingParams(max_new_tokens=16, ignore_eos=True),
              bw.SamplingParams(max_new_tokens=12, temperature=0.8, seed=5, ignore_eos=True),
              bw.SamplingParams(max_new_tokens=16), bw.SamplingParams(max_new_tokens=10, temperature=1.3, seed=9)]
    results = bw.generate(model, prompts, params, engine_config(name, dtype, max_batched_tokens=24))
    for p, sp, r in zip(prompts, params, results):
        want = pl.generate(cfg, w, p, sp.max_new_tokens, sp.temperature, sp.seed, sp.ignore_eos, **tiny.plain_mode(dtype))
        assert r.tokens == want and r.finished
    assert model.config.num_key_value_heads == cfg["num_key_value_heads"] and model.weight_bytes > 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_crowded_engine_equals_solo_to_the_last_bit(folders, dtype):
    """Six requests that share a 24-token prefix, sampled at temperature 0.8 with seeds 0-5, in
    a pool so tight that prefixes are reused and at least one request is preempted and
    recomputed: tokens and logits fingerprints equal each request run alone."""
    name = "B"
    cfg = tiny.read_config(folders[name])
    model = bw.Model.load(folders[name], dtype)
    g = torch.Generator().manual_seed(6)
    shared = torch.randint(0, 500, (24,), generator=g).tolist()
    prompts = [shared + torch.randint(0, 500, (n,), generator=g).tolist() for n in (0, 8, 16, 24, 32, 40)]
    params = [bw.SamplingParams(temperature=0.8, seed=s, max_new_tokens=20, ignore_eos=True) for s in range(6)]
    solo = []
    for p, sp in zip(prompts, params):
        (r,) = bw.generate(model, [p], sp, engine_config(name, dtype, prefix_caching=False, max_batched_tokens=256))
        solo.append(r)
    for tight in (dict(num_blocks=14, max_batched_tokens=32), dict(num_blocks=64, max_batched_tokens=24)):
        eng = bw.Engine(model, None, engine_config(name, dtype, **tight))
        ids = [eng.add_request(p, sp) for p, sp in zip(prompts, params)]
        guard = 0
        while not eng.idle():
            eng.step()
            guard += 1
            assert guard < 5000, eng.debug_state()
        for i, ref in zip(ids, solo):
            assert eng.result(i).tokens == ref.tokens
            assert eng.result(i).logits_fingerprint == ref.logits_fingerprint
        assert eng.free_blocks == tight["num_blocks"]
        assert eng.stats.prefix_hit_tokens > 0
        if tight["num_blocks"] == 14:
            assert eng.stats.preemptions > 0


def test_long_decoding_with_and_without_graphs(folders):
    """200 decoded tokens: graph replay and kernel-by-kernel launches give the same tokens and
    fingerprints, and the tokens are those of the plain implementation."""
    name, dtype = "A", "bfloat16"
    cfg, w = tiny.read_config(folders[name]), tiny.read_weights(folders[name])
    cfg_long = dict(cfg, max_position_embeddings=256)
    folder = folders[name].parent / "tiny_A_long"
    bw.write_random_model(folder, cfg_long, 0, 0.02)
    model = bw.Model.load(folder, dtype)
    prompt = [3, 14, 15, 92, 65]
    sp = bw.SamplingParams(max_new_tokens=100, ignore_eos=True, temperature=0.9, seed=3)
    outs = []
    for graphs in (True, False):
        (r,) = bw.generate(model, [prompt], sp, engine_config(name, dtype, use_graphs=graphs))
        outs.append(r)
    assert outs[0].tokens == outs[1].tokens and outs[0].logits_fingerprint == outs[1].logits_fingerprint
    want = pl.generate(cfg_long, tiny.read_weights(folder), prompt, 100, 0.9, 3, True, **tiny.plain_mode(dtype))
    assert outs[0].tokens == want
    # the same with the decode steps' products as phases of a few launches (what of them can run so at these sizes)
    eng = bw.Engine(model, None, engine_config(name, dtype, decode_phases=True))
    assert eng.exec.runner.chain_rows == 16
    i = eng.add_request(prompt, sp)
    while not eng.idle():
        eng.step()
    assert eng.result(i).tokens == want and eng.result(i).logits_fingerprint == outs[0].logits_fingerprint


def test_many_requests_decode_from_the_large_graph_buckets(gpu):
    """100 and then 200 requests decoding at once (the graph buckets of 128 and 256 rows, where the residual adds
    take their layouts for 65 rows and more inside a captured graph) at SmolLM2's layer widths, one layer: every
    request's tokens and fingerprint are those of the same request run alone, with graphs and without."""
    cfg = {"architectures": ["LlamaForCausalLM"], "model_type": "llama", "hidden_act": "silu", "num_hidden_layers": 1,
           "rms_norm_eps": 1e-5, "max_position_embeddings": 256, "bos_token_id": 1, "eos_token_id": 2,
           "vocab_size": 1000, "hidden_size": 2048, "num_attention_heads": 32, "num_key_value_heads": 32, "head_dim": 64,
           "intermediate_size": 8192, "rope_theta": 130000.0, "tie_word_embeddings": True}
    model = bw.Model.random(cfg, seed=5, dtype="bfloat16", sigma=0.05, on_device=True)
    g = torch.Generator().manual_seed(2)
    prompts = [torch.randint(0, 1000, (int(n),), generator=g).tolist() for n in torch.randint(3, 20, (200,), generator=g)]
    sp = [bw.SamplingParams(max_new_tokens=6, ignore_eos=True, temperature=0.8 if i % 3 else 0.0, seed=i) for i in range(200)]

    replayed = []

    def run(which, graphs, seqs):
        ecfg = bw.EngineConfig(num_blocks=seqs * 4 + 8, max_batched_tokens=2048, max_num_seqs=seqs, prefix_caching=False,
                               block_size=16, dtype="bfloat16", max_model_len=256, use_graphs=graphs)
        eng = bw.Engine(model, None, ecfg)
        ids = [eng.add_request(prompts[i], sp[i]) for i in which]
        most = 0
        while not eng.idle():
            eng.step()
            most = max(most, eng.exec.runner.last_graph_rows)
        replayed.append((seqs, graphs, most))
        return [eng.result(i) for i in ids]

    solo = {i: run([i], False, 1)[0] for i in (0, 1, 57, 99, 100, 199)}
    for count in (100, 200):
        for graphs in (True, False):
            outs = run(range(count), graphs, count)
            assert all(len(o.tokens) == 6 for o in outs)
            for i, want in solo.items():
                if i < count:
                    assert outs[i].tokens == want.tokens and outs[i].logits_fingerprint == want.logits_fingerprint, (count, graphs, i)
    assert (100, True, 100) in replayed and (200, True, 200) in replayed and (200, False, 0) in replayed, replayed


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_randomized_scenarios(gpu, dtype):
    """The scenario simulator on the real engine: page sizes, graphs, steps launched ahead, model lengths, pools
    and budgets drawn per scenario, every request against its solo run with pages of 16 and none of that: no
    wrong token, no other logits, no hang, no page lost; and the scenarios reach preemption, prefix hits,
    requests that end at an end-of-sequence token and cancellations."""
    from bitwise_amd.registry import ARCHITECTURES

    model = bw.Model.random(ARCHITECTURES["LlamaForCausalLM"].tiny_config, 42, dtype, sigma=0.08)
    tally = Simulator(model, dtype).run(24, seed=1)
    print(tally.line(dtype))
    assert tally.violations() == 0, "\n".join(tally.notes[:10])
    assert tally.requests_compared > 60 and tally.preemptions > 0 and tally.prefix_hit_tokens > 0
    assert tally.ended_by_eos > 0 and tally.cancelled > 0
    assert len(tally.knobs_seen["block_size"]) >= 3 and tally.knobs_seen["use_graphs"] == {True, False}
    assert tally.knobs_seen["run_ahead"] == {True, False} and tally.knobs_seen["decode_phases"] == {True, False}


def test_the_simulator_program_catches_every_injected_fault(gpu):
    """python -m bitwise_amd sim --sweep-faults on the GPU: the run without a fault is clean, each of the engine's
    test-only bugs is reported, exit status 0; --fault alone exits with 1; an unknown fault with 2
    (sim/simulate.cpp:239-240, :283-300)."""
    import subprocess
    import sys as _sys

    env = dict(os.environ, PYTHONPATH=str(ROOT))
    base = [_sys.executable, "-m", "bitwise_amd", "sim", "--seed", "3"]
    p = subprocess.run(base + ["--traces", "40", "--sweep-faults"], capture_output=True, text=True, env=env, timeout=900)
    print(p.stdout)
    assert p.returncode == 0, p.stdout[-3000:] + p.stderr[-3000:]
    lines = p.stdout.strip().splitlines()
    assert lines[0].startswith("no fault: 40 scenarios") and "wrong tokens 0" in lines[0]
    assert len(lines) == 6 and lines[-1].startswith("caught 4 of 4 injected faults; violations of the run without a fault: 0")
    assert all("first failing scenario" in l for l in lines[1:5])
    p = subprocess.run(base + ["--traces", "40", "--fault", "5"], capture_output=True, text=True, env=env, timeout=600)
    assert p.returncode == 1 and "pages or slots lost 0" not in p.stdout
    p = subprocess.run(base + ["--fault", "3"], capture_output=True, text=True, env=env, timeout=600)
    assert p.returncode == 2 and "speculative" in p.stderr


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_shared_prefix_trace_of_128_requests_at_real_layer_sizes_equals_solo(gpu, dtype):
    """The hardest workload the reference describes (sim/simulate.cpp:120-210 at the sizes of bench/loadgen.py), whole:
    layers of Llama-3-8B's sizes (width 4096, 32 query heads on 8 key heads of 128, feed-forward 14336, the whole
    vocabulary; two layers), 128 requests with exponential gaps between arrivals, four shared 1,024-token starts and
    suffixes of 16 to 4,096 tokens, 32 to 1,024 new tokens, greedy or temperature 0.7, a tenth given up by the client,
    contexts up to 6,144 in a pool of 96k tokens for up to 64 running requests, so that requests are preempted and
    recomputed; in bfloat16 and in 32-bit.  A seeded sample of 16 finished requests (8 in 32-bit) must have the tokens
    and the logits fingerprints of the same requests run alone."""
    from bitwise_amd import measure

    cfg = {"architectures": ["LlamaForCausalLM"], "model_type": "llama", "hidden_act": "silu", "num_hidden_layers": 2,
           "rms_norm_eps": 1e-5, "max_position_embeddings": 8192, "bos_token_id": 1, "eos_token_id": 2,
           "vocab_size": 128256, "hidden_size": 4096, "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 128,
           "intermediate_size": 14336, "rope_theta": 500000.0, "tie_word_embeddings": False}
    model = bw.Model.random(cfg, seed=9, dtype=dtype, sigma=0.02, on_device=True)
    # arrivals and cancellations by the engine's step count (20 ms a step), so that the run is the same on any machine
    check = 16 if dtype == "bfloat16" else 8                  # (solo runs decode one token a step: the slow part)
    out = measure.measure_trace(bw, torch, model, cfg, dtype, requests=128, seed=7, check=check, clock=lambda steps: steps * 0.02)
    print(dtype, out)
    assert out["differ_from_solo"] == 0 and out["checked_against_solo"] == check and not out["pages_lost"]
    assert out["preemptions"] > 0 and out["prefix_hit_tokens"] >= 64 * 1024 and out["cancelled"] >= 5
    assert out["longest_request"] > 5000 and out["requests"] == 128


def test_command_line(folders):
    p = subprocess.run([sys.executable, "-m", "bitwise_amd", "generate", "--model", str(folders["A"]), "--dtype",
                        "float32", "--prompt-tokens", "5,17,3", "--prompt-tokens", "9", "--max-new-tokens", "6",
                        "--ignore-eos"], capture_output=True, text=True, cwd=str(ROOT), timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    lines = [json.loads(l) for l in p.stdout.strip().splitlines()]
    cfg, w = tiny.read_config(folders["A"]), tiny.read_weights(folders["A"])
    assert lines[0]["tokens"] == pl.generate(cfg, w, [5, 17, 3], 6, ignore_eos=True)
    assert lines[1]["tokens"] == pl.generate(cfg, w, [9], 6, ignore_eos=True)
    p = subprocess.run([sys.executable, "-m", "bitwise_amd", "generate", "--nonsense"], capture_output=True, text=True,
                       cwd=str(ROOT), timeout=120)
    assert p.returncode == 2


def test_command_line_random_config_and_bench(folders, tmp_path):
    """--random-config: a config.json run with seeded random weights, the tokens of the same seed's folder; the
    bench subcommand: one JSON line with a decode rate, its roofline and a prefill; both need one model source."""
    cfg_file = tmp_path / "config.json"
    cfg_file.write_text(json.dumps(tiny.TINY_B))
    common = ["--dtype", "bfloat16", "--block-size", "8", "--prompt-tokens", "7,8,9,10", "--max-new-tokens", "5", "--ignore-eos"]
    run = lambda extra: subprocess.run([sys.executable, "-m", "bitwise_amd", "generate", *extra, *common], capture_output=True,
                                       text=True, cwd=str(ROOT), timeout=300)
    a = run(["--random-config", str(cfg_file), "--weights-seed", "1", "--sigma", "0.05"])
    b = run(["--model", str(folders["B"])])                        # tiny B's folder: seed 1, sigma 0.05
    assert a.returncode == 0 and b.returncode == 0, a.stderr[-2000:] + b.stderr[-2000:]
    assert json.loads(a.stdout)["tokens"] == json.loads(b.stdout)["tokens"]
    assert run([]).returncode == 2 and run(["--model", str(folders["B"]), "--random-config", str(cfg_file)]).returncode == 2
    p = subprocess.run([sys.executable, "-m", "bitwise_amd", "bench", "--model", str(tiny.make_folder(tmp_path, "LONG")), "--batch", "3", "--context", "200",
                        "--steps", "8", "--warmup", "2", "--prefill-tokens", "150"], capture_output=True, text=True, cwd=str(ROOT), timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    line = json.loads(p.stdout.strip().splitlines()[-1])
    assert line["decode"]["tok_s"] > 0 and line["decode"]["roofline"]["bound"] == "hbm" and line["prefill"]["tokens"] == 150


def test_model_errors(folders, tmp_path):
    with pytest.raises(bw.ConfigError, match="cannot open"):
        bw.Model.load(tmp_path / "missing")
    model = bw.Model.load(folders["A"], "float32")
    with pytest.raises(ValueError, match="loaded as float32"):
        bw.Engine(model, None, bw.EngineConfig(dtype="bfloat16"))
    eng = bw.Engine(model, None, bw.EngineConfig(dtype="float32", num_blocks=4))
    with pytest.raises(ValueError, match="never fit"):
        eng.add_request(list(range(60)), bw.SamplingParams(max_new_tokens=8))
    with pytest.raises(ValueError, match="model length"):
        bw.Engine(model, None, bw.EngineConfig(dtype="float32", num_blocks=64)).add_request(
            list(range(100)), bw.SamplingParams(max_new_tokens=60))
    bad = dict(tiny.TINY_A, head_dim=24, hidden_size=96)
    with pytest.raises(ValueError, match="head size 24 is not supported"):
        bw.Model.random(bad, 0, "float32")
