"""Trace replay on the GPU: the same requests whole, with the last 32 tokens one by one, in
portions of changing size, and mixed with other requests so that pages are used again, in
32-bit and in bfloat16, each compared with the plain implementation; and the cuttings
compared with each other bit for bit, which is what the reference's own chunking test asks
(tests/test_main.cpp:219-228)."""

import json
import os
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

import plain_llama as pl
import plain_scalar as ps
import tiny

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parents[1]

import replay_util as ru
from replay_util import MAX_TOL as TOL, check_against_plain

# weights that make attention peaked: larger logits, larger effects of one differing rounding (replay_util)
PEAKED_TOL = {"float32": 2e-5, "bfloat16": 3e-2}


def requests_for(cfg, seed, lengths):
    g = torch.Generator().manual_seed(seed)
    return {f"r{i}": torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist() for i, n in enumerate(lengths)}


def plain_logits(folder, toks, dtype):
    cfg, w = tiny.read_config(folder), tiny.read_weights(folder)
    return pl.forward(cfg, w, toks, **tiny.plain_mode(dtype)).numpy()


def replay(folder, dtype, name, steps, max_tokens, **kw):
    """Run steps through a Replayer; returns {request: [len, vocab] logits} (every position wanted), the
    replayer, and {request: the pages it ever held in group 0}."""
    from bitwise_amd.replay import Replayer

    rp = Replayer(str(folder), dtype, max_tokens, block_size=tiny.CONFIGS[name][3], **kw)
    out, held = {}, {}
    for st in steps:
        lg = rp.step(st["entries"])
        row = 0
        for e in st["entries"]:
            for _ in e["want"]:
                out.setdefault(e["id"], []).append(lg[row])
                row += 1
        for rid, rc in rp.live.items():
            held.setdefault(rid, set()).update(p for p in rc.tables[0] if p >= 0)
        rp.step([], st.get("end", []))          # the requests that end here give back what they hold
        rp.manager.check()
    rp.pages_held = held
    return {k: np.stack(v) for k, v in out.items()}, rp


def all_wanted(rid, toks):
    return {"id": rid, "tokens": toks, "want": list(range(len(toks)))}


def cut(toks, sizes):
    out, pos = [], 0
    for s in sizes:
        out.append(toks[pos:pos + s])
        pos += s
    assert pos == len(toks)
    return out


@pytest.fixture(scope="module")
def folders(tmp_path_factory, gpu):
    tmp = tmp_path_factory.mktemp("models")
    return {n: tiny.make_folder(tmp, n) for n in ("A", "B", "LONG")}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_cuttings_equal_plain_and_each_other(folders, name, dtype):
    cfg = tiny.read_config(folders[name])
    lengths = [100, 67, 41, 33, 20]
    reqs = requests_for(cfg, 11, lengths)
    page = tiny.CONFIGS[name][3]
    refs = {rid: plain_logits(folders[name], toks, dtype) for rid, toks in reqs.items()}

    # 1. each request alone and whole
    whole = {}
    for rid, toks in reqs.items():
        got, _ = replay(folders[name], dtype, name, [{"entries": [all_wanted(rid, toks)], "end": [rid]}], 128)
        whole[rid] = got[rid]
        check_against_plain(got[rid], refs[rid], dtype, f"tiny {name} {rid} whole")
        if dtype == "float32":          # and the bits of the plain scalar 32-bit decoder
            want = ps.forward(cfg, tiny.read_weights(folders[name]), toks)
            same = (got[rid].view(np.uint32) == want.view(np.uint32)).all(axis=1)
            assert same.all(), f"{rid}: first position that is not the scalar decoder's bits: {int(np.argmin(same))}"

    # (the same configuration with one layer, where a differing bfloat16 rounding stays at its position: the
    # median over positions is bounded at 32-bit accuracy)
    from bitwise_amd.model import Model, write_random_model
    one = dict(cfg, num_hidden_layers=1)
    folder1 = write_random_model(folders[name].parent / f"one_layer_{name}", one, tiny.CONFIGS[name][1], tiny.CONFIGS[name][2])
    model1 = Model.load(folder1, dtype)
    for rid, toks in reqs.items():
        ref1 = pl.forward(one, tiny.read_weights(folder1), toks, **tiny.plain_mode(dtype)).numpy()
        check_against_plain(model1.logits(toks, block_size=page), ref1, dtype, f"tiny {name} {rid}, one layer", median=True)

    # 2. most of it in one step, the last 32 tokens one by one
    for rid, toks in reqs.items():
        n = len(toks)
        if n <= 32:
            continue
        steps = [{"entries": [all_wanted(rid, toks[:n - 32])]}]
        steps += [{"entries": [{"id": rid, "tokens": [toks[i]], "want": [0]}]} for i in range(n - 32, n)]
        for use_graphs in (True, False):
            got, _ = replay(folders[name], dtype, name, steps, 128, use_graphs=use_graphs)
            assert np.array_equal(got[rid], whole[rid]), f"{rid}: decoding differs from the whole prompt (graphs={use_graphs})"

    # 3. portions of changing size, down to two tokens and one
    sizes = {100: [3, 17, 1, 19, 2, 30, 2, 26], 67: [2, 2, 31, 1, 1, 30], 41: [40, 1], 33: [16, 16, 1], 20: [2, 16, 2]}
    for rid, toks in reqs.items():
        steps = [{"entries": [all_wanted(rid, part)]} for part in cut(toks, sizes[len(toks)])]
        got, _ = replay(folders[name], dtype, name, steps, 128)
        assert np.array_equal(got[rid], whole[rid]), f"{rid}: portions differ from the whole prompt"

    # 4. mixed: up to four live requests, portions of some beside decoded tokens of others, in a pool smaller
    # than what the five requests need together (20 pages of 16, 36 of 8): pages that come back are filled
    # with NaN at once and must serve a later request
    ids = list(reqs)
    plan = {ids[0]: [30, 1, 1, 1, 20, 1, 1, 45], ids[1]: [2, 5, 1, 1, 1, 57], ids[2]: [41], ids[3]: [1, 1, 31],
            ids[4]: [20]}
    order = [[0], [0, 1], [0, 4, 1, 2], [1, 0, 3], [3, 0, 1], [0, 1, 3], [1, 0], [0]]
    steps = []
    cursor = {rid: 0 for rid in ids}
    progress = {rid: 0 for rid in ids}
    for group in order:
        entries, end = [], []
        for i in group:
            rid = ids[i]
            part = plan[rid][cursor[rid]]
            cursor[rid] += 1
            toks = reqs[rid][progress[rid]:progress[rid] + part]
            progress[rid] += part
            entries.append(all_wanted(rid, toks))
            if progress[rid] == len(reqs[rid]):
                end.append(rid)
        steps.append({"entries": entries, "end": end})
    assert all(progress[r] == len(reqs[r]) for r in ids)
    assert max(len(st["entries"]) for st in steps) == 4
    max_tokens = 144                       # 9 pages of 16, 18 of 8: the most that is ever held at once
    demand = sum((len(t) + page - 1) // page for t in reqs.values())
    assert demand > max_tokens // page, "the pool must be smaller than the requests' pages together"
    got, rp = replay(folders[name], dtype, name, steps, max_tokens, poison_freed_pages=True)
    assert rp.manager.all_free() and not rp.live
    late, early = rp.pages_held[ids[3]], rp.pages_held[ids[2]] | rp.pages_held[ids[4]]
    assert late & early, "the request that came late must have been given pages that an earlier one gave back"
    for rid in ids:
        assert np.array_equal(got[rid], whole[rid]), f"{rid}: the mixed batch differs from the whole prompt"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_context_and_partition_edges(folders, dtype):
    """Hundreds of keys: partitions of 64 keys, pages of 16, the split route of decoded tokens
    (from 256 keys on) and graph replay, all against the plain implementation and each other."""
    name = "LONG"
    cfg = tiny.read_config(folders[name])
    toks = requests_for(cfg, 3, [700])["r0"]
    ref = plain_logits(folders[name], toks, dtype)
    whole, _ = replay(folders[name], dtype, name, [{"entries": [all_wanted("x", toks)]}], 704)
    check_against_plain(whole["x"], ref, dtype, "700 tokens")
    # prompt of 250 tokens, then one by one across the 256-key threshold and several partition edges
    steps = [{"entries": [all_wanted("x", toks[:250])]}]
    steps += [{"entries": [{"id": "x", "tokens": [toks[i]], "want": [0]}]} for i in range(250, 400)]
    steps += [{"entries": [all_wanted("x", toks[400:447])]}, {"entries": [all_wanted("x", toks[447:449])]}]
    steps += [{"entries": [{"id": "x", "tokens": [toks[i]], "want": [0]}]} for i in range(449, 700)]
    for use_graphs in (True, False):
        got, _ = replay(folders[name], dtype, name, steps, 704, use_graphs=use_graphs)
        same = (got["x"] == whole["x"]).all(axis=1)
        assert same.all(), f"first differing position {int(np.argmin(same))} (graphs={use_graphs})"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "LONG"])
def test_peaked_attention_whole_model(gpu, tmp_path, name, dtype):
    """Weights ten times as large as the tiny configurations' own: scores spread over tens of units, so a query
    puts its weight on a few keys and a wrong rotation, scale, key or partition edge moves the logits by far
    more than the bound (with the small weights attention is close to a running mean and hides them).  The
    observed error is printed beside the bound; the cuttings must still agree to the last bit."""
    from bitwise_amd.model import Model, write_random_model
    from bitwise_amd.replay import Replayer

    cfg, seed, _, page = tiny.CONFIGS[name]
    lengths = [300, 129] if name == "LONG" else [100, 41]
    reqs = ru.requests_for(cfg["vocab_size"], 23, lengths)
    # one layer of it first: a differing rounding stays at its position there, so the median over positions shows
    # whether every formula of a layer is the plain one's
    one = dict(cfg, num_hidden_layers=1)
    folder = write_random_model(tmp_path / "peaked1", one, seed + 40, 0.3, "bfloat16")
    model = Model.load(folder, dtype)
    for rid, toks in reqs.items():
        got = ru.run_steps(Replayer("", dtype, 320, block_size=page, model=model), ru.whole_steps(rid, toks))[rid]
        ref = pl.forward(one, tiny.read_weights(folder), toks, **tiny.plain_mode(dtype)).numpy()
        check_against_plain(got, ref, dtype, f"peaked {name} {rid}, one layer", PEAKED_TOL[dtype], median=True)
    folder = write_random_model(tmp_path / "peaked", cfg, seed + 40, 0.3, "bfloat16")
    w = tiny.read_weights(folder)
    model = Model.load(folder, dtype)
    whole = {}
    for rid, toks in reqs.items():
        whole[rid] = ru.run_steps(Replayer("", dtype, 320, block_size=page, model=model), ru.whole_steps(rid, toks))[rid]
        ref = pl.forward(cfg, w, toks, **tiny.plain_mode(dtype)).numpy()
        check_against_plain(whole[rid], ref, dtype, f"peaked {name} {rid}", PEAKED_TOL[dtype])
        top = (whole[rid].argmax(axis=1) == ref.argmax(axis=1)).mean()
        assert top >= (1.0 if dtype == "float32" else 0.97), f"top-1 agreement {top:.3f}"
    for rid, toks in reqs.items():
        got = ru.run_steps(Replayer("", dtype, 320, block_size=page, model=model), ru.tail_steps(rid, toks))
        assert np.array_equal(got[rid], whole[rid]), f"{rid}: decoding differs from the whole prompt"
        got = ru.run_steps(Replayer("", dtype, 320, block_size=page, model=model), ru.portion_steps(rid, toks, 3))
        assert np.array_equal(got[rid], whole[rid]), f"{rid}: portions differ from the whole prompt"
    steps, most = ru.mixed_steps(reqs, seed=9, page=page)
    got = ru.run_steps(Replayer("", dtype, most, block_size=page, model=model, poison_freed_pages=True), steps)
    for rid in reqs:
        assert np.array_equal(got[rid], whole[rid]), f"{rid}: the mixed trace differs from the whole prompt"


def test_the_workspace_stops_growing_while_contexts_grow(folders, tmp_path):
    """Steps launched kernel by kernel bring block tables as wide as the step needs, and decoded tokens of few
    requests split their attention over workgroups that meet in scratch sized by that width: the scratch is made
    once for the widest table the engine can see, so a long run's memory stays where the first such step put it."""
    from bitwise_amd.model import Model, write_random_model
    from bitwise_amd.replay import Replayer

    cfg = dict(tiny.CONFIGS["LONG"][0], max_position_embeddings=2048)
    folder = write_random_model(tmp_path / "long2k", cfg, 6, 0.05)
    model = Model.load(folder, "bfloat16")
    toks = ru.requests_for(cfg["vocab_size"], 8, [900])["r0"]
    other = ru.requests_for(cfg["vocab_size"], 9, [500])["r0"]
    rp = Replayer("", "bfloat16", 2048, block_size=16, model=model, use_graphs=False)
    rp.step([{"id": "a", "tokens": toks[:520], "want": []}])
    sizes, widths = [], set()
    for i in range(520, 900):
        entries = [{"id": "a", "tokens": [toks[i]], "want": [0]}]
        if i >= 600:                              # a second request comes and decodes beside the first
            j = i - 600
            entries.append({"id": "b", "tokens": other[:200] if j == 0 else [other[199 + j]], "want": []})
        rp.step(entries)
        sizes.append(rp.runner.ws.nbytes())
        widths.add(len(rp.live["a"].tables[0]))
    assert len(widths) > 20, "the block table must have grown page by page"
    assert len([k for k in rp.runner.ws._buffers if k[0] == "attn_split"]) == 1, "the split route must have run, on one buffer"
    assert sizes[-1] == sizes[0], f"the workspace grew from {sizes[0]} to {sizes[-1]} bytes"


def test_first_tokens_of_a_sequence(folders):
    """Positions 0 and 1: one key, no rotation at position 0."""
    for name in ("A", "B"):
        for dtype in ("float32", "bfloat16"):
            cfg = tiny.read_config(folders[name])
            toks = requests_for(cfg, 5, [3])["r0"]
            ref = plain_logits(folders[name], toks, dtype)
            one, _ = replay(folders[name], dtype, name, [{"entries": [{"id": "a", "tokens": toks[:1], "want": [0]}]},
                                                       {"entries": [{"id": "a", "tokens": toks[1:2], "want": [0]}]},
                                                       {"entries": [{"id": "a", "tokens": toks[2:], "want": [0]}]}], 64)
            check_against_plain(one["a"], ref, dtype, f"first tokens {name}", median=True)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_order_of_a_steps_entries_changes_nothing(folders, dtype):
    """A step lays its requests' rows out in an order of its own (portions of whole blocks of 16 rows, other portions,
    single tokens); the wanted logits come back in the caller's order, and in any order of the entries they are the
    same bits."""
    from bitwise_amd.engine.batch import Segment, StepContext
    from bitwise_amd.replay import Replayer
    name = "B"
    cfg = tiny.read_config(folders[name])
    reqs = requests_for(cfg, 21, [40, 35, 32, 9])
    first = [{"id": "r0", "tokens": reqs["r0"][:39], "want": []}, {"id": "r3", "tokens": reqs["r3"][:8], "want": []}]
    second = [{"id": "r0", "tokens": reqs["r0"][39:], "want": [0]}, {"id": "r1", "tokens": reqs["r1"], "want": [0, 34]},
              {"id": "r3", "tokens": reqs["r3"][8:], "want": [0]}, {"id": "r2", "tokens": reqs["r2"], "want": [31, 5]}]
    got = []
    for entries in (second, second[::-1], [second[1], second[3], second[0], second[2]]):
        rp = Replayer(str(folders[name]), dtype, 256, block_size=tiny.CONFIGS[name][3])
        rp.step(first)
        lg = rp.step(entries)
        rows, row = {}, 0
        for e in entries:
            for w in e["want"]:
                rows[(e["id"], w)] = lg[row]
                row += 1
        got.append(rows)
    for other in got[1:]:
        assert got[0].keys() == other.keys() and all(np.array_equal(got[0][k], other[k]) for k in got[0])
    ref = plain_logits(folders[name], reqs["r1"], dtype)
    check_against_plain(np.stack([got[0][("r1", 0)], got[0][("r1", 34)]]), ref[[0, 34]], dtype, "a portion between single tokens")
    # the layout itself
    ctx = StepContext([Segment([1], 39, [[0, 1, 2, 3, 4]], 0, [0]), Segment([2] * 35, 0, [[5, 6, 7, 8, 9]], 1, [0, 34]),
                       Segment([3] * 32, 0, [[10, 11, 12, 13]], 2, [31, 5])], 1, rp.runner.ws)
    assert [len(sg.tokens) for sg in ctx.segments] == [32, 35, 1] and ctx.seq_start == [0, 32, 67]
    assert ctx.want_rows.tolist() == [67, 32, 66, 31, 5] and ctx.slots.tolist() == [2, 1, 0]
    assert ctx.row_seq.tolist() == [0] * 32 + [1] * 35 + [2]


def test_trace_run_program(folders, tmp_path):
    """bin/trace_run as a user calls it: JSON steps on standard input, <step>.f32 files, a
    'done <step>' line after every step, exit 0; a request may pause and pages are reused."""
    name, dtype = "B", "bfloat16"
    cfg = tiny.read_config(folders[name])
    reqs = requests_for(cfg, 21, [50, 20, 70])
    a, b, c = reqs["r0"], reqs["r1"], reqs["r2"]
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:30], "want": [0, 29]}], "end": []},
        {"step": 1, "entries": [{"id": "b", "tokens": b, "want": [19]}, {"id": "a", "tokens": a[30:32], "want": []}], "end": ["b"]},
        {"step": 2, "entries": [{"id": "c", "tokens": c[:64], "want": [63]}], "end": []},                  # a pauses
        {"step": 3, "entries": [{"id": "a", "tokens": a[32:33], "want": [0]}, {"id": "c", "tokens": c[64:], "want": [5]}], "end": ["c"]},
        {"step": 4, "entries": [{"id": "a", "tokens": a[33:], "want": [16]}], "end": ["a"]},
    ]
    out = tmp_path / "out"
    env = dict(os.environ, PYTHONPATH=str(ROOT))
    p = subprocess.run([sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(folders[name]), "--dtype", dtype,
                        "--out", str(out), "--max-tokens", "192", "--block-size", "8"],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, env=env,
                       timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert p.stdout.split() == ["done", "0", "done", "1", "done", "2", "done", "3", "done", "4"]
    V = cfg["vocab_size"]
    ra, rb, rc = (plain_logits(folders[name], t, dtype) for t in (a, b, c))
    want = {0: [ra[0], ra[29]], 1: [rb[19]], 2: [rc[63]], 3: [ra[32], rc[69]], 4: [ra[49]]}
    chained = {"a": 1469598103934665603, "b": 1469598103934665603, "c": 1469598103934665603}
    owners = {0: ["a", "a"], 1: ["b"], 2: ["c"], 3: ["a", "c"], 4: ["a"]}
    for step, rows in want.items():
        got = np.fromfile(out / f"{step}.f32", dtype="<f4").reshape(-1, V)
        assert got.shape[0] == len(rows)
        for g, r, rid in zip(got, rows, owners[step]):
            assert np.abs(g - r).max() <= TOL[dtype] * np.abs(r).max()
            chained[rid] = pl.hash_floats(chained[rid], g)
    # every request's fingerprint: the hash chained over the rows it asked for, as the files hold them
    prints = json.loads((out / "fingerprints.json").read_text())
    assert {k: int(v, 16) for k, v in prints.items()} == chained


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_awkward_sizes(gpu, tmp_path, dtype):
    """Configurations whose sizes fall between the kernels' favourite ones (head sizes 48, 80 and 256, 14 heads on 2,
    a width of 64 with heads of 48, a feed-forward of 8, a vocabulary of 17; one segment of K and a bit): every
    fusion that does not take them must step aside, and the logits are the plain ones whatever the cutting."""
    import bitwise_amd as bw
    from bitwise_amd.model import write_random_model

    base = dict(tiny.TINY_A, max_position_embeddings=512)
    configs = [
        dict(base, hidden_size=136, num_attention_heads=6, num_key_value_heads=3, head_dim=80, intermediate_size=344,
             vocab_size=1001, num_hidden_layers=3, tie_word_embeddings=False),
        dict(base, hidden_size=256, num_attention_heads=2, num_key_value_heads=1, head_dim=256, intermediate_size=520,
             vocab_size=4099, num_hidden_layers=2),
        dict(base, hidden_size=64, num_attention_heads=14, num_key_value_heads=2, head_dim=48, intermediate_size=8,
             vocab_size=17, num_hidden_layers=1),
        dict(base, hidden_size=2048 + 64, num_attention_heads=33, num_key_value_heads=33, head_dim=64,
             intermediate_size=2056, vocab_size=1000, num_hidden_layers=1, tie_word_embeddings=False),
    ]
    for i, cfg in enumerate(configs):
        folder = tmp_path / f"awkward{i}"
        write_random_model(folder, cfg, 10 + i, 0.05, "bfloat16")
        model = bw.Model.load(folder, dtype)
        g = torch.Generator().manual_seed(30 + i)
        toks = torch.randint(0, cfg["vocab_size"], (75,), generator=g).tolist()
        whole = model.logits(toks)
        want = pl.forward(cfg, tiny.read_weights(folder), toks, **tiny.plain_mode(dtype)).numpy()
        check_against_plain(whole, want, dtype, f"awkward sizes {i}", median=cfg["num_hidden_layers"] == 1 and cfg["hidden_size"] <= 256)     # (a wide layer has a differing rounding at most positions)
        assert np.array_equal(model.logits(toks, chunk=5), whole) and np.array_equal(model.logits(toks, chunk=1), whole), (i, dtype)


REAL_SHAPES = {
    # SmolLM2-1.7B's layer sizes
    "smollm2": dict(vocab_size=49152, hidden_size=2048, num_attention_heads=32, num_key_value_heads=32, head_dim=64,
                    intermediate_size=8192, rope_theta=130000.0, tie_word_embeddings=True),
    # Llama-3-8B's: heads of 128, four query heads a key head, a feed-forward of seven 2048-segments, an untied head
    "llama3_8b": dict(vocab_size=128256, hidden_size=4096, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
                      intermediate_size=14336, rope_theta=500000.0, tie_word_embeddings=False),
}


@pytest.mark.parametrize("shape,dtype", [("smollm2", "bfloat16"), ("smollm2", "float32"), ("llama3_8b", "bfloat16"),
                                         ("llama3_8b", "float32")])
def test_real_layer_sizes_are_cut_invariant(gpu, shape, dtype):
    """Two layers of real sizes, so that every shape-dependent route of the kernels runs at the shapes it was
    written for (K = 2048, 4096, 8192 and 14336; up to 128,256 columns), in bfloat16 and in 32-bit: a prompt whole;
    in portions of 900, 700, 300, 100, 61, 29 and 10 tokens; with its last 40 tokens decoded one by one from graphs;
    and decoded beside 8 and then 19 other requests; in bfloat16 also with the decode steps' products run as phases of a
    few launches (EngineConfig.decode_phases).  The logits of the last 40 positions are the same bits every time."""
    import bitwise_amd as bw
    from bitwise_amd.replay import Replayer

    cfg = dict({"architectures": ["LlamaForCausalLM"], "model_type": "llama", "hidden_act": "silu", "num_hidden_layers": 2,
                "rms_norm_eps": 1e-5, "max_position_embeddings": 4096, "bos_token_id": 1, "eos_token_id": 2},
               **REAL_SHAPES[shape])
    vocab = cfg["vocab_size"]
    model = bw.Model.random(cfg, seed=3, dtype=dtype, sigma=0.02, on_device=True)
    g = torch.Generator().manual_seed(11)
    toks = torch.randint(0, vocab, (2100,), generator=g).tolist()
    others = {f"o{i}": torch.randint(0, vocab, (30,), generator=g).tolist() for i in range(19)}
    tail = 40
    head = len(toks) - tail

    def last(rp_steps, max_tokens=4096, decode_phases=False):
        rp = Replayer("", dtype, max_tokens, block_size=16, model=model, decode_phases=decode_phases)
        rows = []
        for st in rp_steps:
            lg = rp.step(st["entries"], st.get("end", []))
            row = 0
            for e in st["entries"]:
                for _ in e["want"]:
                    if e["id"] == "r":
                        rows.append(lg[row].copy())
                    row += 1
        if decode_phases:
            rp.runner.check_phases()              # no wait inside a launch gave up
        return np.stack(rows)

    whole = last([{"entries": [{"id": "r", "tokens": toks, "want": list(range(head, len(toks)))}]}])
    assert whole.shape == (tail, vocab) and np.isfinite(whole).all()
    steps, pos = [], 0
    for n in (900, 700, 300, 100, 61, 29, 10):
        want = [i - pos for i in range(max(pos, head), pos + n)]
        steps.append({"entries": [{"id": "r", "tokens": toks[pos:pos + n], "want": want}]})
        pos += n
    assert np.array_equal(last(steps), whole), "portions of 900, 700, 300, 100, 61, 29, 10"
    one = [{"entries": [{"id": "r", "tokens": toks[:head + 1], "want": [head]}]}]
    one += [{"entries": [{"id": "r", "tokens": [t], "want": [0]}]} for t in toks[head + 1:]]
    assert np.array_equal(last(one), whole), "last tokens one by one"
    if dtype == "bfloat16":
        # the decode steps' products as phases of a few launches that wait for each other inside the kernel
        assert np.array_equal(last(one, decode_phases=True), whole), "last tokens one by one, products as phases"
    for crowd in (8, 19):
        names = list(others)[:crowd]
        mixed = [{"entries": [{"id": "r", "tokens": toks[:head + 1], "want": [head]}] +
                             [{"id": n, "tokens": others[n], "want": []} for n in names]}]
        for j, t in enumerate(toks[head + 1:]):
            mixed.append({"entries": [{"id": n, "tokens": [others[n][j % 30]], "want": [0]} for n in names[:crowd // 2]] +
                                     [{"id": "r", "tokens": [t], "want": [0]}] +
                                     [{"id": n, "tokens": [others[n][j % 30]], "want": [0]} for n in names[crowd // 2:]]})
        assert np.array_equal(last(mixed, max_tokens=8192), whole), f"decoded beside {crowd} others"
        if dtype == "bfloat16" and crowd == 8:
            assert np.array_equal(last(mixed, max_tokens=8192, decode_phases=True), whole), "decoded beside 8 others, products as phases"
