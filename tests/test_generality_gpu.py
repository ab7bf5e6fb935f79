"""What another architecture would need, shown with toy parts that are defined here and never become a
model of anyone's: a whole architecture registered from outside the package and run from a folder; a mixer
with per-request device state that can be captured in a graph, through the engine with preemption; two
engines at once on one model; caches with different windows in one model, end to end with pages that come
back NaN-filled."""

from dataclasses import asdict, dataclass

import numpy as np
import pytest
import torch

import bitwise_amd as bw
import plain_llama as pl
import plain_scalar as ps
import tiny
from bitwise_amd.models.assembled import AssembledModel
from bitwise_amd.models.llama import llama_spec
from bitwise_amd.parts import base
from bitwise_amd.parts.base import LayerCall, LayerSpec, ModelSpec, PartSpec, StateSpec, TensorSpec
from bitwise_amd.replay import Replayer
from bitwise_amd.runtime import Runtime
from bitwise_amd.weights import loader

pytestmark = pytest.mark.gpu
F64 = torch.float64


# ----------------------------------------------------------------------------- a toy architecture

@base.register_mixer("toy_decay")
class DecayMixer(base.Mixer):
    """s_t = 0.5 * s_(t-1) + h_t per request, residual_t += gain * s_t.  The state s lives in the request's
    slot on the device.  Steps of one row per request run as dense device operations only (they can be
    captured in a graph; rows with a negative slot are padding and must touch nothing); other steps walk
    their segments from the host."""

    graph_safe = True

    def __init__(self, params, runtime):
        super().__init__(params, runtime)
        self.width = int(params["width"])
        self.gain = None

    def tensors(self):
        return {"gain": TensorSpec((self.width,), "norm")}

    def bind(self, tensors):
        self.gain = tensors["gain"].to(self.rt.device).float()

    def weight_bytes(self):
        return 4 * self.width

    def state_spec(self):
        return StateSpec((self.width,), "float32")

    def forward(self, ctx, call, h, residual):
        state = call.state
        if getattr(ctx, "one_row_per_request", False):
            rows = ctx.rows
            slots = ctx.slots[:rows].long()
            live = slots >= 0
            idx = slots.clamp(min=0)
            s_new = 0.5 * state[idx] + h[:rows].float()
            residual[:rows] += torch.where(live[:, None], self.gain * s_new, torch.zeros_like(s_new))
            # every slot takes the new state of the row that names it, if any: dense, no scatter, no race
            names = (slots[None, :] == torch.arange(state.shape[0], device=state.device)[:, None])
            row_of = names.float().argmax(1)
            state.copy_(torch.where(names.any(1)[:, None], s_new[row_of], state))
            return
        for seg, r0 in zip(ctx.segments, ctx.seq_start):
            s = state[seg.slot].clone()
            for i in range(len(seg.tokens)):
                s = 0.5 * s + h[r0 + i].float()
                residual[r0 + i] += self.gain * s
            state[seg.slot] = s


@dataclass(frozen=True)
class ToyConfig:
    architecture: str
    vocab: int
    width: int
    depth: int
    inter: int
    eps: float
    max_len: int
    eos: int

    @classmethod
    def from_dict(cls, d):
        return cls(d["architectures"][0], int(d["vocab"]), int(d["width"]), int(d["depth"]), int(d["inter"]),
                   float(d["eps"]), int(d["max_len"]), int(d.get("eos", -1)))

    def to_dict(self):
        out = asdict(self)
        out["architectures"] = [out.pop("architecture")]
        return out


HEADS, KV_HEADS, HEAD_DIM, THETA = 2, 1, 16, 1000.0


def toy_spec(cfg: ToyConfig) -> ModelSpec:
    """Even layers mix with the decaying state, odd layers with attention over the paged cache."""
    def norm(prefix):
        return PartSpec("rmsnorm", {"width": cfg.width, "eps": cfg.eps}, prefix)
    rope = PartSpec("rope", {"theta": THETA, "head_dim": HEAD_DIM, "max_positions": cfg.max_len})
    layers = []
    for i in range(cfg.depth):
        if i % 2 == 0:
            mixer = PartSpec("toy_decay", {"width": cfg.width}, f"blocks.{i}.mix.")
        else:
            mixer = PartSpec("attention", {"width": cfg.width, "heads": HEADS, "kv_heads": KV_HEADS, "head_dim": HEAD_DIM,
                                           "window": None, "position": rope}, f"blocks.{i}.att.")
        layers.append(LayerSpec.prenorm(mixer, PartSpec("swiglu", {"width": cfg.width, "inter": cfg.inter}, f"blocks.{i}.ff."),
                                        norm(f"blocks.{i}.n1."), norm(f"blocks.{i}.n2.")))
    return ModelSpec(cfg.architecture, cfg.vocab, cfg.width,
                     PartSpec("embedding", {"vocab": cfg.vocab, "width": cfg.width}, "tok."), layers,
                     [LayerCall(i, i) for i in range(cfg.depth)], norm("out_norm."),
                     PartSpec("lm_head", {"vocab": cfg.vocab, "width": cfg.width, "tied": False}, "out."),
                     cfg.max_len, -1, cfg.eos)


if "ToyDecayForCausalLM" not in bw.ARCHITECTURES:
    bw.register_architecture("ToyDecayForCausalLM", ToyConfig.from_dict, toy_spec)

TOY = {"architectures": ["ToyDecayForCausalLM"], "vocab": 83, "width": 40, "depth": 3, "inter": 56, "eps": 1e-5,
       "max_len": 96, "eos": 7}


def plain_toy(w, toks, rnd):
    """The toy architecture in plain code, whole sequence, float64."""
    n = len(toks)
    x = pl.embed(toks, w["tok.weight"])
    for i in range(TOY["depth"]):
        pre = f"blocks.{i}."
        hn = rnd(pl.rmsnorm(x, w[pre + "n1.weight"], TOY["eps"]))
        if i % 2 == 0:
            s = torch.zeros(TOY["width"], dtype=F64)
            mixed = []
            for t in range(n):
                s = 0.5 * s + hn[t]
                mixed.append(w[pre + "mix.gain"].double() * s)
            x = x + torch.stack(mixed)
        else:
            inv = pl.rope_inv_freq(THETA, HEAD_DIM)
            q = rnd(pl.rope(pl.linear(hn, w[pre + "att.q_proj.weight"]).view(n, HEADS, HEAD_DIM), range(n), inv))
            k = rnd(pl.rope(pl.linear(hn, w[pre + "att.k_proj.weight"]).view(n, KV_HEADS, HEAD_DIM), range(n), inv))
            v = rnd(pl.linear(hn, w[pre + "att.v_proj.weight"]).view(n, KV_HEADS, HEAD_DIM))
            x = x + pl.linear(rnd(pl.attention(q, k, v, rnd)).reshape(n, -1), w[pre + "att.o_proj.weight"])
        hn = rnd(pl.rmsnorm(x, w[pre + "n2.weight"], TOY["eps"]))
        act = rnd(pl.swiglu(pl.linear(hn, w[pre + "ff.gate_proj.weight"]), pl.linear(hn, w[pre + "ff.up_proj.weight"])))
        x = x + pl.linear(act, w[pre + "ff.down_proj.weight"])
    return pl.linear(rnd(pl.rmsnorm(x, w["out_norm.weight"], TOY["eps"])), w["out.weight"])


def plain_toy_generate(w, prompt, n, rnd):
    toks, out = list(prompt), []
    for _ in range(n):
        t = pl.argmax_row(plain_toy(w, toks, rnd)[-1].float().numpy())
        toks.append(t)
        out.append(t)
    return out


@pytest.fixture(scope="module")
def toy_folder(tmp_path_factory, gpu):
    folder = tmp_path_factory.mktemp("toy") / "model"
    bw.write_random_model(folder, TOY, seed=5, sigma=0.2)
    return folder


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_whole_toy_architecture_from_a_folder(toy_folder, dtype):
    """config.json names an architecture that only this file knows; loader, cache manager, step function,
    scheduler, sampler and the entry point run it unchanged; its decode steps are replayed from graphs."""
    assert tiny.read_config(toy_folder)["architectures"] == ["ToyDecayForCausalLM"]
    w = tiny.read_weights(toy_folder)
    assert set(w) == set(bw.describe(TOY))
    model = bw.Model.load(toy_folder, dtype)
    assert isinstance(model.config, ToyConfig) and model.assembled.graph_safe
    assert len(model.assembled.group_specs) == 1 and len(model.assembled.state_specs) == 2
    rnd = pl.round_bf16 if dtype == "bfloat16" else pl.identity
    prompt = [(i * 11 + 3) % TOY["vocab"] for i in range(13)]
    want = plain_toy(w, prompt, rnd).numpy()
    got = model.logits(prompt)
    assert np.abs(got - want).max() <= (2e-2 if dtype == "bfloat16" else 2e-5) * np.abs(want).max()
    sp = bw.SamplingParams(max_new_tokens=12, ignore_eos=True)
    outs = []
    for graphs in (True, False):
        cfg = bw.EngineConfig(num_blocks=8, max_batched_tokens=8, max_num_seqs=4, dtype=dtype, use_graphs=graphs)
        (r,) = bw.generate(model, [prompt], sp, cfg)
        outs.append(r)
    assert outs[0].tokens == outs[1].tokens and outs[0].logits_fingerprint == outs[1].logits_fingerprint
    assert outs[0].tokens == plain_toy_generate(w, prompt, 12, rnd)


def test_stateful_mixer_through_the_engine_with_preemption(toy_folder):
    """Requests of the toy architecture in an engine whose page pool forces preemption: a preempted request
    gives its slot back, takes one again later (zeroed) and is recomputed; its tokens and logits are those
    of a solo run, with graphs on and off."""
    dtype = "float32"
    model = bw.Model.load(toy_folder, dtype)
    # (a part that does not say that all its launches go through ops keeps the engine from holding launches back)
    assert not model.assembled.launches_through_ops
    g = torch.Generator().manual_seed(8)
    prompts = [torch.randint(0, TOY["vocab"], (n,), generator=g).tolist() for n in (9, 17, 5, 12)]
    sp = bw.SamplingParams(max_new_tokens=20, ignore_eos=True)
    solo = [bw.generate(model, [p], sp, bw.EngineConfig(num_blocks=8, max_num_seqs=1, dtype=dtype))[0] for p in prompts]
    for graphs in (True, False):
        eng = bw.Engine(model, None, bw.EngineConfig(num_blocks=7, max_batched_tokens=16, max_num_seqs=4, dtype=dtype,
                                                     use_graphs=graphs))
        resets = []
        real_reset = eng.exec.storage.reset_slot
        eng.exec.storage.reset_slot = lambda slot: (resets.append(slot), real_reset(slot))[1]
        ids = [eng.add_request(p, sp) for p in prompts]
        guard = 0
        while not eng.idle():
            eng.step()
            guard += 1
            assert guard < 2000, eng.debug_state()
        assert eng.stats.preemptions > 0, "the pool was meant to be too small"
        # every admission zeroes its slot (an admission that finds no pages gives the slot back and comes again)
        assert len(resets) >= len(prompts) + eng.stats.preemptions
        for i, ref in zip(ids, solo):
            assert eng.result(i).tokens == ref.tokens
            assert eng.result(i).logits_fingerprint == ref.logits_fingerprint
        assert eng.manager.all_free()


# ----------------------------------------------------------------------------- two engines on one model

@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_two_engines_and_model_logits_share_one_model(gpu, tmp_path, dtype):
    """Two engines with different page sizes and step sizes on one model, their steps interleaved, and
    Model.logits in between: nobody sees anybody else's caches, buffers or page size."""
    folder = tiny.make_folder(tmp_path, "B")
    model = bw.Model.load(folder, dtype)
    g = torch.Generator().manual_seed(3)
    prompts = [torch.randint(0, 500, (n,), generator=g).tolist() for n in (21, 40, 9)]
    sp = [bw.SamplingParams(max_new_tokens=18, ignore_eos=True, temperature=0.7, seed=i) for i in range(3)]
    solo = [bw.generate(model, [p], s, bw.EngineConfig(num_blocks=16, block_size=8, dtype=dtype))[0] for p, s in zip(prompts, sp)]
    whole = model.logits(prompts[1])
    a = bw.Engine(model, None, bw.EngineConfig(num_blocks=40, block_size=8, max_batched_tokens=16, dtype=dtype))
    b = bw.Engine(model, None, bw.EngineConfig(num_blocks=9, block_size=16, max_batched_tokens=64, max_num_seqs=2, dtype=dtype))
    ids_a = [a.add_request(p, s) for p, s in zip(prompts, sp)]
    ids_b = [b.add_request(p, s) for p, s in zip(reversed(prompts), reversed(sp))]
    assert a.exec.storage.keys[0].data_ptr() != b.exec.storage.keys[0].data_ptr()
    assert a.exec.runner.ws is not b.exec.runner.ws
    guard = 0
    while not (a.idle() and b.idle()):
        if not a.idle():
            a.step()
        if guard % 3 == 0:
            assert np.array_equal(model.logits(prompts[1], chunk=7, block_size=32), whole)
        if not b.idle():
            b.step()
        guard += 1
        assert guard < 2000
    for i, ref in zip(ids_a, solo):
        assert a.result(i).tokens == ref.tokens and a.result(i).logits_fingerprint == ref.logits_fingerprint
    for i, ref in zip(ids_b, reversed(solo)):
        assert b.result(i).tokens == ref.tokens and b.result(i).logits_fingerprint == ref.logits_fingerprint
    with pytest.raises(ValueError, match="positions"):
        model.logits(list(range(257)))                       # beyond max_position_embeddings: refused, not read


# ----------------------------------------------------------------------------- windows end to end

def windowed_model(folder, dtype, windows):
    """Tiny B's weights in a model whose layers keep windows of their own: three cache groups."""
    cfg = bw.LlamaConfig.from_dict(tiny.read_config(folder))
    spec = llama_spec(cfg)
    for ls, win in zip(spec.layers, windows):
        ls.parts["mixer"].params["window"] = win
    asm = AssembledModel(spec, Runtime(dtype, "cuda:0"))
    asm.bind_tensors(loader.load_folder(folder, asm.tensor_specs()))
    return bw.Model(cfg, asm)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_windowed_groups_end_to_end(gpu, tmp_path, dtype):
    """Layers with windows of 24 and 40 keys beside one that keeps all keys (three cache groups with pools
    of their own), pages of 8: a prompt in portions down to two tokens, then decoding past several windows,
    while a second request arrives and takes pages the first has given back.  Freed pages are filled with
    NaN.  Graphs on and off; every cutting equals the whole prompt bit for bit and the plain code."""
    folder = tiny.make_folder(tmp_path, "B")
    windows = [24, None, 40]
    model = windowed_model(folder, dtype, windows)
    assert len(model.assembled.group_specs) == 3
    cfg, w = tiny.read_config(folder), tiny.read_weights(folder)
    g = torch.Generator().manual_seed(14)
    x = torch.randint(0, 500, (150,), generator=g).tolist()
    y = torch.randint(0, 500, (70,), generator=g).tolist()
    mode = tiny.plain_mode(dtype)
    refs = {"x": pl.forward(cfg, w, x, windows=windows, **mode).numpy(), "y": pl.forward(cfg, w, y, windows=windows, **mode).numpy()}
    tol = 1e-2 if dtype == "bfloat16" else 2e-5

    def run(steps, max_tokens, **kw):
        rp = Replayer("", dtype, max_tokens, block_size=8, model=model, poison_freed_pages=True, **kw)
        out = {}
        taken = {}
        for st in steps:
            lg = rp.step(st["entries"])
            row = 0
            for e in st["entries"]:
                for _ in e["want"]:
                    out.setdefault(e["id"], []).append(lg[row].copy())
                    row += 1
            for rid, rc in rp.live.items():
                for gi, table in enumerate(rc.tables):
                    taken.setdefault((rid, gi), set()).update(p for p in table if p >= 0)
            rp.step([], st.get("end", []))
            rp.manager.check()
        assert rp.manager.all_free()
        return {k: np.stack(v) for k, v in out.items()}, taken

    def entry(rid, toks):
        return {"id": rid, "tokens": toks, "want": list(range(len(toks)))}

    whole, _ = run([{"entries": [entry("x", x)], "end": ["x"]}, {"entries": [entry("y", y)], "end": ["y"]}], 160)
    for rid in ("x", "y"):
        assert np.abs(whole[rid] - refs[rid]).max() <= tol * np.abs(refs[rid]).max(), rid
    if dtype == "float32":
        want = ps.forward(cfg, w, x, window=windows)
        assert np.array_equal(whole["x"].view(np.uint32), want.view(np.uint32))

    # x: portions 30, 2, 17, 2, 9 then one by one; y arrives when x is 60 tokens in, in portions beside x's tokens
    steps, px = [], 0
    for n in (30, 2, 17, 2, 9):
        steps.append({"entries": [entry("x", x[px:px + n])]})
        px += n
    py = 0
    for n in (25, 2, 1, 1, 41):
        steps.append({"entries": [entry("x", x[px:px + 1]), entry("y", y[py:py + n])]})
        px += 1
        py += n
    steps[-1]["end"] = ["y"]
    while px < len(x):
        steps.append({"entries": [entry("x", x[px:px + 1])]})
        px += 1
    steps[-1]["end"] = ["x"]
    for graphs in (True, False):
        got, taken = run(steps, 232, use_graphs=graphs)       # 29 pages a group: x whole (19) and y whole (9) in the all-keys group
        for rid in ("x", "y"):
            same = (got[rid] == whole[rid]).all(axis=1)
            assert same.all(), f"{rid}: first differing position {int(np.argmin(same))} (graphs={graphs})"
        # in the windowed groups y was served from pages that x had given back
        assert taken[("y", 0)] & taken[("x", 0)] and taken[("y", 2)] & taken[("x", 2)]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prefix_reuse_with_windowed_groups_in_the_engine(gpu, tmp_path, dtype):
    """Three cache groups (windows of 24 and 40 keys beside all keys) in the engine with the prefix cache on:
    requests that share a 40-token start, and one that repeats another's prompt, arrive one after the other
    in a pool that forces preemption; later ones start behind cached pages in every group (for the windowed
    groups only the pages under the window are taken), and everyone's tokens and logits are those of a solo run
    without any of that."""
    folder = tiny.make_folder(tmp_path, "B")
    model = windowed_model(folder, dtype, [24, None, 40])
    g = torch.Generator().manual_seed(21)
    stem = torch.randint(0, 500, (40,), generator=g).tolist()
    prompts = [stem + torch.randint(0, 500, (n,), generator=g).tolist() for n in (9, 30, 3, 17)]
    prompts.append(list(prompts[1]))
    sp = [bw.SamplingParams(max_new_tokens=24, ignore_eos=True, temperature=0.8 if i % 2 else 0.0, seed=i) for i in range(5)]
    solo = [bw.generate(model, [p], s, bw.EngineConfig(num_blocks=32, block_size=8, dtype=dtype, prefix_caching=False,
                                                       use_graphs=False, run_ahead=False))[0] for p, s in zip(prompts, sp)]
    for graphs in (True, False):
        eng = bw.Engine(model, None, bw.EngineConfig(num_blocks=26, block_size=8, max_batched_tokens=32, max_num_seqs=3,
                                                     dtype=dtype, use_graphs=graphs))
        assert eng.manager.prefix_caching and len(eng.manager.pools) == 3
        ids, guard = [], 0
        while len(ids) < len(prompts) or not eng.idle():
            if guard % 4 == 0 and len(ids) < len(prompts):
                ids.append(eng.add_request(prompts[len(ids)], sp[len(ids)]))
            eng.step()
            eng.manager.check()
            guard += 1
            assert guard < 3000, eng.debug_state()
        assert eng.stats.prefix_hit_tokens >= 40 and eng.manager.all_free()
        for i, ref in zip(ids, solo):
            assert eng.result(i).tokens == ref.tokens, (graphs, i)
            assert eng.result(i).logits_fingerprint == ref.logits_fingerprint, (graphs, i)
        assert eng.result(ids[4]).prefix_cached_tokens >= 64      # the repeated prompt: every full page but the last token's


def test_a_mixer_names_its_caches_dtype_and_page_sizes(gpu):
    """A toy mixer that pages 32-bit integers (token ids) in bfloat16 mode and takes pages of 4 or 8 tokens only:
    the storage gives its group pools of that dtype, a page size it does not take is refused by name, and a
    position encoding that rotates part of a head is refused by the attention part."""
    from bitwise_amd.engine.storage import CacheStorage
    from bitwise_amd.parts import base
    from bitwise_amd.parts.base import CacheSpec, LayerCall, LayerSpec, ModelSpec, PartSpec

    @base.register_mixer("toy_token_pager")
    class TokenPager(base.Mixer):
        graph_safe = False

        def cache_spec(self):
            return CacheSpec(1, 1, None, key_width=1, value_width=0, dtype="int32")

        def page_sizes(self):
            return (4, 8)

        def forward(self, ctx, call, h, residual):
            pass

    width = 32
    norm = PartSpec("rmsnorm", {"width": width, "eps": 1e-5}, "n.")
    layers = [LayerSpec.prenorm(PartSpec("toy_token_pager", {}, "m."), PartSpec("swiglu", {"width": width, "inter": 16}, "f."), norm, norm),
              LayerSpec.prenorm(PartSpec("attention", {"width": width, "heads": 2, "kv_heads": 1, "head_dim": 16, "window": None,
                                                       "position": PartSpec("rope", {"theta": 1e4, "head_dim": 16, "max_positions": 32})},
                                         "a."), PartSpec("swiglu", {"width": width, "inter": 16}, "f."), norm, norm)]
    spec = ModelSpec("ToyPager", 20, width, PartSpec("embedding", {"vocab": 20, "width": width}, "e."), layers,
                     [LayerCall(0, 0), LayerCall(1, 1)], norm, PartSpec("lm_head", {"vocab": 20, "width": width, "tied": True}, "h."), 32)
    asm = AssembledModel(spec, Runtime("bfloat16", "cuda:0"))
    assert len(asm.group_specs) == 2
    storage = CacheStorage(asm, num_pages=6, num_slots=2, page_size=8)
    assert storage.keys[0].dtype == torch.int32 and storage.keys[0].shape == (1, 6, 8) and storage.values[0].shape == (1, 6, 0)
    assert storage.keys[1].dtype == torch.bfloat16
    storage.poison_pages(0, [2])
    assert int(storage.keys[0][0, 2, 0]) == -(2 ** 31) and int(storage.keys[0][0, 1, 0]) == 0
    with pytest.raises(ValueError, match="layer 0: its mixer takes pages of \\[4, 8\\] tokens, not of 16"):
        CacheStorage(asm, num_pages=6, num_slots=2, page_size=16)
    with pytest.raises(ValueError, match="layer 1: its mixer takes pages of \\[8, 16, 32, 64\\] tokens, not of 4"):
        CacheStorage(asm, num_pages=6, num_slots=2, page_size=4)

    @base.register_position_encoding("toy_partial_rope")
    class PartialRotary(base.PositionEncoding):
        def __init__(self, params, runtime):
            super().__init__(params, runtime)
            self.rotary_dim = 8

    with pytest.raises(ValueError, match="rotates 8 elements of a head and needs a mixer of its own"):
        base.MIXERS["attention"]({"width": width, "heads": 2, "kv_heads": 1, "head_dim": 16, "window": None,
                                  "position": PartSpec("toy_partial_rope", {})}, Runtime("bfloat16", "cuda:0"))
