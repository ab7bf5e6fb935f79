"""Each part alone against the plain implementation, a toy mixer with state of its own that
is registered, built and stepped without touching the framework, and schedules that name a
layer twice or let a layer read another layer's cache."""

import numpy as np
import pytest
import torch

import plain_llama as pl
import tiny
from bitwise_amd.cache.manager import CacheManager, GroupSpec
from bitwise_amd.engine.batch import Segment, StepContext
from bitwise_amd.engine.runner import ModelRunner
from bitwise_amd.engine.storage import CacheStorage
from bitwise_amd.models.assembled import AssembledModel, CallBinding
from bitwise_amd.parts import base
from bitwise_amd.parts.base import LayerCall, LayerSpec, ModelSpec, PartSpec, StateSpec, TensorSpec
from bitwise_amd.runtime import Runtime, Workspace
from bitwise_amd.weights.loader import random_tensors

pytestmark = pytest.mark.gpu
F64 = torch.float64
TOL = {"float32": 3e-6, "bfloat16": 1.5e-2}


def check_rows(got, ref, mode, what):
    """Maximum over all rows within TOL, and the median over rows at 32-bit accuracy: in bfloat16 mode part and
    plain code round at the same places, so a row differs by more only where a value fell so close to the
    middle between two bfloat16 numbers that the two roundings parted."""
    scale = ref.abs().max()
    per_row = ((got - ref).abs().amax(dim=1) / scale).numpy()
    print(f"{what} {mode}: max {per_row.max():.2e} (bound {TOL[mode]:.1e}), median over rows {np.median(per_row):.2e} (bound 1e-6)")
    assert per_row.max() <= TOL[mode] and np.median(per_row) <= 1e-6, what


def rnd_for(mode):
    return pl.round_bf16 if mode == "bfloat16" else pl.identity


def one_request_ctx(ws, n, groups=1, pages=None):
    pages = pages if pages is not None else list(range((n + ws.page_size - 1) // ws.page_size))
    return StepContext([Segment([0] * n, 0, [pages] * groups, 0, [])], groups, ws)


@pytest.mark.parametrize("mode", ["float32", "bfloat16"])
def test_norm_part(gpu, mode):
    rt, ws = Runtime(mode, gpu), Workspace(gpu, max_rows=32, page_size=8)
    part = base.NORMS["rmsnorm"]({"width": 72, "eps": 1e-3}, rt)
    assert part.tensors() == {"weight": TensorSpec((72,), "norm")}
    w = 1 + 0.1 * torch.randn(72)
    part.bind({"weight": w.bfloat16()})
    x = torch.zeros(32, 72, device=gpu)
    x[:5] = torch.randn(5, 72, device=gpu) * 2
    out = part.forward(one_request_ctx(ws, 5), x)
    assert out.dtype == rt.act_dtype
    ref = pl.rmsnorm(x[:5].double().cpu(), w.bfloat16(), 1e-3)
    assert (out[:5].cpu().double() - ref).abs().max() <= (2 ** -8 if mode == "bfloat16" else 4e-7) * ref.abs().max()


@pytest.mark.parametrize("mode", ["float32", "bfloat16"])
@pytest.mark.parametrize("stored", [torch.bfloat16, torch.float32])
def test_a_projection_with_a_bias(gpu, mode, stored):
    """The reference's architecture has no biases; a part of another one passes ``bias`` to Linear: one 32-bit addition
    behind the product's sum, stored in 32-bit or rounded to bfloat16, or the biased product added whole into the
    residual stream.  Against 64-bit arithmetic at the product's tolerance, and to the bit against the same Linear
    without a bias followed by the addition."""
    from bitwise_amd.parts.linear import Linear
    rt, ws = Runtime(mode, gpu), Workspace(gpu, max_rows=32, page_size=8)
    g = torch.Generator().manual_seed(12)
    n, k, rows = 88, 72, 19
    w = (torch.randn(n, k, generator=g) * 0.3).to(stored)
    b = torch.randn(n, generator=g).bfloat16()
    x = torch.zeros(32, k, device=gpu, dtype=rt.act_dtype)
    x[:rows] = torch.randn(rows, k, generator=g).to(rt.act_dtype).to(gpu)
    with_bias, plain = Linear(w, rt, bias=b), Linear(w, rt)
    ref = pl.linear(x[:rows].cpu().double(), w) + b.double()
    y = torch.zeros(32, n, device=gpu)
    with_bias.store(ws, x, y, rows)
    check_rows(y[:rows].cpu().double(), ref, mode, "biased projection")
    y0 = torch.zeros(32, n, device=gpu)
    plain.store(ws, x, y0, rows)
    assert torch.equal(y[:rows], y0[:rows] + b.float().to(gpu))
    yb = torch.zeros(32, n, device=gpu, dtype=torch.bfloat16)
    with_bias.store(ws, x, yb, rows)
    assert torch.equal(yb[:rows], y[:rows].bfloat16())
    res = torch.randn(32, n, generator=g).to(gpu)
    before = res.clone()
    with_bias.add_into(ws, x, res, rows)
    assert torch.equal(res[:rows], before[:rows] + y[:rows]) and torch.equal(res[rows:], before[rows:])
    assert with_bias.nbytes() == plain.nbytes() + 4 * n
    with pytest.raises(ValueError):
        Linear(w, rt, bias=b[:5])


@pytest.mark.parametrize("mode", ["float32", "bfloat16"])
def test_feed_forward_part(gpu, mode):
    rt, ws = Runtime(mode, gpu), Workspace(gpu, max_rows=64, page_size=8)
    part = base.FEED_FORWARDS["swiglu"]({"width": 40, "inter": 88}, rt)
    specs = part.tensors()
    assert specs["down_proj.weight"].shape == (40, 88) and specs["gate_proj.weight"].shape == (88, 40)
    w = dict(random_tensors(specs, 3, 0.3))
    part.bind(w)
    n = 21
    h = torch.zeros(64, 40, device=gpu, dtype=rt.act_dtype)
    h[:n] = torch.randn(n, 40, device=gpu).to(rt.act_dtype)
    res = torch.randn(64, 40, device=gpu)
    before = res.clone()
    part.forward(one_request_ctx(ws, n), h, res)
    hd = h[:n].cpu().double()
    act = rnd_for(mode)(pl.swiglu(pl.linear(hd, w["gate_proj.weight"]), pl.linear(hd, w["up_proj.weight"])))
    ref = before[:n].cpu().double() + pl.linear(act, w["down_proj.weight"])
    check_rows(res[:n].cpu().double(), ref, mode, "feed-forward part")
    assert torch.equal(res[n:], before[n:])                         # rows beyond the step are not touched


@pytest.mark.parametrize("mode", ["float32", "bfloat16"])
@pytest.mark.parametrize("heads,kvh,hd,window", [(4, 2, 16, None), (3, 1, 32, None), (6, 3, 48, 10)])
def test_attention_part(gpu, mode, heads, kvh, hd, window):
    """The mixer alone: projections, rotation, cache write through a permuted block table,
    attention (with a window as an option) and the output projection added to the residual."""
    width, page = 56, 8
    rt, ws = Runtime(mode, gpu), Workspace(gpu, max_rows=64, page_size=page)
    pos_spec = PartSpec("rope", {"theta": 5000.0, "head_dim": hd, "max_positions": 64})
    part = base.MIXERS["attention"]({"width": width, "heads": heads, "kv_heads": kvh, "head_dim": hd, "window": window,
                                     "position": pos_spec}, rt)
    w = dict(random_tensors(part.tensors(), 5, 0.2))
    part.bind(w)
    assert part.cache_spec().window == window and part.state_spec() is None
    n = 37
    pages = [6, 2, 5, 0, 4]
    cache = torch.zeros(7, part.page_elements(page), device=gpu, dtype=rt.act_dtype)
    call = CallBinding(0, 0, 0, 0, 0, True, k_cache=cache, v_cache=torch.zeros_like(cache))
    h_all = torch.randn(n, width).to(rt.act_dtype)
    res = torch.zeros(64, width, device=gpu)
    # the first 30 positions as one portion, then 7 single tokens: the cache carries over
    h = torch.zeros(64, width, device=gpu, dtype=rt.act_dtype)
    h[:30] = h_all[:30].to(gpu)
    ctx = StepContext([Segment([0] * 30, 0, [pages], 0, [])], 1, ws)
    part.forward(ctx, call, h, res)
    got = [res[:30].cpu().clone()]
    for p in range(30, n):
        h[0] = h_all[p].to(gpu)
        res.zero_()
        part.forward(StepContext([Segment([0], p, [pages], 0, [])], 1, ws), call, h, res)
        got.append(res[:1].cpu().clone())
    got = torch.cat(got).double()
    x = h_all.double()
    rnd = rnd_for(mode)
    inv = pl.rope_inv_freq(5000.0, hd)
    q = rnd(pl.rope(pl.linear(x, w["q_proj.weight"]).view(n, heads, hd), range(n), inv))
    k = rnd(pl.rope(pl.linear(x, w["k_proj.weight"]).view(n, kvh, hd), range(n), inv))
    v = rnd(pl.linear(x, w["v_proj.weight"]).view(n, kvh, hd))
    ref = pl.linear(rnd(pl.attention(q, k, v, rnd, window, partition=64 if mode == "bfloat16" else None)).reshape(n, -1),
                    w["o_proj.weight"])
    check_rows(got, ref, mode, f"attention part {heads}/{kvh}x{hd} window {window}")


# ----------------------------------------------------------------------------- a toy mixer with state

@base.register_mixer("toy_running_mean")
class RunningMean(base.Mixer):
    """Adds gain * (mean of all rows of the request so far) to the residual.  Its per-request
    state (count and running sum) lives in a slot, not in pages."""

    def __init__(self, params, runtime):
        super().__init__(params, runtime)
        self.width = params["width"]
        self.gain = None

    def tensors(self):
        return {"gain": TensorSpec((self.width,), "norm")}

    def bind(self, tensors):
        self.gain = tensors["gain"].to(self.rt.device).float()

    def state_spec(self):
        return StateSpec((self.width + 1,), "float32")

    def forward(self, ctx, call, h, residual):
        for seg, r0 in zip(ctx.segments, ctx.seq_start):
            n = len(seg.tokens)
            st = call.state[seg.slot]
            rows = h[r0:r0 + n].float()
            sums = st[1:] + torch.cumsum(rows, 0)
            counts = st[0] + torch.arange(1, n + 1, device=rows.device, dtype=torch.float32)
            residual[r0:r0 + n] += self.gain * sums / counts[:, None]
            st[0] += n
            st[1:] = sums[-1]


def toy_spec(width=32, vocab=50):
    def layer(i, mixer):
        pre = f"layers.{i}."
        return LayerSpec.prenorm(mixer, PartSpec("swiglu", {"width": width, "inter": 48}, pre + "mlp."),
                                 PartSpec("rmsnorm", {"width": width, "eps": 1e-5}, pre + "norm1."),
                                 PartSpec("rmsnorm", {"width": width, "eps": 1e-5}, pre + "norm2."))
    rope = PartSpec("rope", {"theta": 10000.0, "head_dim": 16, "max_positions": 128})
    attn = PartSpec("attention", {"width": width, "heads": 2, "kv_heads": 1, "head_dim": 16, "window": None,
                                  "position": rope}, "layers.1.attn.")
    layers = [layer(0, PartSpec("toy_running_mean", {"width": width}, "layers.0.toy.")), layer(1, attn)]
    # the toy layer runs twice (two states), the attention layer runs twice: the second call
    # reads the cache the first one wrote
    schedule = [LayerCall(0, 0), LayerCall(1, 1), LayerCall(0, 2), LayerCall(1, 1, writes_cache=False)]
    return ModelSpec("ToyForTests", vocab, width, PartSpec("embedding", {"vocab": vocab, "width": width}, "embed."),
                     layers, schedule, PartSpec("rmsnorm", {"width": width, "eps": 1e-5}, "norm."),
                     PartSpec("lm_head", {"vocab": vocab, "width": width, "tied": True}, "head."), 128)


def plain_toy(w, toks, rnd):
    """The toy model with plain parts, whole sequence."""
    n = len(toks)
    x = pl.embed(toks, w["embed.weight"])

    def mlp(x, pre):
        hn = rnd(pl.rmsnorm(x, w[pre + "norm2.weight"], 1e-5))
        a = rnd(pl.swiglu(pl.linear(hn, w[pre + "mlp.gate_proj.weight"]), pl.linear(hn, w[pre + "mlp.up_proj.weight"])))
        return pl.linear(a, w[pre + "mlp.down_proj.weight"])

    def toy(x):
        hn = rnd(pl.rmsnorm(x, w["layers.0.norm1.weight"], 1e-5))
        mean = torch.cumsum(hn, 0) / torch.arange(1, n + 1, dtype=F64)[:, None]
        x = x + w["layers.0.toy.gain"].double() * mean
        return x + mlp(x, "layers.0.")

    kv = {}

    def attn(x, write):
        hn = rnd(pl.rmsnorm(x, w["layers.1.norm1.weight"], 1e-5))
        inv = pl.rope_inv_freq(10000.0, 16)
        q = rnd(pl.rope(pl.linear(hn, w["layers.1.attn.q_proj.weight"]).view(n, 2, 16), range(n), inv))
        if write:
            kv["k"] = rnd(pl.rope(pl.linear(hn, w["layers.1.attn.k_proj.weight"]).view(n, 1, 16), range(n), inv))
            kv["v"] = rnd(pl.linear(hn, w["layers.1.attn.v_proj.weight"]).view(n, 1, 16))
        a = rnd(pl.attention(q, kv["k"], kv["v"], rnd)).reshape(n, -1)
        x = x + pl.linear(a, w["layers.1.attn.o_proj.weight"])
        return x + mlp(x, "layers.1.")

    x = attn(toy(attn(toy(x), True)), False)
    return pl.linear(rnd(pl.rmsnorm(x, w["norm.weight"], 1e-5)), w["embed.weight"])


@pytest.mark.parametrize("mode", ["float32", "bfloat16"])
def test_toy_mixer_with_state_and_a_schedule_that_repeats_and_shares(gpu, mode):
    rt = Runtime(mode, gpu)
    model = AssembledModel(toy_spec(), rt)
    assert len(model.state_specs) == 2 and len(model.group_specs) == 1 and model.group_caches == [[1]]
    assert not model.graph_safe                                   # the toy part works on the host: no graph capture
    specs = model.tensor_specs()
    assert "layers.0.toy.gain" in specs and "head.weight" not in specs
    w = dict(random_tensors(specs, 9, 0.2))
    model.bind_tensors({k: v.to(gpu) for k, v in w.items()})
    storage = CacheStorage(model, num_pages=12, num_slots=3, page_size=8)
    manager = CacheManager([GroupSpec(None)], 12, 8, 3, prefix_caching=True, has_state=True)
    assert not manager.prefix_caching                             # state outside the pages: no prefix reuse
    runner = ModelRunner(model, storage, max_model_len=128, max_rows=64, use_graphs=True)
    a = [int(t) for t in torch.randint(0, 50, (23,), generator=torch.Generator().manual_seed(1))]
    b = [int(t) for t in torch.randint(0, 50, (11,), generator=torch.Generator().manual_seed(2))]
    rnd = rnd_for(mode)
    ref = {"a": plain_toy(w, a, rnd).numpy(), "b": plain_toy(w, b, rnd).numpy()}
    rcs = {"a": manager.open(), "b": manager.open()}
    for rc in rcs.values():
        storage.reset_slot(rc.slot)
    got = {"a": [], "b": []}
    cuts = [[("a", 9)], [("a", 1), ("b", 5)], [("b", 1), ("a", 2)], [("a", 11), ("b", 5)]]
    prog = {"a": 0, "b": 0}
    toks = {"a": a, "b": b}
    for step in cuts:
        segs = []
        for rid, n in step:
            rc = rcs[rid]
            assert manager.ensure(rc, prog[rid] + n)
            segs.append(Segment(toks[rid][prog[rid]:prog[rid] + n], prog[rid], rc.tables, rc.slot, list(range(n))))
        lg = runner.step(segs).cpu().numpy()
        row = 0
        for rid, n in step:
            got[rid].append(lg[row:row + n])
            row += n
            prog[rid] += n
            manager.advance(rcs[rid], toks[rid], prog[rid])
    for rid in ("a", "b"):
        out = np.concatenate(got[rid])
        assert out.shape == ref[rid].shape
        assert np.abs(out - ref[rid]).max() <= (2e-2 if mode == "bfloat16" else 2e-5) * np.abs(ref[rid]).max()
    # a slot that is taken again starts from zero state
    manager.close(rcs["a"])
    rc = manager.open()
    storage.reset_slot(rc.slot)
    assert manager.ensure(rc, len(b))
    lg = runner.step([Segment(b, 0, rc.tables, rc.slot, list(range(len(b))))]).cpu().numpy()
    assert np.abs(lg - ref["b"]).max() <= (2e-2 if mode == "bfloat16" else 2e-5) * np.abs(ref["b"]).max()


# ----------------------------------------------------------------------------- a toy routed feed-forward, a toy position encoding

@base.register_feed_forward("toy_top1")
class TopOneExperts(base.FeedForward):
    """Two square experts and a router: every row goes through the expert whose router logit (32-bit) is larger,
    ties to the first.  The choice depends on the row alone, so it does not matter what else is in the batch."""

    def __init__(self, params, runtime):
        super().__init__(params, runtime)
        self.width = params["width"]

    def tensors(self):
        return {"router.weight": TensorSpec((2, self.width)), "experts.0.weight": TensorSpec((self.width, self.width)),
                "experts.1.weight": TensorSpec((self.width, self.width))}

    def bind(self, tensors):
        self.router = tensors["router.weight"].to(self.rt.device).float()
        self.experts = [tensors[f"experts.{e}.weight"].to(self.rt.device).float() for e in range(2)]

    def forward(self, ctx, h, residual):
        rows = h[:ctx.rows].float()
        logits = rows @ self.router.T
        second = logits[:, 1] > logits[:, 0]
        out = torch.where(second[:, None], rows @ self.experts[1].T, rows @ self.experts[0].T)
        residual[:ctx.rows] += out


@base.register_position_encoding("toy_stretched_rope")
class StretchedRotary(base.PositionEncoding):
    """Rotary angles of position / stretch (positions interpolated): the tables a mixer's kernels read, built by
    another rule.  params: theta, head_dim, max_positions, stretch."""

    def __init__(self, params, runtime):
        super().__init__(params, runtime)
        hd, n = int(params["head_dim"]), int(params["max_positions"])
        inv = pl.rope_inv_freq(float(params["theta"]), hd)
        places = (np.arange(n, dtype=np.float32) / np.float32(params["stretch"]))[:, None]
        angle = (places * inv[None, :]).astype(np.float32).astype(np.float64)
        self.rotary_dim = hd
        self.cos = torch.from_numpy(np.cos(angle).astype(np.float32)).to(runtime.device).contiguous()
        self.sin = torch.from_numpy(np.sin(angle).astype(np.float32)).to(runtime.device).contiguous()

    def tables(self):
        return self.cos, self.sin


@pytest.mark.parametrize("mode", ["float32", "bfloat16"])
def test_toy_routed_feed_forward_and_another_position_encoding(gpu, mode):
    """A model of one layer whose feed-forward routes rows between two experts and whose attention reads the tables
    of a position encoding defined here: registered, built, stepped in portions and compared with plain code; nothing
    in the framework's files knows of either."""
    width, vocab, hd, stretch = 32, 40, 16, 4.0
    pos = PartSpec("toy_stretched_rope", {"theta": 1000.0, "head_dim": hd, "max_positions": 64, "stretch": stretch})
    attn = PartSpec("attention", {"width": width, "heads": 2, "kv_heads": 2, "head_dim": hd, "window": None, "position": pos},
                    "l.attn.")
    layer = LayerSpec.prenorm(attn, PartSpec("toy_top1", {"width": width}, "l.moe."),
                              PartSpec("rmsnorm", {"width": width, "eps": 1e-5}, "l.norm1."),
                              PartSpec("rmsnorm", {"width": width, "eps": 1e-5}, "l.norm2."))
    spec = ModelSpec("ToyRouted", vocab, width, PartSpec("embedding", {"vocab": vocab, "width": width}, "embed."), [layer],
                     [LayerCall(0, 0)], PartSpec("rmsnorm", {"width": width, "eps": 1e-5}, "norm."),
                     PartSpec("lm_head", {"vocab": vocab, "width": width, "tied": True}, "head."), 64)
    rt = Runtime(mode, gpu)
    model = AssembledModel(spec, rt)
    w = dict(random_tensors(model.tensor_specs(), 17, 0.3))
    model.bind_tensors({k: v.to(gpu) for k, v in w.items()})
    storage = CacheStorage(model, num_pages=8, num_slots=2, page_size=8)
    manager = CacheManager([GroupSpec(None)], 8, 8, 2, prefix_caching=False)
    runner = ModelRunner(model, storage, max_model_len=64, max_rows=32, use_graphs=False)
    toks = [int(t) for t in torch.randint(0, vocab, (21,), generator=torch.Generator().manual_seed(5))]
    rnd = rnd_for(mode)

    # plain: whole sequence, the toy parts written out again
    n = len(toks)
    x = pl.embed(toks, w["embed.weight"])
    hn = rnd(pl.rmsnorm(x, w["l.norm1.weight"], 1e-5))
    inv = pl.rope_inv_freq(1000.0, hd)
    places = [p / stretch for p in range(n)]
    q = rnd(pl.rope(pl.linear(hn, w["l.attn.q_proj.weight"]).view(n, 2, hd), places, inv))
    k = rnd(pl.rope(pl.linear(hn, w["l.attn.k_proj.weight"]).view(n, 2, hd), places, inv))
    v = rnd(pl.linear(hn, w["l.attn.v_proj.weight"]).view(n, 2, hd))
    x = x + pl.linear(rnd(pl.attention(q, k, v, rnd)).reshape(n, -1), w["l.attn.o_proj.weight"])
    hn = rnd(pl.rmsnorm(x, w["l.norm2.weight"], 1e-5))
    logits = hn.float().double() @ w["l.moe.router.weight"].double().T
    chosen = (logits[:, 1] > logits[:, 0]).long()
    assert 0 < int(chosen.sum()) < n                                # both experts get rows
    experts = [w[f"l.moe.experts.{e}.weight"].double() for e in range(2)]
    x = x + torch.stack([hn[i].double() @ experts[int(chosen[i])].T for i in range(n)])
    ref = pl.linear(rnd(pl.rmsnorm(x, w["norm.weight"], 1e-5)), w["embed.weight"]).numpy()

    rc = manager.open()
    got, done = [], 0
    for cut in (8, 1, 5, 7):
        assert manager.ensure(rc, done + cut)
        lg = runner.step([Segment(toks[done:done + cut], done, rc.tables, rc.slot, list(range(cut)))])
        got.append(lg.cpu().numpy())
        done += cut
        manager.advance(rc, toks, done)
    out = np.concatenate(got)
    assert np.abs(out - ref).max() <= (2e-2 if mode == "bfloat16" else 2e-5) * np.abs(ref).max()


def test_schedule_errors(gpu):
    rt = Runtime("float32", gpu)
    spec = toy_spec()
    spec.schedule = [LayerCall(1, 5, writes_cache=False)]
    with pytest.raises(ValueError, match="before any call wrote it"):
        AssembledModel(spec, rt)
    spec.schedule = [LayerCall(1, 0), LayerCall(1, 0)]
    with pytest.raises(ValueError, match="already has a writer"):
        AssembledModel(spec, rt)
    spec.schedule = [LayerCall(7, 0)]
    with pytest.raises(ValueError, match="names layer 7"):
        AssembledModel(spec, rt)
    spec.layers[0].parts["mixer"].kind = "no_such_mixer"
    with pytest.raises(KeyError, match="unknown mixer 'no_such_mixer'"):
        AssembledModel(spec, rt)
