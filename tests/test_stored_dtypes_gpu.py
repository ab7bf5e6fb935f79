"""Checkpoints stored in 32-bit, in float16 and in a mixture, run in both modes.

The reference's converter keeps BF16 and F32 bytes and widens F16 to F32 (tools/convert.py:85-92), and its
engine widens bfloat16 weights exactly and computes in 32-bit whatever was stored (src/kernels.cpp:77-81,
src/model.cpp:135-171).  Here: in 32-bit mode the logits are, bit for bit, the plain scalar decoder's on the
stored values.  In bfloat16 mode the activations are rounded to bfloat16 at the same places whatever dtype a
weight is stored in (a 32-bit weight meets them widened again, in a 32-bit product); the plain counterpart is
the float64 model with those roundings, and the four cuttings give the same bits."""

import json

import numpy as np
import pytest
import torch

import plain_llama as pl
import plain_scalar as ps
import tiny
from replay_util import (check_against_plain, mixed_steps, portion_steps, requests_for, run_steps, tail_steps,
                         whole_steps)

pytestmark = pytest.mark.gpu


def stored_as(name: str, variant: str) -> dict:
    """dtype by tensor name for a variant: all 32-bit, all float16, or a mixture that sends every product of a
    layer down another road (q|k|v and gate|up on the matrix cores, output and down projection in 32-bit, norms
    and embedding in 32-bit, so that a tied head is a 32-bit product too)."""
    from bitwise_amd.model import describe

    cfg = tiny.CONFIGS[name][0]
    out = {}
    for tensor in describe(cfg):
        if variant == "float32":
            out[tensor] = torch.float32
        elif variant == "float16":
            out[tensor] = torch.float16
        elif "norm" in tensor or "embed_tokens" in tensor or "o_proj" in tensor:
            out[tensor] = torch.float32
        elif "down_proj" in tensor:
            out[tensor] = torch.float16
        else:
            out[tensor] = torch.bfloat16
    return out


@pytest.fixture(scope="module")
def stored(tmp_path_factory, gpu):
    """{(configuration, variant, layers: 0 for the configuration's own): folder}"""
    from bitwise_amd.model import describe
    from bitwise_amd.weights import loader, safetensors_io

    tmp = tmp_path_factory.mktemp("stored")
    out = {}
    for name in ("A", "B"):
        cfg, seed, sigma, _ = tiny.CONFIGS[name]
        for variant in ("float32", "float16", "mixed"):
            for layers in (0, 1):
                c = dict(cfg, num_hidden_layers=layers) if layers else cfg
                folder = tmp / f"{name}_{variant}_{layers}"
                folder.mkdir()
                (folder / "config.json").write_text(json.dumps(c))
                dtypes = stored_as(name, variant)
                tensors = ((n, t.to(dtypes[n])) for n, t in loader.random_tensors(describe(c), seed, sigma, torch.float32))
                safetensors_io.write_file(folder / "model.safetensors", tensors)
                out[name, variant, layers] = folder
    return out


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("variant", ["float32", "float16", "mixed"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_stored_dtypes_in_both_modes(stored, name, variant, dtype):
    from bitwise_amd.model import Model
    from bitwise_amd.replay import Replayer

    folder = stored[name, variant, 0]
    cfg, page = tiny.read_config(folder), tiny.CONFIGS[name][3]
    model = Model.load(folder, dtype)
    held = {n: t.dtype for n, t in _bound_tensors(model).items()}
    want_dtypes = {n: (torch.float32 if d == torch.float16 else d) for n, d in stored_as(name, variant).items()}
    assert held == want_dtypes, "a tensor stored in 32-bit stays so, float16 is widened, bfloat16 stays"
    weights = {n: t.float() for n, t in tiny.read_weights(folder).items()}     # widening is exact
    reqs = requests_for(cfg["vocab_size"], 17, [70, 41, 20])

    # one layer of it: the median over positions is bounded at 32-bit accuracy in bfloat16 mode too
    one = stored[name, variant, 1]
    model1, w1 = Model.load(one, dtype), {n: t.float() for n, t in tiny.read_weights(one).items()}
    for rid, toks in reqs.items():
        ref = pl.forward(tiny.read_config(one), w1, toks, **tiny.plain_mode(dtype)).numpy()
        check_against_plain(model1.logits(toks, block_size=page), ref, dtype, f"{name} stored as {variant} {rid}, one layer",
                            median=True)

    def replayer(max_tokens, **kw):
        return Replayer("", dtype, max_tokens, block_size=page, model=model, **kw)

    whole = {}
    for rid, toks in reqs.items():
        whole[rid] = run_steps(replayer(128), whole_steps(rid, toks))[rid]
        if dtype == "float32":
            want = ps.forward(cfg, weights, toks)
            same = (whole[rid].view(np.uint32) == want.view(np.uint32)).all(axis=1)
            assert same.all(), f"{rid}: first position that is not the scalar decoder's bits: {int(np.argmin(same))}"
        ref = pl.forward(cfg, weights, toks, **tiny.plain_mode(dtype)).numpy()
        check_against_plain(whole[rid], ref, dtype, f"{name} stored as {variant} {rid}")
    for rid, toks in reqs.items():
        for use_graphs in (True, False):
            got = run_steps(replayer(128, use_graphs=use_graphs), tail_steps(rid, toks))
            assert np.array_equal(got[rid], whole[rid]), f"{rid}: decoding differs from the whole prompt (graphs={use_graphs})"
        got = run_steps(replayer(128), portion_steps(rid, toks, seed=len(toks)))
        assert np.array_equal(got[rid], whole[rid]), f"{rid}: portions differ from the whole prompt"
    steps, most = mixed_steps(reqs, seed=5, page=page, max_live=2)
    assert most < sum((len(t) + page - 1) // page * page for t in reqs.values()), "pages must come back and be used again"
    rp = replayer(most, poison_freed_pages=True)
    got = run_steps(rp, steps)
    assert rp.manager.all_free() and not rp.live
    for rid in reqs:
        assert np.array_equal(got[rid], whole[rid]), f"{rid}: the mixed trace differs from the whole prompt"


def _bound_tensors(model) -> dict:
    """What the parts hold after loading, by checkpoint name (stacked products by their stack's dtype)."""
    asm, out = model.assembled, {}
    out["model.embed_tokens.weight"] = asm.embedding.weight
    out["model.norm.weight"] = asm.final_norm.weight
    if not asm.lm_head.tied:
        out["lm_head.weight"] = asm.lm_head.linear.weight
    for i, block in enumerate(asm.layers):
        pre = f"model.layers.{i}."
        out[pre + "input_layernorm.weight"] = block.mixer_norm.weight
        out[pre + "post_attention_layernorm.weight"] = block.ffn_norm.weight
        for n in ("q_proj", "k_proj", "v_proj"):
            out[pre + f"self_attn.{n}.weight"] = block.mixer.qkv.weight
        out[pre + "self_attn.o_proj.weight"] = block.mixer.o.weight
        for n in ("gate_proj", "up_proj"):
            out[pre + f"mlp.{n}.weight"] = block.feed_forward.gate_up.weight
        out[pre + "mlp.down_proj.weight"] = block.feed_forward.down.weight
    return out


def test_convert_kernel(gpu):
    """float32 <-> bfloat16 with strided rows: widening is exact; narrowing rounds to nearest, ties to even;
    infinities stay, NaN stays NaN; rows beyond the count and the padding between rows are not touched."""
    from bitwise_amd.csrc import ops

    def f32(bits):
        return torch.tensor(bits, dtype=torch.int64).to(torch.int32).view(torch.float32)

    # exact ties between two bfloat16 values (low half 0x8000): to the even one; just above and below a tie;
    # the largest finite value rounds to infinity; a denormal; signed zeros
    special = f32([0x3F808000, 0x3F818000, 0x3F808001, 0x3F807FFF, 0x7F7FFFFF, 0x7F800000, 0xFF800000, 0x7FC00000,
                   0x00000001, 0x80000000, 0x00008000, 0x00018000, 0x7F7F8000, 0x7FA00000])
    want_bits = [0x3F80, 0x3F82, 0x3F81, 0x3F80, 0x7F80, 0x7F80, 0xFF80, None, 0x0000, 0x8000, 0x0000, 0x0002, 0x7F80, None]
    g = torch.Generator().manual_seed(4)
    rows, cols, pad = 5, 37, 11
    src = torch.randn(rows + 2, cols + pad, generator=g) * 3.0
    src[0, :special.numel()] = special
    src = src.to(gpu)
    dst = torch.full((rows + 2, cols + 5), 7.0, dtype=torch.bfloat16, device=gpu)
    ops.convert(src[:, :cols], dst[:, :cols], rows)
    got = dst.cpu()
    ref = src.cpu()[:, :cols].to(torch.bfloat16)
    got_bits = got[:rows, :cols].view(torch.int16).numpy().astype(np.uint16)
    ref_bits = ref[:rows].view(torch.int16).numpy().astype(np.uint16)
    nan = torch.isnan(ref[:rows]).numpy()
    assert np.array_equal(got_bits[~nan], ref_bits[~nan]) and torch.isnan(got[:rows, :cols])[torch.from_numpy(nan)].all()
    for i, bits in enumerate(want_bits):
        if bits is None:
            assert torch.isnan(got[0, i])
        else:
            assert int(got_bits[0, i]) == bits, (i, hex(int(got_bits[0, i])), hex(bits))
    assert (got[rows:] == 7.0).all() and (got[:, cols:] == 7.0).all(), "rows past the count and the padding stay"
    # widening: exact, strided the other way
    back = torch.full((rows + 1, cols + 3), -1.0, dtype=torch.float32, device=gpu)
    ops.convert(dst[:, :cols], back[:, :cols], rows)
    b = back.cpu()
    wide = got[:rows, :cols].float()
    ok = (b[:rows, :cols] == wide) | (torch.isnan(b[:rows, :cols]) & torch.isnan(wide))
    assert ok.all() and (b[rows:] == -1.0).all() and (b[:, cols:] == -1.0).all()
