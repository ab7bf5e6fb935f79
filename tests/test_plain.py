"""What pins the plain implementation beside the reference's text: special cases that reduce
to library routines, invariants, and known constants, each chosen so that a plausible
mistake (a wrong sign or pairing, a norm in the wrong place, a transposed weight) fails."""

import math
from pathlib import Path

import numpy as np
import pytest
import torch

import plain_llama as pl
from tiny import TINY_A, TINY_B

F64 = torch.float64


def test_linear_orientation():
    w = torch.arange(12, dtype=F64).view(3, 4)            # [out=3, in=4]
    x = torch.zeros(1, 4, dtype=F64)
    x[0, 2] = 1.0
    assert torch.equal(pl.linear(x, w)[0], w[:, 2])       # a one-hot input reads a column of W
    assert pl.linear(torch.ones(2, 4, dtype=F64), w).shape == (2, 3)


def test_rmsnorm_eps_inside_the_root_and_weight_last():
    c, eps = 3.0, 0.5
    x = torch.full((1, 8), c, dtype=F64)
    y = pl.rmsnorm(x, torch.ones(8), eps)
    assert torch.allclose(y, torch.full_like(y, c / math.sqrt(c * c + eps)), rtol=1e-15)
    assert not torch.allclose(y, torch.full_like(y, c / (math.sqrt(c * c) + eps)))      # eps outside the root
    assert torch.equal(pl.rmsnorm(torch.zeros(1, 8, dtype=F64), torch.ones(8), 1e-5), torch.zeros(1, 8, dtype=F64))
    w = torch.tensor([2.0, 0.0, -1.0, 1.0])
    x = torch.tensor([[1.0, 2.0, 3.0, 4.0]], dtype=F64)
    ms = (1 + 4 + 9 + 16) / 4                               # the mean of squares, not the sum
    assert torch.allclose(pl.rmsnorm(x, w, 0.0), x / math.sqrt(ms) * w.to(F64), rtol=1e-15)


def test_rope_pairing_sign_and_invariants():
    hd = 8
    inv = pl.rope_inv_freq(10000.0, hd)
    assert inv[0] == np.float32(1.0) and np.allclose(inv[1], 10000.0 ** (-2 / hd), rtol=1e-6)
    v = torch.randn(3, 2, hd, dtype=F64)
    assert torch.equal(pl.rope(v, [0, 0, 0], inv), v)                         # position 0 is the identity
    e0 = torch.zeros(1, 1, hd, dtype=F64)
    e0[0, 0, 0] = 1.0
    r = pl.rope(e0, [1], inv)[0, 0]
    # rotate-half: index 0 pairs with index hd/2 (interleaved pairing would move it to index 1);
    # positive angle: cos on itself, +sin on its partner
    assert abs(r[0] - math.cos(1.0)) < 1e-7 and abs(r[hd // 2] - math.sin(1.0)) < 1e-7
    assert r[1] == 0 and all(r[i] == 0 for i in range(hd) if i not in (0, hd // 2))
    out = pl.rope(v, [5, 17, 300], inv)
    half = hd // 2
    assert torch.allclose(out[..., :half] ** 2 + out[..., half:] ** 2, v[..., :half] ** 2 + v[..., half:] ** 2, rtol=1e-9)
    q, k = torch.randn(1, 1, hd, dtype=F64), torch.randn(1, 1, hd, dtype=F64)
    dots = [(pl.rope(q, [m], inv) * pl.rope(k, [m - 3], inv)).sum().item() for m in (3, 10, 50)]
    assert max(dots) - min(dots) < 1e-4                                       # only the distance counts
    assert abs(dots[0] - (pl.rope(q, [3], inv) * pl.rope(k, [1], inv)).sum().item()) > 1e-3


def test_attention_reduces_to_the_library_routine():
    torch.manual_seed(0)
    T, heads, hd = 9, 2, 8
    q, k, v = (torch.randn(T, heads, hd, dtype=F64) for _ in range(3))
    got = pl.attention(q, k, v)
    ref = torch.nn.functional.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1),
                                                           is_causal=True).transpose(0, 1)
    assert torch.allclose(got, ref, rtol=1e-12, atol=1e-14)
    assert torch.equal(got[0], v[0])                                          # one key: the output is its value
    zero = pl.attention(torch.zeros_like(q), k, v)
    means = torch.cumsum(v, 0) / torch.arange(1, T + 1, dtype=F64)[:, None, None]
    assert torch.allclose(zero, means, rtol=1e-12)                            # q = 0: running mean in key order


def test_attention_groups_causality_and_window():
    torch.manual_seed(1)
    T, heads, kvh, hd = 7, 6, 2, 4
    q = torch.randn(T, heads, hd, dtype=F64)
    k, v = torch.randn(T, kvh, hd, dtype=F64), torch.randn(T, kvh, hd, dtype=F64)
    got = pl.attention(q, k, v)
    for h in range(heads):                                                    # head h reads kv head h // group
        solo = pl.attention(q[:, h:h + 1], k[:, h // 3:h // 3 + 1], v[:, h // 3:h // 3 + 1])
        assert torch.equal(got[:, h], solo[:, 0])
    k2, v2 = k.clone(), v.clone()
    k2[5:] += 1.0
    v2[5:] -= 2.0
    assert torch.equal(pl.attention(q, k2, v2)[:5], got[:5])                 # later tokens never reach back
    w = pl.attention(q, k, v, window=3)
    assert torch.equal(w[:3], got[:3]) and not torch.allclose(w[5], got[5])
    assert torch.allclose(w[6, 0], pl.attention(q[4:7, :1], k[4:7, :1], v[4:7, :1])[2, 0], rtol=1e-12)


def test_rounding_in_partitions_changes_only_where_a_weight_is_rounded():
    """Without rounding, partitions of keys are the plain formula term for term (any partition size, any shift
    of the positions, with a window); with a rounding, a sequence within one partition is the unpartitioned
    formula, and a partition whose maximum is far below the row's keeps the relative precision of its weights
    (rounded against the row's maximum they would lose it)."""
    torch.manual_seed(2)
    T, heads, hd = 150, 2, 8
    q, k, v = (torch.randn(T, heads, hd, dtype=F64) for _ in range(3))
    base = pl.attention(q, k, v)
    for part, first, window in ((64, 0, None), (64, 37, None), (16, 5, 40), (1, 0, None), (1000, 0, 7)):
        ref = base if window is None else pl.attention(q, k, v, window=window)
        got = pl.attention(q, k, v, window=window, partition=part, first_position=first)
        assert torch.allclose(got, ref, rtol=1e-11, atol=1e-13), (part, first, window)
    short = pl.attention(q[:60], k[:60], v[:60], pl.round_bf16, partition=64)
    assert torch.equal(short, pl.attention(q[:60], k[:60], v[:60], pl.round_bf16))
    assert not torch.equal(pl.attention(q[:60], k[:60], v[:60], pl.round_bf16, partition=64, first_position=30), short)
    # two keys in two partitions, the second score 20 above the first: the first key's weight is e^-20, which the
    # fold applies unrounded to a weight of exactly 1
    q1 = torch.zeros(2, 1, 1, dtype=F64)
    q1[1] = 1.0
    k1 = torch.tensor([0.0, 20.0], dtype=F64).view(2, 1, 1)
    v1 = torch.tensor([1.0, 0.0], dtype=F64).view(2, 1, 1)
    out = pl.attention(q1, k1, v1, pl.round_bf16, partition=1)[1, 0, 0].item()
    exact = math.exp(-20.0) / (1.0 + math.exp(-20.0))
    assert abs(out - exact) < 1e-15 * exact + 1e-22
    rough = pl.attention(q1, k1, v1, pl.round_bf16)[1, 0, 0].item()
    assert abs(rough - exact) > 1e-4 * exact


def test_swiglu():
    g, u = torch.tensor([0.0, 40.0, -40.0, 1.5], dtype=F64), torch.tensor([3.0, 2.0, 2.0, -1.0], dtype=F64)
    out = pl.swiglu(g, u)
    assert out[0] == 0 and abs(out[1] - 80.0) < 1e-12 and abs(out[2]) < 1e-14
    assert torch.allclose(out, torch.nn.functional.silu(g) * u, rtol=1e-14)


@pytest.mark.parametrize("cfg", [TINY_A, TINY_B])
def test_whole_model_structure(cfg):
    """Tied head is the embedding; logits at a position do not depend on later tokens; a shift
    of all positions changes nothing but rounding of the 32-bit angles."""
    from bitwise_amd.model import describe
    from bitwise_amd.weights.loader import random_tensors

    w = dict(random_tensors(describe(cfg), 3, 0.05))
    toks = [(i * 31 + 5) % 97 for i in range(12)]
    base = pl.forward(cfg, w, toks)
    assert base.shape == (12, cfg["vocab_size"])
    other = pl.forward(cfg, w, toks[:8] + [1, 2, 3, 4])
    assert torch.equal(base[:8], other[:8]) and not torch.allclose(base[8:], other[8:])
    shifted = pl.forward(cfg, w, toks, first_position=40)
    assert (shifted - base).abs().max() < 1e-4 * base.abs().max()
    if cfg["tie_word_embeddings"]:
        w2 = dict(w)
        w2["lm_head.weight"] = torch.zeros_like(w["model.embed_tokens.weight"])
        assert torch.equal(pl.forward(cfg, w2, toks), base)                  # a stray head tensor is not used
    else:
        w2 = dict(w)
        w2["lm_head.weight"] = w["lm_head.weight"] * 2
        assert torch.allclose(pl.forward(cfg, w2, toks), base * 2, rtol=1e-12)


def test_residual_and_norm_placement():
    """Pre-norm: with all projections zero the residual stream is the embedding itself, so the
    logits are head @ rmsnorm(embedding); a post-norm or a norm on the residual would differ."""
    from bitwise_amd.model import describe
    from bitwise_amd.weights.loader import random_tensors

    w = {k: v.clone() for k, v in random_tensors(describe(TINY_B), 4, 0.05)}
    for k in w:
        if "o_proj" in k or "down_proj" in k:
            w[k].zero_()
    toks = [5, 9, 200]
    x = pl.embed(toks, w["model.embed_tokens.weight"])
    want = pl.linear(pl.rmsnorm(x, w["model.norm.weight"], 1e-6), w["lm_head.weight"])
    assert torch.allclose(pl.forward(TINY_B, w, toks), want, rtol=1e-13)


def test_constants_and_sampling():
    assert pl.mix64(0x9E3779B97F4A7C15) == 0xE220A8397B1DCDAF          # first output of splitmix64 seeded with 0
    # the chain: another parent, another token or another order gives another hash
    hashes = {pl.block_hash(0, [1, 2, 3]), pl.block_hash(1, [1, 2, 3]), pl.block_hash(0, [1, 3, 2]), pl.block_hash(0, [1, 2]),
              pl.block_hash(pl.block_hash(0, [1, 2, 3]), [1, 2, 3])}
    assert len(hashes) == 5
    # the reference's basis is the FNV-1a offset 14695981039346656037 without its last digit
    # (src/block_manager.cpp:10, src/engine.h:68); its text is followed, not the FNV standard
    assert 1469598103934665603 == 0xCBF29CE484222325 // 10 and 1099511628211 == 0x100000001B3
    assert pl.block_hash(0, []) == ((lambda h: (h ^ (h >> 33)))(((1469598103934665603 ^ (1469598103934665603 >> 33))
                                    * 0xff51afd7ed558ccd) & (2 ** 64 - 1)))
    us = [pl.counter_uniform(s, p, 0) for s in (0, 1, 2 ** 63) for p in (0, 1, 1000)]
    assert all(0.0 <= u < 1.0 for u in us) and len(set(us)) == len(us)
    assert pl.counter_uniform(7, 11, 0) == pl.counter_uniform(7, 11, 0) != pl.counter_uniform(7, 11, 1)
    row = np.array([0.5, 2.0, 2.0, -1.0], np.float32)
    assert pl.argmax_row(row) == 1                                       # ties: the first maximum
    assert pl.sample_row(row, 1.0, 0.0) == 0                             # u = 0: the first token with weight
    assert pl.sample_row(row, 1.0, 1.0 - 2 ** -53) == 3                  # u -> 1: the last
    w = np.exp((row - 2.0).astype(np.float64))
    cdf = np.cumsum(w) / w.sum()
    for u in (0.05, 0.3, 0.6, 0.97):
        assert pl.sample_row(row, 1.0, u) == int(np.searchsorted(cdf, u, side="right"))
    cold = [pl.sample_row(row, 0.05, u) for u in np.linspace(0.01, 0.99, 25)]
    assert set(cold) <= {1, 2}                                           # low temperature: only the maxima
    h1 = pl.hash_floats(1469598103934665603, np.array([1.0, 2.0, 3.0], np.float32))
    assert h1 != pl.hash_floats(1469598103934665603, np.array([1.0, 2.0, 3.0000002], np.float32))


# ----------------------------------------------------------------------------- the scalar 32-bit decoder

def test_scalar_decoder_agrees_with_the_float64_one():
    """Two transcriptions of the same formulas, in different languages and precisions: what one gets wrong
    (a pairing, an order, a transposed weight) the other must get wrong the same way to pass."""
    import plain_scalar as ps
    from bitwise_amd.model import describe
    from bitwise_amd.weights.loader import random_tensors

    for cfg, seed, sigma in ((TINY_A, 0, 0.05), (TINY_B, 1, 0.08)):
        w = dict(random_tensors(describe(cfg), seed, sigma))
        toks = [(i * 31 + 5) % cfg["vocab_size"] for i in range(45)]
        a = ps.forward(cfg, w, toks)
        b = pl.forward(cfg, w, toks).numpy()
        assert np.abs(a - b).max() <= 2e-5 * np.abs(b).max()
        shifted = ps.forward(cfg, w, toks, first_position=9)
        assert np.abs(shifted - a).max() <= 3e-5 * np.abs(b).max()          # only distances count
        assert not np.array_equal(shifted, a)
        windowed = ps.forward(cfg, w, toks, window=11)
        assert np.array_equal(windowed[:11], a[:11]) and not np.array_equal(windowed[11:], a[11:])


def test_scalar_primitives():
    import plain_scalar as ps

    assert ps.expf([0.0])[0] == np.float32(1.0)                            # one key: its value, exactly
    edge = ps.expf([-87.5, -1e30, 89.5, float("inf"), float("-inf")])
    assert list(edge[:2]) == [0.0, 0.0] and np.isinf(edge[2]) and np.isinf(edge[3]) and edge[4] == 0.0
    assert np.isnan(ps.expf([float("nan")])[0])
    x = np.linspace(-80, 80, 20001, dtype=np.float32)
    ref = np.exp(x.astype(np.float64))
    assert (np.abs(ps.expf(x).astype(np.float64) - ref) <= 2.0 * np.spacing(ref.astype(np.float32))).all()
    # the 16 chains and the tree, written out (tests/test_main.cpp:126-131), in exact arithmetic
    from fractions import Fraction
    rng = np.random.default_rng(3)
    for n in (1, 5, 16, 31, 64, 100, 128):
        a, b = rng.standard_normal(n).astype(np.float32), rng.standard_normal(n).astype(np.float32)
        lane = [np.float32(0)] * 16
        for i in range(n):
            exact = Fraction(float(a[i])) * Fraction(float(b[i])) + Fraction(float(lane[i % 16]))
            c = np.float32(float(exact))                                  # float(Fraction) rounds correctly to double;
            lane[i % 16] = c                                              # a double rounds to float32 once more: close
        s8 = [np.float32(lane[i] + lane[i + 8]) for i in range(8)]
        s4 = [np.float32(s8[i] + s8[i + 4]) for i in range(4)]
        want = np.float32(np.float32(s4[0] + s4[2]) + np.float32(s4[1] + s4[3]))
        got = ps.dot_canonical(a, b)
        assert abs(float(got) - float(want)) <= 4 * np.spacing(np.float32(abs(float(want)) + 1e-30))
    w = np.arange(12, dtype=np.float32).reshape(3, 4)
    onehot = np.zeros((1, 4), np.float32)
    onehot[0, 2] = 1
    assert np.array_equal(ps.linear(onehot, w)[0], w[:, 2])
    assert ps.swiglu([0.0], [5.0])[0] == 0.0 and ps.swiglu([30.0], [2.0])[0] == np.float32(60.0)
    y = ps.rmsnorm(np.full((1, 8), 3.0, np.float32), np.ones(8, np.float32), 0.5)
    assert np.allclose(y, 3.0 / math.sqrt(9.5), rtol=1e-6)


def test_the_scalar_decoder_under_the_compilers_memory_and_arithmetic_checks(tmp_path):
    """plain_scalar.cpp built as a program with -fsanitize=address,undefined (the reference builds its own C++
    so for its sanitizer job: CMakeLists.txt:19-22, .github/workflows/ci.yml:29-40) and run on both tiny
    configurations, one with windows: no report, and the bits of the optimised library."""
    import subprocess
    import numpy as np
    import plain_scalar as ps
    from bitwise_amd.model import describe
    from bitwise_amd.weights.loader import random_tensors
    from tiny import TINY_A, TINY_B

    exe = tmp_path / "plain_scalar_checked"
    here = Path(__file__).resolve().parent
    subprocess.run(["g++", "-std=c++17", "-O1", "-g", "-ffp-contract=off", "-fno-fast-math", "-fsanitize=address,undefined",
                    "-fno-sanitize-recover=undefined", str(here / "plain_scalar_main.cpp"), "-o", str(exe)], check=True)
    for cfg, seed, sigma, windows in ((TINY_A, 0, 0.02, [0, 0]), (TINY_B, 1, 0.05, [7, 0, 12])):
        w = dict(random_tensors(describe(cfg), seed, sigma))
        toks = [(i * 31 + 5) % cfg["vocab_size"] for i in range(23)]
        want = ps.forward(cfg, w, toks, window=windows)
        heads, H, L = cfg["num_attention_heads"], cfg["hidden_size"], cfg["num_hidden_layers"]
        hd, kvh, I, V = cfg["head_dim"], cfg["num_key_value_heads"], cfg["intermediate_size"], cfg["vocab_size"]
        cos, sin = ps.rope_tables(cfg["rope_theta"], hd, range(len(toks)))
        names = ["model.embed_tokens.weight"]
        for l in range(L):
            pre = f"model.layers.{l}."
            names += [pre + n for n in ("input_layernorm.weight", "self_attn.q_proj.weight", "self_attn.k_proj.weight",
                                        "self_attn.v_proj.weight", "self_attn.o_proj.weight", "post_attention_layernorm.weight",
                                        "mlp.gate_proj.weight", "mlp.up_proj.weight", "mlp.down_proj.weight")]
        names += ["model.norm.weight", "model.embed_tokens.weight" if cfg["tie_word_embeddings"] else "lm_head.weight"]
        case = tmp_path / "case.bin"
        with open(case, "wb") as f:
            f.write(np.asarray([len(toks), V, H, L, heads, kvh, hd, I], np.int32).tobytes())
            f.write(np.float32(cfg["rms_norm_eps"]).tobytes())
            f.write(np.asarray(windows, np.int32).tobytes() + np.asarray(toks, np.int32).tobytes())
            f.write(np.ascontiguousarray(cos, np.float32).tobytes() + np.ascontiguousarray(sin, np.float32).tobytes())
            for n in names:
                f.write(w[n].float().numpy().astype("<f4").tobytes())
        out = tmp_path / "logits.bin"
        p = subprocess.run([str(exe), str(case), str(out)], capture_output=True, text=True, timeout=300)
        assert p.returncode == 0 and not p.stderr.strip(), (p.returncode, p.stderr[-3000:])
        got = np.fromfile(out, dtype="<f4").reshape(len(toks), V)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
