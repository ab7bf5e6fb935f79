"""The checks can fail: three plausible 'optimisations' that break schedule invariance, patched in for the
test only, each of which the same comparisons that the other tests make must catch.  The reference shows
the same of its own checks: a matrix product specialised by shape (two accumulators over halves of K for
few rows, src/kernels.cpp:140-173) must differ (tests/test_main.cpp:114-117), attention that splits the
keys by shape must differ (:166-167), and a random generator keyed by the engine's step instead of the
request's position gives other tokens (README.md:86-93)."""

import numpy as np
import pytest
import torch

import bitwise_amd as bw
import tiny
from bitwise_amd.csrc import ops
from bitwise_amd.replay import Replayer
from bitwise_amd.sampling import rng
from bitwise_amd.sampling.sampler import Sampler

pytestmark = pytest.mark.gpu


def decode_and_whole(model, toks, tail, page):
    """Logits of the last ``tail`` positions: the prompt whole, and most of it whole with the tail decoded
    token by token (kernel by kernel, no graphs)."""
    n = len(toks)

    def run(steps):
        rp = Replayer("", "float32", 1024, block_size=page, model=model, use_graphs=False)
        rows = []
        for st in steps:
            lg = rp.step(st)
            if lg is not None:
                rows.append(lg)
        return np.concatenate(rows)

    whole = run([[{"id": "a", "tokens": toks, "want": list(range(n - tail, n))}]])
    steps = [[{"id": "a", "tokens": toks[:n - tail], "want": []}]]
    steps += [[{"id": "a", "tokens": [t], "want": [0]}] for t in toks[n - tail:]]
    return run(steps), whole


@pytest.fixture(scope="module")
def long_model(tmp_path_factory, gpu):
    folder = tiny.make_folder(tmp_path_factory.mktemp("neg"), "LONG")
    cfg = tiny.read_config(folder)
    g = torch.Generator().manual_seed(2)
    toks = torch.randint(0, cfg["vocab_size"], (300,), generator=g).tolist()
    return bw.Model.load(folder, "float32"), toks


def test_the_unpatched_engine_passes(long_model):
    model, toks = long_model
    dec, whole = decode_and_whole(model, toks, 24, 16)
    assert np.array_equal(dec, whole)


def test_a_matrix_product_split_over_k_for_few_rows_is_caught(long_model, monkeypatch):
    """Two chains over the halves of K, added, whenever a step has fewer than 4 rows."""
    model, toks = long_model
    real = ops.gemm_f32

    def split_k(x, w, out, rows, accumulate=False):
        K = w.shape[1]
        if rows >= 4 or K < 32:
            return real(x, w, out, rows, accumulate)
        h = K // 2
        parts = []
        for lo, hi in ((0, h), (h, K)):
            y = torch.zeros(rows, w.shape[0], device=out.device)
            real(x[:rows, lo:hi].contiguous(), w[:, lo:hi].contiguous(), y, rows)
            parts.append(y)
        total = parts[0] + parts[1]
        out[:rows] = out[:rows] + total if accumulate else total

    monkeypatch.setattr(ops, "gemm_f32", split_k)
    dec, whole = decode_and_whole(model, toks, 24, 16)
    assert not np.array_equal(dec, whole), "the cut over K went unnoticed"
    assert np.abs(dec - whole).max() < 1e-3 * np.abs(whole).max()          # (it is still a matrix product)


def test_attention_that_splits_the_keys_by_shape_is_caught(long_model, monkeypatch):
    """A decoded token with 64 keys or more folds two halves of its keys separately and merges them by their
    maxima and sums; a prompt portion walks its keys in one pass."""
    model, toks = long_model
    real = ops.attention_f32_tiles

    def split_kv(q, positions, block_table, tiles, num_tiles, tiled, k_cache, v_cache, out, heads, kv_heads, hd, page,
                 window, scale):
        if tiled:
            return real(q, positions, block_table, tiles, num_tiles, tiled, k_cache, v_cache, out, heads, kv_heads, hd,
                        page, window, scale)
        pos, tab = positions.cpu().tolist(), block_table.cpu()
        for row, _, req, _ in tiles[:num_tiles].cpu().tolist():
            p = pos[row]
            pages = tab[req, :p // page + 1].long().to(q.device)
            K = k_cache.view(-1, kv_heads, page, hd)[pages].permute(1, 0, 2, 3).reshape(kv_heads, -1, hd)[:, :p + 1]
            V = v_cache.view(-1, kv_heads, page, hd)[pages].permute(1, 0, 2, 3).reshape(kv_heads, -1, hd)[:, :p + 1]
            for h in range(heads):
                kvh = h // (heads // kv_heads)
                s = (K[kvh] @ q[row, h * hd:(h + 1) * hd]) * scale
                cuts = [(0, (p + 1) // 2), ((p + 1) // 2, p + 1)] if p + 1 >= 64 else [(0, p + 1)]
                ms, ls, os_ = [], [], []
                for lo, hi in cuts:
                    m = s[lo:hi].max()
                    e = torch.exp(s[lo:hi] - m)
                    ms.append(m), ls.append(e.sum()), os_.append(e @ V[kvh, lo:hi])
                m = torch.stack(ms).max()
                l = sum(li * torch.exp(mi - m) for li, mi in zip(ls, ms))
                o = sum(oi * torch.exp(mi - m) for oi, mi in zip(os_, ms))
                out[row, h * hd:(h + 1) * hd] = o / l

    monkeypatch.setattr(ops, "attention_f32_tiles", split_kv)
    dec, whole = decode_and_whole(model, toks, 24, 16)
    assert not np.array_equal(dec, whole), "the split over the keys went unnoticed"
    assert np.abs(dec - whole).max() < 1e-3 * np.abs(whole).max()          # (it is still attention)


def test_randomness_keyed_by_the_engine_s_step_is_caught(gpu, tmp_path, monkeypatch):
    """Uniforms drawn from (seed, how many draws the engine has made) instead of (seed, position): a request's
    tokens then depend on what else the engine has been doing."""
    folder = tiny.make_folder(tmp_path, "B")
    model = bw.Model.load(folder, "bfloat16")
    g = torch.Generator().manual_seed(6)
    prompts = [torch.randint(0, 500, (n,), generator=g).tolist() for n in (12, 30, 21)]
    params = [bw.SamplingParams(temperature=0.8, seed=s, max_new_tokens=16, ignore_eos=True) for s in range(3)]

    def run_all():
        cfg = dict(num_blocks=64, block_size=8, dtype="bfloat16")
        solo = [bw.generate(model, [p], sp, bw.EngineConfig(**cfg))[0].tokens for p, sp in zip(prompts, params)]
        crowd = [r.tokens for r in bw.generate(model, prompts, params, bw.EngineConfig(max_batched_tokens=16, **cfg))]
        return solo, crowd

    solo, crowd = run_all()
    assert solo == crowd                                                     # as it is: the same tokens

    draws = [0]

    def by_step(temperatures, seeds, positions):
        draws[0] += 1
        return np.asarray([rng.counter_uniform(s, draws[0]) if t > 0 else 0.0 for t, s in zip(temperatures, seeds)],
                          np.float64)

    monkeypatch.setattr(Sampler, "uniforms", staticmethod(by_step))
    solo, crowd = run_all()
    assert solo != crowd, "randomness keyed by the step went unnoticed"
