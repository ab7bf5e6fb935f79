"""The 32-bit path against the plain scalar 32-bit decoder (plain_scalar.cpp), bit for bit: each
kernel alone over a grid of shapes (the reference proves vector == scalar the same way,
tests/test_main.cpp:70-93, :122-135), and the whole model's logits at every position."""

import numpy as np
import pytest
import torch

import plain_scalar as ps
import tiny
from bitwise_amd.csrc import ops

pytestmark = pytest.mark.gpu


def bits(a) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(a, dtype=np.float32)).view(np.uint32)


def test_matrix_product_over_the_reference_grid(gpu):
    """m x n x k of tests/test_main.cpp:74-77 (its bias axis does not exist here), 32-bit and bfloat16
    weights, plain store and residual add: every output is the one k-ascending chain."""
    g = torch.Generator().manual_seed(4)
    for wdt in (torch.float32, torch.bfloat16):
        for M in (1, 2, 3, 4, 5, 7, 13, 50):
            for N in (1, 15, 16, 17, 100, 300):
                for K in (1, 16, 33, 64, 600):
                    x = torch.randn(M, K, generator=g)
                    w = (torch.randn(N, K, generator=g) * 0.3).to(wdt)
                    want = ps.linear(x.numpy(), w.float().numpy())
                    y = torch.zeros(M, N, device=gpu)
                    ops.gemm_f32(x.to(gpu), w.to(gpu), y, M)
                    assert np.array_equal(bits(y.cpu().numpy()), bits(want)), (wdt, M, N, K)
                    if (M, N) in ((1, 17), (5, 100), (50, 300)):
                        res = torch.randn(M, N, generator=g)
                        y = res.clone().to(gpu)
                        ops.gemm_f32(x.to(gpu), w.to(gpu), y, M, accumulate=True)
                        assert np.array_equal(bits(y.cpu().numpy()), bits(res.numpy() + want)), ("add", wdt, M, N, K)


def test_matrix_product_at_layer_widths(gpu):
    """The routes long chains take (K = 2048 and 8192, one to 64 rows and a prompt portion's tiles)."""
    g = torch.Generator().manual_seed(5)
    for M, N, K in [(1, 40, 2048), (3, 24, 8192), (20, 33, 2048), (48, 16, 8192), (130, 140, 2048)]:
        x = torch.randn(M, K, generator=g)
        w = (torch.randn(N, K, generator=g) * 0.05).to(torch.bfloat16)
        y = torch.zeros(M, N, device=gpu)
        ops.gemm_f32(x.to(gpu), w.to(gpu), y, M)
        assert np.array_equal(bits(y.cpu().numpy()), bits(ps.linear(x.numpy(), w.float().numpy()))), (M, N, K)


def test_matrix_product_on_the_matrix_cores_is_the_same_chain(gpu):
    """17 to 64 rows and prompt portions run their chains as 32-bit matrix instructions of one step of k each:
    shapes around the kernels' tile edges, 32-bit and bfloat16 weights, store and residual add, against std::fma."""
    g = torch.Generator().manual_seed(15)
    shapes = [(17, 33, 64), (24, 16, 128), (32, 100, 192), (33, 17, 64), (64, 130, 256), (48, 64, 2048),
              (65, 1, 32), (100, 129, 96), (128, 128, 64), (129, 300, 160), (300, 257, 2048), (200, 40, 8192)]
    for wdt in (torch.bfloat16, torch.float32):
        for M, N, K in shapes:
            x = torch.randn(M, K, generator=g)
            x[0, :5] = torch.tensor([0.0, -0.0, 1e-30, -1e-38, 3e38])        # zeros, a tiny and a huge element
            w = (torch.randn(N, K, generator=g) * 0.2).to(wdt)
            want = ps.linear(x.numpy(), w.float().numpy())
            y = torch.zeros(M, N, device=gpu)
            ops.gemm_f32(x.to(gpu), w.to(gpu), y, M)
            same = (bits(y.cpu().numpy()) == bits(want)) | (np.isnan(want) & np.isnan(y.cpu().numpy()))
            assert same.all(), (wdt, M, N, K, int((~same).sum()))
            res = torch.randn(M, N, generator=g)
            y = res.clone().to(gpu)
            ops.gemm_f32(x.to(gpu), w.to(gpu), y, M, accumulate=True)
            want_add = res.numpy() + want
            same = (bits(y.cpu().numpy()) == bits(want_add)) | (np.isnan(want_add) & np.isnan(y.cpu().numpy()))
            assert same.all(), ("add", wdt, M, N, K)


def test_rmsnorm_bits(gpu):
    g = torch.Generator().manual_seed(6)
    for rows, dim, eps in [(1, 1, 1e-5), (3, 5, 1e-6), (4, 16, 1e-5), (2, 31, 0.5), (5, 64, 1e-5), (3, 96, 1e-6),
                           (2, 100, 1e-5), (7, 2048, 1e-5), (2, 4100, 1e-5)]:
        x = torch.randn(rows, dim, generator=g) * 3
        w = 1 + 0.1 * torch.randn(dim, generator=g)
        y = torch.zeros(rows, dim, device=gpu)
        ops.rmsnorm(x.to(gpu), w.to(gpu), y, rows, eps)
        assert np.array_equal(bits(y.cpu().numpy()), bits(ps.rmsnorm(x.numpy(), w.numpy(), eps))), (rows, dim)


def test_swiglu_and_the_exponential_bits(gpu):
    """g * (1/(1+exp(-g))) * u over arguments that reach both ends of the exponential's range, its ties
    of the integer rounding, zero, infinities and NaN."""
    g = torch.Generator().manual_seed(7)
    gate = torch.cat([torch.randn(3000, generator=g) * 4, torch.linspace(-120, 120, 4001),
                      torch.tensor([0.0, -0.0, 87.0, -87.0, 87.00001, 88.7, 88.8, 89.5, -89.5, 1e30, -1e30,
                                    float("inf"), float("-inf"), float("nan")]),
                      (torch.arange(-130, 130).float() + 0.5) * 0.6931472])
    inter = gate.numel()
    up = torch.randn(inter, generator=g)
    gu = torch.cat([gate, up]).view(1, 2 * inter).to(gpu)
    h = torch.zeros(1, inter, device=gpu)
    ops.swiglu_f32(gu, h, 1)
    want = ps.swiglu(gate.numpy(), up.numpy())
    got = h.cpu().numpy()[0]
    same = (bits(got) == bits(want)) | (np.isnan(got) & np.isnan(want))
    assert same.all(), f"first difference at g = {gate[int(np.argmin(same))].item()}"
    # the plain exponential itself: against the library's in double, within 2 units of the last place
    x = np.linspace(-86.9, 88.7, 200001, dtype=np.float32)
    e = ps.expf(x).astype(np.float64)
    ref = np.exp(x.astype(np.float64))
    assert (np.abs(e - ref) <= 2.0 * np.spacing(ref.astype(np.float32)).astype(np.float64)).all()


@pytest.mark.parametrize("heads,kvh,hd,page,window", [(4, 2, 16, 16, 0), (3, 1, 32, 8, 0), (2, 2, 64, 16, 37),
                                                      (2, 1, 128, 16, 0), (5, 5, 80, 32, 0)])
def test_attention_bits(gpu, heads, kvh, hd, page, window):
    """Decoded tokens and prompt tiles over a paged cache with a permuted table against the scalar two-pass
    attention over the contiguous keys."""
    from test_kernels_gpu import paged_setup, run_attention

    n = 333
    pages = n // page + 6
    while pages % 7 == 0:
        pages += 1
    k, v, kc, vc, tab = paged_setup(gpu, False, heads, kvh, hd, page, pages, n, seed=9, poison=True)
    g = torch.Generator().manual_seed(10)
    q_all = torch.randn(n, heads, hd, generator=g)
    want = ps.attention(q_all.numpy(), k.numpy(), v.numpy(), window)          # every position of the sequence
    positions = [0, 1, 5, 17, 63, 64, 200, 301, 332]
    q = q_all[positions].reshape(len(positions), heads * hd)
    got = run_attention(gpu, False, q, positions, tab, kc, vc, heads, kvh, hd, page, window=window).cpu().numpy()
    for r, p in enumerate(positions):
        assert np.array_equal(bits(got[r]), bits(want[p].reshape(-1))), f"decoded token at position {p}"
    if hd <= 128:
        first = 300
        rows = list(range(first, n))
        tiles = [(i, min(16, len(rows) - i), 0, 0) for i in range(0, len(rows), 16)]
        q = q_all[rows].reshape(len(rows), heads * hd)
        got = run_attention(gpu, False, q, rows, tab, kc, vc, heads, kvh, hd, page, window=window, tiles=tiles).cpu().numpy()
        assert np.array_equal(bits(got), bits(want[rows].reshape(len(rows), -1))), "tiles of a prompt portion"


@pytest.mark.parametrize("name", ["A", "B"])
def test_whole_model_logits_are_the_scalar_decoder_s_bits(gpu, tmp_path, name):
    """Tiny A and B in 32-bit: the engine's logits at every position, whole and in portions, are the bits
    of the plain scalar decoder."""
    import bitwise_amd as bw

    folder = tiny.make_folder(tmp_path, name)
    cfg, w = tiny.read_config(folder), tiny.read_weights(folder)
    model = bw.Model.load(folder, "float32")
    g = torch.Generator().manual_seed(12)
    toks = torch.randint(0, cfg["vocab_size"], (90,), generator=g).tolist()
    want = ps.forward(cfg, w, toks)
    page = tiny.CONFIGS[name][3]
    for chunk in (None, 7, 1):
        got = model.logits(toks, chunk=chunk, block_size=page)
        same = (bits(got) == bits(want)).all(axis=1)
        assert same.all(), f"{name} chunk={chunk}: first differing position {int(np.argmin(same))}"
