"""Each kernel alone against its plain reference, at sizes other than the engine's, with
inputs built so that a fault shows: a far key among hundreds, a window's edge, a page's edge,
poisoned memory that must not be read."""

from fractions import Fraction

import numpy as np
import pytest
import torch

import plain_llama as pl
from bitwise_amd.csrc import ops

pytestmark = pytest.mark.gpu
F64 = torch.float64


def f32_round(fr: Fraction) -> np.float32:
    """Round an exact rational to the nearest float32, ties to even."""
    c = np.float32(float(fr))
    best = c
    for cand in (np.nextafter(c, np.float32(-np.inf)), np.nextafter(c, np.float32(np.inf))):
        d_c, d_n = abs(Fraction(float(best)) - fr), abs(Fraction(float(cand)) - fr)
        if d_n < d_c or (d_n == d_c and (cand.view(np.uint32) & 1) == 0):
            best = cand
    return best


def fma32(a, b, c) -> np.float32:
    return f32_round(Fraction(float(a)) * Fraction(float(b)) + Fraction(float(c)))


def chain_dot(x, w) -> np.float32:
    """acc = fma(x[k], w[k], acc) for k ascending from 0.0f (src/kernels.cpp:236-244)."""
    acc = np.float32(0.0)
    for a, b in zip(x, w):
        acc = fma32(a, b, acc)
    return acc


def canonical_sumsq(x) -> np.float32:
    """16 chains lane = i % 16, then the fixed tree (src/kernels.cpp:57-64, tests/test_main.cpp:126-131)."""
    lane = [np.float32(0.0)] * 16
    for i, v in enumerate(x):
        lane[i % 16] = fma32(v, v, lane[i % 16])
    s8 = [np.float32(lane[i] + lane[i + 8]) for i in range(8)]
    s4 = [np.float32(s8[i] + s8[i + 4]) for i in range(4)]
    return np.float32(np.float32(s4[0] + s4[2]) + np.float32(s4[1] + s4[3]))


# ----------------------------------------------------------------------------- matrix products

def test_gemm_f32_is_the_scalar_chain_bit_for_bit(gpu):
    g = torch.Generator().manual_seed(1)
    for M, N, K in [(1, 1, 1), (2, 3, 33), (3, 17, 16), (5, 2, 70)]:
        x, w = torch.randn(M, K, generator=g), torch.randn(N, K, generator=g)
        y = torch.zeros(M, N, device=gpu)
        ops.gemm_f32(x.to(gpu), w.to(gpu), y, M)
        want = np.array([[chain_dot(x[m].numpy(), w[n].numpy()) for n in range(N)] for m in range(M)], np.float32)
        assert np.array_equal(y.cpu().numpy().view(np.uint32), want.view(np.uint32)), (M, N, K)


def test_gemm_f32_grid_rows_and_accumulate(gpu):
    """The reference's shape grid (tests/test_main.cpp:75-77) against float64, every row equal
    to the same row computed alone (tests/test_main.cpp:95-120), bfloat16 weights widened."""
    g = torch.Generator().manual_seed(2)
    for M in (1, 2, 3, 4, 5, 7, 13, 50):
        for N in (1, 15, 16, 17, 100, 300):
            for K in (1, 16, 33, 64, 600):
                x, w = torch.randn(M, K, generator=g).to(gpu), torch.randn(N, K, generator=g).to(gpu)
                y = torch.full((M, N), 7.0, device=gpu)
                ops.gemm_f32(x, w, y, M)
                ref = x.double() @ w.double().T
                assert (y.double() - ref).abs().max() <= 1e-6 * K ** 0.5 * ref.abs().max().clamp(min=1.0)
    x, w = torch.randn(9, 1024, generator=g).to(gpu), torch.randn(200, 1024, generator=g).to(gpu)
    wb = w.bfloat16()
    batch, one = torch.zeros(9, 200, device=gpu), torch.zeros(1, 200, device=gpu)
    for weight in (w, wb):
        ops.gemm_f32(x, weight, batch, 9)
        for r in range(9):
            ops.gemm_f32(x[r:r + 1].contiguous(), weight, one, 1)
            assert torch.equal(one[0], batch[r])
    assert torch.allclose(batch.double(), x.double() @ wb.double().T, rtol=0, atol=1e-4)
    before = batch.clone()
    ops.gemm_f32(x, wb, batch, 9, accumulate=True)
    assert torch.equal(batch, before + before)                     # y + acc, one addition per output
    # prompt portions (128 x 128 tiles, or 64 x 64 where K is no multiple of 16): a row's bits are those of the row alone
    # (and 17 to 64 rows: the chain-per-thread kernel with two or four blocks of rows)
    for M, N, K in [(150, 200, 1024), (129, 130, 64), (300, 77, 48), (70, 140, 1000), (40, 130, 1024), (20, 77, 264),
                    (64, 50, 136), (33, 16, 8)]:
        x, w = torch.randn(M, K, generator=g).to(gpu), torch.randn(N, K, generator=g).to(gpu)
        for weight in (w, w.bfloat16()):
            batch, one = torch.full((M, N), 3.0, device=gpu), torch.zeros(1, N, device=gpu)
            ops.gemm_f32(x, weight, batch, M)
            assert (batch.double() - x.double() @ weight.double().T).abs().max() <= 1e-6 * K ** 0.5 * batch.abs().max()
            for r in sorted({0, min(63, M - 1), min(64, M - 1), M // 2, M - 1}):
                ops.gemm_f32(x[r:r + 1].contiguous(), weight, one, 1)
                assert torch.equal(one[0], batch[r]), (M, N, K, r)
            before = batch.clone()
            ops.gemm_f32(x, weight, batch, M, accumulate=True)
            assert torch.equal(batch, before + before)
    # many columns and up to 16 rows (a wave a row, weights packed in LDS; up to 8 rows with loader waves and the row
    # four elements a register): the bits of the same rows inside a product of 20 rows (matrix cores) and of the
    # chain-per-thread kernel (K + 8 is no whole stage of the first)
    for M, N, K in [(1, 16400, 64), (8, 16384, 2048), (16, 20000, 128), (5, 16385, 192), (13, 16500, 96), (3, 16390, 128),
                    (7, 16384, 320), (2, 17000, 64), (9, 16384, 64)]:
        x, w = torch.randn(20, K + 8, generator=g).to(gpu), (torch.randn(N, K + 8, generator=g) * 0.1).to(gpu)
        for weight in (w, w.bfloat16()):
            xs, ws = x[:, :K].contiguous(), weight[:, :K].contiguous()
            few, many = torch.full((M, N), 3.0, device=gpu), torch.zeros(20, N, device=gpu)
            ops.gemm_f32(xs[:M].contiguous(), ws, few, M)
            ops.gemm_f32(xs, ws, many, 20)
            assert torch.equal(few, many[:M]), (M, N, K, weight.dtype)
            before = few.clone()
            ops.gemm_f32(xs[:M].contiguous(), ws, few, M, accumulate=True)
            assert torch.equal(few, before + before)
            # the longer rows through the other kernel: zeros in the last 8 places of x leave every chain's value
            xz = x[:M].clone()
            xz[:, K:] = 0.0
            longer = torch.zeros(M, N, device=gpu)
            ops.gemm_f32(xz, weight, longer, M)
            assert torch.equal(longer, before), (M, N, K, weight.dtype)


def test_gemm_bf16_rows_shapes_and_epilogues(gpu):
    g = torch.Generator().manual_seed(3)
    for M, N, K in [(1, 16, 32), (5, 100, 64), (16, 64, 96), (17, 500, 96), (50, 300, 608), (130, 96, 224), (33, 72, 40),
                    (40, 4100, 192), (64, 4200, 2048), (17, 4096, 64), (9, 4100, 128), (16, 5000, 64), (30, 4096, 320),   # many columns: x shared through LDS
                    (7, 200, 4160), (16, 5000, 4096), (3, 40, 128), (12, 4104, 6144),   # up to 16 rows streaming through LDS, several segments
                    (50, 1030, 128), (20, 2048, 256),   # 17 to 64 rows, one segment, few columns: narrow tiles for the residual add
                    (130, 96, 256), (200, 300, 1024), (129, 130, 2048),   # wide tiles, K in whole double steps
                    (130, 2048, 256), (500, 2100, 128), (65, 1030, 64), (320, 1024, 2048),   # a residual add of one segment: all blocks of 64 rows in one launch
                    (2100, 2100, 128),                                    # more than 256 tiles: four waves a tile
                    (3, 40, 4096), (8, 64, 8192), (70, 80, 4160), (40, 48, 6144), (150, 200, 4096),
                    (8, 4096, 14336), (5, 2050, 10240), (3, 1000, 16384), (7, 4100, 9280),   # five to eight segments, up to 8 rows: a wave a segment
                    (8, 4096, 4096), (6, 3000, 2112), (9, 4096, 14336),   # one or two segments: half strips; more than 8 rows with seven segments
                    (129, 96, 6144)]:                                     # several 2048-segments of K
        x = torch.randn(M, K, generator=g).bfloat16().to(gpu)
        w = torch.randn(N, K, generator=g).bfloat16().to(gpu)
        y = torch.full((M, N), 3.0, device=gpu)
        ops.gemm_bf16(x, w, y, M, ops.EPI_F32)
        ref = x.double() @ w.double().T
        assert (y.double() - ref).abs().max() <= 2e-6 * K ** 0.5 * ref.abs().max()
        one = torch.zeros(1, N, device=gpu)
        for r in range(0, M, max(1, M // 7)):                      # the skinny and the wide kernel agree bit for bit
            ops.gemm_bf16(x[r:r + 1].contiguous(), w, one, 1, ops.EPI_F32)
            assert torch.equal(one[0], y[r]), (M, N, K, r)
        yb = torch.zeros(M, N, device=gpu, dtype=torch.bfloat16)
        ops.gemm_bf16(x, w, yb, M, ops.EPI_BF16)
        assert torch.equal(yb, y.bfloat16())
        res = torch.randn(M, N, generator=g).to(gpu)
        acc = res.clone()
        ops.gemm_bf16(x, w, acc, M, ops.EPI_ADD_F32)
        want = res.clone()                                         # the chain of segment sums starts at the residual
        for k0 in range(0, K, 2048):
            part = torch.zeros(M, N, device=gpu)
            ops.gemm_bf16(x[:, k0:k0 + 2048].contiguous(), w[:, k0:k0 + 2048].contiguous(), part, M, ops.EPI_F32)
            want = want + part
        assert torch.equal(acc, want), (M, N, K)
    # enough 256 x 256 tiles for the big-tile kernel: the bits of the same rows in slices that other kernels take
    # (3696 columns: SwiGLU outputs of whole 16-byte pieces, which leave that kernel through LDS a row at a time)
    for M, N, K in ((2100, 3700, 192), (2100, 3696, 192)):
        x = torch.randn(M, K, generator=g).bfloat16().to(gpu)
        w = torch.randn(N, K, generator=g).bfloat16().to(gpu)
        y = torch.full((M, N), 3.0, device=gpu)
        ops.gemm_bf16(x, w, y, M, ops.EPI_F32)
        ref = x.double() @ w.double().T
        assert (y.double() - ref).abs().max() <= 2e-6 * K ** 0.5 * ref.abs().max()
        for lo, n in ((0, 300), (1800, 300), (2047, 53), (2099, 1)):
            part = torch.zeros(n, N, device=gpu)
            ops.gemm_bf16(x[lo:lo + n].contiguous(), w, part, n, ops.EPI_F32)
            assert torch.equal(part, y[lo:lo + n]), (lo, n)
        yb = torch.zeros(M, N, device=gpu, dtype=torch.bfloat16)
        ops.gemm_bf16(x, w, yb, M, ops.EPI_BF16)
        assert torch.equal(yb, y.bfloat16())
        inter = N // 2
        hb = torch.zeros(M, inter, device=gpu, dtype=torch.bfloat16)
        ops.gemm_bf16(x, w, hb, M, ops.EPI_SWIGLU_BF16)
        for lo, n in ((0, 300), (1900, 200), (2090, 10)):
            part = torch.zeros(n, inter, device=gpu, dtype=torch.bfloat16)
            ops.gemm_bf16(x[lo:lo + n].contiguous(), w, part, n, ops.EPI_SWIGLU_BF16)
            assert torch.equal(part, hb[lo:lo + n]), (lo, n)
    # a residual add of 17 to 64 rows over several segments of K with scratch: a workgroup per tile and segment; the
    # bits of the add without scratch, twice in a row on the same scratch (full of NaN at first), counters zero after
    for M, N, K in [(64, 2048, 8192), (23, 800, 2048 * 2 + 320), (40, 1100, 4096)]:
        x = torch.randn(M, K, generator=g).bfloat16().to(gpu)
        w = (torch.randn(N, K, generator=g) * 0.05).bfloat16().to(gpu)
        res = torch.randn(M, N, generator=g).to(gpu)
        want = res.clone()
        ops.gemm_bf16(x, w, want, M, ops.EPI_ADD_F32)
        floats, counters = ops.gemm_add_scratch(M, N, K)
        assert floats > 0 and counters > 0 and ops.gemm_add_scratch(8, N, K) == (0, 0)
        scratch = (torch.full((floats,), float("nan"), device=gpu), torch.zeros(counters, dtype=torch.int32, device=gpu))
        for _ in range(2):
            got = res.clone()
            ops.gemm_bf16(x, w, got, M, ops.EPI_ADD_F32, scratch=scratch)
            assert torch.equal(got, want) and not scratch[1].any(), (M, N, K)
    # a residual add of more than 64 rows whose 128 x 128 tiles with all of K would leave compute units idle: up to
    # 128 rows and three segments in blocks of 64 rows through that kernel (its scratch if K has several segments);
    # else a workgroup per tile (128 x 128, 128 x 256, or 256 x 256 from 512 rows) and segment, the segments' sums whole in
    # scratch and joined in order afterwards; or 128 x 256 tiles with all of K where those go round the compute units
    # once (no scratch).  The bits of the rows alone, 16 at a time, with and without scratch,
    # twice on the same scratch (full of NaN at first, larger than needed); ragged edges, a short last segment
    S = lambda K: (K + 2047) // 2048
    # ("at once": up to 512 workgroups of the 64-row kernel, a block of 64 rows, a tile of columns and a segment each, in
    # one launch; their scratch is the same size whatever the shape)
    for M, N, K, kind in [(65, 2048, 4096, "at once"), (128, 1100, 2048 * 2 + 320, "at once"), (100, 2048, 2048, None),
                          (129, 2048, 2048, None), (81, 2048, 4096 + 72, None), (640, 4096, 4096, None),
                          (2048, 4096, 4096, None),       # 128 x 256 tiles, the two segments joined in registers
                          (65, 2048, 8192, "at once"), (145, 2048, 8192, "at once"), (300, 1000, 2 * 2048 + 192, "at once"),
                          (256, 2048, 8192, "at once"), (320, 2048, 8192, "sums"),
                          (768, 2048, 8192, "sums"), (700, 3000, 4 * 2048 + 128, "sums"), (2048, 2048, 8192, "sums"),
                          (1000, 2000, 8128, "sums"),     # 128 x 256 tiles, a workgroup per tile and segment

                          (513, 8192, 4096, "sums")]:
        x = torch.randn(M, K, generator=g).bfloat16().to(gpu)
        w = (torch.randn(N, K, generator=g) * 0.05).bfloat16().to(gpu)
        res = torch.randn(M, N, generator=g).to(gpu)
        want = res.clone()
        for lo in range(0, M, 16):
            n = min(16, M - lo)
            part = res[lo:lo + n].clone()
            ops.gemm_bf16(x[lo:lo + n].contiguous(), w, part, n, ops.EPI_ADD_F32)
            want[lo:lo + n] = part
        got = res.clone()
        ops.gemm_bf16(x, w, got, M, ops.EPI_ADD_F32)
        assert torch.equal(got, want), (M, N, K)
        floats, counters = ops.gemm_add_scratch(M, N, K)
        if kind == "sums":
            assert (floats, counters) == (S(K) * M * N, 1), (M, N, K)
        elif kind == "at once":
            assert (floats, counters) == (512 * 4096, 512), (M, N, K)
        else:
            assert (floats, counters) == (0, 0), (M, N, K)
        if floats:
            scratch = (torch.full((floats + 1000,), float("nan"), device=gpu), torch.zeros(counters, dtype=torch.int32, device=gpu))
            for _ in range(2):
                got = res.clone()
                ops.gemm_bf16(x, w, got, M, ops.EPI_ADD_F32, scratch=scratch)
                assert torch.equal(got, want) and not scratch[1].any(), (M, N, K)
            if kind == "sums":
                with pytest.raises(RuntimeError, match="scratch smaller"):
                    ops.gemm_bf16(x, w, got, M, ops.EPI_ADD_F32, scratch=(scratch[0][:floats - 8], scratch[1]))
    assert ops.gemm_add_scratch(2048, 2048, 2048) == (0, 0)
    # SwiGLU with many columns (x shared through LDS; one, two or four blocks of 16 rows): the plain result, and
    # the bits of the same rows inside a prompt portion's product (another kernel)
    for inter, K in ((2100, 128), (2100, 2048 + 128)):             # the second: two segments of K
        wgu = (torch.randn(2 * inter, K, generator=g) * (0.5 if K > 2048 else 1.0)).bfloat16().to(gpu)
        xl = torch.randn(200, K, generator=g).bfloat16().to(gpu)
        big = torch.zeros(200, inter, device=gpu, dtype=torch.bfloat16)
        ops.gemm_bf16(xl, wgu, big, 200, ops.EPI_SWIGLU_BF16)
        gate, up = xl.double() @ wgu[:inter].double().T, xl.double() @ wgu[inter:].double().T
        want = pl.swiglu(gate.cpu(), up.cpu())
        assert (big.cpu().double() - want).abs().max() <= 2 ** -8 * want.abs().max()
        for M in (1, 13, 16, 29, 41, 64):
            hb = torch.zeros(M, inter, device=gpu, dtype=torch.bfloat16)
            ops.gemm_bf16(xl[100:100 + M].contiguous(), wgu, hb, M, ops.EPI_SWIGLU_BF16)
            assert torch.equal(hb, big[100:100 + M]), (M, K)
    # enough 128 x 128 tiles for two rounds of the compute units and few enough 128 x 256 tiles for one: those run
    # (plain and SwiGLU epilogues, two segments of K joined in registers, ragged last tiles of rows and columns);
    # the plain result, and the bits of the rows 16 at a time (other kernels)
    M, N, K = 300, 11000, 2048 + 192
    w = (torch.randn(N, K, generator=g) * 0.05).bfloat16().to(gpu)
    xl = torch.randn(M, K, generator=g).bfloat16().to(gpu)
    for dt, e, cols in ((torch.float32, ops.EPI_F32, N), (torch.bfloat16, ops.EPI_BF16, N), (torch.bfloat16, ops.EPI_SWIGLU_BF16, N // 2)):
        y = torch.zeros(M, cols, device=gpu, dtype=dt)
        ops.gemm_bf16(xl, w, y, M, e)
        for lo in (0, 64, 128, 250, 288):
            n = min(16, M - lo)
            part = torch.zeros(n, cols, device=gpu, dtype=dt)
            ops.gemm_bf16(xl[lo:lo + n].contiguous(), w, part, n, e)
            assert torch.equal(part, y[lo:lo + n]), (lo, e)
        if e == ops.EPI_SWIGLU_BF16:
            gate, up = xl.double() @ w[:N // 2].double().T, xl.double() @ w[N // 2:].double().T
            ref = gate * torch.sigmoid(gate) * up
        else:
            ref = xl.double() @ w.double().T
        assert (y.double() - ref).abs().max() <= 2 ** -7 * ref.abs().max() + 1e-3, e
    M, inter, K = 19, 56, 96
    x = torch.randn(M, K, generator=g).bfloat16().to(gpu)
    wgu = torch.randn(2 * inter, K, generator=g).bfloat16().to(gpu)
    h = torch.zeros(M, inter, device=gpu, dtype=torch.bfloat16)
    ops.gemm_bf16(x, wgu, h, M, ops.EPI_SWIGLU_BF16)
    gate, up = x.double() @ wgu[:inter].double().T, x.double() @ wgu[inter:].double().T
    want = pl.swiglu(gate.cpu(), up.cpu())
    assert (h.cpu().double() - want).abs().max() <= 2 ** -8 * want.abs().max()     # one bfloat16 rounding
    with pytest.raises(ValueError, match="multiple of 8"):
        ops.gemm_bf16(torch.zeros(2, 12, device=gpu, dtype=torch.bfloat16),
                      torch.zeros(4, 12, device=gpu, dtype=torch.bfloat16), torch.zeros(2, 4, device=gpu), 2, ops.EPI_F32)


def test_gemm_bf16_random_shapes(gpu):
    """Which kernel runs is a matter of the shape: shapes drawn at random (edges of the row blocks, of the strips,
    of the segments of K) through every epilogue, against float64 and, bit for bit, against the same rows alone."""
    import random
    rnd = random.Random(11)
    g = torch.Generator().manual_seed(12)
    ms = [1, 2, 7, 15, 16, 17, 31, 32, 33, 48, 63, 64, 65, 100, 127, 128, 129, 255, 256, 300, 511, 512, 513, 700]
    ns = [8, 16, 24, 40, 64, 72, 128, 136, 200, 256, 264, 1000, 1024, 2048, 2056, 4096, 4104]
    ks = [8, 32, 64, 72, 128, 192, 320, 1024, 2048, 2056, 2112, 4096, 4160]
    done = 0
    while done < 90:
        M, N, K, epi = rnd.choice(ms), rnd.choice(ns), rnd.choice(ks), rnd.choice(["f32", "bf16", "add", "swiglu"])
        if M * N > 1_500_000 or N * K > 9_000_000:
            continue
        done += 1
        x = torch.randn(M, K, generator=g).bfloat16().to(gpu)
        w = (torch.randn(N, K, generator=g) * (0.3 if epi == "swiglu" else 1.0)).bfloat16().to(gpu)
        rows = sorted({0, M - 1, M // 2, min(15, M - 1), min(16, M - 1), min(64, M - 1)})
        what = (M, N, K, epi)
        if epi == "swiglu":
            out = torch.zeros(M, N // 2, device=gpu, dtype=torch.bfloat16)
            one = torch.zeros(1, N // 2, device=gpu, dtype=torch.bfloat16)
            ops.gemm_bf16(x, w, out, M, ops.EPI_SWIGLU_BF16)
            for r in rows:
                ops.gemm_bf16(x[r:r + 1].contiguous(), w, one, 1, ops.EPI_SWIGLU_BF16)
                assert torch.equal(one[0], out[r]), (what, r)
            gate, up = x.double() @ w[:N // 2].double().T, x.double() @ w[N // 2:].double().T
            ref = gate * torch.sigmoid(gate) * up
            assert (out.double() - ref).abs().max() <= 2 ** -7 * ref.abs().max() + 1e-3, what
            continue
        ref = x.double() @ w.double().T
        if epi == "add":
            res = torch.randn(M, N, generator=g).to(gpu)
            out, one = res.clone(), torch.zeros(1, N, device=gpu)
            ops.gemm_bf16(x, w, out, M, ops.EPI_ADD_F32)
            floats, counters = ops.gemm_add_scratch(M, N, K)
            if floats:
                scratch = (torch.full((floats,), float("nan"), device=gpu), torch.zeros(counters, dtype=torch.int32, device=gpu))
                again = res.clone()
                ops.gemm_bf16(x, w, again, M, ops.EPI_ADD_F32, scratch=scratch)
                assert torch.equal(again, out), what
            for r in rows:
                one.copy_(res[r:r + 1])
                ops.gemm_bf16(x[r:r + 1].contiguous(), w, one, 1, ops.EPI_ADD_F32)
                assert torch.equal(one[0], out[r]), (what, r)
            assert (out.double() - res.double() - ref).abs().max() <= 3e-6 * K ** 0.5 * ref.abs().max() + 1e-4, what
            continue
        dt, e = (torch.float32, ops.EPI_F32) if epi == "f32" else (torch.bfloat16, ops.EPI_BF16)
        out, one = torch.zeros(M, N, device=gpu, dtype=dt), torch.zeros(1, N, device=gpu, dtype=dt)
        ops.gemm_bf16(x, w, out, M, e)
        for r in rows:
            ops.gemm_bf16(x[r:r + 1].contiguous(), w, one, 1, e)
            assert torch.equal(one[0], out[r]), (what, r)
        assert (out.double() - ref).abs().max() <= (3e-6 * K ** 0.5 if epi == "f32" else 2 ** -8) * ref.abs().max() + 1e-4, what


def test_gemm_bf16_weight_beyond_two_gib(gpu):
    """A weight of more than 2^31 bytes (a large vocabulary's head): every kernel addresses W through descriptors
    of a tile's rows, so only the tile has to fit 32-bit offsets.  The first and last columns equal the product
    with those rows of W alone, for a decode step, a short portion and a long one."""
    N, K = 270000, 4096                                            # 2.2 GB
    g = torch.Generator(device=gpu).manual_seed(3)
    w = (torch.randn(N, K, device=gpu, generator=g) * 0.05).bfloat16()
    for M in (3, 40, 300):
        x = torch.randn(M, K, device=gpu, generator=g).bfloat16()
        y = torch.zeros(M, N, device=gpu)
        ops.gemm_bf16(x, w, y, M, ops.EPI_F32)
        for lo in (0, N - 200):
            part = torch.zeros(M, 200, device=gpu)
            ops.gemm_bf16(x, w[lo:lo + 200].contiguous(), part, M, ops.EPI_F32)
            assert torch.equal(part, y[:, lo:lo + 200]), (M, lo)
        ref = x[:, :].double() @ w[N - 200:].double().T
        assert (y[:, N - 200:].double() - ref).abs().max() <= 2e-6 * K ** 0.5 * ref.abs().max()


# ----------------------------------------------------------------------------- row kernels

def test_rmsnorm(gpu):
    g = torch.Generator().manual_seed(4)
    for rows, dim, eps in [(1, 1, 1e-5), (3, 33, 1e-6), (7, 96, 1e-5), (21, 100, 0.5), (5, 2048, 1e-5),
                           (18, 8208, 1e-5)]:                      # the last: wider than the per-row kernel's LDS, 16 rows a workgroup
        x, w = torch.randn(rows, dim, generator=g) * 3, torch.randn(dim, generator=g)
        o32 = torch.zeros(rows, dim, device=gpu)
        ob = torch.zeros(rows, dim, device=gpu, dtype=torch.bfloat16)
        ops.rmsnorm(x.to(gpu), w.to(gpu), o32, rows, eps)
        ops.rmsnorm(x.to(gpu), w.bfloat16().to(gpu), ob, rows, eps)
        ref = pl.rmsnorm(x.double(), w, eps)
        assert (o32.cpu().double() - ref).abs().max() <= 4e-7 * ref.abs().max()
        refb = pl.rmsnorm(x.double(), w.bfloat16(), eps)
        assert (ob.cpu().double() - refb).abs().max() <= 2 ** -8 * refb.abs().max()
        if dim <= 100 or dim > 8192:                               # the canonical order, bit for bit
            for r in range(min(rows, 2)):
                xr = x[r].numpy()
                ss = canonical_sumsq(xr)
                inv = np.float32(1.0) / np.sqrt(np.float32(ss / np.float32(dim) + np.float32(eps)), dtype=np.float32)
                want = (xr * inv) * w.numpy()
                assert np.array_equal(o32[r].cpu().numpy().view(np.uint32), want.astype(np.float32).view(np.uint32))
    # bfloat16 out (rows as 16-byte vectors, a row a wave): lane l owns vectors l, l + 64, ... and runs one chain over
    # their elements in ascending order; the lanes are joined by xor butterflies 32, 16, ..., 1.  The three routes
    # (a row in eight vectors a lane, in sixteen, in two passes) against that order spelled out, bit for bit
    for dim in (2048, 2052, 4096, 4100):
        x, w = torch.randn(2, dim, generator=g) * 3, torch.randn(dim, generator=g)
        ob = torch.zeros(2, dim, device=gpu, dtype=torch.bfloat16)
        ops.rmsnorm(x.to(gpu), w.to(gpu), ob, 2, 1e-5)
        xr, nvec = x[1].numpy(), dim // 4
        lanes = [np.float32(0.0)] * 64
        for c in range(nvec):
            for e in range(4):
                lanes[c % 64] = fma32(xr[4 * c + e], xr[4 * c + e], lanes[c % 64])
        for off in (32, 16, 8, 4, 2, 1):
            lanes = [np.float32(lanes[l] + lanes[l ^ off]) for l in range(64)]
        inv = np.float32(1.0) / np.sqrt(np.float32(lanes[0] / np.float32(dim) + np.float32(1e-5)), dtype=np.float32)
        want = torch.from_numpy(((xr * inv) * w.numpy()).astype(np.float32)).bfloat16()
        assert torch.equal(ob[1].cpu(), want), dim
    z = torch.zeros(2, 64, device=gpu)
    out = torch.ones(2, 64, device=gpu)
    ops.rmsnorm(z, torch.ones(64, device=gpu), out, 2, 1e-5)
    assert torch.equal(out, z)                                     # x = 0 gives exactly 0


def test_embed_gather_swiglu_add(gpu):
    g = torch.Generator().manual_seed(5)
    table = torch.randn(37, 24, generator=g).bfloat16().to(gpu)
    toks = torch.tensor([5, 0, 36, -1, 5], dtype=torch.int32, device=gpu)
    out = torch.full((5, 24), 9.0, device=gpu)
    ops.embed(toks, table, out)
    assert torch.equal(out[[0, 1, 2, 4]], table.float()[[5, 0, 36, 5]]) and torch.equal(out[3], torch.zeros(24, device=gpu))
    table32 = torch.randn(37, 24, generator=g).to(gpu)
    ops.embed(toks[:3].contiguous(), table32, out)
    assert torch.equal(out[:3], table32[[5, 0, 36]])
    x = torch.randn(11, 40, generator=g).to(gpu)
    idx = torch.tensor([10, 0, 3, 3], dtype=torch.int32, device=gpu)
    got = torch.zeros(4, 40, device=gpu)
    ops.gather_rows(x, idx, got, 4)
    assert torch.equal(got, x[[10, 0, 3, 3]])
    gu = torch.randn(6, 2 * 28, generator=g).to(gpu) * 4
    gu[0, 0], gu[0, 1], gu[0, 2] = 0.0, 40.0, -40.0
    h = torch.zeros(6, 28, device=gpu)
    ops.swiglu_f32(gu, h, 6)
    want = pl.swiglu(gu[:, :28].double().cpu(), gu[:, 28:].double().cpu())
    assert (h.cpu().double() - want).abs().max() <= 3e-7 * want.abs().max()
    assert h[0, 0] == 0 and abs(h[0, 1].item() - 40.0 * gu[0, 29].item()) < 1e-4 and abs(h[0, 2].item()) < 1e-12
    a, b = torch.randn(5, 16, generator=g).to(gpu), torch.randn(5, 16, generator=g).to(gpu)
    s = a.clone()
    ops.add_(s, b, 4)
    assert torch.equal(s[:4], a[:4] + b[:4]) and torch.equal(s[4], a[4])


def rope_tables(theta, hd, n, gpu):
    inv = pl.rope_inv_freq(theta, hd)
    ang = (np.arange(n, dtype=np.float32)[:, None] * inv[None, :]).astype(np.float32).astype(np.float64)
    return (torch.from_numpy(np.cos(ang).astype(np.float32)).to(gpu), torch.from_numpy(np.sin(ang).astype(np.float32)).to(gpu))


@pytest.mark.parametrize("bf16", [False, True])
def test_rope_and_cache_write(gpu, bf16):
    g = torch.Generator().manual_seed(6)
    heads, kvh, hd, page, pages = 3, 2, 48, 8, 9
    cos, sin = rope_tables(50000.0, hd, 80, gpu)
    positions = [0, 1, 7, 8, 63, 70]
    rows = len(positions)
    width = (heads + 2 * kvh) * hd
    qkv = torch.randn(rows, width, generator=g)
    table = torch.tensor([[8, 2, 5, 0, 7, 1, 3, 6, 4], [4, 6, 3, 1, 7, 0, 5, 2, 8]], dtype=torch.int32, device=gpu)
    row_seq = torch.tensor([0, 0, 1, 1, 0, 1], dtype=torch.int32, device=gpu)
    dt = torch.bfloat16 if bf16 else torch.float32
    poison = 1e30
    kc = torch.full((pages, kvh * page * hd), poison, dtype=dt, device=gpu)
    vc = torch.full((pages, kvh * page * hd), poison, dtype=dt, device=gpu)
    dev = qkv.to(gpu).clone()
    q_out = torch.zeros(rows, heads * hd, dtype=torch.bfloat16, device=gpu) if bf16 else None
    ops.rope_kvwrite(dev, q_out, torch.tensor(positions, dtype=torch.int32, device=gpu), row_seq, table, cos, sin,
                     kc, vc, rows, heads, kvh, hd, page)
    inv = pl.rope_inv_freq(50000.0, hd)
    q_ref = pl.rope(qkv[:, :heads * hd].double().view(rows, heads, hd), positions, inv)
    k_ref = pl.rope(qkv[:, heads * hd:(heads + kvh) * hd].double().view(rows, kvh, hd), positions, inv)
    v_ref = qkv[:, (heads + kvh) * hd:].double().view(rows, kvh, hd)
    tol = 2 ** -8 if bf16 else 2e-7
    q_got = (q_out if bf16 else dev[:, :heads * hd]).cpu().double().view(rows, heads, hd)
    assert (q_got - q_ref).abs().max() <= tol * q_ref.abs().max()
    if bf16:
        assert torch.equal(q_out[0], qkv[0, :heads * hd].bfloat16().to(gpu))          # position 0: no rotation
    else:
        assert torch.equal(dev[0, :(heads + kvh) * hd], qkv[0, :(heads + kvh) * hd].to(gpu))
    kc4 = kc.view(pages, kvh, page, hd).cpu().double()
    vc4 = (vc.view(pages, kvh, hd, page).transpose(2, 3) if bf16 else vc.view(pages, kvh, page, hd)).cpu().double()
    written = set()
    for r, p in enumerate(positions):
        pg = int(table[int(row_seq[r]), p // page])
        assert (kc4[pg, :, p % page] - k_ref[r]).abs().max() <= tol * k_ref.abs().max()
        ref_v = v_ref[r].bfloat16().double() if bf16 else v_ref[r]
        assert torch.equal(vc4[pg, :, p % page], ref_v)                              # v is stored untouched
        written.add((pg, p % page))
    for pg in range(pages):
        for s in range(page):
            if (pg, s) not in written:
                assert (kc4[pg, :, s] == torch.tensor(poison).to(dt).double()).all()      # nothing else was touched


# ----------------------------------------------------------------------------- attention

def paged_setup(gpu, bf16, heads, kvh, hd, page, pages, n_keys, seed, poison=False):
    """A sequence of n_keys keys and values scattered over pages by the reference's table
    (i*7+3) % pages (tests/test_main.cpp:146-147); everything else is poison."""
    g = torch.Generator().manual_seed(seed)
    k, v = torch.randn(n_keys, kvh, hd, generator=g), torch.randn(n_keys, kvh, hd, generator=g)
    dt = torch.bfloat16 if bf16 else torch.float32
    k, v = k.to(dt), v.to(dt)
    fill = float("nan") if poison else 0.0
    kc = torch.full((pages, kvh, page, hd), fill, dtype=dt)
    vc = torch.full((pages, kvh, page, hd), fill, dtype=dt)
    n_pages = (n_keys + page - 1) // page
    table = [(i * 7 + 3) % pages for i in range(n_pages)]
    assert len(set(table)) == n_pages
    for j in range(n_keys):
        kc[table[j // page], :, j % page] = k[j]
        vc[table[j // page], :, j % page] = v[j]
    if bf16:
        vc = vc.transpose(2, 3).contiguous()
    tab = torch.tensor([table], dtype=torch.int32, device=gpu)
    return k, v, kc.reshape(pages, -1).to(gpu), vc.reshape(pages, -1).to(gpu), tab


def run_attention(gpu, bf16, q, positions, tab, kc, vc, heads, kvh, hd, page, window=0, split=False, tiles=None,
                  shared=False, mfma=False):
    """split: the decode kernel (a wave per partition); shared: it may also split a tile over
    workgroups that meet in device scratch (given full of NaN: only what a launch wrote may be read);
    mfma (32-bit): a wave per tile of up to 32 rows, both products on the matrix cores."""
    rows = len(positions)
    pos = torch.tensor(positions, dtype=torch.int32, device=gpu)
    scale = 1.0 / float(hd) ** 0.5
    if not bf16:
        out = torch.zeros(rows, heads * hd, device=gpu)
        if tiles is not None:                      # a workgroup a tile of rows, or (tiles of one row) a tile's row
            t = torch.tensor(tiles, dtype=torch.int32, device=gpu)
            ops.attention_f32_tiles(q.to(gpu), pos, tab, t, len(tiles), 2 if mfma else any(n != 1 for _, n, _, _ in tiles),
                                    kc, vc, out, heads, kvh, hd, page, window, scale)
            return out
        ops.attention_f32(q.to(gpu), pos, torch.zeros(rows, dtype=torch.int32, device=gpu), tab, kc, vc, out, rows,
                          heads, kvh, hd, page, window, scale)
        return out
    out = torch.zeros(rows, heads * hd, device=gpu, dtype=torch.bfloat16)
    if tiles is None:
        tiles = [(r, 1, 0, 0) for r in range(rows)]
    t = torch.tensor(tiles, dtype=torch.int32, device=gpu)
    scratch = None
    if shared:
        floats, counters = ops.attention_decode_scratch(len(tiles), heads, kvh, hd, tab.stride(0), page)
        assert floats > 0 and counters > 0, "this launch was meant to be split over workgroups"
        scratch = (torch.full((floats,), float("nan"), device=gpu), torch.zeros(counters, dtype=torch.int32, device=gpu))
    ops.attention_bf16(q.to(gpu), pos, tab, t, len(tiles), kc, vc, out, heads, kvh, hd, page, window, scale,
                       decode=split, scratch=scratch)
    if shared:                                   # the counters are zero again, and a second launch on them agrees
        assert not scratch[1].any()
        again = torch.zeros_like(out)
        ops.attention_bf16(q.to(gpu), pos, tab, t, len(tiles), kc, vc, again, heads, kvh, hd, page, window, scale,
                           decode=True, scratch=scratch)
        assert torch.equal(again, out) and not scratch[1].any()
    return out


def plain_rows(q, k, v, positions, heads, window=None):
    """Row r is the query at positions[r] over keys 0..positions[r] of the same sequence."""
    hd = q.shape[-1] // heads
    out = []
    for r, p in enumerate(positions):
        qq = torch.zeros(p + 1, heads, hd, dtype=F64)
        qq[p] = q[r].double().view(heads, hd)
        out.append(pl.attention(qq, k[:p + 1].double(), v[:p + 1].double(), window=window)[p].reshape(-1))
    return torch.stack(out)


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("heads,kvh,hd,page", [(4, 2, 16, 16), (3, 1, 32, 8), (5, 5, 80, 32), (2, 1, 128, 16), (6, 2, 64, 64)])
def test_attention_batched_equals_alone_and_plain(gpu, bf16, heads, kvh, hd, page):
    """The reference's invariance test (tests/test_main.cpp:137-169): positions 0, 5, 17, 300,
    301, 302, 511 in one batch equal each row alone, bit for bit; everything outside the
    sequence's written slots is NaN and must not be read."""
    pages = 512 // page + 5
    while pages % 7 == 0:
        pages += 1                                                 # the table (i*7+3) % pages must not repeat
    k, v, kc, vc, tab = paged_setup(gpu, bf16, heads, kvh, hd, page, pages, 512, seed=7, poison=True)
    positions = [0, 5, 17, 300, 301, 302, 511]
    g = torch.Generator().manual_seed(8)
    q = torch.randn(len(positions), heads * hd, generator=g).to(torch.bfloat16 if bf16 else torch.float32)
    batch = run_attention(gpu, bf16, q, positions, tab, kc, vc, heads, kvh, hd, page)
    assert torch.isfinite(batch.float()).all()
    for r, p in enumerate(positions):
        alone = run_attention(gpu, bf16, q[r:r + 1], [p], tab, kc, vc, heads, kvh, hd, page)
        assert torch.equal(alone[0], batch[r]), f"position {p}"
    ref = plain_rows(q, k, v, positions, heads)
    tol = 1.5e-2 if bf16 else 3e-6
    assert (batch.cpu().double() - ref).abs().max() <= tol * ref.abs().max()
    first = v[0].double().repeat_interleave(heads // kvh, dim=0).reshape(-1)
    assert torch.equal(batch[0].cpu().double(), first)            # one key: the output is its value, exactly
    if bf16:                                                      # a wave per partition gives the same bits
        sp = run_attention(gpu, bf16, q, positions, tab, kc, vc, heads, kvh, hd, page, split=True)
        assert torch.equal(sp, batch)
        sh = run_attention(gpu, bf16, q, positions, tab, kc, vc, heads, kvh, hd, page, split=True, shared=True)
        assert torch.equal(sh, batch)             # and so do several workgroups a tile


def test_attention_random_shapes(gpu):
    """Head sizes, groups, page sizes, windows and key counts drawn at random: a prompt portion's tiles, single rows,
    the decode kernel and its split over workgroups agree bit for bit (bfloat16), tiles of rows and single rows
    agree in 32-bit, and all are the plain result."""
    import random
    rnd = random.Random(21)
    for case in range(36):
        bf16 = rnd.random() < 0.6
        hd = rnd.choice([16, 32, 48, 64, 80, 96, 128, 160, 256] if bf16 else [16, 32, 64, 96, 128, 160])
        kvh = rnd.choice([1, 2, 3, 5])
        group = rnd.choice([1, 2, 3, 4, 7] if bf16 else [1, 2, 4])
        heads = kvh * group
        page = rnd.choice([4, 8, 16, 32, 64] if bf16 else [4, 8, 16, 32])
        nkeys = rnd.choice([5, 40, 64, 65, 130, 300])
        pages = (nkeys + page - 1) // page + rnd.choice([1, 2, 3])
        while pages % 7 == 0:
            pages += 1
        window = rnd.choice([0, 0, 3, 50, 200])
        what = (case, bf16, heads, kvh, hd, page, nkeys, window)
        k, v, kc, vc, tab = paged_setup(gpu, bf16, heads, kvh, hd, page, pages, nkeys, seed=100 + case, poison=True)
        g = torch.Generator().manual_seed(200 + case)
        positions = list(range(rnd.randrange(0, nkeys), nkeys))[:40]
        q = torch.randn(len(positions), heads * hd, generator=g).to(torch.bfloat16 if bf16 else torch.float32)
        single = run_attention(gpu, bf16, q, positions, tab, kc, vc, heads, kvh, hd, page, window=window)
        if bf16:
            tpt = max(1, 16 // min(group, 16))
            tiles = [(off, min(tpt, len(positions) - off), 0, 0) for off in range(0, len(positions), tpt)]
            while len(tiles) % ops.fold_group_tiles(hd):
                tiles.append((0, 0, 0, 0))
            assert torch.equal(run_attention(gpu, bf16, q, positions, tab, kc, vc, heads, kvh, hd, page, window=window, tiles=tiles), single), what
            assert torch.equal(run_attention(gpu, bf16, q, positions, tab, kc, vc, heads, kvh, hd, page, window=window, split=True), single), what
            if ops.attention_decode_scratch(len(positions), heads, kvh, hd, tab.stride(0), page)[0]:
                assert torch.equal(run_attention(gpu, bf16, q, positions, tab, kc, vc, heads, kvh, hd, page, window=window, split=True,
                                                 shared=True), single), what
        elif hd <= 128:
            tpt = rnd.choice([1, 3, 16])
            tiles = [(off, min(tpt, len(positions) - off), 0, 0) for off in range(0, len(positions), tpt)]
            assert torch.equal(run_attention(gpu, bf16, q, positions, tab, kc, vc, heads, kvh, hd, page, window=window, tiles=tiles), single), what
            tpt = rnd.choice([1, 5, 32])                          # and on the matrix cores
            tiles = [(off, min(tpt, len(positions) - off), 0, 0) for off in range(0, len(positions), tpt)]
            assert torch.equal(run_attention(gpu, bf16, q, positions, tab, kc, vc, heads, kvh, hd, page, window=window, tiles=tiles,
                                             mfma=True), single), what
        ref = plain_rows(q, k, v, positions, heads, window=window or None)
        assert (single.cpu().double() - ref).abs().max() <= (2e-2 if bf16 else 5e-6) * ref.abs().max().clamp(min=0.05), what


def test_decode_attention_with_many_workgroups(gpu):
    """So many tokens and kv heads that there are several workgroups for every compute unit (the decode kernel then
    runs with fewer waves a workgroup): still the bits of the fold kernel."""
    heads, kvh, hd, page = 32, 32, 16, 16
    k, v, kc, vc, tab = paged_setup(gpu, True, heads, kvh, hd, page, 40, 500, seed=19, poison=True)
    positions = [(37 * i + 5) % 500 for i in range(40)]           # 40 x 32 = 1280 workgroups
    g = torch.Generator().manual_seed(20)
    q = torch.randn(len(positions), heads * hd, generator=g).bfloat16()
    fold = run_attention(gpu, True, q, positions, tab, kc, vc, heads, kvh, hd, page)
    split = run_attention(gpu, True, q, positions, tab, kc, vc, heads, kvh, hd, page, split=True)
    assert torch.equal(split, fold)
    few = run_attention(gpu, True, q[:3], positions[:3], tab, kc, vc, heads, kvh, hd, page, split=True)
    assert torch.equal(few, fold[:3])                              # (and of the same kernel with eight waves)


@pytest.mark.parametrize("heads,kvh,hd,nkeys,window", [(16, 1, 128, 700, 0), (20, 1, 256, 1500, 0), (7, 1, 64, 4000, 0),
                                                       (7, 1, 64, 4000, 2500), (3, 3, 16, 300, 0)])
def test_decode_attention_passes_wide_groups_and_implicit_tiles(gpu, heads, kvh, hd, nkeys, window):
    """The decode kernel where its LDS is tight: sixteen heads a workgroup (more than 64 KB of partials; at 256 only four
    waves' fit), contexts of more partitions than LDS holds at once (the sums wait in LDS between passes), and the
    implicit tile list (tile t = row t of sequence t, whose first pages are asked for before the position is known):
    the bits of the fold kernel, and the plain result."""
    page = 16
    pages = nkeys // page + 3
    while pages % 7 == 0:
        pages += 1
    k, v, kc, vc, tab = paged_setup(gpu, True, heads, kvh, hd, page, pages, nkeys, seed=31, poison=True)
    positions = [nkeys - 1, nkeys // 2, 70, 3, 0, nkeys - 2]
    g = torch.Generator().manual_seed(32)
    q = torch.randn(len(positions), heads * hd, generator=g).bfloat16()
    fold = run_attention(gpu, True, q, positions, tab, kc, vc, heads, kvh, hd, page, window=window)
    assert torch.equal(run_attention(gpu, True, q, positions, tab, kc, vc, heads, kvh, hd, page, window=window, split=True), fold)
    if ops.attention_decode_scratch(len(positions), heads, kvh, hd, tab.stride(0), page)[0]:
        assert torch.equal(run_attention(gpu, True, q, positions, tab, kc, vc, heads, kvh, hd, page, window=window, split=True,
                                         shared=True), fold)
    rows = len(positions)
    out = torch.zeros(rows, heads * hd, device=gpu, dtype=torch.bfloat16)
    ops.attention_bf16(q.to(gpu), torch.tensor(positions, dtype=torch.int32, device=gpu), tab.repeat(rows, 1).contiguous(), None,
                       rows, kc, vc, out, heads, kvh, hd, page, window, 1.0 / float(hd) ** 0.5, decode=True)
    assert torch.equal(out, fold)
    ref = plain_rows(q, k, v, positions, heads, window=window or None)
    assert (fold.cpu().double() - ref).abs().max() <= 2e-2 * ref.abs().max()


@pytest.mark.parametrize("bf16", [False, True])
def test_attention_prompt_tiles_equal_single_rows(gpu, bf16):
    """Rows of a prompt portion share a tile with consecutive positions; each must equal the
    same query run as a single decoded token."""
    heads, kvh, hd, page = 6, 2, 32, 16
    k, v, kc, vc, tab = paged_setup(gpu, bf16, heads, kvh, hd, page, 40, 200, seed=9, poison=True)
    positions = list(range(120, 147))
    g = torch.Generator().manual_seed(10)
    q = torch.randn(len(positions), heads * hd, generator=g).to(torch.bfloat16 if bf16 else torch.float32)
    tpt = 16 // (heads // kvh) if bf16 else 16
    tiles = [(off, min(tpt, len(positions) - off), 0, 0) for off in range(0, len(positions), tpt)]
    portion = run_attention(gpu, bf16, q, positions, tab, kc, vc, heads, kvh, hd, page, tiles=tiles)
    single = run_attention(gpu, bf16, q, positions, tab, kc, vc, heads, kvh, hd, page)
    assert torch.equal(portion, single)
    if not bf16:
        # a window that ends inside the tile's keys, tiles of other sizes, and tiles of one row through the row kernel
        for window, tpt in ((0, 1), (37, 16), (37, 7), (5, 16), (70, 3)):
            tiles = [(off, min(tpt, len(positions) - off), 0, 0) for off in range(0, len(positions), tpt)]
            tiled = run_attention(gpu, bf16, q, positions, tab, kc, vc, heads, kvh, hd, page, window=window, tiles=tiles)
            alone = run_attention(gpu, bf16, q, positions, tab, kc, vc, heads, kvh, hd, page, window=window)
            assert torch.equal(tiled, alone), (window, tpt)
        # the same on the matrix cores (tiles of up to 32 rows)
        for window, tpt in ((0, 32), (0, 1), (37, 32), (37, 7), (5, 16), (70, 3), (33, 27)):
            tiles = [(off, min(tpt, len(positions) - off), 0, 0) for off in range(0, len(positions), tpt)]
            tiled = run_attention(gpu, bf16, q, positions, tab, kc, vc, heads, kvh, hd, page, window=window, tiles=tiles, mfma=True)
            alone = run_attention(gpu, bf16, q, positions, tab, kc, vc, heads, kvh, hd, page, window=window)
            assert torch.equal(tiled, alone), ("matrix cores", window, tpt)
        first = run_attention(gpu, bf16, q[:20], list(range(20)), tab, kc, vc, heads, kvh, hd, page, tiles=[(0, 20, 0, 0)], mfma=True)
        assert torch.equal(first, run_attention(gpu, bf16, q[:20], list(range(20)), tab, kc, vc, heads, kvh, hd, page))
        first = run_attention(gpu, bf16, q[:20], list(range(20)), tab, kc, vc, heads, kvh, hd, page, tiles=[(0, 16, 0, 0), (16, 4, 0, 0)])
        assert torch.equal(first, run_attention(gpu, bf16, q[:20], list(range(20)), tab, kc, vc, heads, kvh, hd, page))
    ref = plain_rows(q, k, v, positions, heads)
    assert (portion.cpu().double() - ref).abs().max() <= (1.5e-2 if bf16 else 3e-6) * ref.abs().max()


@pytest.mark.parametrize("bf16", [False, True])
def test_attention_finds_a_far_key_and_respects_the_window(gpu, bf16):
    """One key among hundreds is made to stand out by scaling it and the query: the output must
    be that key's value.  With a window, the key just outside must be invisible however
    attractive it is, and the key just inside visible."""
    heads, kvh, hd, page, n = 2, 1, 64, 16, 700
    k, v, kc, vc, tab = paged_setup(gpu, bf16, heads, kvh, hd, page, 50, n, seed=11)
    dt = torch.bfloat16 if bf16 else torch.float32
    g = torch.Generator().manual_seed(12)
    for far in (3, 64, 333, 448):                                  # in a first page, at partition and page edges, mid
        q = torch.randn(1, heads * hd, generator=g)
        kk = k.clone()
        kk[far, 0] = (q[0, :hd] * 4).to(dt)                        # head 0 of the query loves key `far`
        kc2 = kc.clone().view(50, kvh, page, hd)
        kc2[(far // page * 7 + 3) % 50, 0, far % page] = kk[far, 0].to(gpu)
        out = run_attention(gpu, bf16, q.to(dt), [n - 1], tab, kc2.view(50, -1), vc, heads, kvh, hd, page)
        assert (out[0, :hd].cpu().double() - v[far, 0].double()).abs().max() < 0.05, f"key {far} not found"
        ref = plain_rows(q.to(dt), kk, v, [n - 1], heads)
        assert (out.cpu().double() - ref).abs().max() <= (1.5e-2 if bf16 else 3e-6) * ref.abs().max()
        # window of 100 keys: the query at position far+99 still sees it, the one at far+100 does not
        for p, visible in ((far + 99, True), (far + 100, False)):
            if p >= n:
                continue
            w = run_attention(gpu, bf16, q.to(dt), [p], tab, kc2.view(50, -1), vc, heads, kvh, hd, page, window=100)
            hit = (w[0, :hd].cpu().double() - v[far, 0].double()).abs().max() < 0.05
            assert hit == visible, f"key {far} from position {p}: visible={hit}"
            refw = plain_rows(q.to(dt), kk, v, [p], heads, window=100)
            assert (w.cpu().double() - refw).abs().max() <= (1.5e-2 if bf16 else 3e-6) * refw.abs().max()
            if bf16:                              # the window's first partition is where a split tile's scratch begins
                ws = run_attention(gpu, bf16, q.to(dt), [p], tab, kc2.view(50, -1), vc, heads, kvh, hd, page, window=100,
                                   split=True, shared=True)
                assert torch.equal(ws, w)


def test_attention_refuses_what_it_cannot_do(gpu):
    z = torch.zeros(1, 40, device=gpu)
    i32 = torch.zeros(1, dtype=torch.int32, device=gpu)
    with pytest.raises(ValueError, match="head size 40"):
        ops.attention_f32(z, i32, i32, i32.view(1, 1), z, z, z, 1, 1, 1, 40, 16, 0, 1.0)
    zb = torch.zeros(1, 64, device=gpu, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="page size"):
        ops.attention_bf16(zb, i32, i32.view(1, 1), torch.zeros(1, 4, dtype=torch.int32, device=gpu), 1,
                           torch.zeros(1, 64 * 24, device=gpu, dtype=torch.bfloat16),
                           torch.zeros(1, 64 * 24, device=gpu, dtype=torch.bfloat16), zb, 1, 1, 64, 24, 0, 1.0)
    with pytest.raises(ValueError, match="no CPU path"):
        ops.rmsnorm(torch.zeros(1, 8), torch.ones(8), torch.zeros(1, 8), 1, 1e-5)


# ----------------------------------------------------------------------------- sampling

def test_sampling_and_fingerprint(gpu):
    g = torch.Generator().manual_seed(13)
    V = 501
    logits = (torch.randn(9, V, generator=g) * 3).to(gpu)
    logits[0, 7] = logits[0, 400] = 50.0                           # a tie: the first maximum wins
    logits[1, V - 1] = 60.0
    temps = [0.0, 0.0, -1.0, 0.8, 0.8, 1.5, 0.3, 1.0, 1.0]
    us = [0.0, 0.0, 0.0, 0.0, 1.0 - 2 ** -53, 0.37, 0.99, 0.5, 0.123456789]
    out = torch.zeros(9, dtype=torch.int32, device=gpu)
    ops.sample(logits, 9, torch.tensor(temps, device=gpu), torch.tensor(us, dtype=torch.float64, device=gpu), out)
    got = out.cpu().tolist()
    host = logits.cpu().numpy()
    assert got[0] == 7 and got[1] == V - 1
    for r in range(9):
        want = pl.argmax_row(host[r]) if temps[r] <= 0 else pl.sample_row(host[r], temps[r], us[r])
        assert got[r] == want, f"row {r}"
    # (blocks of 16 words chained in turn from two sets of registers: none, one, two, three, many, with words and an
    # odd element left over; rows that start on an odd element)
    for Vv in (500, 501, 6, 1, 2, 31, 32, 33, 64, 65, 96, 97, 128, 1000, 49152):
        rows = torch.randn(3, Vv, generator=g).to(gpu)
        basis = [1469598103934665603, 12345, 2 ** 64 - 1]
        h_in = torch.from_numpy(np.asarray(basis, np.uint64).view(np.int64)).to(gpu)
        h_out = torch.zeros(3, dtype=torch.int64, device=gpu)
        ops.fingerprint(rows, 3, h_in, h_out)
        want = [pl.hash_floats(b, rows[i].cpu().numpy()) for i, b in enumerate(basis)]
        assert h_out.cpu().numpy().view(np.uint64).tolist() == want


def test_sampling_at_real_vocabularies(gpu):
    """49,152 and 128,256 logits a row: the device sums its weights in 256 stretches that it joins in order, the
    plain code in one sequential chain of doubles; both use the engine's own 32-bit exponential, so they must
    pick the same token wherever the uniform does not fall within rounding of a boundary."""
    import plain_scalar as ps

    g = torch.Generator().manual_seed(17)
    for V in (49152, 128256):
        rows = 12
        logits = (torch.randn(rows, V, generator=g) * 2.5).to(gpu)
        logits[0, V - 3] = 30.0                                        # nearly all weight on a late token
        temps = [0.7, 0.7, 1.0, 1.3, 0.2, 2.0, 0.9, 0.9, 0.0, 1.0, 0.5, 1.1]
        us = [0.5, 0.001, 0.999, 0.25, 0.75, 0.6180339887, 0.0, 1.0 - 2 ** -53, 0.4, 0.31415926, 0.9, 0.05]
        out = torch.zeros(rows, dtype=torch.int32, device=gpu)
        ops.sample(logits, rows, torch.tensor(temps, device=gpu), torch.tensor(us, dtype=torch.float64, device=gpu), out)
        host = logits.cpu().numpy()
        for r, got in enumerate(out.cpu().tolist()):
            want = pl.argmax_row(host[r]) if temps[r] <= 0 else pl.sample_row(host[r], temps[r], us[r], ps.expf)
            assert got == want, f"V={V} row {r}"


# ----------------------------------------------------------------------------- decode fusions

def test_fused_norm_products_equal_the_separate_kernels(gpu):
    """RMSNorm fused into the product (and rotation plus cache write into the q|k|v product)
    must give the bits of the kernels run one after the other."""
    g = torch.Generator().manual_seed(14)
    for M, K, N in [(1, 64, 48), (5, 128, 500), (8, 2048, 6144), (16, 192, 112), (13, 1024, 72),
                    (16, 192, 4100), (1, 64, 4096), (11, 2048, 4224),    # many columns: another kernel
                    (8, 4096, 4096), (5, 4096, 8200), (3, 2176, 4160), (1, 3968, 4224)]:   # rows of two segments of K, up to 8 of them
        x = (torch.randn(M, K, generator=g) * 2).to(gpu)
        nw = (1 + 0.1 * torch.randn(K, generator=g)).bfloat16().to(gpu)
        w = (torch.randn(N, K, generator=g) * 0.05).bfloat16().to(gpu)
        h = torch.zeros(M, K, device=gpu, dtype=torch.bfloat16)
        ops.rmsnorm(x, nw, h, M, 1e-5)
        sep = torch.zeros(M, N, device=gpu)
        ops.gemm_bf16(h, w, sep, M, ops.EPI_F32)
        fused = torch.full((M, N), 5.0, device=gpu)
        ops.norm_gemm_bf16(x, nw, 1e-5, w, fused, M, ops.EPI_F32)
        assert torch.equal(fused, sep), (M, K, N)
        if N % 2 == 0:
            sep_s = torch.zeros(M, N // 2, device=gpu, dtype=torch.bfloat16)
            ops.gemm_bf16(h, w, sep_s, M, ops.EPI_SWIGLU_BF16)
            fused_s = torch.zeros(M, N // 2, device=gpu, dtype=torch.bfloat16)
            ops.norm_gemm_bf16(x, nw.float(), 1e-5, w, fused_s, M, ops.EPI_SWIGLU_BF16)
            assert torch.equal(fused_s, sep_s), (M, K, N)
    assert not ops.can_fuse_norm(17, w, x) and not ops.can_fuse_norm(4, torch.zeros(8, 4096, dtype=torch.bfloat16), x)
    wide_x, wide_w = torch.zeros(9, 4096), torch.zeros(4096, 4096, dtype=torch.bfloat16)
    assert ops.can_fuse_norm(8, wide_w, wide_x) and not ops.can_fuse_norm(9, wide_w, wide_x)           # wide rows: 8 at most,
    assert not ops.can_fuse_norm(8, wide_w[:4032], wide_x) and ops.can_fuse_norm(8, wide_w[:4032], wide_x, columns=32, stacked=2) is False   # 64 workgroups,
    assert not ops.can_fuse_norm(4, torch.zeros(4096, 4160, dtype=torch.bfloat16), torch.zeros(4, 4160))   # two segments
    assert not ops.can_fuse_norm(4, torch.zeros(8, 96, dtype=torch.bfloat16), torch.zeros(4, 96))   # steps of 64 along the rows
    assert not ops.qkv_rope_head_dim_ok(48, 64) and ops.qkv_rope_head_dim_ok(48, 192) and ops.qkv_rope_head_dim_ok(256, 64)   # the epilogue's LDS

    for heads, kvh, hd, page, K in [(4, 2, 16, 16, 64), (3, 1, 32, 8, 128), (32, 32, 64, 16, 2048), (6, 2, 48, 32, 192),
                                     (2, 1, 128, 16, 256), (3, 3, 96, 16, 128), (40, 12, 64, 32, 128),    # the last two: half a head a workgroup,
                                     (200, 28, 64, 16, 64),                                           # a head a workgroup
                                     (24, 4, 128, 16, 128), (12, 2, 256, 8, 64), (100, 14, 128, 16, 64),      # larger heads: 16 or 32 pairs a workgroup
                                     (32, 8, 128, 16, 4096), (40, 12, 64, 32, 2176)]:                 # rows of two segments of K
        M, pages = 7, 12
        cos, sin = rope_tables(10000.0, hd, 100, gpu)
        x = (torch.randn(M, K, generator=g) * 2).to(gpu)
        nw = (1 + 0.1 * torch.randn(K, generator=g)).bfloat16().to(gpu)
        w = (torch.randn((heads + 2 * kvh) * hd, K, generator=g) * 0.05).bfloat16().to(gpu)
        positions = torch.tensor([0, 1, 17, 63, 64, -1, 95], dtype=torch.int32, device=gpu)
        row_seq = torch.tensor([0, 1, 0, 1, 0, 0, 1], dtype=torch.int32, device=gpu)
        table = torch.tensor([[(i * 5 + 1) % pages for i in range(12)], [(i * 7 + 2) % pages for i in range(12)]],
                             dtype=torch.int32, device=gpu)
        outs = []
        for fused in (False, True):
            kc = torch.full((pages, kvh * page * hd), 3.0, dtype=torch.bfloat16, device=gpu)
            vc = torch.full((pages, kvh * page * hd), 3.0, dtype=torch.bfloat16, device=gpu)
            q = torch.zeros(M, heads * hd, dtype=torch.bfloat16, device=gpu)
            if fused:
                ops.norm_qkv_rope_bf16(x, nw, 1e-6, w, q, positions, row_seq, table, cos, sin, kc, vc, M, heads, kvh,
                                       hd, page)
            else:
                h = torch.zeros(M, K, device=gpu, dtype=torch.bfloat16)
                ops.rmsnorm(x, nw, h, M, 1e-6)
                qkv = torch.zeros(M, w.shape[0], device=gpu)
                ops.gemm_bf16(h, w, qkv, M, ops.EPI_F32)
                ops.rope_kvwrite(qkv, q, positions, row_seq, table, cos, sin, kc, vc, M, heads, kvh, hd, page)
            outs.append((q, kc, vc))
        live = [0, 1, 2, 3, 4, 6]                                  # the row with position -1 is padding
        assert torch.equal(outs[0][0][live], outs[1][0][live])
        assert torch.equal(outs[0][1], outs[1][1]) and torch.equal(outs[0][2], outs[1][2])


def test_prompt_qkv_product_with_rotary_epilogue_equals_the_separate_kernels(gpu):
    """More than 64 rows and heads of 64: the wide product rotates and writes the cache in its
    epilogue; q, the key pages and the value pages must be the bits of product + rope_kvwrite.
    Rows of two requests, a padding row, positions across page edges, a ragged last tile."""
    g = torch.Generator().manual_seed(21)
    for case in [(3, 1, 256, 130, 16), (4, 4, 128, 200, 8), (5, 2, 320, 97, 32),
                                   (5, 2, 96, 150, 16), (2, 2, 40, 190, 8),   # K no multiple of 64: tiles through registers
                                   (40, 10, 128, 2100, 32),        # enough 256 x 256 tiles for the big-tile kernel
                                   (40, 28, 128, 1000, 16), (41, 28, 192, 777, 8),   # 128 x 256 tiles (a ragged last one)
                                   (40, 12, 128, 64, 16), (44, 10, 192, 23, 8), (64, 8, 64, 9, 16),   # up to 64 rows, half a head a workgroup
                                   (200, 28, 64, 40, 16), (208, 24, 64, 12, 8), (230, 13, 128, 64, 32),   # a head a workgroup
                                   (40, 12, 128, 130, 16), (72, 12, 192, 300, 16), (64, 16, 2048, 190, 32),   # blocks of 64 rows in one launch
                                   (32, 8, 4096, 130, 16, 128), (24, 4, 128, 200, 16, 128), (40, 12, 4160, 200, 16),   # ... with larger heads, several segments of K
                                   (40, 12, 4160, 16, 16),                                 # several segments of K
                                   (32, 8, 4096, 8, 16, 128), (24, 4, 128, 40, 8, 128), (100, 14, 64, 12, 16, 128),
                                   (16, 8, 2112, 20, 16, 256)]:                            # larger heads, up to 64 rows
        heads, kvh, K, M, page, hd = (tuple(case) + (64,))[:6]
        pages = 40 if M < 500 else 3 * ((M + page - 1) // page + 2) + 3
        cos, sin = rope_tables(10000.0, hd, max(400, M), gpu)
        h = torch.randn(M, K, generator=g).bfloat16().to(gpu)
        w = (torch.randn((heads + 2 * kvh) * hd, K, generator=g) * 0.05).bfloat16().to(gpu)
        pos = [(r if r < M // 2 else r - M // 2 + 3) for r in range(M)]
        pos[7] = -1
        pos[2] = -1                                                # padding rows, one the second of a pair of rows and one the first
        positions = torch.tensor(pos, dtype=torch.int32, device=gpu)
        row_seq = torch.tensor([0 if r < M // 2 else 1 for r in range(M)], dtype=torch.int32, device=gpu)
        per = (M + page - 1) // page + 2
        table = torch.tensor([[(i * 3 + 1) % pages for i in range(per)], [(i * 3 + 2) % pages for i in range(per)]],
                             dtype=torch.int32, device=gpu)
        outs = []
        for fused in (False, True):
            kc = torch.full((pages, kvh * page * hd), 3.0, dtype=torch.bfloat16, device=gpu)
            vc = torch.full((pages, kvh * page * hd), 3.0, dtype=torch.bfloat16, device=gpu)
            q = torch.zeros(M, heads * hd, dtype=torch.bfloat16, device=gpu)
            if fused:
                assert ops.qkv_rope_gemm_ok(M, hd, K, heads + 2 * kvh)
                ops.gemm_qkv_rope_bf16(h, w, q, positions, row_seq, table, cos, sin, kc, vc, M, heads, kvh, hd, page)
            else:
                qkv = torch.zeros(M, w.shape[0], device=gpu)
                ops.gemm_bf16(h, w, qkv, M, ops.EPI_F32)
                ops.rope_kvwrite(qkv, q, positions, row_seq, table, cos, sin, kc, vc, M, heads, kvh, hd, page)
            outs.append((q, kc, vc))
        live = [r for r in range(M) if pos[r] >= 0]
        assert torch.equal(outs[0][0][live], outs[1][0][live]), (heads, kvh, K, M)
        assert torch.equal(outs[0][1], outs[1][1]) and torch.equal(outs[0][2], outs[1][2]), (heads, kvh, K, M)
    assert not ops.qkv_rope_gemm_ok(64, 64, 256, 63) and not ops.qkv_rope_gemm_ok(200, 128, 256, 96)
    assert not ops.qkv_rope_gemm_ok(64, 64, 96, 96) and not ops.qkv_rope_gemm_ok(8, 96, 128, 200) and not ops.qkv_rope_gemm_ok(700, 64, 4096, 96)
    assert ops.qkv_rope_gemm_ok(200, 64, 4096, 96) and ops.qkv_rope_gemm_ok(320, 128, 4096, 48) and not ops.qkv_rope_gemm_ok(384, 128, 4096, 48)


def test_decode_attention_beyond_one_pass_of_partials(gpu):
    """A context so long that the decode kernel's partials do not fit LDS at once (several
    passes over the partitions): still the bits of the fold kernel, and the plain result."""
    heads, kvh, hd, page = 2, 1, 64, 64
    n = 12600                                                      # 197 partitions of 64 keys; one pass holds 186
    pages = n // page + 4
    while pages % 7 == 0:
        pages += 1
    k, v, kc, vc, tab = paged_setup(gpu, True, heads, kvh, hd, page, pages, n, seed=31, poison=True)
    g = torch.Generator().manual_seed(32)
    positions = [n - 1, 11903, 11904, 5000]                        # at the pass edge, and a short one
    q = torch.randn(len(positions), heads * hd, generator=g).bfloat16()
    fold = run_attention(gpu, True, q, positions, tab, kc, vc, heads, kvh, hd, page)
    split = run_attention(gpu, True, q, positions, tab, kc, vc, heads, kvh, hd, page, split=True)
    assert torch.isfinite(split.float()).all()
    assert torch.equal(split, fold)
    shared = run_attention(gpu, True, q, positions, tab, kc, vc, heads, kvh, hd, page, split=True, shared=True)
    assert torch.equal(shared, fold)
    for r, p in enumerate(positions):                              # softmax(q k^T / sqrt(hd)) v for this one row, in float64
        for h in range(heads):
            qh = q[r].double().view(heads, hd)[h]
            kk, vv = k[:p + 1, h // (heads // kvh)].double(), v[:p + 1, h // (heads // kvh)].double()
            w = torch.softmax(kk @ qh / hd ** 0.5, dim=0)
            want = w @ vv
            got = split[r].cpu().double().view(heads, hd)[h]
            assert (got - want).abs().max() <= 1.5e-2 * want.abs().max().clamp(min=0.05), (p, h)


def _decode_layer_tail(gpu, g, M, width, inter, heads, kvh, hd, page, vocab):
    """What follows a decode step's attention in one layer and opens the next (output projection, RMSNorm + gate|up +
    SwiGLU, down projection, RMSNorm + q|k|v + rotation + cache write) and a head: random operands, and a function
    that runs the five products on fresh outputs, one launch each or as phases (ops.chain)."""
    cos, sin = rope_tables(10000.0, hd, 200, gpu)
    per_row = (90 + page - 1) // page                    # every row a request of its own, with pages of its own
    attn = torch.randn(M, heads * hd, generator=g).bfloat16().to(gpu)
    resid = (torch.randn(M, width, generator=g) * 2).to(gpu)
    w_o = (torch.randn(width, heads * hd, generator=g) * 0.05).bfloat16().to(gpu)
    w_gu = (torch.randn(2 * inter, width, generator=g) * 0.05).bfloat16().to(gpu)
    w_d = (torch.randn(width, inter, generator=g) * 0.05).bfloat16().to(gpu)
    w_qkv = (torch.randn((heads + 2 * kvh) * hd, width, generator=g) * 0.05).bfloat16().to(gpu)
    w_head = (torch.randn(vocab, width, generator=g) * 0.05).bfloat16().to(gpu)
    n1 = (1 + 0.1 * torch.randn(width, generator=g)).bfloat16().to(gpu)
    n2 = (1 + 0.1 * torch.randn(width, generator=g)).bfloat16().to(gpu)
    positions = torch.tensor([(7 * i + 3) % 90 if i != 2 else -1 for i in range(M)], dtype=torch.int32, device=gpu)
    row_seq = torch.arange(M, dtype=torch.int32, device=gpu)
    table = torch.arange(M * per_row, dtype=torch.int32, device=gpu).reshape(M, per_row).contiguous()

    def run(chained, sync=None, err=None, spin=None):
        x = resid.clone()
        h = torch.zeros(M, inter, dtype=torch.bfloat16, device=gpu)
        q = torch.zeros(M, heads * hd, dtype=torch.bfloat16, device=gpu)
        kc = torch.full((M * per_row, kvh * page * hd), 3.0, dtype=torch.bfloat16, device=gpu)
        vc = torch.full((M * per_row, kvh * page * hd), 3.0, dtype=torch.bfloat16, device=gpu)
        logits = torch.zeros(M, vocab, device=gpu)

        def products():
            ops.gemm_bf16(attn, w_o, x, M, ops.EPI_ADD_F32)
            ops.norm_gemm_bf16(x, n1, 1e-5, w_gu, h, M, ops.EPI_SWIGLU_BF16)
            ops.gemm_bf16(h, w_d, x, M, ops.EPI_ADD_F32)
            ops.norm_qkv_rope_bf16(x, n2, 1e-5, w_qkv, q, positions, row_seq, table, cos, sin, kc, vc, M, heads, kvh, hd, page)
            ops.norm_gemm_bf16(x, n1, 1e-5, w_head, logits, M, ops.EPI_F32)
        if chained:
            with (ops.chain(sync, err) if spin is None else ops.chain(sync, err, spin)):
                products()
        else:
            products()
        torch.cuda.synchronize()
        return x, h, q, kc, vc, logits
    return run


@pytest.mark.parametrize("M,width,inter,heads,kvh,hd,vocab", [
    (8, 2048, 8192, 32, 32, 64, 49152),        # the layer sizes the decode benchmark runs (burst, stream with 8 rows a stage)
    (13, 2048, 8192, 32, 32, 64, 4096),        # more than 8 rows (16 rows a stage, two rows a wave to normalise)
    (8, 4096, 14336, 32, 8, 128, 4096),        # rows of two segments; the stream kernel with 16 columns a wave, seven segments
    (3, 1024, 2816, 16, 4, 64, 8192),          # a feed-forward width that is no multiple of 2048
])
def test_products_as_phases_of_one_launch_equal_the_separate_launches(gpu, M, width, inter, heads, kvh, hd, vocab):
    """The decode products run as phases of one launch (ops.chain) give the bits of one launch each; the launch leaves
    its meeting words zero and reports no wait that gave up; and a second launch on the same words works like the first."""
    g = torch.Generator().manual_seed(M * 1000 + width)
    run = _decode_layer_tail(gpu, g, M, width, inter, heads, kvh, hd, 16, vocab)
    sync = torch.zeros(ops.chain_sync_words(), dtype=torch.int32, device=gpu)
    err = torch.zeros(1, dtype=torch.int32, device=gpu)
    plain = run(False)
    for _ in range(2):
        chained = run(True, sync, err)
        assert int(err.item()) == 0
        assert int(sync.abs().sum().item()) == 0
        for name, a, b in zip(("residual", "swiglu", "q", "k cache", "v cache", "logits"), plain, chained):
            assert torch.equal(a, b), name


def test_a_phase_that_gives_up_waiting_says_so_and_nothing_hangs(gpu):
    """With no looks at the flag allowed, a phase that finds the phase before it unfinished gives up at once: the launch
    ends normally, the error word names the phase, and after the caller has cleared the words the next launch is right.
    (Whether a wait gives up depends on how far the phase before has got; with no looks allowed and megabytes of weights
    to stream it has not finished.)"""
    g = torch.Generator().manual_seed(5)
    run = _decode_layer_tail(gpu, g, 8, 2048, 8192, 32, 32, 64, 16, 4096)
    sync = torch.zeros(ops.chain_sync_words(), dtype=torch.int32, device=gpu)
    err = torch.zeros(1, dtype=torch.int32, device=gpu)
    plain = run(False)
    run(True, sync, err, spin=0)                     # returns: nothing hangs
    gave_up = int(err.item())
    assert gave_up != 0 and gave_up < (1 << 6)
    sync.zero_()
    err.zero_()
    chained = run(True, sync, err)
    assert int(err.item()) == 0 and int(sync.abs().sum().item()) == 0
    for a, b in zip(plain, chained):
        assert torch.equal(a, b)
