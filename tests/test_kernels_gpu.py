"""Each HIP kernel alone against a plain float32 expression of the same operation, at
sizes other than the engine's tiny models (head sizes in steps of 16, widths and
vocabularies that are no power of two, one row and many)."""
import math

import numpy as np
import pytest
import torch

from braidinfer_amd import kernels as K
from braidinfer_amd.errors import KernelError

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def rnd(*shape, seed=0, scale=1.0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


def i32(v):
    return torch.tensor(v, dtype=torch.int32, device=DEV)


# ------------------------------------------------------------------ embedding ------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embedding(dtype):
    # reference vector: V=256, H=1024, token 42 (tests/embedding_test.rs:14-65); exact
    table = rnd(257, 1000, dtype=dtype)
    toks = i32([42, 0, 256, 42, 7])
    out = torch.empty(5, 1000, device=DEV)
    K.embedding(table, toks, out)
    assert torch.equal(out, table.float()[toks.long()])


# -------------------------------------------------------------------- RMSNorm ------
@pytest.mark.parametrize("H", [48, 1000, 4096, 5120])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_rmsnorm(H, out_dtype):
    x, w = rnd(7, H, scale=3.0), rnd(H, seed=1) * 0.1 + 1
    out = torch.empty(7, H, device=DEV, dtype=out_dtype)
    K.rmsnorm(x, w, out, 1e-6)
    want = x.double() * torch.rsqrt((x.double() ** 2).mean(-1, keepdim=True) + 1e-6) * w.double()
    tol = 1e-5 if out_dtype == torch.float32 else 2e-2
    assert (out.double() - want).abs().max() < tol * want.abs().max()
    rows = i32([6, 0, 3])
    out2 = torch.empty(3, H, device=DEV, dtype=out_dtype)
    K.rmsnorm(x, w, out2, 1e-6, rows)
    assert torch.equal(out2, out[rows.long()])


def test_rmsnorm_reference_vector():
    # tests/op_rmsnorm_test.rs:51-66,109: H=1024, 4 rows, eps 1e-6, x = sin(0.01 i), w = bf16(1 + 0.001 i), tol 1e-4
    H = 1024
    x = torch.sin(0.01 * torch.arange(4 * H, dtype=torch.float64)).reshape(4, H)
    w = (1 + 0.001 * torch.arange(H, dtype=torch.float32)).bfloat16().float()
    out = torch.empty(4, H, device=DEV)
    K.rmsnorm(x.float().to(DEV), w.to(DEV), out, 1e-6)
    want = x / torch.sqrt((x * x).mean(-1, keepdim=True) + 1e-6) * w.double()
    assert (out.cpu().double() - want).abs().max() < 1e-4


# ----------------------------------------------------------------------- GEMM ------
SHAPES = [(1, 64, 64), (5, 100, 96), (17, 192, 320), (64, 301, 100), (33, 1000, 264), (3, 50, 44),
          (130, 514, 100), (257, 129, 72), (300, 260, 1032), (130, 514, 128), (257, 129, 192), (300, 700, 1024),
          (65, 301, 64), (513, 260, 320),
          # few rows and a long k: what the streaming kernel takes (tiles beyond one per workgroup, a chunk
          # count that the waves do not share evenly)
          (1, 100, 1024), (8, 301, 1152), (9, 48, 2048), (16, 4100, 1024), (3, 9000, 1280),
          # 17 to 64 rows: what the wide streaming kernel takes
          (17, 100, 256), (64, 16500, 384), (33, 301, 1152), (48, 4100, 1024)]


def _skip_unless_kernel_takes(kernel, M, Kd, N=None):
    if kernel == 3 and (Kd % 8 or M > 64):
        pytest.skip("the skinny kernels take M <= 64 and K in steps of 8")
    if (4 <= kernel <= 6 or kernel in (10, 11)) and Kd % 64:
        pytest.skip("the direct-to-LDS tile kernels take K in steps of 64")
    if kernel == 7 and (M > 16 or Kd % 128 or Kd < 1024):
        pytest.skip("the streaming kernel takes M <= 16 and K in steps of 128 from 1024")
    if kernel == 8 and (M <= 16 or M > 64 or Kd % 128 or Kd < 256):
        pytest.skip("the wide streaming kernel takes 16 < M <= 64 and K in steps of 128 from 256")
    if 12 <= kernel <= 15 and (Kd % 64 or N is None or N % 4):
        pytest.skip("the tiles of one wave per SIMD take K in steps of 64 and output rows in steps of 16 bytes")


@pytest.mark.parametrize("M,N,Kd", SHAPES)
def test_gemm_f32(M, N, Kd):
    a, w = rnd(M, Kd, seed=1), rnd(N, Kd, seed=2)
    out = torch.empty(M, N, device=DEV)
    K.gemm(a, w, out)
    want = a.double() @ w.double().T
    assert (out.double() - want).abs().max() < 1e-5 * want.abs().max()
    base = rnd(M, N, seed=3)
    acc = base.clone()
    K.gemm(a, w, acc, accumulate=True)
    assert (acc.double() - (base.double() + want)).abs().max() < 1e-5 * want.abs().max()


def test_gemm_f32_rows_do_not_depend_on_the_batch():
    a, w = rnd(70, 200, seed=1), rnd(90, 200, seed=2)
    full = torch.empty(70, 90, device=DEV)
    K.gemm(a, w, full)
    one = torch.empty(1, 90, device=DEV)
    K.gemm(a[33:34].contiguous(), w, one)
    assert torch.equal(one[0], full[33])


@pytest.mark.parametrize("kernel", [0, 1, 2, 3, 4, 5, 6, 7, 8, 10, 12, 13, 14, 15])
@pytest.mark.parametrize("M,N,Kd", SHAPES)
def test_gemm_bf16(M, N, Kd, kernel):
    _skip_unless_kernel_takes(kernel, M, Kd, N)
    a, w = rnd(M, Kd, seed=1, scale=0.5, dtype=torch.bfloat16), rnd(N, Kd, seed=2, scale=0.5, dtype=torch.bfloat16)
    want = a.double() @ w.double().T
    o32 = torch.empty(M, N, device=DEV)
    K.gemm(a, w, o32, kernel=kernel)
    assert (o32.double() - want).abs().max() < 1e-4 * want.abs().max()        # exact products, float sums
    o16 = torch.empty(M, N, device=DEV, dtype=torch.bfloat16)
    K.gemm(a, w, o16, kernel=kernel)
    assert (o16.double() - want).abs().max() < 1e-2 * want.abs().max()
    base = rnd(M, N, seed=3)
    acc = base.clone()
    K.gemm(a, w, acc, accumulate=True, kernel=kernel)
    assert (acc.double() - (base.double() + want)).abs().max() < 1e-4 * want.abs().max()


def test_gemm_streaming_kernel_rows_and_strides():
    # a row's result does not depend on the rows beside it, nor on the row stride of a or out
    Kd, N = 2048, 530
    a, w = rnd(16, Kd, seed=1, scale=0.5, dtype=torch.bfloat16), rnd(N, Kd, seed=2, scale=0.5, dtype=torch.bfloat16)
    full = torch.empty(16, N, device=DEV)
    K.gemm(a, w, full, kernel=7)
    for rows in (slice(0, 1), slice(5, 6), slice(3, 11), slice(15, 16)):
        part = torch.empty(rows.stop - rows.start, N, device=DEV)
        K.gemm(a[rows].contiguous(), w, part, kernel=7)
        assert torch.equal(part, full[rows])
    wide_a = torch.zeros(7, Kd + 64, device=DEV, dtype=torch.bfloat16)
    wide_a[:, 8:8 + Kd] = a[:7]
    wide_o = torch.full((7, N + 10), 7.0, device=DEV)
    K.gemm(wide_a[:, 8:8 + Kd], w, wide_o[:, 3:3 + N], kernel=7)
    assert torch.equal(wide_o[:, 3:3 + N], full[:7])
    assert bool((wide_o[:, :3] == 7.0).all()) and bool((wide_o[:, 3 + N:] == 7.0).all())
    with pytest.raises(KernelError):
        K.gemm(rnd(17, Kd, dtype=torch.bfloat16), w, torch.empty(17, N, device=DEV), kernel=7)
    with pytest.raises(KernelError):
        K.gemm(rnd(4, 960, dtype=torch.bfloat16), rnd(N, 960, dtype=torch.bfloat16), torch.empty(4, N, device=DEV), kernel=7)


@pytest.mark.parametrize("kernel", [0, 3, 8, 5 + 16 * 2, 6 + 16 * 4])      # 16 * p: the tile kernel with p runs, forced
@pytest.mark.parametrize("M,N,Kd", [(17, 520, 1536), (40, 300, 4096), (64, 4096, 2048), (33, 1000, 1032), (64, 96, 8192),
                                    (100, 520, 4096), (300, 260, 2048), (129, 1000, 1024)])
def test_gemm_split_along_k_with_scratch(M, N, Kd, kernel):
    if kernel in (3, 8) and M > 64:
        pytest.skip("more than 64 rows: the tiles")
    if kernel >= 16 and Kd % 64:
        pytest.skip("the direct-to-LDS tile kernels take K in steps of 64")
    if kernel < 16:
        _skip_unless_kernel_takes(kernel, M, Kd)
    a, w = rnd(M, Kd, seed=1, scale=0.5, dtype=torch.bfloat16), rnd(N, Kd, seed=2, scale=0.5, dtype=torch.bfloat16)
    want = a.double() @ w.double().T
    scratch = torch.full((K.GEMM_SCRATCH_FLOATS,), float("nan"), device=DEV)
    o32 = torch.empty(M, N, device=DEV)
    K.gemm(a, w, o32, scratch=scratch, kernel=kernel)
    assert (o32.double() - want).abs().max() < 1e-4 * want.abs().max()
    again = torch.empty(M, N, device=DEV)
    K.gemm(a, w, again, scratch=scratch, kernel=kernel)
    assert torch.equal(again, o32)                                   # the runs are added in a fixed order
    o16 = torch.empty(M, N, device=DEV, dtype=torch.bfloat16)
    K.gemm(a, w, o16, scratch=scratch, kernel=kernel)
    assert (o16.double() - want).abs().max() < 1e-2 * want.abs().max()
    base = rnd(M, N + 6, seed=3)
    acc = base.clone()
    K.gemm(a, w, acc[:, 3:3 + N], accumulate=True, scratch=scratch, kernel=kernel)
    assert (acc[:, 3:3 + N].double() - (base[:, 3:3 + N].double() + want)).abs().max() < 1e-4 * want.abs().max()
    assert torch.equal(acc[:, :3], base[:, :3]) and torch.equal(acc[:, 3 + N:], base[:, 3 + N:])
    small = torch.empty(16, device=DEV)
    if kernel >= 16:
        with pytest.raises(KernelError):                 # forced runs need their room
            K.gemm(a, w, again, scratch=small, kernel=kernel)
        return
    # too little scratch: the product is not split, and is right all the same
    K.gemm(a, w, again, scratch=small, kernel=kernel)
    assert (again.double() - want).abs().max() < 1e-4 * want.abs().max()


@pytest.mark.parametrize("blocked", [False, True])
@pytest.mark.parametrize("parts", [0, 1, 2, 3])
@pytest.mark.parametrize("rows", [64, 80, 96, 112, 128])
def test_gemm_wide_streaming_kernel_tile_heights_and_runs(rows, parts, blocked):
    # kernel 8 with a forced tile height (rows) and number of runs along k (0: by shape); N is no
    # multiple of any height, and the first shape has more tiles than the chip has compute units
    code = 8 + 16 * (rows // 16 + 16 * parts)
    scratch = torch.full((K.GEMM_SCRATCH_FLOATS,), float("nan"), device=DEV)
    for M, N, Kd in ((64, 257 * rows + 40, 1024), (20, 1000, 1664)):
        a, w = rnd(M, Kd, seed=1, scale=0.5, dtype=torch.bfloat16), rnd(N, Kd, seed=2, scale=0.5, dtype=torch.bfloat16)
        want = a.double() @ w.double().T
        if blocked:
            w = K.block_weight(w)
        o32 = torch.empty(M, N, device=DEV)
        K.gemm(a, w, o32, scratch=scratch, kernel=code)
        assert (o32.double() - want).abs().max() < 1e-4 * want.abs().max()
        o16 = torch.empty(M, N, device=DEV, dtype=torch.bfloat16)
        K.gemm(a, w, o16, scratch=scratch, kernel=code)
        assert (o16.double() - want).abs().max() < 1e-2 * want.abs().max()
        base = rnd(M, N, seed=3)
        acc = base.clone()
        K.gemm(a, w, acc, accumulate=True, scratch=scratch, kernel=code)
        assert (acc.double() - (base.double() + want)).abs().max() < 1e-4 * want.abs().max()
        if parts <= 1:
            I = 264 if M == 20 else 4104
            wg, wu = rnd(I, Kd, seed=4, scale=0.3, dtype=torch.bfloat16), rnd(I, Kd, seed=5, scale=0.3, dtype=torch.bfloat16)
            out = torch.empty(M, I, device=DEV, dtype=torch.bfloat16)
            wgu = K.interleave_gate_up(wg, wu)
            K.gemm_swiglu(a, K.block_weight(wgu) if blocked else wgu, out, kernel=code)
            g, u = a.double() @ wg.double().T, a.double() @ wu.double().T
            want2 = g / (1 + torch.exp(-g)) * u
            assert (out.double() - want2).abs().max() < 1e-2 * want2.abs().max()
        else:
            with pytest.raises(KernelError):             # the runs of a split product need scratch
                K.gemm(a, w, o32, kernel=code)
    with pytest.raises(KernelError):
        K.gemm(a, w, o32, scratch=scratch, kernel=8 + 16 * 3)       # 48 rows: no such tile


@pytest.mark.parametrize("M,H,Kd,N2", [(1, 1024, 1024, 304), (8, 1152, 2048, 4112), (13, 2048, 1280, 96), (16, 1024, 1536, 1000),
                                       (17, 1024, 2048, 304), (40, 2048, 1024, 4112), (64, 1280, 4096, 96)])
@pytest.mark.parametrize("blocked", [False, True])
def test_gemm_prepares_the_next_norm_and_the_next_product_uses_it(M, H, Kd, N2, blocked):
    # x += a W1^T, then rmsnorm(x) W2^T, in two kernels instead of three
    a = rnd(M, Kd, seed=1, scale=0.5, dtype=torch.bfloat16)
    w1 = rnd(H, Kd, seed=2, scale=0.05, dtype=torch.bfloat16)
    w2 = rnd(N2, H, seed=3, scale=0.5, dtype=torch.bfloat16)
    w1_rows, w2_rows = w1, w2
    if blocked:
        w1, w2 = K.block_weight(w1), K.block_weight(w2)
    x0 = rnd(M, H, seed=4) * torch.logspace(-1, 1, M, device=DEV)[:, None]     # rows of very different sizes
    gain = 1.0 + 0.5 * rnd(H, seed=5)
    eps = 1e-5
    x = x0.clone()
    xg = torch.empty(M, H, device=DEV, dtype=torch.bfloat16)
    ssq = torch.full(((H // 16) * K.SSQ_LD,), float("nan"), device=DEV)
    scratch = torch.full((K.GEMM_SCRATCH_FLOATS,), float("nan"), device=DEV) if M > 16 else None
    if M > 16:
        assert K.gemm_wide_parts(M, H, Kd, K.GEMM_SCRATCH_FLOATS) >= 2
    tiles = K.gemm_norm_prepare(a, w1, x, gain, xg, ssq, scratch)
    assert tiles == (H // 16 if M <= 16 else H // 256)
    xw = x0.double() + a.double() @ w1_rows.double().T
    assert (x.double() - xw).abs().max() < 1e-4 * xw.abs().max()
    assert (xg.double() - xw * gain.double()).abs().max() < 1e-2 * (xw * gain.double()).abs().max()
    sums = ssq[:tiles * K.SSQ_LD].view(tiles, K.SSQ_LD)[:, :M].double()
    assert (sums.sum(0) - (xw * xw).sum(-1)).abs().max() < 1e-4 * (xw * xw).sum(-1).max()
    normed = xw / torch.sqrt((xw * xw).mean(-1, keepdim=True) + eps) * gain.double()
    want = normed @ w2_rows.double().T
    o32 = torch.empty(M, N2, device=DEV)
    K.gemm_norm_scaled(xg, ssq, tiles, eps, w2, o32, scratch=scratch)
    assert (o32.double() - want).abs().max() < 1e-2 * want.abs().max()
    # against the same product with the rows normed by the norm kernel: bf16 roundings apart
    h = torch.empty(M, H, device=DEV, dtype=torch.bfloat16)
    K.rmsnorm(x, gain, h, eps, None)
    two = torch.empty(M, N2, device=DEV)
    K.gemm(h, w2, two)
    assert (o32 - two).abs().max() < 1e-2 * want.abs().max()
    o16 = torch.empty(M, N2, device=DEV, dtype=torch.bfloat16)
    K.gemm_norm_scaled(xg, ssq, tiles, eps, w2, o16, scratch=scratch)
    assert (o16.double() - want).abs().max() < 2e-2 * want.abs().max()
    if N2 % 16 == 0:
        out = torch.empty(M, N2 // 2, device=DEV, dtype=torch.bfloat16)
        K.gemm_norm_scaled(xg, ssq, tiles, eps, w2, out, swiglu=True, scratch=scratch)
        gu = want.view(M, N2 // 16, 2, 8)
        g, u = gu[:, :, 0].reshape(M, -1), gu[:, :, 1].reshape(M, -1)
        sw = g / (1 + torch.exp(-g)) * u
        assert (out.double() - sw).abs().max() < 2e-2 * sw.abs().max()
    with pytest.raises(KernelError):
        K.gemm_norm_prepare(rnd(65, Kd, dtype=torch.bfloat16), w1, torch.zeros(65, H, device=DEV), gain,
                            torch.empty(65, H, device=DEV, dtype=torch.bfloat16), ssq, scratch)


@pytest.mark.parametrize("kernel", [0, 4, 5, 6, 7, 8, 9, 10, 5 + 16 * 2, 6 + 16 * 4])
@pytest.mark.parametrize("M,N,Kd", [(1, 100, 1024), (8, 301, 1152), (16, 4100, 1024), (17, 200, 1280), (64, 16500, 1024),
                                    (48, 4100, 2048), (65, 301, 1024), (130, 514, 1152), (300, 700, 1024), (513, 260, 2048)])
def test_gemm_with_blocked_weights(M, N, Kd, kernel):
    # the weight as blocks of 16 rows x 128 k (block_weight): every kernel that takes it, every epilogue
    k = kernel % 16
    if k == 7 and M > 16 or k == 8 and not 16 < M <= 64 or k == 9 and M > 64:
        pytest.skip("not this kernel's rows")
    w_rows = rnd(N, Kd, seed=2, scale=0.5, dtype=torch.bfloat16)
    a, w = rnd(M, Kd, seed=1, scale=0.5, dtype=torch.bfloat16), K.block_weight(w_rows)
    assert w.shape == (-(-N // 16), Kd // 128, 16, 128) and torch.equal(K.unblock_weight(w, N), w_rows)
    want = a.double() @ w_rows.double().T
    scratch = torch.full((K.GEMM_SCRATCH_FLOATS,), float("nan"), device=DEV)
    o32 = torch.empty(M, N, device=DEV)
    K.gemm(a, w, o32, kernel=kernel, scratch=scratch)
    assert (o32.double() - want).abs().max() < 1e-4 * want.abs().max()
    rows = torch.empty(M, N, device=DEV)
    K.gemm(a, w_rows, rows, kernel=kernel, scratch=scratch)
    assert torch.equal(rows, o32)                                    # the layout changes no sum
    o16 = torch.empty(M, N + 8, device=DEV, dtype=torch.bfloat16)[:, 3:3 + N]
    K.gemm(a, w, o16, kernel=kernel, scratch=scratch)
    assert (o16.double() - want).abs().max() < 1e-2 * want.abs().max()
    base = rnd(M, N, seed=3)
    acc = base.clone()
    K.gemm(a, w, acc, accumulate=True, kernel=kernel, scratch=scratch)
    assert (acc.double() - (base.double() + want)).abs().max() < 1e-4 * want.abs().max()
    if kernel < 16:
        I = (N // 2) // 8 * 8
        wg, wu = rnd(I, Kd, seed=4, scale=0.3, dtype=torch.bfloat16), rnd(I, Kd, seed=5, scale=0.3, dtype=torch.bfloat16)
        out = torch.empty(M, I, device=DEV, dtype=torch.bfloat16)
        K.gemm_swiglu(a, K.block_weight(K.interleave_gate_up(wg, wu)), out, kernel=kernel)
        g, u = a.double() @ wg.double().T, a.double() @ wu.double().T
        sw = g / (1 + torch.exp(-g)) * u
        assert (out.double() - sw).abs().max() < 1e-2 * sw.abs().max()
    for bad in (1, 2, 3):
        with pytest.raises(KernelError):                 # these read rows only
            K.gemm(a, w, o32, kernel=bad)
    with pytest.raises(KernelError):
        K.gemm(a, w, torch.empty(M, N + 64, device=DEV))             # a width the blocks do not have
    with pytest.raises(KernelError):
        K.block_weight(rnd(64, 960, dtype=torch.bfloat16))           # K in steps of 128 from 1024


@pytest.mark.parametrize("blocked", [False, True])
@pytest.mark.parametrize("parts", [1, 2, 4])
@pytest.mark.parametrize("kernel", [12, 13, 14, 15])
@pytest.mark.parametrize("M,N,Kd", [(130, 516, 1024), (300, 700, 2048), (513, 264, 1152), (65, 1032, 1280), (260, 1500, 1024)])
def test_gemm_tiles_of_one_wave_per_simd(M, N, Kd, kernel, parts, blocked):
    """The 256x256, 128x256, 256x192 and 256x224 tiles of four waves (written-out instruction order, products kept
    transposed in the matrix-core registers): every epilogue, one run or several along k, either weight
    layout, tiles that hang over every edge; a strided output whose width is no multiple of four (the
    elements that no 16-byte store takes); and what they refuse."""
    code = kernel + (16 * parts if parts > 1 else 0)
    w_rows = rnd(N, Kd, seed=2, scale=0.5, dtype=torch.bfloat16)
    a, w = rnd(M, Kd, seed=1, scale=0.5, dtype=torch.bfloat16), (K.block_weight(w_rows) if blocked else w_rows)
    want = a.double() @ w_rows.double().T
    scratch = torch.full((K.GEMM_SCRATCH_FLOATS,), float("nan"), device=DEV)
    o32 = torch.empty(M, N, device=DEV)
    K.gemm(a, w, o32, kernel=code, scratch=scratch)
    assert (o32.double() - want).abs().max() < 1e-4 * want.abs().max()
    again = torch.full((M, N), float("nan"), device=DEV)
    K.gemm(a, w, again, kernel=code, scratch=scratch)
    assert torch.equal(again, o32)
    o16 = torch.empty(M, N + 8, device=DEV, dtype=torch.bfloat16)[:, 8:8 + N]
    K.gemm(a, w, o16, kernel=code, scratch=scratch)
    assert (o16.double() - want).abs().max() < 1e-2 * want.abs().max()
    base = rnd(M, N + 12, seed=3)
    acc = base.clone()
    K.gemm(a, w, acc[:, 4:4 + N], accumulate=True, kernel=code, scratch=scratch)
    assert (acc[:, 4:4 + N].double() - (base[:, 4:4 + N].double() + want)).abs().max() < 1e-4 * want.abs().max()
    assert torch.equal(acc[:, :4], base[:, :4]) and torch.equal(acc[:, 4 + N:], base[:, 4 + N:])
    I = (N // 2) // 8 * 8
    wg, wu = rnd(I, Kd, seed=4, scale=0.3, dtype=torch.bfloat16), rnd(I, Kd, seed=5, scale=0.3, dtype=torch.bfloat16)
    wgu = K.interleave_gate_up(wg, wu)
    out = torch.empty(M, I, device=DEV, dtype=torch.bfloat16)
    K.gemm_swiglu(a, K.block_weight(wgu) if blocked else wgu, out, kernel=code, scratch=scratch)
    g, u = a.double() @ wg.double().T, a.double() @ wu.double().T
    sw = g / (1 + torch.exp(-g)) * u
    assert (out.double() - sw).abs().max() < 1e-2 * sw.abs().max()
    if parts == 1 and not blocked:
        # a width of N - 2 inside rows of N floats: the last columns go out one by one, the neighbours stay
        wide = torch.full((M, N), 7.0, device=DEV)
        K.gemm(a, w_rows[:N - 2], wide[:, :N - 2], kernel=code)
        assert torch.equal(wide[:, :N - 2], o32[:, :N - 2]) and bool((wide[:, N - 2:] == 7.0).all())
    with pytest.raises(KernelError):                     # rows that no 16-byte store can take
        K.gemm(a, w, torch.empty(M, N + 6, device=DEV)[:, 3:3 + N], kernel=code, scratch=scratch)
    with pytest.raises(KernelError):
        K.gemm(a, w, torch.empty(M, N + 1, device=DEV)[:, :N], kernel=code, scratch=scratch)
    if parts > 1:
        with pytest.raises(KernelError):                 # forced runs need their room
            K.gemm(a, w, again, scratch=torch.empty(16, device=DEV), kernel=code)
    # chosen by shape: the same sums where these tiles are taken, and a right result where they are not
    chosen = torch.empty(M, N + 6, device=DEV)[:, 3:3 + N]
    K.gemm(a, w, chosen, scratch=scratch)
    assert (chosen.double() - want).abs().max() < 1e-4 * want.abs().max()


@pytest.mark.parametrize("mode", [0, 1, 2, 3])
def test_gemm_cut_along_weight_rows_into_whole_rounds_and_a_rest(mode):
    """1,024 x 17,408 x 4,096 is one round of 256x256 tiles over the chip and a sixteenth: the product goes as
    one whole round over the first 16,384 weight rows and another tile over the rest.  Every output mode: the
    same sums as the one tile over all rows, and right against double sums at sampled rows."""
    M, N, Kd = 1024, 17408, 4096
    kernel, parts, n1 = K.gemm_tile_choice(M, N, Kd, mode, K.GEMM_SCRATCH_FLOATS)
    assert 0 < n1 < N and n1 % 256 == 0 and kernel in (12, 13, 14, 15), (kernel, parts, n1)
    a = rnd(M, Kd, seed=1, scale=0.5, dtype=torch.bfloat16)
    w = rnd(N, Kd, seed=2, scale=0.05, dtype=torch.bfloat16)
    scratch = torch.full((K.GEMM_SCRATCH_FLOATS,), float("nan"), device=DEV)
    rows = torch.tensor([0, 1, 255, 256, 700, 1023], device=DEV)
    want = a[rows].double() @ w.double().T
    def run(kern):
        if mode == 3:
            out = torch.empty(M, N // 2, device=DEV, dtype=torch.bfloat16)
            K.gemm_swiglu(a, w, out, kernel=kern, scratch=scratch)
        elif mode == 0:
            out = torch.empty(M, N, device=DEV, dtype=torch.bfloat16)
            K.gemm(a, w, out, kernel=kern, scratch=scratch)
        else:
            out = torch.full((M, N), 0.25, device=DEV)
            K.gemm(a, w, out, accumulate=(mode == 2), kernel=kern, scratch=scratch)
        return out
    chosen, one = run(0), run(12)
    c1 = n1 // 2 if mode == 3 else n1                    # output columns of the first n1 weight rows
    assert torch.equal(chosen[:, :c1], one[:, :c1])      # the same tile, the same sums
    # the rest may be cut along k as well: float sums in another order, then the same rounding
    step = 1e-5 if mode in (1, 2) else 2.0 ** -7
    assert (chosen[:, c1:].float() - one[:, c1:].float()).abs().max() <= step * one.float().abs().max()
    if mode == 3:
        g = want.view(len(rows), N // 16, 2, 8)
        want = (g[:, :, 0] / (1 + torch.exp(-g[:, :, 0])) * g[:, :, 1]).reshape(len(rows), N // 2)
    elif mode == 2:
        want = want + 0.25
    tol = 1e-4 if mode in (1, 2) else 1e-2
    assert (chosen[rows].double() - want).abs().max() < tol * want.abs().max()


def test_gemm_reference_vectors():
    # tests/wmma_gemm_test.rs:27-69,72-114: sin/cos ramps times 0.5 / 0.3, tol 1e-3
    for M, N, Kd in ((32, 32, 64), (256, 256, 1024)):
        a = (0.5 * torch.sin(0.01 * torch.arange(M * Kd))).reshape(M, Kd).bfloat16().to(DEV)
        w = (0.3 * torch.cos(0.01 * torch.arange(N * Kd))).reshape(N, Kd).bfloat16().to(DEV)
        out = torch.empty(M, N, device=DEV)
        K.gemm(a, w, out)
        assert (out.double() - a.double() @ w.double().T).abs().max() < 1e-3


def test_gemm_strided_rows_and_refusals():
    wide = rnd(20, 300, dtype=torch.bfloat16)
    a = wide[:, 100:164]                       # a view: rows 600 bytes apart
    w = rnd(40, 64, seed=5, dtype=torch.bfloat16)
    out = torch.empty(20, 40, device=DEV)
    K.gemm(a, w, out)
    assert (out.double() - a.double() @ w.double().T).abs().max() < 1e-4 * 20
    with pytest.raises(KernelError):
        K.gemm(a, rnd(40, 65, dtype=torch.bfloat16), out)
    with pytest.raises(KernelError):
        K.gemm(a.float(), w, out)
    with pytest.raises(KernelError):
        K.gemm(a.cpu(), w.cpu(), out.cpu())


# ------------------------------------------------------------------ rotary, cache ----
def _rope_ref(x, pos, inv, adjacent):
    th = pos.double()[:, None] * inv.double()[None, :]
    c, s = th.cos()[:, None, :], th.sin()[:, None, :]
    P = inv.numel()
    y = x.double().clone()
    if adjacent:
        a, b = x[..., 0:2 * P:2].double(), x[..., 1:2 * P:2].double()
        y[..., 0:2 * P:2], y[..., 1:2 * P:2] = a * c - b * s, a * s + b * c
    else:
        a, b = x[..., :P].double(), x[..., P:2 * P].double()
        y[..., :P], y[..., P:2 * P] = a * c - b * s, a * s + b * c
    return y


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("adjacent", [False, True])
@pytest.mark.parametrize("nq,nkv,hd,rd", [(8, 2, 256, 64), (5, 5, 48, 48), (4, 1, 80, 80), (3, 1, 40, 20)])
@pytest.mark.parametrize("lens,starts", [([8, 128, 64], [0, 0, 32]), ([70, 128, 100], [0, 0, 32]), ([3, 17, 5], [0, 60, 32])])
def test_rope_and_paged_write(dtype, adjacent, nq, nkv, hd, rd, lens, starts):
    # sizes of tests/mrope_test.rs:5-13 (nq 8, nkv 2, hd 256, rotary 64, theta 1e7) among them;
    # page/offset cases of tests/op_kv_write_paged_batch_test.rs:196-198: starts 0 and 32, across pages.
    # Many tokens in bf16 with sizes in steps of 16 take the kernel that works on 64 tokens at a time,
    # everything else the one that takes a token at a time.
    page, theta = 64, 1e7
    T = sum(lens)
    pos = torch.cat([torch.arange(s, s + n) for s, n in zip(starts, lens)]).int().to(DEV)
    sot = torch.cat([torch.full((n,), b) for b, n in enumerate(lens)]).int().to(DEV)
    slots = i32([2, 0, 3])
    table = torch.full((4, 4), -1, dtype=torch.int32)
    table[2, 0], table[0, 0], table[0, 1], table[3, 0], table[3, 1] = 5, 1, 6, 0, 3
    table[2, 1], table[3, 2] = 2, 4
    table = table.to(DEV)
    inv = (1.0 / theta ** (torch.arange(0, rd, 2, dtype=torch.float32) / rd)).to(DEV)
    cs, sn = torch.empty(T, rd // 2, device=DEV), torch.empty(T, rd // 2, device=DEV)
    K.rope_table(pos, inv, cs, sn)
    th = pos.float()[:, None] * inv[None, :]
    assert (cs - th.cos()).abs().max() < 2e-6 and (sn - th.sin()).abs().max() < 2e-6
    qkv = rnd(T, (nq + 2 * nkv) * hd, dtype=dtype)
    src = qkv.clone()
    cache = torch.full((8, 2, nkv, page, hd), 99.0, device=DEV, dtype=dtype)
    K.rope_kv_write(qkv, cs, sn, pos, sot, slots, table, cache, nq, nkv, hd, rd, adjacent, page, True)
    q_in = src[:, :nq * hd].reshape(T, nq, hd).float()
    k_in = src[:, nq * hd:(nq + nkv) * hd].reshape(T, nkv, hd).float()
    v_in = src[:, (nq + nkv) * hd:].reshape(T, nkv, hd)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    q_want, k_want = _rope_ref(q_in, pos, inv, adjacent), _rope_ref(k_in, pos, inv, adjacent)
    assert (qkv[:, :nq * hd].reshape(T, nq, hd).double() - q_want).abs().max() < tol * q_want.abs().max()
    assert torch.equal(qkv[:, nq * hd:], src[:, nq * hd:])            # k and v rows of the step buffer are untouched
    written = torch.zeros(8, page, dtype=torch.bool)
    written_v = torch.zeros(8, page, dtype=torch.bool)
    for t in range(T):
        p, slot = int(pos[t]), int(slots[int(sot[t])])
        pg = int(table[slot, p // page])
        written[pg, p % page] = True
        assert (cache[pg, 0, :, p % page].double() - k_want[t]).abs().max() < tol * k_want.abs().max()
        vt = cache[pg, 1].reshape(nkv, hd, page)                      # values are stored transposed
        assert torch.equal(vt[:, :, p % page], v_in[t])                # and byte-equal
        written_v[pg, p % page] = True
    assert torch.all(cache[:, 0][~written[:, None, :].expand(8, nkv, page)] == 99.0)
    vt_all = cache[:, 1].reshape(8, nkv, hd, page).permute(0, 1, 3, 2)
    assert torch.all(vt_all[~written_v[:, None, :].expand(8, nkv, page)] == 99.0)
    # a padded sequence (slot -1) stores nothing; write_cache=False stores nothing
    cache2 = torch.full_like(cache, 99.0)
    K.rope_kv_write(src.clone(), cs, sn, pos, sot, i32([-1, -1, -1]), table, cache2, nq, nkv, hd, rd, adjacent, page, True)
    K.rope_kv_write(src.clone(), cs, sn, pos, sot, slots, table, cache2, nq, nkv, hd, rd, adjacent, page, False)
    assert torch.all(cache2 == 99.0)


# ------------------------------------------------------------------ attention ------
def _attn_ref(q, k, v, nq, nkv, window):
    T, hd = q.shape[0], q.shape[-1]
    i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
    mask = j <= i
    if window:
        mask &= j > i - window
    out = torch.zeros(T, nq, hd, dtype=torch.float64)
    for h in range(nq):
        s = q[:, h].double() @ k[:, h // (nq // nkv)].double().T / math.sqrt(hd)
        s = s.masked_fill(~mask, float("-inf"))
        out[:, h] = torch.softmax(s, -1) @ v[:, h // (nq // nkv)].double()
    return out


def _paged(k, v, pages, page, n_pages, dtype):
    """Scatter [T, nkv, hd] keys and values into a cache unit through a page list."""
    T, nkv, hd = k.shape
    cache = torch.zeros(n_pages, 2, nkv, page, hd, dtype=dtype, device=DEV)
    for t in range(T):
        cache[pages[t // page], 0, :, t % page] = k[t]
        cache[pages[t // page], 1].view(nkv, hd, page)[:, :, t % page] = v[t]      # values transposed
    return cache


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nq,nkv,hd,window", [(4, 2, 16, None), (6, 3, 32, 8), (5, 1, 48, 70), (8, 8, 128, None),
                                              (2, 1, 80, 100), (4, 4, 256, None)])
def test_attention_simple(dtype, nq, nkv, hd, window):
    page, T = 64, 150
    q, k, v = (rnd(T, n, hd, seed=s, dtype=dtype) for s, n in ((1, nq), (2, nkv), (3, nkv)))
    pages = [7, 2, 9]
    cache = _paged(k, v, pages, page, 12, dtype)
    table = torch.full((3, 4), -1, dtype=torch.int32); table[1, :3] = torch.tensor(pages); table = table.to(DEV)
    pos, sot, slots = torch.arange(T).int().to(DEV), torch.zeros(T).int().to(DEV), i32([1])
    out = torch.empty(T, nq * hd, device=DEV, dtype=dtype)
    qf = q.reshape(T, nq * hd).contiguous()
    K.attention_simple(qf, nq * hd, out, pos, sot, slots, table, cache, T, nq, nkv, hd, page, window, 1 / math.sqrt(hd))
    want = _attn_ref(q.cpu(), k.cpu(), v.cpu(), nq, nkv, window)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert (out.reshape(T, nq, hd).cpu().double() - want).abs().max() < tol * want.abs().max()
    # the last 20 queries alone (decode-like: queries whose keys were stored earlier)
    out2 = torch.empty(20, nq * hd, device=DEV, dtype=dtype)
    K.attention_simple(qf[-20:].contiguous(), nq * hd, out2, pos[-20:].contiguous(), sot[:20].contiguous(), slots, table,
                       cache, 20, nq, nkv, hd, page, window, 1 / math.sqrt(hd))
    assert torch.equal(out2, out[-20:])


def test_attention_one_key_and_uniform_scores():
    hd, page = 32, 64
    k = torch.zeros(5, 1, hd); v = rnd(5, 1, hd, seed=4).cpu()
    cache = _paged(k.to(DEV), v.to(DEV), [0], page, 1, torch.float32)
    q = rnd(5, 2 * hd, seed=5)
    table = i32([[0]])
    out = torch.empty(5, 2 * hd, device=DEV)
    K.attention_simple(q, 2 * hd, out, i32([0, 1, 2, 3, 4]), i32([0] * 5), i32([0]), table, cache, 5, 2, 1, hd, page, None, 1.0)
    o = out.reshape(5, 2, hd).cpu()
    assert torch.allclose(o[0, 0], v[0, 0], atol=1e-6)                            # one key: its value
    assert torch.allclose(o[4, 1], v[:, 0].mean(0), atol=1e-6)                    # equal scores: the mean


# ----------------------------------------------------------------- elementwise ------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_silu_mul_and_residual(dtype):
    # tests/op_silu_mul_test.rs:37-81: g = 3 sin(0.011 i), u = cos(0.009 i), tol 1e-3
    I = 1025
    i = torch.arange(3 * I, dtype=torch.float32)
    g, u = (3 * torch.sin(0.011 * i)).reshape(3, I), torch.cos(0.009 * i).reshape(3, I)
    gu = torch.cat([g, u], dim=1).to(dtype).to(DEV)
    out = torch.empty(3, I, device=DEV, dtype=dtype)
    K.silu_mul(gu, out)
    gd, ud = gu[:, :I].double(), gu[:, I:].double()
    want = gd / (1 + torch.exp(-gd)) * ud
    assert (out.double() - want).abs().max() < (1e-6 if dtype == torch.float32 else 1e-2)
    x, y = rnd(1000, seed=1), rnd(1000, seed=2, dtype=dtype)
    want = x + y.float()
    K.residual_add(x, y)
    assert torch.equal(x, want)                                                   # tests/op_residual_add_test.rs: exact


def test_gather_and_convert():
    x = rnd(9, 100)
    out = torch.empty(3, 100, device=DEV)
    K.gather_rows(x, i32([8, 0, 8]), out)
    assert torch.equal(out, x[[8, 0, 8]])
    b = torch.empty(9, 100, device=DEV, dtype=torch.bfloat16)
    K.convert(x, b)
    assert torch.equal(b, x.bfloat16())                                           # round to nearest even
    back = torch.empty_like(x)
    K.convert(b, back)
    assert torch.equal(back, b.float())


# -------------------------------------------------------------------- sampling ------
def test_argmax_lowest_index_wins():
    l = rnd(5, 32768 + 3)
    l[1, 100] = l[1, 20000] = 50.0
    l[2, :] = 0.0
    l[3, 32770] = 60.0
    out = torch.empty(5, dtype=torch.int32, device=DEV)
    K.argmax(l, out)
    want = [int(l[0].argmax()), 100, 0, 32770, int(l[4].argmax())]
    assert out.tolist() == want
    # reference vector: greedy on [0.1, 0.5, 0.2, 0.8, 0.3] -> 3 (sampling.rs:232-241)
    K.argmax(torch.tensor([[0.1, 0.5, 0.2, 0.8, 0.3]], device=DEV), out)
    assert out[0].item() == 3


# ------------------------------------------- matrix-core attention kernels (bf16) ----
def _multi_seq_cache(lens, nkv, hd, seed):
    """Keys/values of several sequences scattered over shuffled pages: (k, v lists, cache, table)."""
    page = 64
    n_pages = sum(-(-n // page) for n in lens) + 3
    order = torch.randperm(n_pages, generator=torch.Generator().manual_seed(seed)).tolist()
    # stale, non-zero contents in every page: a kernel that reads beyond a sequence's end shows
    cache = torch.full((n_pages, 2, nkv, page, hd), 7.0, dtype=torch.bfloat16, device=DEV)
    table = torch.full((len(lens) + 2, max(-(-n // page) for n in lens) + 1), -1, dtype=torch.int32)
    ks, vs = [], []
    for b, n in enumerate(lens):
        k, v = rnd(n, nkv, hd, seed=seed + 10 * b + 1, dtype=torch.bfloat16), rnd(n, nkv, hd, seed=seed + 10 * b + 2, dtype=torch.bfloat16)
        ks.append(k); vs.append(v)
        for i in range(-(-n // page)):
            pg = order.pop()
            table[b + 1, i] = pg                       # sequence b lives in slot b + 1
            m = min(page, n - i * page)
            cache[pg, 0, :, :m] = k[i * page:i * page + m].permute(1, 0, 2)
            cache[pg, 1].view(nkv, hd, page)[:, :, :m] = v[i * page:i * page + m].permute(1, 2, 0)
    return ks, vs, cache, table.to(DEV)


@pytest.mark.parametrize("nq,nkv,hd,window", [(4, 2, 16, None), (6, 3, 32, 8), (5, 1, 48, 70), (32, 8, 128, None),
                                              (8, 2, 128, 100), (3, 3, 80, None), (2, 1, 256, 33), (20, 1, 64, None)])
@pytest.mark.parametrize("variant", [1, 2, 3, 4])
def test_attention_prefill_matrix_cores(nq, nkv, hd, window, variant):
    if variant == 4 and hd not in (64, 128):
        pytest.skip("the ring of direct loads takes head sizes 64 and 128")
    lens = [200, 37, 64, 1, 130]             # lengths after the step
    new = [200, 30, 3, 1, 65]                # tokens of this step (the rest is earlier context)
    ks, vs, cache, table = _multi_seq_cache(lens, nkv, hd, seed=nq + hd)
    T = sum(new)
    q = rnd(T, nq, hd, seed=99, dtype=torch.bfloat16)
    cu = [0]
    for n in new:
        cu.append(cu[-1] + n)
    out = torch.full((T, nq * hd), 5.0, device=DEV, dtype=torch.bfloat16)
    K.attention_prefill_bf16(q.reshape(T, nq * hd), nq * hd, out, i32(cu), i32([1, 2, 3, 4, 5]), i32(lens), table, cache,
                             len(lens), max(new), nq, nkv, hd, 64, window, 1 / math.sqrt(hd), variant)
    pos = torch.cat([torch.arange(l - n, l) for l, n in zip(lens, new)]).int().to(DEV)
    sot = torch.cat([torch.full((n,), b) for b, n in enumerate(new)]).int().to(DEV)
    simple = torch.empty_like(out)
    K.attention_simple(q.reshape(T, nq * hd), nq * hd, simple, pos, sot, i32([1, 2, 3, 4, 5]), table, cache, T, nq, nkv, hd,
                       64, window, 1 / math.sqrt(hd))
    for b, (l, n) in enumerate(zip(lens, new)):
        qq = torch.zeros(l, nq, hd); qq[l - n:] = q[cu[b]:cu[b + 1]].float().cpu()
        want = _attn_ref(qq, ks[b].float().cpu(), vs[b].float().cpu(), nq, nkv, window)[l - n:]
        got = out[cu[b]:cu[b + 1]].reshape(n, nq, hd).cpu().double()
        assert torch.isfinite(got).all()
        assert (got - want).abs().max() < 2e-2 * want.abs().max(), f"sequence {b}"
        assert (got - simple[cu[b]:cu[b + 1]].reshape(n, nq, hd).cpu().double()).abs().max() < 2e-2 * want.abs().max()


@pytest.mark.parametrize("variant", [1, 2])
@pytest.mark.parametrize("nsplit", [1, 2, 5, 16])
@pytest.mark.parametrize("nq,nkv,hd,window", [(4, 2, 16, None), (6, 3, 32, 8), (5, 1, 48, 70), (32, 8, 128, None),
                                              (8, 2, 128, 100), (2, 1, 256, 33), (20, 1, 64, None), (8, 4, 64, 70)])
def test_attention_decode_matrix_cores(nq, nkv, hd, window, nsplit, variant):
    if variant == 2 and hd not in (64, 128):
        pytest.skip("the kernel that brings pages through LDS takes head sizes 64 and 128")
    lens = [200, 37, 64, 1, 130, 65, 513]
    ks, vs, cache, table = _multi_seq_cache(lens, nkv, hd, seed=nq + hd + 1)
    B = len(lens)
    q = rnd(B + 1, nq, hd, seed=98, dtype=torch.bfloat16)        # the last row is padding (slot -1)
    slots = i32(list(range(1, B + 1)) + [-1])
    ctx = i32(lens + [0])
    out = torch.full((B + 1, nq * hd), 5.0, device=DEV, dtype=torch.bfloat16)
    part_o = torch.empty((B + 1) * nq * nsplit * hd, device=DEV)
    part_ml = torch.empty((B + 1) * nq * nsplit * 2, device=DEV)
    K.attention_decode_bf16(q.reshape(B + 1, nq * hd), nq * hd, out, slots, ctx, table, cache, B + 1, nq, nkv, hd, 64,
                            window, 1 / math.sqrt(hd), nsplit, part_o, part_ml, variant)
    assert torch.all(out[B] == 0)                                  # padding gives zeros, not garbage
    for b, l in enumerate(lens):
        qq = torch.zeros(l, nq, hd); qq[-1] = q[b].float().cpu()
        want = _attn_ref(qq, ks[b].float().cpu(), vs[b].float().cpu(), nq, nkv, window)[-1]
        got = out[b].reshape(nq, hd).cpu().double()
        assert torch.isfinite(got).all()
        assert (got - want).abs().max() < 2e-2 * want.abs().max(), f"sequence {b} of length {l}"


@pytest.mark.parametrize("rope", [True, False])
@pytest.mark.parametrize("nsplit", [1, 3])
@pytest.mark.parametrize("nq,nkv,hd,window", [(32, 8, 128, None), (8, 2, 128, 100), (16, 1, 64, None), (8, 4, 64, 70)])
def test_attention_decode_with_rotation_and_cache_write_fused(nq, nkv, hd, window, nsplit, rope):
    """The kernel that rotates and stores the new token itself against rope_kv_write followed
    by the same kernel: the cache afterwards and the outputs."""
    lens = [200, 37, 64, 1, 130, 65, 513, 128]                   # the new token included; 64, 65, 128, 1: page edges
    B, page, theta = len(lens), 64, 1e6
    _, _, cache, table = _multi_seq_cache(lens, nkv, hd, seed=nq + hd + 7)
    qkv = rnd(B + 1, (nq + 2 * nkv) * hd, seed=5, dtype=torch.bfloat16)      # the last row is padding (slot -1)
    slots = i32(list(range(1, B + 1)) + [-1])
    ctx = i32(lens + [0])
    pos = i32([l - 1 for l in lens] + [0])
    sot = torch.arange(B + 1).int().to(DEV)
    cs = sn = None
    if rope:
        inv = (1.0 / theta ** (torch.arange(0, hd, 2, dtype=torch.float32) / hd)).to(DEV)
        cs, sn = torch.empty(B + 1, hd // 2, device=DEV), torch.empty(B + 1, hd // 2, device=DEV)
        K.rope_table(pos, inv, cs, sn)
    part = lambda: (torch.empty((B + 1) * nq * nsplit * hd, device=DEV), torch.empty((B + 1) * nq * nsplit * 2, device=DEV))
    # two steps
    qkv2, cache2 = qkv.clone(), cache.clone()
    K.rope_kv_write(qkv2, cs, sn, pos, sot, slots, table, cache2, nq, nkv, hd, hd if rope else 0, False, page, True)
    want = torch.full((B + 1, nq * hd), 5.0, device=DEV, dtype=torch.bfloat16)
    po, pml = part()
    K.attention_decode_bf16(qkv2, qkv2.stride(0), want, slots, ctx, table, cache2, B + 1, nq, nkv, hd, page, window,
                            1 / math.sqrt(hd), nsplit, po, pml, 2)
    # one
    assert K.attention_decode_fuses_rope(hd, nq, nkv, page, table.shape[1], nsplit)
    qkv1, cache1 = qkv.clone(), cache.clone()
    got = torch.full((B + 1, nq * hd), 5.0, device=DEV, dtype=torch.bfloat16)
    po, pml = part()
    K.attention_decode_bf16(qkv1, qkv1.stride(0), got, slots, ctx, table, cache1, B + 1, nq, nkv, hd, page, window,
                            1 / math.sqrt(hd), nsplit, po, pml, 2, True, cs, sn, True)
    assert torch.equal(cache1[:, 1], cache2[:, 1])                             # values: copied
    assert (cache1[:, 0].float() - cache2[:, 0].float()).abs().max() <= 2 ** -7 * cache2[:, 0].float().abs().max()
    assert torch.all(got[B] == 0)
    scale = want[:B].float().abs().max()
    assert (got[:B].float() - want[:B].float()).abs().max() <= 2e-2 * scale
    # write_cache=False leaves the cache alone
    cache3 = cache.clone()
    K.attention_decode_bf16(qkv.clone(), qkv.stride(0), got, slots, ctx, table, cache3, B + 1, nq, nkv, hd, page, window,
                            1 / math.sqrt(hd), nsplit, po, pml, 2, True, cs, sn, False)
    assert torch.equal(cache3, cache)
    with pytest.raises(KernelError):
        K.attention_decode_bf16(qkv1, qkv1.stride(0), got, slots, ctx, table, cache1, B + 1, 34, 2, hd, page, window,
                                1 / math.sqrt(hd), nsplit, po, pml, 2, True, cs, sn, True)


@pytest.mark.parametrize("normed", [False, True])
@pytest.mark.parametrize("rows,nq,nkv,hd,width,window", [(24, 8, 2, 128, 1024, None), (64, 32, 8, 128, 4096, None),
                                                          (40, 16, 1, 64, 512, 70), (17, 4, 4, 64, 1536, None)])
def test_attention_decode_adds_the_runs_of_its_rows_itself(rows, nq, nkv, hd, width, window, normed):
    """A product of 17 to 64 rows that is cut along k may leave its runs' sums, and the fused
    decode attention adds them for the heads it reads: outputs and cache must have the bits
    of the product summed by its own kernel followed by the same attention."""
    B, page, nsplit = rows, 64, 2
    lens = [int(x) for x in np.random.default_rng(rows).integers(1, 400, B)]
    lens[0], lens[1], lens[2] = 64, 65, 1
    _, _, cache, table = _multi_seq_cache(lens, nkv, hd, seed=rows + hd)
    n_out = (nq + 2 * nkv) * hd
    a = rnd(B, width, seed=3, dtype=torch.bfloat16)
    w = rnd(n_out, width, seed=4, scale=0.05, dtype=torch.bfloat16)
    scratch = torch.empty(K.GEMM_SCRATCH_FLOATS, device=DEV)
    slots, ctx = i32(list(range(1, B + 1))), i32(lens)
    pos = i32([l - 1 for l in lens])
    inv = (1.0 / 1e4 ** (torch.arange(0, hd, 2, dtype=torch.float32) / hd)).to(DEV)
    cs, sn = torch.empty(B, hd // 2, device=DEV), torch.empty(B, hd // 2, device=DEV)
    K.rope_table(pos, inv, cs, sn)
    ssq, tiles, eps = None, 0, 1e-5
    if normed:          # the rows as a product before left them for an RMS norm: sums of squares in tiles
        tiles = width // 256
        ssq = torch.zeros(tiles * K.SSQ_LD, device=DEV)
        ssq.view(tiles, K.SSQ_LD)[:, :B] = (a.float() ** 2).view(B, tiles, 256).sum(-1).t()
    part = lambda: (torch.empty(B * nq * nsplit * hd, device=DEV), torch.empty(B * nq * nsplit * 2, device=DEV))
    # the product summed by its own kernel, then attention
    qkv = torch.empty(B, n_out, device=DEV, dtype=torch.bfloat16)
    if normed:
        K.gemm_norm_scaled(a, ssq, tiles, eps, w, qkv, scratch=scratch)
    else:
        K.gemm(a, w, qkv, scratch=scratch)
    cache_a, want = cache.clone(), torch.empty(B, nq * hd, device=DEV, dtype=torch.bfloat16)
    po, pml = part()
    K.attention_decode_bf16(qkv, n_out, want, slots, ctx, table, cache_a, B, nq, nkv, hd, page, window, 1 / math.sqrt(hd),
                            nsplit, po, pml, 2, True, cs, sn, True)
    # the runs left, attention adds them
    scratch.fill_(float("nan"))
    runs = K.gemm_wide_partial(a, w, n_out, scratch, ssq, tiles, eps)
    if K.gemm_wide_parts(B, n_out, width, K.GEMM_SCRATCH_FLOATS) < 2:
        assert runs == 0
        return
    assert runs >= 2
    summed = scratch[:runs * B * n_out].view(runs, B, n_out)
    total = summed[0].clone()
    for r in range(1, runs):
        total += summed[r]
    assert torch.equal(total.to(torch.bfloat16), qkv)
    cache_b, got = cache.clone(), torch.empty(B, nq * hd, device=DEV, dtype=torch.bfloat16)
    po, pml = part()
    K.attention_decode_bf16(torch.empty(0, device=DEV, dtype=torch.bfloat16), n_out, got, slots, ctx, table, cache_b, B,
                            nq, nkv, hd, page, window, 1 / math.sqrt(hd), nsplit, po, pml, 0, True, cs, sn, True, scratch, runs)
    assert torch.equal(cache_a, cache_b) and torch.equal(got, want)
    with pytest.raises(KernelError):      # run sums without the fused rotation
        K.attention_decode_bf16(qkv, n_out, got, slots, ctx, table, cache_b, B, nq, nkv, hd, page, window,
                                1 / math.sqrt(hd), nsplit, po, pml, 0, False, None, None, True, scratch, runs)


def test_attention_kernels_refuse_what_they_do_not_take():
    q = rnd(4, 2 * 24, dtype=torch.bfloat16)
    cache = torch.zeros(2, 2, 1, 64, 24, dtype=torch.bfloat16, device=DEV)
    out = torch.empty(4, 48, device=DEV, dtype=torch.bfloat16)
    with pytest.raises(KernelError, match="multiple of 16"):
        K.attention_decode_bf16(q, 48, out, i32([0, 0, 0, 0]), i32([1, 1, 1, 1]), i32([[0]]), cache, 4, 2, 1, 24, 64, None,
                                1.0, 1, None, None)
    with pytest.raises(KernelError, match="multiple of 16"):
        K.attention_prefill_bf16(q, 48, out, i32([0, 4]), i32([0]), i32([4]), i32([[0]]), cache, 1, 4, 2, 1, 24, 64, None, 1.0)


@pytest.mark.parametrize("kernel", [0, 1, 2, 3, 4, 5, 6, 7, 8, 10, 11, 12, 13, 14, 15])
@pytest.mark.parametrize("M,I,Kd", [(40, 8264, 256), (64, 328, 1152), (1, 64, 64), (8, 192, 96), (17, 320, 64), (64, 1024, 264), (130, 328, 100), (300, 512, 1032),
                                    (300, 512, 1024), (129, 200, 192), (1, 2056, 1024), (8, 328, 1152), (13, 4400, 1280),
                                    (100, 264, 4096), (260, 520, 2048)])
def test_gemm_with_swiglu_epilogue(M, I, Kd, kernel):
    _skip_unless_kernel_takes(kernel, M, Kd, I)
    a = rnd(M, Kd, seed=1, scale=0.5, dtype=torch.bfloat16)
    wg, wu = rnd(I, Kd, seed=2, scale=0.3, dtype=torch.bfloat16), rnd(I, Kd, seed=3, scale=0.3, dtype=torch.bfloat16)
    out = torch.empty(M, I, device=DEV, dtype=torch.bfloat16)
    K.gemm_swiglu(a, K.interleave_gate_up(wg, wu), out, kernel=kernel)
    g, u = a.double() @ wg.double().T, a.double() @ wu.double().T
    want = g / (1 + torch.exp(-g)) * u
    assert (out.double() - want).abs().max() < 1e-2 * want.abs().max()
    if kernel == 0:
        # with scratch a product of few tiles may be cut along k; the sum applies the same epilogue
        out2 = torch.empty_like(out)
        K.gemm_swiglu(a, K.interleave_gate_up(wg, wu), out2, scratch=torch.full((K.GEMM_SCRATCH_FLOATS,), float("nan"), device=DEV))
        assert (out2.double() - want).abs().max() < 1e-2 * want.abs().max()


@pytest.mark.parametrize("blocked", [False, True])
def test_gemm_swiglu_over_two_tile_shapes(blocked):
    # 2,048 x 28,672: the chooser covers 24,576 weight rows with 256x256 tiles (whole rounds of them) and the
    # other 4,096 with 128x256 tiles, in two launches; every tile kernel sums k in the same order, so the
    # result equals that of one tile shape bit for bit
    M, I, Kd = 2048, 14336, 1024
    a = rnd(M, Kd, seed=1, scale=0.5, dtype=torch.bfloat16)
    wg, wu = rnd(I, Kd, seed=2, scale=0.3, dtype=torch.bfloat16), rnd(I, Kd, seed=3, scale=0.3, dtype=torch.bfloat16)
    w = K.interleave_gate_up(wg, wu)
    if blocked:
        w = K.block_weight(w)
    out = torch.full((M, I), float("nan"), device=DEV, dtype=torch.bfloat16)
    K.gemm_swiglu(a, w, out)
    one = torch.empty_like(out)
    K.gemm_swiglu(a, w, one, kernel=5)
    assert torch.equal(out, one)
    g, u = a.float() @ wg.float().T, a.float() @ wu.float().T
    want = g / (1 + torch.exp(-g)) * u
    assert (out.float() - want).abs().max() < 1e-2 * want.abs().max()


# ------------------------------------------------------- long contexts, serving head size ----
def _long_cache(lens, nkv, hd, seed, first_live_page=None):
    """Keys and values of long sequences put into shuffled pages with vector operations:
    (k, v as float64 CPU tensors per sequence, cache, table).  Slots beyond a sequence's end
    hold 7.0, so a kernel that reads past the end shows.  `first_live_page[b]`: pages before it
    are given back (-1 in the table), as the cache does behind a window."""
    page = 64
    pages_of = [-(-n // page) for n in lens]
    n_pages = sum(pages_of) + 5
    g = torch.Generator().manual_seed(seed)
    order = torch.randperm(n_pages, generator=g)
    cache = torch.full((n_pages, 2, nkv, page, hd), 7.0, dtype=torch.bfloat16, device=DEV)
    table = torch.full((len(lens) + 1, max(pages_of) + 2), -1, dtype=torch.int32)
    ks, vs, used = [], [], 0
    for b, n in enumerate(lens):
        np_ = pages_of[b]
        k = torch.randn(np_ * page, nkv, hd, generator=g).to(torch.bfloat16)
        v = torch.randn(np_ * page, nkv, hd, generator=g).to(torch.bfloat16)
        pg = order[used:used + np_]
        used += np_
        table[b + 1, :np_] = pg.int()
        kk, vv = k.clone(), v.clone()
        kk[n:], vv[n:] = 7.0, 7.0
        cache[pg.to(DEV), 0] = kk.view(np_, page, nkv, hd).permute(0, 2, 1, 3).to(DEV)
        cache[pg.to(DEV), 1] = vv.view(np_, page, nkv, hd).permute(0, 2, 3, 1).reshape(np_, nkv, page, hd).to(DEV)   # [hd, token] in memory
        if first_live_page is not None and first_live_page[b] > 0:
            table[b + 1, :first_live_page[b]] = -1
        ks.append(k[:n].double()); vs.append(v[:n].double())
    return ks, vs, cache, table.to(DEV)


def _rows_ref(q_rows, q_pos, k, v, nq, nkv, window):
    """float64 attention of a few query rows (at positions q_pos) over keys 0..pos."""
    hd = q_rows.shape[-1]
    out = torch.zeros(len(q_pos), nq, hd, dtype=torch.float64)
    j = torch.arange(k.shape[0])
    for r, p in enumerate(q_pos):
        see = j <= p
        if window:
            see &= j > p - window
        for h in range(nq):
            kh = h // (nq // nkv)
            s = (k[see, kh] @ q_rows[r, h].double()) / math.sqrt(hd)
            out[r, h] = torch.softmax(s, 0) @ v[see, kh]
    return out


@pytest.mark.parametrize("variant", [1, 2])
@pytest.mark.parametrize("nsplit", [1, 8, 32, 64])
@pytest.mark.parametrize("window", [None, 4096])
def test_attention_decode_over_long_contexts(window, nsplit, variant):
    """Head size 128 and contexts of thousands of tokens: runs of many pages per split, splits
    that get no page at all, a window of 4,096 far into the sequence with the pages behind it
    given back."""
    from braidinfer_amd.parts.attention import decode_splits
    nq, nkv, hd = 8, 2, 128
    lens = [5000, 20000, 32768, 4097, 300]
    first = [max(0, n - window + 1) // 64 if window else 0 for n in lens]
    ks, vs, cache, table = _long_cache(lens, nkv, hd, seed=3, first_live_page=first)
    B = len(lens)
    q = rnd(B, nq, hd, seed=97, dtype=torch.bfloat16)
    want = [_rows_ref(q[b:b + 1].cpu(), [l - 1], ks[b], vs[b], nq, nkv, window)[0] for b, l in enumerate(lens)]
    for ns in {nsplit, decode_splits(B, nkv, max(lens), 64)}:
        out = torch.full((B, nq * hd), 5.0, device=DEV, dtype=torch.bfloat16)
        part_o = torch.full((B * nq * ns * hd,), float("nan"), device=DEV)
        part_ml = torch.full((B * nq * ns * 2,), float("nan"), device=DEV)
        K.attention_decode_bf16(q.reshape(B, nq * hd), nq * hd, out, i32(list(range(1, B + 1))), i32(lens), table, cache, B,
                                nq, nkv, hd, 64, window, 1 / math.sqrt(hd), ns, part_o, part_ml, variant)
        for b in range(B):
            got = out[b].reshape(nq, hd).cpu().double()
            assert torch.isfinite(got).all(), (b, ns)
            assert (got - want[b]).abs().max() < 2e-2 * want[b].abs().max(), f"sequence of {lens[b]}, {ns} splits"


def test_decode_splits_double_beyond_64_pages_a_run():
    from braidinfer_amd.parts.attention import decode_splits
    assert decode_splits(64, 8, 4096, 64) == 1 and decode_splits(1, 8, 2048, 64) == 16
    assert decode_splits(64, 8, 20000, 64) == 8 and decode_splits(64, 8, 32768, 64) == 8       # 313 and 512 pages: runs of at most 64
    assert decode_splits(8, 8, 32768, 64) == 8 and decode_splits(1, 8, 32768, 64) == 32
    for b in (1, 3, 8, 100):
        for ctx in (1, 64, 65, 5000, 100000, 1 << 20):
            n = decode_splits(b, 8, ctx, 64)
            assert 1 <= n < 128 and (n >= 64 or -(-(-(-ctx // 64)) // n) <= 64)
    # a chip with other compute units is filled likewise: about one workgroup each
    assert decode_splits(1, 8, 2048, 64, cus=128) == 16 and decode_splits(1, 8, 4096, 64, cus=304) == 32


@pytest.mark.parametrize("variant", [3, 4])
@pytest.mark.parametrize("window", [None, 4096])
def test_attention_prefill_chunks_over_long_contexts(window, variant):
    """Chunks of 64, 1 and 200 new tokens over 8,192, 20,000 and 4,000 earlier ones at head
    size 128: thousands of earlier keys through the ring, the window's edge inside a page far
    from the start, pages behind the window given back."""
    nq, nkv, hd = 8, 2, 128
    new = [64, 1, 200]
    lens = [8192 + 64, 20001, 4200]
    first = [max(0, (l - n) - window + 1) // 64 if window else 0 for l, n in zip(lens, new)]
    ks, vs, cache, table = _long_cache(lens, nkv, hd, seed=4, first_live_page=first)
    T = sum(new)
    q = rnd(T, nq, hd, seed=96, dtype=torch.bfloat16)
    cu = [0, 64, 65, 265]
    out = torch.full((T, nq * hd), 5.0, device=DEV, dtype=torch.bfloat16)
    K.attention_prefill_bf16(q.reshape(T, nq * hd), nq * hd, out, i32(cu), i32([1, 2, 3]), i32(lens), table, cache, 3,
                             max(new), nq, nkv, hd, 64, window, 1 / math.sqrt(hd), variant)
    for b, (l, n) in enumerate(zip(lens, new)):
        rows = sorted({0, n // 2, n - 1})                         # the chunk's first, middle and last query
        want = _rows_ref(q[cu[b]:cu[b + 1]].cpu()[rows], [l - n + r for r in rows], ks[b], vs[b], nq, nkv, window)
        got = out[cu[b]:cu[b + 1]].reshape(n, nq, hd).cpu().double()[rows]
        assert torch.isfinite(out[cu[b]:cu[b + 1]].float()).all()
        assert (got - want).abs().max() < 2e-2 * want.abs().max(), f"sequence {b}"


def test_stream_copy_and_read():
    n = (1 << 20) + 48
    src = torch.randint(-1000, 1000, (n // 4,), device=DEV).float()
    dst = torch.zeros_like(src)
    K.stream_copy(src, dst)
    assert torch.equal(src, dst)
    sums = torch.zeros(K.device_cus() * 32, device=DEV)
    K.stream_read(src, sums)
    assert sums.double().sum().item() == src.double().sum().item()         # integers: every word read exactly once
    with pytest.raises(KernelError):
        K.stream_copy(src[:-1], dst[:-1])                                    # not a multiple of 16 bytes
