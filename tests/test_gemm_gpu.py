"""GPU parity tests of the fp16 GEMM: the HIP kernels called through the C ABI (ctypes) and through the torch
operators, compared with the CPU oracle on the same seeded inputs. Tolerance (stated by the benchmark definition):
|err| <= 2e-2*sqrt(K/1024) + 1e-2*|ref| element-wise and max|err| / max|ref| <= 1e-2; cases whose exact answer is
representable are compared bit-exactly."""
import os

import numpy as np
import pytest
import torch

import serving_oracle as so

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def run(lib, gpu, a, b, layout="NN", variant=0):
    c = lib.hgemm(a.to(gpu), b.to(gpu), layout, variant=variant)
    torch.cuda.synchronize()
    return c.cpu()


def check(lib, gpu, a, b, layout, K, variant=0):
    c = run(lib, gpu, a, b, layout, variant)
    ok, st = so.gemm_tolerance_ok(c, so.gemm_ref(a, b, layout), K)
    assert ok, (layout, tuple(a.shape), tuple(b.shape), st)
    return c


def operands(M, N, K, layout, seed=0, a_std=1.0, b_std=1.0):
    a, b = so.gemm_inputs(M, N, K, seed, a_std, b_std)
    if layout == "TN":
        a = a.t().contiguous()
    if layout == "NT":
        b = b.t().contiguous()
    return a, b


# ---- benchmark configurations --------------------------------------------------------------------------------
def test_config_g1_1024_cubed(lib, gpu):
    a, b = so.gemm_inputs(1024, 1024, 1024, seed=0)
    check(lib, gpu, a, b, "NN", 1024)


@pytest.mark.parametrize("M,N,K", [(4096, 4096, 4096), (8192, 8192, 8192), (16, 14336, 4096)])
def test_config_g2_llm_projection_shapes(lib, gpu, M, N, K):
    a, b = so.gemm_inputs(M, N, K, seed=0, a_std=1.0, b_std=0.02)
    check(lib, gpu, a, b, "NN", K)


# ---- closed forms: exact answers ---------------------------------------------------------------------------------
@pytest.mark.parametrize("n", [256, 512, 96])
def test_identity_and_permutation_are_exact(lib, gpu, n):
    b = so.randn_fp16((n, n), 3)
    assert torch.equal(run(lib, gpu, torch.eye(n).half(), b), b)
    perm = torch.randperm(n, generator=torch.Generator().manual_seed(1))
    p = torch.zeros(n, n).half()
    p[torch.arange(n), perm] = 1
    assert torch.equal(run(lib, gpu, p, b), b[perm])               # rows of b picked by A
    assert torch.equal(run(lib, gpu, b, p), b[:, torch.argsort(perm)])  # columns of b picked by B
    assert torch.equal(run(lib, gpu, p.t().contiguous(), b, "TN"), b[perm])
    assert torch.equal(run(lib, gpu, p, b.t().contiguous(), "NT"), b[perm])


@pytest.mark.parametrize("K", [64, 1024, 2048])
def test_all_ones_counts_k(lib, gpu, K):
    c = run(lib, gpu, torch.ones(256, K).half(), torch.ones(K, 512).half())
    assert torch.equal(c, torch.full((256, 512), float(K)).half())


def test_power_of_two_operands_single_rounding(lib, gpu):
    # every product and partial sum is exact in fp32, so the only rounding is the final fp32 -> fp16 one
    g = torch.Generator().manual_seed(5)
    a = torch.ldexp(torch.ones(256, 256), torch.randint(-4, 5, (256, 256), generator=g)).half()
    b = torch.ldexp(torch.ones(256, 256), torch.randint(-4, 5, (256, 256), generator=g)).half()
    sign = torch.where(torch.rand(256, 256, generator=g) < 0.5, -1.0, 1.0).half()
    a = a * sign
    assert torch.equal(run(lib, gpu, a, b), so.gemm_ref(a, b).half())


# ---- layouts, non-square and ragged shapes -------------------------------------------------------------------------
@pytest.mark.parametrize("layout", ["NN", "TN", "NT"])
@pytest.mark.parametrize("M,N,K", [(256, 512, 320), (512, 256, 64), (768, 1024, 1088), (100, 70, 50), (1, 1, 1),
                                   (257, 255, 129), (31, 300, 8), (2048, 256, 4096)])
def test_layouts_and_shapes(lib, gpu, layout, M, N, K):
    a, b = operands(M, N, K, layout, seed=M + N + K)
    c = check(lib, gpu, a, b, layout, K)
    assert c.shape == (M, N)


@pytest.mark.parametrize("variant", [0, 1, 2, 3, 4, 5, 6, 7])
@pytest.mark.parametrize("layout", ["NN", "TN", "NT"])
@pytest.mark.parametrize("M,N,K", [(1000, 1000, 1024), (300, 4096, 512), (2056, 1032, 128), (130, 8, 64), (4104, 4096, 256),
                                   (257, 264, 64)])
def test_ragged_m_and_n_on_the_tiled_kernels(lib, gpu, variant, layout, M, N, K):
    # token counts and widths that are not multiples of the tile (multiples of 8 where 16-byte chunks must not straddle the
    # end): same kernels with the out-of-range rows folded back inside; the surrounding memory of C stays untouched
    a, b = operands(M, N, K, layout, seed=M + N)
    ref = so.gemm_ref(a, b, layout)
    c = torch.full((M + 2, N + 8), 9.0, dtype=torch.float16, device=gpu)
    ag, bg = a.to(gpu), b.to(gpu)
    lib.hgemm(ag, bg, layout, out=c[:M, :N], variant=variant)   # variant 0: the public entry point
    torch.cuda.synchronize()
    ok, st = so.gemm_tolerance_ok(c[:M, :N].cpu(), ref, K)
    assert ok, st
    assert bool((c[M:] == 9.0).all()) and bool((c[:, N:] == 9.0).all())


@pytest.mark.parametrize("layout", ["NN", "TN", "NT"])
@pytest.mark.parametrize("M,N,K", [(512, 384, 1072), (1024, 1024, 1040), (256, 256, 80), (16, 4096, 4112), (8, 512, 2096),
                                   (48, 2048, 1056), (1000, 520, 4144), (2048, 2048, 176)])
def test_k_that_is_a_multiple_of_16_but_not_of_the_tile_depth(lib, gpu, layout, M, N, K):
    # the reference's checked wrapper takes K % 16 == 0 (kernels/gemm/pkg/gemm_unified/csrc/auto/gemm_7.cu:115-135): the
    # tiled kernels take the last K % 64 columns in their prologue; with up to 64 rows the small-M kernels do the first
    # K - K % 64 columns and the bounds-checked kernel the last K % 64
    a, b = operands(M, N, K, layout, seed=M + K, b_std=0.05)
    check(lib, gpu, a, b, layout, K)


@pytest.mark.parametrize("variant", [1, 2, 3, 4, 5, 6, 7])
@pytest.mark.parametrize("layout", ["NN", "TN", "NT"])
@pytest.mark.parametrize("M,N,K", [(512, 512, 72), (300, 520, 200), (256, 256, 40), (1000, 264, 1048), (64, 128, 8),
                                   (257, 72, 136)])
def test_k_tail_on_every_tile_shape(lib, gpu, variant, layout, M, N, K):
    # every tiled kernel takes its K % 64 columns in its prologue (out-of-range copies write zeros); K below one tile's
    # depth is all tail
    a, b = operands(M, N, K, layout, seed=M + K + variant, b_std=0.05)
    # LDS keeps what the last kernel left there: a product of NaNs on the same tile shape first, over enough tiles to
    # reach every CU, so that a tail lane whose copy wrote nothing would leave a NaN in the tile
    nan_a = torch.full((4096, 128), float("nan"), dtype=torch.float16, device=gpu)
    lib.hgemm(nan_a, nan_a.t().contiguous() if layout == "NN" else nan_a, "NN" if layout == "NN" else "NT", variant=variant)
    check(lib, gpu, a, b, layout, K, variant=variant)


@pytest.mark.parametrize("layout", ["NN", "TN", "NT"])
@pytest.mark.parametrize("M,N,K", [(512, 384, 1072), (1000, 520, 4144), (300, 264, 40), (48, 2048, 1056), (16, 4096, 4112)])
def test_k_tail_with_a_residual(lib, gpu, layout, M, N, K):
    # a residual on a product whose K is not a multiple of the tile depth: one pass on the tiled kernels. More than 64
    # rows: the plain product takes the same kernel, so the fused result is that product plus the residual bit for bit.
    # Up to 64 rows the plain product is formed in two passes (small-M kernel + bounds-checked tail): within tolerance.
    a, b = operands(M, N, K, layout, seed=M + K, b_std=0.05)
    r = (torch.randn(M, N, generator=torch.Generator().manual_seed(3)) * 2).half()
    got = lib.hgemm(a.to(gpu), b.to(gpu), layout, residual=r.to(gpu))
    if M > 64:
        assert torch.equal(got, lib.hgemm(a.to(gpu), b.to(gpu), layout) + r.to(gpu))
    prod = so.gemm_ref(a, b, layout)
    err = (got.cpu().float() - r.float() - prod).abs()
    bound = 2e-2 * (K / 1024.0) ** 0.5 + 1e-2 * prod.abs() + 2.0 ** -10 * got.cpu().float().abs()
    assert bool((err <= bound).all()), (float(err.max()), int((err > bound).sum()))


@pytest.mark.parametrize("variant", [0, 1, 2, 3, 4, 5, 6, 7])
@pytest.mark.parametrize("layout", ["NN", "TN", "NT"])
@pytest.mark.parametrize("M,N,K,ldc_pad", [(300, 1001, 256, 0), (512, 515, 136, 5), (1000, 77, 64, 3), (130, 3, 512, 0),
                                           (16, 1001, 1024, 0), (48, 2049, 256, 1), (256, 256, 128, 1)])
def test_widths_that_are_no_multiple_of_8_and_unaligned_rows_of_c(lib, gpu, variant, layout, M, N, K, ldc_pad):
    # N need not be a multiple of 8 and C's rows need not be 16-byte aligned (a vocabulary of 50257 or 32001 entries): the
    # tiled kernels store such a C in 16-byte pieces of no stated alignment and the last N % 8 columns element by element
    # (the small-M kernel of layout NT element by element). An operand stored [K,N] is
    # still copied in 16-byte chunks, so its rows must be aligned: ldb is N rounded up to 8, the padding holds NaNs and
    # must stay out of the product. The residual has C's row stride. Nothing outside C[:M, :N] may change.
    a, b = operands(M, N, K, layout, seed=M + N + K, b_std=0.05)
    ldb = (b.shape[1] + 7) // 8 * 8
    lda = (a.shape[1] + 7) // 8 * 8
    ag = torch.full((a.shape[0], lda), float("nan"), dtype=torch.float16, device=gpu)
    bg = torch.full((b.shape[0], ldb), float("nan"), dtype=torch.float16, device=gpu)
    ag[:, :a.shape[1]] = a.to(gpu)
    bg[:, :b.shape[1]] = b.to(gpu)
    ldc = N + ldc_pad
    c = torch.full((M + 1, ldc), 3.0, dtype=torch.float16, device=gpu)
    st = torch.cuda.current_stream(gpu).cuda_stream
    L = lib.load()
    rc = L.mi355_internal_hgemm_variant(ag.data_ptr(), bg.data_ptr(), c.data_ptr(), M, N, K, lda, ldb, ldc, lib.LAYOUTS[layout], 0,
                                        variant, st)
    assert rc == 0
    torch.cuda.synchronize()
    ref = so.gemm_ref(a, b, layout)
    ok, stt = so.gemm_tolerance_ok(c[:M, :N].cpu(), ref, K)
    assert ok, (layout, M, N, K, ldc, stt)
    assert bool((c[M:] == 3.0).all()) and bool((c[:, N:] == 3.0).all())
    if variant == 0:   # with a residual of the same row stride, in place: bit for bit the product plus the residual
        r = (torch.randn(M, N, generator=torch.Generator().manual_seed(1)) * 2).half().to(gpu)
        want = c[:M, :N] + r
        c[:M, :N] = r
        assert L.mi355_hgemm_add(ag.data_ptr(), bg.data_ptr(), c.data_ptr(), c.data_ptr(), M, N, K, lda, ldb, ldc, ldc,
                                 lib.LAYOUTS[layout], st) == 0
        torch.cuda.synchronize()
        assert torch.equal(c[:M, :N], want)
        assert bool((c[M:] == 3.0).all()) and bool((c[:, N:] == 3.0).all())


# ---- split-K: 17 .. 256 rows against a narrow second operand --------------------------------------------------------
SPLIT_K_SHAPES = [(64, 4096, 14336), (17, 4096, 8192), (100, 2048, 4096), (128, 4096, 4096), (48, 1000, 2048), (33, 6144, 4096),
                  (250, 1024, 8192), (40, 72, 16384), (160, 4096, 8192), (192, 4000, 14336),
                  # 193 .. 1024 rows, long K: ranges of K on 128x128 tiles (four ranges, two ranges, ragged M and N)
                  (256, 4096, 14336), (384, 2048, 16384), (500, 4000, 12288), (300, 4096, 8192),
                  # up to 1024 rows: 120 tiles in two ranges, 168 tiles in three, 192 tiles in four, 160 tiles in three
                  (640, 3072, 12288), (896, 3072, 12288), (768, 4096, 14336), (640, 4096, 12288)]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("layout", ["NN", "NT", "TN"])
@pytest.mark.parametrize("M,N,K", SPLIT_K_SHAPES)
def test_split_k_products(lib, gpu, dtype, layout, M, N, K):
    # the ranges of K of a tile run on different workgroups and meet in the library's workspace; the workgroup that
    # arrives last adds them in the order of the ranges, so the result does not depend on the order of arrival: five
    # launches give the same bits, also with launches of other shapes (other tile and range counts, a workspace that
    # grows) in between
    a, b = operands(M, N, K, layout, seed=M + N + K, b_std=0.05)
    a, b = a.to(dtype), b.to(dtype)
    ag, bg = a.to(gpu), b.to(gpu)
    first = lib.hgemm(ag, bg, layout)
    torch.cuda.synchronize()
    ref = so.gemm_ref(a, b, layout)
    if dtype == torch.float16:
        ok, st = so.gemm_tolerance_ok(first.cpu(), ref, K)
        assert ok, (layout, M, N, K, st)
    else:
        assert bf16_close(first, ref, K)[0]
    other_a, other_b = operands(96, 512, 1024, "NT", seed=1)
    for _ in range(4):
        lib.hgemm(other_a.to(gpu), other_b.to(gpu), "NT")
        assert torch.equal(lib.hgemm(ag, bg, layout), first)


@pytest.mark.parametrize("M,N,K", [(72, 1001, 8192), (300, 1001, 12288)])      # 64x64 tiles, 128x128 tiles
def test_split_k_with_residual_in_place_and_unaligned_c(lib, gpu, M, N, K):
    a, b = operands(M, N, K, "NT", seed=3, b_std=0.05)
    ag, bg = a.to(gpu), b.to(gpu)
    c = torch.full((M + 1, N + 3), 3.0, dtype=torch.float16, device=gpu)      # rows of 1004 elements: not 16-byte aligned
    st = torch.cuda.current_stream(gpu).cuda_stream
    lib.hgemm_raw(ag.data_ptr(), bg.data_ptr(), c.data_ptr(), M, N, K, K, K, N + 3, lib.GEMM_NT, st)
    torch.cuda.synchronize()
    ok, stt = so.gemm_tolerance_ok(c[:M, :N].cpu(), so.gemm_ref(a, b, "NT"), K)
    assert ok, stt
    assert bool((c[M:] == 3.0).all()) and bool((c[:, N:] == 3.0).all())
    r = (torch.randn(M, N, generator=torch.Generator().manual_seed(1)) * 2).half().to(gpu)
    want = c[:M, :N] + r
    c[:M, :N] = r
    assert lib.load().mi355_hgemm_add(ag.data_ptr(), bg.data_ptr(), c.data_ptr(), c.data_ptr(), M, N, K, K, K, N + 3, N + 3,
                                      lib.GEMM_NT, st) == 0
    torch.cuda.synchronize()
    assert torch.equal(c[:M, :N], want)
    assert bool((c[M:] == 3.0).all()) and bool((c[:, N:] == 3.0).all())


def test_split_k_on_two_streams_and_under_graph_capture(lib, gpu):
    # every stream has a workspace of its own: interleaved calls on two streams do not disturb each other. A call made
    # while its stream is being captured and has no workspace yet takes the kernels without split-K instead of failing;
    # once the stream has a workspace, the captured call uses it, and replays give the eager result.
    M, N, K = 64, 2048, 8192
    a, b = operands(M, N, K, "NT", seed=5, b_std=0.05)
    ag, bg = a.to(gpu), b.to(gpu)
    ref = lib.hgemm(ag, bg, "NT").clone()
    a2, b2 = operands(120, 1024, 4096, "NT", seed=6, b_std=0.05)
    a2g, b2g = a2.to(gpu), b2.to(gpu)
    ref2 = lib.hgemm(a2g, b2g, "NT").clone()
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(gpu), torch.cuda.Stream(gpu)
    outs1, outs2 = [], []
    for _ in range(6):
        with torch.cuda.stream(s1):
            outs1.append(lib.hgemm(ag, bg, "NT"))
        with torch.cuda.stream(s2):
            outs2.append(lib.hgemm(a2g, b2g, "NT"))
    torch.cuda.synchronize()
    assert all(torch.equal(o, ref) for o in outs1) and all(torch.equal(o, ref2) for o in outs2)
    s3 = torch.cuda.Stream(gpu)                       # a stream that has never made such a call
    out = torch.empty((M, N), dtype=torch.float16, device=gpu)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(s3):
        with torch.cuda.graph(g, stream=s3):
            lib.hgemm(ag, bg, "NT", out=out)          # no workspace yet: the kernels without split-K
    for _ in range(3):
        out.zero_()
        g.replay()
        torch.cuda.synchronize()
        ok, stt = so.gemm_tolerance_ok(out.cpu(), so.gemm_ref(a, b, "NT"), K)
        assert ok, stt


@pytest.mark.parametrize("variant,tile_m,tile_n", [(1, 256, 256), (2, 128, 128), (3, 64, 128), (4, 64, 64), (5, 128, 256), (6, 256, 128), (7, 32, 64)])
@pytest.mark.parametrize("layout", ["NN", "NT"])
@pytest.mark.parametrize("tiles_m,tiles_n,ragged", [(16, 32, 0), (32, 24, 0), (32, 16, 8), (48, 16, 0)])
def test_grids_walked_in_super_blocks(lib, gpu, variant, tile_m, tile_n, layout, tiles_m, tiles_n, ragged):
    # grids of >= 512 tiles whose dimensions are multiples of a 16x16 or 32x8 block of tiles are walked block by block in
    # serpentine order (hgemm.hip: tile_of_block): every tile must still be computed exactly once, also when the last tile
    # row / column is ragged. K = 64 keeps the host product cheap.
    if layout == "NT" and variant == 3:
        tile_m, tile_n = 128, 64
    M, N, K = tiles_m * tile_m - ragged, tiles_n * tile_n - ragged, 64
    a, b = operands(M, N, K, layout, seed=tiles_m + tiles_n + variant)
    check(lib, gpu, a, b, layout, K, variant=variant)


def _seeded_shapes(n, seed):
    """n products drawn with a fixed seed: row counts from one to a few thousand, widths and depths on and off the tile grid
    (multiples of 8, sometimes odd), every layout. The library picks the kernel (variant 0): small-M, one of the four tile
    shapes (with or without a K tail), for few rows the K tail through the bounds-checked kernel, or that kernel alone."""
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(n):
        layout = ["NN", "NT", "TN"][int(rng.integers(3))]
        m = int(rng.choice([1, 7, 16, 24, 64, 100, 128, 200, 384, 520, 1000, 1536, 2048, 3000]))
        nn = int(rng.choice([8, 64, 136, 512, 1000, 1024, 2048, 4096, 5120])) + int(rng.choice([0, 0, 0, 8, 24, 3]))
        k = int(rng.choice([64, 128, 192, 448, 1024, 2048, 4096])) + int(rng.choice([0, 0, 0, 16, 32, 8, 5]))
        if m * nn > 6e6:
            k = min(k, 1100)
        out.append((layout, m, nn, k))
    return out


@pytest.mark.parametrize("layout,M,N,K", _seeded_shapes(40, 20260417))
def test_seeded_random_products_choose_their_own_kernel(lib, gpu, layout, M, N, K):
    a, b = operands(M, N, K, layout, seed=M + 3 * N + 7 * K, b_std=0.05)
    c = torch.full((M + 1, N + 3), 7.0, dtype=torch.float16, device=gpu)
    lib.hgemm(a.to(gpu), b.to(gpu), layout, out=c[:M, :N])
    torch.cuda.synchronize()
    ok, st = so.gemm_tolerance_ok(c[:M, :N].cpu(), so.gemm_ref(a, b, layout), K)
    assert ok, (layout, M, N, K, st)
    assert bool((c[M:] == 7.0).all()) and bool((c[:, N:] == 7.0).all())


@pytest.mark.parametrize("M,N,K", [(5, 512, 256), (13, 4096, 1024), (33, 136, 192), (100, 1024, 512), (300, 2048, 256),
                                   (1001, 1000, 1024), (2050, 512, 128), (12, 4096, 4160)])
def test_layout_tn_with_any_row_count_in_padded_rows(lib, gpu, M, N, K):
    # A stored [K, M] in rows of lda = M rounded up to a multiple of 8 (16-byte aligned rows): the small-M and tiled
    # kernels read whole 16-byte chunks, so up to 7 columns of the padding, which holds NaNs here, and must keep them out
    # of the M rows they store; nothing outside C[:M, :N] may change
    a, b = so.gemm_inputs(M, N, K, seed=M + N, b_std=0.05)
    lda = (M + 7) // 8 * 8
    a_pad = torch.full((K, lda), float("nan"), dtype=torch.float16)
    a_pad[:, :M] = a.t()
    ag, bg = a_pad.to(gpu), b.to(gpu)
    c = torch.full((M + 2, N + 8), 5.0, dtype=torch.float16, device=gpu)
    lib.hgemm_raw(ag.data_ptr(), bg.data_ptr(), c.data_ptr(), M, N, K, lda, N, N + 8, lib.GEMM_TN,
                  torch.cuda.current_stream(gpu).cuda_stream)
    torch.cuda.synchronize()
    ok, st = so.gemm_tolerance_ok(c[:M, :N].cpu(), so.gemm_ref(a, b, "NN"), K)
    assert ok, (M, N, K, st)
    assert bool((c[M:] == 5.0).all()) and bool((c[:, N:] == 5.0).all())


def _seeded_padded_products(n, seed):
    """n products drawn with a fixed seed whose three matrices all live in wider allocations: leading dimensions rounded
    up to a multiple of 8 plus 0, 8 or 64 elements, in every layout, row counts from 1 to 3000, K on and off the tiles'
    depth."""
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(n):
        layout = ["NN", "NT", "TN"][int(rng.integers(3))]
        m = int(rng.choice([1, 2, 5, 8, 9, 15, 16, 17, 31, 32, 48, 63, 64, 65, 100, 127, 128, 129, 200, 255, 256, 257, 384, 500, 512, 1000, 1500, 3000]))
        nn = int(rng.choice([8, 16, 24, 64, 72, 128, 136, 256, 512, 1000, 1024, 2048, 3072, 4096])) + int(rng.choice([0, 0, 0, 8, 16]))
        k = int(rng.choice([32, 64, 96, 128, 192, 256, 448, 512, 1024, 2048, 4096])) + int(rng.choice([0, 0, 0, 0, 16, 32, 8]))
        if m * nn * k > 4e9:
            k = 256
        out.append((layout, m, nn, k, int(rng.choice([0, 0, 8, 64])), int(rng.choice([0, 0, 8, 64])), int(rng.choice([0, 8]))))
    return out


@pytest.mark.parametrize("layout,M,N,K,pad_a,pad_b,pad_c", _seeded_padded_products(48, 1234))
def test_seeded_random_products_in_padded_allocations(lib, gpu, layout, M, N, K, pad_a, pad_b, pad_c):
    # the padding of A and B holds NaNs: whatever a kernel reads of it must stay out of the product; C's padding and
    # the row behind C must come back untouched
    a, b = operands(M, N, K, layout, seed=M + 3 * N + 7 * K + pad_a, b_std=0.05)
    lda = (a.shape[1] + 7) // 8 * 8 + pad_a
    ldb = (b.shape[1] + 7) // 8 * 8 + pad_b
    ldc = N + pad_c
    ag = torch.full((a.shape[0], lda), float("nan"), dtype=torch.float16, device=gpu)
    bg = torch.full((b.shape[0], ldb), float("nan"), dtype=torch.float16, device=gpu)
    ag[:, :a.shape[1]] = a.to(gpu)
    bg[:, :b.shape[1]] = b.to(gpu)
    c = torch.full((M + 1, ldc), 3.0, dtype=torch.float16, device=gpu)
    lib.hgemm_raw(ag.data_ptr(), bg.data_ptr(), c.data_ptr(), M, N, K, lda, ldb, ldc, lib.LAYOUTS[layout],
                  torch.cuda.current_stream(gpu).cuda_stream)
    torch.cuda.synchronize()
    ok, st = so.gemm_tolerance_ok(c[:M, :N].cpu(), so.gemm_ref(a, b, layout), K)
    assert ok, (layout, M, N, K, lda, ldb, ldc, st)
    assert bool((c[M:] == 3.0).all()) and bool((c[:, N:] == 3.0).all())


@pytest.mark.parametrize("variant", [1, 2, 3, 4, 5, 6, 7])
@pytest.mark.parametrize("layout", ["NN", "TN", "NT"])
def test_every_tile_variant(lib, gpu, variant, layout):
    a, b = operands(512, 768, 448, layout, seed=variant)
    check(lib, gpu, a, b, layout, 448, variant=variant)


@pytest.mark.parametrize("layout", ["NN", "NT", "TN"])
@pytest.mark.parametrize("M,N,K", [(16, 4096, 4096), (1, 1000, 512), (64, 304, 128), (33, 24, 192), (7, 72, 96), (16, 64, 4096)])
def test_decode_shaped_small_m(lib, gpu, layout, M, N, K):
    a, b = operands(M, N, K, layout, seed=M * 3 + N, b_std=0.05)
    check(lib, gpu, a, b, layout, K)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M,N,K", [(16, 6144, 4096), (8, 14336, 4096), (13, 14336, 4096), (1, 12288, 4096), (3, 6144, 4096),
                                   (16, 28672, 4096), (16, 6160, 4096)])
def test_generation_step_projections_with_the_activation_rows_kept_in_registers(lib, gpu, dtype, M, N, K):
    # layout NT, K = 4096, up to 16 rows, a few hundred row tiles or more: a workgroup takes two or four row tiles and copies
    # the activation rows only for the first (hgemm_smallm_nt_rega_kernel); 6160 = 385 tiles is not divisible and keeps one
    # tile per workgroup
    a, b = operands(M, N, K, "NT", seed=M + N, b_std=0.05)
    if dtype == torch.bfloat16:
        a, b = a.float().bfloat16(), b.float().bfloat16()
        c = lib.hgemm(a.to(gpu), b.to(gpu), "NT").cpu()
        ok, worst = bf16_close(c, so.gemm_ref(a, b, "NT"), K)
        assert ok, worst
    else:
        check(lib, gpu, a, b, "NT", K)


@pytest.mark.parametrize("layout", ["NN", "NT", "TN"])
@pytest.mark.parametrize("M,N,K", [(24, 14336, 512), (64, 14336, 256), (32, 28672, 128), (40, 4096, 1024), (17, 12800, 192)])
def test_17_to_64_rows_small_m_or_tiles(lib, gpu, layout, M, N, K):
    """Between 17 and 64 rows the dispatcher weighs the small-M kernels (B streamed once per 16 rows) against the 128x128
    tiles (wide products); both sides of that choice, all layouts (TN with M a multiple of 8 has a small-M kernel too)."""
    a, b = operands(M, N, K, layout, seed=9, b_std=0.05)
    check(lib, gpu, a, b, layout, K)


def test_reference_seeded_case_from_golden_fixture(lib, gpu):
    z = np.load(os.path.join(GOLDEN, "gemm_seed0_256.npz"))
    a, b, rows = torch.from_numpy(z["a"]), torch.from_numpy(z["b"]), z["rows"]
    for lay in ("NN", "TN", "NT"):
        c = run(lib, gpu, a, b, lay).float().numpy()[rows]
        ref = z["c_" + lay]
        assert np.all(np.abs(c - ref) <= 2e-2 * 0.5 + 1e-2 * np.abs(ref)), lay


def test_strided_leading_dimensions(lib, gpu):
    # lda/ldb/ldc larger than the logical width (operands that are column slices of wider buffers)
    M, N, K = 512, 256, 192
    abig, bbig = so.randn_fp16((M, K + 64), 1).to(gpu), so.randn_fp16((K, N + 128), 2).to(gpu)
    cbig = torch.zeros((M, N + 32), dtype=torch.float16, device=gpu)
    lib.hgemm_raw(abig.data_ptr(), bbig.data_ptr(), cbig.data_ptr(), M, N, K, K + 64, N + 128, N + 32, lib.GEMM_NN,
                  torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    ok, st = so.gemm_tolerance_ok(cbig[:, :N], so.gemm_ref(abig[:, :K], bbig[:, :N]), K)
    assert ok, st
    assert bool((cbig[:, N:] == 0).all())  # nothing written outside the N columns


@pytest.mark.parametrize("layout", ["NN", "NT"])
def test_leading_dimension_beyond_the_tiled_kernels_reach(lib, gpu, layout):
    """The tiled kernels address a tile with 32-bit byte offsets and take leading dimensions below 2^22 elements; a wider
    operand must take the bounds-checked kernel and still be right (A is a 128 x 64 corner of a 128 x 2^22 buffer)."""
    M, N, K, lda = 128, 64, 64, 1 << 22
    abig = torch.zeros((M, lda), dtype=torch.float16, device=gpu)
    a = so.randn_fp16((M, K), 3)
    abig[:, :K] = a.to(gpu)
    b = so.randn_fp16((N, K) if layout == "NT" else (K, N), 4)
    bg = b.to(gpu)
    c = torch.zeros((M, N), dtype=torch.float16, device=gpu)
    lib.hgemm_raw(abig.data_ptr(), bg.data_ptr(), c.data_ptr(), M, N, K, lda, bg.stride(0), N, lib.LAYOUTS[layout],
                  torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    ok, st = so.gemm_tolerance_ok(c.cpu(), so.gemm_ref(a, b, layout), K)
    assert ok, st


# ---- size-independent properties at the full benchmark size -------------------------------------------------------
def test_full_size_linearity_and_column_selection(lib, gpu):
    n = 8192
    a = so.randn_fp16((n, n), 0).to(gpu)
    # B = one-hot columns scaled by powers of two: C[:, j] = 2^e_j * A[:, src_j], exact in fp16
    g = torch.Generator().manual_seed(2)
    src = torch.randint(0, n, (n,), generator=g)
    e = torch.randint(-2, 3, (n,), generator=g)
    b = torch.zeros(n, n, dtype=torch.float16)
    b[src, torch.arange(n)] = torch.ldexp(torch.ones(n), e).half()
    c = lib.hgemm(a, b.to(gpu))
    expect = a[:, src.to(gpu)] * torch.ldexp(torch.ones(n), e).half().to(gpu)[None, :]
    assert torch.equal(c, expect)


# ---- torch operator path ----------------------------------------------------------------------------------------------
@pytest.mark.parametrize("index", list(range(17)))
def test_torch_operator_every_index(gpu, index):
    import gemm_unified
    layout = so.GEMM_LAYOUT_OF_INDEX[index]
    a, b = operands(384, 512, 256, layout, seed=index)
    c = gemm_unified.ops.fine_gemm(a.to(gpu), b.to(gpu), index)
    assert c.dtype == torch.float16 and c.shape == (384, 512)
    ok, st = so.gemm_tolerance_ok(c, so.fine_gemm_ref(a, b, index), 256)
    assert ok, (index, st)


def test_torch_operator_reference_correctness_script_case(gpu):
    # kernels/gemm/test/correct.py: seed 0, 256x256 randn fp16, indices 13..15 against a @ b.T, 16 against a.T @ b,
    # allclose(rtol=1e-1, atol=1e-1)
    import gemm_unified
    torch.manual_seed(0)
    a = torch.randn(256, 256, dtype=torch.half).to(gpu)
    b = torch.randn(256, 256, dtype=torch.half).to(gpu)
    for idx, ref in ((13, a @ b.T), (14, a @ b.T), (15, a @ b.T), (16, a.T @ b), (0, a @ b)):
        c = gemm_unified.ops.fine_gemm(a, b, idx)
        assert torch.allclose(c, ref, rtol=1e-1, atol=1e-1), idx


def test_torch_operator_noncontiguous_inputs_and_stream(gpu):
    import gemm_unified
    a = so.randn_fp16((512, 300), 1).to(gpu)
    b = so.randn_fp16((300, 512), 2).to(gpu)
    at = a.t().contiguous().t()  # same values, column-major strides
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        c = gemm_unified.ops.fine_gemm(at, b, 0)
    s.synchronize()
    ok, st = so.gemm_tolerance_ok(c, so.gemm_ref(a, b), 300)
    assert ok, st


def test_torch_operator_single_row_operand_with_arbitrary_row_stride(lib, gpu):
    # torch calls a [1, K] tensor contiguous whatever its stride(0) (expand / as_strided / keepdim views produce such
    # tensors); the operators and the ctypes wrapper must pass the logical leading dimension, not that stride
    import gemm_unified
    K, N = 512, 256
    a, b = so.gemm_inputs(1, N, K, seed=5)
    base = torch.zeros(4 * K, dtype=torch.float16, device=gpu)
    base[:K] = a[0].to(gpu)
    for stride0 in (7, 0, 3 * K):
        a1 = base.as_strided((1, K), (stride0, 1))
        assert a1.is_contiguous() and a1.stride(0) == stride0
        for c in (gemm_unified.ops.fine_gemm(a1, b.to(gpu), 0), lib.hgemm(a1, b.to(gpu), "NN"),
                  gemm_unified.ops.fine_gemm(a1, b.t().contiguous().to(gpu), 13)):
            ok, st = so.gemm_tolerance_ok(c, so.gemm_ref(a, b), K)
            assert ok, (stride0, st)
    # the same for a [K, 1] second operand
    a2, b2 = so.gemm_inputs(64, 1, K, seed=6)
    bcol = b2.to(gpu).as_strided((K, 1), (1, 5))
    assert bcol.is_contiguous()
    ok, st = so.gemm_tolerance_ok(gemm_unified.ops.fine_gemm(a2.to(gpu), bcol, 0), so.gemm_ref(a2, b2), K)
    assert ok, st


# ---- bfloat16 ---------------------------------------------------------------------------------------------------------
# Tolerance for bfloat16 results (8 significand bits): |err| <= 2e-2 * sqrt(K / 1024) + 2^-8 |ref| against the fp32 product of
# the bf16-rounded operands (the accumulation slack of the fp16 bound plus one bf16 rounding).
def bf16_close(c, ref, K):
    err = (c.float().cpu() - ref).abs()
    return bool((err <= 2e-2 * (K / 1024) ** 0.5 + 2.0 ** -8 * ref.abs()).all()), float(err.max())


@pytest.mark.parametrize("layout", ["NN", "NT", "TN"])
@pytest.mark.parametrize("M,N,K", [(1024, 1024, 1024), (512, 768, 320), (1000, 264, 128), (16, 4096, 1024), (7, 72, 96),
                                   (100, 70, 50),
                                   (1000, 520, 4144), (2048, 2048, 72), (300, 1001, 264), (16, 515, 1096)])   # K tails, odd widths
def test_bfloat16_gemm(lib, gpu, layout, M, N, K):
    a, b = operands(M, N, K, layout, seed=K, b_std=0.05)
    a, b = a.float().bfloat16(), b.float().bfloat16()
    c = lib.hgemm(a.to(gpu), b.to(gpu), layout)
    assert c.dtype == torch.bfloat16
    ok, worst = bf16_close(c, so.gemm_ref(a, b, layout), K)
    assert ok, worst


def test_bfloat16_gemm_exact_cases_and_torch_operator(lib, gpu):
    import gemm_unified
    n = 256
    b = so.randn_fp16((n, n), 3).float().bfloat16()
    eye = torch.eye(n, dtype=torch.bfloat16)
    assert torch.equal(lib.hgemm(eye.to(gpu), b.to(gpu)).cpu(), b)            # identity: exact
    ones = torch.ones((n, 1024), dtype=torch.bfloat16)
    c = lib.hgemm(ones.to(gpu), torch.ones((1024, n), dtype=torch.bfloat16).to(gpu)).cpu()
    assert bool((c == 1024).all())                                            # 1024 is representable in bf16
    a = so.randn_fp16((n, n), 4).float().bfloat16()
    out = gemm_unified.ops.fine_gemm(a.to(gpu), b.to(gpu), 13)                # NT index, bf16 tensors
    assert out.dtype == torch.bfloat16 and bf16_close(out, so.gemm_ref(a, b, "NT"), n)[0]
    with pytest.raises(RuntimeError, match="dtype"):
        gemm_unified.ops.fine_gemm(a.to(gpu), b.half().to(gpu), 0)


# ---- residual added in the epilogue (mi355_hgemm_add) -----------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("layout", ["NN", "NT", "TN"])
@pytest.mark.parametrize("M,N,K", [(512, 512, 256),      # 128x128 tiles
                                   (4096, 4096, 128),    # 256x256 tiles
                                   (1000, 264, 128),     # ragged tiles
                                   (16, 4096, 1024),     # small-M kernels (NN, NT)
                                   (12, 6144, 4096),     # NT: several row tiles per workgroup, A kept in registers
                                   (8, 72, 192),
                                   (100, 70, 50)])       # bounds-checked kernel
def test_residual_epilogue_equals_product_then_add(lib, gpu, dtype, layout, M, N, K):
    """residual + proj(x) (modeling_llama.py:776,781): the fused form must give, bit for bit, what the product followed by
    an elementwise add in the same type gives, for a separate output, for a residual with a row stride, and in place."""
    a, b = operands(M, N, K, layout, seed=5)
    a, b = a.to(gpu, dtype), b.to(gpu, dtype)
    g = torch.Generator().manual_seed(6)
    wide = (torch.randn(M, N + 8, generator=g) * 3).to(dtype).to(gpu)
    r = wide[:, :N]                                      # row stride N + 8
    want = lib.hgemm(a, b, layout) + r
    got = lib.hgemm(a, b, layout, residual=r)
    assert torch.equal(got, want)
    rc = r.contiguous()
    got2 = lib.hgemm(a, b, layout, out=rc, residual=rc)  # in place
    assert got2.data_ptr() == rc.data_ptr() and torch.equal(rc, want)
    if dtype == torch.float16:
        # and against the oracle: what is left of the result without the residual is the product, to the product's
        # tolerance (which its own rounding to fp16 is part of) plus the rounding of the fp16 sum. The bound goes by the
        # size of the product, not of the sum: where product and residual cancel, the sum still carries the product's
        # rounding.
        prod = so.gemm_ref(a.cpu(), b.cpu(), layout)
        err = (got.cpu().float() - r.cpu().float() - prod).abs()
        bound = 2e-2 * (K / 1024.0) ** 0.5 + 1e-2 * prod.abs() + 2.0 ** -10 * got.cpu().float().abs()
        assert bool((err <= bound).all()), (float(err.max()), int((err > bound).sum()))


def test_residual_epilogue_full_size_projection(lib, gpu):
    """Llama-3-8B down projection at s = 8192 with the residual stream updated in place."""
    M, N, K = 8192, 4096, 14336
    g = torch.Generator(device=gpu).manual_seed(1)
    a = torch.randn(M, K, generator=g, device=gpu, dtype=torch.float16)
    w = (torch.randn(N, K, generator=g, device=gpu) * 0.02).half()
    res = torch.randn(M, N, generator=g, device=gpu, dtype=torch.float16)
    want = lib.hgemm(a, w, "NT") + res
    lib.hgemm(a, w, "NT", out=res, residual=res)
    assert torch.equal(res, want)
