"""Parity of the HIP path against the oracle on a real MI355X.  Every launch goes
through the C ABI (tts_launch): either from the unchanged Triton frontend with
HIPDriver active, or directly on a plan handle.

Bars: bit-exact for fp32 elementwise and all index/mask handling;
max-abs <= 1e-5 for fp32 softmax; <= 1e-2 for fp16 LayerNorm; relative Frobenius
error <= 1e-2 for the bf16 and int8-weight GEMMs."""
import numpy as np
import pytest
import torch
import triton

from conftest import plan_for

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.fixture(scope="module", autouse=True)
def hip_driver():
    import triton_shared_amd as tsa
    drv = tsa.activate()
    yield drv


@pytest.fixture(scope="module")
def K():
    from triton_shared_amd.examples import kernels
    return kernels


def relfro(got, ref):
    return ((got.double() - ref.double()).norm() / ref.double().norm()).item()


# ------------------------------------------------------------------ cfg1
def test_cfg1_vec_add_bit_exact(K, oracle_cpu):
    torch.manual_seed(0)
    n = 98432
    x, y = torch.rand(n), torch.rand(n)
    xd, yd = x.to(DEV), y.to(DEV)
    zd = torch.full((n + 64,), -7.0, device=DEV)           # sentinel after the end
    k = K.vec_add[(triton.cdiv(n, 1024),)](xd, yd, zd, n, BLOCK=1024)
    torch.cuda.synchronize()
    assert k.function.family == "map1d" and k.function.last_kernel == "map1d_f32_kernel"
    assert torch.equal(zd[:n].cpu(), oracle_cpu.vec_add(x, y))
    assert torch.equal(zd[n:].cpu(), torch.full((64,), -7.0))  # the masked tail is not written


@pytest.mark.parametrize("n", [1, 3, 1023, 1024, 1025, 5000, (1 << 22) + 5])
def test_vec_add_sizes_and_unaligned_views(K, oracle_cpu, n):
    torch.manual_seed(n)
    x, y = torch.rand(n + 3), torch.rand(n + 3)
    xd, yd, zd = x.to(DEV), y.to(DEV), torch.zeros(n + 3, device=DEV)
    # views starting 1, 2 and 3 elements into the allocation: no 16-byte alignment
    K.vec_add[(triton.cdiv(n, 1024) + 1,)](xd[1:], yd[2:], zd[3:], n, BLOCK=1024)  # one extra, all-masked program
    torch.cuda.synchronize()
    assert torch.equal(zd[3:3 + n].cpu(), x[1:1 + n] + y[2:2 + n])
    assert zd[:3].abs().sum().item() == 0


def test_map1d_other_ops_through_c_abi(native):
    # the same plan family with other binary ops, launched directly on plan handles
    import extra_kernels as X
    from triton_shared_amd.examples import kernels  # noqa: F401
    torch.manual_seed(1)
    n = 3000
    x, y = torch.randn(n), torch.randn(n) + 2.0
    xd, yd, zd = x.to(DEV), y.to(DEV), torch.zeros(n, device=DEV)
    X.vec_sub_swapped[(triton.cdiv(n, 128),)](xd, yd, zd, n, BLOCK=128)
    torch.cuda.synchronize()
    assert torch.equal(zd.cpu(), y - x)
    plan, _ = plan_for(native, "vec_add.small")
    stream = torch.cuda.current_stream().cuda_stream
    plan.launch((triton.cdiv(n, 64), 1, 1), stream, [xd.data_ptr(), yd.data_ptr(), zd.data_ptr(), n])
    torch.cuda.synchronize()
    assert torch.equal(zd.cpu(), x + y)
    plan.launch((0, 1, 1), stream, [0, 0, 0, n])  # empty grid: nothing is dereferenced


# ------------------------------------------------------------------ cfg2
def test_cfg2_softmax(K, oracle_cpu):
    torch.manual_seed(0)
    x = torch.randn(4096, 781)
    xd = x.to(DEV)
    od = torch.full((4096, 781), 3.0, device=DEV)
    k = K.row_softmax[(4096,)](od, xd, xd.stride(0), od.stride(0), 781, BLOCK=1024)
    torch.cuda.synchronize()
    assert k.function.family == "row_softmax"
    ref = oracle_cpu.row_softmax(x)
    assert (od.cpu() - ref).abs().max().item() <= 1e-5
    assert (od.cpu().double() - torch.softmax(x.double(), 1)).abs().max().item() <= 1e-5
    assert torch.allclose(od.sum(1), torch.ones(4096, device=DEV), atol=1e-5)


@pytest.mark.parametrize("rows,cols,block,pad", [(1823, 781, 1024, 0), (33, 1, 64, 5), (7, 64, 64, 3), (5, 4096, 4096, 0),
                                                (3, 6000, 8192, 8), (9, 130, 256, 1)])
def test_softmax_shapes_and_pitches(K, oracle_cpu, rows, cols, block, pad):
    torch.manual_seed(rows)
    xfull = torch.randn(rows, cols + pad)
    x = xfull[:, :cols]
    xd = xfull.to(DEV)[:, :cols]
    ofull = torch.full((rows, cols + pad), -9.0, device=DEV)
    od = ofull[:, :cols]
    K.row_softmax[(rows,)](od, xd, xd.stride(0), od.stride(0), cols, BLOCK=block)
    torch.cuda.synchronize()
    assert torch.allclose(od.cpu(), torch.softmax(x, 1))   # the reference's assertion (test_softmax.py:65)
    assert (od.cpu() - oracle_cpu.row_softmax(x.contiguous(), BLOCK=block)).abs().max().item() <= 1e-5
    if pad:
        assert torch.equal(ofull[:, cols:].cpu(), torch.full((rows, pad), -9.0))  # columns beyond the mask untouched


# ------------------------------------------------------------------ cfg3
def _ln_inputs(M, N, dtype, seed=0):
    torch.manual_seed(seed)
    x = torch.randn(M, N).to(dtype)
    w = (1 + 0.1 * torch.randn(N)).to(dtype)
    b = (0.1 * torch.randn(N)).to(dtype)
    return x, w, b


def _run_ln(K, x, w, b, eps, block=1024):
    M, N = x.shape
    xd, wd, bd = x.to(DEV), w.to(DEV), b.to(DEV)
    yd = torch.zeros_like(xd)
    mean = torch.zeros(M, dtype=torch.float32, device=DEV)
    rstd = torch.zeros(M, dtype=torch.float32, device=DEV)
    k = K.layer_norm_fwd[(M,)](xd, yd, wd, bd, mean, rstd, xd.stride(0), N, eps, BLOCK=block)
    torch.cuda.synchronize()
    assert k.function.family == "layernorm_fwd"
    return yd.cpu(), mean.cpu(), rstd.cpu()


def test_cfg3_layernorm(K, oracle_cpu):
    x, w, b = _ln_inputs(4096, 8192, torch.float16)
    y, mean, rstd = _run_ln(K, x, w, b, 1e-5)
    yr, mr, rr = oracle_cpu.layer_norm_fwd(x, w, b, 1e-5)
    assert (y.float() - yr.float()).abs().max().item() <= 1e-2
    assert (mean - mr).abs().max().item() <= 1e-5
    assert ((rstd - rr) / rr).abs().max().item() <= 1e-5
    # almost every output is the same fp16 value; the rest differ by one rounding
    assert (y != yr).float().mean().item() < 0.02


@pytest.mark.parametrize("M,N,dtype", [(1151, 8192, torch.float16), (17, 1000, torch.float16), (5, 8191, torch.float16),
                                      (3, 64, torch.float16), (9, 16384, torch.float16), (2, 20000, torch.float16),
                                      (33, 4096, torch.bfloat16), (4, 777, torch.bfloat16),
                                      # enough whole rows for workgroups that walk several rows each, in uneven numbers
                                      (4100, 8192, torch.bfloat16), (8200, 4096, torch.float16), (16390, 2048, torch.float16)])
def test_layernorm_shapes(K, oracle_cpu, M, N, dtype):
    x, w, b = _ln_inputs(M, N, dtype, seed=N)
    y, mean, rstd = _run_ln(K, x, w, b, 1e-5)
    yr, mr, rr = oracle_cpu.layer_norm_fwd(x, w, b, 1e-5)
    tol = 1e-2 if dtype == torch.float16 else 4e-2      # one bf16 ulp at |y| ~ 4
    assert (y.float() - yr.float()).abs().max().item() <= tol
    assert (mean - mr).abs().max().item() <= 1e-5 and ((rstd - rr) / rr).abs().max().item() <= 1e-5


@pytest.mark.parametrize("M,N,kernel", [(4100, 8192, "layernorm_fwd_persistent_kernel"), (8200, 2048, "layernorm_fwd_persistent_kernel"), (300, 4096, "layernorm_fwd_kernel<4>"),
                                       (7, 1001, "layernorm_fwd_kernel<1>"), (5, 8191, "layernorm_fwd_kernel<8>"), (3, 20000, "layernorm_fwd_long_kernel")])
def test_layernorm_on_fp32_tensors(K, M, N, kernel):
    # the same Triton source on fp32 x, y, w, b (no widening or narrowing casts in its TTIR) runs on the same kernels with
    # 16-byte chunks of four elements; pinned by the float64 formula (biased variance) and torch's layer_norm
    x, w, b = _ln_inputs(M, N, torch.float32, seed=N + 1)
    xd, wd, bd = x.to(DEV), w.to(DEV), b.to(DEV)
    yd = torch.full((M + 1, N), -3.0, device=DEV)
    mean = torch.zeros(M, dtype=torch.float32, device=DEV)
    rstd = torch.zeros(M, dtype=torch.float32, device=DEV)
    k = K.layer_norm_fwd[(M,)](xd, yd, wd, bd, mean, rstd, xd.stride(0), N, 1e-5, BLOCK=1024)
    torch.cuda.synchronize()
    assert k.function.family == "layernorm_fwd" and k.function.last_kernel == kernel
    xx = x.double()
    m64 = xx.mean(1)
    v64 = ((xx - m64[:, None]) ** 2).mean(1)
    r64 = 1.0 / torch.sqrt(v64 + 1e-5)
    y64 = (xx - m64[:, None]) * r64[:, None] * w.double() + b.double()
    assert (yd[:M].cpu().double() - y64).abs().max().item() <= 1e-5
    assert (mean.cpu().double() - m64).abs().max().item() <= 1e-6 and ((rstd.cpu().double() - r64) / r64).abs().max().item() <= 1e-5
    assert torch.allclose(yd[:M].cpu(), torch.nn.functional.layer_norm(x, (N,), w, b, 1e-5), atol=1e-5)
    assert torch.equal(yd[M].cpu(), torch.full((N,), -3.0))


# ------------------------------------------------------------------ cfg4
def _run_mm(K, a, b, BM=128, BN=128, BK=64):
    M, Kd = a.shape
    N = b.shape[1]
    ad, bd = a.to(DEV), b.to(DEV)
    cd = torch.full((M, N), 5.0, dtype=a.dtype, device=DEV)
    grid = (triton.cdiv(M, BM) * triton.cdiv(N, BN),)
    k = K.matmul_tiles[grid](ad, bd, cd, M, N, Kd, ad.stride(0), ad.stride(1), bd.stride(0), bd.stride(1),
                             cd.stride(0), cd.stride(1), BM=BM, BN=BN, BK=BK, GROUP_M=8)
    torch.cuda.synchronize()
    assert k.function.family == "gemm"
    return cd


def test_cfg4_gemm_4096(K, oracle_cpu):
    torch.manual_seed(0)
    a = (torch.randn(4096, 4096) * 0.02).bfloat16()
    b = (torch.randn(4096, 4096) * 0.02).bfloat16()
    cd = _run_mm(K, a, b)
    ref = torch.matmul(a.to(DEV).float(), b.to(DEV).float())     # fp32 on the GPU: the full-size check
    assert relfro(cd.float(), ref) <= 1e-2
    # the oracle on four programs of the grid (first, a group boundary, the middle, the last)
    c = cd.cpu()
    for pid in (0, 255, 517, 1023):
        tile = torch.zeros(4096, 4096, dtype=torch.bfloat16)
        oracle_cpu.matmul_tiles(a, b, pids=(pid, pid + 1), out=tile)
        nz = tile.nonzero()
        r0, c0 = nz[:, 0].min().item() // 128 * 128, nz[:, 1].min().item() // 128 * 128
        assert relfro(c[r0:r0 + 128, c0:c0 + 128], tile[r0:r0 + 128, c0:c0 + 128]) <= 1e-2


def test_gemm_exact_against_permutation(K):
    # size-independent property at full size: A @ P for a permutation matrix P permutes columns exactly;
    # a transposed operand, a wrong tile origin or a wrong lane mapping cannot pass
    torch.manual_seed(1)
    n = 4096
    a = torch.randn(n, n).bfloat16()
    perm = torch.randperm(n)
    p = torch.zeros(n, n)
    p[perm, torch.arange(n)] = 1.0
    cd = _run_mm(K, a, p.bfloat16())
    assert torch.equal(cd.cpu(), a[:, perm])


@pytest.mark.parametrize("M,N,Kd,dtype", [(179, 321, 167, torch.bfloat16), (179, 321, 167, torch.float16),
                                         (128, 128, 64, torch.bfloat16), (2, 3, 5, torch.bfloat16),
                                         (130, 257, 72, torch.bfloat16), (256, 384, 200, torch.float16),
                                         (2048, 2304, 96, torch.bfloat16)])
def test_gemm_ragged_shapes(K, oracle_cpu, M, N, Kd, dtype):
    torch.manual_seed(M + N)
    a, b = (torch.randn(M, Kd) * 0.5).to(dtype), (torch.randn(Kd, N) * 0.5).to(dtype)
    cd = _run_mm(K, a, b)
    assert relfro(cd.cpu(), a.double() @ b.double()) <= 1e-2
    if M * N * Kd <= 179 * 321 * 167:
        assert relfro(cd.cpu(), oracle_cpu.matmul_tiles(a, b)) <= 1e-2


@pytest.mark.parametrize("M,N,Kd,dtype,pad", [(256, 256, 32, torch.bfloat16, 0), (256, 512, 64, torch.bfloat16, 0),
                                             (512, 256, 96, torch.bfloat16, 8), (768, 256, 160, torch.float16, 16),
                                             (256, 256, 4096, torch.bfloat16, 0), (1024, 1280, 352, torch.float16, 0),
                                             # enough tiles for the 128 x 256 and the 256 x 128 variants, and for 256 x 256
                                             (4096, 2048, 96, torch.bfloat16, 0), (4096, 2176, 64, torch.float16, 8), (4096, 4096, 32, torch.bfloat16, 0)])
def test_gemm_whole_tile_kernel(K, M, N, Kd, dtype, pad):
    # whole tiles: the direct-to-LDS kernels (256 x 256, 128 x 256, 256 x 128 or 128 x 128 tiles by the number of tiles the
    # problem gives), from one K tile (fewer than the pipeline's stages) upwards
    torch.manual_seed(M + Kd)
    A, B = (torch.randn(M, Kd + pad) * 0.5).to(dtype).to(DEV), (torch.randn(Kd, N + pad) * 0.5).to(dtype).to(DEV)
    Cfull = torch.full((M, N + pad), 5.0, dtype=dtype, device=DEV)
    a, b, c = A[:, :Kd], B[:, :N], Cfull[:, :N]
    k = K.matmul_tiles[(triton.cdiv(M, 128) * triton.cdiv(N, 128),)](a, b, c, M, N, Kd, a.stride(0), 1, b.stride(0), 1,
                                                                   c.stride(0), 1, BM=128, BN=128, BK=64, GROUP_M=8)
    torch.cuda.synchronize()
    want_kernel = {(4096, 2048): "gemm_dma_kernel<128x256>", (4096, 2176): "gemm_dma_kernel<256x128>", (4096, 4096): "gemm_dma_kernel"}.get((M, N), "gemm_dma_kernel<128x128>")
    if (M, N, Kd) == (256, 256, 4096):
        want_kernel += ", K slices"     # four tiles and a long K: cut into slices (test_gemm_in_k_slices_for_skinny_products)
    assert k.function.last_kernel == want_kernel
    assert relfro(c.cpu(), a.cpu().double() @ b.cpu().double()) <= 1e-2
    assert torch.equal(Cfull[:, N:].cpu(), torch.full((M, pad), 5.0, dtype=dtype))
    # exact: B selects and negates columns of A
    perm = torch.randperm(Kd)[:N] if N <= Kd else torch.randint(0, Kd, (N,))
    sel = torch.zeros(Kd, N)
    sel[perm, torch.arange(N)] = -1.0
    B[:, :N] = sel.to(dtype).to(DEV)
    K.matmul_tiles[(triton.cdiv(M, 128) * triton.cdiv(N, 128),)](a, b, c, M, N, Kd, a.stride(0), 1, b.stride(0), 1,
                                                               c.stride(0), 1, BM=128, BN=128, BK=64, GROUP_M=8)
    torch.cuda.synchronize()
    assert torch.equal(c.cpu(), -a.cpu()[:, perm])


@pytest.mark.parametrize("M,N,Kd,dtype,bt", [(128, 4096, 4096, torch.bfloat16, False), (300, 1032, 2048, torch.float16, False), (512, 2048, 8192, torch.bfloat16, True),
                                            (1000, 2048, 4096, torch.bfloat16, False), (64, 8192, 8192, torch.float16, False), (1, 256, 4096, torch.bfloat16, False),
                                            (512, 8192, 8192, torch.bfloat16, False), (500, 4104, 8192, torch.float16, False), (768, 2048, 16384, torch.bfloat16, False)])
def test_gemm_in_k_slices_for_skinny_products(K, M, N, Kd, dtype, bt):
    """Products with too few output tiles for the chip run with K cut into slices (a workgroup per tile and slice, fp32
    partial sums; a second kernel adds them and narrows, or, on 256 x 256 tiles, the slice of a tile that arrives last
    does): exact on small-integer operands whatever the order of
    the sums, ragged rows and columns, a column-major B, the buffer around C untouched; twice on one stream (the second
    launch reuses the workspace) and once more on another stream (a workspace of its own)."""
    g = torch.Generator(device="cpu").manual_seed(M + N + Kd)
    pad = 8
    A = torch.randint(-3, 4, (M, Kd), generator=g).to(dtype).to(DEV)
    Bm = torch.randint(-2, 3, (N + pad, Kd) if bt else (Kd, N + pad), generator=g).to(dtype).to(DEV)
    b = Bm[:N].t() if bt else Bm[:, :N]
    Cfull = torch.full((M + 3, N + pad), 5.0, dtype=dtype, device=DEV)
    c = Cfull[:M, :N]
    grid = (triton.cdiv(M, 128) * triton.cdiv(N, 128),)
    want = A.float() @ b.float()          # |sums| stay far below 2^11 * max: exact in fp32, and in 16 bits when small enough
    exact = want.abs().max().item() <= (256 if dtype == torch.bfloat16 else 2048)
    def launch():
        return K.matmul_tiles[grid](A, b, c, M, N, Kd, A.stride(0), 1, b.stride(0), b.stride(1), c.stride(0), 1, BM=128, BN=128, BK=64, GROUP_M=8)
    for _ in range(2):
        k = launch()
    torch.cuda.synchronize()
    assert k.function.family == "gemm" and k.function.last_kernel.endswith("K slices"), k.function.last_kernel
    assert torch.equal(c.float(), want.to(dtype).float()) if exact else relfro(c.float(), want) <= 1e-2
    assert torch.equal(Cfull[:, N:].cpu(), torch.full((M + 3, pad), 5.0, dtype=dtype)) and torch.equal(Cfull[M:].cpu(), torch.full((3, N + pad), 5.0, dtype=dtype))
    c.fill_(7.0)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        launch()
    side.synchronize()
    assert torch.equal(c.float(), want.to(dtype).float()) if exact else relfro(c.float(), want) <= 1e-2


@pytest.mark.parametrize("case", [
    # (batches, M, N, K, dtype, shared B, expected in the kernel's name)
    (8, 256, 384, 256, torch.bfloat16, False, "gemm_dma_kernel"),       # whole tiles
    (5, 130, 264, 96, torch.float16, False, "gemm_dma_kernel"),          # ragged rows and columns
    (3, 200, 136, 2048, torch.bfloat16, True, "K slices"),               # too few tiles: K slices, one workspace part per product; B shared
    (4, 70, 75, 50, torch.bfloat16, False, "gemm_mfma_kernel"),          # nothing aligned: the any-shape kernel
    (3, 100, 72, 40, torch.float32, False, "gemm_f32_kernel"),           # fp32 operands
])
def test_batched_matmul_runs_on_the_matmul_kernels(K, case):
    """A batch of products of one shape (tiles on program_id(0), the product on program_id(1), every operand at a batch
    stride) is proved product by product (each an exact cover of its own C, evenly spaced, results apart) and runs as
    one launch with the batch on grid.y: exact on small-integer operands, the padding around each C untouched."""
    Bn, M, N, Kd, dtype, shared_b, kernel = case
    g = torch.Generator(device="cpu").manual_seed(Bn * 1000 + M + N + Kd)
    pad = 8
    A = torch.randint(-3, 4, (Bn, M, Kd), generator=g).to(dtype).to(DEV)
    Bm = torch.randint(-2, 3, (1 if shared_b else Bn, Kd, N + pad), generator=g).to(dtype).to(DEV)
    b = Bm[:, :, :N]
    Cfull = torch.full((Bn, M + 2, N + pad), 5.0, dtype=dtype, device=DEV)
    c = Cfull[:, :M, :N]
    grid = (triton.cdiv(M, 128) * triton.cdiv(N, 128), Bn)
    k = K.batched_matmul[grid](A, b, c, M, N, Kd, A.stride(0), A.stride(1), 0 if shared_b else b.stride(0), b.stride(1), c.stride(0), c.stride(1), BM=128, BN=128, BK=32)
    torch.cuda.synchronize()
    assert k.function.family == "gemm" and kernel in k.function.last_kernel, k.function.last_kernel
    want = torch.matmul(A.float(), b.float())           # small integers: the sums are exact in fp32 in any order, and narrowed once
    assert torch.equal(c.float(), want.to(dtype).float())
    assert torch.equal(Cfull[:, :, N:].cpu(), torch.full((Bn, M + 2, pad), 5.0, dtype=dtype)) and torch.equal(Cfull[:, M:].cpu(), torch.full((Bn, 2, N + pad), 5.0, dtype=dtype))


def test_batched_matmul_with_overlapping_results_stays_on_the_generic_family(K):
    # two products whose results land on the same C are not one batch of independent products: the launch falls back to
    # the program-per-tile kernel (here both products are the same, so that the result does not depend on who writes last)
    M = N = Kd = 128
    g = torch.Generator(device="cpu").manual_seed(7)
    A = torch.randint(-3, 4, (1, M, Kd), generator=g).bfloat16().to(DEV)
    Bm = torch.randint(-2, 3, (1, Kd, N), generator=g).bfloat16().to(DEV)
    c = torch.zeros(M, N, dtype=torch.bfloat16, device=DEV)
    k = K.batched_matmul[(1, 2)](A, Bm, c, M, N, Kd, 0, A.stride(1), 0, Bm.stride(1), 0, c.stride(0), BM=128, BN=128, BK=32)
    torch.cuda.synchronize()
    assert k.function.family == "gemm" and k.function.last_kernel == "tile_program (hipRTC)", k.function.last_kernel
    assert torch.equal(c.float(), A[0].float() @ Bm[0].float())


@pytest.mark.parametrize("M,N,Kd,dtype,kernel", [(4000, 2048, 96, torch.bfloat16, "gemm_dma_kernel<128x256>"), (1000, 1032, 64, torch.float16, "gemm_dma_kernel<128x128>"),
                                                (130, 264, 96, torch.bfloat16, "gemm_dma_kernel<128x128>"), (4100, 4104, 64, torch.bfloat16, "gemm_dma_kernel"),
                                                (4090, 2056, 32, torch.float16, "gemm_dma_kernel<256x128>"), (1, 8, 32, torch.bfloat16, "gemm_dma_kernel<128x128>")])
def test_gemm_ragged_rows_and_columns_on_the_whole_k_tile_kernel(K, M, N, Kd, dtype, kernel):
    # any M and any N that is a multiple of 8 (K in whole tiles of 32): the direct-to-LDS kernels clamp the addresses of the
    # tiles that stick out of C and mask their stores; columns next to C in the same buffer stay as they were
    torch.manual_seed(M + N)
    pad = 8
    A, B = (torch.randn(M, Kd) * 0.5).to(dtype).to(DEV), (torch.randn(Kd, N + pad) * 0.5).to(dtype).to(DEV)
    Cfull = torch.full((M + 3, N + pad), 5.0, dtype=dtype, device=DEV)
    a, b, c = A, B[:, :N], Cfull[:M, :N]
    grid = (triton.cdiv(M, 128) * triton.cdiv(N, 128),)
    k = K.matmul_tiles[grid](a, b, c, M, N, Kd, a.stride(0), 1, b.stride(0), 1, c.stride(0), 1, BM=128, BN=128, BK=64, GROUP_M=8)
    torch.cuda.synchronize()
    assert k.function.last_kernel == kernel
    assert relfro(c.cpu(), a.cpu().double() @ b.cpu().double()) <= 1e-2
    assert torch.equal(Cfull[:, N:].cpu(), torch.full((M + 3, pad), 5.0, dtype=dtype)) and torch.equal(Cfull[M:].cpu(), torch.full((3, N + pad), 5.0, dtype=dtype))
    perm = torch.randint(0, Kd, (N,))
    sel = torch.zeros(Kd, N)
    sel[perm, torch.arange(N)] = -1.0
    B[:, :N] = sel.to(dtype).to(DEV)
    K.matmul_tiles[grid](a, b, c, M, N, Kd, a.stride(0), 1, b.stride(0), 1, c.stride(0), 1, BM=128, BN=128, BK=64, GROUP_M=8)
    torch.cuda.synchronize()
    assert torch.equal(c.cpu(), -a.cpu()[:, perm])
    assert torch.equal(Cfull[:, N:].cpu(), torch.full((M + 3, pad), 5.0, dtype=dtype)) and torch.equal(Cfull[M:].cpu(), torch.full((3, N + pad), 5.0, dtype=dtype))


@pytest.mark.parametrize("M,N,Kd,dtype", [(179, 321, 167, torch.bfloat16), (70, 90, 40, torch.float16), (512, 768, 96, torch.bfloat16),
                                         (1000, 130, 264, torch.float16)])
def test_matmul_with_wraparound_operands(K, oracle_cpu, M, N, Kd, dtype):
    # the stock tutorial form: rows of A / columns of B beyond the problem are read modulo M / N, not masked
    # (test_matmul.py:74-75 in the reference); the result must be the dense product, and bit-identical to
    # the masked form of the same kernel, which runs the same device code
    torch.manual_seed(M * 7 + N)
    a, b = (torch.randn(M, Kd) * 0.5).to(dtype), (torch.randn(Kd, N) * 0.5).to(dtype)
    ad, bd = a.to(DEV), b.to(DEV)
    cd = torch.full((M, N), 5.0, dtype=dtype, device=DEV)
    grid = (triton.cdiv(M, 128) * triton.cdiv(N, 128),)
    k = K.matmul_wrapped[grid](ad, bd, cd, M, N, Kd, ad.stride(0), 1, bd.stride(0), 1, cd.stride(0), 1,
                               BM=128, BN=128, BK=64, GROUP_M=8)
    torch.cuda.synchronize()
    assert k.function.family == "gemm"
    assert relfro(cd.cpu(), a.double() @ b.double()) <= 1e-2
    assert torch.equal(cd, _run_mm(K, a, b))
    if M * N * Kd <= 179 * 321 * 167:
        assert relfro(cd.cpu(), oracle_cpu.matmul_tiles(a, b)) <= 1e-2


def test_gemm_with_padded_pitches_and_untouched_border(K):
    torch.manual_seed(3)
    M, N, Kd = 200, 300, 150
    A, B = (torch.randn(M, Kd + 8) * 0.5).bfloat16().to(DEV), (torch.randn(Kd, N + 16) * 0.5).bfloat16().to(DEV)
    Cfull = torch.full((M, N + 8), 5.0, dtype=torch.bfloat16, device=DEV)
    a, b, c = A[:, :Kd], B[:, :N], Cfull[:, :N]
    K.matmul_tiles[(triton.cdiv(M, 128) * triton.cdiv(N, 128),)](a, b, c, M, N, Kd, a.stride(0), 1, b.stride(0), 1,
                                                               c.stride(0), 1, BM=128, BN=128, BK=64, GROUP_M=8)
    torch.cuda.synchronize()
    assert relfro(c.cpu(), a.cpu().double() @ b.cpu().double()) <= 1e-2
    assert torch.equal(Cfull[:, N:].cpu(), torch.full((M, 8), 5.0, dtype=torch.bfloat16))


# ------------------------------------------------------------------ cfg5
def _run_w8(K, a, w, s, BN=128, BK=128):
    M, Kd = a.shape
    N = w.shape[1]
    ad, wd, sd = a.to(DEV), w.to(DEV), s.to(DEV)
    cd = torch.full((M, N), 5.0, dtype=torch.float16, device=DEV)
    k = K.w8a16_matmul[(triton.cdiv(M, 16), triton.cdiv(N, BN))](ad, wd, sd, cd, M, N, Kd, ad.stride(0), 1, wd.stride(0), 1,
                                                                cd.stride(0), 1, BM=16, BN=BN, BK=BK)
    torch.cuda.synchronize()
    assert k.function.family == "gemm_w8a16"
    return cd


def test_cfg5_w8a16(K, oracle_cpu):
    torch.manual_seed(0)
    M, N, Kd = 16, 28672, 8192
    a = torch.randn(M, Kd).half()
    w = torch.randint(-127, 128, (Kd, N), dtype=torch.int8)
    s = (0.001 + 0.009 * torch.rand(N)).half()
    cd = _run_w8(K, a, w, s)
    ref = a.to(DEV).float() @ (w.to(DEV).half() * s.to(DEV)[None, :]).float()   # closed form, full size
    assert relfro(cd.float(), ref) <= 1e-2
    part = torch.zeros(M, N, dtype=torch.float16)
    for y in (0, 100, 223):                                                      # oracle on three column blocks
        oracle_cpu.w8a16_matmul(a, w, s, ys=(y, y + 1), out=part)
        assert relfro(cd.cpu()[:, y * 128:(y + 1) * 128], part[:, y * 128:(y + 1) * 128]) <= 1e-2


@pytest.mark.parametrize("M", [16, 32, 41])
def test_w8a16_exact_selection(K, M):
    # W picks and negates single rows, scales are powers of two: the result is exact in fp16.  At the full size of the
    # weight matrix: 16 rows (the decode shape), 32 (one launch with two groups of rows), 41 (two launches, the last ragged)
    torch.manual_seed(2)
    N, Kd = 28672, 8192
    a = torch.randn(M, Kd).half()
    cols = torch.arange(N)
    rows = (cols * 7) % Kd
    w = torch.zeros(Kd, N, dtype=torch.int8)
    sign = torch.where(cols % 2 == 0, 1, -1).to(torch.int8)
    w[rows, cols] = sign * 3
    s = torch.where(cols % 3 == 0, 0.5, 0.25).half()
    cd = _run_w8(K, a, w, s)
    want = (a[:, rows].float() * (sign.float() * 3 * s.float())[None, :]).half()
    assert torch.equal(cd.cpu(), want)


@pytest.mark.parametrize("M,N,Kd", [(13, 1000, 1000), (16, 256, 512), (1, 130, 70), (16, 4096, 4096), (5, 128, 8192),
                                    (3, 512, 2048), (16, 768, 32)])
def test_w8a16_ragged_shapes(K, oracle_cpu, M, N, Kd):
    torch.manual_seed(N)
    a = torch.randn(M, Kd).half()
    w = torch.randint(-127, 128, (Kd, N), dtype=torch.int8)
    s = (0.001 + 0.009 * torch.rand(N)).half()
    cd = _run_w8(K, a, w, s)
    ref = a.double() @ (w.half() * s[None, :]).double()
    assert relfro(cd.cpu(), ref) <= 1e-2
    if N * Kd <= 1000 * 1000:
        assert relfro(cd.cpu(), oracle_cpu.w8a16_matmul(a, w, s)) <= 1e-2


def test_w8a16_split_k_repeated_launches(K):
    # the K slices meet through a workspace whose arrival counters must be back at zero after every launch
    M, N, Kd = 16, 1024, 4096
    prev = None
    for seed in range(4):
        torch.manual_seed(seed)
        a = torch.randn(M, Kd).half()
        w = torch.randint(-127, 128, (Kd, N), dtype=torch.int8)
        s = (0.001 + 0.009 * torch.rand(N)).half()
        cd = _run_w8(K, a, w, s)
        ref = a.double() @ (w.half() * s[None, :]).double()
        assert relfro(cd.cpu(), ref) <= 1e-2
        again = _run_w8(K, a, w, s)
        assert torch.equal(cd, again)                     # slices are added in slice order: reproducible
        assert prev is None or not torch.equal(prev, cd)
        prev = cd


def test_w8a16_split_k_on_two_streams(K):
    # one plan launched alternately on two streams: each stream has partial tiles and arrival counters of its own, so
    # launches that overlap in time do not mix their K slices; every result equals the single-stream one bit for bit
    M, N, Kd = 16, 1024, 8192
    cases = []
    for seed in range(6):
        torch.manual_seed(100 + seed)
        a = torch.randn(M, Kd).half().to(DEV)
        w = torch.randint(-127, 128, (Kd, N), dtype=torch.int8).to(DEV)
        s = (0.001 + 0.009 * torch.rand(N)).half().to(DEV)
        cases.append((a, w, s, torch.zeros(M, N, dtype=torch.float16, device=DEV), torch.zeros(M, N, dtype=torch.float16, device=DEV)))

    def run(a, w, s, c):
        return K.w8a16_matmul[(1, N // 128)](a, w, s, c, M, N, Kd, a.stride(0), 1, w.stride(0), 1, c.stride(0), 1, BM=16, BN=128, BK=128)
    for a, w, s, want, _ in cases:
        k = run(a, w, s, want)
    torch.cuda.synchronize()
    assert int(k.function.describe_launch((1, N // 128, 1), [a.data_ptr(), w.data_ptr(), s.data_ptr(), want.data_ptr(), M, N, Kd, Kd, N, N])["split"]) > 1
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    for rep in range(20):
        for i, (a, w, s, _, got) in enumerate(cases):
            with torch.cuda.stream(streams[i % 2]):
                run(a, w, s, got)
    torch.cuda.synchronize()
    for a, w, s, want, got in cases:
        assert torch.equal(got, want)


# ----------------------------------------- launches and details the hand-written families decline
@pytest.mark.parametrize("M,N,Kd,dtype,kernel", [(4096, 4096, 4096, torch.bfloat16, "gemm_dma_kernel"), (200, 333, 150, torch.bfloat16, "gemm_mfma_kernel"),
                                                (512, 384, 200, torch.float16, "gemm_mfma_kernel"), (1000, 264, 96, torch.float16, "gemm_dma_kernel<128x128>"),
                                                (4096, 2048, 64, torch.bfloat16, "gemm_dma_kernel<128x256>"), (4090, 2176, 32, torch.bfloat16, "gemm_dma_kernel<256x128>")])
def test_gemm_with_column_major_b(K, M, N, Kd, dtype, kernel):
    # the tutorial's b.T (python/examples/test_matmul.py:129-136 passes b.stride(0), b.stride(1) whatever they are;
    # StructuredToMemref.cpp:105-138 takes any strides): B is stored [N, K], the kernel reads it through strides (1, K)
    torch.manual_seed(M + 1)
    a = (torch.randn(M, Kd) * 0.1).to(dtype).to(DEV)
    bt = (torch.randn(N, Kd) * 0.1).to(dtype).to(DEV)
    b = bt.t()
    c = torch.full((M, N), 5.0, dtype=dtype, device=DEV)
    grid = (triton.cdiv(M, 128) * triton.cdiv(N, 128),)
    k = K.matmul_tiles[grid](a, b, c, M, N, Kd, a.stride(0), a.stride(1), b.stride(0), b.stride(1), c.stride(0), c.stride(1),
                             BM=128, BN=128, BK=64, GROUP_M=8)
    torch.cuda.synchronize()
    # whole K tiles of 32 and N a multiple of 8: the direct-to-LDS kernels (B's stage laid out like A's); else the any-shape one
    assert k.function.family == "gemm" and (k.function.last_kernel == kernel or (kernel == "gemm_mfma_kernel" and k.function.last_kernel.startswith(kernel)))
    assert relfro(c.float(), a.float() @ b.float()) <= 1e-2
    # exact: B^T holds one -1 per column of B, so C is a signed selection of A's columns
    perm = torch.randint(0, Kd, (N,))
    bt.zero_()
    bt[torch.arange(N), perm.to(DEV)] = -1.0
    K.matmul_tiles[grid](a, b, c, M, N, Kd, a.stride(0), a.stride(1), b.stride(0), b.stride(1), c.stride(0), c.stride(1),
                         BM=128, BN=128, BK=64, GROUP_M=8)
    torch.cuda.synchronize()
    assert torch.equal(c.cpu(), -a.cpu()[:, perm])


@pytest.mark.parametrize("M,N,Kd,dtype,b_too,kernel", [(1024, 512, 96, torch.bfloat16, False, "gemm_dma_kernel<128x128>"), (4096, 4096, 64, torch.bfloat16, False, "gemm_dma_kernel"),
                                                      (1000, 264, 64, torch.float16, True, "gemm_dma_kernel<128x128>"), (4096, 2048, 32, torch.float16, True, "gemm_dma_kernel<128x256>"),
                                                      (4088, 2176, 96, torch.bfloat16, False, "gemm_dma_kernel<256x128>"), (1004, 256, 64, torch.bfloat16, False, "gemm_mfma_kernel<128x128x64>")])
def test_gemm_with_column_major_a_on_whole_k_tiles(K, M, N, Kd, dtype, b_too, kernel):
    # A stored [K, M] (the product A^T B of a weight gradient), alone or with a column-major B: whole K tiles of 32 and M a
    # multiple of 8 run on the direct-to-LDS kernels (A's stage laid out like a row-major B's); exact on a selection
    torch.manual_seed(M + N + Kd)
    at = torch.randint(-8, 9, (Kd, M)).to(dtype).to(DEV)
    a = at.t()
    perm = torch.randint(0, Kd, (N,))
    sel = torch.zeros(Kd, N)
    sel[perm, torch.arange(N)] = -1.0
    b = sel.t().contiguous().to(dtype).to(DEV).t() if b_too else sel.to(dtype).to(DEV)
    Cfull = torch.full((M + 2, N + 8), 5.0, dtype=dtype, device=DEV)
    c = Cfull[:M, :N]
    grid = (triton.cdiv(M, 128) * triton.cdiv(N, 128),)
    k = K.matmul_tiles[grid](a, b, c, M, N, Kd, a.stride(0), a.stride(1), b.stride(0), b.stride(1), c.stride(0), c.stride(1),
                             BM=128, BN=128, BK=64, GROUP_M=8)
    torch.cuda.synchronize()
    assert k.function.family == "gemm" and k.function.last_kernel == kernel
    assert torch.equal(c.cpu(), -a.cpu()[:, perm])
    assert torch.equal(Cfull[:, N:].cpu(), torch.full((M + 2, 8), 5.0, dtype=dtype)) and torch.equal(Cfull[M:].cpu(), torch.full((2, N + 8), 5.0, dtype=dtype))
    # and a random product within the family's tolerance
    at.copy_((torch.randn(Kd, M) * 0.5).to(dtype))
    bb = (torch.randn(N, Kd) * 0.5).to(dtype).to(DEV).t() if b_too else (torch.randn(Kd, N) * 0.5).to(dtype).to(DEV)
    K.matmul_tiles[grid](a, bb, c, M, N, Kd, a.stride(0), a.stride(1), bb.stride(0), bb.stride(1), c.stride(0), c.stride(1),
                         BM=128, BN=128, BK=64, GROUP_M=8)
    torch.cuda.synchronize()
    assert relfro(c.float(), a.float() @ bb.float()) <= 1e-2


@pytest.mark.parametrize("M,N,Kd,at,bt,BM,BN,BK", [(179, 321, 167, False, False, 32, 64, 16), (512, 384, 256, False, False, 128, 128, 32), (300, 260, 136, True, False, 64, 64, 32),
                                                  (1000, 1031, 77, False, True, 128, 128, 32), (130, 200, 64, True, True, 64, 128, 16), (1, 5, 3, False, False, 32, 32, 16),
                                                  (2048, 2048, 512, False, False, 128, 128, 32)])
def test_gemm_on_fp32_blocks(K, M, N, Kd, at, bt, BM, BN, BK):
    # tl.dot on fp32 blocks (the dtype of python/examples/test_matmul.py:137-157, whose first shape and blocks these are): the
    # reference multiplies in fp32, and so does the fp32 matrix-core kernel; any shape, any alignment, either layout of A and B
    torch.manual_seed(M + N + Kd)
    A = torch.randint(-8, 9, (Kd, M) if at else (M, Kd)).float().to(DEV)
    B = torch.randint(-8, 9, (N, Kd) if bt else (Kd, N)).float().to(DEV)
    a, b = (A.t() if at else A), (B.t() if bt else B)
    Cf = torch.full((M + 1, N + 3), 5.0, device=DEV)
    c = Cf[:M, :N]
    grid = (triton.cdiv(M, BM) * triton.cdiv(N, BN),)
    k = K.matmul_tiles[grid](a, b, c, M, N, Kd, a.stride(0), a.stride(1), b.stride(0), b.stride(1), c.stride(0), c.stride(1), BM=BM, BN=BN, BK=BK, GROUP_M=8)
    torch.cuda.synchronize()
    assert k.function.family == "gemm" and k.function.last_kernel == "gemm_f32_kernel"
    assert torch.equal(c.cpu(), (a.cpu().double() @ b.cpu().double()).float())      # integers: every partial sum is exact in fp32
    assert torch.equal(Cf[M].cpu(), torch.full((N + 3,), 5.0)) and torch.equal(Cf[:, N:].cpu(), torch.full((M + 1, 3), 5.0))
    # random data: fp32 products and sums, so far inside the reference's own atol=1e-2 (test_matmul.py:157)
    A.copy_(torch.randn_like(A))
    B.copy_(torch.randn_like(B))
    K.matmul_tiles[grid](a, b, c, M, N, Kd, a.stride(0), a.stride(1), b.stride(0), b.stride(1), c.stride(0), c.stride(1), BM=BM, BN=BN, BK=BK, GROUP_M=8)
    torch.cuda.synchronize()
    want = a.cpu().double() @ b.cpu().double()
    assert (c.cpu().double() - want).abs().max().item() <= 1e-3 and relfro(c.cpu(), want) <= 1e-5


def test_gemm_with_column_major_a_and_with_strides_no_kernel_takes(K):
    torch.manual_seed(11)
    M, N, Kd = 300, 260, 136
    at = (torch.randn(Kd, M) * 0.1).bfloat16().to(DEV)
    a = at.t()                                                            # strides (1, M)
    b = (torch.randn(Kd, N) * 0.1).bfloat16().to(DEV)
    c = torch.full((M, N), 5.0, dtype=torch.bfloat16, device=DEV)
    grid = (triton.cdiv(M, 128) * triton.cdiv(N, 128),)
    k = K.matmul_tiles[grid](a, b, c, M, N, Kd, a.stride(0), a.stride(1), b.stride(0), b.stride(1), c.stride(0), c.stride(1),
                             BM=128, BN=128, BK=64, GROUP_M=8)
    torch.cuda.synchronize()
    assert k.function.last_kernel.startswith("gemm_mfma_kernel")
    assert relfro(c.float(), a.float() @ b.float()) <= 1e-2
    # every second column of a wider B: neither stride of B is 1, which none of the matrix-product kernels reads; the
    # launch goes to the generic family's kernel for the same program instead of failing
    wide = (torch.randn(Kd, 2 * N) * 0.1).bfloat16().to(DEV)
    b2 = wide[:, ::2]
    c.fill_(5.0)
    k = K.matmul_tiles[grid](a, b2, c, M, N, Kd, a.stride(0), a.stride(1), b2.stride(0), b2.stride(1), c.stride(0), c.stride(1),
                             BM=128, BN=128, BK=64, GROUP_M=8)
    torch.cuda.synchronize()
    assert k.function.family == "gemm" and k.function.last_kernel == "tile_program (hipRTC)"
    assert relfro(c.float(), a.float() @ b2.float()) <= 1e-2


@pytest.mark.parametrize("M,N,Kd,BM,kernel", [(17, 384, 512, 16, "gemm_w8a16_kernel"), (64, 384, 512, 16, "gemm_w8a16_kernel"),
                                             (40, 512, 1024, 16, "gemm_w8a16_wide_kernel"), (100, 1024, 2048, 64, "gemm_w8a16_wide_kernel"),
                                             (33, 200, 100, 32, "gemm_w8a16_kernel"),
                                             # from 193 rows: the weights widened to fp16 once, then the tiled matmul kernels
                                             (193, 512, 1024, 16, "gemm_w8a16_widen_kernel + matmul"), (300, 1032, 2048, 64, "gemm_w8a16_widen_kernel + matmul"),
                                             (200, 260, 96, 64, "gemm_w8a16_kernel")])   # (N not a multiple of 8: the decode kernels, 13 launches)
def test_w8a16_beyond_the_decode_shape(K, oracle_cpu, M, N, Kd, BM, kernel):
    # the reference's matmul lowering has no shape limit (ConversionPatterns.hpp:1128-1201); the decode kernels take 16
    # or 32 rows, more rows run as one launch of them per group of rows (the last group ragged), whatever the program's BM
    torch.manual_seed(M)
    a = torch.randn(M, Kd).half()
    w = torch.randint(-127, 128, (Kd, N), dtype=torch.int8)
    s = (0.001 + 0.009 * torch.rand(N)).half()
    ad, wd, sd = a.to(DEV), w.to(DEV), s.to(DEV)
    cd = torch.full((M + 3, N), 5.0, dtype=torch.float16, device=DEV)
    for _ in range(2):   # twice: every launch leaves the split-K counters ready for the next
        k = K.w8a16_matmul[(triton.cdiv(M, BM), triton.cdiv(N, 128))](ad, wd, sd, cd, M, N, Kd, ad.stride(0), 1, wd.stride(0), 1,
                                                                      cd.stride(0), 1, BM=BM, BN=128, BK=128)
    torch.cuda.synchronize()
    assert k.function.family == "gemm_w8a16" and k.function.last_kernel == kernel
    assert relfro(cd[:M].cpu(), oracle_cpu.w8a16_matmul(a, w, s)) <= 1e-2
    assert relfro(cd[:M].cpu(), a.double() @ (w.half() * s[None, :]).double()) <= 1e-2
    assert torch.equal(cd[M:].cpu(), torch.full((3, N), 5.0, dtype=torch.float16))


@pytest.mark.parametrize("R,C,BR,BC", [(150, 700, 32, 256), (64, 64, 32, 32), (33, 1000, 8, 128), (40, 300, 16, 64)])
def test_programs_keep_their_ids_when_the_launcher_swaps_the_grid(R, C, BR, BC):
    # a program whose stores are contiguous along the dimension program_id(1) walks is launched with the grid's x and y
    # exchanged (neighbouring workgroups then write neighbouring columns); program_id and num_programs must not notice
    import extra_kernels as X
    import numpy as np
    out = torch.full((R + 1, C), -1, dtype=torch.int32, device=DEV)
    g0, g1 = triton.cdiv(R, BR), triton.cdiv(C, BC)
    k = X.stamp_tiles[(g0, g1)](out, R, C, BR=BR, BC=BC)
    torch.cuda.synchronize()
    assert k.function.family == "tile_program"
    rows, cols = np.arange(R)[:, None] // BR, np.arange(C)[None, :] // BC
    want = rows * 100 + cols + 10000 * g0 + 1000000 * g1
    assert np.array_equal(out[:R].cpu().numpy(), want)
    assert bool((out[R] == -1).all())


@pytest.mark.parametrize("R,C,BR,BC", [(200, 300, 64, 64), (513, 130, 32, 128), (64, 64, 64, 64), (1000, 77, 128, 32)])
def test_tiled_transpose_goes_through_lds(R, C, BR, BC):
    # tl.trans of a loaded tile: the load is copied to LDS (pitch = columns + 1) and read back transposed, so that both
    # the loads and the stores of a wavefront are contiguous; ragged edges in both dimensions, square and oblong tiles
    import extra_kernels as X
    torch.manual_seed(R + C)
    x = torch.randn(R, C, device=DEV)
    out = torch.full((C + 1, R), -7.0, device=DEV)
    k = X.transpose_tiles[(triton.cdiv(R, BR), triton.cdiv(C, BC))](x, out, R, C, BR=BR, BC=BC)
    torch.cuda.synchronize()
    assert k.function.family == "tile_program"
    assert torch.equal(out[:C], (x * 2.0).t())
    assert torch.equal(out[C], torch.full((R,), -7.0, device=DEV))


@pytest.mark.parametrize("rows,cols,pitch,block,dtype", [(64, 4096, 4096, 4096, torch.float16), (33, 781, 781, 1024, torch.float16), (5, 40000, 40000, 65536, torch.bfloat16),
                                                        (40, 784, 790, 1024, torch.bfloat16), (300, 1024, 1024, 1024, torch.float16), (7, 8, 8, 64, torch.float16)])
def test_row_softmax_on_16_bit_rows(K, rows, cols, pitch, block, dtype):
    # the same source on fp16 / bf16 tensors (widened after the load, narrowed before the store; the arithmetic is the fp32
    # kernel's): whole 16-byte chunks where rows are multiples of 8 elements and 16-byte aligned, element by element elsewhere
    torch.manual_seed(rows + cols)
    x = torch.randn(rows, pitch).to(dtype)[:, :cols]
    xd = x.to(DEV)
    full = torch.full((rows + 1, pitch), -9.0, dtype=dtype, device=DEV)
    od = full[:, :cols]
    k = K.row_softmax[(rows,)](od, xd, xd.stride(0), od.stride(0), cols, BLOCK=block)
    torch.cuda.synchronize()
    assert k.function.family == "row_softmax"
    want = torch.softmax(x.float(), 1)
    ulp = 2.0 ** -11 if dtype == torch.float16 else 2.0 ** -8
    assert (od[:rows].cpu().float() - want).abs().max().item() <= ulp        # results lie in [0, 1]: one rounding to 16 bits
    assert (od[:rows].cpu() != want.to(dtype)).float().mean().item() < 0.01   # and nearly all are the correctly rounded value
    assert torch.equal(full[rows].cpu(), torch.full((pitch,), -9.0, dtype=dtype)) and torch.equal(full[:, cols:].cpu(), torch.full((rows + 1, pitch - cols), -9.0, dtype=dtype))


@pytest.mark.parametrize("H,seq,D,BM,BN", [(3, 200, 64, 64, 64), (2, 80, 32, 32, 32), (4, 1024, 64, 64, 32), (1, 33, 64, 32, 64), (2, 300, 128, 32, 64)])
def test_flash_attention_forward(H, seq, D, BM, BN):
    # two tile products per step and an online softmax: the running maximum and sum are loop-carried vectors that the
    # [BM, BN] scores and the [BM, D] accumulator read as columns, so they are kept in LDS next to their owners' registers
    import extra_kernels as X
    torch.manual_seed(seq + D)
    q, k, v = (torch.randn(H, seq, D, device=DEV).half() for _ in range(3))
    o = torch.full((H + 1, seq, D), 3.0, device=DEV, dtype=torch.float16)
    kern = X.attention_fwd[(triton.cdiv(seq, BM), H)](q, k, v, o, D ** -0.5, seq, seq * D, D, BM=BM, BN=BN, D=D)
    torch.cuda.synchronize()
    assert kern.function.family == "tile_program"
    s = torch.einsum("hqd,hkd->hqk", q.double(), k.double()) * D ** -0.5
    want = torch.einsum("hqk,hkd->hqd", torch.softmax(s, -1), v.double())
    assert (o[:H].double() - want).abs().max().item() <= 4e-3          # fp16 probabilities and output
    assert torch.equal(o[H], torch.full((seq, D), 3.0, device=DEV, dtype=torch.float16))


def test_softmax_rows_the_row_kernel_declines(K, oracle_cpu):
    import extra_kernels as X
    torch.manual_seed(5)
    # rows of 32768 and 65536 columns: 8 and 16 wavefronts per row on the row kernel; 131072: more than it keeps in registers
    for cols, block, family in [(30000, 32768, "row_softmax"), (40001, 65536, "row_softmax"), (70000, 131072, "tile_program")]:
        x = torch.randn(6, cols)
        xd = x.to(DEV)
        od = torch.full((7, cols), -9.0, device=DEV)
        k = K.row_softmax[(6,)](od, xd, xd.stride(0), od.stride(0), cols, BLOCK=block)
        torch.cuda.synchronize()
        assert k.function.family == family
        assert torch.allclose(od[:6].cpu(), torch.softmax(x, 1))
        assert (od[:6].cpu() - oracle_cpu.row_softmax(x, BLOCK=block)).abs().max().item() <= 1e-5
        assert torch.equal(od[6].cpu(), torch.full((cols,), -9.0))
    # every third element of the input row
    x = torch.randn(40, 3 * 700)
    xd = x.to(DEV)
    od = torch.full((40, 700), -9.0, device=DEV)
    k = X.strided_row_softmax[(40,)](od, xd, xd.stride(0), od.stride(0), 3, 700, BLOCK=1024)
    torch.cuda.synchronize()
    assert k.function.family == "tile_program"
    assert torch.allclose(od.cpu(), torch.softmax(x[:, ::3], 1))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_vec_add_in_16_bit_floats(K, dtype):
    torch.manual_seed(7)
    n = 70000
    x, y = torch.randn(n).to(dtype).to(DEV), torch.randn(n).to(dtype).to(DEV)
    z = torch.zeros(n + 8, dtype=dtype, device=DEV)
    k = K.vec_add[(triton.cdiv(n, 1024),)](x, y, z, n, BLOCK=1024)
    torch.cuda.synchronize()
    assert k.function.family == "fused_map"
    assert torch.equal(z[:n], x + y) and z[n:].abs().sum().item() == 0


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_narrowing_rounds_to_nearest_even_in_both_generated_families(dtype):
    """arith.truncf f32 -> bf16 / f16 rounds to nearest even (the reference lowers it to LLVM's fptrunc): ties, values a
    bit above and below them, denormal results, overflow to infinity, signed zeros and NaNs, through an elementwise pass and
    through a program with a reduction.  Every float32 whose low 16 bits are a tie or next to one, over all exponents."""
    import extra_kernels as X
    hi = torch.arange(0, 1 << 16, dtype=torch.int64)                         # every sign / exponent / high mantissa pattern
    lows = torch.tensor([0x0000, 0x0001, 0x7FFF, 0x8000, 0x8001, 0xFFFF, 0x1000, 0x9000, 0x0FFF, 0xEFFF], dtype=torch.int64)
    bits = ((hi[:, None] << 16) | lows[None, :]).reshape(-1)
    x = torch.from_numpy(bits.numpy().astype("uint32").view("float32").copy())
    n = x.numel()
    want = x.to(dtype)
    nan = torch.isnan(x)
    xd = x.to(DEV)
    y = torch.zeros(n + 8, dtype=dtype, device=DEV)
    k = X.narrow_scaled[(triton.cdiv(n, 1024),)](xd, y, n, 1.0, BLOCK=1024)
    torch.cuda.synchronize()
    assert k.function.family == "fused_map"
    got = y[:n].cpu()
    assert torch.equal(got.view(torch.int16)[~nan], want.view(torch.int16)[~nan]) and torch.isnan(got[nan]).all()
    assert y[n:].abs().sum().item() == 0
    cols = 1000
    rows = n // cols
    y2 = torch.zeros(rows * cols, dtype=dtype, device=DEV)
    m = torch.zeros(rows, device=DEV)
    k = X.narrow_scaled_with_row_max[(rows,)](xd, y2, m, cols, 1.0, BLOCK=1024)
    torch.cuda.synchronize()
    assert k.function.family == "tile_program"
    got = y2.cpu()
    sel = ~nan[:rows * cols]
    assert torch.equal(got.view(torch.int16)[sel], want[:rows * cols].view(torch.int16)[sel]) and torch.isnan(got[~sel]).all()


def test_tile_program_while_loops():
    """`while` (scf.while whose condition passes the loop's arguments on, the form the frontend writes) runs as a loop
    that every thread of a program leaves together: a trip count that depends on an argument, and one that depends on
    the data and differs from program to program (small integers: the sums are exact)."""
    import extra_kernels as X
    for n in (1, 2, 1000, 1025):
        x = torch.randn(n, device=DEV)
        y = torch.full((n + 3,), 9.0, device=DEV)
        k = X.while_halve[(triton.cdiv(n, 256),)](x, y, n, BLOCK=256)
        torch.cuda.synchronize()
        assert k.function.family == "tile_program"
        assert torch.equal(y[:n], x * 0.5 ** (n.bit_length() - 1)) and torch.equal(y[n:].cpu(), torch.full((3,), 9.0))
    rows, n, B = 9, 3000, 256
    g = torch.Generator(device="cpu").manual_seed(5)
    x = torch.randint(0, 4, (rows, n + 5), generator=g).float()
    x[3] = 0.0                                    # never reaches the limit: runs to the end of the row
    x[4, 0] = 1000.0                              # reaches it in the first piece
    limit = 700.0
    out = torch.zeros(rows, device=DEV)
    cnt = torch.zeros(rows, dtype=torch.int32, device=DEV)
    k = X.while_sum_until[(rows,)](x.to(DEV), out, cnt, x.stride(0), n, limit, BLOCK=B)
    torch.cuda.synchronize()
    assert k.function.family == "tile_program"
    want_sum, want_cnt = [], []
    for r in range(rows):
        kk, acc = 0, 0.0
        while kk < n and acc < limit:
            acc += float(x[r, kk:min(kk + B, n)].sum())
            kk += B
        want_sum.append(acc)
        want_cnt.append(kk)
    assert out.cpu().tolist() == want_sum and cnt.cpu().tolist() == want_cnt
    assert len(set(want_cnt)) > 2                 # the programs did leave after different numbers of rounds
    # a carried block of pointers; a `while` inside a `for`
    xs = torch.randint(-3, 4, (5, 1000 + 7), generator=g).float()
    out = torch.zeros(5, device=DEV)
    X.while_carried_pointer[(5,)](xs.to(DEV), out, xs.stride(0), 1000, BLOCK=256)
    torch.cuda.synchronize()
    assert torch.equal(out.cpu(), xs[:, :1000].sum(1))
    xv = torch.randint(-2, 3, (256,), generator=g).float()
    out = torch.zeros(256, device=DEV)
    X.while_inside_for[(1,)](xv.to(DEV), out, 37, BLOCK=256)
    torch.cuda.synchronize()
    total = 0
    for i in range(37):
        kk = i
        while kk > 0:
            total += kk
            kk //= 2
    assert torch.equal(out.cpu(), xv * total)


@pytest.mark.parametrize("rows,N,BLOCK", [(7, 5000, 1024), (3, 1024, 1024), (5, 777, 256), (2, 1, 64)])
def test_tile_program_carries_scalars_through_a_loop(rows, N, BLOCK):
    """Scalars that are not index expressions (a running maximum and sum, a count) carried by a loop: the reference
    carries them as scf.for iter_args like any other value.  An online softmax over rows read in pieces against
    torch.softmax (1e-6: the pieces rescale the sum), the count of positive elements exact."""
    import extra_kernels as X
    torch.manual_seed(N)
    x = torch.randn(rows, N + 3, device=DEV)
    y = torch.full_like(x, -1.0)
    cnt = torch.zeros(rows, dtype=torch.int32, device=DEV)
    k = X.softmax_row_in_pieces[(rows,)](x, y, cnt, x.stride(0), N, BLOCK=BLOCK)
    torch.cuda.synchronize()
    assert k.function.family == "tile_program"
    assert (y[:, :N] - torch.softmax(x[:, :N], 1)).abs().max().item() <= 1e-6
    assert torch.equal(y[:, N:].cpu(), torch.full((rows, 3), -1.0))
    assert torch.equal(cnt.cpu(), (x[:, :N] > 0).sum(1).int().cpu())


@pytest.mark.parametrize("dtype", [torch.float32, torch.int32])
def test_tile_program_load_after_store_sees_the_store(dtype):
    # the serial reference finishes the store before the next load of the same buffer starts
    import extra_kernels as X
    torch.manual_seed(9)
    n = 5000
    p = (torch.randn(n) * 8).to(dtype).to(DEV)
    p0 = p.clone()
    q = torch.zeros(n, dtype=dtype, device=DEV)
    k = X.double_in_place_then_square[(triton.cdiv(n, 1024),)](p, q, n, BLOCK=1024)
    torch.cuda.synchronize()
    assert k.function.family == "tile_program"
    assert torch.equal(p, p0 + p0) and torch.equal(q, (p0 + p0) * (p0 + p0))


def test_tile_program_scalar_read_modify_write():
    import extra_kernels as X
    acc = torch.tensor([41], dtype=torch.int32, device=DEV)
    out = torch.zeros(2048, dtype=torch.int32, device=DEV)
    for step in range(3):
        X.bump_counter_and_report[(1,)](acc, out, BLOCK=1024)
        torch.cuda.synchronize()
        assert acc.item() == 42 + step
        assert torch.equal(out[:1024], torch.full((1024,), 41 + step, dtype=torch.int32, device=DEV))   # the value read before the write
        assert torch.equal(out[1024:], torch.full((1024,), 42 + step, dtype=torch.int32, device=DEV))   # and the one read after it


# ------------------------------------------------------------- fused maps
def _lanes(name, n, scalars, inputs, out_dtype, block=1024):
    from conftest import golden_ttir
    from oracle import ttir_lanes
    mem = {i: a for i, a in enumerate(inputs)}
    out = np.zeros(n, dtype=out_dtype)
    mem[len(inputs)] = out
    ttir_lanes.Interpreter(golden_ttir(name)).run(((n + block - 1) // block,), [None] * (len(inputs) + 1) + [n] + list(scalars), mem)
    return out


@pytest.mark.parametrize("n", [1, 1023, 5000, (1 << 20) + 3])
def test_fused_map_gelu(K, n):
    torch.manual_seed(n)
    x, b = torch.randn(n) * 2, torch.randn(n)
    xd, bd, yd = x.to(DEV), b.to(DEV), torch.full((n + 8,), 5.0, device=DEV)
    k = K.gelu_tanh_bias[(triton.cdiv(n, 1024),)](xd, bd, yd, n, BLOCK=1024)
    torch.cuda.synchronize()
    assert k.function.family == "fused_map" and k.function.last_kernel == "fused_map (hipRTC)"
    v = (x + b).double()
    want = 0.5 * v * (1 + torch.tanh(0.7978845608028654 * (v + 0.044715 * v ** 3)))
    assert (yd[:n].cpu().double() - want).abs().max().item() <= 2e-6
    assert torch.equal(yd[n:].cpu(), torch.full((8,), 5.0))               # nothing past the mask is written
    if n <= 5000:                                                          # the oracle: every op as the lanes do it
        ref = _lanes("gelu_tanh_bias", n, [], [x.numpy().copy(), b.numpy().copy()], np.float32)
        assert np.abs(yd[:n].cpu().numpy() - ref).max() <= 1e-6


def test_fused_map_scalars_compare_select(K):
    n = 4099
    torch.manual_seed(5)
    x, y = torch.randn(n), torch.randn(n)
    x[:4] = torch.tensor([float("nan"), 1.0, float("-inf"), 0.5])
    y[:4] = torch.tensor([0.0, float("nan"), 2.0, 0.5])
    xd, yd, od = x.to(DEV), y.to(DEV), torch.zeros(n, device=DEV)
    k = K.clamp_scale_where[(triton.cdiv(n, 1024),)](xd, yd, od, n, -0.5, 1.25, 3.0, BLOCK=1024)
    torch.cuda.synchronize()
    assert k.function.family == "fused_map"
    ref = _lanes("clamp_scale_where", n, [-0.5, 1.25, 3.0], [x.numpy().copy(), y.numpy().copy()], np.float32)
    got = od.cpu().numpy()
    assert np.array_equal(np.isnan(got), np.isnan(ref))
    assert np.array_equal(got[~np.isnan(ref)], ref[~np.isnan(ref)])      # one IEEE op per value and exact selects: bit-exact
    # other scalar arguments reuse the plan with new immediates
    K.clamp_scale_where[(triton.cdiv(n, 1024),)](xd, yd, od, n, 0.0, 0.25, -2.0, BLOCK=1024)
    ref = _lanes("clamp_scale_where", n, [0.0, 0.25, -2.0], [x.numpy().copy(), y.numpy().copy()], np.float32)
    got = od.cpu().numpy()
    assert np.array_equal(got[~np.isnan(ref)], ref[~np.isnan(ref)])


@pytest.mark.parametrize("n", [7, 4096, 100003])
def test_fused_map_fp16_io(K, n):
    torch.manual_seed(n)
    g, u = (torch.randn(n) * 3).half(), torch.randn(n).half()
    gd, ud, od = g.to(DEV), u.to(DEV), torch.zeros(n, dtype=torch.float16, device=DEV)
    k = K.silu_mul_f16[(triton.cdiv(n, 1024),)](gd, ud, od, n, BLOCK=1024)
    torch.cuda.synchronize()
    assert k.function.family == "fused_map"
    want = (g.double() / (1 + torch.exp(-g.double())) * u.double())
    assert ((od.cpu().double() - want).abs() <= 1e-3 * want.abs() + 1e-4).all()     # half an fp16 ulp is 4.9e-4 relative
    if n <= 4096:
        ref = _lanes("silu_mul_f16", n, [], [g.numpy().copy(), u.numpy().copy()], np.float16)
        # fp32 exp differs in the last bit between libm and the device: at most one fp16 ulp after the final rounding
        assert np.abs(od.cpu().numpy().astype(np.float32) - ref.astype(np.float32)).max() <= 2e-3 * max(1.0, np.abs(ref.astype(np.float32)).max())


@pytest.mark.parametrize("kernel", ["gelu", "where", "silu"])
def test_fused_map_interpreter_and_compiled_kernel_agree(K, kernel, monkeypatch):
    # the register program runs either on the interpreter kernel or as a kernel compiled from the same program:
    # every instruction is the same expression in both, so the outputs are the same bits
    n = 70001
    torch.manual_seed(11)
    x, y = (torch.randn(n) * 3).to(DEV), torch.randn(n).to(DEV)
    outs = []
    for mode in ("interpreter", "compiled"):
        if mode == "interpreter":
            monkeypatch.setenv("TTS_FUSED_MAP", "interpreter")
        else:
            monkeypatch.delenv("TTS_FUSED_MAP", raising=False)
        if kernel == "gelu":
            o = torch.zeros(n, device=DEV)
            k = K.gelu_tanh_bias[(triton.cdiv(n, 1024),)](x, y, o, n, BLOCK=1024)
        elif kernel == "where":
            o = torch.zeros(n, device=DEV)
            k = K.clamp_scale_where[(triton.cdiv(n, 1024),)](x, y, o, n, -0.75, 0.5, 1.5, BLOCK=1024)
        else:
            o = torch.zeros(n, dtype=torch.float16, device=DEV)
            k = K.silu_mul_f16[(triton.cdiv(n, 1024),)](x.half(), y.half(), o, n, BLOCK=1024)
        torch.cuda.synchronize()
        assert k.function.last_kernel == ("mapn_kernel" if mode == "interpreter" else "fused_map (hipRTC)")
        outs.append(o)
    assert torch.equal(outs[0], outs[1])


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("rows,n_cols,BLOCK,rows_on_x", [(37, 100, 16, True), (37, 100, 16, False), (5, 1000, 64, True), (300, 70, 32, False),
                                                         (3, 5000, 1024, True), (9, 3000, 512, False), (1, 8, 8, True), (70000, 24, 8, False)])
def test_fused_map_small_blocks_share_a_workgroup(rows, n_cols, BLOCK, rows_on_x, dtype):
    """Programs whose blocks need fewer than 256 threads share a workgroup, and the launch walks the grid along the
    axis on which the output advances least: every element still comes from its own program (bit-exact against the
    same two roundings in torch), ragged last column blocks stay masked, the padding between rows is untouched."""
    import extra_kernels as X
    torch.manual_seed(rows + n_cols)
    stride = n_cols + 5
    x = torch.randn(rows, stride, device=DEV).to(dtype)
    y = torch.randn(rows, stride, device=DEV).to(dtype)
    out = torch.full((rows, stride), 7.0, dtype=dtype, device=DEV)
    nb = triton.cdiv(n_cols, BLOCK)
    grid = (rows, nb) if rows_on_x else (nb, rows)
    k = X.scale_add_2d[grid](x, y, out, n_cols, stride, 0.5, ROWS_ON_X=rows_on_x, BLOCK=BLOCK)
    torch.cuda.synchronize()
    assert k.function.family == "fused_map" and k.function.last_kernel == "fused_map (hipRTC)", k.function.last_kernel
    want = ((0.5 * x[:, :n_cols].float()).to(dtype) + y[:, :n_cols]) if dtype != torch.float32 else 0.5 * x[:, :n_cols] + y[:, :n_cols]
    assert torch.equal(out[:, :n_cols], want)
    assert torch.equal(out[:, n_cols:].cpu(), torch.full((rows, 5), 7.0, dtype=dtype))


@pytest.mark.parametrize("seq,heads,half", [(33, 5, 64), (7, 3, 16), (2, 1, 128)])
def test_fused_map_rotary_embedding(K, seq, heads, half):
    # a program per (position, head) on blocks of `half` elements, two outputs: fp32 products and differences rounded
    # one by one, as torch rounds them, then narrowed: bit-exact
    torch.manual_seed(seq)
    x = torch.randn(seq, heads * 2 * half, device=DEV).half()
    c, sn = torch.randn(seq, half, device=DEV), torch.randn(seq, half, device=DEV)
    out = torch.zeros_like(x)
    k = K.rotary_embedding[(seq, heads)](x, c, sn, out, x.stride(0), HALF=half)
    torch.cuda.synchronize()
    assert k.function.family == "fused_map" and k.function.last_kernel == "fused_map (hipRTC)"
    xv = x.float().view(seq, heads, 2, half)
    x1, x2 = xv[:, :, 0], xv[:, :, 1]
    cc, ss = c[:, None, :], sn[:, None, :]
    want = torch.stack([x1 * cc - x2 * ss, x2 * cc + x1 * ss], 2).half().view(seq, -1)
    assert torch.equal(out, want)


def test_fused_map_two_ops(K):
    import extra_kernels as X
    n = 3000
    torch.manual_seed(1)
    a, b = torch.randn(n), torch.randn(n)
    zd = torch.zeros(n, device=DEV)
    k = X.fused_mul_add[(triton.cdiv(n, 256),)](a.to(DEV), b.to(DEV), zd, n, BLOCK=256)
    torch.cuda.synchronize()
    assert k.function.family == "fused_map"
    assert torch.equal(zd.cpu(), a * b + a)                              # two roundings, no contraction into an fma


# ------------------------------------------------------------- tile programs (generic family)
# Expected values marked "reference golden" are the literal tensors the reference's own functional tests assert
# (python/examples/test_modulo.py, test_mask.py); the kernels are ours, written to the same access patterns.
def _run_wrap(kernel, M, N, *consts, **kw):
    a = torch.arange(0, M * N, dtype=torch.float32, device=DEV).reshape(M, N)
    out = torch.full((M, N), 88888.0, device=DEV)
    k = kernel[(1,)](a, out, M, N, a.stride(0), a.stride(1), out.stride(0), out.stride(1), **kw)
    torch.cuda.synchronize()
    assert k.function.family == "tile_program"
    return out.cpu().int()


def test_tile_program_wraparound_reference_goldens():
    import extra_kernels as X
    F = 88888
    got = _run_wrap(X.wrap_rows_loop, 4, 8, BK=4)            # test_modulo.py:53-57 (stacked)
    assert got.tolist() == [list(range(16, 24)), list(range(24, 32)), list(range(0, 8)), list(range(8, 16))]
    got = _run_wrap(X.wrap_cols_row, 8, 8)                   # test_modulo.py:91-100 (one row)
    assert got.tolist() == [[62, 63, 56, 57, F, F, F, F]] + [[F] * 8] * 7
    got = _run_wrap(X.wrap_cols_tile, 8, 8)                  # test_modulo.py:136-145 (side by side)
    assert got.tolist() == [[22, 23, 16, 17, F, F, F, F], [30, 31, 24, 25, F, F, F, F], [38, 39, 32, 33, F, F, F, F],
                            [46, 47, 40, 41, F, F, F, F]] + [[F] * 8] * 4
    got = _run_wrap(X.wrap_cols_masked_loop, 12, 8, BK=4)    # test_modulo.py:193-206 (mask, other=-99, loop down the rows)
    assert got.tolist() == [[22, 23, 16, 17, 54, 55, 48, 49], [30, 31, 24, 25, 62, 63, 56, 57], [-99] * 8, [-99] * 8] + [[F] * 8] * 8


def test_tile_program_all_masked_load_reference_golden():
    import extra_kernels as X
    inp = torch.arange(0, 8, dtype=torch.int32, device=DEV)
    out = torch.full((8,), -2, dtype=torch.int32, device=DEV)
    k = X.masked_gather_const[(1,)](inp, out)
    torch.cuda.synchronize()
    assert k.function.family == "tile_program" and k.function.last_kernel == "tile_program (hipRTC)"
    assert out.cpu().tolist() == [-1, -1, -1, -1, -2, -2, -2, -2]  # test_mask.py:38


def test_tile_program_scalar_condition_in_mask_reference_goldens():
    import extra_kernels as X
    inp = torch.arange(0, 8, dtype=torch.int32, device=DEV)
    for bound, value, want in [(4, 3, [0, 1, 2, 3, -1, -1, -1, -1]),      # test_mask.py:57-58: the scalar condition holds
                               (4, 8, [-1] * 8)]:                          # test_mask.py:64-65: it does not
        out = torch.full((8,), -2, dtype=torch.int32, device=DEV)
        X.mask_with_scalar[(1,)](inp, out, bound, value)
        torch.cuda.synchronize()
        assert out.cpu().tolist() == want


def test_tile_program_block_pointers():
    # tl.make_block_ptr / tl.advance arrive as ordinary pointer arithmetic on i64 tensors with `0 <= i < shape` masks
    # (the frontend's rewrite_tensor_pointer pass); boundary checks become the per-dimension extents
    import extra_kernels as X
    for rows, cols, BR, BC in [(512, 256, 4, 2), (37, 50, 16, 32)]:
        x = torch.arange(0, rows * cols, dtype=torch.float32, device=DEV).reshape(rows, cols)
        y = torch.full((rows, cols), -1.0, device=DEV)
        k = X.block_ptr_affine[(triton.cdiv(rows, BR), triton.cdiv(cols, BC))](x, y, rows, cols, x.stride(0), x.stride(1), BR=BR, BC=BC)
        torch.cuda.synchronize()
        assert k.function.family == "tile_program"
        assert torch.equal(y, 2 * x + 1)                                    # test_load_2d_tensor_block.py's expectation
    x = torch.randn(21, 100, device=DEV)
    y = torch.zeros(21, 100, device=DEV)
    X.block_ptr_row_walk[(triton.cdiv(21, 8),)](x, y, 21, 100, x.stride(0), BR=8, BC=32)
    torch.cuda.synchronize()
    assert torch.equal(y, x * 0.5)


def test_tile_program_block_pointer_ops():
    """The same kernels with tt.make_tensor_ptr / tt.advance kept as ops (raw_block_pointers=True): a block pointer is a
    structured access whose boundaryCheck dimensions are cut at the parent tensor's extent, loop-carried ones carry their
    position.  Checked on test_load_2d_tensor_block.py's expectation, exact integer-valued products and the lane interpreter."""
    import extra_kernels as X
    from test_planner import compile_ttir
    from oracle import ttir_lanes
    for rows, cols, BR, BC in [(512, 256, 4, 2), (37, 50, 16, 32)]:
        x = torch.arange(0, rows * cols, dtype=torch.float32, device=DEV).reshape(rows, cols)
        y = torch.full((rows, cols), -1.0, device=DEV)
        k = X.block_ptr_affine[(triton.cdiv(rows, BR), triton.cdiv(cols, BC))](x, y, rows, cols, x.stride(0), x.stride(1), BR=BR, BC=BC, raw_block_pointers=True)
        torch.cuda.synchronize()
        assert k.function.family == "tile_program" and "tt.make_tensor_ptr" in k.asm["ttir"]
        assert torch.equal(y, 2 * x + 1)
    x = torch.randn(21, 100, device=DEV)
    y = torch.zeros(21, 100, device=DEV)
    k = X.block_ptr_row_walk[(triton.cdiv(21, 8),)](x, y, 21, 100, x.stride(0), BR=8, BC=32, raw_block_pointers=True)
    torch.cuda.synchronize()
    assert "tt.advance" in k.asm["ttir"] and torch.equal(y, x * 0.5)
    g = torch.Generator(device="cpu").manual_seed(3)
    sig = {"a_ptr": "*bf16", "b_ptr": "*bf16", "c_ptr": "*fp32", "M": "i32", "N": "i32", "K": "i32", "sam": "i32", "sbk": "i32",
           "scm": "i32", "BM": "constexpr", "BN": "constexpr", "BK": "constexpr", "PAD": "constexpr"}
    for pad, (M, N, Kd), (BM, BN, BK) in [("zero", (200, 150, 72), (64, 64, 32)), ("nan", (130, 70, 64), (64, 64, 32)), ("nan", (40, 50, 24), (32, 32, 16))]:
        a = torch.randint(-2, 3, (M, Kd), generator=g).to(torch.bfloat16).to(DEV)
        b = torch.randint(-2, 3, (Kd, N), generator=g).to(torch.bfloat16).to(DEV)
        c = torch.full((M, N), -7.0, device=DEV)
        grid = (triton.cdiv(M, BM), triton.cdiv(N, BN))
        k = X.block_ptr_matmul[grid](a, b, c, M, N, Kd, a.stride(0), b.stride(0), c.stride(0), BM=BM, BN=BN, BK=BK, PAD=pad, raw_block_pointers=True)
        torch.cuda.synchronize()
        assert k.function.family == "tile_program" and "tt.make_tensor_ptr" in k.asm["ttir"]
        if Kd % BK == 0 or pad == "zero":
            assert torch.equal(c, a.float() @ b.float())
        else:
            assert torch.isnan(c).all()
        if M * N <= 4096:
            ttir = compile_ttir(X.block_ptr_matmul, sig, {"BM": BM, "BN": BN, "BK": BK, "PAD": pad}, raw_block_pointers=True)
            mem = {0: a.view(torch.int16).cpu().numpy().view(np.uint16).reshape(-1).copy(), 1: b.view(torch.int16).cpu().numpy().view(np.uint16).reshape(-1).copy(),
                   2: np.full(M * N, -7, np.float32)}
            ttir_lanes.Interpreter(ttir).run(grid, [None, None, None, M, N, Kd, Kd, N, N], mem)
            assert np.array_equal(mem[2].reshape(M, N), c.cpu().numpy(), equal_nan=True)


def test_tile_program_pointer_blocks_chosen_by_branch_and_where():
    """A block of pointers yielded by an if / else (gathered on one side, strided on the other) and tl.where between two
    blocks of pointers: both become blocks of 64-bit offsets from the one argument.  Exact against the index arithmetic
    in numpy and against the lane interpreter."""
    import extra_kernels as X
    from test_planner import compile_ttir
    from oracle import ttir_lanes
    g = torch.Generator(device="cpu").manual_seed(11)
    src = torch.randn(64 * 80, generator=g).to(DEV)
    idx = torch.randint(0, 64, (64,), generator=g, dtype=torch.int32).to(DEV)
    sig = {"src": "*fp32", "idx": "*i32", "dst": "*fp32", "flag": "i32", "pitch": "i32", "BLOCK": "constexpr"}
    ttir = compile_ttir(X.pointer_blocks_by_branch, sig, {"BLOCK": 64})
    for flag in (0, 1, 7):
        dst = torch.zeros(3 * 64, device=DEV)
        k = X.pointer_blocks_by_branch[(3,)](src, idx, dst, flag, 80, BLOCK=64)
        torch.cuda.synchronize()
        assert k.function.family == "tile_program"
        offs = np.arange(64)
        p = idx.cpu().numpy() * 80 + offs if flag == 0 else offs * 2
        want = np.concatenate([src.cpu().numpy()[np.where(offs % 2 == 0, p, offs + pid)] for pid in range(3)])
        assert np.array_equal(dst.cpu().numpy(), want)
        mem = {0: src.cpu().numpy().copy(), 1: idx.cpu().numpy().copy(), 2: np.zeros(3 * 64, np.float32)}
        ttir_lanes.Interpreter(ttir).run((3,), [None, None, None, flag, 80], mem)
        assert np.array_equal(mem[2], want)


def test_tile_program_same_width_pointer_cast():
    """`ptr.to(tl.pointer_type(tl.int32))` on a float buffer (tt.bitcast of a scalar pointer to a type of the same width):
    the same addresses, read and written as bit patterns.  Exact against numpy views and against the lane interpreter."""
    import extra_kernels as X
    from test_planner import compile_ttir
    from oracle import ttir_lanes
    n = 1000
    x = torch.randn(n, generator=torch.Generator(device="cpu").manual_seed(2)).to(DEV)
    bits = torch.zeros(n, dtype=torch.int32, device=DEV)
    y = torch.zeros(n, device=DEV)
    k = X.float_bits_through_pointer_cast[(4,)](x, bits, y, n, BLOCK=256)
    torch.cuda.synchronize()
    assert k.function.family == "tile_program" and "tt.bitcast" in k.asm["ttir"]
    assert torch.equal(bits, x.view(torch.int32)) and torch.equal(y, x.abs())
    sig = {"x_ptr": "*fp32", "bits_ptr": "*i32", "y_ptr": "*fp32", "n": "i32", "BLOCK": "constexpr"}
    mem = {0: x.cpu().numpy().copy(), 1: np.zeros(n, np.int32), 2: np.zeros(n, np.float32)}
    ttir_lanes.Interpreter(compile_ttir(X.float_bits_through_pointer_cast, sig, {"BLOCK": 256})).run((4,), [None, None, None, n], mem)
    assert np.array_equal(mem[1], bits.cpu().numpy()) and np.array_equal(mem[2], y.cpu().numpy())


def test_tile_program_in_place_swap():
    import extra_kernels as X
    torch.manual_seed(0)
    x, y = torch.rand(10240, device=DEV), torch.rand(10240, device=DEV)
    x0, y0 = x.clone(), y.clone()
    X.swap_blocks[(10,)](x, y, BLOCK=1024)                    # test_swap.py: both loads before either store
    torch.cuda.synchronize()
    assert torch.equal(x, y0) and torch.equal(y, x0)


def test_tile_program_splat_scalar_walk_and_2d_tiles():
    import extra_kernels as X
    out = torch.empty(256, 512, device=DEV)
    X.fill_rows[(128,)](123.456, out, out.stride(0), out.stride(1), BC=512)        # test_splat.py
    torch.cuda.synchronize()
    assert torch.equal(out.cpu(), torch.full((256, 512), 123.456))
    inp, o = torch.arange(0, 11, dtype=torch.float32, device=DEV), torch.zeros(11, device=DEV)
    X.scalar_walk[(1,)](inp, o)                                                    # test_addptr.py
    torch.cuda.synchronize()
    assert torch.equal(inp, o)
    for rows, cols, BR, BC in [(512, 256, 4, 2), (100, 70, 32, 64), (33, 1000, 16, 256)]:
        x = torch.randn(rows, cols, device=DEV)
        y = torch.full((rows, cols), -1.0, device=DEV)
        k = X.affine_tile_2d[(triton.cdiv(rows, BR), triton.cdiv(cols, BC))](x, y, rows, cols, x.stride(0), 1, BR=BR, BC=BC)
        torch.cuda.synchronize()
        assert k.function.family == "tile_program"
        assert torch.equal(y, 2 * x + 1)
    # different row pitches for input and output are different strides: transposed read
    x = torch.randn(64, 48, device=DEV)
    xt = x.t().contiguous().t()                                  # same values, column-major storage
    y = torch.zeros(64, 48, device=DEV)
    X.copy_tile_strided[(2, 3)](xt, y, 64, 48, xt.stride(0), xt.stride(1), y.stride(0), y.stride(1), BR=32, BC=16)
    torch.cuda.synchronize()
    assert torch.equal(y, x)


def test_tile_program_against_lane_interpreter():
    # random wraparound windows, checked element by element against the lane-level oracle
    import extra_kernels as X
    from test_planner import compile_ttir
    from oracle import ttir_lanes
    sig = {"a_ptr": "*fp32", "c_ptr": "*fp32", "M": "i32", "N": "i32", "s_am": "i32", "s_an": "i32", "s_cm": "i32", "s_cn": "i32",
           "BK": "constexpr"}
    ttir = compile_ttir(X.wrap_cols_masked_loop, sig, {"BK": 4})
    rng = np.random.default_rng(3)
    for M, N in [(12, 8), (10, 7), (16, 9)]:
        a = rng.standard_normal((M, N)).astype(np.float32)
        ref = np.full((M, 8), 88888.0, np.float32)
        ttir_lanes.Interpreter(ttir).run((1,), [None, None, M, N, N, 1, 8, 1], {0: a.reshape(-1).copy(), 1: ref.reshape(-1)})
        ad, od = torch.from_numpy(a).to(DEV), torch.full((M, 8), 88888.0, device=DEV)
        X.wrap_cols_masked_loop[(1,)](ad, od, M, N, N, 1, 8, 1, BK=4)
        torch.cuda.synchronize()
        assert np.array_equal(od.cpu().numpy(), ref.reshape(M, 8))


# ------------------------------------------------------------- error paths
def test_errors_surface_as_python_exceptions(K):
    import extra_kernels as X
    x = torch.zeros(1024, device=DEV)
    with pytest.raises(TypeError, match="device"):
        K.vec_add[(1,)](torch.zeros(1024), x, x, 1024, BLOCK=1024)     # host tensor
    with pytest.raises(NotImplementedError):
        X.atomic_accumulate[(4,)](x, x, 1024, BLOCK=256)               # no structured lowering: refused, no fallback
    with pytest.raises(NotImplementedError, match="bytes of LDS"):
        big = torch.zeros(128 * 128, device=DEV)
        X.small_dot[(1,)](big, big, big, B=128)                        # a large product outside the tiled matmul shapes


def test_gemm_with_a_grid_that_is_not_the_tile_grid_runs_program_by_program(K):
    # three programs for four output tiles: not a dense product, so the matrix-product kernels decline at launch and
    # the generic family runs the three programs, as the reference's serial loop would; the fourth tile stays untouched
    torch.manual_seed(4)
    a = (torch.randn(256, 256) * 0.1).bfloat16().to(DEV)
    b = (torch.randn(256, 256) * 0.1).bfloat16().to(DEV)
    c = torch.full((256, 256), 5.0, dtype=torch.bfloat16, device=DEV)
    k = K.matmul_tiles[(3,)](a, b, c, 256, 256, 256, 256, 1, 256, 1, 256, 1, BM=128, BN=128, BK=64, GROUP_M=8)
    torch.cuda.synchronize()
    assert k.function.family == "gemm" and k.function.last_kernel == "tile_program (hipRTC)"
    ref = a.float() @ b.float()
    for tm, tn in [(0, 0), (1, 0), (0, 1)]:      # programs 0, 1, 2 in the kernel's grouped order
        blk = (slice(128 * tm, 128 * tm + 128), slice(128 * tn, 128 * tn + 128))
        assert relfro(c[blk].float(), ref[blk]) <= 1e-2
    assert torch.equal(c[128:, 128:].cpu(), torch.full((128, 128), 5.0, dtype=torch.bfloat16))


def test_plan_handle_is_loaded_once(K):
    # the launcher must keep the native plan (and its binding cache) across launches
    x = torch.zeros(2048, device=DEV)
    k1 = K.vec_add[(2,)](x, x, x, 2048, BLOCK=1024)
    h1 = k1.function
    k2 = K.vec_add[(2,)](x, x, x, 2048, BLOCK=1024)
    assert k2 is k1 and k2.function is h1


# ------------------------------------------------------------- gathers and scatters (generic family)
def _gather_case(kernel):
    # python/examples/test_gather_scatter.py:91-105: 128 int32 inputs 2..129, output preset to -1, one program
    src = torch.arange(2, 130, dtype=torch.int32, device=DEV)
    dst = torch.full((128,), -1, dtype=torch.int32, device=DEV)
    k = kernel[(1,)](src, dst)
    torch.cuda.synchronize()
    assert k.function.family == "tile_program"
    return dst.cpu().tolist()


def _runs(*pairs):
    out = []
    for value, times in pairs:
        out += [value] * times
    return out


def test_gather_scatter_reference_goldens():
    """Expected values are the literal tensors python/examples/test_gather_scatter.py asserts (written here as runs)."""
    import extra_kernels as X
    assert _gather_case(X.gather_div10) == _runs(*[(v, 10) for v in range(7, 13)], (13, 4), (14, 10), (15, 54))     # :108-117
    quarter = lambda fill: _runs(*[(v, 4) for v in range(2, 10)], (fill, 32), *[(v, 4) for v in range(18, 26)], (fill, 32))
    assert _gather_case(X.gather_quarter_masked) == quarter(0)                                                      # :119-128
    assert _gather_case(X.gather_quarter_masked_other) == quarter(-1)                                               # :131-140
    assert _gather_case(X.gather_div12_masked_store) == _runs(*[(v, 12) for v in range(2, 7)], (7, 17), (-1, 51))   # :143-152
    assert _gather_case(X.gather_scatter_nested) == (                                                               # :155-164
        list(range(2, 13)) + [-1] * 4 + [17, 18, -1, 20, 21, -1, 23, 24, 25, -1, -1, 28] + [-1] * 5 + [0] * 11 + [-1] * 85)


def test_index_select_against_torch():
    # python/examples/test_index_select.py:67-81: rows picked through an index vector plus a modulo of the row number
    import extra_kernels as X
    torch.manual_seed(5)
    src = torch.randn(16, 16, device=DEV)
    rows = torch.tensor([1, 3, 5, 7], dtype=torch.int32, device=DEV)
    for period in (2, 3):
        dst = torch.empty(4, 16, device=DEV)
        k = X.select_rows[(1,)](src, dst, rows, rows.stride(0), src.stride(0), dst.stride(0), period, R=4, C=16)
        torch.cuda.synchronize()
        assert k.function.family == "tile_program"
        want = torch.index_select(src, 0, (rows + torch.arange(0, 4, device=DEV, dtype=torch.int32) % period).long())
        assert torch.equal(dst, want)


def test_gather_and_scatter_through_an_index_vector():
    import extra_kernels as X
    from oracle import ttir_lanes
    from test_planner import compile_ttir
    torch.manual_seed(6)
    n = 3000
    src = torch.randn(n, device=DEV)
    perm = torch.randperm(n, device=DEV).int()
    # scatter: dst[perm[i]] = src[i]
    dst = torch.zeros(n, device=DEV)
    k = X.scatter_by_index[(triton.cdiv(n, 256),)](src, perm, dst, n, BLOCK=256)
    torch.cuda.synchronize()
    assert k.function.family == "tile_program"
    want = torch.zeros(n, device=DEV)
    want[perm.long()] = src
    assert torch.equal(dst, want)
    # ... and the lane-level oracle agrees
    ttir = compile_ttir(X.scatter_by_index, {"src": "*fp32", "idx": "*i32", "dst": "*fp32", "n": "i32", "BLOCK": "constexpr"}, {"BLOCK": 256})
    ref = np.zeros(n, dtype=np.float32)
    ttir_lanes.Interpreter(ttir).run((triton.cdiv(n, 256),), [None, None, None, n], {0: src.cpu().numpy(), 1: perm.cpu().numpy(), 2: ref})
    assert np.array_equal(ref, dst.cpu().numpy())
    # gather: dst[i] = src[idx[i]], whole blocks
    idx = torch.randint(0, n, (1024,), device=DEV, dtype=torch.int32)
    out = torch.zeros(1024, device=DEV)
    for b in range(4):
        X.gather_rows[(1,)](src, idx[b * 256:], out[b * 256:], BLOCK=256)
    torch.cuda.synchronize()
    assert torch.equal(out, src[idx.long()])


# ------------------------------------------------------------- reductions and scans (generic family)
def test_tile_program_axis_reductions():
    """2-D reductions along either axis (ConversionPatterns.hpp:1343-1364), checked against torch; float sums to 1e-5
    relative (the order of a sum differs from the reference's sequential one when a line is cut into pieces), max / min
    exactly."""
    import extra_kernels as X
    torch.manual_seed(7)
    rows, cols = 37, 100
    x = torch.randn(rows, cols, device=DEV)
    for kind, want in [(0, x.sum(1)), (1, x.max(1).values), (2, x.min(1).values)]:
        out = torch.full((rows,), 7.0, device=DEV)
        k = X.reduce_rows_2d[(triton.cdiv(rows, 8),)](x, out, rows, cols, x.stride(0), BR=8, BC=128, KIND=kind)
        torch.cuda.synchronize()
        assert k.function.family == "tile_program"
        if kind == 0:
            torch.testing.assert_close(out, want, rtol=1e-5, atol=1e-5)
        else:
            assert torch.equal(out, want)
    out = torch.zeros(cols, device=DEV)
    X.reduce_cols_2d[(triton.cdiv(cols, 64),)](x[:16], out, 16, cols, x.stride(0), BR=16, BC=64)
    torch.cuda.synchronize()
    torch.testing.assert_close(out, x[:16].sum(0), rtol=1e-5, atol=1e-5)


def test_tile_program_reduction_feeding_the_block():
    import extra_kernels as X
    from oracle import ttir_lanes
    from test_planner import compile_ttir
    torch.manual_seed(8)
    x = torch.randn(9, 1000, device=DEV)
    y = torch.zeros_like(x)
    k = X.centre_rows[(9,)](x, y, 1000, x.stride(0), BC=1024)
    torch.cuda.synchronize()
    assert k.function.family == "tile_program"
    torch.testing.assert_close(y, x - x.mean(1, keepdim=True), rtol=1e-5, atol=1e-5)
    ttir = compile_ttir(X.centre_rows, {"x_ptr": "*fp32", "y_ptr": "*fp32", "n_cols": "i32", "pitch": "i32", "BC": "constexpr"}, {"BC": 1024})
    ref = np.zeros(9 * 1000, dtype=np.float32)
    ttir_lanes.Interpreter(ttir).run((9,), [None, None, 1000, 1000], {0: x.cpu().numpy().reshape(-1).copy(), 1: ref})
    assert np.abs(ref.reshape(9, 1000) - y.cpu().numpy()).max() <= 1e-5


def test_tile_program_integer_reductions_are_exact():
    import extra_kernels as X
    g = torch.Generator().manual_seed(9)
    x = torch.randint(-2**31, 2**31 - 1, (300,), generator=g, dtype=torch.int64).to(torch.int32)
    out = torch.zeros(4, dtype=torch.int32, device=DEV)
    X.int_reductions[(1,)](x.to(DEV), out, 300, BLOCK=512)
    torch.cuda.synchronize()
    v = np.concatenate([x.numpy(), np.zeros(212, np.int32)])
    assert out.cpu().tolist() == [int(v.sum(dtype=np.int32)), int(v.max()), int(v.min()), int(np.bitwise_xor.reduce(v))]


def test_tile_program_argmax_argmin_first_index_wins():
    # ConversionPatterns.hpp:1443-1769: the two-operand reduction with the tie-breaking combiner
    import extra_kernels as X
    g = torch.Generator().manual_seed(10)
    x = torch.randint(0, 6, (33, 200), generator=g).float()          # many ties
    hi = torch.zeros(33, dtype=torch.int32, device=DEV)
    lo = torch.zeros(33, dtype=torch.int32, device=DEV)
    xd = x.to(DEV)
    k = X.arg_extremes_rows[(33,)](xd, hi, lo, 200, xd.stride(0), BC=256)
    torch.cuda.synchronize()
    assert k.function.family == "tile_program"
    assert hi.cpu().tolist() == x.numpy().argmax(1).tolist()
    assert lo.cpu().tolist() == x.numpy().argmin(1).tolist()


def test_tile_program_cumsum():
    import extra_kernels as X
    torch.manual_seed(11)
    n = 5000
    x = torch.randn(n, device=DEV)
    y = torch.zeros(n, device=DEV)
    k = X.running_sum[(triton.cdiv(n, 1024),)](x, y, n, BLOCK=1024)
    torch.cuda.synchronize()
    assert k.function.family == "tile_program"
    want = torch.cat([c.double().cumsum(0) for c in x.split(1024)]).float()
    torch.testing.assert_close(y, want, rtol=1e-5, atol=1e-4)
    xi = torch.arange(1, 1025, dtype=torch.float32, device=DEV)        # exact in f32: any order gives the same sums
    yi = torch.zeros(1024, device=DEV)
    X.running_sum[(1,)](xi, yi, 1024, BLOCK=1024)
    torch.cuda.synchronize()
    assert torch.equal(yi, xi.cumsum(0))
    for axis, (BR, BC) in [(1, (4, 8)), (0, (64, 32)), (1, (16, 256))]:
        x2 = torch.randn(BR, BC, device=DEV)
        y2 = torch.zeros_like(x2)
        X.running_sum_2d[(1,)](x2, y2, x2.stride(0), BR=BR, BC=BC, AXIS=axis)
        torch.cuda.synchronize()
        torch.testing.assert_close(y2, x2.double().cumsum(axis).float(), rtol=1e-5, atol=1e-5)


def test_block_sum_runs_in_the_generic_family():
    import extra_kernels as X
    x = torch.arange(0, 1000, dtype=torch.float32, device=DEV)
    out = torch.zeros(4, device=DEV)
    k = X.block_sum[(4,)](x, out, 1000, BLOCK=256)
    torch.cuda.synchronize()
    assert k.function.family == "tile_program"
    assert out.cpu().tolist() == [float(sum(range(b * 256, min(1000, (b + 1) * 256)))) for b in range(4)]


# ------------------------------------------------------------- the reference's functional tests, case by case
def _reference_case_ids():
    import reference_cases
    return [c["name"] for c in reference_cases.cases()]


@pytest.mark.parametrize("name", _reference_case_ids())
def test_reference_functional_case(name):
    """tests/reference_cases.py: inputs and expectations of python/examples/*.py; the same cases pin the lane oracle."""
    import extra_kernels as X
    import reference_cases
    case = next(c for c in reference_cases.cases() if c["name"] == name)
    args = case["args"]()
    dev = [torch.from_numpy(a).to(DEV) if isinstance(a, np.ndarray) else a for a in args]
    k = getattr(X, case["kernel"])[case["grid"]](*dev, **case["consts"])
    torch.cuda.synchronize()
    assert k.function.family == "tile_program"
    case["check"]([d.cpu().numpy() for d in dev if isinstance(d, torch.Tensor)])


def test_tile_program_blocks_past_the_register_budget():
    """Reductions of blocks too large to stage (one thread per line, in index order), in-place blocks of more than 16384
    elements (still two phases: every load before any store), a tile product with 32768 outputs."""
    import core_kernels
    import extra_kernels as X
    rng = np.random.default_rng(21)
    x = rng.integers(-8, 9, (512, 256)).astype(np.float32)           # small integers: every order of summation is exact
    for axis in (0, 1):
        for kind, want in ((0, x.sum(axis)), (1, x.max(axis))):
            out = torch.zeros(x.shape[1 - axis], device=DEV)
            k = X.reduce_big_block_2d[(1,)](torch.from_numpy(x).to(DEV), out, R=512, C=256, AXIS=axis, KIND=kind)
            torch.cuda.synchronize()
            assert k.function.family == "tile_program"
            assert np.array_equal(out.cpu().numpy(), want), (axis, kind)
    xi = rng.integers(-1000, 1000, 50000).astype(np.int32)
    out = torch.zeros(3, dtype=torch.int32, device=DEV)
    X.block_total_and_extremes[(1,)](torch.from_numpy(xi).to(DEV), out, 50000, BLOCK=65536)
    torch.cuda.synchronize()
    assert out.cpu().tolist() == [int(xi.sum()), max(int(xi.max()), 0), min(int(xi.min()), 0)]
    x3 = rng.integers(-8, 9, (8, 16, 32)).astype(np.float32)
    for axis in (0, 1, 2):
        for kind, want in ((0, x3.sum(axis)), (1, x3.max(axis))):
            out = torch.zeros(want.size, device=DEV)
            X.reduce_3d[(1,)](torch.from_numpy(x3).to(DEV), out, A=8, B=16, C=32, AXIS=axis, KIND=kind)
            torch.cuda.synchronize()
            assert np.array_equal(out.cpu().numpy().reshape(want.shape), want), (axis, kind)
    for R, C in ((64, 128), (256, 128), (512, 128)):                 # 8192 (registers), 32768 and 65536 (two phases all the same)
        v = rng.standard_normal(R * C + 1).astype(np.float32)
        d = torch.from_numpy(v).to(DEV)
        X.shift_left_in_place[(1,)](d, R=R, C=C)
        torch.cuda.synchronize()
        assert np.array_equal(d.cpu().numpy(), np.concatenate([v[1:], v[-1:]])), (R, C)
    a = rng.integers(-3, 4, (128, 64)).astype(np.float16)
    b = rng.integers(-3, 4, (64, 256)).astype(np.float16)
    c = torch.zeros(128 * 256, device=DEV)
    core_kernels.dot_in_half_precision[(1,)](torch.from_numpy(a).to(DEV), torch.from_numpy(b).to(DEV), c, M=128, N=256, K=64, ACC_IN=0)
    torch.cuda.synchronize()
    assert np.array_equal(c.cpu().numpy().reshape(128, 256), a.astype(np.float32) @ b.astype(np.float32))


def _core_case_ids():
    import core_cases
    return [c["name"] for c in core_cases.cases()]


@pytest.mark.parametrize("name", _core_case_ids())
def test_core_language_case(name):
    """tests/core_cases.py: one kernel per language feature the reference enables from Triton's core tests
    (python/examples/conftest.py:52-92), closed-form expectations; the same cases pin the lane oracle."""
    import core_cases
    import core_kernels
    case = next(c for c in core_cases.cases() if c["name"] == name)
    dev = []
    for a, ty in zip(case["args"](), [t for t in case["sig"].values() if t != "constexpr"]):
        if isinstance(a, np.ndarray):
            a = torch.from_numpy(a).to(DEV)
            a = a.view(torch.bfloat16) if ty == "*bf16" else a
        dev.append(a)
    getattr(core_kernels, case["kernel"])[case["grid"]](*dev, **case["consts"])
    torch.cuda.synchronize()
    case["check"]([(d.view(torch.uint16) if d.dtype == torch.bfloat16 else d).cpu().numpy() for d in dev if isinstance(d, torch.Tensor)])


def test_tile_program_nested_pointer_walk_against_lane_interpreter():
    # python/examples/test_nested_loops.py is a template without expectations: the oracle provides them
    import extra_kernels as X
    from oracle import ttir_lanes
    from test_planner import compile_ttir
    src = torch.arange(0, 2 * 64, dtype=torch.float32, device=DEV)
    dst = torch.full((2 * 64,), -1.0, device=DEV)
    k = X.nested_walk[(1,)](src, dst, 64, 1)
    torch.cuda.synchronize()
    assert k.function.family == "tile_program"
    ttir = compile_ttir(X.nested_walk, {"src": "*fp32", "dst": "*fp32", "pitch_m": "i32", "pitch_n": "i32"}, {})
    ref = np.full(128, -1.0, dtype=np.float32)
    ttir_lanes.Interpreter(ttir).run((1,), [None, None, 64, 1], {0: src.cpu().numpy(), 1: ref})
    assert np.array_equal(ref, dst.cpu().numpy()) and (ref != -1).sum() > 40


# ------------------------------------------------------------- small matrix products (generic family)
def test_tile_program_small_dot_and_loop_peeled_matmul():
    """tt.dot outside the tiled matmul kernels: a one-shot 32x32 product, and the structure of python/examples/test_mm.py
    (whole K blocks unmasked, a masked remainder block, wrapped operand rows / columns), against torch.matmul; products
    are folded in k order in fp32, so the tolerance only covers torch's own summation order."""
    import extra_kernels as X
    torch.manual_seed(12)
    a = torch.randn(32, 32, device=DEV)
    b = torch.randn(32, 32, device=DEV)
    c = torch.zeros(32, 32, device=DEV)
    k = X.small_dot[(1,)](a, b, c, B=32)
    torch.cuda.synchronize()
    assert k.function.family == "tile_program"
    torch.testing.assert_close(c, (a.double() @ b.double()).float(), rtol=1e-5, atol=1e-5)
    for dtype, tol in [(torch.float32, 1e-5), (torch.float16, 2e-3), (torch.bfloat16, 2e-2)]:
        for M, N, K in [(37, 53, 70), (64, 32, 32), (5, 100, 33)]:
            a = torch.randn(M, K, device=DEV).to(dtype)
            b = torch.randn(K, N, device=DEV).to(dtype)
            c = torch.full((M, N), 7.0, device=DEV, dtype=dtype)
            grid = (triton.cdiv(M, 32) * triton.cdiv(N, 32),)
            k = X.mm_peeled[grid](a, b, c, M, N, K, a.stride(0), a.stride(1), b.stride(0), b.stride(1), c.stride(0), c.stride(1), BM=32, BN=32, BK=32)
            torch.cuda.synchronize()
            assert k.function.family == "tile_program"
            want = a.double() @ b.double()
            err = (c.double() - want).norm() / want.norm()
            assert err <= tol, (dtype, M, N, K, float(err))


def test_tile_program_integer_bit_and_conversion_ops_are_exact():
    """The op classes of test_core's whitelisted test_bin_op / test_bitwise_op / test_shift_op / test_umulhi / test_abs /
    test_clamp / test_floordiv / test_precise_math (python/examples/conftest.py:48-91), bit for bit against numpy."""
    import extra_kernels as X
    import op_zoo
    n = 1000
    x, y = op_zoo.int_inputs(n)
    out = torch.zeros(12 * n, dtype=torch.int32, device=DEV)
    k = X.int_ops[(4,)](torch.from_numpy(x).to(DEV), torch.from_numpy(y).to(DEV), out, n, BLOCK=256)
    torch.cuda.synchronize()
    assert k.function.family == "tile_program"
    got, want = out.cpu().numpy().reshape(12, n), op_zoo.int_expected(x, y)
    for plane in range(12):
        assert np.array_equal(got[plane], want[plane]), plane
    xf, yf = op_zoo.float_inputs(n)
    outf = torch.zeros(8 * n, device=DEV)
    X.float_ops[(4,)](torch.from_numpy(xf).to(DEV), torch.from_numpy(yf).to(DEV), outf, n, -50.0, 75.5, BLOCK=256)
    torch.cuda.synchronize()
    gotf, wantf = outf.cpu().numpy().reshape(8, n), op_zoo.float_expected(xf, yf, -50.0, 75.5)
    for plane in range(8):
        assert np.array_equal(gotf[plane], wantf[plane]), plane


def test_tile_program_transpose_and_reshape():
    import extra_kernels as X
    torch.manual_seed(13)
    for R, C in [(16, 32), (32, 32)]:                     # the square case: same block shape on both sides of the transpose
        x = torch.randn(R, C, device=DEV)
        y = torch.zeros(C, R, device=DEV)
        k = X.transpose_tile[(1,)](x, y, R=R, C=C)
        torch.cuda.synchronize()
        assert k.function.family == "tile_program"
        assert torch.equal(y, x.t() + torch.arange(R, device=DEV, dtype=torch.float32)[None, :])
    x = torch.randn(512, device=DEV)
    y = torch.zeros(8 + 512, device=DEV)
    X.fold_and_sum[(1,)](x, y, R=8, C=64)
    torch.cuda.synchronize()
    torch.testing.assert_close(y[:8], x.reshape(8, 64).double().sum(1).float(), rtol=1e-5, atol=1e-5)
    assert torch.equal(y[8:], x * 2)


def test_tile_program_extern_functions():
    # libdevice-style functions by symbol name run on the device math library: a few ulp from the float64 values
    import extra_kernels as X
    torch.manual_seed(14)
    n = 500
    x = torch.randn(n, device=DEV) * 3
    y = torch.randn(n, device=DEV)
    out = torch.zeros(6 * n, device=DEV)
    k = X.extern_math[(2,)](x, y, out, n, BLOCK=256)
    torch.cuda.synchronize()
    assert k.function.family == "tile_program"
    xd, yd = x.double().cpu(), y.double().cpu()
    want = torch.stack([xd.abs() ** yd, torch.atan2(xd, yd), torch.log1p(xd.abs()), torch.tanh(yd), torch.trunc(xd), torch.asin(yd.clamp(-1, 1))])
    got = out.cpu().double().reshape(6, n)
    err = (got - want).abs().amax(1) / want.abs().amax(1)
    assert (err <= 1e-6).all(), err


def test_tile_program_large_blocks():
    """Blocks of up to 16384 elements are held in registers (64 per thread): a one-dimensional block of 8192 reduced and
    rescaled, and a 64 x 128 block reduced along its rows through the LDS-staged path."""
    import extra_kernels as X
    torch.manual_seed(15)
    x = torch.randn(3, 8000, device=DEV)
    y = torch.zeros_like(x)
    k = X.centre_rows[(3,)](x, y, 8000, x.stride(0), BC=8192)
    torch.cuda.synchronize()
    assert k.function.family == "tile_program"
    torch.testing.assert_close(y, x - x.mean(1, keepdim=True), rtol=1e-5, atol=2e-5)
    x = torch.randn(100, 100, device=DEV)
    out = torch.zeros(100, device=DEV)
    X.reduce_rows_2d[(2,)](x, out, 100, 100, x.stride(0), BR=64, BC=128, KIND=0)
    torch.cuda.synchronize()
    torch.testing.assert_close(out, x.sum(1), rtol=1e-5, atol=2e-5)


# ------------------------------------------------------------- tutorial-style kernels on the generic family
def test_tile_program_seeded_dropout_is_exact():
    import extra_kernels as X
    import op_zoo
    n = 100_000
    x = torch.randn(n, device=DEV)
    out = torch.zeros(n, device=DEV)
    k = X.seeded_dropout[(triton.cdiv(n, 1024),)](x, out, n, 0.3, 1234, BLOCK=1024)
    torch.cuda.synchronize()
    assert k.function.family == "tile_program"
    u = op_zoo.philox_uniform(1234, np.arange(n))
    xs = x.cpu().numpy()
    want = np.where(u > np.float32(0.3), xs / (np.float32(1) - np.float32(0.3)), np.float32(0))
    assert np.array_equal(out.cpu().numpy(), want)


def test_tile_program_norms_and_reductions_of_the_tutorials():
    import extra_kernels as X
    torch.manual_seed(16)
    # RMSNorm, fp16 rows of 4000 in blocks of 4096
    x = torch.randn(7, 4000, device=DEV).half()
    w = (1 + 0.1 * torch.randn(4000, device=DEV)).half()
    y = torch.zeros_like(x)
    k = X.rms_norm_rows[(7,)](x, w, y, x.stride(0), 4000, 1e-6, BLOCK=4096)
    torch.cuda.synchronize()
    assert k.function.family == "tile_program"
    xf = x.float()
    want = xf / torch.sqrt((xf * xf).mean(1, keepdim=True) + 1e-6) * w.float()
    assert (y.float() - want).abs().max() <= 1e-2
    # column sums with a [32, 128] accumulator carried down the rows (the dw / db kernel of the LayerNorm tutorial)
    a = torch.randn(1000, 300, device=DEV)
    out = torch.zeros(300, device=DEV)
    X.column_sums_looped[(triton.cdiv(300, 128),)](a, out, 1000, 300, a.stride(0), BR=32, BC=128)
    torch.cuda.synchronize()
    torch.testing.assert_close(out, a.double().sum(0).float(), rtol=1e-5, atol=1e-4)
    # log-sum-exp of rows
    b = torch.randn(50, 2000, device=DEV) * 5
    lse = torch.zeros(50, device=DEV)
    X.log_sum_exp_rows[(50,)](b, lse, b.stride(0), 2000, BLOCK=2048)
    torch.cuda.synchronize()
    torch.testing.assert_close(lse, torch.logsumexp(b.double(), 1).float(), rtol=1e-6, atol=1e-5)


@pytest.mark.parametrize("dtype", ["float16", "bfloat16"])
@pytest.mark.parametrize("n_cols,block,pitch,lead", [
    (8192, 8192, 8192, 0),     # whole rows, every group moves in one access
    (5000, 8192, 5000, 0),     # rows end on a group boundary; the groups behind are invalid as a whole
    (4001, 4096, 4008, 0),     # rows end inside a group
    (4001, 4096, 4001, 0),     # odd row pitch: every other row starts off a 16-byte boundary
    (4096, 4096, 4096, 3),     # the tensors themselves start off a 16-byte boundary
    (2048, 2048, 2056, 8),
])
def test_tile_program_wide_16_bit_rows(dtype, n_cols, block, pitch, lead):
    """Blocks of 16-bit elements with whole groups of 2048 along the contiguous dimension give every thread eight
    neighbouring elements and move them in 16-byte accesses where a group is aligned, element by element where it is not:
    RMSNorm and the input gradient of LayerNorm on aligned, ragged and misaligned rows against float64 closed forms."""
    torch.manual_seed(n_cols + lead)
    dt = getattr(torch, dtype)
    rows = 9
    def rows_view(fill):
        buf = torch.full((lead + rows * pitch + 16,), fill, device=DEV, dtype=dt)
        return buf, buf[lead:lead + rows * pitch].view(rows, pitch)[:, :n_cols]
    xb, x = rows_view(7.0)
    x.copy_(torch.randn(rows, n_cols, device=DEV))
    wb = torch.zeros(lead + n_cols, device=DEV, dtype=dt)
    w = wb[lead:]
    w.copy_(1 + 0.1 * torch.randn(n_cols, device=DEV))
    yb, y = rows_view(5.0)
    k = K_mod().rms_norm_rows[(rows,)](x, w, y, pitch, n_cols, 1e-6, BLOCK=block)
    torch.cuda.synchronize()
    assert k.function.family == "tile_program"
    xd = x.double()
    want = xd / torch.sqrt((xd * xd).mean(1, keepdim=True) + 1e-6) * w.double()
    tol = 2e-2 if dtype == "bfloat16" else 4e-3
    assert (y.double() - want).abs().max() <= tol * max(1.0, want.abs().max().item())
    keep = torch.ones_like(yb, dtype=torch.bool)
    keep[lead:lead + rows * pitch].view(rows, pitch)[:, :n_cols] = False
    assert (yb[keep] == 5.0).all()                              # nothing written outside the rows
    # the gradient: three 16-bit row tensors, two scalars per row, two reductions
    dyb, dy = rows_view(3.0)
    dy.copy_(torch.randn(rows, n_cols, device=DEV))
    mean, rstd = torch.randn(rows, device=DEV) * 0.1, 0.5 + torch.rand(rows, device=DEV)
    dxb, dx = rows_view(5.0)
    K_mod().layer_norm_dx_rows[(rows,)](dx, dy, x, w, mean, rstd, pitch, n_cols, BLOCK=block)
    torch.cuda.synchronize()
    xhat = (xd - mean.double()[:, None]) * rstd.double()[:, None]
    wdy = w.double() * dy.double()
    want = (wdy - (xhat * (xhat * wdy).mean(1, keepdim=True) + wdy.mean(1, keepdim=True))) * rstd.double()[:, None]
    assert (dx.double() - want).abs().max() <= tol * max(1.0, want.abs().max().item())
    assert (dxb[keep] == 5.0).all()


def test_tile_program_wide_blocks_of_rows_loops_and_mixed_widths():
    """The wide element order next to what shares a program with it: tiles of rows with a row reduction and a vector of
    another shape, a carried accumulator in a loop, 4-byte stores next to 16-bit loads."""
    import extra_kernels as X
    torch.manual_seed(5)
    for dt in (torch.float16, torch.bfloat16):
        n_rows, n_cols, pitch = 11, 4100, 4104
        xb = torch.randn(n_rows, pitch, device=DEV).to(dt)
        x = xb[:, :n_cols]
        s = torch.randn(n_cols, device=DEV)
        yb = torch.full_like(xb, 5.0)
        sums = torch.zeros(3, n_rows, device=DEV)
        k = X.scale_tile_and_row_sums[(triton.cdiv(n_rows, 4), triton.cdiv(n_cols, 2048))](x, s, yb, sums, n_rows, n_cols, pitch, BR=4, BC=2048)
        torch.cuda.synchronize()
        assert k.function.family == "tile_program"
        want = (x.double() * s.double()).to(dt)
        assert (yb[:, :n_cols].double() - want.double()).abs().max() <= (0.07 if dt == torch.bfloat16 else 0.01)
        assert (yb[:, n_cols:] == 5.0).all()
        for j in range(3):
            torch.testing.assert_close(sums[j].double(), x[:, j * 2048:(j + 1) * 2048].double().sum(1), rtol=1e-5, atol=1e-4)
        # a carried accumulator
        n_rows, n_cols = 6, 4096 + 24
        x = torch.randn(n_rows, n_cols, device=DEV).to(dt)
        y = torch.zeros_like(x)
        X.running_mean_of_rows[(triton.cdiv(n_cols, 2048),)](x, y, n_rows, n_cols, n_cols, BLOCK=2048)
        torch.cuda.synchronize()
        want = x.double().cumsum(0) / torch.arange(1, n_rows + 1, device=DEV).double()[:, None]
        assert (y.double() - want).abs().max() <= (0.03 if dt == torch.bfloat16 else 4e-3)
        # 4-byte results of 16-bit loads, off a 16-byte boundary as well
        for lead in (0, 2):
            n = 3 * 2048 + 77
            xs = torch.randn(lead + n, device=DEV).to(dt)[lead:]
            yf = torch.full((lead + n + 8,), 5.0, device=DEV)
            ki = torch.full((lead + n + 8,), 5, device=DEV, dtype=torch.int32)
            X.widen_and_count[(triton.cdiv(n, 2048),)](xs, yf[lead:], ki[lead:], n, BLOCK=2048)
            torch.cuda.synchronize()
            assert torch.equal(yf[lead:lead + n], xs.float() * 2) and (yf[lead + n:] == 5).all() and (yf[:lead] == 5).all()
            o = torch.arange(n, device=DEV, dtype=torch.int32)
            assert torch.equal(ki[lead:lead + n], torch.where(xs.float() > 0, o, -o)) and (ki[lead + n:] == 5).all()


def test_tile_program_persistent_programs_walk_the_whole_grid():
    """A program whose block of weights is the same for every program runs as a loop over programs in a launch of a few
    workgroups per CU: more programs than such a launch has workgroups, on one- and two-dimensional grids."""
    import extra_kernels as X
    torch.manual_seed(3)
    rows, n = 5000, 2048
    x = torch.randn(rows, n, device=DEV).half()
    w = (1 + 0.1 * torch.randn(n, device=DEV)).half()
    y = torch.zeros_like(x)
    k = K_mod().rms_norm_rows[(rows,)](x, w, y, n, n, 1e-6, BLOCK=2048)
    torch.cuda.synchronize()
    assert k.function.family == "tile_program"
    xd = x.double()
    want = xd / torch.sqrt((xd * xd).mean(1, keepdim=True) + 1e-6) * w.double()
    assert (y.double() - want).abs().max() <= 4e-3 * want.abs().max().item()
    batches, rows, n = 3, 700, 2040
    x = torch.randn(batches, rows, n, device=DEV).bfloat16()
    w = torch.randn(n, device=DEV).bfloat16()
    y = torch.zeros_like(x)
    X.scale_rows_on_a_2d_grid[(rows, batches)](x, w, y, rows, n, BLOCK=2048)
    torch.cuda.synchronize()
    shift = torch.arange(batches, device=DEV)[:, None, None] - torch.arange(rows, device=DEV)[None, :, None]
    want = (x.float() * w.float() + shift.float()).bfloat16()
    assert torch.equal(y, want)


def test_tile_program_wide_and_ordinary_element_order_agree(monkeypatch):
    """The same program planned with and without the wide element order (and with and without the program loop) writes
    the same bits: an elementwise program exactly, a program with a row reduction to within the reduction's rounding."""
    import extra_kernels as X
    from triton_shared_amd import _native as native
    from test_planner import compile_ttir
    torch.manual_seed(21)
    stream = torch.cuda.current_stream().cuda_stream
    batches, rows, n = 2, 37, 2040
    x = torch.randn(batches, rows, n, device=DEV).bfloat16()
    w = torch.randn(n, device=DEV).bfloat16()
    sig = {"x_ptr": "*bf16", "w_ptr": "*bf16", "y_ptr": "*bf16", "n_rows": "i32", "n_cols": "i32", "BLOCK": "constexpr"}
    ttir = compile_ttir(X.scale_rows_on_a_2d_grid, sig, {"BLOCK": 2048})
    sig2 = {"x_ptr": "*bf16", "w_ptr": "*bf16", "y_ptr": "*bf16", "pitch": "i32", "n_cols": "i32", "eps": "fp32", "BLOCK": "constexpr"}
    ttir2 = compile_ttir(K_mod().rms_norm_rows, sig2, {"BLOCK": 2048})
    outs, norms = [], []
    for wide, persistent in (("1", "1"), ("1", "0"), ("0", "0")):
        monkeypatch.setenv("TTS_TILE_WIDE", wide)
        monkeypatch.setenv("TTS_TILE_PERSISTENT", persistent)
        plan = native.PlanHandle(native.structured_to_plan(native.ttir_to_structured(ttir))[0])
        y = torch.zeros_like(x)
        plan.launch((rows, batches, 1), stream, [x.data_ptr(), w.data_ptr(), y.data_ptr(), rows, n])
        plan2 = native.PlanHandle(native.structured_to_plan(native.ttir_to_structured(ttir2))[0])
        z = torch.zeros(batches * rows, n, device=DEV, dtype=torch.bfloat16)
        plan2.launch((batches * rows, 1, 1), stream, [x.data_ptr(), w.data_ptr(), z.data_ptr(), n, n, 1e-6])
        torch.cuda.synchronize()
        outs.append(y)
        norms.append(z)
    assert torch.equal(outs[0], outs[2]) and torch.equal(outs[1], outs[2])
    for z in norms[:2]:
        assert (z.float() - norms[2].float()).abs().max() <= 2e-2 * norms[2].float().abs().max()


def test_tile_program_wide_rows_of_random_extent_and_alignment():
    """Seeded random row counts, row lengths, pitches and starting offsets through a wide, persistent elementwise program
    (16-bit rows scaled by a shared vector): bit-exact against torch, nothing written outside the rows."""
    import extra_kernels as X
    rng = torch.Generator(device="cpu").manual_seed(77)
    for trial in range(24):
        dt = (torch.float16, torch.bfloat16)[trial % 2]
        batches = int(torch.randint(1, 4, (1,), generator=rng))
        rows = int(torch.randint(1, 40, (1,), generator=rng))
        n = int(torch.randint(1, 2049, (1,), generator=rng))
        lead = int(torch.randint(0, 9, (1,), generator=rng))
        total = batches * rows * n
        xb = torch.randn(lead + total + 8, device=DEV).to(dt)
        wb = torch.randn(lead + n + 8, device=DEV).to(dt)
        yb = torch.full((lead + total + 8,), 5.0, device=DEV, dtype=dt)
        x, w, y = xb[lead:lead + total].view(batches, rows, n), wb[lead:lead + n], yb[lead:lead + total].view(batches, rows, n)
        X.scale_rows_on_a_2d_grid[(rows, batches)](x, w, y, rows, n, BLOCK=2048)
        torch.cuda.synchronize()
        shift = torch.arange(batches, device=DEV)[:, None, None] - torch.arange(rows, device=DEV)[None, :, None]
        want = (x.float() * w.float() + shift.float()).to(dt)
        assert torch.equal(y, want), (trial, batches, rows, n, lead)
        assert (yb[:lead] == 5.0).all() and (yb[lead + total:] == 5.0).all(), (trial, batches, rows, n, lead)


@pytest.mark.parametrize("n_cols,pitch,lead", [(4096, 4096, 0), (4000, 4000, 0), (4093, 4099, 0), (2048, 2048, 5)])
def test_tile_program_wide_rows_with_int8_neighbours(n_cols, pitch, lead):
    """Row-wise int8 quantisation and its inverse: 1-byte blocks next to 16-bit ones take the wide element order too
    (eight bytes per thread, one 8-byte access where a group is whole and aligned); exact against torch."""
    import extra_kernels as X
    torch.manual_seed(n_cols)
    rows = 7
    xb = torch.zeros(lead + rows * pitch, device=DEV, dtype=torch.float16)
    x = xb[lead:].view(rows, pitch)[:, :n_cols]
    x.copy_(torch.randn(rows, n_cols, device=DEV))
    qb = torch.full((lead + rows * pitch + 8,), 5, device=DEV, dtype=torch.int8)
    q = qb[lead:lead + rows * pitch].view(rows, pitch)[:, :n_cols]
    s = torch.zeros(rows, device=DEV)
    k = X.quantize_rows_int8[(rows,)](x, q, s, n_cols, pitch, BLOCK=4096)
    torch.cuda.synchronize()
    assert k.function.family == "tile_program"
    xf = x.float().cpu()                                              # (on the host: IEEE division, as the kernel's is)
    scale = xf.abs().amax(1) / torch.full((rows,), 127.0)
    assert torch.equal(s.cpu(), scale)
    t = xf / scale[:, None]
    want = torch.where(t >= 0, t + 0.5, t - 0.5).to(torch.int8)      # (the conversion truncates toward zero, as the kernel's does)
    assert torch.equal(q.cpu(), want)
    keep = torch.ones_like(qb, dtype=torch.bool)
    keep[lead:lead + rows * pitch].view(rows, pitch)[:, :n_cols] = False
    assert (qb[keep] == 5).all()
    yb = torch.full((lead + rows * pitch,), 3.0, device=DEV, dtype=torch.float16)
    y = yb[lead:].view(rows, pitch)[:, :n_cols]
    X.dequantize_rows_int8[(rows,)](q, s, y, n_cols, pitch, BLOCK=4096)
    torch.cuda.synchronize()
    assert torch.equal(y.cpu(), (want.float() * scale[:, None]).half())


def test_compiled_kernels_are_cached_on_disk(tmp_path, monkeypatch):
    """The code object of a run-time compiled kernel is written to the cache directory at the first launch and loaded
    from there by the next plan of the same source (the reference caches its compiled launchers the same way,
    backend/driver.py:274-282)."""
    import extra_kernels as X
    from triton_shared_amd import _native as native
    from test_planner import compile_ttir
    monkeypatch.setenv("TTS_RTC_CACHE", str(tmp_path))
    sig = {"x_ptr": "*fp32", "out_ptr": "*fp32", "n": "i32", "BLOCK": "constexpr"}
    plan_bytes, _ = native.structured_to_plan(native.ttir_to_structured(compile_ttir(X.block_sum, sig, {"BLOCK": 512})))
    x = torch.arange(0, 1024, dtype=torch.float32, device=DEV)
    stream = torch.cuda.current_stream().cuda_stream
    for attempt in range(2):
        out = torch.zeros(2, device=DEV)
        plan = native.PlanHandle(plan_bytes)                      # a fresh plan: compiles (or loads) at its first launch
        plan.launch((2, 1, 1), stream, [x.data_ptr(), out.data_ptr(), 1024])
        torch.cuda.synchronize()
        assert out.tolist() == [float(sum(range(512))), float(sum(range(512, 1024)))]
        files = sorted(p.name for p in tmp_path.iterdir())
        assert len(files) == 1 and files[0].endswith(".hsaco"), files
        if attempt == 0:
            stamp = (tmp_path / files[0]).stat().st_mtime_ns
        else:
            assert (tmp_path / files[0]).stat().st_mtime_ns == stamp   # loaded, not rewritten


def test_reference_matmul_test_in_fp32():
    """python/examples/test_matmul.py:137-157 as it stands: fp32 operands, 179 x 167 @ 167 x 321, blocks 32 x 64 x 16,
    GROUP_M 8, operand rows / columns wrapped, and the reference's own assertion (atol 1e-2, rtol 0).  fp32 products run
    on the fp32 matrix-core kernel of the matmul family."""
    torch.manual_seed(0)
    a = torch.randn(179, 167, device=DEV)
    b = torch.randn(167, 321, device=DEV)
    for kernel in (K_mod().matmul_wrapped, K_mod().matmul_tiles):
        c = torch.empty(179, 321, device=DEV)
        grid = (triton.cdiv(179, 32) * triton.cdiv(321, 64),)
        k = kernel[grid](a, b, c, 179, 321, 167, a.stride(0), a.stride(1), b.stride(0), b.stride(1), c.stride(0), c.stride(1),
                         BM=32, BN=64, BK=16, GROUP_M=8)
        torch.cuda.synchronize()
        assert k.function.family == "gemm" and k.function.last_kernel == "gemm_f32_kernel"
        torch.testing.assert_close(c, torch.matmul(a, b), atol=1e-2, rtol=0)
        assert ((c.double() - a.double() @ b.double()).norm() / (a.double() @ b.double()).norm()) < 1e-6


def K_mod():
    from triton_shared_amd.examples import kernels
    return kernels


def test_tile_program_join_split_cat():
    # TritonArithToLinalg/join.mlir, split.mlir and tl.cat: index shuffles of rank-1 blocks
    import extra_kernels as X
    a = torch.arange(0, 64, dtype=torch.float32, device=DEV)
    b = 100 + torch.arange(0, 64, dtype=torch.float32, device=DEV)
    out = torch.zeros(6 * 64, device=DEV)
    k = X.join_split_cat[(1,)](a, b, out, N=64)
    torch.cuda.synchronize()
    assert k.function.family == "tile_program"
    assert torch.equal(out, torch.cat([torch.stack([a, b], 1).reshape(-1), a + 1, b + 1, b, a]))


def test_tile_program_if_with_results():
    # an if / else on a loaded scalar that yields a block, and an integer scalar that later feeds float arithmetic
    import extra_kernels as X
    torch.manual_seed(17)
    x = torch.randn(128, device=DEV)
    flags = torch.tensor([3, -2, 0, 5], dtype=torch.int32, device=DEV)
    out = torch.zeros(4, 128, device=DEV)
    k = X.branch_with_results[(4,)](x, flags, out, N=128)
    torch.cuda.synchronize()
    assert k.function.family == "tile_program"
    want = torch.stack([(x * 2 + 1 + float(3 * f)) if f > 0 else (x - 1 - 1 + float(7 - f)) for f in flags.tolist()])
    assert torch.equal(out, want)


def test_tile_program_persistent_softmax():
    """The grid-stride softmax of the current tutorial on the generic family, with the reference's own shape and assertion
    (python/examples/test_softmax.py:60-65) and the 1e-5 max-abs bar against float64."""
    import extra_kernels as X
    torch.manual_seed(0)
    x = torch.randn(1823, 781, device=DEV)
    y = torch.empty_like(x)
    k = X.softmax_persistent[(256,)](y, x, x.stride(0), y.stride(0), 1823, 781, BLOCK=1024)
    torch.cuda.synchronize()
    assert k.function.family == "tile_program"
    assert torch.allclose(y, torch.softmax(x, 1))
    assert (y.double() - torch.softmax(x.double(), 1)).abs().max() <= 1e-5


def test_gemm_epilogue_in_the_grouped_tile_order(K):
    """The stock tutorial kernel with its activation (one-dimensional grid, tiles in groups of 8 rows, wrapped operands), and
    a kernel in the same tile order whose epilogue adds a value per row and per column: exact on small integers."""
    import extra_kernels as X
    g = torch.Generator(device="cpu").manual_seed(5)
    M, N, Kd = 700, 520, 96
    a = torch.randint(-1, 2, (M, Kd), generator=g).to(torch.bfloat16).to(DEV)
    b = torch.randint(-1, 2, (Kd, N), generator=g).to(torch.bfloat16).to(DEV)
    c = torch.zeros(M, N, dtype=torch.bfloat16, device=DEV)
    grid = (triton.cdiv(M, 64) * triton.cdiv(N, 128),)
    k = K.matmul_wrapped[grid](a, b, c, M, N, Kd, a.stride(0), 1, b.stride(0), 1, c.stride(0), 1, BM=64, BN=128, BK=32, GROUP_M=8, ACTIVATION="leaky_relu")
    torch.cuda.synchronize()
    assert k.function.family == "gemm" and "epilogue" in k.function.last_kernel
    z = a.float() @ b.float()
    assert torch.equal(c.float(), torch.where(z >= 0, z, (z * 0.01).bfloat16().float()))
    bias = torch.cat([torch.randint(-4, 5, (N,), generator=g), torch.randint(-2, 3, (M,), generator=g)]).float().to(DEV)
    k = X.matmul_grouped_order_plus_bias[grid](a, b, c, bias, M, N, Kd, a.stride(0), b.stride(0), c.stride(0), BM=64, BN=128, BK=32, GROUP_M=8)
    torch.cuda.synchronize()
    assert k.function.family == "gemm" and "epilogue" in k.function.last_kernel
    assert torch.equal(c.float(), z + bias[:N][None, :] + 16.0 * bias[N:][:, None])


@pytest.mark.parametrize("dtype,BM,family", [(torch.bfloat16, 128, "gemm"), (torch.float16, 128, "gemm"), (torch.bfloat16, 64, "tile_program")])
def test_matmul_with_gathered_rows(dtype, BM, family):
    """Tile products whose A rows come through an index vector and whose weights are picked by a loaded expert id
    (examples/kernels.py:expert_rows_matmul, the shape of unstructured_ptr_used_in_loop.mlir): with blocks of 128 rows
    the matrix-product kernel takes the index vector and the ids as they are; with smaller blocks the program runs as
    small-product code of the generic family."""
    from triton_shared_amd.examples import kernels
    torch.manual_seed(18)
    tokens, kd, nd, experts = 300, 150, 256, 3
    a = torch.randn(512, kd, device=DEV).to(dtype)
    b = torch.randn(experts, kd, nd, device=DEV).to(dtype)
    rows = torch.randint(0, 512, (tokens,), device=DEV, dtype=torch.int32)
    blocks = triton.cdiv(tokens, BM)
    ids = torch.tensor([2, -1, 0, 1, -1][:blocks], device=DEV, dtype=torch.int32)
    c = torch.zeros(tokens, nd, device=DEV, dtype=dtype)
    k = kernels.expert_rows_matmul[(blocks, 2)](a, b, c, rows, ids, tokens, kd, nd, kd, kd * nd, nd, nd, BM=BM, BN=128, BK=64)
    torch.cuda.synchronize()
    assert k.function.family == family
    if family == "gemm":
        assert k.function.last_kernel.startswith("gemm_mfma_kernel")
    want = torch.zeros(tokens, nd, dtype=torch.float64, device=DEV)
    for blk, e in enumerate(ids.tolist()):
        r = slice(blk * BM, min(tokens, blk * BM + BM))
        if e >= 0:
            want[r] = a[rows[r].long()].double() @ b[e].double()
        else:
            assert torch.equal(c[r], torch.zeros_like(c[r]))          # a block whose expert id is negative is left alone
    assert ((c.double() - want).norm() / want.norm()) <= 1e-2


def test_matmul_with_gathered_rows_is_exact_on_selections():
    # every expert's matrix selects and negates columns of its input rows: the result is exact, so a wrong row index, a
    # wrong expert, a wrong pitch or a transposed operand cannot pass; 16-byte aligned pitches (the vector path) and
    # rows picked more than once
    import extra_kernels as X
    torch.manual_seed(19)
    tokens, kd, nd, experts = 1000, 256, 384, 4
    a = torch.randint(-8, 9, (700, kd), device=DEV).bfloat16()
    pick = torch.randint(0, kd, (experts, nd), device=DEV)
    b = torch.zeros(experts, kd, nd, device=DEV, dtype=torch.bfloat16)
    for e in range(experts):
        b[e, pick[e], torch.arange(nd, device=DEV)] = -1.0
    rows = torch.randint(0, 700, (tokens,), device=DEV, dtype=torch.int32)
    ids = torch.randint(-1, experts, (triton.cdiv(tokens, 128),), device=DEV, dtype=torch.int32)
    c = torch.full((tokens, nd), 5.0, device=DEV, dtype=torch.bfloat16)
    k = X.grouped_rows_matmul[(triton.cdiv(tokens, 128), triton.cdiv(nd, 128))](a, b, c, rows, ids, tokens, kd, nd, kd, kd * nd, nd, nd, BM=128, BN=128, BK=64)
    torch.cuda.synchronize()
    assert k.function.family == "gemm" and k.function.last_kernel == "gemm_dma_kernel<128x128>"   # a ragged last row tile
    want = torch.full((tokens, nd), 5.0, device=DEV, dtype=torch.bfloat16)
    for blk, e in enumerate(ids.tolist()):
        r = slice(blk * 128, min(tokens, blk * 128 + 128))
        if e >= 0:
            want[r] = -a[rows[r].long()][:, pick[e]]
    assert torch.equal(c, want)


@pytest.mark.parametrize("case", [(1024, 256, 512, 4, "gemm_dma_kernel<128x128>"), (4096, 64, 2048, 8, "gemm_dma_kernel<128x256>"),
                                                         (384, 96, 128, 5, "gemm_dma_kernel<128x128>"),
                                                         # more row tiles than the kernel sorts (256): taken in memory order
                                                         (128 * 300, 32, 128, 6, "gemm_dma_kernel<128x128>"),
                                                         # enough K tiles for the wavefront that touches B's lines ahead of the others
                                                         # (uneven numbers of row tiles per matrix: uneven shares of the lines); fewer K
                                                         # tiles than matrix ids (the K walk starts at id % tiles); a ragged last column
                                                         # tile; fp16
                                                         (4096, 640, 2048, 8, "gemm_dma_kernel<128x256>"), (4096, 96, 2048, 8, "gemm_dma_kernel<128x256>"),
                                                         (4096, 416, 2040, 7, "gemm_dma_kernel<128x256>"), (4224, 320, 2048, 3, "gemm_dma_kernel<128x256>", torch.float16)])
def test_matmul_with_gathered_rows_on_whole_tiles(case):
    tokens, kd, nd, experts, kernel = case[:5]
    dtype = case[5] if len(case) > 5 else torch.bfloat16
    # whole 128-row tiles go to the direct-to-LDS kernel, which walks the row tiles in the order of their matrix ids (so
    # that the tiles of one matrix share an L2): ids dealt out of order, repeated and negative; exact as above
    import extra_kernels as X
    g = torch.Generator(device="cpu").manual_seed(tokens + nd)
    a = torch.randint(-8, 9, (tokens + 77, kd), generator=g).to(dtype).to(DEV)
    pick = torch.randint(0, kd, (experts, nd), generator=g)
    b = torch.zeros(experts, kd, nd, dtype=dtype)
    for e in range(experts):
        b[e, pick[e], torch.arange(nd)] = -1.0
    b = b.to(DEV)
    rows = torch.randint(0, tokens + 77, (tokens,), generator=g, dtype=torch.int32).to(DEV)
    ids = torch.randint(-1, experts, (tokens // 128,), generator=g, dtype=torch.int32)
    ids[0] = experts - 1
    ids = ids.to(DEV)
    c = torch.full((tokens, nd), 5.0, device=DEV, dtype=dtype)
    k = X.grouped_rows_matmul[(tokens // 128, triton.cdiv(nd, 128))](a, b, c, rows, ids, tokens, kd, nd, kd, kd * nd, nd, nd, BM=128, BN=128, BK=64)
    torch.cuda.synchronize()
    assert k.function.family == "gemm" and k.function.last_kernel == kernel
    want = torch.full((tokens, nd), 5.0, device=DEV, dtype=dtype)
    for blk, e in enumerate(ids.tolist()):
        r = slice(blk * 128, blk * 128 + 128)
        if e >= 0:
            want[r] = -a[rows[r].long()][:, pick[e].to(DEV)]
    assert torch.equal(c, want)


@pytest.mark.parametrize("M,N,K,kernel", [(512, 768, 96, "gemm_dma_kernel + epilogue"), (200, 300, 150, "gemm_mfma_kernel<128x128x64> + epilogue"),
                                          (521, 776, 96, "gemm_dma_kernel + epilogue"),
                                          (2100, 2060, 72, "gemm_mfma_kernel<128x128x64> + epilogue")])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_gemm_with_fused_epilogue(M, N, K, kernel, dtype):
    """The tutorial matmul's fused activation (test_matmul.py:98-99, 112-117): ops on the accumulator alone are compiled into
    the epilogue of the matmul kernels.  Operands of -1 / 0 / 1 and a slope of 1/2 make every value exact in 16 bits, so
    the result must equal leaky_relu(A @ B) bit for bit, on each of the three kernels the launcher chooses from."""
    import extra_kernels as X
    g = torch.Generator(device="cpu").manual_seed(M + K)
    a = torch.randint(-1, 2, (M, K), generator=g).to(dtype).to(DEV)
    b = torch.randint(-1, 2, (K, N), generator=g).to(dtype).to(DEV)
    c = torch.full((M, N), 7, device=DEV, dtype=dtype)
    k = X.matmul_leaky[(triton.cdiv(M, 128), triton.cdiv(N, 128))](a, b, c, M, N, K, a.stride(0), b.stride(0), c.stride(0), 0.5, BM=128, BN=128, BK=64)
    torch.cuda.synchronize()
    assert k.function.family == "gemm" and k.function.last_kernel.startswith(kernel), k.function.last_kernel
    want = torch.nn.functional.leaky_relu(a.float() @ b.float(), 0.5)
    assert torch.equal(c.float(), want)
    # epilogues that depend on the element's position: a bias per column before the activation, then slope * acc + what
    # the output held (the kernels find the Triton program that owns an element through the table of tile owners)
    bias = torch.randint(-4, 5, (N,), generator=g).float().to(DEV)
    X.matmul_leaky[(triton.cdiv(M, 128), triton.cdiv(N, 128))](a, b, c, M, N, K, a.stride(0), b.stride(0), c.stride(0), 0.5, BM=128, BN=128, BK=64,
                                                               ACT=2, bias_ptr=bias)
    torch.cuda.synchronize()
    assert torch.equal(c.float(), torch.nn.functional.leaky_relu(a.float() @ b.float() + bias, 0.5))
    held = torch.randint(-8, 9, (M, N), generator=g).to(dtype).to(DEV)
    c.copy_(held)
    k = X.matmul_leaky[(triton.cdiv(M, 128), triton.cdiv(N, 128))](a, b, c, M, N, K, a.stride(0), b.stride(0), c.stride(0), 0.5, BM=128, BN=128, BK=64, ACT=3)
    torch.cuda.synchronize()
    assert k.function.family == "gemm" and k.function.last_kernel.startswith(kernel)
    assert torch.equal(c.float(), (a.float() @ b.float()) * 0.5 + held.float())
    # a smooth activation: within the tolerance of the family
    a = torch.randn(M, K, device=DEV).to(dtype)
    b = torch.randn(K, N, device=DEV).to(dtype)
    X.matmul_leaky[(triton.cdiv(M, 128), triton.cdiv(N, 128))](a, b, c, M, N, K, a.stride(0), b.stride(0), c.stride(0), 0.25, BM=128, BN=128, BK=64, ACT=1)
    torch.cuda.synchronize()
    z = a.double() @ b.double()
    want = z * torch.sigmoid(z * 0.25)
    assert ((c.double() - want).norm() / want.norm()) <= 1e-2


# ------------------------------------------------------------------ grids beyond the device's extents
def test_grid_extents_beyond_the_device_limit():
    """The reference's launcher loops over any grid (backend/driver.py:116-133); the device's grid holds 65535 along y and
    z.  A (3, 70000) grid and a (2, 3, 66000) one run as one-dimensional launches whose kernels number the programs
    themselves: every program must see its own ids and the grid's extents (closed form; the small grid of the same kernel
    is checked against the lane interpreter as well)."""
    import extra_kernels as X
    from oracle import ttir_lanes
    BLOCK = 16

    def expect(gx, gy, gz):
        z, y, x, o = np.meshgrid(np.arange(gz), np.arange(gy), np.arange(gx), np.arange(BLOCK), indexing="ij")
        return (x * 1000003 + y * 7 + z * 131 + o * 3 + gz).astype(np.int32).reshape(-1)

    for grid in [(3, 5, 2), (3, 70000, 1), (2, 3, 66000)]:
        gx, gy, gz = grid
        out = torch.full((gx * gy * gz * BLOCK + 8,), -1, dtype=torch.int32, device=DEV)
        k = X.grid_stamp[grid](out, BLOCK=BLOCK)
        torch.cuda.synchronize()
        assert k.function.family == "tile_program"
        got = out.cpu().numpy()
        assert np.array_equal(got[:-8], expect(gx, gy, gz)), grid
        assert (got[-8:] == -1).all()
        if grid == (3, 5, 2):
            mem = {0: np.full(gx * gy * gz * BLOCK, -1, np.int32)}
            ttir_lanes.Interpreter(k.asm["ttir"]).run(grid, [None], mem)
            assert np.array_equal(mem[0], expect(gx, gy, gz))
    # the hand-written elementwise family (or the compiled fused map, whichever takes it) on rows along program_id(1)
    rows, n_cols = 66000, 1500
    g = torch.Generator(device="cpu").manual_seed(1)
    x = torch.rand(rows, n_cols, generator=g).to(DEV)
    y = torch.rand(rows, n_cols, generator=g).to(DEV)
    z = torch.full((rows, n_cols), -1.0, device=DEV)
    k = X.add_rows_2d[(triton.cdiv(n_cols, 1024), rows)](x, y, z, n_cols, BLOCK=1024)
    torch.cuda.synchronize()
    assert k.function.family in ("map1d", "fused_map"), k.function.family
    assert torch.equal(z, x + y)     # one IEEE addition per element: bit for bit
