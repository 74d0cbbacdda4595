"""tts_launch_noalloc (the launch for callers that cannot allocate device memory) against tts_launch, through the C ABI.

Both run the same kernels and add the K slices in slice order, so the int8-weight product must come out bit for bit
the same whether its partial tiles sit in the plan's own workspace (tts_launch) or in the library's static scratch
array (tts_launch_noalloc).  Two calls in a row share that array; the second is a smaller problem."""
import pytest
import torch

from conftest import plan_for

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _inputs(M, N, Kd, seed):
    torch.manual_seed(seed)
    a = torch.randn(M, Kd).half().to(DEV)
    w = torch.randint(-127, 128, (Kd, N), dtype=torch.int8).to(DEV)
    s = (0.001 + 0.009 * torch.rand(N)).half().to(DEV)
    return a, w, s


def _values(a, w, s, c, M, N, Kd):
    # w8a16_matmul(a, w, scale, c, M, N, K, stride_am, stride_wk, stride_cm): the unit inner strides are constants
    return [a.data_ptr(), w.data_ptr(), s.data_ptr(), c.data_ptr(), M, N, Kd, a.stride(0), w.stride(0), c.stride(0)]


def test_noalloc_launch_matches_the_allocating_launch(native):
    plan, _ = plan_for(native, "w8a16_matmul")
    assert plan.family == "gemm_w8a16"
    stream = torch.cuda.current_stream().cuda_stream
    # a split-K shape on the wide kernel (counters and partial tiles), then a smaller one on the same scratch array,
    # then a shape that the narrow kernel and its separate reduce kernel take
    for seed, (M, N, Kd) in enumerate([(16, 2048, 8192), (16, 1024, 4096), (13, 384, 4096)]):
        a, w, s = _inputs(M, N, Kd, seed)
        grid = (1, (N + 127) // 128, 1)
        want = torch.full((M, N), 5.0, dtype=torch.float16, device=DEV)
        got = torch.full((M, N), 7.0, dtype=torch.float16, device=DEV)
        vals = _values(a, w, s, want, M, N, Kd)
        d = plan.describe_launch(grid, vals)
        assert int(d["split"]) > 1, d            # the case that needs scratch memory
        plan.launch(grid, stream, vals)
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        plan.launch_noalloc(grid, stream, _values(a, w, s, got, M, N, Kd))
        torch.cuda.synchronize()
        if seed > 0:                             # the first call on a device looks up the scratch array's address
            assert torch.cuda.mem_get_info()[0] >= free_before
        assert torch.equal(got, want), (M, N, Kd)
        ref = a.double() @ (w.half() * s[None, :]).double()
        assert ((got.double() - ref).norm() / ref.norm()).item() <= 1e-2


def test_noalloc_launch_refuses_a_plan_that_still_has_to_compile(native):
    # a fused map is compiled into a kernel of its own at its first launch, which allocates: the no-allocation launch
    # says so instead of compiling (nothing is dereferenced before the refusal)
    plan, _ = plan_for(native, "gelu_tanh_bias")
    assert plan.family == "fused_map"
    n = 4096
    x = torch.randn(n, device=DEV)
    b = torch.randn(n, device=DEV)
    y = torch.zeros(n, device=DEV)
    stream = torch.cuda.current_stream().cuda_stream
    vals = [x.data_ptr(), b.data_ptr(), y.data_ptr(), n]
    with pytest.raises(NotImplementedError, match="allocates"):
        plan.launch_noalloc((4, 1, 1), stream, vals)
    plan.launch((4, 1, 1), stream, vals)         # compiles
    want = y.clone()
    y.zero_()
    plan.launch_noalloc((4, 1, 1), stream, vals)  # now there is nothing left to allocate
    torch.cuda.synchronize()
    assert torch.equal(y, want) and want.abs().sum().item() > 0


def test_noalloc_launch_runs_a_skinny_matmul_in_k_slices_from_the_static_array(native):
    # a matrix product with too few output tiles for the chip runs in K slices, whose fp32 partial sums tts_launch keeps in
    # the stream's workspace and tts_launch_noalloc in the static array, in as many slices as fit there (8 MiB: eight
    # slices of 128 x 2048); with the same number of slices the results agree bit for bit, both adding them in slice order.
    # A product of which not even two slices fit (1024 x 2048) runs without slices in the call that may not allocate,
    # which changes the order of the sums: within the tolerance of the family
    plan, _ = plan_for(native, "matmul_tiles")
    assert plan.family == "gemm"
    stream = torch.cuda.current_stream().cuda_stream
    for seed, (M, N, Kd, fits) in enumerate([(128, 2048, 8192, True), (64, 1024, 4096, True), (1000, 2048, 4096, False)]):
        torch.manual_seed(seed)
        a = (torch.randn(M, Kd) * 0.1).bfloat16().to(DEV)
        b = (torch.randn(Kd, N) * 0.1).bfloat16().to(DEV)
        want = torch.full((M, N), 5.0, dtype=torch.bfloat16, device=DEV)
        got = torch.full((M, N), 7.0, dtype=torch.bfloat16, device=DEV)
        grid = (((M + 127) // 128) * ((N + 127) // 128), 1, 1)
        plan.launch(grid, stream, [a.data_ptr(), b.data_ptr(), want.data_ptr(), M, N, Kd, Kd, N, N])
        torch.cuda.synchronize()
        assert plan.last_kernel.endswith("K slices"), plan.last_kernel
        # (the entry point's first call on a device looks the static array's address up, which is when the runtime gives
        # the array its memory: free memory is compared around a later call)
        plan.launch_noalloc(grid, stream, [a.data_ptr(), b.data_ptr(), got.data_ptr(), M, N, Kd, Kd, N, N])
        torch.cuda.synchronize()
        got.fill_(7.0)
        free_before = torch.cuda.mem_get_info()[0]
        plan.launch_noalloc(grid, stream, [a.data_ptr(), b.data_ptr(), got.data_ptr(), M, N, Kd, Kd, N, N])
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] >= free_before
        assert plan.last_kernel.endswith("K slices") == fits, plan.last_kernel
        ref = a.double() @ b.double()
        assert ((got.double() - ref).norm() / ref.norm()).item() <= 1e-2
        if fits and M * N * 4 * 16 <= (8 << 20):   # (at most 16 slices are ever taken: then both calls took the same number)
            assert torch.equal(got, want), (M, N, Kd)


def test_noalloc_refusal_leaves_a_matmul_with_epilogue_on_its_kernel(native):
    """A matrix product with a fused epilogue needs a compiled kernel and, per launch shape, a device table of tile
    owners: the launch that may not allocate refuses both, and the refusal must not be remembered as "this launch belongs
    to the generic family" -- the same launch through tts_launch afterwards runs the product kernel with its epilogue."""
    import triton
    import triton_shared_amd as tsa
    import extra_kernels as X
    tsa.activate()
    g = torch.Generator(device="cpu").manual_seed(3)
    stream = torch.cuda.current_stream().cuda_stream

    def operands(M, N, K):
        a = torch.randint(-1, 2, (M, K), generator=g).to(torch.bfloat16).to(DEV)
        b = torch.randint(-1, 2, (K, N), generator=g).to(torch.bfloat16).to(DEV)
        return a, b, torch.full((M, N), 7, device=DEV, dtype=torch.bfloat16)

    M, N, K = 512, 768, 96
    a, b, c = operands(M, N, K)
    grid = (triton.cdiv(M, 128), triton.cdiv(N, 128), 1)
    k = X.matmul_leaky[grid[:2]](a, b, c, M, N, K, a.stride(0), b.stride(0), c.stride(0), 0.5, BM=128, BN=128, BK=64)
    torch.cuda.synchronize()
    assert k.function.family == "gemm" and k.function.last_kernel.startswith("gemm_dma_kernel + epilogue")
    want = torch.nn.functional.leaky_relu(a.float() @ b.float(), 0.5)
    assert torch.equal(c.float(), want)
    n_args = len(k.function.arg_kinds)

    def values(a, b, c, M, N, K):
        vals = [a.data_ptr(), b.data_ptr(), c.data_ptr(), M, N, K, a.stride(0), b.stride(0), c.stride(0), 0.5]
        assert len(vals) == n_args, (n_args, k.function.arg_kinds)
        return vals

    # (1) a plan that has compiled nothing yet: refused, then launched the ordinary way on the product kernel
    fresh = native.PlanHandle(k.kernel)
    c.fill_(7)
    with pytest.raises(NotImplementedError, match="allocates"):
        fresh.launch_noalloc(grid, stream, values(a, b, c, M, N, K))
    torch.cuda.synchronize()
    assert torch.all(c == 7)                     # nothing ran
    fresh.launch(grid, stream, values(a, b, c, M, N, K))
    torch.cuda.synchronize()
    assert fresh.last_kernel.startswith("gemm_dma_kernel + epilogue"), fresh.last_kernel
    assert torch.equal(c.float(), want)
    c.fill_(7)
    fresh.launch_noalloc(grid, stream, values(a, b, c, M, N, K))   # kernel compiled, table of this shape built: runs
    torch.cuda.synchronize()
    assert fresh.last_kernel.startswith("gemm_dma_kernel + epilogue") and torch.equal(c.float(), want)
    # (2) the kernel is compiled, but a new shape needs a new table of tile owners: refused, not rebound to the generic
    # family; a smaller problem than the first, as the second call of two in a row
    M2, N2, K2 = 256, 512, 64
    a2, b2, c2 = operands(M2, N2, K2)
    grid2 = (triton.cdiv(M2, 128), triton.cdiv(N2, 128), 1)
    with pytest.raises(NotImplementedError, match="allocates"):
        fresh.launch_noalloc(grid2, stream, values(a2, b2, c2, M2, N2, K2))
    d = fresh.describe_launch(grid2, values(a2, b2, c2, M2, N2, K2))
    assert d["kernel"] == "gemm_mfma", d
    fresh.launch(grid2, stream, values(a2, b2, c2, M2, N2, K2))
    torch.cuda.synchronize()
    assert fresh.last_kernel.startswith("gemm_dma_kernel + epilogue"), fresh.last_kernel
    assert torch.equal(c2.float(), torch.nn.functional.leaky_relu(a2.float() @ b2.float(), 0.5))
