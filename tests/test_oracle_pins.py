"""Pins the oracle (oracle/cpu_path.c and oracle/ttir_lanes.py) before anything
is compared against it: closed forms, library routines, brute force on tiny
inputs, and agreement of the two independent restatements.  No GPU."""
import numpy as np
import pytest
import torch

from conftest import golden_ttir
from oracle import ttir_lanes


# ---------------------------------------------------------------- primitives
def test_valid_extent_matches_counting_true_lanes(oracle_cpu):
    # MaskAnalysis.cpp:568-585: dims = max(min(start+size, bound), start) - start.  A dropped max()
    # (negative extent when bound < start) or a swapped min/max fails this.
    L = oracle_cpu.lib()
    for start in (-3, 0, 5, 64, 1000):
        for size in (1, 16, 64):
            for bound in (-10, 0, 3, 5, 6, 64, 70, 1000, 1063, 1064, 5000):
                lanes = start + np.arange(size)
                assert L.oracle_valid_extent(start, size, bound) == int((lanes < bound).sum())


def test_half_conversions_match_torch(oracle_cpu):
    L = oracle_cpu.lib()
    rng = np.random.default_rng(0)
    vals = np.concatenate([rng.standard_normal(4000).astype(np.float32) * 10.0 ** rng.integers(-9, 6, 4000),
                           np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 65536.0, 1e-8, 2.0 ** -24, 2.0 ** -25,
                                     2.0 ** -25 * 1.0001, 6.1e-5, 6.0e-8, np.inf, -np.inf], dtype=np.float32)])
    t = torch.from_numpy(vals)
    want16 = t.half().view(torch.int16).numpy().view(np.uint16)
    wantbf = t.bfloat16().view(torch.int16).numpy().view(np.uint16)
    for v, h, b in zip(vals, want16, wantbf):
        assert L.oracle_f32_to_f16(float(v)) == h, v
        assert L.oracle_f32_to_bf16(float(v)) == b, v
    all16 = np.arange(65536, dtype=np.uint16)
    back = torch.from_numpy(all16.view(np.int16)).view(torch.float16).float().numpy()
    for h in list(range(0, 65536, 97)) + [0x7c00, 0xfc00, 0x0001, 0x03ff, 0x0400]:
        got = L.oracle_f16_to_f32(int(h))
        assert got == back[h] or (np.isnan(got) and np.isnan(back[h]))


# -------------------------------------------------- C restatement vs closed forms
def test_vec_add_is_ieee_addition(oracle_cpu):
    torch.manual_seed(0)
    for n in (1, 127, 1024, 98432):
        x, y = torch.rand(n), torch.rand(n)
        assert torch.equal(oracle_cpu.vec_add(x, y), x + y)  # bit-exact


def test_softmax_matches_torch_and_float64(oracle_cpu):
    torch.manual_seed(0)
    x = torch.randn(1823, 781)  # the reference's own test shape (python/examples/test_softmax.py:60-65)
    y = oracle_cpu.row_softmax(x)
    assert torch.allclose(y, torch.softmax(x, 1))  # the reference's assertion
    assert (y.double() - torch.softmax(x.double(), 1)).abs().max() <= 1e-6
    assert torch.allclose(y.sum(1), torch.ones(1823), atol=1e-5)


def _layernorm_f64(x, w, b, eps):
    xf = x.double()
    mu = xf.mean(1)
    var = ((xf - mu[:, None]) ** 2).mean(1)  # biased
    rs = 1 / torch.sqrt(var + eps)
    return (xf - mu[:, None]) * rs[:, None] * w.double() + b.double(), mu, rs


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("N", [8192, 1000, 64])
def test_layernorm_matches_float64_formula(oracle_cpu, dtype, N):
    torch.manual_seed(1)
    x = (torch.randn(37, N) * 1.5 - 0.3).to(dtype)
    w, b = (1 + 0.1 * torch.randn(N)).to(dtype), (0.1 * torch.randn(N)).to(dtype)
    y, mean, rstd = oracle_cpu.layer_norm_fwd(x, w, b, 1e-5, BLOCK=1024 if N > 64 else 64)
    yr, mu, rs = _layernorm_f64(x, w, b, 1e-5)
    tol = 1e-2 if dtype == torch.float16 else 5e-2
    assert (y.double() - yr).abs().max() <= tol
    assert (mean.double() - mu).abs().max() <= 1e-5
    assert ((rstd.double() - rs) / rs).abs().max() <= 1e-5


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_matmul_matches_float64(oracle_cpu, dtype):
    torch.manual_seed(2)
    # ragged in every dimension, as python/examples/test_matmul.py:137-157 (179x167x321)
    a, b = (torch.randn(179, 167) * 0.5).to(dtype), (torch.randn(167, 321) * 0.5).to(dtype)
    c = oracle_cpu.matmul_tiles(a, b, BM=32, BN=64, BK=16, GROUP_M=8)
    ref = a.double() @ b.double()
    assert torch.allclose(c.double(), ref, atol=1e-2 * ref.abs().max().item(), rtol=0)
    assert (c.double() - ref).norm() / ref.norm() <= 1e-2
    # negative check: an oracle that read an operand transposed would compute another product; on a square problem
    # (where such a mistake still has matching shapes) the oracle's result is far from both wrong products
    a, b = (torch.randn(96, 96) * 0.5).to(dtype), (torch.randn(96, 96) * 0.5).to(dtype)
    c = oracle_cpu.matmul_tiles(a, b, BM=32, BN=64, BK=16, GROUP_M=8).double()
    ref = a.double() @ b.double()
    assert (c - ref).norm() / ref.norm() <= 1e-2
    for wrong in (a.double().T @ b.double(), a.double() @ b.double().T, b.double() @ a.double()):
        assert (c - wrong).norm() / ref.norm() > 0.5


def test_w8a16_matches_closed_form(oracle_cpu):
    torch.manual_seed(3)
    a = torch.randn(16, 300).half()
    w = torch.randint(-127, 128, (300, 200), dtype=torch.int8)
    s = (0.001 + 0.009 * torch.rand(200)).half()
    c = oracle_cpu.w8a16_matmul(a, w, s, BN=64, BK=64)
    ref = a.double() @ (w.half() * s[None, :]).double()  # dequantised weights rounded to fp16 first
    assert (c.double() - ref).norm() / ref.norm() <= 2e-3
    # scale per *output channel*: scaling rows instead would fail
    wrong = a.double() @ (w.double() * s.double()[:200][None, :].flip(1))
    assert (c.double() - wrong).norm() / ref.norm() > 0.1


# ---------------------------------- lane interpreter vs C restatement (independent)
def _u16(t):
    return t.view(torch.int16).numpy().view(np.uint16).reshape(-1)


def test_lanes_vs_c_vec_add(oracle_cpu):
    torch.manual_seed(0)
    n, B = 333, 64
    x, y, z = torch.rand(n), torch.rand(n), torch.zeros(n)
    it = ttir_lanes.Interpreter(golden_ttir("vec_add.small"))
    grid = (n + B - 1) // B + 2  # two programs entirely past the end: all-masked
    log = it.run((grid,), [None, None, None, n], {0: x.numpy(), 1: y.numpy(), 2: z.numpy()})
    assert torch.equal(z, oracle_cpu.vec_add(x, y, BLOCK=B))
    counts = [len(a[2]) for a in (prog[2] for prog in log)]
    assert counts == [oracle_cpu.lib().oracle_valid_extent(p * B, B, n) for p in range(grid)]
    assert counts[-1] == 0 and counts[-2] == 0 and counts[5] == 333 - 320


def test_lanes_vs_c_softmax(oracle_cpu):
    torch.manual_seed(0)
    x, o = torch.randn(9, 50), torch.zeros(9, 50)
    it = ttir_lanes.Interpreter(golden_ttir("row_softmax.small"))
    it.run((9,), [None, None, 50, 50, 50], {0: o.numpy().reshape(-1), 1: x.numpy().reshape(-1)})
    ref = oracle_cpu.row_softmax(x, BLOCK=64)
    assert (o - ref).abs().max() <= 1e-7  # np.exp vs libm expf
    assert torch.allclose(o, torch.softmax(x, 1))


def test_lanes_vs_c_layernorm(oracle_cpu):
    torch.manual_seed(0)
    M, N = 5, 150
    x, w, b = torch.randn(M, N).half(), torch.randn(N).half(), torch.randn(N).half()
    y, mean, rstd = torch.zeros(M, N).half(), torch.zeros(M), torch.zeros(M)
    it = ttir_lanes.Interpreter(golden_ttir("layer_norm_fwd.small"))
    it.run((M,), [None] * 6 + [N, N, 1e-5], {0: x.numpy().reshape(-1), 1: y.numpy().reshape(-1), 2: w.numpy(),
                                             3: b.numpy(), 4: mean.numpy(), 5: rstd.numpy()})
    y2, m2, r2 = oracle_cpu.layer_norm_fwd(x, w, b, 1e-5, BLOCK=64)
    assert torch.equal(y, y2) and torch.equal(mean, m2) and torch.equal(rstd, r2)


def test_lanes_vs_c_matmul(oracle_cpu):
    torch.manual_seed(0)
    M, N, K = 70, 90, 40
    a, b = (torch.randn(M, K) * 0.5).bfloat16(), (torch.randn(K, N) * 0.5).bfloat16()
    c = torch.zeros(M, N).bfloat16()
    it = ttir_lanes.Interpreter(golden_ttir("matmul_tiles.small"))
    grid = ((M + 31) // 32) * ((N + 31) // 32)
    it.run((grid,), [None, None, None, M, N, K, K, N, N], {0: _u16(a), 1: _u16(b), 2: _u16(c)})
    assert torch.equal(c, oracle_cpu.matmul_tiles(a, b, BM=32, BN=32, BK=16, GROUP_M=2))


def test_lanes_vs_c_w8a16(oracle_cpu):
    torch.manual_seed(0)
    M, N, K = 13, 70, 100
    a = torch.randn(M, K).half()
    w = torch.randint(-127, 128, (K, N), dtype=torch.int8)
    s = (0.001 + 0.009 * torch.rand(N)).half()
    c = torch.zeros(M, N).half()
    it = ttir_lanes.Interpreter(golden_ttir("w8a16_matmul.small"))
    it.run((1, (N + 31) // 32), [None] * 4 + [M, N, K, K, N, N],
           {0: a.numpy().reshape(-1), 1: w.numpy().reshape(-1), 2: s.numpy(), 3: c.numpy().reshape(-1)})
    assert torch.equal(c, oracle_cpu.w8a16_matmul(a, w, s, BM=16, BN=32, BK=32))


# ---- fused elementwise maps: the lane interpreter is the oracle; pin its ops by closed forms in float64
def _run_lanes(name, n, scalars, inputs, out_dtype, block=1024):
    it = ttir_lanes.Interpreter(golden_ttir(name))
    mem = {i: a for i, a in enumerate(inputs)}
    out = np.zeros(n, dtype=out_dtype)
    mem[len(inputs)] = out
    it.run(((n + block - 1) // block,), [None] * (len(inputs) + 1) + [n] + list(scalars), mem)
    return out


def test_lanes_fused_maps_against_closed_forms():
    rng = np.random.default_rng(0)
    n = 3000
    x, y = rng.standard_normal(n).astype(np.float32) * 2, rng.standard_normal(n).astype(np.float32)
    got = _run_lanes("gelu_tanh_bias", n, [], [x.copy(), y.copy()], np.float32)
    v = x.astype(np.float64) + y
    want = 0.5 * v * (1 + np.tanh(0.7978845608028654 * (v + 0.044715 * v ** 3)))
    assert np.abs(got - want).max() <= 2e-6
    got = _run_lanes("clamp_scale_where", n, [-0.5, 1.25, 3.0], [x.copy(), y.copy()], np.float32)
    want = np.where(x > y, 3.0 * np.clip(x, -0.5, 1.25), np.sqrt(np.abs(y.astype(np.float64))))
    assert np.abs(got - want).max() <= 1e-6
    g, u = x.astype(np.float16), y.astype(np.float16)
    got = _run_lanes("silu_mul_f16", n, [], [g.copy(), u.copy()], np.float16)
    g64, u64 = g.astype(np.float64), u.astype(np.float64)
    want = g64 / (1 + np.exp(-g64)) * u64
    assert np.abs(got.astype(np.float64) - want).max() <= 2e-3 * np.abs(want).max()
    # special values through the comparison and min/max ops: NaN compares false, maxnumf/minnumf drop it
    xs = np.array([np.nan, 1.0, -np.inf, 0.5], np.float32)
    ys = np.array([0.0, np.nan, 2.0, 0.5], np.float32)
    got = _run_lanes("clamp_scale_where", 4, [-0.5, 1.25, 3.0], [xs.copy(), ys.copy()], np.float32)
    assert got[0] == 0.0 and np.isnan(got[1]) and got[2] == np.float32(np.sqrt(2.0)) and got[3] == np.float32(np.sqrt(0.5))


def test_lanes_gathers_and_scatters_against_reference_goldens():
    """The lane interpreter on data-dependent addresses, carried offset blocks and nested loops: the expected outputs are
    the literal tensors python/examples/test_gather_scatter.py:108-164 asserts (written as runs)."""
    import extra_kernels as X
    from test_planner import compile_ttir

    def runs(*pairs):
        out = []
        for value, times in pairs:
            out += [value] * times
        return out

    quarter = lambda fill: runs(*[(v, 4) for v in range(2, 10)], (fill, 32), *[(v, 4) for v in range(18, 26)], (fill, 32))
    want = {
        "gather_div10": runs(*[(v, 10) for v in range(7, 13)], (13, 4), (14, 10), (15, 54)),
        "gather_quarter_masked": quarter(0),
        "gather_quarter_masked_other": quarter(-1),
        "gather_div12_masked_store": runs(*[(v, 12) for v in range(2, 7)], (7, 17), (-1, 51)),
        "gather_scatter_nested": list(range(2, 13)) + [-1] * 4 + [17, 18, -1, 20, 21, -1, 23, 24, 25, -1, -1, 28] + [-1] * 5 + [0] * 11 + [-1] * 85,
    }
    for name, expected in want.items():
        assert len(expected) == 128
        ttir = compile_ttir(getattr(X, name), {"src": "*i32", "dst": "*i32"}, {})
        src = np.arange(2, 130, dtype=np.int32)
        dst = np.full(128, -1, dtype=np.int32)
        ttir_lanes.Interpreter(ttir).run((1,), [None, None], {0: src, 1: dst})
        assert dst.tolist() == expected, name


def test_lanes_reductions_with_regions_and_scans_against_numpy():
    """Combiner regions (argmax / argmin with ties, first index wins), integer reductions with wraparound, and scans along
    either axis, against numpy's closed forms."""
    import extra_kernels as X
    from test_planner import compile_ttir
    P, I = "*fp32", "*i32"
    rng = np.random.default_rng(0)
    x = rng.integers(0, 6, (5, 200)).astype(np.float32)          # many ties
    t = compile_ttir(X.arg_extremes_rows, {"x_ptr": P, "max_ptr": I, "min_ptr": I, "n_cols": "i32", "pitch": "i32", "BC": "constexpr"}, {"BC": 256})
    hi, lo = np.zeros(5, np.int32), np.zeros(5, np.int32)
    ttir_lanes.Interpreter(t).run((5,), [None, None, None, 200, 200], {0: x.reshape(-1).copy(), 1: hi, 2: lo})
    assert hi.tolist() == x.argmax(1).tolist() and lo.tolist() == x.argmin(1).tolist()
    for axis, (BR, BC) in [(1, (4, 8)), (0, (64, 32))]:
        sig = {"x_ptr": P, "y_ptr": P, "pitch": "i32", "BR": "constexpr", "BC": "constexpr", "AXIS": "constexpr"}
        t = compile_ttir(X.running_sum_2d, sig, {"BR": BR, "BC": BC, "AXIS": axis})
        x = rng.standard_normal((BR, BC)).astype(np.float32)
        y = np.zeros(BR * BC, np.float32)
        ttir_lanes.Interpreter(t).run((1,), [None, None, BC], {0: x.reshape(-1).copy(), 1: y})
        assert np.abs(y.reshape(BR, BC) - np.cumsum(x.astype(np.float64), axis=axis)).max() < 1e-5
    t = compile_ttir(X.int_reductions, {"x_ptr": I, "out_ptr": I, "n": "i32", "BLOCK": "constexpr"}, {"BLOCK": 512})
    xi = rng.integers(-2**31, 2**31, 300).astype(np.int32)
    out = np.zeros(4, np.int32)
    ttir_lanes.Interpreter(t).run((1,), [None, None, 300], {0: xi.copy(), 1: out})
    pad = np.concatenate([xi, np.zeros(212, np.int32)])
    assert out.tolist() == [int(pad.sum(dtype=np.int32)), int(pad.max()), int(pad.min()), int(np.bitwise_xor.reduce(pad))]


def test_lanes_on_the_reference_functional_cases():
    """The lane interpreter against the expectations of the reference's functional tests (tests/reference_cases.py):
    early return, scalar stores from nested loops, a loaded 64-bit offset, block pointers, index arithmetic with // and %,
    grid-stride loops, loop-carried offset blocks, masks read from memory, an einsum with carried accumulators."""
    import extra_kernels as X
    import reference_cases
    from test_planner import compile_ttir
    for case in reference_cases.cases():
        ttir = compile_ttir(getattr(X, case["kernel"]), case["sig"], case["consts"])
        args = case["args"]()
        arrays = [a for a in args if isinstance(a, np.ndarray)]
        values = [None if isinstance(a, np.ndarray) else a for a in args]
        log = ttir_lanes.Interpreter(ttir).run(case["grid"], values, dict(enumerate(arrays)))
        case["check"](arrays)
        for program in log:                      # and no lane of any program leaves its buffer
            for _kind, arg, offsets in program:
                o = np.asarray(offsets)
                assert o.size == 0 or (o.min() >= 0 and o.max() < arrays[arg].size), (case["name"], arg)


def test_lanes_on_the_core_language_cases():
    """The lane interpreter against closed forms for the language features the reference enables from Triton's core tests
    (tests/core_cases.py): umulhi, 64-bit loop indices, calls of functions kept out of line, new axes, tl.full in every
    type, double precision, early returns through merged blocks, NaN rules of min / max / clamp, permutes up to rank 4,
    broadcasts, products of constants, masked scalar loads, fma, const pointers, arange, every fp16 value widened, abs,
    cache hints, unary ops, // and %, argument specialisation, unary math, fp16 products."""
    import core_cases
    import core_kernels
    from test_planner import compile_ttir
    for case in core_cases.cases():
        ttir = compile_ttir(getattr(core_kernels, case["kernel"]), case["sig"], case["consts"])
        args = case["args"]()
        arrays = [a for a in args if isinstance(a, np.ndarray)]
        values = [None if isinstance(a, np.ndarray) else a for a in args]
        log = ttir_lanes.Interpreter(ttir).run(case["grid"], values, dict(enumerate(arrays)))
        case["check"](arrays)
        for program in log:
            for _kind, arg, offsets in program:
                o = np.asarray(offsets)
                assert o.size == 0 or (o.min() >= 0 and o.max() < arrays[arg].size), (case["name"], arg)


def test_lanes_integer_bit_and_conversion_ops_against_numpy():
    """Unsigned division / remainder / compare / max, shifts, umulhi, abs, bit casts, float <-> integer conversions, clamp,
    correctly rounded sqrt / divide and fma: every plane bit for bit against tests/op_zoo.py."""
    import extra_kernels as X
    import op_zoo
    from test_planner import compile_ttir
    n = 1000
    x, y = op_zoo.int_inputs(n)
    t = compile_ttir(X.int_ops, {"x_ptr": "*i32", "y_ptr": "*i32", "out_ptr": "*i32", "n": "i32", "BLOCK": "constexpr"}, {"BLOCK": 256})
    out = np.zeros(12 * n, np.int32)
    ttir_lanes.Interpreter(t).run((4,), [None, None, None, n], {0: x, 1: y, 2: out})
    assert np.array_equal(out.reshape(12, n), op_zoo.int_expected(x, y))
    xf, yf = op_zoo.float_inputs(n)
    sig = {"x_ptr": "*fp32", "y_ptr": "*fp32", "out_ptr": "*fp32", "n": "i32", "lo": "fp32", "hi": "fp32", "BLOCK": "constexpr"}
    t = compile_ttir(X.float_ops, sig, {"BLOCK": 256})
    outf = np.zeros(8 * n, np.float32)
    ttir_lanes.Interpreter(t).run((4,), [None, None, None, n, -50.0, 75.5], {0: xf, 1: yf, 2: outf})
    assert np.array_equal(outf.reshape(8, n), op_zoo.float_expected(xf, yf, -50.0, 75.5))


def test_lanes_transpose_and_reshape_against_numpy():
    import extra_kernels as X
    from test_planner import compile_ttir
    P = "*fp32"
    for R, C in [(16, 32), (32, 32)]:
        t = compile_ttir(X.transpose_tile, {"src": P, "dst": P, "R": "constexpr", "C": "constexpr"}, {"R": R, "C": C})
        x = np.random.default_rng(0).standard_normal((R, C)).astype(np.float32)
        y = np.zeros(R * C, np.float32)
        ttir_lanes.Interpreter(t).run((1,), [None, None], {0: x.reshape(-1).copy(), 1: y})
        assert np.array_equal(y.reshape(C, R), x.T + np.arange(R, dtype=np.float32)[None, :])
    t = compile_ttir(X.fold_and_sum, {"src": P, "dst": P, "R": "constexpr", "C": "constexpr"}, {"R": 8, "C": 64})
    x = np.random.default_rng(1).standard_normal(512).astype(np.float32)
    y = np.zeros(8 + 512, np.float32)
    ttir_lanes.Interpreter(t).run((1,), [None, None], {0: x.copy(), 1: y})
    assert np.abs(y[:8] - x.reshape(8, 64).astype(np.float64).sum(1)).max() < 1e-5 and np.array_equal(y[8:], x * 2)


def test_lanes_extern_functions_against_float64():
    """tt.extern_elementwise by symbol name (test/Conversion/TritonToLinalg/convert_extern_elementwise.mlir): each plane
    within 2e-7 relative of the float64 value."""
    import extra_kernels as X
    from test_planner import compile_ttir
    t = compile_ttir(X.extern_math, {"x_ptr": "*fp32", "y_ptr": "*fp32", "out_ptr": "*fp32", "n": "i32", "BLOCK": "constexpr"}, {"BLOCK": 256})
    rng = np.random.default_rng(0)
    n = 500
    x = (rng.standard_normal(n) * 3).astype(np.float32)
    y = rng.standard_normal(n).astype(np.float32)
    out = np.zeros(6 * n, np.float32)
    ttir_lanes.Interpreter(t).run((2,), [None, None, None, n], {0: x, 1: y, 2: out})
    x64, y64 = x.astype(np.float64), y.astype(np.float64)
    want = np.stack([np.abs(x64) ** y64, np.arctan2(x64, y64), np.log1p(np.abs(x64)), np.tanh(y64), np.trunc(x64), np.arcsin(np.clip(y64, -1, 1))])
    assert (np.abs(out.reshape(6, n) - want).max(axis=1) <= 2e-7 * np.abs(want).max(axis=1)).all()


def test_lanes_philox_dropout_against_an_independent_philox():
    """tl.rand expands into ~60 integer ops per element (umulhi, xor, shifts, wrapping adds); the oracle's result equals
    tests/op_zoo.philox_uniform, written from the published algorithm, bit for bit."""
    import extra_kernels as X
    import op_zoo
    from test_planner import compile_ttir
    sig = {"x_ptr": "*fp32", "out_ptr": "*fp32", "n": "i32", "p": "fp32", "seed": "i32", "BLOCK": "constexpr"}
    t = compile_ttir(X.seeded_dropout, sig, {"BLOCK": 1024})
    n = 3000
    x = np.random.default_rng(0).standard_normal(n).astype(np.float32)
    out = np.zeros(n, np.float32)
    ttir_lanes.Interpreter(t).run((3,), [None, None, n, 0.3, 1234], {0: x, 1: out})
    u = op_zoo.philox_uniform(1234, np.arange(n))
    assert np.array_equal(out, np.where(u > np.float32(0.3), x / (np.float32(1) - np.float32(0.3)), np.float32(0)))


def test_lanes_join_split_cat_against_numpy():
    import extra_kernels as X
    from test_planner import compile_ttir
    t = compile_ttir(X.join_split_cat, {"a_ptr": "*fp32", "b_ptr": "*fp32", "out_ptr": "*fp32", "N": "constexpr"}, {"N": 64})
    a = np.arange(64, dtype=np.float32)
    b = 100 + np.arange(64, dtype=np.float32)
    out = np.zeros(6 * 64, np.float32)
    ttir_lanes.Interpreter(t).run((1,), [None, None, None], {0: a, 1: b, 2: out})
    assert np.array_equal(out, np.concatenate([np.stack([a, b], 1).reshape(-1), a + 1, b + 1, b, a]))


def test_lanes_if_with_results_against_numpy():
    import extra_kernels as X
    from test_planner import compile_ttir
    t = compile_ttir(X.branch_with_results, {"x_ptr": "*fp32", "flag_ptr": "*i32", "out_ptr": "*fp32", "N": "constexpr"}, {"N": 128})
    x = np.random.default_rng(2).standard_normal(128).astype(np.float32)
    flags = np.array([3, -2, 0, 5], dtype=np.int32)
    out = np.zeros(4 * 128, np.float32)
    ttir_lanes.Interpreter(t).run((4,), [None, None, None], {0: x, 1: flags, 2: out})
    want = np.stack([(x * 2 + 1 + np.float32(3 * f)) if f > 0 else (x - 1 - 1 + np.float32(7 - f)) for f in flags])
    assert np.array_equal(out.reshape(4, 128), want.astype(np.float32))


def test_lanes_flash_attention_forward_matches_the_closed_form():
    """The lane interpreter on a flash-attention forward (two tile products per step, online softmax with carried vectors):
    softmax(Q K^T / sqrt(D)) V in float64, on a sequence that is not a multiple of the blocks."""
    import extra_kernels as X
    from test_planner import compile_ttir
    sig = {"Q": "*fp16", "K": "*fp16", "V": "*fp16", "O": "*fp16", "sm_scale": "fp32", "seq": "i32", "stride_h": "i32", "stride_s": "i32",
           "BM": "constexpr", "BN": "constexpr", "D": "constexpr"}
    t = compile_ttir(X.attention_fwd, sig, {"BM": 32, "BN": 32, "D": 32})
    rng = np.random.default_rng(0)
    H, seq, D = 2, 80, 32
    q, k, v = (rng.standard_normal((H, seq, D)).astype(np.float16) for _ in range(3))
    bufs = {0: q.reshape(-1).copy(), 1: k.reshape(-1).copy(), 2: v.reshape(-1).copy(), 3: np.zeros(H * seq * D, np.float16)}
    ttir_lanes.Interpreter(t).run(((seq + 31) // 32, H), [None, None, None, None, np.float32(D ** -0.5), seq, seq * D, D], bufs)
    s = np.einsum("hqd,hkd->hqk", q.astype(np.float64), k.astype(np.float64)) * D ** -0.5
    p = np.exp(s - s.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    want = np.einsum("hqk,hkd->hqd", p, v.astype(np.float64))
    assert np.abs(bufs[3].reshape(H, seq, D).astype(np.float64) - want).max() <= 2e-3
