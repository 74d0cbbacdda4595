"""Host-side tests of the native planner: TTIR text -> structured program ->
kernel family + bindings.  The expectations are hand-encoded from the CHECK lines
of the reference's lit tests (read, not copied) and pinned by brute force with
the independent lane interpreter.  No GPU."""
import re

import numpy as np
import pytest
import torch

from conftest import golden_ttir, plan_for
from oracle import ttir_lanes


def accesses(structured):
    """[(kind, readable comment)] of every load/store line, in program order."""
    out = []
    for line in structured.splitlines():
        m = re.match(r"\s*(load|store|scalar_store|scalar_load)\b.*? ; (.*)$", line)
        if m:
            out.append((m.group(1), m.group(2)))
    return out


def compile_ttir(fn, sig, consts, **opts):
    import os
    import triton
    from triton.backends.compiler import GPUTarget
    from triton.compiler import ASTSource
    import triton_shared_amd as tsa
    tsa.register_backend()
    os.environ.setdefault("TRITON_ALWAYS_COMPILE", "1")
    # stop after the TTIR stage by asking for the asm of a kernel that may not match any family
    from triton_shared_amd.backend.compiler import HIPBackend
    src = ASTSource(fn, signature=sig, constexprs=consts)
    target = GPUTarget(tsa.BACKEND_NAME, "gfx950", 64)
    backend = HIPBackend(target)
    from triton._C.libtriton import ir
    ctx = ir.context()
    ir.load_dialects(ctx)
    options = backend.parse_options(opts)
    mod = src.make_ir(target, options, backend.get_codegen_implementation(options), backend.get_module_map(), ctx)
    return str(backend.make_ttir(mod, {}, options))


# ------------------------------------------------- goldens from the lit tests
def test_vec_add_structured_matches_reference_golden(native):
    # test/Conversion/TritonToStructured/kernel-01-vector-add.mlir CHECK :27-65:
    # sizes [1024], strides [1], offsets [index_cast(pid*1024)], dims = max(min(off+1024, n), off) - off,
    # the same for both loads and the store; addf on the two loaded tiles.
    s = native.ttir_to_structured(golden_ttir("vec_add"))
    acc = accesses(s)
    assert [k for k, _ in acc] == ["load", "load", "store"]
    dims = "dims=[(max((1024 * pid.x), min(((1024 * pid.x) + 1024), arg3)) - (1024 * pid.x))]"
    for (kind, text), arg in zip(acc, ("%x_ptr", "%y_ptr", "%z_ptr")):
        assert text.startswith(arg + " offsets=[(1024 * pid.x)] strides=[1] " + dims), text
    assert "sizes=[1024]" in s and s.count("name=arith.addf") == 1
    assert " other" not in s  # tail lanes are left as they are: no fill


def test_softmax_structured_matches_reference_golden(native):
    # kernel-02-fused-softmax.mlir CHECK :46-75 (there with block 128): offsets [index_cast(pid*stride)],
    # dims = max(min(n_cols, BLOCK), 0), other = -inf on the load, none on the store.
    s = native.ttir_to_structured(golden_ttir("row_softmax"))
    (k0, ld), (k1, st) = accesses(s)
    assert (k0, k1) == ("load", "store")
    assert ld == "%in_ptr offsets=[(arg2 * pid.x)] strides=[1] dims=[max(0, min(1024, arg4))] other=-inf"
    assert st == "%out_ptr offsets=[(pid.x * arg3)] strides=[1] dims=[max(0, min(1024, arg4))]"
    names = re.findall(r"name=([\w.]+)", s)
    assert names == ["arith.maxnumf", "arith.subf", "math.exp", "arith.addf", "arith.divf"]


def test_matmul_structured_matches_reference_golden(native):
    # kernel-03-matrix-multiplication.mlir CHECK :155-190: loop-carried offsets, the K advance of both
    # operands lands in dimension 0 (a splat constant is an offset of the outermost dimension,
    # PtrAnalysis.cpp:1068-1100), strides [stride_am, 1] / [stride_bk, 1], 2-D store mask as a min per dim.
    s = native.ttir_to_structured(golden_ttir("matmul_tiles"))
    iters = re.findall(r"int_iter .*? ; (it0\.\d) = (.*) then (.*)$", s, re.M)
    by = {n: (init, nxt) for n, init, nxt in iters}
    assert by["it0.0"][1] == "(it0.0 + 64)" and by["it0.0"][0].startswith("(arg6 * (128 * ")   # A: row0*stride_am, += BK
    assert by["it0.1"] == ("0", "it0.1")
    assert by["it0.2"] == ("arg6", "it0.2") and by["it0.3"] == ("1", "it0.3")
    assert by["it0.4"] == ("0", "(it0.4 + (arg7 * 64))")                                      # B: += BK*stride_bk
    assert by["it0.5"][1] == "it0.5" and by["it0.6"] == ("arg7", "it0.6") and by["it0.7"] == ("1", "it0.7")
    acc = accesses(s)
    assert [k for k, _ in acc] == ["load", "load", "store"]
    assert "strides=[arg8, 1]" in acc[2][1]
    assert acc[2][1].count("min(128, ") == 2          # minsi(dim, 128) on both store dims (CHECK :188-189)
    assert "for loop=0" in s and "0 to ((63 + arg5) / 64) step 1" in s
    assert s.count(" dot ") == 1 and "name=arith.truncf" in s


def test_layernorm_structured(native):
    # kernel-05-layer-norm-fwd.mlir: three scf.for over column blocks, scalar stores of mean and rstd
    # at offset pid, masked loads padding with 0.
    s = native.ttir_to_structured(golden_ttir("layer_norm_fwd"))
    acc = accesses(s)
    assert [k for k, _ in acc] == ["load", "load", "scalar_store", "scalar_store", "load", "load", "load", "store"]
    assert acc[2][1].startswith("%Mean offsets=[pid.x]") and acc[3][1].startswith("%Rstd offsets=[pid.x]")
    assert acc[0][1] == "%X offsets=[((arg6 * pid.x) + iv0)] strides=[1] dims=[(max(iv0, min((iv0 + 1024), arg7)) - iv0)] other=0"
    assert acc[4][1].startswith("%W offsets=[iv2] strides=[1]") and "other" not in acc[4][1]
    assert s.count("for loop=") == 3 and s.count("0 to arg7 step 1024") == 3


def test_masked_2d_window_matches_reference_golden(native):
    # test/Conversion/TritonToStructured/masked_ldst_2d.mlir CHECK :75-98: sizes [128, 256],
    # strides [1, 1024], offsets [2, 3072], dims [min(max(min(rows,130),2)-2,128), min(max(min(cols,259),3)-3,256)],
    # other = -inf.
    import extra_kernels as X
    ttir = compile_ttir(X.masked_copy_2d, {"src": "*bf16", "dst": "*bf16", "rows": "i32", "cols": "i32"}, {})
    s = native.ttir_to_structured(ttir)
    (k0, ld), (k1, st) = accesses(s)
    assert "sizes=[128,256]" in s
    want = ("offsets=[2, 3072] strides=[1, 1024] "
            "dims=[min(128, (max(2, min(130, arg2)) - 2)), min(256, (max(3, min(259, arg3)) - 3))]")
    assert ld == "%src " + want + " other=-inf"
    assert st == "%dst " + want
    plan = native.PlanHandle(native.structured_to_plan(s)[0])
    assert plan.family == "tile_program"                   # a masked 2-D copy runs on the generic family


# ---------------------------------------------------------------- text form
@pytest.mark.parametrize("name", ["vec_add", "row_softmax", "layer_norm_fwd", "matmul_tiles", "matmul_wrapped", "w8a16_matmul"])
def test_family_and_signature(native, name):
    plan, structured = plan_for(native, name)
    want = {"vec_add": "map1d", "row_softmax": "row_softmax", "layer_norm_fwd": "layernorm_fwd",
            "matmul_tiles": "gemm", "matmul_wrapped": "gemm", "w8a16_matmul": "gemm_w8a16"}[name]
    assert plan.family == want and plan.kernel_name == name
    # the small-block variant has the same op structure, hence the same signature
    small, _ = plan_for(native, name + ".small")
    assert small.signature == plan.signature and small.family == want


def test_plan_bytes_are_self_contained(native):
    structured = native.ttir_to_structured(golden_ttir("row_softmax"))
    plan_bytes, name = native.structured_to_plan(structured)
    assert name == "row_softmax" and plan_bytes.startswith(b"tts.plan 1 family=row_softmax\n")
    with pytest.raises(ValueError):
        native.PlanHandle(b"garbage")
    with pytest.raises(ValueError, match="disagree"):
        native.PlanHandle(plan_bytes.replace(b"family=row_softmax", b"family=gemm", 1))


# ------------------------------------------------------------------ refusals
def test_unsupported_kernels_are_refused(native):
    import extra_kernels as X
    sig = {"src": "*fp32", "dst": "*fp32", "M": "i32", "BLOCK": "constexpr"}
    wrapped = native.ttir_to_structured(compile_ttir(X.wraparound_rows, sig, {"BLOCK": 64}))
    assert "wraps=[arg2]" in wrapped                       # the structured stage carries the period (tts.make_tptr shape)
    assert native.PlanHandle(native.structured_to_plan(wrapped)[0]).family == "tile_program"   # ... and the generic family runs it
    sig = {"src": "*fp32", "idx": "*i32", "dst": "*fp32", "BLOCK": "constexpr"}
    gathered = native.ttir_to_structured(compile_ttir(X.gather_rows, sig, {"BLOCK": 64}))
    assert "gather=" in gathered                           # data-dependent addresses: an unstructured access
    assert native.PlanHandle(native.structured_to_plan(gathered)[0]).family == "tile_program"
    sig = {"x_ptr": "*fp32", "out_ptr": "*fp32", "n": "i32", "BLOCK": "constexpr"}
    s = native.ttir_to_structured(compile_ttir(X.block_sum, sig, {"BLOCK": 256}))
    assert native.PlanHandle(native.structured_to_plan(s)[0]).family == "tile_program"      # a reduction outside softmax / LayerNorm
    with pytest.raises(NotImplementedError, match="tt.atomic_rmw"):
        native.ttir_to_structured(compile_ttir(X.atomic_accumulate, sig, {"BLOCK": 256}))
    dot_sig = {"a_ptr": "*fp32", "b_ptr": "*fp32", "c_ptr": "*fp32", "B": "constexpr"}
    s = native.ttir_to_structured(compile_ttir(X.small_dot, dot_sig, {"B": 32}))
    assert native.PlanHandle(native.structured_to_plan(s)[0]).family == "tile_program"      # a small product: generic family
    s = native.ttir_to_structured(compile_ttir(X.small_dot, dot_sig, {"B": 128}))
    with pytest.raises(NotImplementedError, match="bytes of LDS"):                            # a large one outside the matmul shapes
        native.structured_to_plan(s)
    with pytest.raises(NotImplementedError):
        native.ttir_to_structured("module {\n  tt.func public @k(%a: !tt.ptr<f32>) {\n    %0 = foo.bar %a : i32\n    tt.return\n  }\n}\n")


def test_operand_order_is_kept(native):
    import extra_kernels as X
    sig = {"x_ptr": "*fp32", "y_ptr": "*fp32", "z_ptr": "*fp32", "n": "i32", "BLOCK": "constexpr"}
    s = native.ttir_to_structured(compile_ttir(X.vec_sub_swapped, sig, {"BLOCK": 128}))
    plan = native.PlanHandle(native.structured_to_plan(s)[0])
    d = plan.describe_launch((4, 1, 1), [0, 0, 0, 500])
    assert d["kernel"] == "map1d_f32" and d["op"] == "1" and d["swap"] == "1" and d["block"] == "128"


# --------------------------------- bindings vs brute force (lane interpreter)
def affine(text, x, y=0, z=0):
    c0, cx, cy, cz = [int(v) for v in re.match(r"(-?\d+)\+(-?\d+)\*x\+(-?\d+)\*y\+(-?\d+)\*z", text).groups()]
    return c0 + cx * x + cy * y + cz * z


@pytest.mark.parametrize("n", [333, 64, 1, 640])
def test_map1d_binding_matches_every_lane(native, n):
    B = 64
    grid = (n + B - 1) // B + 1  # one extra, fully masked program
    plan, _ = plan_for(native, "vec_add.small")
    d = plan.describe_launch((grid, 1, 1), [0, 0, 0, n])
    x = np.zeros(n + 2 * B, np.float32)
    log = ttir_lanes.Interpreter(golden_ttir("vec_add.small")).run((grid,), [None, None, None, n],
                                                                     {0: x, 1: x.copy(), 2: x.copy()})
    for p, prog in enumerate(log):
        extent = int(np.clip(int(d["bound"]) - affine(d["m_start"], p), 0, int(d["block"])))
        for (kind, arg, offs), key in zip(prog, ("x_off", "y_off", "z_off")):
            start = affine(d[key], p)
            assert np.array_equal(offs, np.arange(start, start + extent)), (p, kind, arg)


def test_softmax_binding_matches_every_lane(native):
    plan, _ = plan_for(native, "row_softmax.small")
    rows, n_cols, pitch_in, pitch_out = 7, 50, 70, 60
    d = plan.describe_launch((rows, 1, 1), [0, 0, pitch_in, pitch_out, n_cols])
    o, x = np.zeros(rows * pitch_out, np.float32), np.ones(rows * pitch_in, np.float32)
    log = ttir_lanes.Interpreter(golden_ttir("row_softmax.small")).run(
        (rows,), [None, None, pitch_in, pitch_out, n_cols], {0: o, 1: x})
    assert d["other"] == "-inf" and d["block"] == "64"
    for p, ((k0, a0, ld), (k1, a1, st)) in enumerate(log):
        assert (a0, a1) == (1, 0)
        assert np.array_equal(ld, affine(d["in_off"], p) + np.arange(int(d["d_in"])))
        assert np.array_equal(st, affine(d["out_off"], p) + np.arange(int(d["d_out"])))
    # n_cols above the block is clamped, a negative one gives 0 (the max with start)
    assert plan.describe_launch((1, 1, 1), [0, 0, 70, 60, 1000])["d_in"] == "64"
    assert plan.describe_launch((1, 1, 1), [0, 0, 70, 60, -5])["d_in"] == "0"


def test_layernorm_binding_matches_every_lane(native):
    plan, _ = plan_for(native, "layer_norm_fwd.small")
    M, N, pitch = 3, 150, 160
    d = plan.describe_launch((M, 1, 1), [0] * 6 + [pitch, N, 1e-5])
    assert d["N"] == str(N) and abs(float(d["eps"]) - 1e-5) < 1e-12
    mem = {0: np.ones(M * pitch, np.float16), 1: np.zeros(M * pitch, np.float16), 2: np.ones(N, np.float16),
           3: np.ones(N, np.float16), 4: np.zeros(M, np.float32), 5: np.zeros(M, np.float32)}
    log = ttir_lanes.Interpreter(golden_ttir("layer_norm_fwd.small")).run((M,), [None] * 6 + [pitch, N, 1e-5], mem)
    for p, prog in enumerate(log):
        touched = {}
        for kind, arg, offs in prog:
            touched.setdefault((kind, arg), []).append(offs)
        row = np.arange(N)
        for (kind, arg), key in ((("load", 0), "x_off"), (("store", 1), "y_off"), (("load", 2), "w_off"),
                                 (("load", 3), "b_off")):
            got = np.unique(np.concatenate(touched[(kind, arg)]))
            assert np.array_equal(got, affine(d[key], p) + row), (p, kind, arg)
        assert touched[("store", 4)][0][0] == affine(d["mean_off"], p)
        assert touched[("store", 5)][0][0] == affine(d["rstd_off"], p)


@pytest.mark.parametrize("kernel", ["matmul_tiles.small", "matmul_wrapped.small"])
@pytest.mark.parametrize("shape", [(70, 90, 40), (32, 32, 16), (33, 1, 17)])
def test_gemm_binding_matches_every_lane(native, shape, kernel):
    # matmul_wrapped reads rows of A / columns of B modulo M / N (the stock tutorial form): the lanes it
    # touches are still exactly the dense operands, and the launcher binds it to the same dense problem
    M, N, K = shape
    plan, _ = plan_for(native, kernel)
    grid = ((M + 31) // 32) * ((N + 31) // 32)
    lda, ldb, ldc = K + 3, N + 5, N + 1
    d = plan.describe_launch((grid, 1, 1), [0, 0, 0, M, N, K, lda, ldb, ldc])
    assert (d["M"], d["N"], d["K"], d["lda"], d["ldb"], d["ldc"]) == tuple(str(v) for v in (M, N, K, lda, ldb, ldc))
    mem = {0: np.zeros(M * lda, np.uint16), 1: np.zeros(K * ldb, np.uint16), 2: np.zeros(M * ldc, np.uint16)}
    log = ttir_lanes.Interpreter(golden_ttir(kernel)).run(
        (grid,), [None, None, None, M, N, K, lda, ldb, ldc], mem)
    loads = {0: [], 1: []}
    stores = []
    for prog in log:
        for kind, arg, offs in prog:
            (stores if kind == "store" else loads[arg]).append(offs)
    dense = lambda r, c, ld: (np.arange(r)[:, None] * ld + np.arange(c)[None, :]).ravel()
    assert np.array_equal(np.unique(np.concatenate(loads[0])), dense(M, K, lda))
    assert np.array_equal(np.unique(np.concatenate(loads[1])), dense(K, N, ldb))
    all_stores = np.concatenate(stores)
    assert np.array_equal(np.sort(all_stores), dense(M, N, ldc))  # every element of C exactly once


def test_gemm_launches_the_product_kernels_decline_go_to_the_generic_family(native):
    # what the matrix-product family can only check at launch (the grid's shape, strides) does not end the launch:
    # the same program runs on the generic family's kernel, and the launch description says why
    plan, _ = plan_for(native, "matmul_tiles.small")
    d = plan.describe_launch((5, 1, 1), [0, 0, 0, 70, 90, 40, 40, 90, 90])
    assert d["kernel"] == "tile_program" and "one program per output tile" in d["fallback_reason"]
    # a pitch so large that BK * ldb wraps in 32 bits: the pointer advance is no longer one K block
    d = plan.describe_launch((9, 1, 1), [0, 0, 0, 70, 90, 40, 40, 2 ** 31 - 1, 90])
    assert d["kernel"] == "tile_program" and "advance" in d["fallback_reason"]
    # the ordinary launch stays on the product kernels
    d = plan.describe_launch((9, 1, 1), [0, 0, 0, 70, 90, 40, 40, 90, 90])
    assert d["kernel"] == "gemm_mfma" and d["a_trans"] == "0" and d["b_trans"] == "0"


def test_gemm_declines_negative_pitches(native):
    # a negative pitch of A or B would become an unsigned byte offset in the product kernels, and a pitch of C that is
    # not positive makes the rows of C overlap or run backwards: such launches go to the generic family's kernel
    plan, _ = plan_for(native, "matmul_tiles.small")
    for vals in ([0, 0, 0, 70, 90, 40, -40, 90, 90], [0, 0, 0, 70, 90, 40, 40, -90, 90], [0, 0, 0, 70, 90, 40, 40, 90, -90],
                 [0, 0, 0, 70, 90, 40, 40, 90, 0]):
        d = plan.describe_launch((9, 1, 1), vals)
        assert d["kernel"] == "tile_program" and "pitch" in d["fallback_reason"], (vals, d)
    d = plan.describe_launch((9, 1, 1), [0, 0, 0, 70, 90, 40, 0, 90, 90])    # a pitch of 0: one row of A for every row of C
    assert d["kernel"] == "gemm_mfma" and d["lda"] == "0"


def test_w8a16_binding(native):
    plan, _ = plan_for(native, "w8a16_matmul.small")
    M, N, K = 13, 70, 100
    d = plan.describe_launch((1, 3, 1), [0, 0, 0, 0, M, N, K, K, N, N])
    assert (d["M"], d["N"], d["K"], d["lda"], d["ldw"], d["ldc"]) == ("13", "70", "100", "100", "70", "70")
    d = plan.describe_launch((2, 3, 1), [0, 0, 0, 0, 20, N, K, K, N, N])   # beyond the decode shape: the same kernels, a launch per 16 rows
    assert d["kernel"] == "gemm_w8a16" and d["M"] == "20"
    # what the family can only decline at launch goes to the generic family's kernel: a pitch so large that BK * ldw wraps
    d = plan.describe_launch((1, 3, 1), [0, 0, 0, 0, M, N, K, K, 2 ** 31 - 1, N])
    assert d["kernel"] == "tile_program" and "fallback_reason" in d


def test_index_overflow_is_detected(native):
    plan, _ = plan_for(native, "row_softmax")
    # pid * in_pitch overflows i32 at the last program: the reference would wrap, so must we not assume linearity
    with pytest.raises(ValueError, match="overflow"):
        plan.describe_launch((4096, 1, 1), [0, 0, 2 ** 20, 781, 781])


def test_argument_checks(native):
    plan, _ = plan_for(native, "vec_add")
    with pytest.raises(ValueError, match="arguments"):
        plan.describe_launch((1, 1, 1), [0, 0, 0])
    assert plan.describe_launch((0, 1, 1), [0, 0, 0, 5]) == {"kernel": "none"}


# ------------------------------------------------------------------ gathers and scatters
def test_unstructured_accesses_keep_offsets_and_masks_as_data(native):
    """What PtrAnalysis cannot express stays a tensor of offsets (and a tensor mask) on the access; block values carried
    around loops, integer ones included, become loop-carried block arguments (StructuredToMemref.cpp:855-993,1034-1157)."""
    import extra_kernels as X
    s = native.ttir_to_structured(compile_ttir(X.gather_div12_masked_store, {"src": "*i32", "dst": "*i32"}, {}))
    loads = [l for l in s.splitlines() if l.strip().startswith("load ")]
    stores = [l for l in s.splitlines() if l.strip().startswith("store ")]
    assert len(loads) == 1 and len(stores) == 1
    assert "gather=" in loads[0] and "maskv=-1" not in loads[0] and "other_i=99" in loads[0]
    assert "gather=" in stores[0] and "maskv=-1" not in stores[0]
    assert s.count("tile_iter") == 2
    plan = native.PlanHandle(native.structured_to_plan(s)[0])
    assert plan.family == "tile_program"
    # a structured store next to a gathered load stays structured
    s = native.ttir_to_structured(compile_ttir(X.gather_div10, {"src": "*i32", "dst": "*i32"}, {}))
    store = [l for l in s.splitlines() if l.strip().startswith("store ")][0]
    assert "gather=" not in store and "strides=[1]" in store
    # a rank-1 index vector feeding a rank-2 gather
    sig = {"src": "*fp32", "dst": "*fp32", "rows": "*i32", "pitch_rows": "i32", "pitch_src": "i32", "pitch_dst": "i32", "period": "i32",
           "R": "constexpr", "C": "constexpr"}
    s = native.ttir_to_structured(compile_ttir(X.select_rows, sig, {"R": 4, "C": 16}))
    assert native.PlanHandle(native.structured_to_plan(s)[0]).family == "tile_program"


# ------------------------------------------------------------------ reductions and scans outside the hand-written families
def test_reductions_and_scans_lower_to_the_generic_family(native):
    import extra_kernels as X
    P, I = "*fp32", "*i32"
    sig = {"x_ptr": P, "max_ptr": I, "min_ptr": I, "n_cols": "i32", "pitch": "i32", "BC": "constexpr"}
    s = native.ttir_to_structured(compile_ttir(X.arg_extremes_rows, sig, {"BC": 256}))
    reduces = [l for l in s.splitlines() if l.strip().startswith("reduce ")]
    assert len(reduces) == 2 and all("name=region" in l and "region=1" in l for l in reduces)   # two operands, a combiner region
    assert s.count("region_arg") == 8 and s.count("region_result") == 4
    plan_bytes, _ = native.structured_to_plan(s)
    assert native.PlanHandle(plan_bytes).family == "tile_program"
    assert native.structured_to_plan(s)[0] == plan_bytes                                         # the text form round-trips
    sig = {"x_ptr": P, "y_ptr": P, "n": "i32", "BLOCK": "constexpr"}
    s = native.ttir_to_structured(compile_ttir(X.running_sum, sig, {"BLOCK": 1024}))
    assert "scan " in s and "name=arith.addf" in s
    assert native.PlanHandle(native.structured_to_plan(s)[0]).family == "tile_program"
    sig = {"x_ptr": P, "out_ptr": P, "n_rows": "i32", "n_cols": "i32", "pitch": "i32", "BR": "constexpr", "BC": "constexpr", "KIND": "constexpr"}
    s = native.ttir_to_structured(compile_ttir(X.reduce_rows_2d, sig, {"BR": 8, "BC": 128, "KIND": 0}))
    assert "reduce " in s and "axis=1" in s
    assert native.PlanHandle(native.structured_to_plan(s)[0]).family == "tile_program"
    # a block too large to stage is reduced by one thread per line; a scan of that size is refused with the reason
    big = native.structured_to_plan(native.ttir_to_structured(compile_ttir(X.reduce_rows_2d, sig, {"BR": 256, "BC": 128, "KIND": 0})))
    assert native.PlanHandle(big[0]).family == "tile_program"
    sig = {"x_ptr": P, "y_ptr": P, "n": "i32", "BLOCK": "constexpr"}
    with pytest.raises(NotImplementedError, match="a scan over a block of more than 16384 elements"):
        native.structured_to_plan(native.ttir_to_structured(compile_ttir(X.running_sum, sig, {"BLOCK": 32768})))


# ------------------------------------------------- the reference's lit inputs, all of them
_LIT = "/root/reference/test/Conversion"


def _lit_functions(text):
    """One module per public tt.func of a lit file (private functions go with every piece); comment lines dropped."""
    lines = [l for l in text.splitlines() if not l.lstrip().startswith("//")]
    funcs, i = [], 0
    while i < len(lines):
        if not lines[i].lstrip().startswith("tt.func"):
            i += 1
            continue
        j, depth, seen = i, 0, False
        while True:
            depth += lines[j].count("{") - lines[j].count("}")
            seen = seen or "{" in lines[j]
            if seen and depth <= 0:
                break
            j += 1
        funcs.append("\n".join(lines[i:j + 1]))
        i = j + 1
    private = [f for f in funcs if "private" in f.split("@")[0]]
    return ["module {\n" + "\n".join([f] + private) + "\n}" for f in funcs if "private" not in f.split("@")[0]]


@pytest.mark.skipif(not __import__("os").path.isdir(_LIT), reason="the reference tree is not here")
def test_reference_lit_inputs_plan_or_are_refused_for_a_known_reason(native):
    """Every tt.func in the reference's conversion tests (test/Conversion/*/*.mlir, hand-written IR included) goes through
    the reader, the analyses and the planner.  What is refused is refused for one of the reasons listed here, each with
    the number of functions it may account for; anything else, or more of the same, fails."""
    import collections
    import glob
    known = {  # reason (prefix) -> functions
        "tensor-typed kernel argument": 18,                       # blocks of pointers as arguments: no launcher can pass them
        "operation tensor.empty": 9,                              # tensor dialect ops written by hand into triton_assert.mlir
        "tt.func with results is not a kernel": 6,
        "tile_program: a loop-carried block value of more than 32768 elements": 3,   # 256 x 256 accumulators in one program (kernel-05-layer-norm-dwdb.mlir)
        "tile_program: an argument is both stored to and read by a load that is not": 4,   # dot.mlir: the [128, 256] accumulator is read from the tensor the result goes to
        "tile_program: elementwise op extern.some_symbol": 3,     # the reference refuses it too (unsupported_extern_elementwise.mlir)
        "pointer-valued operation": 7,                            # int_to_ptr / cat on pointers (the reference's TritonToPtr fallback)
        "scalar integer operation tt.ptr_to_int": 1,              # cast_with_int_ptr.mlir: addresses as integers
        "pointer cast that changes the element width": 2,         # i32 <-> i64 / i8 views of one buffer: every offset would be rescaled
        "scalar pointer produced by arith.select": 1,             # a choice between two arguments (mixed_structured_unstructured.mlir)
        "unsupported type 'f8E4M3FN'": 1,
        "unsupported type '[": 3,                                 # tts / memref dialect inputs of later stages
        "unsupported type '}'": 1,
    }
    planned, refused = 0, collections.Counter()
    for path in sorted(glob.glob(_LIT + "/*/*.mlir")):
        text = open(path).read()
        if "tt.func" not in text:
            continue
        for module in _lit_functions(text):
            try:
                native.PlanHandle(native.structured_to_plan(native.ttir_to_structured(module))[0])
                planned += 1
            except NotImplementedError as e:
                why = next((k for k in known if k in str(e)), None)
                assert why is not None, (path, str(e)[:300])
                refused[why] += 1
    for why, n in refused.items():
        assert n <= known[why], (why, n)
    assert planned >= 345, (planned, dict(refused))


def test_block_pointer_ops_plan_and_agree_with_the_frontend_rewrite(native):
    """tt.make_tensor_ptr / tt.advance / boundaryCheck + padding as ops (raw_block_pointers=True keeps them; the lit inputs
    block_ptr_advance.mlir, block_ptr_complex_offset.mlir, make_tensor_ptr*.mlir hold the same forms): the program plans,
    and the lane interpreter gives the same memory image for the raw ops as for what the frontend's rewrite to plain
    pointer arithmetic makes of the same kernel - which pins the interpreter's reading of the ops on the frontend's."""
    import numpy as np
    import extra_kernels as X
    from oracle import ttir_lanes
    sig = {"a_ptr": "*bf16", "b_ptr": "*bf16", "c_ptr": "*fp32", "M": "i32", "N": "i32", "K": "i32", "sam": "i32", "sbk": "i32",
           "scm": "i32", "BM": "constexpr", "BN": "constexpr", "BK": "constexpr", "PAD": "constexpr"}
    rng = np.random.default_rng(1)
    for pad, (M, N, K) in [("zero", (40, 50, 24)), ("nan", (40, 50, 32)), ("nan", (33, 20, 24))]:
        a = (rng.integers(-2, 3, M * K).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
        b = (rng.integers(-2, 3, K * N).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
        images = []
        for raw in (False, True):
            ttir = compile_ttir(X.block_ptr_matmul, sig, {"BM": 32, "BN": 32, "BK": 16, "PAD": pad}, raw_block_pointers=raw)
            assert ("tt.make_tensor_ptr" in ttir) == raw and ("tt.advance" in ttir) == raw
            plan = native.structured_to_plan(native.ttir_to_structured(ttir))[0]
            assert plan.startswith(b"tts.plan 1 family=tile_program")
            c = np.full(M * N, -7, np.float32)
            ttir_lanes.Interpreter(ttir).run((2, 2), [None, None, None, M, N, K, K, N, N], {0: a.copy(), 1: b.copy(), 2: c})
            images.append(c)
        assert np.array_equal(images[0], images[1], equal_nan=True)
        if K % 16 == 0:          # no padding inside the products: the plain product, NaN padding or not
            want = (a.astype(np.uint32) << 16).view(np.float32).reshape(M, K) @ (b.astype(np.uint32) << 16).view(np.float32).reshape(K, N)
            assert np.array_equal(images[1].reshape(M, N), want)
        elif pad == "nan":       # K tiles stick out of A: NaN-padded columns meet zero-padded rows of B, NaN everywhere
            assert np.isnan(images[1]).all()


def test_every_functional_case_plans(native):
    """The kernels of tests/reference_cases.py and tests/core_cases.py (run on the GPU by the gpu tests, on the lane oracle by
    test_oracle_pins.py) all get a plan here, without a GPU; the structured text survives a round trip through its reader."""
    import core_cases
    import core_kernels
    import extra_kernels
    import reference_cases
    families = set()
    for cases, kernels in ((reference_cases.cases(), extra_kernels), (core_cases.cases(), core_kernels)):
        for case in cases:
            text = native.ttir_to_structured(compile_ttir(getattr(kernels, case["kernel"]), case["sig"], case["consts"]))
            plan_bytes, _names = native.structured_to_plan(text)
            families.add(native.PlanHandle(plan_bytes).family)
    assert families == {"tile_program", "fused_map"}, families


def _generic_source(tmp_path, ttir):
    """HIP source of the generic family's kernel for a program, from the tts-opt tool."""
    import os
    import subprocess
    from conftest import ROOT
    f = tmp_path / "k.ttir"
    f.write_text(ttir)
    res = subprocess.run([os.path.join(ROOT, "triton-shared_amd", "csrc", "tts-opt"), "--source", str(f)], text=True, capture_output=True)
    assert res.returncode == 0, res.stderr
    return res.stdout


def test_memory_effects_keep_their_order_inside_a_program(native, tmp_path):
    import extra_kernels as X
    # a load after a store to the same argument: the vectorised map (all loads first) must decline, and the generic
    # family must start a new phase at that load, behind a barrier
    sig = {"p_ptr": "*fp32", "q_ptr": "*fp32", "n": "i32", "BLOCK": "constexpr"}
    ttir = compile_ttir(X.double_in_place_then_square, sig, {"BLOCK": 1024})
    plan = native.PlanHandle(native.structured_to_plan(native.ttir_to_structured(ttir))[0])
    assert plan.family == "tile_program"
    body = _generic_source(tmp_path, ttir)
    stores = [m.start() for m in re.finditer(r"\(\(float \*\)p\.ptr\[\d\]\)\[[^;]*\] = ", body)]
    loads = [m.start() for m in re.finditer(r"ld\d+\[n\] = \(\(const float \*\)p\.ptr\[0\]\)", body)]
    assert len(stores) == 2 and len(loads) == 2, body
    assert loads[0] < stores[0] < loads[1] < stores[1]                      # program order
    assert "__syncthreads();" in body[stores[0]:loads[1]]                   # and a barrier between the store and the re-load
    # scalar read-modify-write of one address: barriers keep thread 0's store apart from the other threads' reads
    sig = {"acc_ptr": "*i32", "out_ptr": "*i32", "BLOCK": "constexpr"}
    ttir = compile_ttir(X.bump_counter_and_report, sig, {"BLOCK": 1024})
    assert native.PlanHandle(native.structured_to_plan(native.ttir_to_structured(ttir))[0]).family == "tile_program"
    body = _generic_source(tmp_path, ttir)
    first_read = body.index("const int s")
    write = body.index("if (threadIdx.x == 0")
    second_read = body.index("const int s", write)
    assert first_read < write < second_read
    assert "__syncthreads();" in body[first_read:write] and "__syncthreads();" in body[write:second_read]


def test_generic_source_asks_for_a_swapped_grid_when_program_id_1_walks_the_contiguous_dimension(native, tmp_path):
    # tiles of a row-major matrix with rows on program_id(0) and columns on program_id(1): the hardware starts workgroups
    # along x first, so the launcher is asked to exchange x and y (the mark at the top of the source).  A transpose, whose
    # stores are contiguous along what program_id(0) walks, is left as it is.
    import extra_kernels as X
    sig = {"out_ptr": "*i32", "R": "i32", "C": "i32", "BR": "constexpr", "BC": "constexpr"}
    body = _generic_source(tmp_path, compile_ttir(X.stamp_tiles, sig, {"BR": 32, "BC": 256}))
    assert body.startswith("// tts: swap_xy\n") and "swap_xy ? blockIdx.y : blockIdx.x" in body
    sig = {"src": "*fp32", "dst": "*fp32", "R": "i32", "C": "i32", "BR": "constexpr", "BC": "constexpr"}
    body = _generic_source(tmp_path, compile_ttir(X.transpose_tiles, sig, {"BR": 64, "BC": 64}))
    assert not body.startswith("// tts: swap_xy")


def test_declined_details_of_a_handwritten_family_fall_through(native):
    import extra_kernels as X
    from triton_shared_amd.examples import kernels as K
    # the op structure of the two-input map in fp16 / bf16: the fused map takes it
    for t in ("fp16", "bf16"):
        sig = {"x_ptr": "*" + t, "y_ptr": "*" + t, "z_ptr": "*" + t, "n": "i32", "BLOCK": "constexpr"}
        text = native.ttir_to_structured(compile_ttir(K.vec_add, sig, {"BLOCK": 1024}))
        assert native.PlanHandle(native.structured_to_plan(text)[0]).family == "fused_map"
    # a softmax whose input row is strided, and one whose rows are longer than the row kernel holds: the generic family
    sig = {"out_ptr": "*fp32", "in_ptr": "*fp32", "in_pitch": "i32", "out_pitch": "i32", "col_stride": "i32", "n_cols": "i32", "BLOCK": "constexpr"}
    text = native.ttir_to_structured(compile_ttir(X.strided_row_softmax, sig, {"BLOCK": 1024}))
    assert native.PlanHandle(native.structured_to_plan(text)[0]).family == "tile_program"
    sig = {"out_ptr": "*fp32", "in_ptr": "*fp32", "in_pitch": "i32", "out_pitch": "i32", "n_cols": "i32", "BLOCK": "constexpr"}
    text = native.ttir_to_structured(compile_ttir(K.row_softmax, sig, {"BLOCK": 131072}))
    assert native.PlanHandle(native.structured_to_plan(text)[0]).family == "tile_program"
    text = native.ttir_to_structured(compile_ttir(K.row_softmax, sig, {"BLOCK": 65536}))
    assert native.PlanHandle(native.structured_to_plan(text)[0]).family == "row_softmax"


def test_gemm_binds_column_major_operands(native):
    from triton_shared_amd.examples import kernels as K
    # the tutorial's b.T: stride_bk == 1 is specialised to a constant and stride_bn is the pitch
    sig = {"a_ptr": "*bf16", "b_ptr": "*bf16", "c_ptr": "*bf16", "M": "i32", "N": "i32", "K": "i32", "s_am": "i32", "s_ak": "constexpr",
           "s_bk": "constexpr", "s_bn": "i32", "s_cm": "i32", "s_cn": "constexpr", "BM": "constexpr", "BN": "constexpr", "BK": "constexpr",
           "GROUP_M": "constexpr"}
    text = native.ttir_to_structured(compile_ttir(K.matmul_tiles, sig, {"s_ak": 1, "s_bk": 1, "s_cn": 1, "BM": 128, "BN": 128, "BK": 64, "GROUP_M": 8}))
    plan = native.PlanHandle(native.structured_to_plan(text)[0])
    assert plan.family == "gemm"
    d = plan.describe_launch((4 * 3, 1, 1), [0, 0, 0, 512, 384, 200, 208, 216, 392])
    assert (d["kernel"], d["a_trans"], d["b_trans"], d["lda"], d["ldb"], d["ldc"]) == ("gemm_mfma", "0", "1", "208", "216", "392")
    # both strides of B run-time values, neither of them 1: the generic family
    sig["s_bk"] = "i32"
    text = native.ttir_to_structured(compile_ttir(K.matmul_tiles, sig, {"s_ak": 1, "s_cn": 1, "BM": 128, "BN": 128, "BK": 64, "GROUP_M": 8}))
    plan = native.PlanHandle(native.structured_to_plan(text)[0])
    d = plan.describe_launch((4 * 3, 1, 1), [0, 0, 0, 512, 384, 200, 208, 2, 432, 392])
    assert d["kernel"] == "tile_program" and "neither stride of B is 1" in d["fallback_reason"]


def test_gathered_rows_matmul_binds_to_the_matrix_product_family(native):
    # the mixture-of-experts product (rows of A through an index vector, the weight matrix of a block of rows picked by an
    # id read from memory; test/Conversion/TritonToUnstructured/unstructured_ptr_used_in_loop.mlir has this shape)
    import extra_kernels as X
    from triton_shared_amd.examples import kernels as K
    sig = {"a_ptr": "*bf16", "b_ptr": "*bf16", "c_ptr": "*bf16", "rows_ptr": "*i32", "expert_ptr": "*i32", "n_rows": "i32", "K": "i32", "N": "i32",
           "s_am": "i32", "s_be": "i32", "s_bk": "i32", "s_cm": "i32", "BM": "constexpr", "BN": "constexpr", "BK": "constexpr"}
    for fn in (K.expert_rows_matmul, X.grouped_rows_matmul):
        text = native.ttir_to_structured(compile_ttir(fn, sig, {"BM": 128, "BN": 128, "BK": 64}))
        plan = native.PlanHandle(native.structured_to_plan(text)[0])
        assert plan.family == "gemm"
        tokens, kd, nd = 300, 150, 256
        vals = [0, 0, 0, 0, 0, tokens, kd, nd, kd + 2, kd * nd, nd + 8, nd + 16]
        d = plan.describe_launch((3, 2, 1), vals)
        assert (d["kernel"], d["gathered"], d["M"], d["N"], d["K"], d["lda"], d["ldb"], d["ldc"], d["block_rows"], d["block_stride"]) == \
               ("gemm_mfma", "1", "300", "256", "150", str(kd + 2), str(nd + 8), str(nd + 16), "128", str(kd * nd))
        # a grid that is not one program per tile: the generic family's kernel for the same program
        d = plan.describe_launch((2, 2, 1), vals)
        assert d["kernel"] == "tile_program" and "one program per output tile" in d["fallback_reason"]
    # blocks of rows smaller than the kernel's tile, and fp32 data: the generic family from the start
    text = native.ttir_to_structured(compile_ttir(K.expert_rows_matmul, sig, {"BM": 64, "BN": 128, "BK": 64}))
    assert native.PlanHandle(native.structured_to_plan(text)[0]).family == "tile_program"
    sig32 = {k: (v.replace("bf16", "fp32")) for k, v in sig.items()}
    text = native.ttir_to_structured(compile_ttir(K.expert_rows_matmul, sig32, {"BM": 32, "BN": 32, "BK": 32}))
    assert native.PlanHandle(native.structured_to_plan(text)[0]).family == "tile_program"


def test_batched_matmul_and_carried_scalars_plan(native):
    """A batch index on another grid axis leaves the matmul in its family (the launcher proves the batch's structure
    from the arguments); a loop that carries a running maximum and sum as scalars is a generic program whose source
    keeps them in one variable per thread."""
    from triton_shared_amd.examples import kernels as K
    import extra_kernels as X
    sig = {"a_ptr": "*bf16", "b_ptr": "*bf16", "c_ptr": "*bf16", "M": "i32", "N": "i32", "K": "i32", "s_ab": "i32", "s_am": "i32", "s_bb": "i32",
           "s_bk": "i32", "s_cb": "i32", "s_cm": "i32", "BM": "constexpr", "BN": "constexpr", "BK": "constexpr"}
    s = native.ttir_to_structured(compile_ttir(K.batched_matmul, sig, {"BM": 128, "BN": 128, "BK": 64}))
    assert native.PlanHandle(native.structured_to_plan(s)[0]).family == "gemm"
    sig = {"x_ptr": "*fp32", "y_ptr": "*fp32", "cnt_ptr": "*i32", "stride": "i32", "N": "i32", "BLOCK": "constexpr"}
    s = native.ttir_to_structured(compile_ttir(X.softmax_row_in_pieces, sig, {"BLOCK": 1024}))
    plan = native.PlanHandle(native.structured_to_plan(s)[0])
    assert plan.family == "tile_program"
    # `while`: a counted loop with an exit (an If without a body, ival = 2) that dead-code elimination keeps
    sig = {"x_ptr": "*fp32", "out_ptr": "*fp32", "cnt_ptr": "*i32", "stride": "i32", "n": "i32", "limit": "fp32", "BLOCK": "constexpr"}
    s = native.ttir_to_structured(compile_ttir(X.while_sum_until, sig, {"BLOCK": 256}))
    assert "ub=" in s and "2147483647" in s and "ival=2" in s
    assert native.PlanHandle(native.structured_to_plan(s)[0]).family == "tile_program"
