"""Inputs and closed-form expectations for tests/core_kernels.py, in the format of reference_cases.py:
(kernel name, signature, constexprs, grid, argument builder, checker).  The expectations are numpy
expressions of the language definition, never a run of the code under test; both the lane-level
oracle (CPU) and the GPU backend go through the same cases."""
import math

import numpy as np

I, P, H = "*i32", "*fp32", "*fp16"
C = "constexpr"


def _eq(got, want):
    got, want = np.asarray(got), np.asarray(want)
    assert got.shape == want.shape and np.array_equal(got, want, equal_nan=got.dtype.kind == "f"), (got.ravel()[:16].tolist(), want.ravel()[:16].tolist())


def _bits_eq(got, want):
    got, want = np.asarray(got), np.asarray(want)
    assert got.dtype == want.dtype and np.array_equal(got.view(f"u{got.itemsize}"), want.view(f"u{want.itemsize}")), (got.ravel()[:16].tolist(), want.ravel()[:16].tolist())


def _close(got, want, tol):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    assert np.allclose(got, want, rtol=tol, atol=tol, equal_nan=True), float(np.nanmax(np.abs(got - want)))


def bf16_bits(x):
    """float32 -> bfloat16 storage (uint16), round to nearest even."""
    u = np.asarray(x, np.float32).view(np.uint32).astype(np.uint64)
    return (((u + 0x7FFF + ((u >> 16) & 1)) >> 16) & 0xFFFF).astype(np.uint16)


def cases():
    out = []

    def add(name, kernel, sig, consts, grid, args, check):
        out.append(dict(name=name, kernel=kernel, sig=sig, consts=consts, grid=grid, args=args, check=check))

    rng = np.random.default_rng(11)

    # umulhi: the high word of the unsigned 64-bit product
    ux = rng.integers(0, 1 << 32, 256, dtype=np.uint64).astype(np.uint32)
    uy = rng.integers(0, 1 << 32, 256, dtype=np.uint64).astype(np.uint32)
    ux[:4] = [0, 0xFFFFFFFF, 0xFFFFFFFF, 0x80000000]
    uy[:4] = [5, 0xFFFFFFFF, 1, 2]
    add("umulhi", "umulhi_pairs", {"x_ptr": "*u32", "y_ptr": "*u32", "out_ptr": "*u32", "BLOCK": C}, {"BLOCK": 256}, (1,),
        lambda: [ux.copy(), uy.copy(), np.zeros(256, np.uint32)],
        lambda a: _eq(a[2], ((ux.astype(np.uint64) * uy.astype(np.uint64)) >> 32).astype(np.uint32)))

    # loop induction variable in 64 bits, several steps
    for lo, hi, step in [(0, 10, 1), (2 ** 35, 2 ** 35 + 20, 2), (2 ** 35, 2 ** 35 + 20, 3), (-7, 30, 4)]:
        add(f"for_iv_{lo}_{step}", "sum_of_loop_indices", {"out_ptr": "*i64", "lo": "i64", "hi": "i64", "STEP": C}, {"STEP": step}, (1,),
            lambda lo=lo, hi=hi: [np.zeros(1, np.int64), lo, hi],
            lambda a, lo=lo, hi=hi, step=step: _eq(a[0], [sum(range(lo, hi, step))]))

    # calls: an inlined helper, then functions kept out of line: a store inside, a call graph, a branch around calls,
    # a tile product inside, two results
    tile = rng.integers(-2, 3, (16, 16)).astype(np.float32)
    for kind, x, y, want in [(0, 3.0, 4.0, [10.0, 0.0]), (1, 3.0, 4.0, [7.0, 0.0]), (2, 3.0, 4.0, [10.0, 0.0]), (3, 3.0, 4.0, [8.0, 0.0]),
                             (3, -3.0, 4.0, [3.0, 0.0]), (5, 3.0, 4.0, [7.0, -1.0])]:
        add(f"call_kind{kind}_{x}", "calls_helpers", {"x_ptr": P, "y_ptr": P, "dst_ptr": P, "KIND": C}, {"KIND": kind}, (1,),
            lambda x=x, y=y: [np.full(1, x, np.float32), np.full(1, y, np.float32), np.zeros(2, np.float32)], lambda a, want=want: _eq(a[2], want))
    add("call_kind4_tile", "calls_helpers", {"x_ptr": P, "y_ptr": P, "dst_ptr": P, "KIND": C}, {"KIND": 4}, (1,),
        lambda: [np.full(1, 3, np.float32), np.full(1, 4, np.float32), tile.reshape(-1).copy()], lambda a: _eq(a[2].reshape(16, 16), tile @ tile + 7))

    # indexing with new axes
    xi = rng.integers(0, 90, 32).astype(np.int32)

    def check_index(a):
        _eq(a[1].reshape(32, 32), xi[:, None] * 100 + xi[None, :])
        _eq(a[2].reshape(2, 32, 4), xi[None, :, None] + (np.arange(2) * 1000)[:, None, None] + (np.arange(4) * 100000)[None, None, :])
    add("index_new_axes", "index_with_new_axes", {"x_ptr": I, "z2_ptr": I, "z3_ptr": I, "N": C, "A": C, "C": C}, {"N": 32, "A": 2, "C": 4}, (1,),
        lambda: [xi.copy(), np.zeros(32 * 32, np.int32), np.zeros(2 * 32 * 4, np.int32)], check_index)

    # tl.full in every storage type
    def check_full(a):
        _eq(a[0], np.full(64, -7, np.int8)); _eq(a[1], np.full(64, -300, np.int16)); _eq(a[2], np.full(64, 1 << 20, np.int32))
        _eq(a[3], np.full(64, -(1 << 40), np.int64)); _eq(a[4], np.full(64, 200, np.uint8))
        _eq(a[5], np.full(64, 0.333251953125, np.float16)); _eq(a[6], np.full(64, bf16_bits(-2.5), np.uint16))
        _eq(a[7], np.full(64, 3.1415927410125732, np.float32)); _eq(a[8], np.full(64, math.e, np.float64))
    add("full", "fill_constants", {"i8_ptr": "*i8", "i16_ptr": "*i16", "i32_ptr": "*i32", "i64_ptr": "*i64", "u8_ptr": "*u8", "f16_ptr": "*fp16",
                                    "bf16_ptr": "*bf16", "f32_ptr": "*fp32", "f64_ptr": "*fp64", "BLOCK": C}, {"BLOCK": 64}, (1,),
        lambda: [np.zeros(64, t) for t in (np.int8, np.int16, np.int32, np.int64, np.uint8, np.float16, np.uint16, np.float32, np.float64)], check_full)

    # double precision: IEEE operations are exact to the bit; the block sum is compared within rounding of its length
    dx, dy = rng.standard_normal(700), rng.standard_normal(700) + 3.0
    ds = rng.standard_normal(700).astype(np.float32)

    def check_f64(a):
        o = a[3].reshape(7, 700)
        want = [dx + dy * 0.5, dx / dy, np.sqrt(np.abs(dx)), np.maximum(dx, dy), ds.astype(np.float64) * dx, np.where(dx > dy, dx, -dy),
                np.trunc(dx * 1000.0)]
        for got, w in zip(o, want):
            _bits_eq(got, w)
        sums = [dx[b * 256:(b + 1) * 256].sum() for b in range(3)]
        _close(a[4], sums, 1e-13)
    add("f64_ops", "double_precision_ops", {"x_ptr": "*fp64", "y_ptr": "*fp64", "s_ptr": P, "out_ptr": "*fp64", "sum_ptr": "*fp64", "k": "fp32", "n": "i32", "BLOCK": C},
        {"BLOCK": 256}, (3,), lambda: [dx.copy(), dy.copy(), ds.copy(), np.zeros(7 * 700), np.zeros(3), 0.5, 700], check_f64)

    add("empty_kernel", "does_nothing", {"x_ptr": I, "SIZE": C}, {"SIZE": 32}, (3,),
        lambda: [np.arange(4, dtype=np.int32)], lambda a: _eq(a[0], np.arange(4)))

    for mode, flag, want in [(0, 1, [1, -1]), (0, 0, [2, -1]), (1, 3, [1, -1]), (1, -9, [3, -1]), (1, -2, [-1, 4])]:
        add(f"if_return_{mode}_{flag}", "return_inside_if", {"flag_ptr": I, "out_ptr": I, "MODE": C}, {"MODE": mode}, (1,),
            lambda flag=flag: [np.full(1, flag, np.int32), np.full(2, -1, np.int32)], lambda a, want=want: _eq(a[1], want))

    # minimum / maximum / clamp: NaN lost by default, kept with propagate_nan=ALL
    nan = np.float32("nan")
    mx = np.array([1, nan, 3, nan, -0.0, 0.0, -2, 5] * 16, np.float32)
    my = np.array([2, 1, nan, nan, 0.0, -0.0, -3, 0.5] * 16, np.float32)

    def check_nan(a):
        o = a[2].reshape(6, 128)
        _eq(o[0], np.fmin(mx, my)); _eq(o[1], np.fmax(mx, my)); _eq(o[2], np.minimum(mx, my)); _eq(o[3], np.maximum(mx, my))
        _eq(o[4], np.fmin(np.fmax(mx, np.float32(-1)), np.float32(1))); _eq(o[5], np.minimum(np.maximum(mx, np.float32(-1)), np.float32(1)))
    add("propagate_nan", "min_max_nan_rules", {"x_ptr": P, "y_ptr": P, "out_ptr": P, "BLOCK": C}, {"BLOCK": 128}, (1,),
        lambda: [mx.copy(), my.copy(), np.zeros(6 * 128, np.float32)], check_nan)

    cx = rng.standard_normal(1000).astype(np.float32) * 3
    clo = -np.abs(rng.standard_normal(1000)).astype(np.float32)
    chi = np.abs(rng.standard_normal(1000)).astype(np.float32)
    add("clamp", "clamp_between_blocks", {"x_ptr": P, "lo_ptr": P, "hi_ptr": P, "out_ptr": P, "n": "i32", "BLOCK": C}, {"BLOCK": 256}, (4,),
        lambda: [cx.copy(), clo.copy(), chi.copy(), np.zeros(1000, np.float32), 1000], lambda a: _eq(a[3], np.clip(cx, clo, chi)))

    p3 = rng.standard_normal((4, 8, 16)).astype(np.float32)
    add("permute_3d", "permute_3d", {"src_ptr": P, "dst_ptr": P, "A": C, "B": C, "C": C}, {"A": 4, "B": 8, "C": 16}, (1,),
        lambda: [p3.reshape(-1).copy(), np.zeros(p3.size, np.float32)], lambda a: _eq(a[1].reshape(16, 4, 8), p3.transpose(2, 0, 1)))
    for shape in [(2, 2, 8, 64), (4, 4, 4, 16), (1, 8, 2, 32)]:
        p4 = rng.standard_normal(shape).astype(np.float32)
        add("permute_4d_" + "x".join(map(str, shape)), "permute_4d_block_ptr", {"src_ptr": P, "dst_ptr": P, "S0": C, "S1": C, "S2": C, "S3": C},
            dict(zip(("S0", "S1", "S2", "S3"), shape)), (1,),
            lambda p4=p4: [p4.reshape(-1).copy(), np.zeros(p4.size, np.float32)], lambda a, p4=p4: _eq(a[1], p4.transpose(3, 1, 0, 2).reshape(-1)))

    bx = rng.standard_normal(32).astype(np.float32)
    by = rng.standard_normal((32, 32)).astype(np.float32)
    add("broadcast", "broadcast_pair", {"x_ptr": P, "y_ptr": P, "out_ptr": P, "M": C, "N": C}, {"M": 32, "N": 32}, (1,),
        lambda: [bx.copy(), by.reshape(-1).copy(), np.zeros(32 * 32, np.float32)],
        lambda a: _eq(a[2].reshape(32, 32), (bx[:, None] * np.float32(2) + by) + bx[None, :] * np.float32(3)))

    add("dot_without_load", "dot_of_constants", {"out_ptr": P, "B": C}, {"B": 32}, (1,),
        lambda: [np.zeros(32 * 32, np.float32)], lambda a: _eq(a[0], np.full(32 * 32, 48.0, np.float32)))

    # small integers in float: every product and partial sum is exact, so any summation order gives the same bits
    da = rng.integers(-4, 5, (16, 32)).astype(np.float32)
    db = rng.integers(-4, 5, (32, 16)).astype(np.float32)
    add("dot_mulbroadcasted", "product_by_broadcast_and_sum", {"a_ptr": P, "b_ptr": P, "c_ptr": P, "M": C, "N": C, "K": C}, {"M": 16, "N": 16, "K": 32}, (1,),
        lambda: [da.reshape(-1).copy(), db.reshape(-1).copy(), np.zeros(16 * 16, np.float32)], lambda a: _eq(a[2].reshape(16, 16), da @ db))

    sv = np.arange(10, 18, dtype=np.float32)
    for index, want in [(3, 13.0), (8, -5.0), (100, -5.0)]:
        add(f"masked_load_scalar_{index}", "scalar_load_under_mask", {"src_ptr": P, "dst_ptr": P, "index": "i32", "n": "i32", "OTHER": C}, {"OTHER": -5.0}, (1,),
            lambda index=index: [sv.copy(), np.zeros(1, np.float32), index, 8], lambda a, want=want: _eq(a[1], [want]))

    for order in (0, 1):
        for size in (1, 128):
            ap = rng.standard_normal(size).astype(np.float32)
            add(f"addptr_order{order}_size{size}", "copy_with_offsets_first", {"x_ptr": P, "y_ptr": P, "ORDER": C, "SIZE": C}, {"ORDER": order, "SIZE": size}, (1,),
                lambda ap=ap: [ap.copy(), np.zeros(ap.size, np.float32)], lambda a, ap=ap: _eq(a[1], ap))

    for flag, want in [(3, [7, -1]), (-3, [-1, 8])]:
        add(f"masked_store_scalar_{flag}", "scalar_store_under_mask", {"dst_ptr": I, "flag": "i32", "value": "i32"}, {}, (1,),
            lambda flag=flag: [np.full(2, -1, np.int32), flag, 7], lambda a, want=want: _eq(a[0], want))

    fx, fy, fz = (rng.standard_normal(256).astype(np.float32) for _ in range(3))
    fx[0], fy[0], fz[0] = np.float32(1 + 2 ** -12), np.float32(1 + 2 ** -12), np.float32(-1)     # the product's low bits survive only when fused
    add("fma", "fused_multiply_add", {"x_ptr": P, "y_ptr": P, "z_ptr": P, "out_ptr": P, "BLOCK": C}, {"BLOCK": 256}, (1,),
        lambda: [fx.copy(), fy.copy(), fz.copy(), np.zeros(256, np.float32)],
        lambda a: _eq(a[3], (fx.astype(np.float64) * fy.astype(np.float64) + fz.astype(np.float64)).astype(np.float32)))

    cs = rng.standard_normal(700).astype(np.float32)
    add("const_pointer", "copy_from_const", {"src_ptr": "*kfp32", "dst_ptr": P, "n": "i32", "BLOCK": C}, {"BLOCK": 256}, (3,),
        lambda: [cs.copy(), np.zeros(700, np.float32), 700], lambda a: _eq(a[1], cs))

    for start in (0, 1, 7, 16):
        add(f"arange_{start}", "arange_from", {"out_ptr": I, "START": C, "BLOCK": C}, {"START": start, "BLOCK": 128}, (1,),
            lambda: [np.zeros(128, np.int32)], lambda a, start=start: _eq(a[0], np.arange(start, start + 128)))

    halves = np.arange(1 << 16, dtype=np.uint16).view(np.float16)             # every fp16 value: subnormals, infinities, NaNs
    add("fp16_to_fp32_all_values", "widen_halves", {"src_ptr": H, "dst_ptr": P, "BLOCK": C}, {"BLOCK": 1024}, (64,),
        lambda: [halves.copy(), np.zeros(1 << 16, np.float32)], lambda a: _eq(a[1], halves.astype(np.float32)))

    ai = rng.integers(-1000, 1000, 128).astype(np.int32)
    af = rng.standard_normal(128).astype(np.float32); af[:3] = [-0.0, -np.inf, nan]
    ah = rng.standard_normal(128).astype(np.float16); ah[:2] = [-0.0, -np.inf]

    def check_abs(a):
        _eq(a[3], np.abs(ai)); _bits_eq(a[4], np.abs(af)); _bits_eq(a[5], np.abs(ah))
    add("abs", "absolute_values", {"xi_ptr": I, "xf_ptr": P, "xh_ptr": H, "oi_ptr": I, "of_ptr": P, "oh_ptr": H, "BLOCK": C}, {"BLOCK": 128}, (1,),
        lambda: [ai.copy(), af.copy(), ah.copy(), np.zeros(128, np.int32), np.zeros(128, np.float32), np.zeros(128, np.float16)], check_abs)

    hs = rng.standard_normal(2000).astype(np.float32)
    add("hints_and_cache_modifiers", "hinted_copy", {"src_ptr": P, "dst_ptr": P, "n": "i32", "BLOCK": C}, {"BLOCK": 512}, (4,),
        lambda: [hs.copy(), np.zeros(2000, np.float32), 2000], lambda a: _eq(a[1], hs + np.float32(1)))
    add("volatile_and_cache_modifiers", "volatile_copy", {"src_ptr": P, "dst_ptr": P, "BLOCK": C}, {"BLOCK": 256}, (1,),
        lambda: [hs[:256].copy(), np.zeros(256, np.float32)], lambda a: _eq(a[1], hs[:256]))

    ui = rng.integers(-5, 5, 128).astype(np.int32)
    uf = rng.standard_normal(128).astype(np.float32); uf[0] = 0.0

    def check_unary(a):
        _eq(a[2].reshape(3, 128), [-ui, ~ui, (ui == 0).astype(np.int32)]); _bits_eq(a[3], np.float32(0) - uf)     # -x is 0 - x: -0.0 stays out
    add("unary_ops", "unary_ops", {"xi_ptr": I, "xf_ptr": P, "oi_ptr": I, "of_ptr": P, "BLOCK": C}, {"BLOCK": 128}, (1,),
        lambda: [ui.copy(), uf.copy(), np.zeros(3 * 128, np.int32), np.zeros(128, np.float32)], check_unary)

    # // and % on signed integers follow C (truncation towards zero; the remainder has the dividend's sign)
    qx = rng.integers(-1000, 1000, 256).astype(np.int32)
    qy = rng.integers(1, 50, 256).astype(np.int32) * rng.choice([-1, 1], 256).astype(np.int32)
    qx[:4], qy[:4] = [-7, 7, -7, 7], [2, -2, -2, 2]

    def check_div(a):
        q = np.trunc(qx.astype(np.float64) / qy).astype(np.int32)
        _eq(a[2], q); _eq(a[3], qx - q * qy)
    add("floordiv", "floor_division", {"x_ptr": I, "y_ptr": I, "q_ptr": I, "r_ptr": I, "BLOCK": C}, {"BLOCK": 256}, (1,),
        lambda: [qx.copy(), qy.copy(), np.zeros(256, np.int32), np.zeros(256, np.int32)], check_div)

    vs = rng.integers(-100, 100, 64).astype(np.int32)
    for k, ty in [(1, "i32"), (-3, "i32"), (2 ** 31 - 1, "i32"), (2 ** 31, "i64"), (-2 ** 40, "i64")]:
        add(f"value_specialization_{k}", "scale_by_argument", {"x_ptr": I, "out_ptr": "*i64", "k": ty, "BLOCK": C}, {"BLOCK": 64}, (1,),
            lambda k=k: [vs.copy(), np.zeros(64, np.int64), k], lambda a, k=k: _eq(a[1], vs.astype(np.int64) * k))

    um = (rng.standard_normal(256) * 3).astype(np.float32)

    def check_math(a):
        o = a[1].reshape(12, 256)
        x = um.astype(np.float64)
        from math import erf
        want = [np.exp(x), np.log(np.abs(x) + 1), np.cos(x), np.sin(x), np.sqrt(np.abs(x)), 1 / np.sqrt(np.abs(x) + 0.5),
                np.array([erf(v) for v in x]), np.floor(x), np.ceil(x), np.exp2(x), np.log2(np.abs(x) + 1), 1 / (1 + np.exp(-x))]
        for got, w in zip(o, want):
            _close(got, w, 2e-6 * max(1.0, float(np.max(np.abs(w)))))
        _eq(o[7], np.floor(um)); _eq(o[8], np.ceil(um)); _eq(o[4], np.sqrt(np.abs(um)))
    add("unary_math", "unary_math", {"x_ptr": P, "out_ptr": P, "BLOCK": C}, {"BLOCK": 256}, (1,),
        lambda: [um.copy(), np.zeros(12 * 256, np.float32)], check_math)

    ha = rng.integers(-3, 4, (32, 64)).astype(np.float16)
    hb = rng.integers(-3, 4, (64, 32)).astype(np.float16)
    hc = rng.integers(-9, 9, (32, 32)).astype(np.float32)
    for acc in (0, 1):
        add(f"dot_fp16_acc{acc}", "dot_in_half_precision", {"a_ptr": H, "b_ptr": H, "c_ptr": P, "M": C, "N": C, "K": C, "ACC_IN": C}, {"M": 32, "N": 32, "K": 64, "ACC_IN": acc}, (1,),
            lambda: [ha.reshape(-1).copy(), hb.reshape(-1).copy(), hc.reshape(-1).copy()],
            lambda a, acc=acc: _eq(a[2].reshape(32, 32), ha.astype(np.float32) @ hb.astype(np.float32) + (hc if acc else 0)))
    add("dot_fp16_out_fp16", "dot_accumulating_in_half", {"a_ptr": H, "b_ptr": H, "c_ptr": H, "M": C, "N": C, "K": C}, {"M": 32, "N": 32, "K": 64}, (1,),
        lambda: [ha.reshape(-1).copy(), hb.reshape(-1).copy(), np.zeros(32 * 32, np.float16)],
        lambda a: _eq(a[2].reshape(32, 32), (ha.astype(np.float32) @ hb.astype(np.float32)).astype(np.float16)))

    fx_ = rng.standard_normal(1024).astype(np.float32)
    falt = rng.standard_normal(1024).astype(np.float32)
    add("other_is_data", "fill_values_that_are_data", {"x_ptr": P, "alt_ptr": P, "out_ptr": P, "n": "i32", "fill": "i32", "BLOCK": C}, {"BLOCK": 256}, (4,),
        lambda: [fx_.copy(), falt.copy(), np.zeros(2048, np.float32), 700, -7],
        lambda a: _eq(a[2], np.concatenate([np.where(np.arange(1024) < 700, fx_, np.float32(-7)), np.where(np.arange(1024) < 700, fx_, falt)])))

    # tile products with the epilogues of the core dot test; small integers so that every order of summation is exact
    for dt, name in [(np.float32, "fp32"), (np.float16, "fp16"), (np.int8, "i8")]:
        M, N, K = 32, 32, 64
        dx_ = rng.integers(-3, 4, (M, K)).astype(dt)
        dy_ = rng.integers(-3, 4, (K, N)).astype(dt)
        dw_ = rng.integers(-2, 3, (N, N)).astype(dt)
        acc_t = np.int32 if dt == np.int8 else np.float32
        dz_ = rng.integers(-9, 10, (M, N)).astype(acc_t)
        prod = dx_.astype(np.int64) @ dy_.astype(np.int64)
        sig = {"x_ptr": "*" + name, "y_ptr": "*" + name, "w_ptr": "*" + name, "z_ptr": "*i32" if dt == np.int8 else P, "M": C, "N": C, "K": C, "EPI": C}
        for epi in range(7):
            if epi == 4 and dt == np.int8:
                continue
            if epi == 5 and dt == np.float16:       # the first product is narrowed to fp16 before the second: keep it exact
                prod5 = np.clip(prod, -2048, 2048)
                assert np.array_equal(prod5, prod)

            def check(a, epi=epi, prod=prod, dz_=dz_, dw_=dw_, acc_t=acc_t, M=M, N=N):
                got = a[3].reshape(N, M).T if epi == 6 else a[3].reshape(M, N)
                if epi == 4:
                    e = np.exp((prod - prod.max(1, keepdims=True)).astype(np.float64))
                    return _close(got, e / e.sum(1, keepdims=True), 1e-6)
                want = [prod, prod + dz_, prod + dz_[:, :1], prod + dz_[:1, :], None, prod @ dw_.astype(np.int64), prod][epi]
                _eq(got, want.astype(acc_t))
            add(f"dot_{name}_epilogue{epi}", "dot_with_epilogue", sig, {"M": M, "N": N, "K": K, "EPI": epi}, (1,),
                lambda dx_=dx_, dy_=dy_, dw_=dw_, dz_=dz_: [dx_.reshape(-1).copy(), dy_.reshape(-1).copy(), dw_.reshape(-1).copy(), dz_.reshape(-1).copy()], check)

    # integer arithmetic, bit operations, shifts and comparisons in every width and signedness
    for dt, name in [(np.int8, "i8"), (np.int16, "i16"), (np.int32, "i32"), (np.int64, "i64"), (np.uint8, "u8"), (np.uint16, "u16"), (np.uint32, "u32"), (np.uint64, "u64")]:
        info = np.iinfo(dt)
        n = 600
        ix = rng.integers(info.min, info.max, n, dtype=dt, endpoint=True)
        iy = rng.integers(info.min, info.max, n, dtype=dt, endpoint=True)
        iy[iy == 0] = 3
        if info.min < 0:
            iy[iy == -1] = 5                                        # min // -1 overflows: undefined in the source language
        ix[:3] = [info.min, info.max, 0]

        def check_int(a, dt=dt, ix=ix, iy=iy, n=n, info=info):
            o = a[2].reshape(13, n)
            X, Y = [int(v) for v in ix], [int(v) for v in iy]
            bits = info.bits

            def wrap(v):
                v &= (1 << bits) - 1
                return v - (1 << bits) if info.min < 0 and v >> (bits - 1) else v
            tdiv = lambda p, q: abs(p) // abs(q) * (1 if (p < 0) == (q < 0) else -1)       # C division: towards zero
            planes = [[wrap(p + q) for p, q in zip(X, Y)], [wrap(p - q) for p, q in zip(X, Y)], [wrap(p * q) for p, q in zip(X, Y)],
                      [wrap(tdiv(p, q)) for p, q in zip(X, Y)], [wrap(p - tdiv(p, q) * q) for p, q in zip(X, Y)],
                      [wrap(p & q) for p, q in zip(X, Y)], [wrap(p | q) for p, q in zip(X, Y)], [wrap(p ^ q) for p, q in zip(X, Y)],
                      [wrap(p << (q & 3)) for p, q in zip(X, Y)], [wrap(p >> (q & 3)) for p, q in zip(X, Y)],
                      [(p < q) + 2 * (p <= q) + 4 * (p == q) for p, q in zip(X, Y)], [wrap(max(p, q) - min(p, q)) for p, q in zip(X, Y)],
                      [max(p, q) for p, q in zip(X, Y)]]
            for k, (got, want) in enumerate(zip(o, planes)):
                assert [int(v) for v in got] == want, (k, [int(v) for v in got][:8], want[:8])
        add(f"int_ops_{name}", "integer_ops_any_width", {"x_ptr": "*" + name, "y_ptr": "*" + name, "out_ptr": "*" + name, "n": "i32", "BLOCK": C}, {"BLOCK": 256}, (3,),
            lambda ix=ix, iy=iy, dt=dt, n=n: [ix.copy(), iy.copy(), np.zeros(13 * n, dt), n], check_int)
    return out
