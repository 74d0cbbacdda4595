"""Inputs and expected outputs of the reference's functional tests (python/examples/*.py) for the kernels in
extra_kernels.py that restate them.  Each case: (kernel name, signature, constexprs, grid, argument builder, checker).
The builders return numpy arrays / scalars in kernel-argument order; `check(arrays)` asserts on the arrays after the
run.  Both the lane-level oracle (CPU) and the GPU backend are run through the same cases."""
import numpy as np

I, P = "*i32", "*fp32"


def _eq(got, want):
    assert np.array_equal(np.asarray(got), np.asarray(want)), (np.asarray(got).tolist(), np.asarray(want).tolist())


def cases():
    out = []

    def add(name, kernel, sig, consts, grid, args, check):
        out.append(dict(name=name, kernel=kernel, sig=sig, consts=consts, grid=grid, args=args, check=check))

    # test_early_return.py:37-65
    add("early_return_taken", "stop_on_flag", {"flags": I, "dst": I}, {}, (1,),
        lambda: [np.full(8, -1, np.int32), np.full(8, -1, np.int32)], lambda a: _eq(a[1], [-1] * 8))
    add("early_return_not_taken", "stop_on_flag", {"flags": I, "dst": I}, {}, (1,),
        lambda: [np.arange(8, dtype=np.int32), np.full(8, -1, np.int32)], lambda a: _eq(a[1], [1, 2, 3, 4, -1, -1, -1, -1]))
    # test_scalar_store.py:37-55
    add("scalar_store_nested", "count_up_scalars", {"dst": P, "N": "constexpr"}, {"N": 8}, (1,),
        lambda: [np.full(8, -99, np.float32)], lambda a: _eq(a[0], np.arange(8, dtype=np.float32)))
    # test_sign_extend.py:30-48
    add("sign_extend", "window_at_loaded_offset", {"start_ptr": I, "src": I, "dst": I, "n": "i32"}, {}, (1,),
        lambda: [np.full(1, 1, np.int32), np.arange(4, dtype=np.int32), np.full(4, -1, np.int32), 4], lambda a: _eq(a[2], [1, 2, 3, 11]))
    # test_blockptr_complex_offset.py:33-40
    add("blockptr_shifted_base", "block_ptr_shifted_base", {"src": P, "dst": P}, {}, (1,),
        lambda: [np.arange(16, dtype=np.float32), np.full(4, -1, np.float32)], lambda a: _eq(a[1], np.arange(8, 12, dtype=np.float32)))
    # test_gather_scatter_continuous.py:24-89 (rows of a [2, 4, 8] view; the column variants move the split to the other index)
    sig3 = {"src": I, "dst": I, "X": "constexpr", "Y": "constexpr", "Z": "constexpr", "MASK": "constexpr"}
    src3 = np.arange(2, 66, dtype=np.int32)

    def want3(mask):
        ref = src3.reshape(2, 4, 8).copy()
        if mask:
            ref[:, :, 4:] = 0 if mask == 1 else -1
        return ref.reshape(-1)
    for mask in (0, 1, 2):
        add(f"gather_row_mask{mask}", "copy_as_3d", sig3, {"X": 2, "Y": 4, "Z": 8, "MASK": mask}, (1,),
            lambda: [src3.copy(), np.full(64, -1, np.int32)], lambda a, mask=mask: _eq(a[1], want3(mask)))
    # test_load_2d_tensor_col.py:49-67
    x42 = np.arange(8, dtype=np.float32)
    add("blockptr_column", "block_ptr_column", {"src": P, "dst": P, "n_rows": "i32", "n_cols": "i32", "BR": "constexpr", "PITCH": "constexpr"},
        {"BR": 4, "PITCH": 2}, (2,), lambda: [x42.copy(), np.full(8, -1, np.float32), 4, 2], lambda a: _eq(a[1], x42))
    # test_mask_loop_iter_arg.py:55-70 (three of its 36 shapes)
    for b, h in [(1, 16), (3, 128), (8, 1024)]:
        rng = np.random.default_rng(b * h)
        xs = rng.standard_normal(b * h).astype(np.float32)
        add(f"mask_loop_{b}x{h}", "grid_stride_copy", {"dst": P, "src": P, "total": "i64", "BLOCK": "constexpr"}, {"BLOCK": 2}, (2,),
            lambda xs=xs: [np.zeros_like(xs), xs.copy(), xs.size], lambda a, xs=xs: _eq(a[0], xs))
    # test_reduce.py:34-46
    rng = np.random.default_rng(3)
    xr = rng.random((32, 16)).astype(np.float32)
    add("blockptr_row_sum", "block_ptr_row_sum", {"x_ptr": P, "out_ptr": P, "pitch": "i32", "n": "i32", "BLOCK": "constexpr"}, {"BLOCK": 16}, (32,),
        lambda: [xr.reshape(-1).copy(), np.zeros(32, np.float32), 16, 16],
        lambda a: np.testing.assert_allclose(a[1], xr.astype(np.float64).sum(1), rtol=1e-3, atol=1e-5))
    # test_tensor_index_iterargs.py:11-108
    add("carried_offsets_masked", "carried_offsets_masked", {"src": I, "dst": I, "bound": "i32"}, {}, (1,),
        lambda: [np.arange(17, dtype=np.int32), np.full(17, -1, np.int32), 14], lambda a: _eq(a[1], list(range(14)) + [-11, -11, -1]))
    add("carried_offsets_nested", "carried_offsets_nested", {"src": I, "dst": I}, {}, (1,),
        lambda: [np.arange(64, dtype=np.int32), np.full(64, -1, np.int32)],
        lambda a: _eq(a[1], [0, 1, 2, 3, 4, 5, 6, 7, 11, 12, 13, 14, 21, 22, 23, 24, 27, 28, 29, 30, 31, 32, 33, 34, 38, 39, 40, 41, 48, 49, 50, 51]
                      + [-1] * 32))
    add("store_carried_block", "store_carried_block", {"dst": I}, {}, (1,), lambda: [np.full(8, -1, np.int32)],
        lambda a: _eq(a[0], np.arange(8, dtype=np.int32)))
    # test_unstructured_mask.py:33-66, 107-147
    m, n, M, N = 6, 16, 8, 16
    xin = np.arange(2, 2 + m * n, dtype=np.float32).reshape(m, n)
    keep_r = np.array([1, 0, 1, 0, 1, 0], dtype=np.int8)
    keep_c = np.array([0, 1, 0, 1, 0, 1, 0, 1, 1, 0, 1, 0, 1, 0, 1, 0], dtype=np.int8)

    def want_masks():
        v = np.full_like(xin, -2)
        v[keep_r != 0, :] = xin[keep_r != 0, :]
        w = np.full_like(xin, -1)
        w[:, keep_c != 0] = v[:, keep_c != 0]
        return w.reshape(-1)
    add("masks_from_memory_2d", "masks_from_memory_2d",
        {"src": P, "dst": P, "keep_rows": "*i8", "keep_cols": "*i8", "m": "i32", "n": "i32", "M": "constexpr", "N": "constexpr"}, {"M": M, "N": N}, (1,),
        lambda: [xin.reshape(-1).copy(), np.full(m * n, -1, np.float32), keep_r.copy(), keep_c.copy(), m, n], lambda a: _eq(a[1], want_masks()))
    idx = np.array([1, 3, 7], dtype=np.int32)

    def want_rows():
        w = np.full((3, n), -2, dtype=np.float32)
        ok = idx[idx < m]
        w[:len(ok), :] = xin[ok, :]
        return w.reshape(-1)
    add("rows_by_index_masked", "rows_by_index_masked",
        {"src": P, "dst": P, "idx": I, "n_idx": "i32", "m": "i32", "n": "i32", "pitch_m": "i32", "pitch_n": "i32", "IM": "constexpr", "N": "constexpr"},
        {"IM": 4, "N": 16}, (1,), lambda: [xin.reshape(-1).copy(), np.full(3 * n, -1, np.float32), idx.copy(), 3, m, n, n, 1],
        lambda a: _eq(a[1], want_rows()))
    # test_unstructured_mask.py:69-110 (the batched form), 167-211 (columns through an index), 215-325 (both in three
    # dimensions), 328-375 (masks from comparisons with the program id)
    b3 = 4
    x3 = np.arange(2, 2 + b3 * m * n, dtype=np.float32).reshape(b3, m, n)

    def want_masks_3d():
        v = np.full_like(x3, -2)
        v[:, keep_r != 0, :] = x3[:, keep_r != 0, :]
        w = np.full_like(x3, -1)
        w[:, :, keep_c != 0] = v[:, :, keep_c != 0]
        return w.reshape(-1)
    add("masks_from_memory_3d", "masks_from_memory_3d",
        {"src": P, "dst": P, "keep_rows": "*i8", "keep_cols": "*i8", "b": "i32", "m": "i32", "n": "i32", "B": "constexpr", "M": "constexpr", "N": "constexpr"},
        {"B": 4, "M": M, "N": N}, (1,),
        lambda: [x3.reshape(-1).copy(), np.full(x3.size, -1, np.float32), keep_r.copy(), keep_c.copy(), b3, m, n], lambda a: _eq(a[1], want_masks_3d()))
    idx_n = np.array([10, 20, 15, 1, 3, 5, 7, 0, 2, 4, 6, 8], dtype=np.int32)

    def want_columns(src):
        w = np.full_like(src, -1)
        ok = idx_n < n
        w[..., idx_n[ok]] = src[..., :len(idx_n)][..., ok]
        return w.reshape(-1)
    add("columns_by_index_masked", "columns_by_index_masked",
        {"src": P, "dst": P, "idx": I, "n_idx": "i32", "m": "i32", "n": "i32", "pitch_m": "i32", "pitch_n": "i32", "M": "constexpr", "IN": "constexpr"},
        {"M": 8, "IN": 16}, (1,), lambda: [xin.reshape(-1).copy(), np.full(m * n, -1, np.float32), idx_n.copy(), len(idx_n), m, n, n, 1],
        lambda a: _eq(a[1], want_columns(xin)))

    def want_rows_3d():
        w = np.full((b3, 3, n), -2, dtype=np.float32)
        ok = idx[idx < m]
        w[:, :len(ok), :] = x3[:, ok, :]
        return w.reshape(-1)
    add("rows_by_index_masked_3d", "rows_by_index_masked_3d",
        dict([("src", P), ("dst", P), ("idx", I)] + [(k, "i32") for k in "n_idx b m n s_b s_m s_n d_b d_m d_n".split()] + [(k, "constexpr") for k in ("B", "IM", "N")]),
        {"B": 4, "IM": 4, "N": 16}, (1,),
        lambda: [x3.reshape(-1).copy(), np.full(b3 * 3 * n, -1, np.float32), idx.copy(), 3, b3, m, n, m * n, n, 1, 3 * n, n, 1], lambda a: _eq(a[1], want_rows_3d()))
    add("columns_by_index_masked_3d", "columns_by_index_masked_3d",
        dict([("src", P), ("dst", P), ("idx", I)] + [(k, "i32") for k in "n_idx b m n s_b s_m s_n".split()] + [(k, "constexpr") for k in ("B", "M", "IN")]),
        {"B": 4, "M": 8, "IN": 16}, (1,),
        lambda: [x3.reshape(-1).copy(), np.full(x3.size, -1, np.float32), idx_n.copy(), len(idx_n), b3, m, n, m * n, n, 1], lambda a: _eq(a[1], want_columns(x3)))
    xp = np.arange(2, 2 + 3 * m * n, dtype=np.float32).reshape(3, m, n)

    def want_above_pid():
        w = np.full_like(xp, -1)
        for pid in range(3):
            t = np.full((m, n), -2, np.float32)
            t[np.arange(m) > pid, :] = xp[pid][np.arange(m) > pid, :]
            w[pid][:, np.arange(n) > pid] = t[:, np.arange(n) > pid]
        return w.reshape(-1)
    add("masks_above_program_id", "masks_above_program_id",
        dict([("src", P), ("dst", P)] + [(k, "i32") for k in "m n s_pid s_m s_n".split()] + [("M", "constexpr"), ("N", "constexpr")]), {"M": 8, "N": 16}, (3,),
        lambda: [xp.reshape(-1).copy(), np.full(xp.size, -1, np.float32), m, n, m * n, n, 1], lambda a: _eq(a[1], want_above_pid()))
    # a mixture-of-experts product (the kernel of test/Conversion/TritonToLinalgExperimental/unstructured_ptr_used_in_loop.mlir,
    # which has no runtime test in the reference): small integers, so every summation order gives the same bits
    rng = np.random.default_rng(6)
    n_tok, Kd, Nd, E = 40, 48, 24, 3
    Am = rng.integers(-3, 4, (64, Kd)).astype(np.float32)
    Bm = rng.integers(-3, 4, (E, Kd, Nd)).astype(np.float32)
    rows = rng.integers(0, 64, n_tok).astype(np.int32)
    experts = np.array([2, -1, 0], dtype=np.int32)                      # per block of 16 rows; -1: nothing to do

    def want_moe():
        w = np.full((n_tok, Nd), -1, np.float32)
        for blk, e in enumerate(experts):
            if e >= 0:
                r = slice(blk * 16, min(n_tok, blk * 16 + 16))
                w[r] = Am[rows[r]] @ Bm[e]
        return w.reshape(-1)
    add("grouped_rows_matmul", "grouped_rows_matmul",
        dict([("a_ptr", P), ("b_ptr", P), ("c_ptr", P), ("rows_ptr", I), ("expert_ptr", I)] + [(k, "i32") for k in "n_rows K N s_am s_be s_bk s_cm".split()]
             + [(k, "constexpr") for k in ("BM", "BN", "BK")]), {"BM": 16, "BN": 16, "BK": 32}, (3, 2),
        lambda: [Am.reshape(-1).copy(), Bm.reshape(-1).copy(), np.full(n_tok * Nd, -1, np.float32), rows.copy(), experts.copy(), n_tok, Kd, Nd, Kd, Kd * Nd, Nd, Nd],
        lambda a: _eq(a[2], want_moe()))
    # test/Conversion/TritonToStructured/conditional_ptr_as_src.mlir (a lit input without a runtime test in the reference)
    for which, first in [(5, 16), (3, 9)]:
        add(f"pointer_picked_by_branch_{which}", "pointer_picked_by_branch", {"src": P, "dst": P, "which": "i32"}, {}, (1,),
            lambda which=which: [np.arange(32, dtype=np.float32), np.full(4, -1, np.float32), which],
            lambda a, first=first: _eq(a[1], np.arange(first, first + 4, dtype=np.float32)))
    # test_einsum_qhmd_hmpd_to_qhmp.py:150-165
    Q, H, Mm, D, Pp = 1, 2, 2, 2, 4
    rng = np.random.default_rng(4)
    A = rng.standard_normal((Q, H, Mm, D)).astype(np.float32)
    B = rng.standard_normal((H, Mm, Pp, D)).astype(np.float32)
    st = lambda t: [s // t.itemsize for s in t.strides]
    sig_e = dict([("a_ptr", P), ("b_ptr", P), ("c_ptr", P)] +
                 [(k, "i32") for k in "Q H M P D a_q a_h a_m a_d b_h b_m b_p b_d c_q c_h c_m c_p".split()] + [("BQ", "constexpr"), ("BP", "constexpr")])
    C = np.zeros((Q, H, Mm, Pp), np.float32)
    add("einsum_qhmd_hmpd", "einsum_qhmd_hmpd", sig_e, {"BQ": 2, "BP": 2}, (Q * H * Mm // 2, Pp // 2),
        lambda: [A.reshape(-1).copy(), B.reshape(-1).copy(), np.zeros(C.size, np.float32), Q, H, Mm, Pp, D] + st(A) + st(B) + st(C),
        lambda a: np.testing.assert_allclose(a[2].reshape(C.shape), np.einsum("qhmd,hmpd->qhmp", A.astype(np.float64), B.astype(np.float64)),
                                             rtol=1e-5, atol=1e-5))
    return out
