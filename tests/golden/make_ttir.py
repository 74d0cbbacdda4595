"""Regenerates tests/golden/*.ttir: the TTIR text of the five hot-path kernels as
the installed Triton frontend emits it under the reference's TTIR pass list
(backend/compiler.py:244-260).  Needs no GPU.  The files are inputs for the planner
tests (the role the .mlir inputs under test/Conversion/ play for the reference's
lit tests); nothing of the reference is run or read by this script.

    python tests/golden/make_ttir.py
"""
import os
import re
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

import triton  # noqa: E402
from triton.backends.compiler import GPUTarget  # noqa: E402
from triton.compiler import ASTSource  # noqa: E402

import triton_shared_amd as tsa  # noqa: E402
from triton_shared_amd.examples import kernels as K  # noqa: E402

SIGS = {
    "vec_add": (K.vec_add, {"x_ptr": "*fp32", "y_ptr": "*fp32", "z_ptr": "*fp32", "n": "i32", "BLOCK": "constexpr"},
                {"BLOCK": 1024}),
    "row_softmax": (K.row_softmax, {"out_ptr": "*fp32", "in_ptr": "*fp32", "in_pitch": "i32", "out_pitch": "i32",
                                    "n_cols": "i32", "BLOCK": "constexpr"}, {"BLOCK": 1024}),
    "layer_norm_fwd": (K.layer_norm_fwd, {"X": "*fp16", "Y": "*fp16", "W": "*fp16", "B": "*fp16", "Mean": "*fp32",
                                          "Rstd": "*fp32", "pitch": "i32", "N": "i32", "eps": "fp32",
                                          "BLOCK": "constexpr"}, {"BLOCK": 1024}),
    "matmul_tiles": (K.matmul_tiles, {"a_ptr": "*bf16", "b_ptr": "*bf16", "c_ptr": "*bf16", "M": "i32", "N": "i32",
                                      "K": "i32", "s_am": "i32", "s_ak": "constexpr", "s_bk": "i32", "s_bn": "constexpr",
                                      "s_cm": "i32", "s_cn": "constexpr", "BM": "constexpr", "BN": "constexpr",
                                      "BK": "constexpr", "GROUP_M": "constexpr"},
                     {"s_ak": 1, "s_bn": 1, "s_cn": 1, "BM": 128, "BN": 128, "BK": 64, "GROUP_M": 8}),
    "matmul_wrapped": (K.matmul_wrapped, {"a_ptr": "*bf16", "b_ptr": "*bf16", "c_ptr": "*bf16", "M": "i32", "N": "i32",
                                          "K": "i32", "s_am": "i32", "s_ak": "constexpr", "s_bk": "i32", "s_bn": "constexpr",
                                          "s_cm": "i32", "s_cn": "constexpr", "BM": "constexpr", "BN": "constexpr",
                                          "BK": "constexpr", "GROUP_M": "constexpr"},
                       {"s_ak": 1, "s_bn": 1, "s_cn": 1, "BM": 128, "BN": 128, "BK": 64, "GROUP_M": 8}),
    "w8a16_matmul": (K.w8a16_matmul, {"a_ptr": "*fp16", "w_ptr": "*i8", "s_ptr": "*fp16", "c_ptr": "*fp16", "M": "i32",
                                      "N": "i32", "K": "i32", "s_am": "i32", "s_ak": "constexpr", "s_wk": "i32",
                                      "s_wn": "constexpr", "s_cm": "i32", "s_cn": "constexpr", "BM": "constexpr",
                                      "BN": "constexpr", "BK": "constexpr"},
                     {"s_ak": 1, "s_wn": 1, "s_cn": 1, "BM": 16, "BN": 128, "BK": 128}),
    "gelu_tanh_bias": (K.gelu_tanh_bias, {"x_ptr": "*fp32", "b_ptr": "*fp32", "y_ptr": "*fp32", "n": "i32", "BLOCK": "constexpr"},
                       {"BLOCK": 1024}),
    "clamp_scale_where": (K.clamp_scale_where, {"x_ptr": "*fp32", "y_ptr": "*fp32", "out_ptr": "*fp32", "n": "i32", "lo": "fp32",
                                                "hi": "fp32", "alpha": "fp32", "BLOCK": "constexpr"}, {"BLOCK": 1024}),
    "silu_mul_f16": (K.silu_mul_f16, {"g_ptr": "*fp16", "u_ptr": "*fp16", "out_ptr": "*fp16", "n": "i32", "BLOCK": "constexpr"},
                     {"BLOCK": 1024}),
}
# small-block variants for the brute-force tests
SMALL = {
    "vec_add.small": ("vec_add", {"BLOCK": 64}),
    "row_softmax.small": ("row_softmax", {"BLOCK": 64}),
    "layer_norm_fwd.small": ("layer_norm_fwd", {"BLOCK": 64}),
    "matmul_tiles.small": ("matmul_tiles", {"BM": 32, "BN": 32, "BK": 16, "GROUP_M": 2}),
    "matmul_wrapped.small": ("matmul_wrapped", {"BM": 32, "BN": 32, "BK": 16, "GROUP_M": 2}),
    "w8a16_matmul.small": ("w8a16_matmul", {"BM": 16, "BN": 32, "BK": 32}),
}


def strip_loc(text):
    out, i = [], 0
    while i < len(text):
        if text.startswith(" loc(", i):
            j, depth = i + 5, 1
            while depth:
                depth += {"(": 1, ")": -1}.get(text[j], 0)
                j += 1
            i = j
        else:
            out.append(text[i])
            i += 1
    return "\n".join(l for l in "".join(out).splitlines() if not re.match(r"\s*#loc", l)) + "\n"


def ttir_of(fn, sig, consts):
    """TTIR only: the frontend plus the reference's TTIR pass list, without the later stages (a kernel
    need not belong to a kernel family to have a fixture)."""
    from triton._C.libtriton import ir
    from triton_shared_amd.backend.compiler import HIPBackend
    tsa.register_backend()
    src = ASTSource(fn, signature=sig, constexprs=consts)
    target = GPUTarget(tsa.BACKEND_NAME, "gfx950", 64)
    backend = HIPBackend(target)
    ctx = ir.context()
    ir.load_dialects(ctx)
    options = backend.parse_options({})
    mod = src.make_ir(target, options, backend.get_codegen_implementation(options), backend.get_module_map(), ctx)
    return str(backend.make_ttir(mod, {}, options))


def main():
    for name, (fn, sig, consts) in SIGS.items():
        with open(os.path.join(HERE, name + ".ttir"), "w") as f:
            f.write(strip_loc(ttir_of(fn, sig, consts)))
    for name, (base, over) in SMALL.items():
        fn, sig, consts = SIGS[base]
        with open(os.path.join(HERE, name + ".ttir"), "w") as f:
            f.write(strip_loc(ttir_of(fn, sig, dict(consts, **over))))
    print("wrote", len(SIGS) + len(SMALL), "files to", HERE)


if __name__ == "__main__":
    main()
