"""The drop-in boundary without a GPU: the C-ABI library loads and exports every
symbol include/tts_hip.h declares, the Python plugin surface has the members the
reference's CPUDriver/CPUBackend have (backend/driver.py:361-464,
backend/compiler.py:206-275), and the launcher marshals arguments as the
reference launcher does (driver.py:140-223).  Nothing here launches a kernel."""
import ctypes
import os
import re

import pytest

from conftest import ROOT, plan_for


def test_library_exports_every_declared_symbol(native):
    header = open(os.path.join(ROOT, "include", "tts_hip.h")).read()
    declared = set(re.findall(r"\b(tts_[a-z_0-9]+)\s*\(", header))
    assert {"tts_launch", "tts_plan_load", "tts_ttir_to_structured", "tts_structured_to_plan", "tts_free",
            "tts_last_error", "tts_plan_describe_launch"} <= declared
    lib = ctypes.CDLL(native.LIB_PATH)
    for sym in sorted(declared):
        assert hasattr(lib, sym), f"{sym} is declared in include/tts_hip.h but not exported"


def test_full_frontend_compile_without_gpu():
    # the whole unchanged frontend path: @triton.jit source -> ttir -> ttsharedir -> obj
    import triton
    from triton.backends.compiler import GPUTarget
    from triton.compiler import ASTSource
    import triton_shared_amd as tsa
    from triton_shared_amd.examples import kernels as K
    tsa.register_backend()
    src = ASTSource(K.row_softmax, signature={"out_ptr": "*fp32", "in_ptr": "*fp32", "in_pitch": "i32",
                                              "out_pitch": "i32", "n_cols": "i32", "BLOCK": "constexpr"},
                    constexprs={"BLOCK": 1024})
    k = triton.compile(src, target=GPUTarget(tsa.BACKEND_NAME, "gfx950", 64))
    assert list(k.asm.keys())[-3:] == ["ttir", "ttsharedir", "obj"]
    assert k.metadata.name == "row_softmax"
    assert k.asm["obj"].startswith(b"tts.plan 1 family=row_softmax")
    assert k.asm["ttsharedir"].startswith("tts.program 1 @row_softmax")


def test_backend_and_driver_surface():
    from triton.backends.compiler import GPUTarget
    import triton_shared_amd as tsa
    target = GPUTarget(tsa.BACKEND_NAME, "gfx950", 64)
    assert tsa.HIPBackend.supports_target(target)
    assert not tsa.HIPBackend.supports_target(GPUTarget("cpu", 0, 0))
    assert not tsa.HIPBackend.supports_target(GPUTarget("hip", "gfx950", 64))  # never shadows Triton's own AMD backend
    be = tsa.HIPBackend(target)
    opts = be.parse_options({"num_warps": 8, "debug": True})
    assert opts.num_warps == 8 and opts.arch == "gfx950" and opts.enable_fp_fusion is False
    assert be.get_codegen_implementation(opts)["min_dot_size"](None, None) == (1, 1, 1)
    assert be.binary_ext == "obj" and be.get_module_map() == {} and isinstance(be.hash(), str)
    stages = {}
    be.add_stages(stages, opts, None)
    assert list(stages) == ["ttir", "ttsharedir", "obj"]

    class Meta:
        num_warps, num_ctas, shared, cluster_dims, name = 4, 1, 0, (1, 1, 1), "k"

    assert be.pack_metadata(Meta)[6] == "k" and len(be.pack_metadata(Meta)) == 7
    drv = tsa.HIPDriver()
    assert tsa.HIPDriver.is_active() is False          # never auto-selected (driver.py:428-432)
    assert drv.get_current_target() == target
    assert drv.binary_ext == "obj" and drv.launcher_cls is tsa.HIPLauncher and drv.utils is tsa.HIPUtils()
    assert drv.map_python_to_cpp_type("*fp16") == "void*" and drv.map_python_to_cpp_type("i1") == "int32_t"
    assert drv.map_python_to_cpp_type("fp32") == "float" and drv.map_python_to_cpp_type("u64") == "uint64_t"
    with pytest.raises(TypeError):
        drv.map_python_to_cpp_type("fp16")             # unsupported in the reference as well (driver.py:57-60)
    assert str(drv.get_active_torch_device()) == "cuda"


class _Src:
    class fn:
        arg_names = ["x_ptr", "y_ptr", "z_ptr", "n", "BLOCK"]
    signature = {"x_ptr": "*fp32", "y_ptr": "*fp32", "z_ptr": "*fp32", "n": "i32", "BLOCK": "constexpr"}
    constants = {"BLOCK": 1024}


def test_launcher_marshalling(native):
    import torch
    import triton_shared_amd as tsa
    plan, _ = plan_for(native, "vec_add")
    launcher = tsa.HIPLauncher(_Src, None)
    assert launcher.slots == [(0, True), (1, True), (2, True), (3, False)]   # the constexpr is not forwarded
    events = []
    enter = lambda md: events.append(("enter", md))
    leave = lambda md: events.append(("exit", md))
    # a grid with zero volume is a no-op, hooks still run (driver.py:117,197-218)
    launcher(0, 1, 1, None, plan, (4, 1, 0, 1, 1, 1, "vec_add"), "meta", enter, leave, 1 << 20, 2 << 20, None, 10, 1024)
    assert events == [("enter", "meta"), ("exit", "meta")]
    with pytest.raises(TypeError, match="device"):      # host memory is refused
        launcher(1, 1, 1, None, plan, None, None, None, None, torch.zeros(4), 0, 0, 4, 1024)
    with pytest.raises(TypeError, match="data_ptr"):
        launcher(1, 1, 1, None, plan, None, None, None, None, "not a pointer", 0, 0, 4, 1024)
    with pytest.raises(RuntimeError, match="load_binary"):
        launcher(1, 1, 1, None, b"raw bytes", None, None, None, None, 0, 0, 0, 4, 1024)


def test_load_binary_tuple(native):
    import sys
    import triton_shared_amd as tsa
    structured = native.ttir_to_structured(open(os.path.join(ROOT, "tests/golden/vec_add.ttir")).read())
    plan_bytes, _ = native.structured_to_plan(structured)
    mod, fn, n_regs, n_spills, n_max = tsa.HIPUtils.load_binary("vec_add", plan_bytes, 0, 0)
    assert mod is fn and fn.family == "map1d" and n_max == sys.maxsize and fn.arg_kinds == [0, 0, 0, 1]


def test_missing_extension_fails_loudly(monkeypatch):
    import triton_shared_amd as tsa
    monkeypatch.setattr(tsa._native, "_lib", None)
    monkeypatch.setattr(tsa._native, "LIB_PATH", "/nonexistent/libtts_hip.so")
    with pytest.raises(RuntimeError, match="has not been built"):
        tsa.HIPDriver()


def test_product_does_not_import_the_oracle():
    bad = []
    pkg = os.path.join(ROOT, "triton-shared_amd")
    for d, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".cpp", ".hip", ".h")):
                text = open(os.path.join(d, f)).read()
                if re.search(r"\boracle\b", text) or "cpu_path" in text or "ttir_lanes" in text:
                    bad.append(os.path.join(d, f))
    assert not bad, f"product files mention the oracle: {bad}"
