"""Triton compiler backend for the MI355X execution backend.

Counterpart of the reference's `CPUBackend` (backend/compiler.py:206-275) with the
same plugin surface: `supports_target`, `parse_options`, `get_codegen_implementation`,
`pack_metadata` (7-tuple, kernel name last), `load_dialects`, `add_stages`, `hash`,
`get_module_map`, `binary_ext`.  The stages are

    ttir        the reference's own TTIR pass list (backend/compiler.py:244-260)
    ttsharedir  structured program text produced by the native planner
                (replaces the triton-shared-opt subprocess, compiler.py:48-67)
    obj         launch plan bytes: kernel family + bindings
                (replaces mlir-opt / mlir-translate / llc, compiler.py:75-175)

A kernel that matches no hand-written kernel family fails at the `obj` stage with
NotImplementedError; there is no fallback path.
"""
import functools
import hashlib
import os
from dataclasses import dataclass
from types import ModuleType
from typing import Any, Dict, Tuple

from triton._C.libtriton import ir, passes
from triton.backends.compiler import BaseBackend, GPUTarget

from .. import _native

BACKEND_NAME = "mi355x"


def _dump(name: str, text):
    """TRITON_SHARED_DUMP_PATH keeps the intermediate files, as in the reference
    (backend/compiler.py:30-35)."""
    path = os.getenv("TRITON_SHARED_DUMP_PATH", "")
    if not path:
        return
    mode = "wb" if isinstance(text, bytes) else "w"
    with open(os.path.join(path, name), mode) as f:
        f.write(text)


def ttir_to_ttsharedir(mod) -> str:
    ttir_text = str(mod)
    _dump("tt.mlir", ttir_text)
    text = _native.ttir_to_structured(ttir_text)
    _dump("ttshared.txt", text)
    return text


def ttsharedir_to_obj(structured: str, metadata) -> bytes:
    plan, name = _native.structured_to_plan(structured)
    metadata["name"] = name
    _dump("plan.bin", plan)
    return plan


@dataclass(frozen=True)
class HIPOptions:
    debug: bool = False
    arch: str = "gfx950"
    num_warps: int = 4          # accepted for source compatibility; the kernels pick their own shape
    num_ctas: int = 1
    num_stages: int = 1
    enable_warp_specialization: bool = False
    enable_fp_fusion: bool = False   # no FMA contraction, as on the reference CPU path
    extern_libs = None
    cluster_dims: tuple = (1, 1, 1)
    shared: int = 0
    supported_fp8_dtypes: Tuple[str] = ()
    deprecated_fp8_dot_operand_dtypes: Tuple[str] = ()
    allow_fp8e4nv: bool = False
    allowed_dot_input_precisions: Tuple[str] = ("ieee", )
    default_dot_input_precision: str = "ieee"
    max_num_imprecise_acc_default: int = 0
    sanitize_overflow: bool = True
    launch_cooperative_grid: bool = False
    instrumentation_mode: str = ""
    backend_name: str = BACKEND_NAME
    # True: tl.make_block_ptr / tl.advance reach the planner as tt.make_tensor_ptr / tt.advance ops instead of being
    # rewritten to plain pointer arithmetic first (the default, and what the reference's pass list does)
    raw_block_pointers: bool = os.environ.get("TTS_RAW_BLOCK_POINTERS", "0") == "1"

    def hash(self):
        key = "_".join(f"{k}-{v}" for k, v in sorted(self.__dict__.items()))
        return hashlib.sha256(key.encode("utf-8")).hexdigest()


class HIPBackend(BaseBackend):
    binary_ext = "obj"

    @staticmethod
    def supports_target(target: GPUTarget):
        return target.backend == BACKEND_NAME

    def __init__(self, target: GPUTarget) -> None:
        super().__init__(target)

    def parse_options(self, opts) -> Any:
        args = {"arch": self.target.arch}
        args.update({k: opts[k] for k in HIPOptions.__dataclass_fields__.keys() if k in opts and opts[k] is not None})
        return HIPOptions(**args)

    def get_codegen_implementation(self, options):
        return {"min_dot_size": lambda lhs_type, rhs_type: (1, 1, 1)}

    def pack_metadata(self, metadata):
        return (metadata.num_warps, metadata.num_ctas, metadata.shared, metadata.cluster_dims[0],
                metadata.cluster_dims[1], metadata.cluster_dims[2], metadata.name)

    def load_dialects(self, ctx):
        return

    @staticmethod
    def make_ttir(mod, metadata, options):
        pm = ir.pass_manager(mod.context)
        pm.enable_debug()
        passes.common.add_inliner(pm)
        if not options.raw_block_pointers:
            passes.ttir.add_rewrite_tensor_pointer(pm)
        passes.ttir.add_rewrite_tensor_descriptor_to_pointer(pm)
        passes.common.add_canonicalizer(pm)
        passes.ttir.add_combine(pm)
        passes.ttir.add_reorder_broadcast(pm)
        passes.common.add_cse(pm)
        passes.ttir.add_triton_licm(pm)
        passes.common.add_symbol_dce(pm)
        passes.ttir.add_loop_unroll(pm)
        passes.common.add_cse(pm)
        pm.run(mod, "make_ttir")
        return mod

    def add_stages(self, stages, options, language=None):
        stages["ttir"] = lambda src, metadata: self.make_ttir(src, metadata, options)
        stages["ttsharedir"] = lambda src, metadata: ttir_to_ttsharedir(src)
        stages["obj"] = lambda src, metadata: ttsharedir_to_obj(src, metadata)

    @functools.lru_cache()
    def hash(self):
        # the planner is part of the compiler: a rebuilt library invalidates cached plans
        h = hashlib.sha256()
        h.update(str(self.target).encode())
        try:
            with open(_native.LIB_PATH, "rb") as f:
                h.update(f.read())
        except OSError:
            pass
        return h.hexdigest()

    def get_module_map(self) -> Dict[str, ModuleType]:
        return {}
