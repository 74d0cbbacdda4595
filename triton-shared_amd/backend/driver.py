"""Triton driver for the MI355X execution backend.

Counterpart of the reference's `CPUDriver` / `CPULauncher` / `CPUUtils`
(backend/driver.py:361-464) with the same surface and the same launcher call
signature (driver.py:262-265).  Differences that follow from running on a GPU:

  * `load_binary` parses the plan bytes once into a native handle, instead of
    handing the object file to a per-kernel launcher that g++ builds at first
    launch (driver.py:249-358);
  * the launch is asynchronous on the HIP stream Triton passes in (torch's
    current stream); the reference runs the grid serially on the calling thread
    and ignores the stream (driver.py:116-133, 441-442);
  * pointer arguments must be device memory: a CPU tensor is rejected.
"""
import sys

from triton.backends.compiler import GPUTarget
from triton.backends.driver import DriverBase

from .. import _native
from .compiler import BACKEND_NAME


def _ty_to_cpp(ty):
    """Scalar typing table of the reference launcher (driver.py:41-64): fp16/bf16
    scalars are not supported there either."""
    if ty[0] == "*":
        return "void*"
    if ty == "constexpr":
        return "PyObject*"
    table = {
        "i1": "int32_t", "i8": "int8_t", "i16": "int16_t", "i32": "int32_t", "i64": "int64_t",
        "u1": "uint32_t", "u8": "uint8_t", "u16": "uint16_t", "u32": "uint32_t", "u64": "uint64_t",
        "fp32": "float", "f32": "float", "fp64": "double",
    }
    if ty not in table:
        raise TypeError(f"scalar kernel arguments of type {ty} are not supported")
    return table[ty]


def _device_pointer(obj, index):
    """int, None or an object with data_ptr(), as driver.py:140-171; host tensors are refused."""
    if obj is None:
        return 0
    if isinstance(obj, int):
        return obj
    data_ptr = getattr(obj, "data_ptr", None)
    if data_ptr is None:
        raise TypeError("Pointer argument must be either uint64 or have data_ptr method")
    device = getattr(obj, "device", None)
    if device is not None and getattr(device, "type", "cuda") != "cuda":
        raise TypeError(f"pointer argument {index} lives on device '{device}'; this backend needs GPU memory")
    p = data_ptr()
    if not isinstance(p, int):
        raise TypeError("data_ptr method of Pointer object must return 64-bit int")
    return p


class HIPLauncher(object):
    """launch(gridX, gridY, gridZ, stream, function, kernel_metadata, launch_metadata,
    launch_enter_hook, launch_exit_hook, *args) -- the call Triton's JIT makes."""

    def __init__(self, src, metadata):
        constants = src.constants if hasattr(src, "constants") else dict()
        arg_index = lambda i: src.fn.arg_names.index(i) if isinstance(i, str) else i
        self.constants = {arg_index(k): v for k, v in constants.items()}
        signature = {arg_index(k): v for k, v in src.signature.items()}
        # positions (in *args) of the runtime arguments, i.e. everything the
        # compiled kernel still takes: constexprs are parsed but not forwarded
        self.slots = []
        for i, ty in signature.items():
            if ty == "constexpr":
                continue
            _ty_to_cpp(ty)
            self.slots.append((i, ty[0] == "*"))

    def __call__(self, gridX, gridY, gridZ, stream, function, kernel_metadata, launch_metadata,
                 launch_enter_hook, launch_exit_hook, *args):
        plan = function
        if not isinstance(plan, _native.PlanHandle):
            raise RuntimeError("kernel was not loaded through HIPUtils.load_binary")
        if launch_enter_hook is not None:
            launch_enter_hook(launch_metadata)
        values = []
        for pos, is_ptr in self.slots:
            v = args[pos]
            values.append(_device_pointer(v, pos) if is_ptr else v)
        if len(values) != len(plan.arg_kinds):
            # arguments specialised to constants (e.g. stride == 1) are not kernel arguments
            raise RuntimeError(
                f"kernel {plan.kernel_name} expects {len(plan.arg_kinds)} runtime arguments, launcher has {len(values)}")
        if gridX * gridY * gridZ > 0:
            plan.launch((gridX, gridY, gridZ), stream, values)
        if launch_exit_hook is not None:
            launch_exit_hook(launch_metadata)


class HIPUtils(object):

    def __new__(cls):
        if not hasattr(cls, "instance"):
            cls.instance = super(HIPUtils, cls).__new__(cls)
        return cls.instance

    @staticmethod
    def get_device_properties(device):
        import torch
        props = torch.cuda.get_device_properties(device)
        return {
            "max_shared_mem": 160 * 1024,
            "multiprocessor_count": props.multi_processor_count,
            "sm_clock_rate": getattr(props, "clock_rate", None),
            "mem_clock_rate": getattr(props, "memory_clock_rate", None),
            "mem_bus_width": getattr(props, "memory_bus_width", None),
        }

    @staticmethod
    def load_binary(name, kernel_obj, shared, device):
        plan = _native.PlanHandle(kernel_obj)
        # (module, function, n_regs, n_spills, n_max_threads).  The module slot must not be None:
        # Triton treats a None module as "handles not initialised yet" and would reload the plan, and
        # with it drop the plan's binding cache, on every launch.
        return (plan, plan, None, None, sys.maxsize)


class HIPDriver(DriverBase):

    def __init__(self):
        super().__init__()
        _native.lib()  # fail now, loudly, if the HIP extension is missing
        self.utils = HIPUtils()
        self.launcher_cls = HIPLauncher
        self.binary_ext = "obj"

    # Never chosen automatically; activate with triton.runtime.driver.set_active(HIPDriver())
    @staticmethod
    def is_active():
        return False

    def get_benchmarker(self):
        from triton.testing import do_bench
        return do_bench

    def get_device_capability(self):
        return ("gfx950", 0)

    def get_current_stream(self, device):
        import torch
        return torch.cuda.current_stream(device).cuda_stream

    def get_current_device(self):
        import torch
        return torch.cuda.current_device()

    def set_current_device(self, device):
        import torch
        torch.cuda.set_device(device)

    def get_current_target(self):
        return GPUTarget(BACKEND_NAME, "gfx950", 64)

    def get_active_torch_device(self):
        import torch
        return torch.device("cuda")

    def get_device_interface(self):
        import torch
        return torch.cuda

    def get_empty_cache_for_benchmark(self):
        import torch
        return torch.empty(256 * 1024 * 1024 // 4, dtype=torch.int, device="cuda")

    def clear_cache(self, cache):
        cache.zero_()

    def assemble_tensormap_to_arg(self, tensormaps_info, args):
        return args

    def map_python_to_cpp_type(self, ty: str) -> str:
        return _ty_to_cpp(ty)
