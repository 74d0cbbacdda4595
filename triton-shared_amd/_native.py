"""ctypes binding of libtts_hip.so (C ABI declared in include/tts_hip.h)."""
import ctypes
import os
import subprocess

_CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
LIB_PATH = os.path.join(_CSRC, "libtts_hip.so")

TTS_OK, TTS_UNSUPPORTED, TTS_INVALID, TTS_HIP_ERROR = 0, 1, 2, 3
ARG_PTR, ARG_INT, ARG_FLOAT = 0, 1, 2


class _ArgValue(ctypes.Union):
    _fields_ = [("ptr", ctypes.c_void_p), ("i", ctypes.c_int64), ("f", ctypes.c_double)]


class TtsArg(ctypes.Structure):
    _fields_ = [("kind", ctypes.c_int32), ("reserved", ctypes.c_int32), ("v", _ArgValue)]


def build(verbose=False):
    """Compiles the library in-tree with hipcc for gfx950 (cross-compiles without a GPU)."""
    cmd = ["make", "-C", _CSRC, "-j8", "all"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("building libtts_hip.so failed:\n" + res.stdout[-4000:] + res.stderr[-4000:])
    if verbose:
        print(res.stdout)
    return LIB_PATH


_lib = None


def lib():
    """Loads the library; fails loudly if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: the HIP extension has not been built "
            "(run `python -c 'import __graft_entry__ as g; g.build()'` or `make -C triton-shared_amd/csrc`)")
    L = ctypes.CDLL(LIB_PATH)
    c_char_pp = ctypes.POINTER(ctypes.c_char_p)
    L.tts_last_error.restype = ctypes.c_char_p
    L.tts_free.argtypes = [ctypes.c_void_p]
    L.tts_ttir_to_structured.argtypes = [ctypes.c_char_p, ctypes.POINTER(ctypes.c_void_p)]
    L.tts_structured_to_plan.argtypes = [ctypes.c_char_p, ctypes.POINTER(ctypes.c_void_p),
                                         ctypes.POINTER(ctypes.c_size_t), ctypes.POINTER(ctypes.c_void_p)]
    L.tts_plan_load.argtypes = [ctypes.c_char_p, ctypes.c_size_t, ctypes.POINTER(ctypes.c_void_p)]
    L.tts_plan_destroy.argtypes = [ctypes.c_void_p]
    for name in ("tts_plan_kernel_name", "tts_plan_family", "tts_plan_signature", "tts_plan_last_kernel"):
        getattr(L, name).argtypes = [ctypes.c_void_p]
        getattr(L, name).restype = ctypes.c_char_p
    L.tts_plan_num_args.argtypes = [ctypes.c_void_p]
    L.tts_plan_arg_kind.argtypes = [ctypes.c_void_p, ctypes.c_int]
    L.tts_plan_describe_launch.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                           ctypes.POINTER(TtsArg), ctypes.c_int, ctypes.POINTER(ctypes.c_void_p)]
    L.tts_launch.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
                             ctypes.POINTER(TtsArg), ctypes.c_int]
    L.tts_launch_noalloc.argtypes = L.tts_launch.argtypes
    _lib = L
    return L


def _raise(status):
    msg = lib().tts_last_error().decode("utf-8", "replace")
    if status == TTS_UNSUPPORTED:
        raise NotImplementedError(msg)
    if status == TTS_INVALID:
        raise ValueError(msg)
    raise RuntimeError(msg)


def _take_string(p):
    s = ctypes.string_at(p).decode("utf-8")
    lib().tts_free(p)
    return s


def ttir_to_structured(ttir_text: str) -> str:
    out = ctypes.c_void_p()
    st = lib().tts_ttir_to_structured(ttir_text.encode("utf-8"), ctypes.byref(out))
    if st != TTS_OK:
        _raise(st)
    return _take_string(out)


def structured_to_plan(structured_text: str):
    """Returns (plan_bytes, kernel_name)."""
    out, name, n = ctypes.c_void_p(), ctypes.c_void_p(), ctypes.c_size_t()
    st = lib().tts_structured_to_plan(structured_text.encode("utf-8"), ctypes.byref(out), ctypes.byref(n),
                                      ctypes.byref(name))
    if st != TTS_OK:
        _raise(st)
    data = ctypes.string_at(out, n.value)
    lib().tts_free(out)
    return data, _take_string(name)


class PlanHandle:
    """Owns a tts_plan*."""

    def __init__(self, plan_bytes: bytes):
        h = ctypes.c_void_p()
        st = lib().tts_plan_load(plan_bytes, len(plan_bytes), ctypes.byref(h))
        if st != TTS_OK:
            _raise(st)
        self._h = h
        L = lib()
        self.kernel_name = L.tts_plan_kernel_name(h).decode()
        self.family = L.tts_plan_family(h).decode()
        self.signature = L.tts_plan_signature(h).decode()
        self.arg_kinds = [L.tts_plan_arg_kind(h, i) for i in range(L.tts_plan_num_args(h))]

    def __del__(self):
        try:
            if self._h:
                lib().tts_plan_destroy(self._h)
                self._h = None
        except Exception:
            pass

    def pack(self, values):
        """values: one Python value per kernel argument (int pointer / int / float)."""
        n = len(self.arg_kinds)
        if len(values) != n:
            raise ValueError(f"kernel {self.kernel_name} takes {n} arguments, got {len(values)}")
        arr = (TtsArg * n)()
        for i, (k, v) in enumerate(zip(self.arg_kinds, values)):
            arr[i].kind = k
            if k == ARG_PTR:
                arr[i].v.ptr = v
            elif k == ARG_INT:
                arr[i].v.i = int(v)
            else:
                arr[i].v.f = float(v)
        return arr

    def describe_launch(self, grid, values):
        arr = self.pack(values)
        out = ctypes.c_void_p()
        st = lib().tts_plan_describe_launch(self._h, grid[0], grid[1], grid[2], arr, len(values), ctypes.byref(out))
        if st != TTS_OK:
            _raise(st)
        text = _take_string(out)
        return dict(line.split("=", 1) for line in text.strip().splitlines())

    def launch_packed(self, grid, stream, arr, n):
        st = lib().tts_launch(self._h, grid[0], grid[1], grid[2], stream, arr, n)
        if st != TTS_OK:
            _raise(st)

    def launch_noalloc(self, grid, stream, values):
        """tts_launch_noalloc: the launch for callers that cannot allocate device memory."""
        arr = self.pack(values)
        st = lib().tts_launch_noalloc(self._h, grid[0], grid[1], grid[2], stream, arr, len(values))
        if st != TTS_OK:
            _raise(st)

    def launch(self, grid, stream, values):
        arr = self.pack(values)
        self.launch_packed(grid, stream, arr, len(values))

    @property
    def last_kernel(self):
        return lib().tts_plan_last_kernel(self._h).decode()
