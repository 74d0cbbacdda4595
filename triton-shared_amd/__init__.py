"""MI355X (gfx950) execution backend behind triton-shared's plugin surface.

    import triton, triton_shared_amd
    triton_shared_amd.activate()          # registers the backend, sets HIPDriver active
    kernel[grid](*args)                   # unchanged Triton frontend

`activate()` is the counterpart of the reference's
`triton.runtime.driver.set_active(CPUDriver())` (README.md:69-75,
python/examples/conftest.py:5-7).
"""
from . import _native
from .backend.compiler import BACKEND_NAME, HIPBackend, HIPOptions
from .backend.driver import HIPDriver, HIPLauncher, HIPUtils

__all__ = ["BACKEND_NAME", "HIPBackend", "HIPOptions", "HIPDriver", "HIPLauncher", "HIPUtils", "register_backend",
           "activate", "build"]


def register_backend():
    """Makes the backend discoverable by triton.compiler.make_backend without an
    installed entry point: Triton scans the `triton.backends.backends` dict."""
    import triton.backends as tb
    if BACKEND_NAME not in tb.backends:
        tb.backends[BACKEND_NAME] = tb.Backend(compiler=HIPBackend, driver=HIPDriver)


def activate():
    import triton
    register_backend()
    drv = HIPDriver()
    triton.runtime.driver.set_active(drv)
    return drv


def build(verbose=False):
    return _native.build(verbose)
