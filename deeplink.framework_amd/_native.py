"""Loads the backend's shared libraries. There is no fallback: a missing library is an error."""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_DIR = os.path.join(HERE, "lib")
RT_PATH = os.path.join(LIB_DIR, "libdipu_amd_rt.so")
IMPL_PATH = os.path.join(LIB_DIR, "libdiopi_impl.so")

_rt = None
_impl = None


class NativeLibraryMissing(RuntimeError):
    pass


def _require(path):
    if not os.path.exists(path):
        raise NativeLibraryMissing(
            f"{path} is not built. Run `python {os.path.join(HERE, 'build.py')}` (needs hipcc); "
            "this backend has no CPU or PyTorch fallback path.")


def runtime():
    """libdipu_amd_rt.so, loaded RTLD_GLOBAL so its diopirt callbacks resolve for the impl library."""
    global _rt
    if _rt is None:
        _require(RT_PATH)
        # torch owns device memory and streams in this host; importing it first makes the HIP
        # runtime it ships (same SONAME) the one these libraries bind to, so stream handles and
        # device pointers are shared rather than belonging to a second runtime instance.
        import torch  # noqa: F401
        _rt = ctypes.CDLL(RT_PATH, mode=ctypes.RTLD_GLOBAL)
    return _rt


def impl():
    """libdiopi_impl.so (the DIOPI operator entry points)."""
    global _impl
    if _impl is None:
        runtime()
        _require(IMPL_PATH)
        _impl = ctypes.CDLL(IMPL_PATH, mode=ctypes.RTLD_GLOBAL)
    return _impl
