"""llm_hip: MI355X (gfx950) kernels and host engine for PPLNN's dynamic-batching attention path.

The compute path is the HIP kernel library `lib/libppl_llm_kernel_hip.so` (C ABI declared in
include/ppl_llm_kernel_hip.h). There is no CPU fallback: loading fails loudly when the library is missing.
"""
import ctypes
import os

from . import cabi

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libppl_llm_kernel_hip.so")
_LIB = None


class LibraryMissing(RuntimeError):
    pass


def load_library():
    """dlopen the kernel library and bind every declared symbol. Raises LibraryMissing if it is not built."""
    global _LIB
    if _LIB is None:
        if not os.path.exists(LIB_PATH):
            raise LibraryMissing(
                f"{LIB_PATH} is not built; run `python __graft_entry__.py` (hipcc, --offload-arch=gfx950). "
                "There is no CPU fallback for the attention kernels.")
        # The tests and the bench own device memory through torch, which ships its own HIP runtime under the
        # same soname: load torch's first so that this library binds to that one runtime instead of a second copy.
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        _LIB = cabi.bind(ctypes.CDLL(LIB_PATH))
        _assert_single_hip_runtime()
    return _LIB


def _assert_single_hip_runtime():
    paths = set()
    try:
        with open("/proc/self/maps") as f:
            for line in f:
                if "libamdhip64" in line:
                    paths.add(os.path.realpath(line.split()[-1]))
    except OSError:
        return
    if len(paths) > 1:
        raise RuntimeError(f"two HIP runtimes are loaded in this process: {sorted(paths)}")


def check(rc, what=""):
    if rc != cabi.RC_SUCCESS:
        msg = load_library().pplhip_last_error().decode()
        raise RuntimeError(f"{what} failed: {cabi.RC_NAMES.get(rc, rc)}: {msg}")
