"""llm_hip: MI355X (gfx950) kernels and host engine for PPLNN's dynamic-batching attention path.

The compute path is the HIP kernel library `lib/libppl_llm_kernel_hip.so` (C ABI declared in
include/ppl_llm_kernel_hip.h). There is no CPU fallback: loading fails loudly when the library is missing.
"""
import ctypes
import os

from . import cabi

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libppl_llm_kernel_hip.so")
CONSERVATIVE_WAITS_LIB_PATH = os.path.join(_HERE, "lib", "libppl_llm_kernel_hip_conservative_waits.so")
PROBES_LIB_PATH = os.path.join(_HERE, "lib", "libppl_llm_kernel_hip_probes.so")
_LIB = None
_CHECK_LIB = None
_PROBES = None


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


def load_conservative_waits_library():
    """The checking build of the kernel library (every hand-counted wait of the decode kernel replaced by a wait
    for everything in flight). For tests that compare it bit for bit with the product build; nothing else loads it."""
    global _CHECK_LIB
    if _CHECK_LIB is None:
        if not os.path.exists(CONSERVATIVE_WAITS_LIB_PATH):
            raise LibraryMissing(f"{CONSERVATIVE_WAITS_LIB_PATH} is not built; run `python __graft_entry__.py`")
        load_library()
        _CHECK_LIB = cabi.bind(ctypes.CDLL(CONSERVATIVE_WAITS_LIB_PATH))
        _assert_single_hip_runtime()
    return _CHECK_LIB


def load_probe_library():
    """The roofline probes and the quantiser enumeration (measurement / verification aids; not part of the drop-in
    ABI): for the benchmark and the tests only."""
    global _PROBES
    if _PROBES is None:
        if not os.path.exists(PROBES_LIB_PATH):
            raise LibraryMissing(f"{PROBES_LIB_PATH} is not built; run `python __graft_entry__.py`")
        load_library()
        _PROBES = cabi.bind(ctypes.CDLL(PROBES_LIB_PATH), cabi.PROBE_PROTOTYPES)
        _assert_single_hip_runtime()
    return _PROBES


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


ENGINE_LIB_PATH = os.path.join(_HERE, "lib", "libpplnn_llm_hip.so")
_ENGINE = None


def load_engine_library():
    """dlopen the llm_hip host engine (C++) and bind its flat C entry points."""
    global _ENGINE
    if _ENGINE is None:
        load_library()  # the kernel library (and torch's HIP runtime, when present) first
        if not os.path.exists(ENGINE_LIB_PATH):
            raise LibraryMissing(f"{ENGINE_LIB_PATH} is not built; run `python __graft_entry__.py`.")
        L = ctypes.CDLL(ENGINE_LIB_PATH)
        vp, u32, u64, i64p = ctypes.c_void_p, ctypes.c_uint32, ctypes.c_uint64, ctypes.POINTER(ctypes.c_int64)
        sig = {
            "pplnn_hip_last_error": (ctypes.c_char_p, []),
            "pplnn_hip_set_log_level": (None, [ctypes.c_int]),
            "pplnn_hip_engine_create": (vp, [u32, u32]),
            "pplnn_hip_engine_create_on_stream": (vp, [u32, u32, vp]),
            "pplnn_hip_engine_name": (ctypes.c_char_p, [vp]),
            "pplnn_hip_engine_configure_u32": (u32, [vp, u32, u32]),
            "pplnn_hip_engine_destroy": (None, [vp]),
            "pplnn_hip_builder_create": (vp, []),
            "pplnn_hip_builder_load_model": (u32, [vp, ctypes.c_char_p, u64]),
            "pplnn_hip_builder_load_model_file": (u32, [vp, ctypes.c_char_p]),
            "pplnn_hip_builder_set_engine": (u32, [vp, vp]),
            "pplnn_hip_builder_preprocess": (u32, [vp]),
            "pplnn_hip_builder_create_runtime": (vp, [vp]),
            "pplnn_hip_builder_destroy": (None, [vp]),
            "pplnn_hip_engine_configure_str": (u32, [vp, u32, ctypes.c_char_p]),
            "pplnn_hip_runtime_set_inputs_from_files": (u32, [vp, ctypes.c_char_p]),
            "pplnn_hip_runtime_save_outputs": (u32, [vp, ctypes.c_char_p]),
            "pplnn_hip_builder_serialize_op": (u32, [vp, ctypes.c_char_p, vp, ctypes.c_uint64,
                                                     ctypes.POINTER(ctypes.c_uint64)]),
            "pplnn_hip_builder_deserialize_op": (u32, [vp, ctypes.c_char_p, ctypes.c_char_p, ctypes.c_uint64]),
            "pplnn_hip_runtime_input_count": (u32, [vp]),
            "pplnn_hip_runtime_output_count": (u32, [vp]),
            "pplnn_hip_runtime_input": (vp, [vp, u32]),
            "pplnn_hip_runtime_output": (vp, [vp, u32]),
            "pplnn_hip_runtime_run": (u32, [vp]),
            "pplnn_hip_runtime_run_async": (u32, [vp]),
            "pplnn_hip_runtime_synchronize": (u32, [vp]),
            "pplnn_hip_runtime_set_profiling": (u32, [vp, u32]),
            "pplnn_hip_runtime_profiling": (u32, [vp, ctypes.POINTER(u64), ctypes.POINTER(u32), u32]),
            "pplnn_hip_runtime_destroy": (None, [vp]),
            "pplnn_hip_tensor_name": (ctypes.c_char_p, [vp]),
            "pplnn_hip_tensor_reshape": (None, [vp, i64p, u32]),
            "pplnn_hip_tensor_dims": (u32, [vp, i64p, u32]),
            "pplnn_hip_tensor_dtype": (u32, [vp]),
            "pplnn_hip_tensor_set_buffer_ptr": (None, [vp, vp]),
            "pplnn_hip_tensor_buffer_ptr": (vp, [vp]),
            "pplnn_hip_tensor_copy_from_host": (u32, [vp, vp]),
            "pplnn_hip_tensor_copy_to_host": (u32, [vp, vp]),
            "pplnn_hip_tensor_use_host_device": (None, [vp]),
            "pplnn_hip_selftest_registry": (u32, []),
            "pplnn_x86_engine_create": (vp, []),
            "pplnn_x86_set_num_threads": (None, [ctypes.c_int]),
            "pplnn_x86_get_num_threads": (ctypes.c_int, []),
            "pplnn_hip_arena_create_host": (vp, [u64, u64]),
            "pplnn_hip_arena_create_host_with_policy": (vp, [u64, u64, u32]),
            "pplnn_hip_arena_alloc": (u32, [vp, u64, ctypes.POINTER(vp), ctypes.POINTER(u64)]),
            "pplnn_hip_arena_free": (None, [vp, vp]),
            "pplnn_hip_arena_buffered_bytes": (u64, [vp]),
            "pplnn_hip_arena_used_bytes": (u64, [vp]),
            "pplnn_hip_arena_destroy": (None, [vp]),
        }
        for name, (res, args) in sig.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _ENGINE = L
    return _ENGINE
