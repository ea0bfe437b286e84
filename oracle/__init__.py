"""TEST INFRASTRUCTURE ONLY: ctypes loader for the scalar CPU oracle (oracle/liboracle.so).

May be imported from tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg only.
Argument blocks are the ctypes structures of the product's C ABI, filled with HOST pointers.
"""
import ctypes as C
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def build():
    subprocess.check_call(["make", "-C", _HERE, "-s"])


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(path):
            build()
        L = C.CDLL(path)
        vp, i64 = C.c_void_p, C.c_int64
        L.oracle_half_to_float.argtypes = [vp, vp, i64]
        L.oracle_float_to_half.argtypes = [vp, vp, i64]
        L.oracle_kv_quantize_groups.argtypes = [vp, vp, vp, i64]
        L.oracle_kv_dequant_groups.argtypes = [vp, vp, vp, i64]
        L.oracle_kv_quantize_write.argtypes = [vp]
        L.oracle_kv_quantize_write.restype = C.c_int
        L.oracle_mhca_forward.argtypes = [vp, vp]
        L.oracle_mhca_forward.restype = C.c_int
        L.oracle_mha_forward.argtypes = [vp, vp]
        L.oracle_mha_forward.restype = C.c_int
        L.oracle_rope_forward.argtypes = [vp]
        L.oracle_rope_forward.restype = C.c_int
        L.oracle_position_index.argtypes = [vp, vp, i64, vp]
        L.oracle_position_index.restype = C.c_int
        L.oracle_kv_cache_forward.argtypes = [vp]
        L.oracle_kv_cache_forward.restype = C.c_int
        L.oracle_pack_tables.argtypes = [vp]
        L.oracle_pack_tables.restype = C.c_int
        _LIB = L
    return _LIB
