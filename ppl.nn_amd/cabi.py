"""ctypes mirror of include/ppl_llm_kernel_hip.h (field order and types must match the header exactly)."""
import ctypes as C

RC_SUCCESS = 0
RC_OTHER_ERROR = 1
RC_UNSUPPORTED = 2
RC_OUT_OF_MEMORY = 3
RC_INVALID_VALUE = 4
RC_EXISTS = 5
RC_NOT_FOUND = 6
RC_PERMISSION_DENIED = 7
RC_HOST_MEMORY_ERROR = 8
RC_DEVICE_MEMORY_ERROR = 9
RC_DEVICE_RUNTIME_ERROR = 10
RC_OUT_OF_RANGE = 11
RC_INTERNAL_ERROR = 12

RC_NAMES = {
    0: "RC_SUCCESS", 1: "RC_OTHER_ERROR", 2: "RC_UNSUPPORTED", 3: "RC_OUT_OF_MEMORY", 4: "RC_INVALID_VALUE",
    5: "RC_EXISTS", 6: "RC_NOT_FOUND", 7: "RC_PERMISSION_DENIED", 8: "RC_HOST_MEMORY_ERROR",
    9: "RC_DEVICE_MEMORY_ERROR", 10: "RC_DEVICE_RUNTIME_ERROR", 11: "RC_OUT_OF_RANGE", 12: "RC_INTERNAL_ERROR",
}

_p = C.c_void_p
_i32 = C.c_int32
_i64 = C.c_int64


class MhcaArgs(C.Structure):
    _fields_ = [
        ("d_query", _p), ("d_current_key", _p), ("d_current_value", _p), ("d_attn_mask", _p),
        ("d_seqstarts", _p), ("d_kvstarts", _p), ("d_cachestarts", _p), ("d_start_pos", _p),
        ("d_alibi_slopes", _p),
        ("is_causal", _i32),
        ("batch", _i64), ("decoding_batches", _i64), ("max_seqlen", _i64), ("max_kvlen", _i64),
        ("layer_idx", _i32), ("num_layer", _i32), ("num_heads", _i32), ("num_kv_heads", _i32),
        ("head_dim", _i32), ("cache_mode", _i32), ("page_size", _i32),
        ("cache_stride_s", _i64), ("cache_stride_l", _i64), ("cache_stride_h", _i64), ("cache_stride_kv", _i64),
        ("cachestart_stride_b", _i64),
        ("enable_cache_prefill", _i32), ("enable_decoding_sharemem_mhca", _i32),
        ("enable_decoding_infinity_mhca", _i32), ("enable_decoding_infinity_gqca", _i32),
        ("specify_decoding_attn_split_k", _i32), ("specify_decoding_attn_tpb", _i32),
        ("d_cache", _p), ("d_scale", _p), ("d_output", _p),
        ("total_new_tokens", _i64),
        ("attn_mask_stride_h", _i64), ("attn_mask_stride_q", _i64),
    ]


class MhcaPlan(C.Structure):
    _fields_ = [
        ("workspace_bytes", C.c_uint64),
        ("decode_num_ranges", _i32), ("decode_heads_per_block", _i32), ("decode_waves_per_block", _i32),
        ("prefill_q_tile", _i32), ("prefill_num_q_tiles", _i32),
        ("prefill_staging", _i32), ("prefill_staging_offset_256", _i32),
        ("general_kernel", _i32), ("general_decode_splits", _i32),
    ]


class KvWriteArgs(C.Structure):
    _fields_ = [
        ("d_current_key", _p), ("d_current_value", _p),
        ("d_seqstarts", _p), ("d_cachestarts", _p), ("d_start_pos", _p),
        ("batch", _i64), ("total_new_tokens", _i64),
        ("layer_idx", _i32), ("num_layer", _i32), ("num_kv_heads", _i32), ("head_dim", _i32),
        ("cache_stride_s", _i64), ("cache_stride_l", _i64), ("cache_stride_h", _i64), ("cache_stride_kv", _i64),
        ("d_cache", _p), ("d_scale", _p),
        ("cache_mode", _i32), ("page_size", _i32), ("cachestart_stride_b", _i64),
    ]


class KvCacheArgs(C.Structure):
    _fields_ = [
        ("write", KvWriteArgs),
        ("d_kvstarts", _p),
        ("total_kv_tokens", _i64), ("max_kvlen", _i64),
        ("num_repeat", _i32), ("cache_mode", _i32), ("cache_layout", _i32), ("reserved", _i32),
        ("d_key_out", _p), ("d_value_out", _p),
    ]


class MhaArgs(C.Structure):
    _fields_ = [
        ("d_query", _p), ("d_key", _p), ("d_value", _p), ("d_attn_mask", _p),
        ("d_seqstarts", _p), ("d_kvstarts", _p),
        ("is_causal", _i32), ("is_alibi", _i32),
        ("batch", _i64), ("decoding_batches", _i64), ("max_seqlen", _i64), ("max_kvlen", _i64),
        ("num_heads", _i32), ("num_kv_heads", _i32), ("head_dim", _i32), ("reserved", _i32),
        ("d_output", _p),
        ("attn_mask_stride_h", _i64), ("attn_mask_stride_q", _i64),
    ]


class RopeArgs(C.Structure):
    _fields_ = [
        ("d_query", _p), ("d_key", _p), ("d_start_pos", _p), ("d_seqstarts", _p),
        ("theta", C.c_float), ("bypass_key", _i32), ("rotary_dim", _i32), ("pair_layout", _i32),
        ("batch", _i64), ("total_tokens", _i64),
        ("num_heads", _i32), ("num_key_heads", _i32), ("head_dim", _i32), ("max_position_embeddings", _i32),
        ("max_seqlen", _i64),
        ("scaling_type", _i32), ("scaling_factor", C.c_float),
        ("d_rotated_query", _p), ("d_rotated_key", _p),
    ]


ROPE_PAIRS_INTERLEAVED, ROPE_PAIRS_HALF_SPLIT = 0, 1
ROPE_SCALING_NONE, ROPE_SCALING_LINEAR, ROPE_SCALING_DYNAMIC = 0, 1, 2


class PackArgs(C.Structure):
    _fields_ = [
        ("d_slot_kvlen", _p), ("d_slot_newlen", _p), ("d_slot_cachestart", _p),
        ("num_slots", _i32), ("advance_slots", _i32),
        ("d_seqstarts", _p), ("d_kvstarts", _p), ("d_cachestarts", _p), ("d_start_pos", _p),
        ("d_batch_slots", _p), ("d_header", _p),
    ]


# name -> (restype, argtypes); every symbol the header declares
PROTOTYPES = {
    "pplhip_last_error": (C.c_char_p, []),
    "pplhip_version": (_i32, []),
    "pplhip_init": (_i32, []),
    "pplhip_mhca_prepare": (_i32, [C.POINTER(MhcaArgs), C.POINTER(MhcaPlan)]),
    "pplhip_mhca_forward": (_i32, [C.POINTER(MhcaArgs), C.POINTER(MhcaPlan), _p, _p]),
    "pplhip_mhca_forward_noalloc": (_i32, [C.POINTER(MhcaArgs), C.POINTER(MhcaPlan), _p]),
    "pplhip_mha_forward": (_i32, [C.POINTER(MhaArgs), _p]),
    "pplhip_rope_forward": (_i32, [C.POINTER(RopeArgs), _p]),
    "pplhip_rope_kv_write_forward": (_i32, [C.POINTER(RopeArgs), C.POINTER(KvWriteArgs), _p]),
    "pplhip_position_index": (_i32, [_p, _p, _i64, _i64, _i64, _p, _p]),
    "pplhip_kv_quantize_write": (_i32, [C.POINTER(KvWriteArgs), _p]),
    "pplhip_kv_cache_forward": (_i32, [C.POINTER(KvCacheArgs), _p]),
    "pplhip_pack_tables": (_i32, [C.POINTER(PackArgs), _p]),
    "pplhip_advance_slots": (_i32, [_p, _p, _i32, _p]),
    "pplhip_check_tables": (_i32, [C.POINTER(MhcaArgs), _i64, _p, _p]),
    "pplhip_check_tables_host": (_i32, [C.POINTER(MhcaArgs), _i64, _p]),
}

# the measurement / verification aids of libppl_llm_kernel_hip_probes.so (include/ppl_llm_kernel_hip_probes.h)
PROBE_PROTOTYPES = {
    "pplhip_probe_last_error": (C.c_char_p, []),
    "pplhip_probe_mfma_f16": (_i32, [_p, _p, _i32, _i32, C.POINTER(C.c_double), _p]),
    "pplhip_probe_hbm_read": (_i32, [_p, C.c_uint64, _p, _i32, C.POINTER(C.c_uint64), _p]),
    "pplhip_probe_quantizer": (_i32, [_p, _p]),
    "pplhip_probe_slab_row": (_i32, [_i64, _i64, _i64, _i64, _i32, _i64, _i32, _i32, C.POINTER(_i64), C.POINTER(_i64)]),
}

TABLES_OK, TABLES_BAD_SEQSTARTS, TABLES_BAD_KVSTARTS, TABLES_KVLEN_MISMATCH = 0, 1, 2, 3
TABLES_BAD_DECODE_ORDER, TABLES_MAX_EXCEEDED, TABLES_SLAB_RANGE, TABLES_PAGE_TABLE_TOO_SHORT = 4, 5, 6, 7


def bind(lib, prototypes=None):
    """Attach prototypes to a loaded CDLL; raises AttributeError when a declared symbol is missing."""
    for name, (res, args) in (PROTOTYPES if prototypes is None else prototypes).items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


def cache_strides_layout0(num_layer, num_kv_heads, head_dim):
    """(MaxT, L, 2, KVH, Dh) strides, as computed at multi_head_cache_attention_kernel.cc:141-148."""
    return dict(
        cache_stride_s=num_layer * 2 * num_kv_heads * head_dim,
        cache_stride_l=2 * num_kv_heads * head_dim,
        cache_stride_h=head_dim,
        cache_stride_kv=num_kv_heads * head_dim,
    )


def cache_strides_layout3(num_layer, num_kv_heads, head_dim, max_tokens):
    """(L, 2, KVH, MaxT, Dh) strides, as computed at multi_head_cache_attention_kernel.cc:149-155."""
    return dict(
        cache_stride_s=head_dim,
        cache_stride_l=2 * num_kv_heads * max_tokens * head_dim,
        cache_stride_h=max_tokens * head_dim,
        cache_stride_kv=num_kv_heads * max_tokens * head_dim,
    )
