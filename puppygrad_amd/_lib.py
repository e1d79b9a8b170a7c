"""ctypes binding of libpuppygrad_hip.so (the C ABI in include/puppygrad_hip.h).

The library is loaded from the package directory.  If it has not been built the
loader builds it once with hipcc; if that is impossible it raises, so no caller
ever runs on a silent substitute.
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path

from . import build as _build

PG_OK, PG_ASSET, PG_INVALID_CONFIG, PG_INVALID_INPUT, PG_INVALID_WEIGHTS, PG_BACKEND = range(6)
PG_STORE_F32, PG_STORE_BF16, PG_STORE_INT8 = 0, 1, 2
PG_DECODE_AUTO, PG_DECODE_KERNELS, PG_DECODE_PERSISTENT = 0, 1, 2


class pg_gpt2_config(C.Structure):
    _fields_ = [("vocab_size", C.c_uint64), ("n_positions", C.c_uint64), ("n_embd", C.c_uint64),
                ("n_layer", C.c_uint64), ("n_head", C.c_uint64), ("n_inner", C.c_uint64),
                ("layer_norm_epsilon", C.c_float)]


class pg_tensor(C.Structure):
    _fields_ = [("data", C.POINTER(C.c_float)), ("len", C.c_uint64)]


BLOCK_FIELDS = ["ln_1_g", "ln_1_b", "c_attn_w", "c_attn_b", "c_proj_w", "c_proj_b", "ln_2_g",
                "ln_2_b", "c_fc_w", "c_fc_b", "c_proj_mlp_w", "c_proj_mlp_b"]


class pg_gpt2_block_view(C.Structure):
    _fields_ = [(name, pg_tensor) for name in BLOCK_FIELDS]


class pg_gpt2_weights_view(C.Structure):
    _fields_ = [("wte", pg_tensor), ("wpe", pg_tensor), ("ln_f_g", pg_tensor),
                ("ln_f_b", pg_tensor), ("blocks", C.POINTER(pg_gpt2_block_view)),
                ("n_blocks", C.c_uint64)]


class pg_hip_options(C.Structure):
    _fields_ = [("device", C.c_int32), ("weight_storage", C.c_uint32),
                ("decode_path", C.c_uint32), ("prefill_path", C.c_uint32),
                ("attn_item_keys", C.c_uint32), ("attn_blocks_per_cu", C.c_uint32),
                ("gemm_split_items_per_cu", C.c_uint32), ("gemm_b9_min_rows", C.c_uint32),
                ("seq_gemm_min_tokens", C.c_uint32), ("reserved", C.c_uint32)]


class pg_sampling(C.Structure):
    _fields_ = [("temperature", C.c_float), ("has_top_p", C.c_int32), ("top_p", C.c_float),
                ("has_top_k", C.c_int32), ("top_k", C.c_uint64), ("repeat_penalty", C.c_float),
                ("repeat_last_n", C.c_uint64)]


class pg_rng_state(C.Structure):
    _fields_ = [("state", C.c_uint64)]


class pg_generation_stats(C.Structure):
    _fields_ = [("prompt_tokens", C.c_uint64), ("generated_tokens", C.c_uint64),
                ("prefill_s", C.c_double), ("decode_s", C.c_double),
                ("first_token_s", C.c_double), ("gpu_decode_s", C.c_double)]


class pg_gpt2_operation_profile(C.Structure):
    _fields_ = [(name, C.c_double) for name in (
        "tokenization_s", "layer_norm_s", "qkv_projection_s", "attention_s",
        "attention_projection_s", "mlp_fc_projection_s", "mlp_projection_s", "final_logits_s",
        "decoding_s")]


class pg_device_info(C.Structure):
    _fields_ = [("name", C.c_char * 128), ("arch", C.c_char * 64), ("compute_units", C.c_uint32),
                ("total_mem_bytes", C.c_uint64), ("lds_bytes_per_block", C.c_uint32)]


ON_TOKEN = C.CFUNCTYPE(C.c_int, C.c_uint32, C.c_void_p)

_f32p = C.POINTER(C.c_float)
_u32p = C.POINTER(C.c_uint32)
_vp = C.c_void_p

# name -> (restype, argtypes); every symbol include/puppygrad_hip.h declares.
SIGNATURES = {
    "pg_last_error_message": (C.c_char_p, []),
    "pg_gpt2_create": (C.c_int, [C.POINTER(pg_gpt2_config), C.POINTER(pg_gpt2_weights_view),
                                 C.POINTER(pg_hip_options), C.POINTER(_vp)]),
    "pg_gpt2_destroy": (None, [_vp]),
    "pg_gpt2_get_config": (C.c_int, [_vp, C.POINTER(pg_gpt2_config)]),
    "pg_gpt2_describe": (C.c_int, [_vp, C.c_char_p, C.c_size_t]),
    "pg_kv_cache_create": (C.c_int, [_vp, C.c_uint32, C.POINTER(_vp)]),
    "pg_kv_cache_destroy": (None, [_vp]),
    "pg_kv_cache_clear": (C.c_int, [_vp]),
    "pg_kv_cache_seq_len": (C.c_uint64, [_vp]),
    "pg_kv_cache_max_seq_len": (C.c_uint64, [_vp]),
    "pg_kv_cache_batch": (C.c_uint32, [_vp]),
    "pg_kv_cache_set_seq_len": (C.c_int, [_vp, C.c_uint64]),
    "pg_kv_cache_read_layer": (C.c_int, [_vp, C.c_uint32, C.c_uint32, C.c_uint32, _f32p,
                                         C.c_size_t]),
    "pg_gpt2_prefill": (C.c_int, [_vp, _vp, _u32p, C.c_size_t, C.POINTER(_vp)]),
    "pg_gpt2_forward_one": (C.c_int, [_vp, _vp, C.c_uint32, C.POINTER(_vp)]),
    "pg_gpt2_forward": (C.c_int, [_vp, _u32p, C.c_size_t, _f32p, C.c_size_t]),
    "pg_gpt2_prefill_batch": (C.c_int, [_vp, _vp, _u32p, C.c_size_t, C.POINTER(_vp)]),
    "pg_gpt2_forward_one_batch": (C.c_int, [_vp, _vp, _u32p, C.POINTER(_vp)]),
    "pg_logits_rows": (C.c_uint32, [_vp]),
    "pg_logits_vocab": (C.c_uint64, [_vp]),
    "pg_logits_argmax": (C.c_int, [_vp, _u32p]),
    "pg_logits_copy_to_host": (C.c_int, [_vp, _f32p, C.c_size_t]),
    "pg_sampling_validate": (C.c_int, [C.POINTER(pg_sampling)]),
    "pg_rng_seed": (None, [C.POINTER(pg_rng_state), C.c_uint64]),
    "pg_rng_next_u64": (C.c_uint64, [C.POINTER(pg_rng_state)]),
    "pg_rng_next_unit_f64": (C.c_double, [C.POINTER(pg_rng_state)]),
    "pg_logits_sample": (C.c_int, [_vp, C.c_uint32, _u32p, C.c_size_t, C.POINTER(pg_sampling),
                                   C.POINTER(pg_rng_state), _u32p]),
    "pg_gpt2_decode_greedy": (C.c_int, [_vp, _vp, C.c_uint32, C.c_int64, _u32p, _u32p,
                                        C.POINTER(pg_generation_stats)]),
    "pg_gpt2_decode_greedy_batch": (C.c_int, [_vp, _vp, C.c_uint32, _u32p,
                                              C.POINTER(pg_generation_stats)]),
    "pg_gpt2_stream_token_ids_with_stats": (C.c_int, [_vp, _u32p, C.c_size_t, C.c_uint32,
                                                      C.c_int64, C.POINTER(pg_sampling),
                                                      C.c_uint64, ON_TOKEN, _vp, _u32p,
                                                      C.POINTER(C.c_size_t),
                                                      C.POINTER(pg_generation_stats)]),
    "pg_gpt2_stream_token_ids_profiled": (C.c_int, [_vp, _u32p, C.c_size_t, C.c_uint32,
                                                    C.c_int64, C.POINTER(pg_sampling),
                                                    C.c_uint64, ON_TOKEN, _vp, _u32p,
                                                    C.POINTER(C.c_size_t),
                                                    C.POINTER(pg_generation_stats),
                                                    C.POINTER(pg_gpt2_operation_profile)]),
    "pg_gpt2_prefill_profiled": (C.c_int, [_vp, _vp, _u32p, C.c_size_t, C.POINTER(_vp),
                                           C.POINTER(pg_gpt2_operation_profile)]),
    "pg_op_dense": (C.c_int, [C.c_int32, _f32p, C.c_uint64, C.c_uint64, C.c_uint64, _f32p, _f32p,
                              _f32p]),
    "pg_op_layer_norm": (C.c_int, [C.c_int32, _f32p, C.c_uint64, C.c_uint64, _f32p, _f32p,
                                   C.c_float]),
    "pg_op_gelu": (C.c_int, [C.c_int32, _f32p, C.c_uint64]),
    "pg_op_softmax": (C.c_int, [C.c_int32, _f32p, C.c_uint64, C.c_uint64]),
    "pg_op_add": (C.c_int, [C.c_int32, _f32p, _f32p, C.c_uint64]),
    "pg_op_attention_decode": (C.c_int, [C.c_int32, _f32p, C.c_uint64, _f32p, _f32p, C.c_uint64,
                                         C.c_uint64, C.c_uint64, _f32p]),
    "pg_op_argmax": (C.c_int, [C.c_int32, _f32p, C.c_uint64, _u32p]),
    "pg_device_alloc": (C.c_int, [C.c_int32, C.c_size_t, C.POINTER(_vp)]),
    "pg_device_free": (C.c_int, [C.c_int32, _vp]),
    "pg_device_upload": (C.c_int, [C.c_int32, _vp, _vp, C.c_size_t]),
    "pg_device_download": (C.c_int, [C.c_int32, _vp, _vp, C.c_size_t]),
    "pg_op_dense_dev": (C.c_int, [C.c_int32, _vp, _vp, C.c_uint64, C.c_uint64, C.c_uint64, _vp, _vp, _vp]),
    "pg_op_quantize_rows_dev": (C.c_int, [C.c_int32, _vp, _vp, C.c_uint64, C.c_uint64, _vp, _vp]),
    "pg_op_quantized_dense_dev": (C.c_int, [C.c_int32, _vp, _vp, C.c_uint64, C.c_uint64, C.c_uint64, _vp, _vp, _vp, _vp]),
    "pg_op_dense_in_out_dev": (C.c_int, [C.c_int32, _vp, _vp, C.c_uint64, C.c_uint64, C.c_uint64, _vp,
                                         _vp, _vp]),
    "pg_op_layer_norm_dev": (C.c_int, [C.c_int32, _vp, _vp, C.c_uint64, C.c_uint64, _vp, _vp, C.c_float]),
    "pg_op_gelu_dev": (C.c_int, [C.c_int32, _vp, _vp, C.c_uint64]),
    "pg_op_softmax_dev": (C.c_int, [C.c_int32, _vp, _vp, C.c_uint64, C.c_uint64]),
    "pg_op_add_dev": (C.c_int, [C.c_int32, _vp, _vp, _vp, C.c_uint64]),
    "pg_op_argmax_dev": (C.c_int, [C.c_int32, _vp, _vp, C.c_uint64, _vp]),
    "pg_op_attention_dev": (C.c_int, [C.c_int32, _vp, _vp, _vp, _vp, C.c_uint64, C.c_uint64, C.c_uint64,
                                      C.c_uint64, C.c_int32, _vp]),
    "pg_op_attention_decode_noalloc": (C.c_int, [C.c_int32, _vp, _vp, C.c_uint64, _vp, _vp,
                                                 C.c_uint64, C.c_uint64, C.c_uint64, _vp]),
    "pg_debug_sample_counts": (None, [C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]),
    "pg_debug_sample_train": (C.c_int, [C.c_int]),
    "pg_kv_cache_debug_epoch": (C.c_uint32, [_vp]),
    "pg_kv_cache_debug_set_epoch": (C.c_int, [_vp, C.c_uint32]),
    "pg_tensor_store_open": (C.c_int, [C.c_char_p, C.POINTER(_vp)]),
    "pg_tensor_store_close": (None, [_vp]),
    "pg_tensor_store_len": (C.c_uint64, [_vp]),
    "pg_tensor_store_required_f32": (C.c_int, [_vp, C.c_char_p, C.POINTER(C.c_uint64), C.c_size_t,
                                               C.POINTER(pg_tensor)]),
    "pg_tensor_store_optional_f32": (C.c_int, [_vp, C.c_char_p, C.POINTER(C.c_uint64), C.c_size_t,
                                               C.POINTER(C.c_int32), C.POINTER(pg_tensor)]),
    "pg_gpt2_load_config": (C.c_int, [C.c_char_p, C.POINTER(pg_gpt2_config)]),
    "pg_hip_load_tuning": (C.c_int, [C.c_char_p, C.POINTER(pg_hip_options), C.POINTER(C.c_int32)]),
    "pg_gpt2_create_from_dir": (C.c_int, [C.c_char_p, C.POINTER(pg_hip_options), C.POINTER(_vp)]),
    "pg_synth_normal_f32": (None, [_f32p, C.c_uint64, C.c_uint64, C.c_uint64, C.c_double]),
    "pg_synth_token_ids": (None, [_u32p, C.c_uint64, C.c_uint64, C.c_uint64]),
    "pg_device_query": (C.c_int, [C.c_int32, C.POINTER(pg_device_info)]),
}

_lib = None


def lib_path() -> Path:
    """The built library; PUPPYGRAD_HIP_LIB names another build of it (e.g. one with the
    decode kernel's development timestamps compiled in)."""
    import os
    override = os.environ.get("PUPPYGRAD_HIP_LIB")
    return Path(override) if override else _build.LIB_PATH


def load() -> C.CDLL:
    """Load the built library (building it first only if no built file exists)."""
    global _lib
    if _lib is not None:
        return _lib
    path = lib_path()
    if not path.exists():
        _build.build_library(verbose=False)
    lib = C.CDLL(str(path))
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError here means header and library disagree
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def f32p(arr):
    return arr.ctypes.data_as(_f32p)


def u32p(arr):
    return arr.ctypes.data_as(_u32p)
