"""ctypes loader of ``lib/libmummu_moe.so`` (the HIP library behind include/mummu_moe.h).

The library is built in-tree by ``python -m mummu_amd.build``.  Loading fails loudly when it
is missing: there is no CPU fallback anywhere in this package.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libmummu_moe.so")

F32, F16, Q8_0, Q4_K, BF16 = 0, 1, 8, 12, 30
Q4_0, Q4_1, Q5_0, Q5_1, Q5_K, Q6_K = 2, 3, 6, 7, 13, 14
# ggml type id -> (elements per block, bytes per block)
BLOCKS = {F32: (1, 4), F16: (1, 2), BF16: (1, 2), Q4_0: (32, 18), Q4_1: (32, 20), Q5_0: (32, 22), Q5_1: (32, 24),
          Q8_0: (32, 34), Q4_K: (256, 144), Q5_K: (256, 176), Q6_K: (256, 210)}
ROUTER_SPARSE_MOE, ROUTER_QWEN4EXP = 0, 1

(OK, ERR_CONFIG, ERR_TYPE, ERR_BLOCKS, ERR_TOPK, ERR_SHAPE, ERR_NONFINITE, ERR_RANGE, ERR_NOT_LOADED, ERR_TOKENS,
 ERR_DEVICE, ERR_ARG, ERR_IO, ERR_GGUF, ERR_SAFETENSORS, ERR_STALE) = range(16)

STATUS_NAMES = ["ok", "config", "type", "blocks", "topk", "shape", "nonfinite", "range", "not_loaded", "tokens",
                "device", "arg", "io", "gguf", "safetensors", "stale"]


class Config(C.Structure):
    """mummu_moe_config."""
    _fields_ = [
        ("hidden_size", C.c_int32), ("expert_intermediate_size", C.c_int32), ("num_experts", C.c_int32),
        ("num_experts_per_tok", C.c_int32), ("norm_topk_prob", C.c_int32), ("router_flavour", C.c_int32),
        ("num_layers", C.c_int32), ("max_tokens", C.c_int32), ("rms_norm_eps", C.c_float),
    ]


class GgufTensor(C.Structure):
    """mummu_gguf_tensor."""
    _fields_ = [
        ("name", C.c_char_p), ("n_dims", C.c_int32), ("dims", C.c_int64 * 4), ("ggml_type", C.c_int32),
        ("shard", C.c_int32), ("file_offset", C.c_uint64), ("nbytes", C.c_uint64), ("path", C.c_char_p),
    ]


class StTensor(C.Structure):
    """mummu_st_tensor."""
    _fields_ = [
        ("name", C.c_char_p), ("dtype", C.c_char_p), ("n_dims", C.c_int32), ("dims", C.c_int64 * 8), ("shard", C.c_int32),
        ("file_offset", C.c_uint64), ("nbytes", C.c_uint64), ("path", C.c_char_p),
    ]


class GgufMoeLayer(C.Structure):
    """mummu_gguf_moe_layer."""
    _fields_ = [("router", C.c_int32), ("gate", C.c_int32), ("up", C.c_int32), ("down", C.c_int32), ("norm", C.c_int32)]


# name -> (restype, argtypes); the list the header declares, checked against the .so by the tests
_P, _I, _I64, _SZ = C.c_void_p, C.c_int, C.c_int64, C.c_size_t
SIGNATURES = {
    "mummu_device_count": (_I, []),
    "mummu_moe_last_error": (C.c_char_p, [_P]),
    "mummu_moe_create": (_I, [C.POINTER(Config), C.POINTER(_P)]),
    "mummu_moe_destroy": (None, [_P]),
    "mummu_moe_load_layer": (_I, [_P, _I, _P, _I, _P, _I, _P, _I, _P, _I, _P]),
    "mummu_moe_load_shared_expert": (_I, [_P, _I, _I, _P, _I, _P, _I, _P, _I, _P, _I]),
    "mummu_moe_get_config": (_I, [_P, _P]),
    "mummu_moe_resident_bytes": (C.c_uint64, [_P]),
    "mummu_moe_batched_from": (C.c_int, [_P, C.c_int]),
    "mummu_moe_forward_typed": (_I, [_P, _I, _P, _I, _I64, _I, _I, _P]),
    "mummu_moe_forward": (_I, [_P, _I, _P, _I64, _I, _I, _P]),
    "mummu_moe_route": (_I, [_P, _I, _P, _I64, _I, _I, _P, _P, _P]),
    "mummu_route_logits": (_I, [_P, _P, _I64, _I, _I, _I, _I, _P, _P]),
    "mummu_moe_routed": (_I, [_P, _I, _P, _P, _I64, _I, _P]),
    "mummu_moe_apply_routing": (_I, [_P, _I, _P, _P, _P, _I64, _I, _P]),
    "mummu_expert_run": (_I, [_P, _I, _I, _P, _I64, _I, _P]),
    "mummu_expert_run_device": (_I, [_P, _I, _I, _P, _I64, _I, _P, _P]),
    "mummu_expert_gate_energy": (_I, [_P, _I, _I, _P, _I64, _I, _P]),
    "mummu_packed_last_error": (C.c_char_p, []),
    "mummu_packed_weight_create": (_I, [_P, _P, _I, _I, _I, _P]),
    "mummu_packed_weight_wrap_device": (_I, [_P, _P, _I, _I, _I, _P]),
    "mummu_packed_weight_destroy": (None, [_P]),
    "mummu_packed_weight_bytes": (C.c_uint64, [_P]),
    "mummu_q4s_gemv": (_I, [_P, _P, _I64, _I, _P]),
    "mummu_q4s_gemv_device": (_I, [_P, _P, _I64, _I, _P, _P]),
    "mummu_moe_take_hits": (_I, [_P, _I, _P]),
    "mummu_moe_stack_forward": (_I, [_P, _P, _I64, _I, _I, _P, _P]),
    "mummu_dequantize": (_I, [_I, _P, _SZ, _P]),
    "mummu_moe_dequantize_expert": (_I, [_P, _I, _I, _I, _P]),
    "mummu_moe_forward_device": (_I, [_P, _I, _P, _I64, _I, _I, _P, _P]),
    "mummu_moe_forward_device_noalloc": (_I, [_P, _I, _P, _I64, _I, _I, _P, _P]),
    "mummu_moe_stack_forward_device": (_I, [_P, _P, _I64, _I, _I, _P, _P]),
    "mummu_moe_set_router_exchange": (_I, [_P, _I, C.c_uint]),
    "mummu_moe_router_exchange_state": (_I, [_P, C.POINTER(C.c_int), C.POINTER(C.c_uint64)]),
    "mummu_moe_set_layer_fusion": (_I, [_P, _I]),
    "mummu_moe_set_deferred_combine": (_I, [_P, _I]),
    "mummu_moe_set_tile_order": (_I, [_P, _I]),
    "mummu_moe_flush": (_I, [_P]),
    "mummu_moe_check": (_I, [_P, _P]),
    "mummu_moe_last_routing": (_I, [_P, _I64, _I, _P, _P]),
    "mummu_device_alloc": (_P, [_SZ]),
    "mummu_device_free": (None, [_P]),
    "mummu_copy_to_device": (_I, [_P, _P, _SZ]),
    "mummu_copy_to_host": (_I, [_P, _P, _SZ]),
    "mummu_device_synchronize": (_I, []),
    "mummu_device_name": (_I, [C.c_char_p, _SZ]),
    "mummu_moe_stream": (_P, [_P]),
    "mummu_graph_begin": (_I, [_P]),
    "mummu_graph_end": (_I, [_P, C.POINTER(_P)]),
    "mummu_graph_launch": (_I, [_P, _P]),
    "mummu_graph_launch_timed": (_I, [_P, _P, _I, C.POINTER(C.c_float)]),
    "mummu_graph_destroy": (None, [_P]),
    "mummu_timer_start": (_I, [_P]),
    "mummu_timer_stop": (_I, [_P, C.POINTER(C.c_float)]),
    "mummu_probe_copy": (_I, [_P, _P, _SZ, _P]),
    "mummu_probe_read": (_I, [_P, _SZ, _I, _I, _P]),
    "mummu_gguf_last_error": (C.c_char_p, []),
    "mummu_gguf_open": (_I, [C.c_char_p, C.POINTER(_P)]),
    "mummu_gguf_close": (None, [_P]),
    "mummu_gguf_version": (_I, [_P]),
    "mummu_gguf_alignment": (_I64, [_P]),
    "mummu_gguf_shard_count": (_I, [_P]),
    "mummu_gguf_tensor_count": (_I, [_P]),
    "mummu_gguf_kv_count": (_I, [_P]),
    "mummu_gguf_find_tensor": (_I, [_P, C.c_char_p]),
    "mummu_gguf_tensor_info": (_I, [_P, _I, C.POINTER(GgufTensor)]),
    "mummu_gguf_tensor_data": (_I, [_P, _I, C.POINTER(_P), C.POINTER(C.c_uint64)]),
    "mummu_gguf_get_u64": (_I, [_P, C.c_char_p, C.POINTER(C.c_uint64)]),
    "mummu_gguf_get_f64": (_I, [_P, C.c_char_p, C.POINTER(C.c_double)]),
    "mummu_gguf_get_str": (C.c_char_p, [_P, C.c_char_p]),
    "mummu_gguf_moe_config": (_I, [_P, C.POINTER(Config)]),
    "mummu_gguf_locate_moe_layer": (_I, [_P, _I, C.POINTER(GgufMoeLayer)]),
    "mummu_moe_load_gguf": (_I, [_P, _P, _I, _I]),
    "mummu_st_last_error": (C.c_char_p, []),
    "mummu_st_open": (_I, [C.c_char_p, C.POINTER(_P)]),
    "mummu_st_close": (None, [_P]),
    "mummu_st_shard_count": (_I, [_P]),
    "mummu_st_tensor_count": (_I, [_P]),
    "mummu_st_find_tensor": (_I, [_P, C.c_char_p]),
    "mummu_st_tensor_info": (_I, [_P, _I, C.POINTER(StTensor)]),
    "mummu_olmoe_config_from_json": (_I, [C.c_char_p, _SZ, C.POINTER(Config)]),
    "mummu_st_moe_config": (_I, [_P, C.POINTER(Config)]),
    "mummu_st_check_moe_layer": (_I, [_P, _I]),
    "mummu_moe_load_safetensors": (_I, [_P, _P, _I, _I]),
    "mummu_moe_kernel_timing": (_I, [_P, _I]),
    "mummu_moe_kernel_times": (_I, [_P, C.POINTER(C.c_char_p), C.POINTER(C.c_double), C.POINTER(C.c_int64), _I]),
}

_lib = None


def load() -> C.CDLL:
    """The HIP library, loaded once.  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build the HIP library first (python -m mummu_amd.build). "
                "This package has no CPU path.")
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def device_count() -> int:
    return load().mummu_device_count()
