"""ctypes binding of libucm_hip.so (declarations mirror include/ucm_hip.h)."""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libucm_hip.so")

OK, EINVAL, ENOTSUP, EHIP, ENOMEM = 0, -22, -95, -5, -12
DTYPE_F32, DTYPE_BF16, DTYPE_F16 = 0, 1, 2
MEAN_F32, MEAN_BF16_ROUND, MEAN_BF16_STORE = 0, 1, 2
MEAN_ABS = 4        # or-ed to a mode: the mean of the absolute values
MEAN_KEYS_F16 = 8   # or-ed to MEAN_F32 / MEAN_BF16_ROUND: fp16 key cache; the rounding is then to fp16

_p, _i, _i64, _sz, _f = C.c_void_p, C.c_int, C.c_int64, C.c_size_t, C.c_float

# name -> argtypes, in the order of include/ucm_hip.h
SIGNATURES = {
    "ucm_version": [],
    "ucm_last_error": [],
    "ucm_block_mean": [_p, _i, _i, _p, _p, _i, _i, _i, _i, _p, _i, _i64, _i, _p],
    "ucm_score_blocks": [_p, _i, _i64, _p, _i, _p, _i, _i64, _i64, _i, _p, _p, _i, _i, _i64, _i, _i, _i, _p, _i64, _f, _i, _p],
    "ucm_score_select": [_p, _p],
    "ucm_kvstar_block_repre": [_p, _i, _i, _p, _p, _i, _i, _i, _i, _i, _p, _i64, _p, _i, _i, _i, _p, _i, _i64, _i64, _i64, _p],
    "ucm_kvstar_block_repre_keys": [_p, _i, _i, _i, _p, _p, _i, _i, _i, _i, _i, _p, _i64, _p, _i, _i, _i, _p, _i, _i64, _i64, _i64, _p],
    "ucm_kvstar_park_queries": [_p, _i, _i64, _i, _p, _p, _i, _p, _i64, _p],
    "ucm_kvstar_workspace_floats": [_i, _i, _i, _i, _i, _i, _i, _p, _p],
    "ucm_kvstar_votes": [_p, _i64, _p, _i, _i, _i, _p, _i, _p, _p, _i64, _i64, _i64, _p, _p, _i, _i, _i, _i, _i, _i, _p, _i64, _p, _i64, _p, _i, _p],
    "ucm_kvstar_votes_tables": [_p, _i64, _p, _i, _i, _i, _p, _i, _p, _p, _p, _i64, _p, _p, _i, _i, _i, _i, _i, _i, _p, _i64, _p, _i64, _p, _i64, _i, _p],
    "ucm_kvstar_topk": [_p, _i64, _p, _p, _p, _i, _i, _p, _i, _p, _p],
    "ucm_kvstar_order": [_p, _i64, _p, _p, _i, _i, _p, _i, _p, _p],
    "ucm_topk_windows": [_p, _i64, _i64, _p, _p, _p, _i, _i, _i, _i, _i, _p, _i, _p, _p, _i, _p, _p, _i, _p, _p],
    "ucm_esa_retrieve": [_p, _i, _i, _p, _p, _i, _i, _i, _p, _p, _p, _p, _i, _p],
    "ucm_esa_retrieve_static": [_p, _i, _i, _p, _p, _i, _i, _i, _p, _p, _p, _i, _p],
    "ucm_esa_retrieve_rows": [_p, _i, _i, _p, _p, _i, _i, _i, _p, _i, _p, _i, _p, _p, _p, _p, _p, _i, _p],
    "ucm_delta_plan_rows": [_p, _p, _p, _p, _i, _i, _i, _i, _p, _i, _p, _p, _p, _p],
    "ucm_kv_load_planned": [_p, _i, _sz, _sz, _i, _p, _i64, _sz, _i, _p, _i, _p, _i, _p, _i, _i64, _p, _p, _i, _i, _p],
    "ucm_kv_load_planned_tp": [_p, _i, _sz, _sz, _i, _p, _i64, _sz, _i, _p, _i, _p, _i, _p, _i, _i64, _p, _p, _i, _i, _i, _i, _p],
    "ucm_prefetch_plan": [_p, _p, _p, _i, _i, _p, _i, _p, _p, _p, _i, _i, _i, _i, _p, _p, _p, _p, _p, _p, _p, _p, _p],
    "ucm_delta_plan": [_p, _p, _p, _i, _i, _i, _p, _i, _p, _p, _p, _p],
    "ucm_hash_encode_blocks": [_p, _i, _i, _p, _p, _i, _i, _i, _i, _p, _i, _i, _p, _i64, _p, _i64, _p, _i64, _i, _p],
    "ucm_hash_encode_blocks_f16": [_p, _i, _i, _p, _p, _i, _i, _i, _i, _p, _i, _i, _p, _i64, _p, _i64, _p, _i64, _i, _p],
    "ucm_hash_encode_queries": [_p, _i64, _p, _i, _i, _i, _i, _i, _p, _i, _p, _p, _p, _p],
    "ucm_hash_encode_queries_f16": [_p, _i64, _p, _i, _i, _i, _i, _i, _p, _i, _p, _p, _p, _p],
    "ucm_hash_score_blocks": [_i, _p, _p, _p, _i64, _p, _i64, _i64, _p, _p, _i, _i64, _i, _i, _i, _p, _i64, _i, _p],
    "ucm_copy_batch": [_p, _p, _sz, _sz, _p],
    "ucm_park_rows": [_p, _i64, _p, _p, _i64, _p, _i, _sz, _p],
    "ucm_kernel_can_access": [_p, _sz],
    "ucm_device_create": [_i, _sz, _sz, _p],
    "ucm_device_destroy": [_p],
    "ucm_device_get_buffer": [_p, _sz],
    "ucm_device_release_buffer": [_p, _p],
    "ucm_device_h2d_sync": [_p, _p, _p, _sz],
    "ucm_device_d2h_sync": [_p, _p, _p, _sz],
    "ucm_device_h2d_async": [_p, _p, _p, _sz],
    "ucm_device_d2h_async": [_p, _p, _p, _sz],
    "ucm_device_append_callback": [_p, _p, _p],
    "ucm_device_synchronized": [_p],
    "ucm_device_h2d_batch_sync": [_p, _p, _p, _sz, _sz],
    "ucm_device_d2h_batch_sync": [_p, _p, _p, _sz, _sz],
    "ucm_device_stream": [_p],
    "ucm_kv_gather_blocks": [_p, _i, _sz, _sz, _i, _p, _i, _p, _p],
    "ucm_kv_scatter_blocks": [_p, _i, _sz, _sz, _i, _p, _i, _p, _p],
    "ucm_kv_gather_blocks_tp": [_p, _i, _sz, _sz, _i, _p, _i, _p, _i, _i, _p],
    "ucm_kv_scatter_blocks_tp": [_p, _i, _sz, _sz, _i, _p, _i, _p, _i, _i, _p],
    "ucm_kv_gather_selected": [_p, _i, _sz, _sz, _i, _p, _p, _i, _i, _p, _p, _i, _p, _i64, _p],
}


# entry points that do not return a status code
RESTYPES = {
    "ucm_last_error": C.c_char_p,
    "ucm_device_destroy": None,
    "ucm_device_get_buffer": C.c_void_p,
    "ucm_device_release_buffer": None,
    "ucm_device_stream": C.c_void_p,
}

DEVICE_CALLBACK = C.CFUNCTYPE(None, C.c_int, C.c_void_p)


class ScoreSelectArgs(C.Structure):
    """ucm_score_select_args_t (include/ucm_hip.h), field for field."""
    _fields_ = [
        ("struct_size", _sz), ("q", _p), ("q_dtype", _i), ("q_heads", _i), ("q_layer_stride", _i64), ("q_rows", _p),
        ("repre", _p), ("repre_dtype", _i), ("num_repre", _i), ("repre_layer_stride", _i64), ("repre_rows", _i64),
        ("seg_off", _p), ("seg_len", _p), ("topk_len", _p), ("n_req", _i), ("max_seg_len", _i), ("first_layer", _i),
        ("n_layers", _i), ("kv_heads", _i), ("head_dim", _i), ("scores", _p), ("scores_layer_stride", _i64),
        ("scale", _f), ("tile_blocks", _i), ("start_w", _i), ("end_w", _i), ("idx_out", _p), ("count_out", _p),
        ("out_stride", _i), ("bt_stride", _i), ("block_tables", _p), ("phys_out", _p), ("seq_lens", _p),
        ("sparse_seq_lens", _p), ("block_size", _i), ("reserved", _i), ("tickets", _p),
        ("idx_layer_stride", _i64), ("count_layer_stride", _i64), ("total_blocks", _i64),
    ]

    def __init__(self, **kw):
        super().__init__(struct_size=C.sizeof(ScoreSelectArgs), num_repre=1, scale=1.0, n_layers=1, **kw)


class UcmHipError(RuntimeError):
    def __init__(self, fn: str, code: int, text: str):
        super().__init__(f"{fn} failed with {code}: {text}")
        self.code = code


def load() -> C.CDLL:
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python unified-cache-management_amd/build.py` "
            "(the HIP library is the only implementation; there is no CPU fallback)"
        )
    lib = C.CDLL(LIB_PATH)
    for name, argtypes in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the library does not export a declared symbol
        fn.argtypes = argtypes
        fn.restype = RESTYPES.get(name, C.c_int)
    return lib


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        _lib = load()
    return _lib


def call(name: str, *args) -> None:
    rc = getattr(lib(), name)(*args)
    if rc != OK:
        raise UcmHipError(name, rc, lib().ucm_last_error().decode())
