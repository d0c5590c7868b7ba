"""ctypes binding of libmoeflux_attn_hip.so — the C ABI in include/moeflux_attn.h.

The library is loaded from moeflux_amd/lib/ (built in-tree by
``python -m moeflux_amd.build``).  A missing library is an error: there is no
other implementation to fall back to.
"""
from __future__ import annotations

import ctypes as C
import os

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib",
                         "libmoeflux_attn_hip.so")

OK, ERR_INVALID, ERR_SHAPE, ERR_OVERFLOW, ERR_LAYER, ERR_HIP, ERR_STATE, ERR_NO_CHECKPOINT = 0, -1, -2, -3, -4, -5, -6, -7
KV_F32, KV_BF16 = 0, 1

i32, f32, vp, u16p, f32p = C.c_int32, C.c_float, C.c_void_p, C.c_void_p, C.c_void_p


class mfa_matvec_spec(C.Structure):
    _fields_ = [("w_packed", C.c_void_p), ("scales", C.c_void_p), ("biases", C.c_void_p), ("x", C.c_void_p),
                ("out", C.c_void_p), ("out_dim", C.c_int32), ("in_dim", C.c_int32)]


class mfa_config(C.Structure):
    _fields_ = [
        ("num_layers", i32), ("full_attn_interval", i32), ("num_attn_heads", i32),
        ("num_kv_heads", i32), ("head_dim", i32), ("kv_capacity", i32), ("kv_dtype", i32),
        ("linear_num_k_heads", i32), ("linear_num_v_heads", i32), ("linear_key_dim", i32),
        ("linear_value_dim", i32), ("conv_kernel_size", i32), ("rms_norm_eps", f32),
    ]


# name -> (restype, argtypes); every symbol include/moeflux_attn.h declares.
SIGNATURES = {
    "mfa_ctx_create": (vp, [C.POINTER(mfa_config)]),
    "mfa_ctx_destroy": (None, [vp]),
    "mfa_last_error_string": (C.c_char_p, []),
    "mfa_sync": (C.c_int, [vp]),
    "mfa_stream": (vp, [vp]),
    "mfa_set_linear_weights": (C.c_int, [vp, i32, u16p, f32p, u16p, u16p]),
    "mfa_set_num_splits": (C.c_int, [vp, i32]),
    "mfa_set_partial_only": (C.c_int, [vp, i32]),
    "mfa_set_step_launches": (C.c_int, [vp, i32]),
    "mfa_host_alloc": (vp, [C.c_int64]),
    "mfa_host_free": (None, [vp]),
    "mfa_kv_append": (C.c_int, [vp, i32, f32p, f32p]),
    "mfa_kv_append_dev": (C.c_int, [vp, i32, f32p, f32p]),
    "mfa_kv_len": (i32, [vp, i32]),
    "mfa_sdpa_decode": (C.c_int, [vp, i32, f32p, f32p, f32p]),
    "mfa_sdpa_decode_dev": (C.c_int, [vp, i32, f32p, f32p, f32p]),
    "mfa_sdpa_decode_static_dev": (C.c_int, [vp, i32, f32p, f32p, f32p]),
    "mfa_prefill_attn": (C.c_int, [vp, i32, i32, f32p, f32p, f32p, f32p, f32p]),
    "mfa_prefill_attn_dev": (C.c_int, [vp, i32, i32, f32p, f32p, f32p, f32p, f32p]),
    "mfa_gdn_step": (C.c_int, [vp, i32, f32p, f32p, f32p, f32p, f32p]),
    "mfa_gdn_step_dev": (C.c_int, [vp, i32, f32p, f32p, f32p, f32p, f32p]),
    "mfa_prefill_gdn": (C.c_int, [vp, i32, i32, f32p, f32p, f32p, f32p, f32p]),
    "mfa_prefill_gdn_dev": (C.c_int, [vp, i32, i32, f32p, f32p, f32p, f32p, f32p]),
    "mfa_set_full_weights": (C.c_int, [vp, C.c_int32, u16p, u16p]),
    "mfa_set_rope": (C.c_int, [vp, C.c_float, C.c_int32]),
    "mfa_attn_prologue": (C.c_int, [vp, C.c_int32, C.c_int32, f32p, f32p, f32p, f32p, f32p]),
    "mfa_attn_prologue_dev": (C.c_int, [vp, C.c_int32, C.c_int32, f32p, f32p, f32p, f32p, f32p]),
    "mfa_full_attn_step": (C.c_int, [vp, C.c_int32, C.c_int32, f32p, f32p, f32p, f32p]),
    "mfa_full_attn_step_dev": (C.c_int, [vp, C.c_int32, C.c_int32, f32p, f32p, f32p, f32p]),
    "mfa_prefill_full_attn": (C.c_int, [vp, C.c_int32, C.c_int32, C.c_int32, f32p, f32p, f32p, f32p]),
    "mfa_prefill_full_attn_dev": (C.c_int, [vp, C.c_int32, C.c_int32, C.c_int32, f32p, f32p, f32p, f32p]),
    "mfa_dequant_matvec_4bit_dev": (C.c_int, [vp, C.c_int32, vp]),
    "mfa_dequant_matvec_4bit_tiled_dev": (C.c_int, [vp, C.c_int32, vp]),
    "mfa_matvec_tiled_words": (C.c_int64, [C.c_int32, C.c_int32]),
    "mfa_matvec_tile_weights_dev": (C.c_int, [vp, C.c_int32, C.c_int32, vp, vp, vp, vp]),
    "mfa_dequant_matvec_4bit": (C.c_int, [C.c_int32, C.c_int32, C.c_int32, vp, u16p, u16p, f32p, f32p]),
    "mfa_mla_sdpa_folded_dev": (C.c_int, [vp, C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_float,
                                          f32p, f32p, f32p, f32p, f32p]),
    "mfa_mla_sdpa_folded": (C.c_int, [C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_float,
                                      f32p, f32p, f32p, f32p, f32p]),
    "mfa_state_size": (C.c_int64, [vp]),
    "mfa_state_save": (C.c_int64, [vp, vp, C.c_int64]),
    "mfa_state_load": (C.c_int, [vp, vp, C.c_int64]),
    "mfa_checkpoint_pos": (C.c_int, [vp, i32]),
    "mfa_restore_to": (C.c_int, [vp, i32]),
    "mfa_set_max_checkpoints": (C.c_int, [vp, i32]),
    "mfa_checkpoint_count": (i32, [vp]),
    "mfa_set_sweep_per_layer": (C.c_int, [vp, C.c_int32]),
    "mfa_token_sweep_dev": (C.c_int, [vp, f32p, f32p, f32p, f32p, f32p, f32p, f32p, f32p]),
    "mfa_reset": (C.c_int, [vp]),
    "mfa_truncate": (C.c_int, [vp, i32, i32]),
    "mfa_pos_max": (i32, [vp]),
    "mfa_kv_export": (C.c_int, [vp, i32, i32, f32p, f32p]),
    "mfa_kv_import": (C.c_int, [vp, i32, i32, f32p, f32p]),
    "mfa_kv_import_bf16": (C.c_int, [vp, i32, i32, u16p, u16p]),
    "mfa_linear_state_export": (C.c_int, [vp, i32, f32p, f32p]),
    "mfa_linear_state_import": (C.c_int, [vp, i32, f32p, f32p]),
    "mfa_timer_start": (C.c_int, [vp]),
    "mfa_timer_stop": (C.c_int, [vp, C.POINTER(C.c_float)]),
    "mfa_sdpa": (C.c_int, [i32, i32, i32, i32, f32p, f32p, f32p, f32p, f32p]),
    "mfa_sdpa_bf16kv": (C.c_int, [i32, i32, i32, i32, f32p, f32p, u16p, u16p, f32p]),
    "mfa_attn_scores_batched": (C.c_int, [i32, i32, i32, i32, f32p, f32p, f32, f32p]),
    "mfa_attn_softmax_batched": (C.c_int, [i32, i32, f32p]),
    "mfa_attn_values_batched": (C.c_int, [i32, i32, i32, i32, f32p, f32p, f32p]),
    "mfa_sigmoid_gate": (C.c_int, [i32, f32p, f32p]),
    "mfa_conv1d_step": (C.c_int, [i32, i32, f32p, f32p, u16p, f32p]),
    "mfa_rms_norm_qk": (C.c_int, [i32, i32, f32p, f32p]),
    "mfa_rms_norm_bare": (C.c_int, [i32, f32, f32p, f32p]),
    "mfa_compute_decay_beta": (C.c_int, [i32, f32p, f32p, f32p, u16p, f32p, f32p]),
    "mfa_gated_delta_net_step": (C.c_int, [i32, i32, i32, i32, f32p, f32p, f32p, f32p, f32p, f32p, f32p]),
    "mfa_gated_delta_recurrence": (C.c_int, [f32p, u16p, f32p, f32p, f32p, f32p, f32p, i32, i32, i32, i32, f32p, f32p]),
    "mfa_gated_rms_norm": (C.c_int, [i32, i32, f32, f32p, f32p, u16p, f32p]),
    "mfa_debug_kv_offset": (C.c_int64, [i32, i32, C.c_int64, i32, i32]),
    "mfa_debug_num_splits": (i32, [i32, i32, i32, i32, C.c_int64, i32, i32]),
    "mfa_debug_max_splits": (i32, [i32, i32, i32, i32, C.c_int64, i32, i32]),
    "mfa_debug_copy_dev": (C.c_int, [vp, vp, vp, C.c_size_t]),
    "mfa_debug_read_dev": (C.c_int, [vp, vp, C.c_size_t, C.c_int32]),
    "mfa_debug_fill_workspace": (C.c_int, [vp, C.c_uint32]),
}

_lib = None


def lib_path() -> str:
    return _LIB_PATH


def load() -> C.CDLL:
    """Load the library and attach prototypes.  Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        raise ImportError(
            f"{_LIB_PATH} is missing: build it with `python -m moeflux_amd.build` "
            "(hipcc, gfx950). There is no CPU fallback.")
    lib = C.CDLL(_LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def last_error() -> str:
    return load().mfa_last_error_string().decode("utf-8", "replace")
