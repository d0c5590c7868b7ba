"""ctypes front end of the CPU oracle (oracle/mfa_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by ``__graft_entry__.smoke()`` and
by the ``cpu_baseline`` leg of ``bench.py`` as the checker.  The shipped package
never imports it.

Every wrapper takes and returns numpy arrays; arrays the reference mutates in
place (conv state, recurrent state, score rows) are copied first and the new
value is returned, so a test can keep its inputs.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libmfa_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile oracle/mfa_oracle.c with gcc (a second or two)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libmfa_oracle.so"],
                              stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.orc_f32_to_bf16.restype = C.c_uint16
        _lib.orc_f32_to_bf16.argtypes = [C.c_float]
    return _lib


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _u16(a):
    return np.ascontiguousarray(a, dtype=np.uint16)


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def _check(rc, name):
    if rc != 0:
        raise ValueError(f"{name} rejected its arguments (rc={rc})")


# -- bf16 helpers -------------------------------------------------------------

def f32_to_bf16(x) -> np.ndarray:
    x = _f32(x)
    out = np.empty(x.shape, dtype=np.uint16)
    lib().orc_f32_to_bf16_array(_p(x), _p(out), C.c_int64(x.size))
    return out


def bf16_to_f32(x) -> np.ndarray:
    x = _u16(x)
    out = np.empty(x.shape, dtype=np.float32)
    lib().orc_bf16_to_f32_array(_p(x), _p(out), C.c_int64(x.size))
    return out


# -- full attention -----------------------------------------------------------

def sdpa(kv_len, num_attn_heads, num_kv_heads, head_dim, q, q_gate, k_cache, v_cache):
    q, q_gate = _f32(q), _f32(q_gate)
    out = np.empty(num_attn_heads * head_dim, dtype=np.float32)
    if k_cache.dtype == np.uint16:
        k_cache, v_cache = _u16(k_cache), _u16(v_cache)
        fn = lib().orc_sdpa_bf16kv
    else:
        k_cache, v_cache = _f32(k_cache), _f32(v_cache)
        fn = lib().orc_sdpa
    rc = fn(C.c_int32(kv_len), C.c_int32(num_attn_heads), C.c_int32(num_kv_heads),
            C.c_int32(head_dim), _p(q), _p(q_gate), _p(k_cache), _p(v_cache), _p(out))
    _check(rc, "orc_sdpa")
    return out


def attn_scores(num_heads, num_kv_heads, head_dim, seq_len, q, k_cache, scale, seq_stride=None):
    seq_stride = seq_len if seq_stride is None else seq_stride
    q, k_cache = _f32(q), _f32(k_cache)
    out = np.zeros(num_heads * seq_stride, dtype=np.float32)
    rc = lib().orc_attn_scores(C.c_int32(num_heads), C.c_int32(num_kv_heads),
                               C.c_int32(head_dim), C.c_int32(seq_len), C.c_int32(seq_stride),
                               _p(q), _p(k_cache), C.c_float(scale), _p(out))
    _check(rc, "orc_attn_scores")
    return out


def attn_softmax(num_heads, seq_len, scores, seq_stride=None):
    seq_stride = seq_len if seq_stride is None else seq_stride
    s = _f32(scores).copy()
    rc = lib().orc_attn_softmax(C.c_int32(num_heads), C.c_int32(seq_len),
                                C.c_int32(seq_stride), _p(s))
    _check(rc, "orc_attn_softmax")
    return s


def attn_values(num_heads, num_kv_heads, head_dim, seq_len, scores, v_cache, seq_stride=None):
    seq_stride = seq_len if seq_stride is None else seq_stride
    scores, v_cache = _f32(scores), _f32(v_cache)
    out = np.empty(num_heads * head_dim, dtype=np.float32)
    rc = lib().orc_attn_values(C.c_int32(num_heads), C.c_int32(num_kv_heads),
                               C.c_int32(head_dim), C.c_int32(seq_len), C.c_int32(seq_stride),
                               _p(scores), _p(v_cache), _p(out))
    _check(rc, "orc_attn_values")
    return out


def sigmoid_gate(gate, x):
    gate, x = _f32(gate), _f32(x).copy()
    rc = lib().orc_sigmoid_gate(C.c_int32(x.size), _p(gate), _p(x))
    _check(rc, "orc_sigmoid_gate")
    return x


# -- gated delta net ----------------------------------------------------------

def conv1d_step(conv_state, new_input, weight_bf16, channels, kernel_size):
    conv_state, new_input, weight_bf16 = _f32(conv_state), _f32(new_input), _u16(weight_bf16)
    out = np.empty(channels, dtype=np.float32)
    rc = lib().orc_conv1d_step(_p(conv_state), _p(new_input), _p(weight_bf16),
                               C.c_int32(channels), C.c_int32(kernel_size), _p(out))
    _check(rc, "orc_conv1d_step")
    return out


def conv_state_shift(conv_state, new_input, channels, kernel_size):
    s, new_input = _f32(conv_state).copy(), _f32(new_input)
    rc = lib().orc_conv_state_shift(_p(s), _p(new_input), C.c_int32(channels),
                                    C.c_int32(kernel_size))
    _check(rc, "orc_conv_state_shift")
    return s


def rms_norm_bare(x, eps):
    x = _f32(x)
    out = np.empty_like(x)
    rc = lib().orc_rms_norm_bare(C.c_int32(x.size), C.c_float(eps), _p(x), _p(out))
    _check(rc, "orc_rms_norm_bare")
    return out


def rms_norm_qk(num_k_heads, key_dim, q, k):
    q, k = _f32(q).copy(), _f32(k).copy()
    rc = lib().orc_rms_norm_qk(C.c_int32(num_k_heads), C.c_int32(key_dim), _p(q), _p(k))
    _check(rc, "orc_rms_norm_qk")
    return q, k


def rms_norm_gated(x, z, w_bf16, eps):
    x, z, w_bf16 = _f32(x), _f32(z), _u16(w_bf16)
    out = np.empty_like(x)
    rc = lib().orc_rms_norm_gated(C.c_int32(x.size), C.c_float(eps), _p(x), _p(z),
                                  _p(w_bf16), _p(out))
    _check(rc, "orc_rms_norm_gated")
    return out


def decay_beta(alpha, beta, a_log, dt_bias_bf16):
    alpha, beta, a_log, dt_bias_bf16 = _f32(alpha), _f32(beta), _f32(a_log), _u16(dt_bias_bf16)
    g = np.empty_like(alpha)
    b = np.empty_like(alpha)
    rc = lib().orc_decay_beta(C.c_int32(alpha.size), _p(alpha), _p(beta), _p(a_log),
                              _p(dt_bias_bf16), _p(g), _p(b))
    _check(rc, "orc_decay_beta")
    return g, b


def delta_net_step(v_heads, k_heads, key_dim, value_dim, g_decay, beta_gate, q, k, v, ssm_state):
    g_decay, beta_gate, q, k, v = map(_f32, (g_decay, beta_gate, q, k, v))
    s = _f32(ssm_state).copy()
    out = np.empty(v_heads * value_dim, dtype=np.float32)
    rc = lib().orc_delta_net_step(C.c_int32(v_heads), C.c_int32(k_heads), C.c_int32(key_dim),
                                  C.c_int32(value_dim), _p(g_decay), _p(beta_gate), _p(q),
                                  _p(k), _p(v), _p(s), _p(out))
    _check(rc, "orc_delta_net_step")
    return s, out


def gated_delta_recurrence(a_log, dt_bias_bf16, alpha, beta, q, k, v, v_heads, k_heads,
                           key_dim, value_dim, ssm_state):
    a_log, alpha, beta, q, k, v = map(_f32, (a_log, alpha, beta, q, k, v))
    dt_bias_bf16 = _u16(dt_bias_bf16)
    s = _f32(ssm_state).copy()
    out = np.empty(v_heads * value_dim, dtype=np.float32)
    rc = lib().orc_gated_delta_recurrence(_p(a_log), _p(dt_bias_bf16), _p(alpha), _p(beta),
                                          _p(q), _p(k), _p(v), C.c_int32(v_heads),
                                          C.c_int32(k_heads), C.c_int32(key_dim),
                                          C.c_int32(value_dim), _p(s), _p(out))
    _check(rc, "orc_gated_delta_recurrence")
    return s, out


def gdn_step(k_heads, v_heads, key_dim, value_dim, kernel_size, eps, conv_w_bf16, a_log,
             dt_bias_bf16, norm_w_bf16, qkv_in, z, alpha, beta, conv_state, ssm_state):
    """Returns (out, new_conv_state, new_ssm_state)."""
    conv_w_bf16, dt_bias_bf16, norm_w_bf16 = map(_u16, (conv_w_bf16, dt_bias_bf16, norm_w_bf16))
    a_log, qkv_in, z, alpha, beta = map(_f32, (a_log, qkv_in, z, alpha, beta))
    cs, ss = _f32(conv_state).copy(), _f32(ssm_state).copy()
    out = np.empty(v_heads * value_dim, dtype=np.float32)
    rc = lib().orc_gdn_step(C.c_int32(k_heads), C.c_int32(v_heads), C.c_int32(key_dim),
                            C.c_int32(value_dim), C.c_int32(kernel_size), C.c_float(eps),
                            _p(conv_w_bf16), _p(a_log), _p(dt_bias_bf16), _p(norm_w_bf16),
                            _p(qkv_in), _p(z), _p(alpha), _p(beta), _p(cs), _p(ss), _p(out))
    _check(rc, "orc_gdn_step")
    return out, cs, ss


def prefill_attn(T, kv_len0, num_attn_heads, num_kv_heads, head_dim, q, q_gate, k_cache, v_cache):
    q, q_gate, k_cache, v_cache = map(_f32, (q, q_gate, k_cache, v_cache))
    out = np.empty(T * num_attn_heads * head_dim, dtype=np.float32)
    rc = lib().orc_prefill_attn(C.c_int32(T), C.c_int32(kv_len0), C.c_int32(num_attn_heads),
                                C.c_int32(num_kv_heads), C.c_int32(head_dim), _p(q),
                                _p(q_gate), _p(k_cache), _p(v_cache), _p(out))
    _check(rc, "orc_prefill_attn")
    return out


def prefill_gdn(T, k_heads, v_heads, key_dim, value_dim, kernel_size, eps, conv_w_bf16, a_log,
                dt_bias_bf16, norm_w_bf16, qkv_in, z, alpha, beta, conv_state, ssm_state):
    """Returns (out [T, v_heads*value_dim], new_conv_state, new_ssm_state)."""
    conv_w_bf16, dt_bias_bf16, norm_w_bf16 = map(_u16, (conv_w_bf16, dt_bias_bf16, norm_w_bf16))
    a_log, qkv_in, z, alpha, beta = map(_f32, (a_log, qkv_in, z, alpha, beta))
    cs, ss = _f32(conv_state).copy(), _f32(ssm_state).copy()
    out = np.empty(T * v_heads * value_dim, dtype=np.float32)
    rc = lib().orc_prefill_gdn(C.c_int32(T), C.c_int32(k_heads), C.c_int32(v_heads),
                               C.c_int32(key_dim), C.c_int32(value_dim),
                               C.c_int32(kernel_size), C.c_float(eps), _p(conv_w_bf16),
                               _p(a_log), _p(dt_bias_bf16), _p(norm_w_bf16), _p(qkv_in), _p(z),
                               _p(alpha), _p(beta), _p(cs), _p(ss), _p(out))
    _check(rc, "orc_prefill_gdn")
    return out.reshape(T, v_heads * value_dim), cs, ss


def rms_norm_per_head(num_heads, head_dim, eps, weight_bf16, x):
    x = _f32(x).copy()
    rc = lib().orc_rms_norm_per_head(C.c_int32(num_heads), C.c_int32(head_dim), C.c_float(eps),
                                     _p(_u16(weight_bf16)), _p(x))
    _check(rc, "orc_rms_norm_per_head")
    return x


def rope_inv_freq(theta, rotary_dim):
    out = np.empty(rotary_dim // 2, dtype=np.float32)
    _check(lib().orc_rope_inv_freq(C.c_float(theta), C.c_int32(rotary_dim), _p(out)), "orc_rope_inv_freq")
    return out


def apply_rotary_emb(pos, num_heads, num_kv_heads, head_dim, rotary_dim, theta, q, k):
    """Returns (q, k) rotated at position pos."""
    q, k = _f32(q).copy(), _f32(k).copy()
    rc = lib().orc_apply_rotary_emb(C.c_int32(pos), C.c_int32(num_heads), C.c_int32(num_kv_heads),
                                    C.c_int32(head_dim), C.c_int32(rotary_dim), C.c_float(theta),
                                    _p(q), _p(k))
    _check(rc, "orc_apply_rotary_emb")
    return q, k


def attn_prologue(pos, num_heads, num_kv_heads, head_dim, rotary_dim, theta, eps, q_norm_bf16,
                  k_norm_bf16, q_proj_out, k_in, v_in):
    """Returns (q, q_gate, k_row, v_row): the attention core's inputs and the row appended to the cache."""
    q_proj_out, k_in, v_in = map(_f32, (q_proj_out, k_in, v_in))
    qd, kd = num_heads * head_dim, num_kv_heads * head_dim
    q, g = np.empty(qd, np.float32), np.empty(qd, np.float32)
    kr, vr = np.empty(kd, np.float32), np.empty(kd, np.float32)
    rc = lib().orc_attn_prologue(C.c_int32(pos), C.c_int32(num_heads), C.c_int32(num_kv_heads),
                                 C.c_int32(head_dim), C.c_int32(rotary_dim), C.c_float(theta),
                                 C.c_float(eps), _p(_u16(q_norm_bf16)), _p(_u16(k_norm_bf16)),
                                 _p(q_proj_out), _p(k_in), _p(v_in), _p(q), _p(g), _p(kr), _p(vr))
    _check(rc, "orc_attn_prologue")
    return q, g, kr, vr


def dequant_matvec_4bit(packed, scales_bf16, biases_bf16, in_dim, out_dim, x):
    packed = np.ascontiguousarray(packed, dtype=np.uint32)
    out = np.empty(out_dim, dtype=np.float32)
    rc = lib().orc_dequant_matvec_4bit(_p(packed), _p(_u16(scales_bf16)), _p(_u16(biases_bf16)),
                                       C.c_int32(in_dim), C.c_int32(out_dim), _p(_f32(x)), _p(out))
    _check(rc, "orc_dequant_matvec_4bit")
    return out


def mla_sdpa_folded(num_heads, kv_lora_rank, qk_rope_head_dim, cache_len, softmax_scale, q_prime, q_pe,
                    latent_cache, rope_k_cache):
    q_prime, q_pe, latent_cache, rope_k_cache = map(_f32, (q_prime, q_pe, latent_cache, rope_k_cache))
    out = np.empty(num_heads * kv_lora_rank, dtype=np.float32)
    rc = lib().orc_mla_sdpa_folded(C.c_int32(num_heads), C.c_int32(kv_lora_rank), C.c_int32(qk_rope_head_dim),
                                   C.c_int32(cache_len), C.c_float(softmax_scale), _p(q_prime), _p(q_pe),
                                   _p(latent_cache), _p(rope_k_cache), _p(out))
    _check(rc, "orc_mla_sdpa_folded")
    return out

