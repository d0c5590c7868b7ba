"""Host-side mirror, for the attention core, of the reference's `RsCtx`
(crates/moeflux/src/riir/mod.rs): the production calls the layer composers make
(KV append + SDPA, the Gated-DeltaNet chain), the state operations
(`memory_clear`, `memory_seq_rm`, `memory_seq_pos_max`) and the per-kernel
hooks the reference's differential tests drive (`sdpa_cpu`, `attn_*_batched`,
`sigmoid_gate`, `conv1d_step_cpu`, ...).  Everything computes on the GPU through
the C ABI; the names keep the reference's so its tests read the same here.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass

import numpy as np

from . import ffi


class MfaError(RuntimeError):
    """A negative return code from the library (the reference maps its kernel
    errors to `RsError::EvalFailed`, riir/mod.rs:2218-2239)."""

    def __init__(self, code: int, where: str):
        self.code = code
        super().__init__(f"{where}: error {code}: {ffi.last_error()}")


def _chk(rc: int, where: str) -> int:
    if rc < 0:
        raise MfaError(rc, where)
    return rc


def _f32(a, n=None, name="array"):
    a = np.ascontiguousarray(a, dtype=np.float32)
    if n is not None and a.size != n:
        raise ValueError(f"{name} has {a.size} elements, expected {n}")
    return a


def _u16(a, n=None, name="array"):
    a = np.ascontiguousarray(a, dtype=np.uint16)
    if n is not None and a.size != n:
        raise ValueError(f"{name} has {a.size} elements, expected {n}")
    return a


def _p(a):
    return a.ctypes.data


@dataclass
class Config:
    """Run-time shapes; the fields of `Variant` (riir/variants.rs:383-465) the path reads."""
    num_layers: int = 1
    full_attn_interval: int = 1
    num_attn_heads: int = 32
    num_kv_heads: int = 2
    head_dim: int = 256
    kv_capacity: int = 8192
    kv_dtype: int = ffi.KV_F32
    linear_num_k_heads: int = 16
    linear_num_v_heads: int = 32
    linear_key_dim: int = 128
    linear_value_dim: int = 128
    conv_kernel_size: int = 4
    rms_norm_eps: float = 1e-6

    @property
    def q_dim(self):
        return self.num_attn_heads * self.head_dim

    @property
    def kv_dim(self):
        return self.num_kv_heads * self.head_dim

    @property
    def conv_dim(self):
        return 2 * self.linear_num_k_heads * self.linear_key_dim + self.v_total

    @property
    def v_total(self):
        return self.linear_num_v_heads * self.linear_value_dim

    @property
    def ssm_elems(self):
        return self.v_total * self.linear_key_dim

    def is_full(self, layer: int) -> bool:
        return (layer + 1) % self.full_attn_interval == 0

    def to_c(self) -> ffi.mfa_config:
        return ffi.mfa_config(self.num_layers, self.full_attn_interval, self.num_attn_heads,
                              self.num_kv_heads, self.head_dim, self.kv_capacity, self.kv_dtype,
                              self.linear_num_k_heads, self.linear_num_v_heads,
                              self.linear_key_dim, self.linear_value_dim, self.conv_kernel_size,
                              self.rms_norm_eps)


class Ctx:
    """Owns the device-resident attention state of one model instance."""

    def __init__(self, cfg: Config):
        self.lib = ffi.load()
        self.cfg = cfg
        c = cfg.to_c()
        self.h = self.lib.mfa_ctx_create(C.byref(c))
        if not self.h:
            raise MfaError(ffi.ERR_INVALID, "mfa_ctx_create")

    def close(self):
        if getattr(self, "h", None):
            self.lib.mfa_ctx_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    # ---- weights / tuning ---------------------------------------------------
    def set_linear_weights(self, layer, conv_w_bf16, a_log, dt_bias_bf16, norm_w_bf16):
        cfg = self.cfg
        cw = _u16(conv_w_bf16, cfg.conv_dim * cfg.conv_kernel_size, "conv weight")
        al = _f32(a_log, cfg.linear_num_v_heads, "A_log")
        dt = _u16(dt_bias_bf16, cfg.linear_num_v_heads, "dt_bias")
        nw = _u16(norm_w_bf16, cfg.linear_value_dim, "norm weight")
        _chk(self.lib.mfa_set_linear_weights(self.h, layer, _p(cw), _p(al), _p(dt), _p(nw)),
             "mfa_set_linear_weights")

    def set_num_splits(self, n: int):
        _chk(self.lib.mfa_set_num_splits(self.h, n), "mfa_set_num_splits")

    def set_step_launches(self, launches: int):
        """Launches of full_attn_step: 2 (prologue inside the attention launch) or 3."""
        _chk(self.lib.mfa_set_step_launches(self.h, launches), "mfa_set_step_launches")

    # ---- full attention -------------------------------------------------------
    def kv_append(self, layer, k, v):
        k, v = _f32(k, self.cfg.kv_dim, "k"), _f32(v, self.cfg.kv_dim, "v")
        _chk(self.lib.mfa_kv_append(self.h, layer, _p(k), _p(v)), "mfa_kv_append")

    def kv_len(self, layer) -> int:
        return _chk(self.lib.mfa_kv_len(self.h, layer), "mfa_kv_len")

    def sdpa_decode(self, layer, q, q_gate) -> np.ndarray:
        q, g = _f32(q, self.cfg.q_dim, "q"), _f32(q_gate, self.cfg.q_dim, "q_gate")
        out = np.empty(self.cfg.q_dim, dtype=np.float32)
        _chk(self.lib.mfa_sdpa_decode(self.h, layer, _p(q), _p(g), _p(out)), "mfa_sdpa_decode")
        return out

    def set_full_weights(self, layer, q_norm_bf16, k_norm_bf16):
        qn = _u16(q_norm_bf16, self.cfg.head_dim, "q_norm weight")
        kn = _u16(k_norm_bf16, self.cfg.head_dim, "k_norm weight")
        _chk(self.lib.mfa_set_full_weights(self.h, layer, _p(qn), _p(kn)), "mfa_set_full_weights")

    def set_rope(self, theta: float, rotary_dim: int):
        _chk(self.lib.mfa_set_rope(self.h, theta, rotary_dim), "mfa_set_rope")

    def attn_prologue(self, layer, pos, q_proj_out, k, v):
        """(q, q_gate) for the attention core; the token's k (normed, rotated) and v are appended."""
        cfg = self.cfg
        qp = _f32(q_proj_out, 2 * cfg.q_dim, "q_proj_out")
        k, v = _f32(k, cfg.kv_dim, "k"), _f32(v, cfg.kv_dim, "v")
        q, g = np.empty(cfg.q_dim, np.float32), np.empty(cfg.q_dim, np.float32)
        _chk(self.lib.mfa_attn_prologue(self.h, layer, pos, _p(qp), _p(k), _p(v), _p(q), _p(g)), "mfa_attn_prologue")
        return q, g

    def full_attn_step(self, layer, pos, q_proj_out, k, v) -> np.ndarray:
        cfg = self.cfg
        qp = _f32(q_proj_out, 2 * cfg.q_dim, "q_proj_out")
        k, v = _f32(k, cfg.kv_dim, "k"), _f32(v, cfg.kv_dim, "v")
        out = np.empty(cfg.q_dim, np.float32)
        _chk(self.lib.mfa_full_attn_step(self.h, layer, pos, _p(qp), _p(k), _p(v), _p(out)), "mfa_full_attn_step")
        return out

    def prefill_full_attn(self, layer, pos0, q_proj_out, k, v) -> np.ndarray:
        """The layer step for a chunk of tokens at positions pos0, pos0 + 1, ...: [T, q_dim]."""
        cfg = self.cfg
        qp = _f32(q_proj_out)
        T = qp.size // (2 * cfg.q_dim)
        qp = _f32(qp, 2 * T * cfg.q_dim, "q_proj_out")
        k, v = _f32(k, T * cfg.kv_dim, "k"), _f32(v, T * cfg.kv_dim, "v")
        out = np.empty((T, cfg.q_dim), dtype=np.float32)
        _chk(self.lib.mfa_prefill_full_attn(self.h, layer, pos0, T, _p(qp), _p(k), _p(v), _p(out)),
             "mfa_prefill_full_attn")
        return out

    def prefill_attn(self, layer, q, q_gate, k, v) -> np.ndarray:
        q = _f32(q)
        T = q.size // self.cfg.q_dim
        g = _f32(q_gate, q.size, "q_gate")
        k, v = _f32(k, T * self.cfg.kv_dim, "k"), _f32(v, T * self.cfg.kv_dim, "v")
        out = np.empty((T, self.cfg.q_dim), dtype=np.float32)
        _chk(self.lib.mfa_prefill_attn(self.h, layer, T, _p(q), _p(g), _p(k), _p(v), _p(out)),
             "mfa_prefill_attn")
        return out

    # ---- gated delta net --------------------------------------------------------
    def gdn_step(self, layer, qkv_in, z, alpha, beta) -> np.ndarray:
        cfg = self.cfg
        x, z = _f32(qkv_in, cfg.conv_dim, "qkv_in"), _f32(z, cfg.v_total, "z")
        a, b = _f32(alpha, cfg.linear_num_v_heads, "alpha"), _f32(beta, cfg.linear_num_v_heads, "beta")
        out = np.empty(cfg.v_total, dtype=np.float32)
        _chk(self.lib.mfa_gdn_step(self.h, layer, _p(x), _p(z), _p(a), _p(b), _p(out)), "mfa_gdn_step")
        return out

    def prefill_gdn(self, layer, qkv_in, z, alpha, beta) -> np.ndarray:
        cfg = self.cfg
        x = _f32(qkv_in)
        T = x.size // cfg.conv_dim
        z = _f32(z, T * cfg.v_total, "z")
        a = _f32(alpha, T * cfg.linear_num_v_heads, "alpha")
        b = _f32(beta, T * cfg.linear_num_v_heads, "beta")
        out = np.empty((T, cfg.v_total), dtype=np.float32)
        _chk(self.lib.mfa_prefill_gdn(self.h, layer, T, _p(x), _p(z), _p(a), _p(b), _p(out)),
             "mfa_prefill_gdn")
        return out

    # ---- state operations (riir/mod.rs:1950-2125) -----------------------------------
    def memory_clear(self):
        _chk(self.lib.mfa_reset(self.h), "mfa_reset")

    def memory_seq_rm(self, p0: int, p1: int = -1):
        _chk(self.lib.mfa_truncate(self.h, p0, p1), "mfa_truncate")

    def memory_seq_pos_max(self) -> int:
        return self.lib.mfa_pos_max(self.h)

    def kv_export(self, layer):
        n = self.kv_len(layer)
        k = np.zeros((n, self.cfg.kv_dim), dtype=np.float32)
        v = np.zeros((n, self.cfg.kv_dim), dtype=np.float32)
        _chk(self.lib.mfa_kv_export(self.h, layer, n, _p(k), _p(v)), "mfa_kv_export")
        return k, v

    def kv_import(self, layer, k, v):
        if np.asarray(k).dtype == np.uint16:
            k, v = _u16(k), _u16(v)
            n = k.size // self.cfg.kv_dim
            _chk(self.lib.mfa_kv_import_bf16(self.h, layer, n, _p(k), _p(v)), "mfa_kv_import_bf16")
        else:
            k, v = _f32(k), _f32(v)
            n = k.size // self.cfg.kv_dim
            _chk(self.lib.mfa_kv_import(self.h, layer, n, _p(k), _p(v)), "mfa_kv_import")

    def linear_state_export(self, layer):
        cfg = self.cfg
        conv = np.empty(((cfg.conv_kernel_size - 1), cfg.conv_dim), dtype=np.float32)
        ssm = np.empty(cfg.ssm_elems, dtype=np.float32)
        _chk(self.lib.mfa_linear_state_export(self.h, layer, _p(conv), _p(ssm)),
             "mfa_linear_state_export")
        return conv, ssm

    def linear_state_import(self, layer, conv_state, ssm_state):
        cfg = self.cfg
        conv = _f32(conv_state, (cfg.conv_kernel_size - 1) * cfg.conv_dim, "conv_state")
        ssm = _f32(ssm_state, cfg.ssm_elems, "ssm_state")
        _chk(self.lib.mfa_linear_state_import(self.h, layer, _p(conv), _p(ssm)),
             "mfa_linear_state_import")

    def state_size(self) -> int:
        n = self.lib.mfa_state_size(self.h)
        if n < 0:
            _chk(int(n), "mfa_state_size")
        return int(n)

    def state_save(self) -> bytes:
        """The snapshot in the reference's 'MFLX' wire format (state_snapshot.rs)."""
        buf = np.empty(self.state_size(), dtype=np.uint8)
        n = self.lib.mfa_state_save(self.h, _p(buf), buf.size)
        if n < 0:
            _chk(int(n), "mfa_state_save")
        return buf[:int(n)].tobytes()

    def state_load(self, blob: bytes):
        buf = np.frombuffer(blob, dtype=np.uint8)
        _chk(self.lib.mfa_state_load(self.h, _p(buf) if buf.size else None, buf.size), "mfa_state_load")

    # checkpoints by position (riir/mod.rs:2015-2100)
    def checkpoint_pos(self, pos: int):
        _chk(self.lib.mfa_checkpoint_pos(self.h, pos), "mfa_checkpoint_pos")

    def restore_to(self, pos: int):
        """Raises MfaError with code ffi.ERR_NO_CHECKPOINT when nothing is stored at `pos`."""
        _chk(self.lib.mfa_restore_to(self.h, pos), "mfa_restore_to")

    def set_max_checkpoints(self, n: int):
        _chk(self.lib.mfa_set_max_checkpoints(self.h, n), "mfa_set_max_checkpoints")

    def checkpoint_count(self) -> int:
        return _chk(self.lib.mfa_checkpoint_count(self.h), "mfa_checkpoint_count")

    def sync(self):
        _chk(self.lib.mfa_sync(self.h), "mfa_sync")


# ---- per-kernel hooks (riir/mod.rs:444-684), stateless -------------------------------

def sdpa_cpu(kv_len, num_attn_heads, num_kv_heads, head_dim, q, q_gate, k_cache, v_cache):
    """`RsCtx::sdpa_cpu` (riir/mod.rs:444) on the GPU; k/v may be f32 or uint16 bf16 bits."""
    lib = ffi.load()
    qd = num_attn_heads * head_dim
    q, g = _f32(q, qd, "q"), _f32(q_gate, qd, "q_gate")
    out = np.empty(qd, dtype=np.float32)
    n = max(kv_len, 0) * num_kv_heads * head_dim
    if np.asarray(k_cache).dtype == np.uint16:
        k, v = _u16(k_cache, n, "k_cache"), _u16(v_cache, n, "v_cache")
        rc = lib.mfa_sdpa_bf16kv(kv_len, num_attn_heads, num_kv_heads, head_dim, _p(q), _p(g),
                                 _p(k), _p(v), _p(out))
    else:
        k, v = _f32(k_cache, n, "k_cache"), _f32(v_cache, n, "v_cache")
        rc = lib.mfa_sdpa(kv_len, num_attn_heads, num_kv_heads, head_dim, _p(q), _p(g), _p(k),
                          _p(v), _p(out))
    _chk(rc, "mfa_sdpa")
    return out


def attn_scores_batched(num_heads, num_kv_heads, head_dim, seq_len, q, k_cache, scale):
    lib = ffi.load()
    q = _f32(q, num_heads * head_dim, "q")
    k = _f32(k_cache, seq_len * num_kv_heads * head_dim, "k_cache")
    out = np.empty(num_heads * seq_len, dtype=np.float32)
    _chk(lib.mfa_attn_scores_batched(num_heads, num_kv_heads, head_dim, seq_len, _p(q), _p(k),
                                     scale, _p(out)), "mfa_attn_scores_batched")
    return out


def attn_softmax_batched(num_heads, seq_len, scores):
    lib = ffi.load()
    s = _f32(scores, num_heads * seq_len, "scores").copy()
    _chk(lib.mfa_attn_softmax_batched(num_heads, seq_len, _p(s)), "mfa_attn_softmax_batched")
    return s


def attn_values_batched(num_heads, num_kv_heads, head_dim, seq_len, scores, v_cache):
    lib = ffi.load()
    s = _f32(scores, num_heads * seq_len, "scores")
    v = _f32(v_cache, seq_len * num_kv_heads * head_dim, "v_cache")
    out = np.empty(num_heads * head_dim, dtype=np.float32)
    _chk(lib.mfa_attn_values_batched(num_heads, num_kv_heads, head_dim, seq_len, _p(s), _p(v),
                                     _p(out)), "mfa_attn_values_batched")
    return out


def sigmoid_gate(gate, x):
    lib = ffi.load()
    x = _f32(x).copy()
    g = _f32(gate, x.size, "gate")
    _chk(lib.mfa_sigmoid_gate(x.size, _p(g), _p(x)), "mfa_sigmoid_gate")
    return x


def conv1d_step(conv_state, new_input, weight_bf16, channels, kernel_size):
    """The GPU kernel's contract: returns (out, rolled_state)."""
    lib = ffi.load()
    s = _f32(conv_state, (kernel_size - 1) * channels, "conv_state").copy()
    x = _f32(new_input, channels, "new_input")
    w = _u16(weight_bf16, channels * kernel_size, "weight")
    out = np.empty(channels, dtype=np.float32)
    _chk(lib.mfa_conv1d_step(channels, kernel_size, _p(s), _p(x), _p(w), _p(out)), "mfa_conv1d_step")
    return out, s


def rms_norm_qk(num_k_heads, key_dim, q, k):
    lib = ffi.load()
    q = _f32(q, num_k_heads * key_dim, "q").copy()
    k = _f32(k, num_k_heads * key_dim, "k").copy()
    _chk(lib.mfa_rms_norm_qk(num_k_heads, key_dim, _p(q), _p(k)), "mfa_rms_norm_qk")
    return q, k


def rms_norm_bare_cpu(x, eps):
    lib = ffi.load()
    x = _f32(x)
    out = np.empty_like(x)
    _chk(lib.mfa_rms_norm_bare(x.size, eps, _p(x), _p(out)), "mfa_rms_norm_bare")
    return out


def compute_decay_beta(alpha, beta, a_log, dt_bias_bf16):
    lib = ffi.load()
    a = _f32(alpha)
    b, al, dt = _f32(beta, a.size), _f32(a_log, a.size), _u16(dt_bias_bf16, a.size)
    g, bo = np.empty_like(a), np.empty_like(a)
    _chk(lib.mfa_compute_decay_beta(a.size, _p(a), _p(b), _p(al), _p(dt), _p(g), _p(bo)),
         "mfa_compute_decay_beta")
    return g, bo


def gated_delta_net_step(v_heads, k_heads, key_dim, value_dim, g_decay, beta_gate, q, k, v,
                         ssm_state):
    lib = ffi.load()
    g, b = _f32(g_decay, v_heads), _f32(beta_gate, v_heads)
    q, k = _f32(q, k_heads * key_dim, "q"), _f32(k, k_heads * key_dim, "k")
    v = _f32(v, v_heads * value_dim, "v")
    s = _f32(ssm_state, v_heads * value_dim * key_dim, "ssm_state").copy()
    out = np.empty(v_heads * value_dim, dtype=np.float32)
    _chk(lib.mfa_gated_delta_net_step(v_heads, k_heads, key_dim, value_dim, _p(g), _p(b), _p(q),
                                      _p(k), _p(v), _p(s), _p(out)), "mfa_gated_delta_net_step")
    return s, out


def gated_delta_recurrence_cpu(a_log, dt_bias_bf16, alpha, beta, q, k, v, v_heads, k_heads,
                               key_dim, value_dim, ssm_state):
    lib = ffi.load()
    al, dt = _f32(a_log, v_heads), _u16(dt_bias_bf16, v_heads)
    a, b = _f32(alpha, v_heads), _f32(beta, v_heads)
    q, k = _f32(q, k_heads * key_dim, "q"), _f32(k, k_heads * key_dim, "k")
    v = _f32(v, v_heads * value_dim, "v")
    s = _f32(ssm_state, v_heads * value_dim * key_dim, "ssm_state").copy()
    out = np.empty(v_heads * value_dim, dtype=np.float32)
    _chk(lib.mfa_gated_delta_recurrence(_p(al), _p(dt), _p(a), _p(b), _p(q), _p(k), _p(v), v_heads,
                                        k_heads, key_dim, value_dim, _p(s), _p(out)),
         "mfa_gated_delta_recurrence")
    return s, out


def gated_rms_norm(num_heads, dim, eps, x, z, weight_bf16):
    lib = ffi.load()
    x, z = _f32(x, num_heads * dim, "x"), _f32(z, num_heads * dim, "z")
    w = _u16(weight_bf16, dim, "weight")
    out = np.empty_like(x)
    _chk(lib.mfa_gated_rms_norm(num_heads, dim, eps, _p(x), _p(z), _p(w), _p(out)),
         "mfa_gated_rms_norm")
    return out


def rms_norm_gated_cpu(x, z, weight_bf16, eps):
    """`RsCtx::rms_norm_gated_cpu` (riir/mod.rs:526): the one-head case."""
    x = _f32(x)
    return gated_rms_norm(1, x.size, eps, x, z, weight_bf16)


def dequant_matvec_4bit_cpu(packed, scales_bf16, biases_bf16, in_dim, out_dim, x):
    """The reference hook of the same name (cpu_matvec.rs:83-160), computed on the GPU."""
    lib = ffi.load()
    packed = np.ascontiguousarray(packed, dtype=np.uint32).reshape(-1)
    if packed.size != out_dim * (in_dim // 8):
        raise ValueError(f"packed has {packed.size} words, expected {out_dim * (in_dim // 8)}")
    sc = _u16(scales_bf16, out_dim * (in_dim // 64), "scales")
    bi = _u16(biases_bf16, out_dim * (in_dim // 64), "biases")
    x = _f32(x, in_dim, "x")
    out = np.empty(out_dim, dtype=np.float32)
    _chk(lib.mfa_dequant_matvec_4bit(out_dim, in_dim, 64, _p(packed), _p(sc), _p(bi), _p(x), _p(out)),
         "mfa_dequant_matvec_4bit")
    return out


def mla_sdpa_folded(num_heads, kv_lora_rank, qk_rope_head_dim, cache_len, softmax_scale, q_prime, q_pe,
                    latent_cache, rope_k_cache):
    """Attention of one token over a latent cache, the folded form (encode_mla_sdpa_folded,
    gpu_mla.rs:146-200; kernel shaders.metal:1688-1816), host arrays in and out."""
    lib = ffi.load()
    qp = _f32(q_prime, num_heads * kv_lora_rank, "q_prime")
    qe = _f32(q_pe, num_heads * qk_rope_head_dim, "q_pe")
    lat = _f32(latent_cache, cache_len * kv_lora_rank, "latent_cache")
    rk = _f32(rope_k_cache, cache_len * qk_rope_head_dim, "rope_k_cache")
    out = np.empty(num_heads * kv_lora_rank, dtype=np.float32)
    _chk(lib.mfa_mla_sdpa_folded(num_heads, kv_lora_rank, qk_rope_head_dim, cache_len, softmax_scale,
                                 _p(qp), _p(qe), _p(lat), _p(rk), _p(out)), "mfa_mla_sdpa_folded")
    return out

