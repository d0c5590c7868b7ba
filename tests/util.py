"""Shared helpers for the tests: seeded inputs, the reference's closed-form test
inputs, and the error measures the tolerances are stated in."""
import numpy as np

from oracle import cref

# north-star tolerances
TOL_F32 = 1e-5    # fp32 paths: max|a-b| / max|b|
TOL_BF16 = 1e-2   # bf16-KV paths


def rel_err(a, b) -> float:
    """max|a-b| / max|b| — the reference's own measure (tests/diff_oracle.rs:2771-2772
    uses max_abs_diff / max_abs_out)."""
    a = np.asarray(a, np.float64).reshape(-1)
    b = np.asarray(b, np.float64).reshape(-1)
    return float(np.abs(a - b).max() / max(np.abs(b).max(), 1e-30))


def rel_err_rows(a, b, row_len) -> float:
    """The same measure taken per row of `row_len` values (one head of one token), worst row:
    max over rows of max|a_row - b_row| / max|b_row|.  A row of small values is held to its own
    scale instead of hiding under a large neighbour."""
    a = np.asarray(a, np.float64).reshape(-1, row_len)
    b = np.asarray(b, np.float64).reshape(-1, row_len)
    return float((np.abs(a - b).max(axis=1) / np.maximum(np.abs(b).max(axis=1), 1e-30)).max())


def cosine(a, b) -> float:
    a = np.asarray(a, np.float64).reshape(-1)
    b = np.asarray(b, np.float64).reshape(-1)
    return float(a @ b / (np.linalg.norm(a) * np.linalg.norm(b) + 1e-300))


def idx(n):
    return np.arange(n, dtype=np.float32)


def synth(seed, n, s):
    """tests/diff_oracle.rs:2698-2705: sin(phi)*s + cos(1.7 phi)*s/2, phi = 0.13 seed + 0.017 i."""
    phi = np.float32(0.13) * np.float32(seed) + np.float32(0.017) * idx(n)
    return (np.sin(phi) * np.float32(s) + np.cos(np.float32(1.7) * phi) * np.float32(s) / 2).astype(np.float32)


def sdpa_reference_inputs(Hq, Hkv, d, kv_len):
    """tests/diff_oracle.rs:1555-1571."""
    q = (np.sin(0.011 * idx(Hq * d)) * 0.6 + 0.05).astype(np.float32)
    g = (np.cos(0.007 * idx(Hq * d)) * 1.2 - 0.1).astype(np.float32)
    k = (np.sin(0.013 * idx(kv_len * Hkv * d)) * 0.5 + 0.02).astype(np.float32)
    v = (np.cos(0.017 * idx(kv_len * Hkv * d)) * 0.4 - 0.05).astype(np.float32)
    return q, g, k, v


def sdpa_random_inputs(seed, Hq, Hkv, d, L, bf16=False, qscale=None):
    rng = np.random.default_rng(seed)
    qs = 1.0 / np.sqrt(d) if qscale is None else qscale
    q = (rng.standard_normal(Hq * d) * qs).astype(np.float32)
    g = rng.standard_normal(Hq * d).astype(np.float32)
    if bf16:
        k = cref.f32_to_bf16(rng.standard_normal((L, Hkv * d)).astype(np.float32))
        v = cref.f32_to_bf16(rng.standard_normal((L, Hkv * d)).astype(np.float32))
    else:
        ks = 1.0 / np.sqrt(d)
        k = (rng.standard_normal((L, Hkv * d)) * ks).astype(np.float32)
        v = (rng.standard_normal((L, Hkv * d)) * ks).astype(np.float32)
    return q, g, k, v


class GdnCase:
    """One Gated-DeltaNet layer's constants, state and T tokens of inputs."""

    def __init__(self, seed, Hk, Hv, dk, dv, K=4, T=1, zero_state=False, plain=False):
        rng = np.random.default_rng(seed)
        self.Hk, self.Hv, self.dk, self.dv, self.K, self.T = Hk, Hv, dk, dv, K, T
        self.C = C = 2 * Hk * dk + Hv * dv
        self.eps = 1e-6
        self.conv_w = cref.f32_to_bf16(rng.standard_normal(C * K) * 0.5)
        if plain:  # the plain step shape: A_log = 0, dt_bias = 0, norm weight = 1
            self.a_log = np.zeros(Hv, np.float32)
            self.dt_bias = cref.f32_to_bf16(np.zeros(Hv))
            self.norm_w = cref.f32_to_bf16(np.ones(dv))
        else:
            self.a_log = (rng.standard_normal(Hv) * 0.5).astype(np.float32)
            self.dt_bias = cref.f32_to_bf16(rng.standard_normal(Hv) * 0.5)
            self.norm_w = cref.f32_to_bf16(1.0 + 0.2 * rng.standard_normal(dv))
        if zero_state:
            self.conv_state = np.zeros((K - 1) * C, np.float32)
            self.ssm_state = np.zeros(Hv * dv * dk, np.float32)
        else:
            self.conv_state = rng.standard_normal((K - 1) * C).astype(np.float32)
            self.ssm_state = (rng.standard_normal(Hv * dv * dk) * 0.02).astype(np.float32)
        self.qkv = rng.standard_normal((T, C)).astype(np.float32)
        self.z = rng.standard_normal((T, Hv * dv)).astype(np.float32)
        self.alpha = rng.standard_normal((T, Hv)).astype(np.float32)
        self.beta = rng.standard_normal((T, Hv)).astype(np.float32)

    def oracle(self):
        """(out [T, Hv*dv], conv_state, ssm_state) after T steps."""
        return cref.prefill_gdn(self.T, self.Hk, self.Hv, self.dk, self.dv, self.K, self.eps,
                                self.conv_w, self.a_log, self.dt_bias, self.norm_w, self.qkv,
                                self.z, self.alpha, self.beta, self.conv_state, self.ssm_state)
