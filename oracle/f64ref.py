"""Float64 reference of the attention path, written from the mathematics.

TEST INFRASTRUCTURE ONLY.  This is the independent check that pins
oracle/mfa_oracle.c: it is vectorised numpy in float64 built on library
routines (``np.einsum``, ``scipy.special.softmax``/``expit``), shares no code
and no loop structure with the C restatement, and so a dropped term, a wrong
sign, a transposed operand or a wrong GQA map in either one shows up as a
mismatch far above float32 rounding.

Formulas (the reference lines they describe are cited in mfa_oracle.c):
  SDPA   out[h] = softmax_p(scale * q[h] . K[p, h // hpk]) @ V[:, h // hpk] * sigmoid(gate[h])
  conv   y[c] = silu(sum_k hist[k, c] * w[c, k]) with hist = [state(3 rows); new input]
  q/k    q^ = q / sqrt(mean q^2 + 1e-6) / dk ;  k^ = k / sqrt(mean k^2 + 1e-6) / sqrt(dk)
  decay  g = exp(-exp(A_log) * log1p(exp(alpha + dt_bias))) ; beta = sigmoid(b)
  delta  S <- g S ; S <- S + beta (v - S k^) k^T ; o = S q^            (S is [dv, dk])
  norm   y = o / sqrt(mean o^2 + eps) * w * silu(z)
"""
from __future__ import annotations

import numpy as np
from scipy.special import expit, softmax


def bf16_bits_to_f64(bits) -> np.ndarray:
    b = np.asarray(bits, dtype=np.uint16).astype(np.uint32) << 16
    return b.view(np.float32).astype(np.float64)


def silu(x):
    return x * expit(x)


def sdpa(kv_len, Hq, Hkv, d, q, gate, K, V):
    q = np.asarray(q, np.float64).reshape(Hq, d)
    gate = np.asarray(gate, np.float64).reshape(Hq, d)
    K = np.asarray(K, np.float64).reshape(-1, Hkv, d)[:kv_len]
    V = np.asarray(V, np.float64).reshape(-1, Hkv, d)[:kv_len]
    hpk = Hq // Hkv
    Kx = np.repeat(K, hpk, axis=1)          # [L, Hq, d]
    Vx = np.repeat(V, hpk, axis=1)
    s = np.einsum("hd,lhd->hl", q, Kx) / np.sqrt(d)
    w = softmax(s, axis=1)
    o = np.einsum("hl,lhd->hd", w, Vx)
    return (o * expit(gate)).reshape(-1)


def attn_scores(Hq, Hkv, d, L, q, K, scale):
    q = np.asarray(q, np.float64).reshape(Hq, d)
    K = np.repeat(np.asarray(K, np.float64).reshape(L, Hkv, d), Hq // Hkv, axis=1)
    return (np.einsum("hd,lhd->hl", q, K) * scale).reshape(-1)


def attn_softmax(Hq, L, scores):
    return softmax(np.asarray(scores, np.float64).reshape(Hq, L), axis=1).reshape(-1)


def attn_values(Hq, Hkv, d, L, scores, V):
    s = np.asarray(scores, np.float64).reshape(Hq, L)
    V = np.repeat(np.asarray(V, np.float64).reshape(L, Hkv, d), Hq // Hkv, axis=1)
    return np.einsum("hl,lhd->hd", s, V).reshape(-1)


def conv1d_step(conv_state, new_input, w_bf16, C, K):
    hist = np.concatenate([np.asarray(conv_state, np.float64).reshape(K - 1, C),
                           np.asarray(new_input, np.float64).reshape(1, C)], axis=0)  # [K, C]
    w = bf16_bits_to_f64(w_bf16).reshape(C, K)
    return silu(np.einsum("kc,ck->c", hist, w))


def conv_state_shift(conv_state, new_input, C, K):
    s = np.asarray(conv_state, np.float64).reshape(K - 1, C)
    return np.concatenate([s[1:], np.asarray(new_input, np.float64).reshape(1, C)], 0).reshape(-1)


def rms_norm_bare(x, eps):
    x = np.asarray(x, np.float64)
    return x / np.sqrt(np.mean(x * x) + eps)


def rms_norm_qk(Hk, dk, q, k):
    q = np.asarray(q, np.float64).reshape(Hk, dk)
    k = np.asarray(k, np.float64).reshape(Hk, dk)
    qn = q / np.sqrt(np.mean(q * q, axis=1, keepdims=True) + 1e-6) / dk
    kn = k / np.sqrt(np.mean(k * k, axis=1, keepdims=True) + 1e-6) / np.sqrt(dk)
    return qn.reshape(-1), kn.reshape(-1)


def rms_norm_gated(x, z, w_bf16, eps):
    x = np.asarray(x, np.float64)
    z = np.asarray(z, np.float64)
    return x / np.sqrt(np.mean(x * x) + eps) * bf16_bits_to_f64(w_bf16) * silu(z)


def decay_beta(alpha, beta, a_log, dt_bias_bf16):
    alpha = np.asarray(alpha, np.float64)
    sp = np.log1p(np.exp(alpha + bf16_bits_to_f64(dt_bias_bf16)))
    g = np.exp(-np.exp(np.asarray(a_log, np.float64)) * sp)
    return g, expit(np.asarray(beta, np.float64))


def delta_net_step(Hv, Hk, dk, dv, g, b, q, k, v, S):
    """Matrix form of the delta rule; S [Hv, dv, dk]."""
    S = np.asarray(S, np.float64).reshape(Hv, dv, dk)
    rep = Hv // Hk
    q = np.repeat(np.asarray(q, np.float64).reshape(Hk, dk), rep, axis=0)   # [Hv, dk]
    k = np.repeat(np.asarray(k, np.float64).reshape(Hk, dk), rep, axis=0)
    v = np.asarray(v, np.float64).reshape(Hv, dv)
    g = np.asarray(g, np.float64).reshape(Hv, 1, 1)
    b = np.asarray(b, np.float64).reshape(Hv, 1)
    Sd = g * S
    err = (v - np.einsum("hvk,hk->hv", Sd, k)) * b                           # [Hv, dv]
    Sn = Sd + np.einsum("hv,hk->hvk", err, k)
    o = np.einsum("hvk,hk->hv", Sn, q)
    return Sn.reshape(-1), o.reshape(-1)


def gdn_step(Hk, Hv, dk, dv, K, eps, conv_w, a_log, dt_bias, norm_w, qkv_in, z, alpha, beta,
             conv_state, ssm_state):
    """Returns (out, new_conv_state, new_ssm_state), all float64."""
    C = 2 * Hk * dk + Hv * dv
    y = conv1d_step(conv_state, qkv_in, conv_w, C, K)
    cs = conv_state_shift(conv_state, qkv_in, C, K)
    qn, kn = rms_norm_qk(Hk, dk, y[:Hk * dk], y[Hk * dk:2 * Hk * dk])
    g, b = decay_beta(alpha, beta, a_log, dt_bias)
    Sn, o = delta_net_step(Hv, Hk, dk, dv, g, b, qn, kn, y[2 * Hk * dk:], ssm_state)
    o = o.reshape(Hv, dv)
    zz = np.asarray(z, np.float64).reshape(Hv, dv)
    w = bf16_bits_to_f64(norm_w)
    out = o / np.sqrt(np.mean(o * o, axis=1, keepdims=True) + eps) * w * silu(zz)
    return out.reshape(-1), cs, Sn


def prefill_attn(T, kv_len0, Hq, Hkv, d, q, gate, K, V):
    """Causal-mask matrix form (not a loop of decodes)."""
    L = kv_len0 + T
    q = np.asarray(q, np.float64).reshape(T, Hq, d)
    gate = np.asarray(gate, np.float64).reshape(T, Hq, d)
    hpk = Hq // Hkv
    Kx = np.repeat(np.asarray(K, np.float64).reshape(-1, Hkv, d)[:L], hpk, axis=1)
    Vx = np.repeat(np.asarray(V, np.float64).reshape(-1, Hkv, d)[:L], hpk, axis=1)
    s = np.einsum("thd,lhd->thl", q, Kx) / np.sqrt(d)
    mask = np.arange(L)[None, :] <= (kv_len0 + np.arange(T))[:, None]         # [T, L]
    s = np.where(mask[:, None, :], s, -np.inf)
    w = softmax(s, axis=2)
    o = np.einsum("thl,lhd->thd", w, Vx)
    return (o * expit(gate)).reshape(-1)


def rms_norm_per_head(H, d, eps, w_bf16, x):
    x = np.asarray(x, np.float64).reshape(H, d)
    return (x / np.sqrt((x * x).mean(axis=1, keepdims=True) + eps) * bf16_bits_to_f64(w_bf16)).reshape(-1)


def rotary(pos, H, d, rotary_dim, theta, x):
    """The rotation as a complex product: channels (i, i + rotary_dim/2) of each head form
    x_i + j x_{i+half}, multiplied by exp(j pos theta^(-2i/rotary_dim))."""
    x = np.asarray(x, np.float64).reshape(H, d).copy()
    half = rotary_dim // 2
    zc = (x[:, :half] + 1j * x[:, half:rotary_dim]) * np.exp(1j * pos * theta ** (-2.0 * np.arange(half) / rotary_dim))
    x[:, :half], x[:, half:rotary_dim] = zc.real, zc.imag
    return x.reshape(-1)


def attn_prologue(pos, Hq, Hkv, d, rotary_dim, theta, eps, q_norm_bf16, k_norm_bf16, q_proj_out, k_in, v_in):
    qp = np.asarray(q_proj_out, np.float64).reshape(Hq, 2, d)
    q = rotary(pos, Hq, d, rotary_dim, theta, rms_norm_per_head(Hq, d, eps, q_norm_bf16, qp[:, 0]))
    k = rotary(pos, Hkv, d, rotary_dim, theta, rms_norm_per_head(Hkv, d, eps, k_norm_bf16, k_in))
    return q, qp[:, 1].reshape(-1).copy(), k, np.asarray(v_in, np.float64).copy()


def mla_sdpa_folded(H, R, P, L, scale, q_prime, q_pe, latent, rope_k):
    """Attention over a latent cache: scores over [latent | rope_k], softmax, weighted sum of latent."""
    qp = np.asarray(q_prime, np.float64).reshape(H, R)
    qe = np.asarray(q_pe, np.float64).reshape(H, P)
    lat = np.asarray(latent, np.float64).reshape(L, R)
    rk = np.asarray(rope_k, np.float64).reshape(L, P)
    s = (np.einsum("hr,lr->hl", qp, lat) + np.einsum("hp,lp->hl", qe, rk)) * scale
    return np.einsum("hl,lr->hr", softmax(s, axis=1), lat)


def dequant_matvec_4bit(packed, scales_bf16, biases_bf16, in_dim, out_dim, x):
    """Group-64 affine 4-bit weights: nibble n of word w of a row is input 8 w + n."""
    pk = np.asarray(packed, np.uint32).reshape(out_dim, in_dim // 8)
    nib = np.stack([(pk >> (4 * n)) & 0xF for n in range(8)], axis=-1).reshape(out_dim, in_dim).astype(np.float64)
    sc = np.repeat(bf16_bits_to_f64(scales_bf16).reshape(out_dim, in_dim // 64), 64, axis=1)
    bi = np.repeat(bf16_bits_to_f64(biases_bf16).reshape(out_dim, in_dim // 64), 64, axis=1)
    return (nib * sc + bi) @ np.asarray(x, np.float64)

