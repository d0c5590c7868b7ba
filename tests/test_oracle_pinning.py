"""Pins the CPU oracle (oracle/mfa_oracle.c) before anything is compared with it.

The reference holds no numeric vectors for the attention kernels (its tests store
input formulas and tolerances, tests/diff_oracle.rs), so every function of the
oracle is held in place by
  (1) the committed float64 fixtures tests/golden/attention_f64.json (vectorised
      library-routine formulation, independent of the C loops),
  (2) closed forms and invariants the mathematics fixes, chosen so that a dropped
      term, a wrong sign, a wrong GQA map or a transposed operand fails,
  (3) the reference's own three unit tests (linear_attn.rs:420-445).
Runs on the CPU.
"""
import json
import os

import numpy as np
import pytest

from oracle import cref, f64ref
from tests.util import rel_err

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "attention_f64.json")))
F32 = 2e-6  # float32 evaluation of a float64 expected value, small shapes


def a32(x):
    return np.asarray(x, dtype=np.float32)


def u16(x):
    return np.asarray(x, dtype=np.uint16)


# ---- (1) golden fixtures -----------------------------------------------------

@pytest.mark.parametrize("c", GOLD["sdpa"], ids=lambda c: f"Hq{c['Hq']}Hkv{c['Hkv']}d{c['d']}L{c['L']}")
def test_golden_sdpa(c):
    out = cref.sdpa(c["L"], c["Hq"], c["Hkv"], c["d"], a32(c["q"]), a32(c["gate"]), a32(c["k"]), a32(c["v"]))
    assert rel_err(out, c["out"]) <= F32
    # the bf16-cache twin on bf16-exact inputs is the same function
    kb, vb = cref.f32_to_bf16(a32(c["k"])), cref.f32_to_bf16(a32(c["v"]))
    out_b = cref.sdpa(c["L"], c["Hq"], c["Hkv"], c["d"], a32(c["q"]), a32(c["gate"]), kb, vb)
    exp_b = f64ref.sdpa(c["L"], c["Hq"], c["Hkv"], c["d"], c["q"], c["gate"],
                        f64ref.bf16_bits_to_f64(kb), f64ref.bf16_bits_to_f64(vb))
    assert rel_err(out_b, exp_b) <= F32


@pytest.mark.parametrize("c", GOLD["sdpa"], ids=lambda c: f"L{c['L']}")
def test_golden_attn_kernels(c):
    Hq, Hkv, d, L = c["Hq"], c["Hkv"], c["d"], c["L"]
    scale = 1.0 / np.sqrt(d)
    s = cref.attn_scores(Hq, Hkv, d, L, a32(c["q"]), a32(c["k"]), scale)
    assert rel_err(s, f64ref.attn_scores(Hq, Hkv, d, L, c["q"], c["k"], scale)) <= F32
    p = cref.attn_softmax(Hq, L, s)
    assert rel_err(p, f64ref.attn_softmax(Hq, L, s)) <= F32
    o = cref.attn_values(Hq, Hkv, d, L, p, a32(c["v"]))
    assert rel_err(o, f64ref.attn_values(Hq, Hkv, d, L, p, c["v"])) <= F32
    # the four kernels chained are sdpa
    assert rel_err(cref.sigmoid_gate(a32(c["gate"]), o), c["out"]) <= F32
    # strided score rows (production uses stride GPU_KV_SEQ) hold the same values
    s2 = cref.attn_scores(Hq, Hkv, d, L, a32(c["q"]), a32(c["k"]), scale, seq_stride=L + 3)
    assert np.array_equal(s2.reshape(Hq, L + 3)[:, :L].reshape(-1), s)


@pytest.mark.parametrize("c", GOLD["gdn_step"], ids=lambda c: f"Hk{c['Hk']}Hv{c['Hv']}dk{c['dk']}dv{c['dv']}K{c['K']}")
def test_golden_gdn_step(c):
    cs, ss = a32(c["conv_state0"]), a32(c["ssm_state0"])
    for t in range(c["T"]):
        o, cs, ss = cref.gdn_step(c["Hk"], c["Hv"], c["dk"], c["dv"], c["K"], c["eps"], u16(c["conv_w"]),
                                  a32(c["a_log"]), u16(c["dt_bias"]), u16(c["norm_w"]), a32(c["qkv"][t]),
                                  a32(c["z"][t]), a32(c["alpha"][t]), a32(c["beta"][t]), cs, ss)
        assert rel_err(o, c["out"][t]) <= 5e-6, t
    assert np.array_equal(cs, a32(c["conv_state"]))
    assert rel_err(ss, c["ssm_state"]) <= 5e-6
    # the chunk form is the same loop
    T = c["T"]
    out, cs2, ss2 = cref.prefill_gdn(T, c["Hk"], c["Hv"], c["dk"], c["dv"], c["K"], c["eps"],
                                     u16(c["conv_w"]), a32(c["a_log"]), u16(c["dt_bias"]),
                                     u16(c["norm_w"]), a32(c["qkv"]), a32(c["z"]), a32(c["alpha"]),
                                     a32(c["beta"]), a32(c["conv_state0"]), a32(c["ssm_state0"]))
    assert rel_err(out, np.asarray(c["out"])) <= 5e-6
    assert np.array_equal(cs2, cs) and np.array_equal(ss2, ss)


@pytest.mark.parametrize("c", GOLD["conv1d"], ids=lambda c: f"C{c['C']}K{c['K']}")
def test_golden_conv1d(c):
    out = cref.conv1d_step(a32(c["state"]), a32(c["x"]), u16(c["w"]), c["C"], c["K"])
    assert rel_err(out, c["out"]) <= F32
    assert np.array_equal(cref.conv_state_shift(a32(c["state"]), a32(c["x"]), c["C"], c["K"]), a32(c["shifted"]))


@pytest.mark.parametrize("c", GOLD["rms_norm_qk"], ids=lambda c: f"Hk{c['Hk']}dk{c['dk']}")
def test_golden_rms_norm_qk(c):
    qn, kn = cref.rms_norm_qk(c["Hk"], c["dk"], a32(c["q"]), a32(c["k"]))
    assert rel_err(qn, c["qn"]) <= F32 and rel_err(kn, c["kn"]) <= F32


def test_golden_decay_beta_delta_step_gated_norm():
    c = GOLD["decay_beta"][0]
    g, b = cref.decay_beta(a32(c["alpha"]), a32(c["beta"]), a32(c["a_log"]), u16(c["dt_bias"]))
    assert rel_err(g, c["g"]) <= F32 and rel_err(b, c["b"]) <= F32
    for c in GOLD["delta_net_step"]:
        S, o = cref.delta_net_step(c["Hv"], c["Hk"], c["dk"], c["dv"], a32(c["g"]), a32(c["b"]),
                                   a32(c["q"]), a32(c["k"]), a32(c["v"]), a32(c["S"]))
        assert rel_err(S, c["S_new"]) <= F32 and rel_err(o, c["out"]) <= F32
    c = GOLD["rms_norm_gated"][0]
    assert rel_err(cref.rms_norm_gated(a32(c["x"]), a32(c["z"]), u16(c["w"]), c["eps"]), c["out"]) <= F32


@pytest.mark.parametrize("c", GOLD["prefill_attn"], ids=lambda c: f"T{c['T']}L0{c['L0']}")
def test_golden_prefill_attn(c):
    out = cref.prefill_attn(c["T"], c["L0"], c["Hq"], c["Hkv"], c["d"], a32(c["q"]), a32(c["gate"]),
                            a32(c["k"]), a32(c["v"]))
    assert rel_err(out, c["out"]) <= F32


# ---- (2) closed forms and invariants: full attention -------------------------------

def _rand_sdpa(seed, Hq=8, Hkv=2, d=16, L=12):
    rng = np.random.default_rng(seed)
    return (Hq, Hkv, d, L, rng.standard_normal(Hq * d).astype(np.float32),
            rng.standard_normal(Hq * d).astype(np.float32),
            rng.standard_normal((L, Hkv * d)).astype(np.float32),
            rng.standard_normal((L, Hkv * d)).astype(np.float32))


def sig(x):
    return 1.0 / (1.0 + np.exp(-np.asarray(x, np.float64)))


def test_sdpa_one_position_returns_gated_v():
    Hq, Hkv, d, _, q, g, k, v = _rand_sdpa(1, L=1)
    out = cref.sdpa(1, Hq, Hkv, d, q, g, k, v).reshape(Hq, d)
    vexp = np.repeat(v.reshape(Hkv, d), Hq // Hkv, axis=0) * sig(g).reshape(Hq, d)
    assert rel_err(out, vexp) <= F32


def test_sdpa_equal_keys_or_zero_query_average_v():
    Hq, Hkv, d, L, q, g, k, v = _rand_sdpa(2)
    mean_v = np.repeat(v.reshape(L, Hkv, d).mean(0), Hq // Hkv, axis=0) * sig(g).reshape(Hq, d)
    k_same = np.tile(k[:1], (L, 1))
    assert rel_err(cref.sdpa(L, Hq, Hkv, d, q, g, k_same, v), mean_v) <= F32
    assert rel_err(cref.sdpa(L, Hq, Hkv, d, np.zeros_like(q), g, k, v), mean_v) <= F32


def test_sdpa_zero_gate_halves():
    Hq, Hkv, d, L, q, g, k, v = _rand_sdpa(3)
    big = cref.sdpa(L, Hq, Hkv, d, q, np.full_like(g, 40.0), k, v)   # sigmoid -> 1
    half = cref.sdpa(L, Hq, Hkv, d, q, np.zeros_like(g), k, v)
    assert rel_err(half, 0.5 * big) <= F32


def test_sdpa_invariant_to_score_shift_and_position_permutation():
    Hq, Hkv, d, L, q, g, k, v = _rand_sdpa(4)
    base = cref.sdpa(L, Hq, Hkv, d, q, g, k, v)
    u = np.random.default_rng(5).standard_normal(Hkv * d).astype(np.float32)
    assert rel_err(cref.sdpa(L, Hq, Hkv, d, q, g, k + u, v), base) <= 2e-5  # every score + q.u
    perm = np.random.default_rng(6).permutation(L)
    assert rel_err(cref.sdpa(L, Hq, Hkv, d, q, g, k[perm], v[perm]), base) <= F32


def test_sdpa_gqa_map_is_h_div_heads_per_kv():
    Hq, Hkv, d, L, q, g, k, v = _rand_sdpa(7)
    q = q.reshape(Hq, d).copy()
    g = g.reshape(Hq, d).copy()
    q[:] = q[0]
    g[:] = g[0]
    out = cref.sdpa(L, Hq, Hkv, d, q, g, k, v).reshape(Hq, d)
    hpk = Hq // Hkv
    for h in range(Hq):
        same = (h // hpk) == 0
        assert np.array_equal(out[h], out[0]) == same, h   # consecutive heads share a kv head


def test_sdpa_dominant_key_selects_its_value():
    Hq, Hkv, d, L, q, g, k, v = _rand_sdpa(8, Hq=4, Hkv=4)
    k = (0.01 * k).reshape(L, Hkv, d)
    qh = q.reshape(Hq, d)
    k[5] = 40.0 * qh / np.linalg.norm(qh, axis=1, keepdims=True)   # score gap >> 30 for every head
    out = cref.sdpa(L, Hq, Hkv, d, q, np.full_like(g, 40.0), k.reshape(L, -1), v).reshape(Hq, d)
    assert rel_err(out, v.reshape(L, Hkv, d)[5]) <= F32


def test_sdpa_rejects_what_the_reference_rejects():
    Hq, Hkv, d, L, q, g, k, v = _rand_sdpa(9)
    with pytest.raises(ValueError):
        cref.sdpa(0, Hq, Hkv, d, q, g, k, v)            # sdpa.rs:71
    with pytest.raises(ValueError):
        cref.sdpa(L, 6, 4, d, q[:6 * d], g[:6 * d], np.zeros((L, 4 * d), np.float32),
                  np.zeros((L, 4 * d), np.float32))      # gpu_attn.rs:262


def test_softmax_rows_sum_to_one_and_order_preserved():
    s = np.random.default_rng(10).standard_normal(5 * 40).astype(np.float32) * 4
    p = cref.attn_softmax(5, 40, s).reshape(5, 40)
    assert np.allclose(p.sum(1), 1.0, atol=1e-6)
    assert np.array_equal(np.argsort(p, axis=1), np.argsort(s.reshape(5, 40), axis=1))


# ---- closed forms: gated delta net ----------------------------------------------------

def test_conv_identity_tap_and_state_roll():
    C, K = 7, 4
    rng = np.random.default_rng(11)
    w = np.zeros((C, K), np.float32)
    w[:, K - 1] = 1.0
    wb = cref.f32_to_bf16(w)
    state = rng.standard_normal((K - 1) * C).astype(np.float32)
    xs = rng.standard_normal((3, C)).astype(np.float32)
    out = cref.conv1d_step(state, xs[0], wb, C, K)
    assert rel_err(out, f64ref.silu(xs[0].astype(np.float64))) <= F32   # taps [0,0,0,1] => silu(in)
    for x in xs:
        state = cref.conv_state_shift(state, x, C, K)
    assert np.array_equal(state.reshape(3, C), xs)                        # last three inputs, oldest first


def test_conv_equals_numpy_convolve_over_a_sequence():
    C, K, T = 3, 4, 9
    rng = np.random.default_rng(12)
    wb = cref.f32_to_bf16(rng.standard_normal((C, K)).astype(np.float32))
    w = cref.bf16_to_f32(wb).astype(np.float64)
    xs = rng.standard_normal((T, C)).astype(np.float32)
    state = np.zeros((K - 1) * C, np.float32)
    got = []
    for x in xs:
        got.append(cref.conv1d_step(state, x, wb, C, K))
        state = cref.conv_state_shift(state, x, C, K)
    got = np.array(got)
    for c in range(C):
        full = np.convolve(xs[:, c].astype(np.float64), w[c, ::-1])[:T]   # causal, tap K-1 on the newest
        assert rel_err(got[:, c], f64ref.silu(full)) <= F32


def test_qk_norm_lengths_and_scale_equivariance():
    Hk, dk = 3, 128
    rng = np.random.default_rng(13)
    q, k = rng.standard_normal(Hk * dk).astype(np.float32), rng.standard_normal(Hk * dk).astype(np.float32)
    qn, kn = cref.rms_norm_qk(Hk, dk, q, k)
    assert np.allclose(np.linalg.norm(kn.reshape(Hk, dk), axis=1), 1.0, atol=1e-5)
    assert np.allclose(np.linalg.norm(qn.reshape(Hk, dk), axis=1), 1.0 / np.sqrt(dk), atol=1e-6)
    q2, k2 = cref.rms_norm_qk(Hk, dk, 7.0 * q, 0.25 * k)
    assert rel_err(q2, qn) <= 1e-5 and rel_err(k2, kn) <= 1e-5


def test_decay_beta_special_values():
    z = np.zeros(3, np.float32)
    zb = cref.f32_to_bf16(z)
    g, b = cref.decay_beta(z, z, z, zb)
    assert np.allclose(g, 0.5, atol=1e-7) and np.allclose(b, 0.5, atol=1e-7)   # exp(-ln 2), sigmoid(0)
    g, _ = cref.decay_beta(np.full(3, -60.0, np.float32), z, z, zb)
    assert np.allclose(g, 1.0, atol=1e-7)                                        # alpha -> -inf
    g, _ = cref.decay_beta(np.full(3, 100.0, np.float32), z, z, zb)
    assert np.all(g == 0.0)              # naive softplus overflows to +inf, as the reference's does
    # dt_bias enters the decay only, never beta (infer.m:2701-2702)
    g1, b1 = cref.decay_beta(z, z, z, cref.f32_to_bf16(np.ones(3)))
    assert np.allclose(g1, np.exp(-np.log1p(np.e)), atol=1e-6) and np.allclose(b1, 0.5)


def test_delta_rule_closed_forms():
    Hv, Hk, dk, dv = 4, 2, 16, 8
    rng = np.random.default_rng(14)
    q, k = rng.standard_normal(Hk * dk).astype(np.float32), rng.standard_normal(Hk * dk).astype(np.float32)
    qn, kn = cref.rms_norm_qk(Hk, dk, q, k)
    v = rng.standard_normal(Hv * dv).astype(np.float32)
    g = rng.uniform(0.3, 0.9, Hv).astype(np.float32)
    b = rng.uniform(0.2, 0.8, Hv).astype(np.float32)
    rep = Hv // Hk
    kx = np.repeat(kn.reshape(Hk, dk), rep, axis=0).astype(np.float64)
    qx = np.repeat(qn.reshape(Hk, dk), rep, axis=0).astype(np.float64)
    # from S = 0:  S' = beta v k^T,  out = beta v (k.q)
    S, o = cref.delta_net_step(Hv, Hk, dk, dv, g, b, qn, kn, v, np.zeros(Hv * dv * dk, np.float32))
    S_exp = b[:, None, None] * v.reshape(Hv, dv)[:, :, None] * kx[:, None, :]
    assert rel_err(S, S_exp) <= F32
    assert rel_err(o, (b[:, None] * v.reshape(Hv, dv)) * (kx * qx).sum(1)[:, None]) <= F32
    # beta = 0:  S' = g S,  out = g S q
    S0 = rng.standard_normal(Hv * dv * dk).astype(np.float32)
    S, o = cref.delta_net_step(Hv, Hk, dk, dv, g, np.zeros(Hv, np.float32), qn, kn, v, S0)
    assert rel_err(S, g[:, None, None] * S0.reshape(Hv, dv, dk)) <= F32
    assert rel_err(o, np.einsum("hvk,hk->hv", g[:, None, None] * S0.reshape(Hv, dv, dk), qx)) <= F32
    # g = 1, beta = 1, |k| = 1:  the rule writes v at key k  (S' k = v)
    one = np.ones(Hv, np.float32)
    S, _ = cref.delta_net_step(Hv, Hk, dk, dv, one, one, qn, kn, v, S0)
    assert rel_err(np.einsum("hvk,hk->hv", S.reshape(Hv, dv, dk), kx), v.reshape(Hv, dv)) <= 1e-5
    # the update is delta k^T (rows = value index), not k delta^T
    assert S.reshape(Hv, dv, dk).shape == (Hv, dv, dk)
    d_rows = (S.reshape(Hv, dv, dk) - S0.reshape(Hv, dv, dk))[0]
    assert np.linalg.matrix_rank(d_rows.astype(np.float64), tol=1e-5) == 1
    assert rel_err(d_rows[0] / np.linalg.norm(d_rows[0]) * np.sign(d_rows[0] @ kx[0]), kx[0] / np.linalg.norm(kx[0])) <= 1e-4


def test_gated_norm_closed_forms_and_reference_unit_tests():
    dv = 16
    rng = np.random.default_rng(15)
    x = rng.standard_normal(dv).astype(np.float32)
    ones = cref.f32_to_bf16(np.ones(dv))
    assert not cref.rms_norm_gated(x, np.zeros(dv, np.float32), ones, 1e-6).any()   # z = 0 => 0
    z = np.full(dv, 30.0, np.float32)                                               # silu(z) -> z
    exp = x.astype(np.float64) / np.sqrt(np.mean(x.astype(np.float64) ** 2) + 1e-6) * 30.0
    assert rel_err(cref.rms_norm_gated(x, z, ones, 1e-6), exp) <= F32
    # linear_attn.rs:420-445
    assert np.all(np.abs(cref.rms_norm_bare(np.ones(16, np.float32), 1e-6) - 1.0) < 1e-3)
    w = cref.f32_to_bf16(np.array([[1.0]], np.float32))
    assert cref.conv1d_step(np.zeros(0, np.float32), np.zeros(1, np.float32), w, 1, 1)[0] == 0.0   # silu(0)
    assert abs(cref.conv1d_step(np.zeros(0, np.float32), np.full(1, 10.0, np.float32), w, 1, 1)[0] - 10.0) < 1e-3


def test_gdn_rejects_what_the_reference_rejects():
    with pytest.raises(ValueError):   # v_heads % k_heads != 0 (linear_attn.rs:306)
        cref.delta_net_step(3, 2, 4, 4, np.ones(3), np.ones(3), np.zeros(8), np.zeros(8), np.zeros(12),
                            np.zeros(48))
    with pytest.raises(ValueError):   # zero dim (linear_attn.rs:166)
        cref.rms_norm_bare(np.zeros(0, np.float32), 1e-6)


# ---- what precedes the attention core: per-head norm, rotation, q/gate split ------------

PRO = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "attn_prologue_f64.json")))


@pytest.mark.parametrize("c", PRO["attn_prologue"], ids=lambda c: f"Hq{c['Hq']}d{c['d']}rd{c['rotary_dim']}pos{c['pos']}")
def test_golden_attn_prologue(c):
    q, g, kr, vr = cref.attn_prologue(c["pos"], c["Hq"], c["Hkv"], c["d"], c["rotary_dim"], c["theta"], c["eps"],
                                      u16(c["q_norm"]), u16(c["k_norm"]), a32(c["q_proj_out"]), a32(c["k"]),
                                      a32(c["v"]))
    assert rel_err(q, a32(c["q_out"])) <= 1e-5 and rel_err(kr, a32(c["k_row"])) <= 1e-5
    assert np.array_equal(g, a32(c["gate_out"])) and np.array_equal(vr, a32(c["v_row"]))


def test_rope_position_zero_is_the_identity():
    """rope.rs:352-383 (the reference's own unit test): cos = 1, sin = 0 leave every channel as it was."""
    Hq, Hkv, d = 4, 2, 32
    q = (np.arange(Hq * d) * 0.001).astype(np.float32)
    k = (np.arange(Hkv * d) * 0.001).astype(np.float32)
    q2, k2 = cref.apply_rotary_emb(0, Hq, Hkv, d, d // 4, 1e7, q, k)
    assert np.array_equal(q, q2) and np.array_equal(k, k2)


def test_rope_is_a_rotation_of_the_paired_channels_only():
    """Pairs (i, i + half) keep their norm, channels past rotary_dim are untouched, channel 0's
    pair turns by exactly pos radians (theta^0 = 1), and two rotations compose: R(a) R(b) = R(a+b)
    on the first pair, which a wrong sign in either output line breaks."""
    rng = np.random.default_rng(3)
    H, d, rd = 3, 32, 8
    half = rd // 2
    x = rng.standard_normal(H * d).astype(np.float32)
    y, _ = cref.apply_rotary_emb(7, H, 1, d, rd, 1e7, x, x[:d])
    X, Y = x.reshape(H, d), y.reshape(H, d)
    assert np.array_equal(X[:, rd:], Y[:, rd:])
    assert np.allclose(X[:, :half] ** 2 + X[:, half:rd] ** 2, Y[:, :half] ** 2 + Y[:, half:rd] ** 2, rtol=1e-5)
    ang = np.arctan2(Y[:, half], Y[:, 0]) - np.arctan2(X[:, half], X[:, 0])
    assert np.allclose(np.mod(ang - 7.0 + np.pi, 2 * np.pi) - np.pi, 0.0, atol=1e-5)
    y2, _ = cref.apply_rotary_emb(5, H, 1, d, rd, 1e7, y, y[:d])
    y12, _ = cref.apply_rotary_emb(12, H, 1, d, rd, 1e7, x, x[:d])
    assert np.allclose(y2.reshape(H, d)[:, [0, half]], y12.reshape(H, d)[:, [0, half]], atol=2e-6)


def test_rope_frequency_table():
    f = cref.rope_inv_freq(1e7, 64)
    assert f[0] == 1.0 and np.all(np.diff(f) < 0)
    assert np.allclose(f, 1e7 ** (-2.0 * np.arange(32) / 64), rtol=3e-7)


def test_rms_norm_per_head_properties():
    """Unit weight: every head leaves with mean square 1; a head's scale does not leak into
    another head; scaling the input leaves the output unchanged (up to eps)."""
    rng = np.random.default_rng(4)
    H, d = 5, 64
    one = cref.f32_to_bf16(np.ones(d))
    x = rng.standard_normal(H * d).astype(np.float32)
    y = cref.rms_norm_per_head(H, d, 1e-6, one, x).reshape(H, d)
    assert np.allclose((y.astype(np.float64) ** 2).mean(axis=1), 1.0, rtol=1e-5)
    x2 = x.copy().reshape(H, d)
    x2[2] *= 37.0
    y2 = cref.rms_norm_per_head(H, d, 1e-6, one, x2).reshape(H, d)
    assert np.array_equal(np.delete(y, 2, axis=0), np.delete(y2, 2, axis=0)) and rel_err(y2[2], y[2]) <= 1e-6
    w = cref.f32_to_bf16(1.0 + 0.2 * rng.standard_normal(d))
    yw = cref.rms_norm_per_head(H, d, 1e-6, w, x).reshape(H, d)
    assert rel_err(yw, y * cref.bf16_to_f32(w)) <= 1e-6


# ---- 4-bit dequantising matvec (the projections either side of the attention core) -------

def test_dequant_matvec_reference_unit_tests():
    """cpu_matvec.rs:366-417, the reference's own known-answer tests: all nibbles 1 with
    scale 1 bias 0 against ones gives 64; a zero input gives zero whatever the bias; nibble 0
    with bias 2 against ones gives 128."""
    ones = np.ones(64, np.float32)
    assert cref.dequant_matvec_4bit(np.full(8, 0x11111111, np.uint32), [0x3F80], [0x0000], 64, 1, ones)[0] == 64.0
    out = cref.dequant_matvec_4bit(np.full(16, 0xFFFFFFFF, np.uint32), [0x3F80] * 2, [0x3F80] * 2, 64, 2,
                                   np.zeros(64, np.float32))
    assert np.array_equal(out, np.zeros(2, np.float32))
    assert cref.dequant_matvec_4bit(np.zeros(8, np.uint32), [0x40A0], [0x4000], 64, 1, ones)[0] == 128.0


def test_dequant_matvec_against_float64_matrix_product():
    """Unpack the nibbles with numpy (bit n*4 of each word is input 8*word + n), build the
    dequantised matrix in float64 and multiply: pins nibble order, group stride and row stride."""
    rng = np.random.default_rng(8)
    out_dim, in_dim = 7, 256
    packed = rng.integers(0, 2 ** 32, size=(out_dim, in_dim // 8), dtype=np.uint64).astype(np.uint32)
    sc = cref.f32_to_bf16(rng.standard_normal((out_dim, in_dim // 64)) * 0.1)
    bi = cref.f32_to_bf16(rng.standard_normal((out_dim, in_dim // 64)) * 0.5)
    x = rng.standard_normal(in_dim).astype(np.float32)
    nib = ((packed[:, :, None] >> (4 * np.arange(8, dtype=np.uint32))) & 0xF).reshape(out_dim, in_dim).astype(np.float64)
    W = nib * np.repeat(cref.bf16_to_f32(sc).astype(np.float64), 64, axis=1) + \
        np.repeat(cref.bf16_to_f32(bi).astype(np.float64), 64, axis=1)
    got = cref.dequant_matvec_4bit(packed, sc, bi, in_dim, out_dim, x)
    assert rel_err(got, (W @ x.astype(np.float64)).astype(np.float32)) <= 2e-6
    # linear in x; a one-hot x picks one dequantised column
    e = np.zeros(in_dim, np.float32)
    e[77] = 1.0
    assert np.allclose(cref.dequant_matvec_4bit(packed, sc, bi, in_dim, out_dim, e), W[:, 77], rtol=1e-6)


# ---- attention over a latent cache (MLA, folded form) ---------------------------------

def _mla_inputs(seed, H, R, P, L):
    rng = np.random.default_rng(seed)
    return (rng.standard_normal((H, R)).astype(np.float32) * 0.3, rng.standard_normal((H, P)).astype(np.float32) * 0.3,
            rng.standard_normal((L, R)).astype(np.float32), rng.standard_normal((L, P)).astype(np.float32))


@pytest.mark.parametrize("H,R,P,L", [(3, 8, 4, 1), (3, 8, 4, 7), (16, 64, 16, 33), (5, 32, 8, 130)])
def test_mla_against_float64_softmax(H, R, P, L):
    from scipy.special import softmax
    qp, qe, lat, rk = _mla_inputs(L, H, R, P, L)
    scale = 0.37
    s = (qp.astype(np.float64) @ lat.astype(np.float64).T + qe.astype(np.float64) @ rk.astype(np.float64).T) * scale
    want = softmax(s, axis=1) @ lat.astype(np.float64)
    got = cref.mla_sdpa_folded(H, R, P, L, scale, qp, qe, lat, rk).reshape(H, R)
    assert rel_err(got, want.astype(np.float32)) <= F32


def test_mla_is_multi_query_attention_over_the_concatenated_key():
    """The folded form is MQA with key [latent | rope_k], value latent, one kv head and no gate:
    the already pinned orc_sdpa, fed the concatenation (value padded to the key's width, query
    rescaled to its 1/sqrt(d), gate large so the sigmoid is 1), must agree."""
    H, R, P, L = 4, 48, 16, 57
    qp, qe, lat, rk = _mla_inputs(2, H, R, P, L)
    scale = 0.21
    d = R + P
    q = np.concatenate([qp, qe], axis=1) * (scale * np.sqrt(d))
    k = np.concatenate([lat, rk], axis=1)
    v = np.concatenate([lat, np.zeros((L, P), np.float32)], axis=1)
    ref = cref.sdpa(L, H, 1, d, q.astype(np.float32), np.full(H * d, 40.0, np.float32), k, v).reshape(H, d)[:, :R]
    got = cref.mla_sdpa_folded(H, R, P, L, scale, qp, qe, lat, rk).reshape(H, R)
    assert rel_err(got, ref) <= 3e-6


def test_mla_closed_forms():
    H, R, P, L = 3, 16, 4, 9
    qp, qe, lat, rk = _mla_inputs(4, H, R, P, L)
    f = lambda *a: cref.mla_sdpa_folded(H, R, P, len(a[2]), 0.5, *a).reshape(H, R)
    # one position: the output is that latent row, whatever the query
    assert np.allclose(f(qp, qe, lat[:1], rk[:1]), np.broadcast_to(lat[0], (H, R)), rtol=1e-6)
    # zero query: uniform weights, the mean latent row
    z = f(qp * 0, qe * 0, lat, rk)
    assert np.allclose(z, np.broadcast_to(lat.mean(axis=0), (H, R)), atol=2e-7, rtol=1e-5)
    # only the rope part differs between positions with equal latent rows: output is that row
    same = np.broadcast_to(lat[0], (L, R)).copy()
    assert np.allclose(f(qp, qe, same, rk), np.broadcast_to(lat[0], (H, R)), rtol=1e-5, atol=1e-6)
    # a rope key far along q_pe takes all the weight: this pins that the rope term enters the score
    rk2 = rk.copy()
    rk2[5] = 60.0 * qe[1] / np.dot(qe[1], qe[1])
    out = f(qp * 0, qe, lat, rk2)
    assert np.allclose(out[1], lat[5], rtol=1e-4, atol=1e-5)


# ---- committed float64 fixtures for the functions around the core --------------------

ATC = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "around_the_core_f64.json")))


@pytest.mark.parametrize("case", ATC["mla_sdpa_folded"], ids=lambda c: f"H{c['H']}_L{c['L']}")
def test_mla_golden(case):
    c = case
    got = cref.mla_sdpa_folded(c["H"], c["R"], c["P"], c["L"], c["scale"], np.array(c["q_prime"], np.float32),
                               np.array(c["q_pe"], np.float32), np.array(c["latent"], np.float32),
                               np.array(c["rope_k"], np.float32))
    assert rel_err(got, np.array(c["out"])) <= F32


@pytest.mark.parametrize("case", ATC["dequant_matvec_4bit"], ids=lambda c: f"{c['out_dim']}x{c['in_dim']}")
def test_dequant_matvec_golden(case):
    c = case
    got = cref.dequant_matvec_4bit(np.array(c["packed"], np.uint32), np.array(c["scales"], np.uint16),
                                   np.array(c["biases"], np.uint16), c["in_dim"], c["out_dim"],
                                   np.array(c["x"], np.float32))
    # a row is a signed sum of in_dim terms accumulated in f32, as the reference accumulates it: the
    # rounding of the partial sums is relative to their size, not to the (cancelled) result
    assert rel_err(got, np.array(c["out"])) <= 1e-5

