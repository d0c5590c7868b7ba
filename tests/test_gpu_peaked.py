"""GPU parity of the attention kernels where the soft-max is NOT flat: wide score spreads, a key
that dominates, keys that are all equal.  These are the inputs under which the running maximum
moves by hundreds of log2 units in the middle of a walk, the accumulators are rescaled by factors
far from 1, a split's merge weight is exactly 0 or exactly 1, and the decode step's own token
either carries the whole result or none of it (the reference's adversarial list: large score
spread, kv_len = 1, all-equal keys; its own test inputs reach |score| = 2.4,
tests/diff_oracle.rs:1555-1571; the latent-cache precedent is tests/mla_sdpa_tiled.rs:176-216).

Every case goes through the C ABI and is held to the CPU oracle at the north-star tolerances
(1e-5 for f32 caches, 1e-2 for bf16 caches).  Where scores reach tens of units the oracle's own
f32 sums are a few 1e-6 from exact, so each case also measures the oracle and the kernel against
a float64 evaluation and prints the three distances; the error of the bf16 path's two-part
operand split grows with |score| (about 2^-17 |s|) and is on record in that output.
"""
import numpy as np
import pytest

from tests.util import TOL_BF16, TOL_F32, GdnCase, rel_err

pytestmark = pytest.mark.gpu

THETA = 1.0e7


def _f64_sdpa(L, Hq, Hkv, d, q, g, k, v):
    """Float64 soft-max attention with the sigmoid gate, one kv head at a time."""
    q = np.asarray(q, np.float64).reshape(Hq, d)
    g = np.asarray(g, np.float64).reshape(Hq, d)
    k = np.asarray(k, np.float64).reshape(-1, Hkv, d)[:L]
    v = np.asarray(v, np.float64).reshape(-1, Hkv, d)[:L]
    hpk = Hq // Hkv
    out = np.empty((Hq, d))
    for kvh in range(Hkv):
        s = q[kvh * hpk:(kvh + 1) * hpk] @ k[:, kvh].T / np.sqrt(d)
        w = np.exp(s - s.max(axis=1, keepdims=True))
        w /= w.sum(axis=1, keepdims=True)
        out[kvh * hpk:(kvh + 1) * hpk] = w @ v[:, kvh]
    return (out / (1.0 + np.exp(-g))).reshape(-1)


def _widen(oracle, a):
    return oracle.bf16_to_f32(a) if np.asarray(a).dtype == np.uint16 else a


def _report(name, out, ref, exact):
    e_ref, e_exact, o_exact = rel_err(out, ref), rel_err(out, exact), rel_err(ref, exact)
    print(f"\n[peaked] {name}: kernel-oracle {e_ref:.2e}  kernel-f64 {e_exact:.2e}  oracle-f64 {o_exact:.2e}")
    return e_ref, e_exact, o_exact


def _inputs(oracle, seed, Hq, Hkv, d, L, bf16, score_std):
    """q, gate, K, V whose scaled scores q.k/sqrt(d) have the given standard deviation."""
    rng = np.random.default_rng(seed)
    g = rng.standard_normal(Hq * d).astype(np.float32)
    if bf16:
        q = (rng.standard_normal(Hq * d) * score_std).astype(np.float32)
        k = oracle.f32_to_bf16(rng.standard_normal((L, Hkv * d)).astype(np.float32))
        v = oracle.f32_to_bf16(rng.standard_normal((L, Hkv * d)).astype(np.float32))
    else:
        q = (rng.standard_normal(Hq * d) * score_std).astype(np.float32)
        k = rng.standard_normal((L, Hkv * d)).astype(np.float32)
        v = rng.standard_normal((L, Hkv * d)).astype(np.float32)
    return q, g, k, v


def _decode(mfa, Hq, Hkv, d, L, bf16, q, g, k, v, splits=(0,)):
    from moeflux_amd import Config
    outs = []
    with mfa.Ctx(Config(num_layers=1, full_attn_interval=1, num_attn_heads=Hq, num_kv_heads=Hkv, head_dim=d,
                        kv_capacity=L, kv_dtype=1 if bf16 else 0)) as c:
        c.kv_import(0, k, v)
        for ns in splits:
            c.set_num_splits(ns)
            outs.append(c.sdpa_decode(0, q, g))
    return outs


# The f32 oracle sums sequentially and rounds its dot products at the magnitude of the score; with
# scores of tens of units it is itself up to 1e-5 .. 1e-4 from the exact value (printed as
# oracle-f64).  The f32 criterion is therefore applied with the oracle's own distance from exact
# allowed for, and the kernel may be no further from the exact value than the tolerance or the
# oracle, whichever is larger.
def _check(name, out, ref, exact, bf16):
    e_ref, e_exact, o_exact = _report(name, out, ref, exact)
    if bf16:
        assert e_ref <= TOL_BF16, name
        assert e_exact <= 2e-3, name                      # 2^-17 |s| at |s| of several tens
    else:
        assert e_ref <= TOL_F32 + o_exact, name
        assert e_exact <= max(TOL_F32, o_exact), name


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("score_std", [4.0, 16.0])
@pytest.mark.parametrize("Hq,Hkv,d,L", [(32, 2, 256, 4097), (32, 4, 128, 2500), (8, 8, 64, 700), (32, 2, 256, 40000)])
def test_decode_wide_score_spread(mfa, oracle, Hq, Hkv, d, L, score_std, bf16):
    """Scores with standard deviation 4 and 16 (weights spread over e^-60..1): default split plan
    and forced plans of 1, 3 and 64 splits agree with the oracle and with each other."""
    if L == 40000 and not bf16:
        pytest.skip("the long case runs on the bf16 cache")
    q, g, k, v = _inputs(oracle, 300 + L + int(score_std), Hq, Hkv, d, L, bf16, score_std)
    kf, vf = _widen(oracle, k), _widen(oracle, v)
    ref = oracle.sdpa(L, Hq, Hkv, d, q, g, k, v)
    exact = _f64_sdpa(L, Hq, Hkv, d, q, g, kf, vf)
    outs = _decode(mfa, Hq, Hkv, d, L, bf16, q, g, k, v, splits=(0, 1, 3, 64))
    for ns, out in zip((0, 1, 3, 64), outs):
        _check(f"decode std {score_std} {'bf16' if bf16 else 'f32'} {Hq}/{Hkv}/{d} L={L} splits={ns}", out, ref,
               exact, bf16)


def _plant(q, k, Hq, Hkv, d, head, pos, nats, bf16, oracle):
    """Make position `pos` the key that query head `head` scores `nats` above zero: the key row of
    the head's kv head becomes a multiple of the query."""
    hpk = Hq // Hkv
    qh = q.reshape(Hq, d)[head].astype(np.float64)
    row = (qh * (nats * np.sqrt(d) / (qh @ qh))).astype(np.float32)
    k.reshape(-1, Hkv, d)[pos, head // hpk] = oracle.f32_to_bf16(row) if bf16 else row


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("nats", [30.0, 300.0])
def test_decode_dominant_keys_in_first_and_late_blocks(mfa, oracle, bf16, nats):
    """One key per kv head that a query head scores 30 (weight of everything else e^-30) or 300
    (exactly 0 in f32) above the rest: in block 0 for a head of kv head 0, so that every later block
    is rescaled into nothing; in the last block of a late split for a head of kv head 1, so that the
    maximum jumps by hundreds of log2 units at the end of one workgroup's walk and that split takes
    the whole merge.  The head's output is then the planted position's value row."""
    Hq, Hkv, d, L = 32, 2, 256, 32768 + 37
    q, g, k, v = _inputs(oracle, 77, Hq, Hkv, d, L, bf16, 1.0)
    blk = 32 if bf16 else 16
    late = (L // blk - 3) * blk + blk - 1          # last position of a block near the end
    _plant(q, k, Hq, Hkv, d, 3, 5, nats, bf16, oracle)
    _plant(q, k, Hq, Hkv, d, 16 + 9, late, nats, bf16, oracle)
    kf, vf = _widen(oracle, k), _widen(oracle, v)
    ref = oracle.sdpa(L, Hq, Hkv, d, q, g, k, v)
    exact = _f64_sdpa(L, Hq, Hkv, d, q, g, kf, vf)
    sig = 1.0 / (1.0 + np.exp(-g.reshape(Hq, d).astype(np.float64)))
    for ns, out in zip((0, 1, 7, 200), _decode(mfa, Hq, Hkv, d, L, bf16, q, g, k, v, splits=(0, 1, 7, 200))):
        _check(f"dominant +{nats} {'bf16' if bf16 else 'f32'} splits={ns}", out, ref, exact, bf16)
        o = out.reshape(Hq, d)
        # the textbook limit: the planted rows' values, gated
        assert rel_err(o[3], vf.reshape(-1, Hkv, d)[5, 0] * sig[3]) <= (1e-2 if nats < 100 else 1e-6)
        assert rel_err(o[25], vf.reshape(-1, Hkv, d)[late, 1] * sig[25]) <= (1e-2 if nats < 100 else 1e-6)


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("L", [4097, 32768])
def test_decode_equal_keys_and_zero_query(mfa, oracle, bf16, L):
    """All keys equal, and a zero query: every weight is exactly 1/L whatever the split plan, so
    the output is the mean value row (gated)."""
    Hq, Hkv, d = 32, 2, 256
    q, g, k, v = _inputs(oracle, 5 + L, Hq, Hkv, d, L, bf16, 3.0)
    k[:] = k[0]
    kf, vf = _widen(oracle, k), _widen(oracle, v)
    mean = np.repeat(vf.reshape(L, Hkv, d).astype(np.float64).mean(axis=0), Hq // Hkv, axis=0)
    sig = 1.0 / (1.0 + np.exp(-g.reshape(Hq, d).astype(np.float64)))
    ref = oracle.sdpa(L, Hq, Hkv, d, q, g, k, v)
    for ns, out in zip((0, 5), _decode(mfa, Hq, Hkv, d, L, bf16, q, g, k, v, splits=(0, 5))):
        e_ref, e_exact, _ = _report(f"equal keys L={L} {'bf16' if bf16 else 'f32'} splits={ns}", out, ref, mean * sig)
        assert e_exact <= TOL_F32 and e_ref <= 4e-5      # the oracle's sequential sum over L values is the further one
    q0 = np.zeros_like(q)
    _, _, k2, _ = _inputs(oracle, 6 + L, Hq, Hkv, d, L, bf16, 1.0)
    ref = oracle.sdpa(L, Hq, Hkv, d, q0, g, k2, v)
    out, = _decode(mfa, Hq, Hkv, d, L, bf16, q0, g, k2, v)
    e_ref, e_exact, _ = _report(f"zero query L={L} {'bf16' if bf16 else 'f32'}", out, ref, mean * sig)
    assert e_exact <= TOL_F32 and e_ref <= 4e-5


def _step_ctx(mfa, Hq, Hkv, d, cap, bf16, qn, kn):
    from moeflux_amd import Config
    c = mfa.Ctx(Config(num_layers=1, full_attn_interval=1, num_attn_heads=Hq, num_kv_heads=Hkv, head_dim=d,
                       kv_capacity=cap, kv_dtype=1 if bf16 else 0))
    c.set_full_weights(0, qn, kn)
    return c


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("launches", [2, 3])
@pytest.mark.parametrize("sign", [+1.0, -1.0], ids=["token-dominates", "token-50-below"])
def test_step_whose_own_token_dominates_or_vanishes(mfa, oracle, bf16, launches, sign):
    """One decode token through a full-attention layer behind 3000 cached positions.  Its key is
    its own query direction (every query head of a group the same vector), with norm weights of
    1.8: after the norms its score is +-sqrt(d) 1.8^2 = +-52 while the cache's scores stay within a
    few units.  With +, the token's weight in the merge is 1 and every split's is e^-45; with -, the
    token weighs e^-55 against the cache.  Two-launch form (the token enters the merge as one more
    split) and three-launch form."""
    Hq, Hkv, d, L0 = 32, 2, 256, 3000
    rng = np.random.default_rng(11)
    w = oracle.f32_to_bf16(np.full(d, 1.8, np.float32))
    kc = rng.standard_normal((L0, Hkv * d)).astype(np.float32)
    vc = rng.standard_normal((L0, Hkv * d)).astype(np.float32)
    if bf16:
        kc, vc = (oracle.bf16_to_f32(oracle.f32_to_bf16(a)) for a in (kc, vc))
    base = rng.standard_normal((Hkv, d)).astype(np.float32)
    qp = rng.standard_normal((Hq, 2, d)).astype(np.float32)
    hpk = Hq // Hkv
    for h in range(Hq):
        qp[h, 0] = base[h // hpk]
    k_new = (sign * base).reshape(-1).astype(np.float32)
    v_new = rng.standard_normal(Hkv * d).astype(np.float32)
    rq, rg, rk, rv = oracle.attn_prologue(L0, Hq, Hkv, d, d // 4, THETA, 1e-6, w, w, qp.reshape(-1), k_new, v_new)
    if bf16:
        rk, rv = (oracle.bf16_to_f32(oracle.f32_to_bf16(a)) for a in (rk, rv))
    kall, vall = np.vstack([kc, rk[None]]), np.vstack([vc, rv[None]])
    score = float(rq.reshape(Hq, d)[0] @ rk.reshape(Hkv, d)[0] / np.sqrt(d))
    assert abs(abs(score) - 51.8) < 1.5 and np.sign(score) == sign
    ref = oracle.sdpa(L0 + 1, Hq, Hkv, d, rq, rg, kall, vall)
    exact = _f64_sdpa(L0 + 1, Hq, Hkv, d, rq, rg, kall, vall)
    with _step_ctx(mfa, Hq, Hkv, d, L0 + 8, bf16, w, w) as c:
        c.kv_import(0, kc, vc)
        c.set_step_launches(launches)
        out = c.full_attn_step(0, L0, qp.reshape(-1), k_new, v_new)
    name = f"step {'+' if sign > 0 else '-'}52 {'bf16' if bf16 else 'f32'} {launches} launches"
    e_ref, e_exact, o_exact = _report(name, out, ref, exact)
    # the query handed to the core is the kernel's own norm and rotation (1e-6 from the oracle's),
    # which a score of 52 turns into a few 1e-5 of weight when the token does not dominate
    assert e_ref <= (TOL_BF16 if bf16 else 1e-4)
    if sign > 0:
        sig = 1.0 / (1.0 + np.exp(-rg.reshape(Hq, d).astype(np.float64)))
        assert rel_err(out.reshape(Hq, d)[0], rv.reshape(Hkv, d)[0] * sig[0]) <= 1e-6


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("T,L0", [(160, 0), (200, 1000), (6, 5000)])
def test_prompt_chunk_wide_spread_and_dominant_keys(mfa, oracle, bf16, T, L0):
    """Prompt chunks with score standard deviation 6 and planted keys: 160 tokens from an empty
    cache and 200 behind 1000 positions run the chunk kernel (lazy rescale of the accumulators: the
    planted key raises a row's maximum by far more than 2^8 in the middle of its walk, once), 6
    tokens behind 5000 positions run the split-K path with per-row causal limits."""
    Hq, Hkv, d = 32, 4, 128
    rng = np.random.default_rng(T + L0)
    n = L0 + T
    k = rng.standard_normal((n, Hkv * d)).astype(np.float32)
    v = rng.standard_normal((n, Hkv * d)).astype(np.float32)
    q = (rng.standard_normal((T, Hq * d)) * 6.0).astype(np.float32)
    g = rng.standard_normal((T, Hq * d)).astype(np.float32)
    hpk = Hq // Hkv
    # planted keys: one in the cached part (or early in the chunk), one inside the chunk, each aimed
    # at one head of the chunk's last token and scoring 250 above zero
    for head, pos in ((1, max(L0 // 2, 3)), (hpk + 2, L0 + T // 2), (2 * hpk, n - 1)):
        qh = q[T - 1].reshape(Hq, d)[head].astype(np.float64)
        k.reshape(n, Hkv, d)[pos, head // hpk] = (qh * (250.0 * np.sqrt(d) / (qh @ qh))).astype(np.float32)
    if bf16:
        k, v = (oracle.bf16_to_f32(oracle.f32_to_bf16(a)) for a in (k, v))
    ref = oracle.prefill_attn(T, L0, Hq, Hkv, d, q, g, k, v).reshape(T, Hq * d)
    from moeflux_amd import Config
    with mfa.Ctx(Config(num_layers=1, full_attn_interval=1, num_attn_heads=Hq, num_kv_heads=Hkv, head_dim=d,
                        kv_capacity=n, kv_dtype=1 if bf16 else 0)) as c:
        if L0:
            c.kv_import(0, k[:L0], v[:L0])
        out = c.prefill_attn(0, q, g, k[L0:], v[L0:])
    worst_ref = worst_exact = worst_oracle = 0.0
    for t in sorted({0, 1, T // 3, T // 2, T - 2, T - 1}):
        exact = _f64_sdpa(L0 + t + 1, Hq, Hkv, d, q[t], g[t], k, v)
        worst_ref = max(worst_ref, rel_err(out[t], ref[t]))
        worst_exact = max(worst_exact, rel_err(out[t], exact))
        worst_oracle = max(worst_oracle, rel_err(ref[t], exact))
    print(f"\n[peaked] chunk T={T} L0={L0} {'bf16' if bf16 else 'f32'}: kernel-oracle {worst_ref:.2e}  "
          f"kernel-f64 {worst_exact:.2e}  oracle-f64 {worst_oracle:.2e}")
    if bf16:
        assert rel_err(out, ref) <= TOL_BF16 and worst_exact <= 2e-3
    else:
        assert worst_ref <= TOL_F32 + worst_oracle and worst_exact <= max(TOL_F32, worst_oracle)
        assert rel_err(out, ref) <= 1e-4
    # the last token's planted heads return the planted positions' value rows
    sig = 1.0 / (1.0 + np.exp(-g[T - 1].reshape(Hq, d).astype(np.float64)))
    vv = v.reshape(n, Hkv, d)
    for head, pos in ((1, max(L0 // 2, 3)), (hpk + 2, L0 + T // 2), (2 * hpk, n - 1)):
        assert rel_err(out[T - 1].reshape(Hq, d)[head], vv[pos, head // hpk] * sig[head]) <= 1e-5, (head, pos)


def _gdn_ctx(mfa, case):
    from moeflux_amd import Config
    c = mfa.Ctx(Config(num_layers=1, full_attn_interval=2, linear_num_k_heads=case.Hk, linear_num_v_heads=case.Hv,
                       linear_key_dim=case.dk, linear_value_dim=case.dv, conv_kernel_size=case.K,
                       rms_norm_eps=case.eps))
    c.set_linear_weights(0, case.conv_w, case.a_log, case.dt_bias, case.norm_w)
    return c


@pytest.mark.parametrize("T", [1, 5, 130])
def test_gdn_gates_at_their_extremes(mfa, T):
    """alpha = 100 (the reference's naive softplus log(1 + exp(x)) overflows to +inf there, so the
    decay is exactly 0 and the state is forgotten; linear_attn.rs:357-370), alpha = -100 (decay 1),
    beta logits of +-30 (beta = 1 - 1e-13 and 1e-13): through the single step (T = 1), the
    token-by-token chunk (5) and the blocked chunk (130, two blocks and a ragged third)."""
    case = GdnCase(41 + T, 2, 4, 128, 128, T=T)
    Hv = case.Hv
    pattern_a = np.array([100.0, -100.0, 0.3, 100.0], np.float32)[:Hv]
    pattern_b = np.array([30.0, -30.0, 30.0, 0.1], np.float32)[:Hv]
    for t in range(T):
        if t % 3 != 1:                       # every third token keeps its random gates
            case.alpha[t] = np.roll(pattern_a, t)
            case.beta[t] = np.roll(pattern_b, t)
    ref_out, ref_conv, ref_ssm = case.oracle()
    assert np.isfinite(ref_out).all()
    with _gdn_ctx(mfa, case) as c:
        c.linear_state_import(0, case.conv_state, case.ssm_state)
        if T == 1:
            out = c.gdn_step(0, case.qkv[0], case.z[0], case.alpha[0], case.beta[0])[None]
        else:
            out = c.prefill_gdn(0, case.qkv, case.z, case.alpha, case.beta)
        conv, ssm = c.linear_state_export(0)
    assert np.isfinite(out).all() and np.isfinite(ssm).all()
    e_out, e_ssm = rel_err(out, ref_out), rel_err(ssm, ref_ssm)
    print(f"\n[peaked] gdn extreme gates T={T}: out {e_out:.2e} state {e_ssm:.2e}")
    assert e_out <= TOL_F32 and e_ssm <= TOL_F32
    assert np.array_equal(conv.reshape(-1), ref_conv)
    if T == 1:   # the value head whose decay is exactly 0 and whose beta is 1: S' = (v - 0) k^T, of rank one
        S = ssm.reshape(Hv, case.dv, case.dk)
        R = ref_ssm.reshape(Hv, case.dv, case.dk)
        sv = np.linalg.svd(S[0].astype(np.float64), compute_uv=False)
        assert rel_err(S[0], R[0]) <= TOL_F32 and sv[1] <= 1e-5 * sv[0]
