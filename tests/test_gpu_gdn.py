"""GPU parity of the Gated-DeltaNet path against the CPU oracle, through the C ABI."""
import numpy as np
import pytest

from tests.util import TOL_F32, GdnCase, idx, rel_err

pytestmark = pytest.mark.gpu


def _ctx(mfa, case, num_layers=1):
    from moeflux_amd import Config
    c = mfa.Ctx(Config(num_layers=num_layers, full_attn_interval=num_layers + 1,
                       linear_num_k_heads=case.Hk, linear_num_v_heads=case.Hv,
                       linear_key_dim=case.dk, linear_value_dim=case.dv,
                       conv_kernel_size=case.K, rms_norm_eps=case.eps))
    for l in range(num_layers):
        c.set_linear_weights(l, case.conv_w, case.a_log, case.dt_bias, case.norm_w)
    return c


@pytest.mark.parametrize("Hk,Hv,dk,dv", [(16, 32, 128, 128), (16, 64, 128, 128), (2, 2, 128, 128),
                                          (4, 8, 64, 64), (1, 3, 128, 128)])
def test_gdn_step_matches_oracle(mfa, Hk, Hv, dk, dv):
    case = GdnCase(5 + Hv, Hk, Hv, dk, dv, T=6)
    ref_out, ref_conv, ref_ssm = case.oracle()
    with _ctx(mfa, case) as c:
        c.linear_state_import(0, case.conv_state, case.ssm_state)
        for t in range(case.T):
            out = c.gdn_step(0, case.qkv[t], case.z[t], case.alpha[t], case.beta[t])
            assert rel_err(out, ref_out[t]) <= TOL_F32, f"step {t}"
        conv, ssm = c.linear_state_export(0)
    assert np.array_equal(conv.reshape(-1), ref_conv)  # the history is copied, never computed
    assert rel_err(ssm, ref_ssm) <= TOL_F32


def test_config2_from_zero_state_and_prefill(mfa):
    """The 16 / 32-head, dk = dv = 128 step shape with A_log = dt_bias = 0 and unit norm weight; the
    chunk call equals the token loop."""
    case = GdnCase(0xC0FFEE + 2, 16, 32, 128, 128, T=9, zero_state=True, plain=True)
    ref_out, ref_conv, ref_ssm = case.oracle()
    with _ctx(mfa, case, num_layers=2) as c:
        out = c.prefill_gdn(1, case.qkv, case.z, case.alpha, case.beta)
        conv, ssm = c.linear_state_export(1)
        conv0, ssm0 = c.linear_state_export(0)
    assert rel_err(out, ref_out) <= TOL_F32
    assert np.array_equal(conv.reshape(-1), ref_conv)
    assert rel_err(ssm, ref_ssm) <= TOL_F32
    assert not conv0.any() and not ssm0.any()  # the other layer is untouched


def test_gdn_kernel_hooks(mfa, oracle):
    """The five reference kernels one at a time (inputs of tests/diff_oracle.rs:2091-2260)."""
    Hk, Hv, dk, dv, K = 16, 32, 128, 128, 4
    case = GdnCase(3, Hk, Hv, dk, dv)
    C = case.C
    state = (np.sin(0.013 * idx(3 * C)) * 0.4 + 0.02).astype(np.float32)
    x = (np.cos(0.019 * idx(C)) * 0.5 - 0.1).astype(np.float32)
    out, rolled = mfa.conv1d_step(state, x, case.conv_w, C, K)
    assert rel_err(out, oracle.conv1d_step(state, x, case.conv_w, C, K)) <= TOL_F32
    assert np.array_equal(rolled, oracle.conv_state_shift(state, x, C, K))

    q = (np.sin(0.011 * idx(Hk * dk)) * 0.4 + 0.05).astype(np.float32)
    k = (np.cos(0.019 * idx(Hk * dk)) * 0.5 - 0.1).astype(np.float32)
    v = (np.sin(0.023 * idx(Hv * dv)) * 0.6 + 0.02).astype(np.float32)
    qn, kn = mfa.rms_norm_qk(Hk, dk, q, k)
    qr, kr = oracle.rms_norm_qk(Hk, dk, q, k)
    assert rel_err(qn, qr) <= TOL_F32 and rel_err(kn, kr) <= TOL_F32

    xb = (np.sin(0.011 * idx(128)) * 0.6 + 0.05).astype(np.float32)
    zb = (np.cos(0.017 * idx(128)) * 1.2 - 0.1).astype(np.float32)
    assert rel_err(mfa.rms_norm_bare_cpu(xb, 1e-6), oracle.rms_norm_bare(xb, 1e-6)) <= TOL_F32
    assert rel_err(mfa.rms_norm_gated_cpu(xb, zb, case.norm_w, 1e-6),
                   oracle.rms_norm_gated(xb, zb, case.norm_w, 1e-6)) <= TOL_F32

    alpha = (np.sin(0.013 * idx(Hv)) * 0.3).astype(np.float32)
    beta = (np.cos(0.017 * idx(Hv)) * 0.5).astype(np.float32)
    g, b = mfa.compute_decay_beta(alpha, beta, case.a_log, case.dt_bias)
    gr, br = oracle.decay_beta(alpha, beta, case.a_log, case.dt_bias)
    assert rel_err(g, gr) <= TOL_F32 and rel_err(b, br) <= TOL_F32

    s1, o1 = mfa.gated_delta_net_step(Hv, Hk, dk, dv, gr, br, qr, kr, v, case.ssm_state)
    s2, o2 = oracle.delta_net_step(Hv, Hk, dk, dv, gr, br, qr, kr, v, case.ssm_state)
    assert rel_err(o1, o2) <= TOL_F32 and rel_err(s1, s2) <= TOL_F32

    zero = np.zeros_like(case.ssm_state)  # the reference's test starts from a zero state
    s1, o1 = mfa.gated_delta_recurrence_cpu(case.a_log, case.dt_bias, alpha, beta, qr, kr, v, Hv,
                                            Hk, dk, dv, zero)
    s2, o2 = oracle.gated_delta_recurrence(case.a_log, case.dt_bias, alpha, beta, qr, kr, v, Hv,
                                           Hk, dk, dv, zero)
    assert rel_err(o1, o2) <= TOL_F32 and rel_err(s1, s2) <= TOL_F32

    z = case.z[0]
    y1 = mfa.gated_rms_norm(Hv, dv, 1e-6, o2, z, case.norm_w)
    y2 = np.concatenate([oracle.rms_norm_gated(o2[h * dv:(h + 1) * dv], z[h * dv:(h + 1) * dv],
                                               case.norm_w, 1e-6) for h in range(Hv)])
    assert rel_err(y1, y2) <= TOL_F32


@pytest.mark.parametrize("T", [2, 3, 4, 5, 37, 47, 48, 64, 65, 100, 200])
def test_chunk_equals_token_loop(mfa, T):
    """The chunk kernels do, token for token, the operations of the single-step kernel
    (riir/mod.rs:1196-1214: a prompt is a loop of steps) and differ from it only in f32
    rounding: below 48 tokens in how a state row's dot products are grouped over lanes, from
    48 tokens on by the blocked form of the recurrence.  The conv history is copied and must
    be identical.  T below, at and above the conv width exercises the history ring on both
    sides of the chunk boundary; 47/48 and 64/65 the switch of algorithm and a block edge."""
    case = GdnCase(40 + T, 4, 8, 128, 128, T=T)
    with _ctx(mfa, case, num_layers=2) as c:
        for layer in (0, 1):
            c.linear_state_import(layer, case.conv_state, case.ssm_state)
        chunk = c.prefill_gdn(0, case.qkv, case.z, case.alpha, case.beta)
        loop = np.stack([c.gdn_step(1, case.qkv[t], case.z[t], case.alpha[t], case.beta[t])
                         for t in range(T)])
        s0, s1 = c.linear_state_export(0), c.linear_state_export(1)
        # a further single step continues correctly from the chunk's ring and state
        extra = GdnCase(99, 4, 8, 128, 128, T=1)
        n0 = c.gdn_step(0, extra.qkv[0], extra.z[0], extra.alpha[0], extra.beta[0])
        n1 = c.gdn_step(1, extra.qkv[0], extra.z[0], extra.alpha[0], extra.beta[0])
    tol = 2e-6 if T < 48 else TOL_F32
    assert rel_err(chunk, loop) <= tol
    assert np.array_equal(s0[0], s1[0]) and rel_err(s0[1], s1[1]) <= tol
    assert rel_err(n0, n1) <= tol
    ref_out, ref_conv, ref_ssm = case.oracle()
    assert rel_err(chunk, ref_out) <= TOL_F32
    assert np.array_equal(s0[0].reshape(-1), ref_conv) and rel_err(s0[1], ref_ssm) <= TOL_F32


@pytest.mark.parametrize("T", [50, 64, 129])
def test_chunk_blocked_form_dk64(mfa, T):
    """Chunks of 48 tokens and more take the blocked form (64-token blocks on the matrix
    cores); here at the 64-wide head shape, from a non-zero state, with a ragged last block."""
    case = GdnCase(70 + T, 2, 4, 64, 64, T=T)
    ref_out, ref_conv, ref_ssm = case.oracle()
    with _ctx(mfa, case) as c:
        c.linear_state_import(0, case.conv_state, case.ssm_state)
        out = c.prefill_gdn(0, case.qkv, case.z, case.alpha, case.beta)
        conv, ssm = c.linear_state_export(0)
    assert rel_err(out, ref_out) <= TOL_F32
    assert np.array_equal(conv.reshape(-1), ref_conv)
    assert rel_err(ssm, ref_ssm) <= TOL_F32


def test_config4_gdn_chunk_of_512_from_zero_state(mfa):
    """The DeltaNet half of the 512-token prompt chunk: 512 tokens of the 16 / 32-head step shape from a zero state,
    against 512 sequential oracle steps; outputs and the final state."""
    case = GdnCase(0xC0FFEE + 4, 16, 32, 128, 128, T=512, zero_state=True)
    ref_out, ref_conv, ref_ssm = case.oracle()
    with _ctx(mfa, case) as c:
        out = c.prefill_gdn(0, case.qkv, case.z, case.alpha, case.beta)
        conv, ssm = c.linear_state_export(0)
    assert rel_err(out, ref_out) <= TOL_F32
    worst = max(rel_err(out[t], ref_out[t]) for t in range(0, 512, 37))
    assert worst <= 5e-5
    assert np.array_equal(conv.reshape(-1), ref_conv)
    assert rel_err(ssm, ref_ssm) <= TOL_F32


def _same_tokens(c):
    c.qkv[:] = c.qkv[0]


def _same_tokens_beta_one(c):
    c.qkv[:] = c.qkv[0]
    c.beta[:] = 20.0
    c.alpha[:] = -20.0


def _drift(c):
    d = np.random.default_rng(1).standard_normal(c.qkv.shape).astype(np.float32) * 0.02
    c.qkv[:] = c.qkv[0] + np.cumsum(d, axis=0)


def _strong_decay(c):
    c.alpha[:] = 8.0
    c.a_log[:] = 1.5


def _big(c):
    c.qkv *= 30.0


@pytest.mark.parametrize("mutate", [_same_tokens, _same_tokens_beta_one, _drift, _strong_decay, _big],
                         ids=["identical-tokens", "identical-tokens-beta1-g1", "drifting-tokens", "strong-decay",
                              "inputs-x30"])
def test_blocked_form_on_hard_inputs(mfa, mutate):
    """The blocked form inverts I + A per 64-token block, A built from key-key products: keys that
    repeat or drift slowly make A dense with entries near beta, gates at their extremes stretch the
    decay factors (e^{L_C} underflows under strong decay).  Same criterion as everywhere."""
    case = GdnCase(5, 2, 4, 128, 128, T=256)
    mutate(case)
    ref_out, ref_conv, ref_ssm = case.oracle()
    with _ctx(mfa, case) as c:
        c.linear_state_import(0, case.conv_state, case.ssm_state)
        out = c.prefill_gdn(0, case.qkv, case.z, case.alpha, case.beta)
        conv, ssm = c.linear_state_export(0)
    assert np.isfinite(out).all()
    assert rel_err(out, ref_out) <= TOL_F32 and rel_err(ssm, ref_ssm) <= TOL_F32
    assert np.array_equal(conv.reshape(-1), ref_conv)


def test_chunk_at_the_a17b_head_counts(mfa):
    """16 key heads, 64 value heads (variants.rs:396-397), a ragged 130-token chunk."""
    case = GdnCase(6, 16, 64, 128, 128, T=130)
    ref_out, ref_conv, ref_ssm = case.oracle()
    with _ctx(mfa, case) as c:
        c.linear_state_import(0, case.conv_state, case.ssm_state)
        out = c.prefill_gdn(0, case.qkv, case.z, case.alpha, case.beta)
        _, ssm = c.linear_state_export(0)
    assert rel_err(out, ref_out) <= TOL_F32 and rel_err(ssm, ref_ssm) <= TOL_F32


def test_prompt_longer_than_one_segment(mfa):
    """A prompt of more than 4096 tokens goes through the chunk kernels in 4096-token segments; the
    ring and the state carry from one segment to the next as they do between calls."""
    case = GdnCase(8, 2, 4, 64, 64, T=4096 + 70)
    ref_out, ref_conv, ref_ssm = case.oracle()
    with _ctx(mfa, case) as c:
        c.linear_state_import(0, case.conv_state, case.ssm_state)
        out = c.prefill_gdn(0, case.qkv, case.z, case.alpha, case.beta)
        conv, ssm = c.linear_state_export(0)
    assert rel_err(out, ref_out) <= TOL_F32 and rel_err(ssm, ref_ssm) <= TOL_F32
    assert rel_err(out[4090:], ref_out[4090:]) <= 5e-5
    assert np.array_equal(conv.reshape(-1), ref_conv)


def test_random_shapes_and_conv_widths(mfa):
    """Seeded random head counts, both head widths, conv widths 2 to 8 and chunk lengths on either
    side of the switch to the blocked form: a chunk after a few single steps, against the oracle's
    sequential steps; outputs, the conv history (bit for bit) and the recurrent state."""
    rng = np.random.default_rng(77)
    shapes = [(128, 2, 4, 8, 5, 70), (64, 1, 2, 2, 0, 130), (128, 1, 1, 5, 9, 48), (64, 2, 8, 8, 17, 64)]
    for _ in range(14):
        Hk = int(rng.choice([1, 2, 4]))
        K = int(rng.choice([2, 3, 4, 5, 8]))
        shapes.append((int(rng.choice([64, 128])), Hk, Hk * int(rng.choice([1, 2, 4])), K, int(rng.integers(0, 2 * K)),
                       int(rng.choice([1, 2, 7, 40, 48, 63, 64, 65, 130]))))
    for case_no, (dk, Hk, Hv, K, pre, T) in enumerate(shapes):
        case = GdnCase(500 + case_no, Hk, Hv, dk, dk, K=K, T=pre + T)
        ref_out, ref_conv, ref_ssm = case.oracle()
        with _ctx(mfa, case) as c:
            c.linear_state_import(0, case.conv_state, case.ssm_state)
            outs = [c.gdn_step(0, case.qkv[t], case.z[t], case.alpha[t], case.beta[t]) for t in range(pre)]
            outs.extend(c.prefill_gdn(0, case.qkv[pre:], case.z[pre:], case.alpha[pre:], case.beta[pre:]))
            conv, ssm = c.linear_state_export(0)
        what = (case_no, Hk, Hv, dk, K, pre, T)
        assert rel_err(np.stack(outs), ref_out) <= TOL_F32, what
        assert np.array_equal(conv.reshape(-1), ref_conv), what
        assert rel_err(ssm, ref_ssm) <= TOL_F32, what
