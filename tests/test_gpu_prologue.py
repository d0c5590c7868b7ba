"""GPU parity of what precedes the attention core in a full-attention layer (q/gate split,
per-head RMS norms, partial rotation, cache append) against the CPU oracle, through the C ABI."""
import numpy as np
import pytest

from tests.util import TOL_F32, rel_err

pytestmark = pytest.mark.gpu

THETA = 1.0e7


def _case(seed, Hq, Hkv, d):
    rng = np.random.default_rng(seed)
    from oracle import cref
    qn = cref.f32_to_bf16(1.0 + 0.3 * rng.standard_normal(d))
    kn = cref.f32_to_bf16(1.0 + 0.3 * rng.standard_normal(d))
    return rng, qn, kn


def _ctx(mfa, Hq, Hkv, d, cap, bf16=False):
    from moeflux_amd import Config
    return mfa.Ctx(Config(num_layers=1, full_attn_interval=1, num_attn_heads=Hq, num_kv_heads=Hkv, head_dim=d,
                          kv_capacity=cap, kv_dtype=1 if bf16 else 0))


@pytest.mark.parametrize("Hq,Hkv,d", [(32, 2, 256), (32, 4, 128), (8, 2, 64)])
@pytest.mark.parametrize("pos", [0, 1, 777, 32767])
def test_prologue_matches_oracle(mfa, oracle, Hq, Hkv, d, pos):
    """q and the gate handed to the attention core, and the cache row: the reference's order of
    operations (full_attn_forward.rs:238-293) at the default rotation (theta 1e7, d/4 channels)."""
    rng, qn, kn = _case(pos + d, Hq, Hkv, d)
    qp = rng.standard_normal(Hq * 2 * d).astype(np.float32)
    k, v = rng.standard_normal(Hkv * d).astype(np.float32), rng.standard_normal(Hkv * d).astype(np.float32)
    rq, rg, rk, rv = oracle.attn_prologue(pos, Hq, Hkv, d, d // 4, THETA, 1e-6, qn, kn, qp, k, v)
    with _ctx(mfa, Hq, Hkv, d, 8) as c:
        c.set_full_weights(0, qn, kn)
        q, g = c.attn_prologue(0, pos, qp, k, v)
        assert c.kv_len(0) == 1
        ke, ve = c.kv_export(0)
    assert np.array_equal(g, rg)
    assert rel_err(q, rq) <= TOL_F32
    assert rel_err(ke[0], rk) <= TOL_F32 and np.array_equal(ve[0], rv)


def test_prologue_other_rotation_and_bf16_cache(mfa, oracle):
    """theta 1e4 over the whole head (the other variant family's constants, variants.rs:369-371),
    and a bf16 cache: the stored row is the oracle's row rounded to bf16."""
    Hq, Hkv, d, pos = 8, 2, 64, 41
    rng, qn, kn = _case(5, Hq, Hkv, d)
    qp = rng.standard_normal(Hq * 2 * d).astype(np.float32)
    k, v = rng.standard_normal(Hkv * d).astype(np.float32), rng.standard_normal(Hkv * d).astype(np.float32)
    rq, rg, rk, rv = oracle.attn_prologue(pos, Hq, Hkv, d, d, 1.0e4, 1e-6, qn, kn, qp, k, v)
    with _ctx(mfa, Hq, Hkv, d, 8, bf16=True) as c:
        c.set_full_weights(0, qn, kn)
        c.set_rope(1.0e4, d)
        q, g = c.attn_prologue(0, pos, qp, k, v)
        ke, ve = c.kv_export(0)
    assert rel_err(q, rq) <= TOL_F32 and np.array_equal(g, rg)
    assert rel_err(ke[0], rk) <= 2 ** -8 and np.array_equal(ve[0], oracle.bf16_to_f32(oracle.f32_to_bf16(rv)))


@pytest.mark.parametrize("bf16", [False, True])
def test_full_attn_steps_equal_the_reference_composition(mfa, oracle, bf16):
    """Twelve tokens through prologue + attention core in one call each: equals the oracle's
    prologue, cache append and sdpa composed as full_attn_layer_forward composes them
    (full_attn_forward.rs:234-389); with a bf16 cache the oracle attends over the rounded rows."""
    Hq, Hkv, d, n = 32, 2, 256, 12
    rng, qn, kn = _case(9, Hq, Hkv, d)
    kc, vc = np.zeros((n, Hkv * d), np.float32), np.zeros((n, Hkv * d), np.float32)
    with _ctx(mfa, Hq, Hkv, d, 16, bf16=bf16) as c:
        c.set_full_weights(0, qn, kn)
        for t in range(n):
            qp = rng.standard_normal(Hq * 2 * d).astype(np.float32)
            k, v = rng.standard_normal(Hkv * d).astype(np.float32), rng.standard_normal(Hkv * d).astype(np.float32)
            out = c.full_attn_step(0, t, qp, k, v)
            rq, rg, rk, rv = oracle.attn_prologue(t, Hq, Hkv, d, d // 4, THETA, 1e-6, qn, kn, qp, k, v)
            if bf16:
                rk, rv = (oracle.bf16_to_f32(oracle.f32_to_bf16(a)) for a in (rk, rv))
            kc[t], vc[t] = rk, rv
            ref = oracle.sdpa(t + 1, Hq, Hkv, d, rq, rg, kc[:t + 1], vc[:t + 1])
            assert rel_err(out, ref) <= (2e-3 if bf16 else TOL_F32), t
        assert c.kv_len(0) == n


def test_prologue_errors(mfa):
    Hq, Hkv, d = 8, 2, 64
    from moeflux_amd import MfaError
    z = np.zeros(Hq * 2 * d, np.float32)
    kv = np.zeros(Hkv * d, np.float32)
    w = np.zeros(d, np.uint16)
    with _ctx(mfa, Hq, Hkv, d, 1) as c:
        with pytest.raises(MfaError):
            c.attn_prologue(0, 0, z, kv, kv)        # weights not set
        c.set_full_weights(0, w, w)
        with pytest.raises(MfaError):
            c.attn_prologue(0, -1, z, kv, kv)       # negative position (rope.rs:70-72)
        with pytest.raises(MfaError):
            c.set_rope(1.0e7, 7)                    # odd rotary_dim
        c.attn_prologue(0, 0, z, kv, kv)
        with pytest.raises(MfaError):
            c.attn_prologue(0, 1, z, kv, kv)        # cache full (full_attn_forward.rs:283-288)
        assert c.kv_len(0) == 1
