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


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("Hq,Hkv,d,L0,T", [(32, 2, 256, 0, 70), (8, 2, 64, 5, 3), (32, 4, 128, 100, 513), (16, 4, 64, 37, 1)])
def test_chunk_layer_step_equals_the_token_loop(mfa, oracle, bf16, Hq, Hkv, d, L0, T):
    """A chunk of T tokens through norms, rotation, append and causal attention in one call, after
    L0 tokens fed one by one: the same cache rows and, to the tolerance, the same outputs as the
    loop of single-token steps that eval_prompt runs (riir/mod.rs:1196-1214); and the oracle's
    composition for the chunk's last token."""
    rng, qn, kn = _case(T + L0, Hq, Hkv, d)
    n = L0 + T
    qp = rng.standard_normal((n, Hq * 2 * d)).astype(np.float32)
    k = rng.standard_normal((n, Hkv * d)).astype(np.float32)
    v = rng.standard_normal((n, Hkv * d)).astype(np.float32)
    with _ctx(mfa, Hq, Hkv, d, n + 1, bf16=bf16) as a, _ctx(mfa, Hq, Hkv, d, n + 1, bf16=bf16) as b:
        for c in (a, b):
            c.set_full_weights(0, qn, kn)
            for t in range(L0):
                c.full_attn_step(0, t, qp[t], k[t], v[t])
        loop = np.stack([a.full_attn_step(0, L0 + t, qp[L0 + t], k[L0 + t], v[L0 + t]) for t in range(T)])
        chunk = b.prefill_full_attn(0, L0, qp[L0:], k[L0:], v[L0:])
        assert a.kv_len(0) == b.kv_len(0) == n
        (ka, va), (kb, vb) = a.kv_export(0), b.kv_export(0)
        assert np.array_equal(ka, kb) and np.array_equal(va, vb)
        assert chunk.shape == loop.shape and rel_err(chunk, loop) <= (1e-4 if bf16 else TOL_F32)
        # a further single step continues from the chunk's cache as from the loop's
        x = rng.standard_normal(Hq * 2 * d).astype(np.float32)
        nk, nv = rng.standard_normal(Hkv * d).astype(np.float32), rng.standard_normal(Hkv * d).astype(np.float32)
        assert np.array_equal(a.full_attn_step(0, n, x, nk, nv), b.full_attn_step(0, n, x, nk, nv))
    rq, rg, _, _ = oracle.attn_prologue(n - 1, Hq, Hkv, d, d // 4, THETA, 1e-6, qn, kn, qp[-1], k[-1], v[-1])
    ref = oracle.sdpa(n, Hq, Hkv, d, rq, rg, ka, va)
    assert rel_err(chunk[-1], ref) <= (1e-4 if bf16 else TOL_F32)


def test_chunk_layer_step_errors_append_nothing(mfa):
    Hq, Hkv, d = 8, 2, 64
    from moeflux_amd import MfaError, ffi
    w = np.full(d, 0x3F80, np.uint16)
    qp, kv = np.ones((4, Hq * 2 * d), np.float32), np.ones((4, Hkv * d), np.float32)
    with _ctx(mfa, Hq, Hkv, d, 6) as c:
        with pytest.raises(MfaError):
            c.prefill_full_attn(0, 0, qp, kv, kv)         # weights not set
        c.set_full_weights(0, w, w)
        c.prefill_full_attn(0, 0, qp, kv, kv)
        with pytest.raises(MfaError) as e:
            c.prefill_full_attn(0, 4, qp, kv, kv)         # 4 + 4 > 6
        assert e.value.code == ffi.ERR_OVERFLOW and c.kv_len(0) == 4
        with pytest.raises(MfaError):
            c.prefill_full_attn(0, -1, qp[:1], kv[:1], kv[:1])
        assert c.kv_len(0) == 4
        c.prefill_full_attn(0, 4, qp[:2], kv[:2], kv[:2])
        assert c.kv_len(0) == 6


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


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("Hq,Hkv,d,L0", [(32, 2, 256, 0), (32, 2, 256, 1000), (32, 2, 256, 9000), (32, 4, 128, 4100),
                                         (8, 2, 64, 33), (16, 1, 128, 300), (4, 4, 64, 17), (40, 2, 64, 70)])
def test_two_launch_step_equals_three_launch_step(mfa, oracle, bf16, Hq, Hkv, d, L0):
    """A decode step whose attention launch norms and rotates its own query heads and whose merge
    takes the new token as one more split, against the prologue / attention / merge chain: the same
    cache rows bit for bit, the same outputs to the tolerance, and the oracle's composition
    (full_attn_forward.rs:234-389) for every step; from an empty cache, across a block edge, with
    16 and more than 16 query heads per kv head."""
    rng, qn, kn = _case(L0 + d + Hq, Hq, Hkv, d)
    steps = 3
    k0 = rng.standard_normal((L0, Hkv * d)).astype(np.float32)
    v0 = rng.standard_normal((L0, Hkv * d)).astype(np.float32)
    if bf16:
        k0, v0 = (oracle.bf16_to_f32(oracle.f32_to_bf16(a)) for a in (k0, v0))
    kc = np.concatenate([k0, np.zeros((steps, Hkv * d), np.float32)])
    vc = np.concatenate([v0, np.zeros((steps, Hkv * d), np.float32)])
    tol = 1e-4 if bf16 else TOL_F32
    with _ctx(mfa, Hq, Hkv, d, L0 + steps, bf16=bf16) as a, _ctx(mfa, Hq, Hkv, d, L0 + steps, bf16=bf16) as b:
        b.set_step_launches(3)
        for c in (a, b):
            c.set_full_weights(0, qn, kn)
            if L0:
                c.kv_import(0, k0, v0)
        for t in range(steps):
            pos = L0 + t
            qp = rng.standard_normal(Hq * 2 * d).astype(np.float32)
            k, v = rng.standard_normal(Hkv * d).astype(np.float32), rng.standard_normal(Hkv * d).astype(np.float32)
            o2, o3 = a.full_attn_step(0, pos, qp, k, v), b.full_attn_step(0, pos, qp, k, v)
            rq, rg, rk, rv = oracle.attn_prologue(pos, Hq, Hkv, d, d // 4, THETA, 1e-6, qn, kn, qp, k, v)
            if bf16:
                rk, rv = (oracle.bf16_to_f32(oracle.f32_to_bf16(x)) for x in (rk, rv))
            kc[pos], vc[pos] = rk, rv
            ref = oracle.sdpa(pos + 1, Hq, Hkv, d, rq, rg, kc[:pos + 1], vc[:pos + 1])
            assert rel_err(o2, o3) <= tol, (t, rel_err(o2, o3))
            assert rel_err(o2, ref) <= (2e-3 if bf16 else TOL_F32), (t, rel_err(o2, ref))
            heads = np.abs(o2.reshape(Hq, d) - ref.reshape(Hq, d)).max(axis=1) / np.abs(ref.reshape(Hq, d)).max(axis=1)
            assert heads.max() <= (4e-3 if bf16 else 2e-5), (t, heads.max())
        assert a.kv_len(0) == b.kv_len(0) == L0 + steps
        (ka, va), (kb, vb) = a.kv_export(0), b.kv_export(0)
        assert np.array_equal(ka, kb) and np.array_equal(va, vb)


@pytest.mark.parametrize("L0", [31, 32, 255, 256, 257, 2047, 2048, 2049, 8191, 8192, 8193])
def test_two_launch_step_at_the_edges_of_the_split_plan(mfa, oracle, L0):
    """The token rides in the last split's workgroup: lengths at which that split is full, holds one
    block, or holds a single position, either side of the lengths at which the plan changes."""
    Hq, Hkv, d, steps = 32, 2, 256, 2
    rng, qn, kn = _case(7 * L0 + 1, Hq, Hkv, d)
    k0 = oracle.bf16_to_f32(oracle.f32_to_bf16(rng.standard_normal((L0, Hkv * d)).astype(np.float32)))
    v0 = oracle.bf16_to_f32(oracle.f32_to_bf16(rng.standard_normal((L0, Hkv * d)).astype(np.float32)))
    kc = np.concatenate([k0, np.zeros((steps, Hkv * d), np.float32)])
    vc = np.concatenate([v0, np.zeros((steps, Hkv * d), np.float32)])
    with _ctx(mfa, Hq, Hkv, d, L0 + steps, bf16=True) as a, _ctx(mfa, Hq, Hkv, d, L0 + steps, bf16=True) as b:
        b.set_step_launches(3)
        for c in (a, b):
            c.set_full_weights(0, qn, kn)
            c.kv_import(0, k0, v0)
        for t in range(steps):
            pos = L0 + t
            qp = rng.standard_normal(Hq * 2 * d).astype(np.float32)
            k, v = rng.standard_normal(Hkv * d).astype(np.float32), rng.standard_normal(Hkv * d).astype(np.float32)
            o2, o3 = a.full_attn_step(0, pos, qp, k, v), b.full_attn_step(0, pos, qp, k, v)
            rq, rg, rk, rv = oracle.attn_prologue(pos, Hq, Hkv, d, d // 4, THETA, 1e-6, qn, kn, qp, k, v)
            kc[pos], vc[pos] = (oracle.bf16_to_f32(oracle.f32_to_bf16(x)) for x in (rk, rv))
            ref = oracle.sdpa(pos + 1, Hq, Hkv, d, rq, rg, kc[:pos + 1], vc[:pos + 1])
            assert rel_err(o2, o3) <= 1e-4, (t, rel_err(o2, o3))
            assert rel_err(o2, ref) <= 2e-3, (t, rel_err(o2, ref))
        (ka, va), (kb, vb) = a.kv_export(0), b.kv_export(0)
        assert np.array_equal(ka, kb) and np.array_equal(va, vb)


def test_two_launch_step_on_seeded_random_shapes(mfa, oracle):
    """Head counts, widths, cache kinds, lengths and forced split counts drawn at random (seeded):
    two launches against three and against the oracle's composition."""
    rng0 = np.random.default_rng(20240611)
    for case in range(14):
        d = int(rng0.choice([64, 128, 256]))
        Hkv = int(rng0.choice([1, 2, 4]))
        hpk = int(rng0.choice([1, 4, 8, 16, 20]))
        Hq = Hkv * hpk
        bf16 = bool(rng0.integers(0, 2))
        L0 = int(rng0.choice([0, 1, 15, 16, 17, 100, 513, 1999, 5000]))
        forced = int(rng0.choice([0, 0, 1, 2, 5, 37]))
        rng, qn, kn = _case(1000 + case, Hq, Hkv, d)
        k0 = rng.standard_normal((L0, Hkv * d)).astype(np.float32)
        v0 = rng.standard_normal((L0, Hkv * d)).astype(np.float32)
        if bf16:
            k0, v0 = (oracle.bf16_to_f32(oracle.f32_to_bf16(a)) for a in (k0, v0))
        kc = np.concatenate([k0, np.zeros((2, Hkv * d), np.float32)])
        vc = np.concatenate([v0, np.zeros((2, Hkv * d), np.float32)])
        tag = (case, Hq, Hkv, d, bf16, L0, forced)
        with _ctx(mfa, Hq, Hkv, d, L0 + 2, bf16=bf16) as a, _ctx(mfa, Hq, Hkv, d, L0 + 2, bf16=bf16) as b:
            b.set_step_launches(3)
            for c in (a, b):
                c.set_full_weights(0, qn, kn)
                if forced:
                    c.set_num_splits(forced)
                if L0:
                    c.kv_import(0, k0, v0)
            for t in range(2):
                pos = L0 + t
                qp = rng.standard_normal(Hq * 2 * d).astype(np.float32)
                k, v = rng.standard_normal(Hkv * d).astype(np.float32), rng.standard_normal(Hkv * d).astype(np.float32)
                o2, o3 = a.full_attn_step(0, pos, qp, k, v), b.full_attn_step(0, pos, qp, k, v)
                rq, rg, rk, rv = oracle.attn_prologue(pos, Hq, Hkv, d, d // 4, THETA, 1e-6, qn, kn, qp, k, v)
                if bf16:
                    rk, rv = (oracle.bf16_to_f32(oracle.f32_to_bf16(x)) for x in (rk, rv))
                kc[pos], vc[pos] = rk, rv
                ref = oracle.sdpa(pos + 1, Hq, Hkv, d, rq, rg, kc[:pos + 1], vc[:pos + 1])
                assert rel_err(o2, o3) <= (1e-4 if bf16 else TOL_F32), (tag, t, rel_err(o2, o3))
                assert rel_err(o2, ref) <= (2e-3 if bf16 else TOL_F32), (tag, t, rel_err(o2, ref))
            (ka, va), (kb, vb) = a.kv_export(0), b.kv_export(0)
            assert np.array_equal(ka, kb) and np.array_equal(va, vb), tag


def test_two_launch_step_with_forced_splits_and_errors(mfa, oracle):
    """The split count does not change the two-launch step's result beyond rounding, a full cache
    is refused before anything is appended, and weights must be set."""
    Hq, Hkv, d, L0 = 32, 2, 256, 700
    from moeflux_amd import MfaError, ffi
    rng, qn, kn = _case(3, Hq, Hkv, d)
    k0, v0 = rng.standard_normal((L0, Hkv * d)).astype(np.float32), rng.standard_normal((L0, Hkv * d)).astype(np.float32)
    qp = rng.standard_normal(Hq * 2 * d).astype(np.float32)
    k, v = rng.standard_normal(Hkv * d).astype(np.float32), rng.standard_normal(Hkv * d).astype(np.float32)
    outs = []
    for splits in (0, 1, 3, 44):
        with _ctx(mfa, Hq, Hkv, d, L0 + 1) as c:
            with pytest.raises(MfaError):
                c.full_attn_step(0, L0, qp, k, v)       # weights not set
            c.set_full_weights(0, qn, kn)
            c.kv_import(0, k0, v0)
            c.set_num_splits(splits)
            outs.append(c.full_attn_step(0, L0, qp, k, v))
            with pytest.raises(MfaError) as e:
                c.full_attn_step(0, L0 + 1, qp, k, v)   # the cache is full
            assert e.value.code == ffi.ERR_OVERFLOW and c.kv_len(0) == L0 + 1
    for o in outs[1:]:
        assert rel_err(o, outs[0]) <= TOL_F32
