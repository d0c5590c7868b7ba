"""GPU tests of the stateful surface: prompt chunks, the whole-stack sweep, and the
state operations (memory_clear / memory_seq_rm / pos_max, export / import), through
the C ABI, against the CPU oracle."""
import ctypes as C

import numpy as np
import pytest

from tests.util import TOL_F32, GdnCase, rel_err, rel_err_rows, sdpa_random_inputs

pytestmark = pytest.mark.gpu


def _full_ctx(mfa, Hq, Hkv, d, cap, bf16=False, layers=1):
    from moeflux_amd import Config
    return mfa.Ctx(Config(num_layers=layers, full_attn_interval=1, num_attn_heads=Hq,
                          num_kv_heads=Hkv, head_dim=d, kv_capacity=cap, kv_dtype=1 if bf16 else 0))


@pytest.mark.parametrize("T,L0", [(1, 0), (5, 0), (33, 0), (17, 40), (64, 31)])
def test_prefill_attn_equals_the_token_loop(mfa, oracle, T, L0):
    """A chunk of T tokens after L0 cached positions: row t is decode with kv_len = L0+t+1
    (riir/mod.rs:1196-1214)."""
    Hq, Hkv, d = 32, 4, 128
    rng = np.random.default_rng(T * 100 + L0)
    k = (rng.standard_normal((L0 + T, Hkv * d)) / np.sqrt(d)).astype(np.float32)
    v = (rng.standard_normal((L0 + T, Hkv * d)) / np.sqrt(d)).astype(np.float32)
    q = (rng.standard_normal((T, Hq * d)) / np.sqrt(d)).astype(np.float32)
    g = rng.standard_normal((T, Hq * d)).astype(np.float32)
    ref = oracle.prefill_attn(T, L0, Hq, Hkv, d, q, g, k, v).reshape(T, Hq * d)
    with _full_ctx(mfa, Hq, Hkv, d, 128) as c:
        if L0:
            c.kv_import(0, k[:L0], v[:L0])
        out = c.prefill_attn(0, q, g, k[L0:], v[L0:])
        assert c.kv_len(0) == L0 + T
        ke, ve = c.kv_export(0)
    assert rel_err(out, ref) <= TOL_F32
    for t in range(T):
        assert rel_err(out[t], ref[t]) <= 5e-5, t
    assert np.array_equal(ke, k) and np.array_equal(ve, v)


@pytest.mark.parametrize("bf16", [False, True])
def test_prefill_attn_few_tokens_after_a_long_cache(mfa, oracle, bf16):
    """A short chunk behind a long cache has too few rows to fill the machine, so the cache
    is split over workgroups (the decode kernel on 16-row groups of (token, head)) and
    merged; a ragged last row group (5 tokens x 4 heads = 20 rows) is part of the case."""
    Hq, Hkv, d, T, L0 = 8, 2, 128, 5, 3000
    rng = np.random.default_rng(31)
    k = (rng.standard_normal((L0 + T, Hkv * d)) / np.sqrt(d)).astype(np.float32)
    v = (rng.standard_normal((L0 + T, Hkv * d)) / np.sqrt(d)).astype(np.float32)
    if bf16:
        k, v = (oracle.bf16_to_f32(oracle.f32_to_bf16(a)) for a in (k, v))
    q = (rng.standard_normal((T, Hq * d)) / np.sqrt(d)).astype(np.float32)
    g = rng.standard_normal((T, Hq * d)).astype(np.float32)
    ref = oracle.prefill_attn(T, L0, Hq, Hkv, d, q, g, k, v).reshape(T, Hq * d)
    with _full_ctx(mfa, Hq, Hkv, d, 3072, bf16=bf16) as c:
        c.kv_import(0, k[:L0], v[:L0])
        out = c.prefill_attn(0, q, g, k[L0:], v[L0:])
    assert rel_err(out, ref) <= (1e-4 if bf16 else TOL_F32)


def test_prefill_attn_short_chunks_random_shapes(mfa, oracle):
    """Seeded random short chunks behind caches of random length: the split-K path with per-row
    causal limits under the default split planning, every head_dim, f32 and bf16 caches, ragged
    row groups."""
    rng = np.random.default_rng(77)
    for case in range(12):
        d = int(rng.choice([64, 128, 256]))
        Hkv = int(rng.choice([1, 2, 4]))
        Hq = Hkv * int(rng.choice([1, 3, 4, 8, 16]))
        T = int(rng.integers(2, 13))
        L0 = int(rng.choice([511, 2047, 2049, 4096, 6145])) if case % 2 else int(rng.integers(300, 9000))
        bf16 = bool(case % 3)
        k = (rng.standard_normal((L0 + T, Hkv * d)) / np.sqrt(d)).astype(np.float32)
        v = (rng.standard_normal((L0 + T, Hkv * d)) / np.sqrt(d)).astype(np.float32)
        if bf16:
            k, v = (oracle.bf16_to_f32(oracle.f32_to_bf16(a)) for a in (k, v))
        q = (rng.standard_normal((T, Hq * d)) / np.sqrt(d)).astype(np.float32)
        g = rng.standard_normal((T, Hq * d)).astype(np.float32)
        ref = oracle.prefill_attn(T, L0, Hq, Hkv, d, q, g, k, v).reshape(T, Hq * d)
        with _full_ctx(mfa, Hq, Hkv, d, L0 + T, bf16=bf16) as c:
            c.kv_import(0, k[:L0], v[:L0])
            out = c.prefill_attn(0, q, g, k[L0:], v[L0:])
        err = rel_err(out, ref)
        assert err <= (1e-4 if bf16 else TOL_F32), (case, d, Hq, Hkv, T, L0, bf16, err)


@pytest.mark.parametrize("Hq,Hkv,d,T,L0,bf16", [(32, 2, 256, 70, 100, True), (8, 2, 64, 200, 0, False),
                                                (32, 2, 256, 40, 9, False), (16, 4, 64, 130, 77, True),
                                                (32, 4, 128, 1100, 50, True), (32, 16, 64, 2100, 0, True),
                                                (32, 16, 64, 2050, 3, False), (4, 1, 64, 4200, 100, True),
                                                (2, 1, 128, 4100, 0, False)])
@pytest.mark.parametrize("q_exact", [False, True])
def test_prefill_attn_shapes(mfa, oracle, Hq, Hkv, d, T, L0, bf16, q_exact):
    """The chunk kernel (one wave per 16-row group, K/V blocks staged in LDS) over head
    dims, group sizes, ragged row counts and one or two row groups per wave; with a query that is
    exact in bf16 the waves of a bf16 cache take the path without the low parts' products."""
    if q_exact and not bf16:
        pytest.skip("an f32 cache has one path")
    rng = np.random.default_rng(T + L0)
    k = rng.standard_normal((L0 + T, Hkv * d)).astype(np.float32)
    v = rng.standard_normal((L0 + T, Hkv * d)).astype(np.float32)
    if bf16:
        k, v = (oracle.bf16_to_f32(oracle.f32_to_bf16(a)) for a in (k, v))
    q = (rng.standard_normal((T, Hq * d)) / np.sqrt(d)).astype(np.float32)
    if q_exact:
        q = oracle.bf16_to_f32(oracle.f32_to_bf16(q))
    g = rng.standard_normal((T, Hq * d)).astype(np.float32)
    ref = oracle.prefill_attn(T, L0, Hq, Hkv, d, q, g, k, v).reshape(T, Hq * d)
    with _full_ctx(mfa, Hq, Hkv, d, L0 + T, bf16=bf16) as c:
        if L0:
            c.kv_import(0, k[:L0], v[:L0])
        out = c.prefill_attn(0, q, g, k[L0:], v[L0:])
    assert rel_err(out, ref) <= (1e-4 if bf16 else TOL_F32)


def test_prefill_attn_bf16_chunk_of_512(mfa, oracle):
    """The attention half of the 512-token prompt chunk: 512 tokens, 32 Q / 4 KV heads, d=128, bf16 values,
    from an empty cache."""
    Hq, Hkv, d, T = 32, 4, 128, 512
    rng = np.random.default_rng(0xC0FFEE + 4)
    kb = oracle.f32_to_bf16(rng.standard_normal((T, Hkv * d)).astype(np.float32))
    vb = oracle.f32_to_bf16(rng.standard_normal((T, Hkv * d)).astype(np.float32))
    k, v = oracle.bf16_to_f32(kb), oracle.bf16_to_f32(vb)
    q = oracle.bf16_to_f32(oracle.f32_to_bf16((rng.standard_normal((T, Hq * d)) / np.sqrt(d)).astype(np.float32)))
    g = rng.standard_normal((T, Hq * d)).astype(np.float32)
    ref = oracle.prefill_attn(T, 0, Hq, Hkv, d, q, g, k, v).reshape(T, Hq * d)
    with _full_ctx(mfa, Hq, Hkv, d, 512, bf16=True) as c:
        out = c.prefill_attn(0, q, g, k, v)
    assert rel_err(out, ref) <= 1e-2      # the stated tolerance of the bf16 path
    assert rel_err(out, ref) <= 1e-4


@pytest.mark.parametrize("per_layer,ragged", [(0, False), (1, False), (0, True)])
def test_token_sweep_equals_independent_calls(mfa, oracle, per_layer, ragged):
    """One token's attention launches over a hybrid stack (every 4th layer full attention,
    variants.rs:258-264) equal the per-layer calls: launched once per layer kind, launched
    layer by layer, and with layers at different positions (kv lengths and conv ring slots
    differ, so the sweep has to fall back to the loop)."""
    from moeflux_amd import Config, ffi
    from moeflux_amd.hip import DeviceArray
    NL, Hq, Hkv, d, L = 8, 32, 2, 256, 200
    case = GdnCase(9, 16, 32, 128, 128)
    cfg = Config(num_layers=NL, full_attn_interval=4, num_attn_heads=Hq, num_kv_heads=Hkv, head_dim=d,
                 kv_capacity=256, kv_dtype=1)
    rng = np.random.default_rng(77)
    n_full, n_lin = 2, 6
    qs, gs, ks, vs = [], [], [], []
    with mfa.Ctx(cfg) as c:
        lib = c.lib
        for i in range(NL):
            if cfg.is_full(i):
                Li = L - 7 * len(qs) if ragged else L
                q, g, k, v = sdpa_random_inputs(300 + i, Hq, Hkv, d, Li, bf16=True)
                c.kv_import(i, k, v)
                qs.append(q); gs.append(g); ks.append(k); vs.append(v)
            else:
                c.set_linear_weights(i, case.conv_w, case.a_log, case.dt_bias, case.norm_w)
        lin_states = [((rng.standard_normal(3 * case.C)).astype(np.float32),
                       (rng.standard_normal(32 * 128 * 128) * 0.02).astype(np.float32)) for _ in range(n_lin)]
        lin_idx = [i for i in range(NL) if not cfg.is_full(i)]
        for (cs, ss), i in zip(lin_states, lin_idx):
            c.linear_state_import(i, cs, ss)
        x = rng.standard_normal((n_lin, case.C)).astype(np.float32)
        z = rng.standard_normal((n_lin, 32 * 128)).astype(np.float32)
        al = rng.standard_normal((n_lin, 32)).astype(np.float32)
        be = rng.standard_normal((n_lin, 32)).astype(np.float32)
        dq, dg = DeviceArray.from_host(np.array(qs)), DeviceArray.from_host(np.array(gs))
        dfo = DeviceArray((n_full, Hq * d), np.float32, zero=True)
        dx, dz, da, db = (DeviceArray.from_host(a) for a in (x, z, al, be))
        dlo = DeviceArray((n_lin, 32 * 128), np.float32, zero=True)
        assert lib.mfa_set_sweep_per_layer(c.h, per_layer) == 0
        if ragged:   # one extra token on the second linear layer: its ring slot differs
            x0 = rng.standard_normal(case.C).astype(np.float32)
            z0, a0, b0 = z[1] * 0.5, al[1] * 0.5, be[1] * 0.5
            c.gdn_step(lin_idx[1], x0, z0, a0, b0)
            _, rc0, rs0 = oracle.gdn_step(16, 32, 128, 128, 4, 1e-6, case.conv_w, case.a_log, case.dt_bias,
                                          case.norm_w, x0, z0, a0, b0, *lin_states[1])
            lin_states[1] = (rc0, rs0)
        rc = lib.mfa_token_sweep_dev(c.h, dq.ptr, dg.ptr, dfo.ptr, dx.ptr, dz.ptr, da.ptr, db.ptr, dlo.ptr)
        assert rc == 0, ffi.last_error()
        c.sync()
        fo, lo = dfo.to_host(), dlo.to_host()
        new_states = [c.linear_state_export(i) for i in lin_idx]
    for j in range(n_full):
        assert rel_err(fo[j], oracle.sdpa(len(ks[j]), Hq, Hkv, d, qs[j], gs[j], ks[j], vs[j])) <= 1e-4
    for j in range(n_lin):
        ro, rc_, rs = oracle.gdn_step(16, 32, 128, 128, 4, 1e-6, case.conv_w, case.a_log, case.dt_bias,
                                      case.norm_w, x[j], z[j], al[j], be[j], *lin_states[j])
        assert rel_err(lo[j], ro) <= TOL_F32
        assert np.array_equal(new_states[j][0].reshape(-1), rc_)
        assert rel_err(new_states[j][1], rs) <= TOL_F32


@pytest.mark.parametrize("forced", [0, 5])
def test_stale_workspace_contents_never_reach_a_result(mfa, oracle, forced):
    """A chunk whose first row group cannot see the cache's last split: 20 tokens of 32 Q / 2 KV
    heads behind 1020 f32 positions are 65 blocks in 5 splits of 16, and token 0's rows end in
    block 63, so their fifth split is empty and writes no partial rows.  The workspace is filled
    with NaN bit patterns first: the merge must give such a split the weight 0 without touching
    its rows.  Also with the split count forced."""
    Hq, Hkv, d, T, L0 = 32, 2, 256, 20, 1020
    rng = np.random.default_rng(1020)
    k = (rng.standard_normal((L0 + T, Hkv * d)) / np.sqrt(d)).astype(np.float32)
    v = (rng.standard_normal((L0 + T, Hkv * d)) / np.sqrt(d)).astype(np.float32)
    q = (rng.standard_normal((T, Hq * d)) / np.sqrt(d)).astype(np.float32)
    g = rng.standard_normal((T, Hq * d)).astype(np.float32)
    ref = oracle.prefill_attn(T, L0, Hq, Hkv, d, q, g, k, v).reshape(T, Hq * d)
    with _full_ctx(mfa, Hq, Hkv, d, L0 + T + 8) as c:
        c.kv_import(0, k[:L0], v[:L0])
        if forced:
            c.set_num_splits(forced)
        # a first call sizes the workspace for the chunk; the second runs over NaN
        out0 = c.prefill_attn(0, q, g, k[L0:], v[L0:])
        c.memory_seq_rm(L0)
        assert c.lib.mfa_debug_fill_workspace(c.h, 0x7FC00000) == 0
        out = c.prefill_attn(0, q, g, k[L0:], v[L0:])
    assert np.isfinite(out).all()
    assert np.array_equal(out, out0)
    assert rel_err(out, ref) <= TOL_F32
    assert rel_err_rows(out, ref, d) <= 3e-5


@pytest.mark.parametrize("per_layer", [0, 1])
def test_config5_full_size_sweep(mfa, oracle, per_layer):
    """The 48-layer hybrid stack at its own size: layers 3, 7, ..., 47 full attention
    (variants.rs:258-264) with 32 Q / 2 KV heads, head_dim 256 and 8192 cached bf16 positions
    each, the other 36 Gated-DeltaNet layers (16 / 32 heads, 128 x 128 states); distinct caches,
    states, weights and inputs per layer.  One token's attention (the layer loop of
    riir/mod.rs:1769-1888), launched once per layer kind and layer by layer: every layer's
    output, conv history (bit for bit) and recurrent state against the oracle."""
    from moeflux_amd import Config, ffi
    from moeflux_amd.hip import DeviceArray
    NL, Hq, Hkv, d, L = 48, 32, 2, 256, 8192
    Hk, Hv, dk, dv, K = 16, 32, 128, 128, 4
    cfg = Config(num_layers=NL, full_attn_interval=4, num_attn_heads=Hq, num_kv_heads=Hkv, head_dim=d,
                 kv_capacity=L, kv_dtype=1, linear_num_k_heads=Hk, linear_num_v_heads=Hv)
    full_idx = [i for i in range(NL) if cfg.is_full(i)]
    lin_idx = [i for i in range(NL) if not cfg.is_full(i)]
    assert full_idx == list(range(3, NL, 4)) and len(lin_idx) == 36
    rng = np.random.default_rng(0xC0FFEE + 5)
    fulls = [sdpa_random_inputs(500 + i, Hq, Hkv, d, L, bf16=True) for i in full_idx]
    cases = [GdnCase(600 + i, Hk, Hv, dk, dv) for i in lin_idx]
    with mfa.Ctx(cfg) as c:
        for i, (q, g, k, v) in zip(full_idx, fulls):
            c.kv_import(i, k, v)
        for i, cs in zip(lin_idx, cases):
            c.set_linear_weights(i, cs.conv_w, cs.a_log, cs.dt_bias, cs.norm_w)
            c.linear_state_import(i, cs.conv_state, cs.ssm_state)
        dq = DeviceArray.from_host(np.array([f[0] for f in fulls]))
        dg = DeviceArray.from_host(np.array([f[1] for f in fulls]))
        dfo = DeviceArray((len(fulls), Hq * d), np.float32, zero=True)
        dx = DeviceArray.from_host(np.array([cs.qkv[0] for cs in cases]))
        dz = DeviceArray.from_host(np.array([cs.z[0] for cs in cases]))
        da = DeviceArray.from_host(np.array([cs.alpha[0] for cs in cases]))
        db = DeviceArray.from_host(np.array([cs.beta[0] for cs in cases]))
        dlo = DeviceArray((len(cases), Hv * dv), np.float32, zero=True)
        assert c.lib.mfa_set_sweep_per_layer(c.h, per_layer) == 0
        assert c.lib.mfa_debug_fill_workspace(c.h, 0x7FC00000) == 0
        rc = c.lib.mfa_token_sweep_dev(c.h, dq.ptr, dg.ptr, dfo.ptr, dx.ptr, dz.ptr, da.ptr, db.ptr, dlo.ptr)
        assert rc == 0, ffi.last_error()
        c.sync()
        fo, lo = dfo.to_host(), dlo.to_host()
        states = [c.linear_state_export(i) for i in lin_idx]
    for j, (q, g, k, v) in enumerate(fulls):
        ref = oracle.sdpa(L, Hq, Hkv, d, q, g, k, v)
        assert rel_err(fo[j], ref) <= 1e-4, full_idx[j]
        assert rel_err_rows(fo[j], ref, d) <= 1e-4, full_idx[j]
    for j, cs in enumerate(cases):
        ro, rconv, rssm = cs.oracle()
        assert rel_err(lo[j], ro) <= TOL_F32, lin_idx[j]
        assert rel_err_rows(lo[j], ro, dv) <= 3e-5, lin_idx[j]
        assert np.array_equal(states[j][0].reshape(-1), rconv), lin_idx[j]
        assert rel_err(states[j][1], rssm) <= TOL_F32, lin_idx[j]


def test_state_operations_follow_the_reference(mfa, oracle):
    """memory_seq_rm keeps [0, p0) of every KV cache and zero-fills the rest, resets every
    DeltaNet layer (state.rs:431-455); memory_clear empties everything; pos_max is the
    largest KV length (state.rs:457-473)."""
    from moeflux_amd import Config
    Hq, Hkv, d = 8, 2, 64
    case = GdnCase(4, 2, 4, 64, 64)
    cfg = Config(num_layers=4, full_attn_interval=2, num_attn_heads=Hq, num_kv_heads=Hkv, head_dim=d,
                 kv_capacity=64, linear_num_k_heads=2, linear_num_v_heads=4, linear_key_dim=64,
                 linear_value_dim=64)
    q, g, k, v = sdpa_random_inputs(5, Hq, Hkv, d, 40)
    with mfa.Ctx(cfg) as c:
        assert c.memory_seq_pos_max() == 0
        for layer in (1, 3):
            c.kv_import(layer, k[:40 if layer == 1 else 25], v[:40 if layer == 1 else 25])
        for layer in (0, 2):
            c.set_linear_weights(layer, case.conv_w, case.a_log, case.dt_bias, case.norm_w)
            c.linear_state_import(layer, case.conv_state, case.ssm_state)
            c.gdn_step(layer, case.qkv[0], case.z[0], case.alpha[0], case.beta[0])
        assert c.memory_seq_pos_max() == 40
        c.memory_seq_rm(30, -1)
        assert c.kv_len(1) == 30 and c.kv_len(3) == 25 and c.memory_seq_pos_max() == 30
        assert rel_err(c.sdpa_decode(1, q, g), oracle.sdpa(30, Hq, Hkv, d, q, g, k, v)) <= TOL_F32
        for layer in (0, 2):
            cs, ss = c.linear_state_export(layer)
            assert not cs.any() and not ss.any()
        # the dropped rows are zero: re-append one row and export
        c.kv_append(1, k[30], v[30])
        ke, ve = c.kv_export(1)
        assert np.array_equal(ke, k[:31]) and np.array_equal(ve, v[:31])
        # a DeltaNet layer restarted from zero behaves like a fresh one
        o = c.gdn_step(0, case.qkv[0], case.z[0], case.alpha[0], case.beta[0])
        ro, _, _ = oracle.gdn_step(2, 4, 64, 64, 4, 1e-6, case.conv_w, case.a_log, case.dt_bias, case.norm_w,
                                   case.qkv[0], case.z[0], case.alpha[0], case.beta[0],
                                   np.zeros_like(case.conv_state), np.zeros_like(case.ssm_state))
        assert rel_err(o, ro) <= TOL_F32
        c.memory_seq_rm(100, -1)          # past the end: no-op for KV, DeltaNet still reset
        assert c.kv_len(1) == 31
        c.memory_clear()
        assert c.memory_seq_pos_max() == 0 and c.kv_len(1) == 0 and c.kv_len(3) == 0


def test_error_paths_leave_the_context_usable(mfa, oracle):
    from moeflux_amd import Config, MfaError, ffi
    Hq, Hkv, d = 8, 2, 64
    cfg = Config(num_layers=2, full_attn_interval=2, num_attn_heads=Hq, num_kv_heads=Hkv, head_dim=d,
                 kv_capacity=3, linear_num_k_heads=2, linear_num_v_heads=4, linear_key_dim=64,
                 linear_value_dim=64)
    q, g, k, v = sdpa_random_inputs(6, Hq, Hkv, d, 4)
    with mfa.Ctx(cfg) as c:
        with pytest.raises(MfaError) as e:
            c.sdpa_decode(1, q, g)                       # empty cache: kv_len <= 0 (sdpa.rs:71)
        assert e.value.code == ffi.ERR_INVALID
        with pytest.raises(MfaError) as e:
            c.sdpa_decode(0, q, g)                       # layer 0 is a DeltaNet layer
        assert e.value.code == ffi.ERR_LAYER
        with pytest.raises(MfaError) as e:
            c.kv_len(7)
        assert e.value.code == ffi.ERR_LAYER
        for p in range(3):
            c.kv_append(1, k[p], v[p])
        with pytest.raises(MfaError) as e:
            c.kv_append(1, k[3], v[3])                   # overflow (full_attn_forward.rs:283-288)
        assert e.value.code == ffi.ERR_OVERFLOW
        case = GdnCase(4, 2, 4, 64, 64)
        with pytest.raises(MfaError) as e:
            c.gdn_step(0, case.qkv[0], case.z[0], case.alpha[0], case.beta[0])   # weights not set
        assert e.value.code == ffi.ERR_INVALID
        assert c.lib.mfa_sdpa_decode(c.h, 1, None, None, None) == ffi.ERR_INVALID
        # still works after all of that
        assert rel_err(c.sdpa_decode(1, q, g), oracle.sdpa(3, Hq, Hkv, d, q, g, k, v)) <= TOL_F32


@pytest.mark.parametrize("L0", [0, 1000])
def test_prefill_attn_query_exact_in_bf16_skips_nothing_that_counts(mfa, oracle, L0):
    """The chunk kernel leaves out the products of the query's low bf16 parts in a wave all of whose
    rows are exact in bf16.  One element of one row made inexact sends that row's wave down the
    general path: every other row, those of the same wave included, must come out bit for bit as in
    the run where the whole query is exact; both runs agree with the oracle."""
    Hq, Hkv, d, T = 32, 4, 128, 256
    rng = np.random.default_rng(77 + L0)
    k = oracle.bf16_to_f32(oracle.f32_to_bf16(rng.standard_normal((L0 + T, Hkv * d)).astype(np.float32)))
    v = oracle.bf16_to_f32(oracle.f32_to_bf16(rng.standard_normal((L0 + T, Hkv * d)).astype(np.float32)))
    q = oracle.bf16_to_f32(oracle.f32_to_bf16((rng.standard_normal((T, Hq * d)) / np.sqrt(d)).astype(np.float32)))
    g = rng.standard_normal((T, Hq * d)).astype(np.float32)
    q2 = q.copy()
    tok, head = 100, 3
    q2[tok, head * d + 5] *= np.float32(1 + 2.0 ** -12)      # no longer a bf16 value
    assert not np.array_equal(oracle.bf16_to_f32(oracle.f32_to_bf16(q2)), q2)
    outs = []
    for qq in (q, q2):
        ref = oracle.prefill_attn(T, L0, Hq, Hkv, d, qq, g, k, v).reshape(T, Hq * d)
        with _full_ctx(mfa, Hq, Hkv, d, L0 + T, bf16=True) as c:
            if L0:
                c.kv_import(0, k[:L0], v[:L0])
            outs.append(c.prefill_attn(0, qq, g, k[L0:], v[L0:]))
        assert rel_err(outs[-1], ref) <= 1e-4
    a, b = (o.reshape(T, Hq, d) for o in outs)
    same = np.ones((T, Hq), bool)
    same[tok, head] = False
    assert np.array_equal(a[same], b[same])
    assert not np.array_equal(a[tok, head], b[tok, head])
