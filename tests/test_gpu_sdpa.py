"""GPU parity of the full-attention path against the CPU oracle, through the C ABI."""
import numpy as np
import pytest

from tests.util import (TOL_BF16, TOL_F32, rel_err, rel_err_rows, sdpa_random_inputs, sdpa_reference_inputs, synth)

pytestmark = pytest.mark.gpu

# Per-head bounds (max|a-b| over one head / max|b| over the same head).  The oracle sums
# sequentially in f32: over L positions its own sums are about sqrt(L) * 6e-8 from exact, which is
# what these leave room for; the kernel's own error is a few 1e-7.
PER_HEAD_F32 = 3e-5     # up to a few thousand positions
PER_HEAD_LONG = 1e-4    # 32768 positions


@pytest.mark.parametrize("Hq,Hkv,d", [(32, 4, 128), (32, 2, 256), (16, 2, 256), (8, 8, 64), (40, 2, 128)])
@pytest.mark.parametrize("L", [1, 2, 7, 16, 33, 64, 257, 1000])
def test_sdpa_f32_matches_oracle(mfa, oracle, Hq, Hkv, d, L):
    q, g, k, v = sdpa_random_inputs(100 + L, Hq, Hkv, d, L)
    ref = oracle.sdpa(L, Hq, Hkv, d, q, g, k, v)
    out = mfa.sdpa_cpu(L, Hq, Hkv, d, q, g, k, v)
    assert rel_err(out, ref) <= TOL_F32


@pytest.mark.parametrize("Hq,Hkv,d", [(32, 2, 256), (32, 4, 128), (16, 2, 256), (4, 1, 64)])
@pytest.mark.parametrize("L", [1, 5, 31, 32, 33, 100, 1025])
def test_sdpa_bf16kv_matches_oracle(mfa, oracle, Hq, Hkv, d, L):
    q, g, k, v = sdpa_random_inputs(200 + L, Hq, Hkv, d, L, bf16=True)
    ref = oracle.sdpa(L, Hq, Hkv, d, q, g, k, v)
    out = mfa.sdpa_cpu(L, Hq, Hkv, d, q, g, k, v)
    # north-star tolerance for the bf16 cache is 1e-2; the hi/lo operand split
    # keeps the kernel at f32-level agreement, which is asserted as well
    assert rel_err(out, ref) <= TOL_BF16
    assert rel_err(out, ref) <= 1e-4


@pytest.mark.parametrize("kv_len", [1, 8, 64, 512])
def test_sdpa_reference_test_inputs(mfa, oracle, kv_len):
    """The reference's own sdpa inputs (tests/diff_oracle.rs:1541-1615), A17B shape."""
    Hq, Hkv, d = 32, 2, 256
    q, g, k, v = sdpa_reference_inputs(Hq, Hkv, d, kv_len)
    ref = oracle.sdpa(kv_len, Hq, Hkv, d, q, g, k, v)
    out = mfa.sdpa_cpu(kv_len, Hq, Hkv, d, q, g, k, v)
    assert rel_err(out, ref) <= TOL_F32


def test_sdpa_random_shapes_default_split_planning(mfa, oracle):
    """Seeded random shapes and lengths through the default split planning (whole passes per
    workgroup, two workgroups per CU up to head_dim 128): lengths around pass and block edges,
    every head_dim, f32 and bf16 caches."""
    rng = np.random.default_rng(2024)
    edges = [255, 256, 257, 2047, 2048, 2049, 4095, 4097, 6143, 6145, 8191, 8193, 12289, 16383, 16385, 20481]
    for case in range(28):
        d = int(rng.choice([64, 128, 256]))
        Hkv = int(rng.choice([1, 2, 4, 8]))
        hpk = int(rng.choice([1, 2, 5, 8, 16, 20]))
        Hq = Hkv * hpk
        L = int(rng.choice(edges)) if case % 2 == 0 else int(rng.integers(1, 9000))
        bf16 = bool(case % 3)
        q, g, k, v = sdpa_random_inputs(7000 + case, Hq, Hkv, d, L, bf16=bf16)
        ref = oracle.sdpa(L, Hq, Hkv, d, q, g, k, v)
        out = mfa.sdpa_cpu(L, Hq, Hkv, d, q, g, k, v)
        tol = 1e-4 if bf16 else TOL_F32
        assert rel_err(out, ref) <= tol, (case, d, Hq, Hkv, L, bf16, rel_err(out, ref))


def test_config1_full_size(mfa, oracle):
    """The 4K f32 decode shape: 32 Q / 4 KV heads, d=128, L=4096, fp32."""
    Hq, Hkv, d, L = 32, 4, 128, 4096
    q, g, k, v = sdpa_random_inputs(0xC0FFEE + 1, Hq, Hkv, d, L)
    ref = oracle.sdpa(L, Hq, Hkv, d, q, g, k, v)
    out = mfa.sdpa_cpu(L, Hq, Hkv, d, q, g, k, v)
    assert rel_err(out, ref) <= TOL_F32
    # every head against its own largest value (a head of small values cannot hide under a neighbour)
    assert rel_err_rows(out, ref, d) <= PER_HEAD_F32


@pytest.mark.parametrize("seq_len", [32, 64, 128, 512])
def test_attn_kernel_hooks(mfa, oracle, seq_len):
    """Per-kernel hooks with the reference's synthetic inputs (tests/diff_oracle.rs:2712-2955)."""
    Hq, Hkv, d = 32, 2, 256
    q = synth(11, Hq * d, 0.6)
    k = synth(22, seq_len * Hkv * d, 0.5)
    v = synth(33, seq_len * Hkv * d, 0.4)
    scale = 1.0 / np.sqrt(d)
    s_ref = oracle.attn_scores(Hq, Hkv, d, seq_len, q, k, scale)
    s = mfa.attn_scores_batched(Hq, Hkv, d, seq_len, q, k, scale)
    assert rel_err(s, s_ref) <= TOL_F32
    p_ref = oracle.attn_softmax(Hq, seq_len, s_ref)
    p = mfa.attn_softmax_batched(Hq, seq_len, s_ref)
    assert rel_err(p, p_ref) <= TOL_F32
    o_ref = oracle.attn_values(Hq, Hkv, d, seq_len, p_ref, v)
    o = mfa.attn_values_batched(Hq, Hkv, d, seq_len, p_ref, v)
    assert rel_err(o, o_ref) <= TOL_F32


def test_sigmoid_gate_hook(mfa, oracle):
    x, gate = synth(101, 32 * 256, 0.7), synth(202, 32 * 256, 1.2)
    assert rel_err(mfa.sigmoid_gate(gate, x), oracle.sigmoid_gate(gate, x)) <= 1e-6


def _ctx(mfa, **kw):
    from moeflux_amd import Config
    return mfa.Ctx(Config(**kw))


@pytest.mark.parametrize("bf16", [False, True])
def test_ctx_append_decode_and_split_invariance(mfa, oracle, bf16):
    """Token-by-token append + decode through a context, then the same query at
    split counts 1, 2, 7, 64 (tests/mla_sdpa_tiled.rs:176-216 is the precedent)."""
    Hq, Hkv, d, L = 32, 2, 256, 300
    q, g, k, v = sdpa_random_inputs(7, Hq, Hkv, d, L, bf16=bf16)
    kf = oracle.bf16_to_f32(k) if bf16 else k
    vf = oracle.bf16_to_f32(v) if bf16 else v
    with _ctx(mfa, num_layers=2, full_attn_interval=1, num_attn_heads=Hq, num_kv_heads=Hkv,
              head_dim=d, kv_capacity=512, kv_dtype=1 if bf16 else 0) as c:
        for p in range(L):
            c.kv_append(1, kf[p], vf[p])
            if p in (0, 1, 31, 32, 150, L - 1):
                ref = oracle.sdpa(p + 1, Hq, Hkv, d, q, g, k, v)
                assert rel_err(c.sdpa_decode(1, q, g), ref) <= (1e-4 if bf16 else TOL_F32)
        assert c.kv_len(1) == L and c.kv_len(0) == 0
        ref = oracle.sdpa(L, Hq, Hkv, d, q, g, k, v)
        outs = []
        for ns in (1, 2, 7, 64, 0):
            c.set_num_splits(ns)
            outs.append(c.sdpa_decode(1, q, g))
            assert rel_err(outs[-1], ref) <= (1e-4 if bf16 else TOL_F32)
        for o in outs[1:]:
            assert rel_err(o, outs[0]) <= 1e-5
        ke, ve = c.kv_export(1)
        assert np.array_equal(ke, kf) and np.array_equal(ve, vf)


@pytest.mark.parametrize("bf16", [False, True])
def test_merge_of_several_hundred_splits(mfa, oracle, bf16):
    """More splits than the 256 whose statistics the merge keeps in registers (the rest are read
    in loops), and more than the 128 whose rows a thread requests up front: forced split counts
    of 300, 512 and 1024 over a cache long enough to give every split a unit of the kernel's work
    (64 positions of an f32 cache, 128 of a bf16 cache at this head width, so the plans end at 625
    and 547 splits).  The oracle's sequential f32 sums over tens of thousands of positions are
    themselves 1e-5 from exact, so the kernel is also held to a float64 evaluation."""
    Hq, Hkv, d = 8, 1, 64
    L = 70000 if bf16 else 40000
    q, g, k, v = sdpa_random_inputs(71, Hq, Hkv, d, L, bf16=bf16)
    kf = oracle.bf16_to_f32(k) if bf16 else k
    vf = oracle.bf16_to_f32(v) if bf16 else v
    ref = oracle.sdpa(L, Hq, Hkv, d, q, g, k, v)
    s = q.reshape(Hq, d).astype(np.float64) @ kf.reshape(L, d).astype(np.float64).T / np.sqrt(d)
    w = np.exp(s - s.max(axis=1, keepdims=True))
    exact = ((w / w.sum(axis=1, keepdims=True)) @ vf.reshape(L, d).astype(np.float64)
             / (1.0 + np.exp(-g.reshape(Hq, d).astype(np.float64)))).reshape(-1)
    with _ctx(mfa, num_layers=1, full_attn_interval=1, num_attn_heads=Hq, num_kv_heads=Hkv,
              head_dim=d, kv_capacity=L, kv_dtype=1 if bf16 else 0) as c:
        c.kv_import(0, kf, vf)
        base = c.sdpa_decode(0, q, g)
        assert rel_err(base, exact) <= (1e-4 if bf16 else TOL_F32)
        assert rel_err(base, ref) <= (1e-4 if bf16 else TOL_F32 + rel_err(ref, exact))
        seen = set()
        for ns in (300, 512, 1024):
            c.set_num_splits(ns)
            seen.add(c.lib.mfa_debug_num_splits(1 if bf16 else 0, Hq, Hkv, d, L, 256, ns))
            out = c.sdpa_decode(0, q, g)
            assert rel_err(out, exact) <= (1e-4 if bf16 else TOL_F32), ns
            assert rel_err(out, base) <= 1e-5, ns
        assert max(seen) > 256


def test_config3_full_size_bf16(mfa, oracle):
    """The 32K bf16 decode shape (the headline workload): 32 Q / 2 KV heads, d=256, L=32768, bf16 K/V, via bulk import."""
    Hq, Hkv, d, L = 32, 2, 256, 32768
    q, g, k, v = sdpa_random_inputs(0xC0FFEE + 3, Hq, Hkv, d, L, bf16=True)
    ref = oracle.sdpa(L, Hq, Hkv, d, q, g, k, v)
    with _ctx(mfa, num_layers=1, full_attn_interval=1, num_attn_heads=Hq, num_kv_heads=Hkv,
              head_dim=d, kv_capacity=L, kv_dtype=1) as c:
        c.kv_import(0, k, v)
        out = c.sdpa_decode(0, q, g)
    assert rel_err(out, ref) <= TOL_BF16
    assert rel_err(out, ref) <= 1e-4
    assert rel_err_rows(out, ref, d) <= PER_HEAD_LONG


def test_cache_of_131072_positions_bf16(mfa, oracle):
    """Four times the 32K decode shape's length: 4096 blocks per kv head, 268 MB per layer, four passes
    per workgroup; the byte offsets of the last blocks pass 2^27."""
    Hq, Hkv, d, L = 32, 2, 256, 131072
    q, g, k, v = sdpa_random_inputs(0xC0FFEE + 13, Hq, Hkv, d, L, bf16=True)
    ref = oracle.sdpa(L, Hq, Hkv, d, q, g, k, v)
    with _ctx(mfa, num_layers=1, full_attn_interval=1, num_attn_heads=Hq, num_kv_heads=Hkv,
              head_dim=d, kv_capacity=L, kv_dtype=1) as c:
        c.kv_import(0, k, v)
        out = c.sdpa_decode(0, q, g)
    assert rel_err(out, ref) <= 1e-4


@pytest.mark.parametrize("Hq,Hkv,d,bf16", [(32, 2, 256, True), (32, 4, 128, True), (8, 2, 64, True), (8, 2, 64, False)])
def test_shares_of_a_single_unit(mfa, oracle, Hq, Hkv, d, bf16):
    """Where a ring of loads is more than one unit's K (these shapes), a share of one unit is streamed
    as one ring holding its K and its V: forced plans that give every workgroup exactly one unit, one
    unit or two, and a last unit that is only partly filled, against the oracle and against a single
    split."""
    unit = 128 if (bf16 and d == 64) else 64      # positions of a unit of the plan
    tol = 1e-4 if bf16 else 1e-5
    for L, splits in ((unit * 6, 6), (unit * 6 + 17, 7), (unit * 9, 6), (unit - 14, 1), (unit * 3 - 1, 64)):
        q, g, k, v = sdpa_random_inputs(L + splits, Hq, Hkv, d, L, bf16=bf16)
        kf = oracle.bf16_to_f32(k) if bf16 else k
        vf = oracle.bf16_to_f32(v) if bf16 else v
        ref = oracle.sdpa(L, Hq, Hkv, d, q, g, k, v)
        with _ctx(mfa, num_layers=1, full_attn_interval=1, num_attn_heads=Hq, num_kv_heads=Hkv, head_dim=d,
                  kv_capacity=L, kv_dtype=1 if bf16 else 0) as c:
            c.kv_import(0, kf, vf)
            c.set_num_splits(splits)
            out = c.sdpa_decode(0, q, g)
            c.set_num_splits(1)
            one = c.sdpa_decode(0, q, g)
        assert rel_err(out, ref) <= tol, (L, splits)
        assert rel_err(out, one) <= tol, (L, splits)
