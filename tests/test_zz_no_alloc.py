"""The decode entry point that allocates nothing (mfa_sdpa_decode_static_dev): its split-K
partials live in a file-scope device array of the library.  Through the C ABI, against
mfa_sdpa_decode_dev on the same inputs: bit-identical, on two calls in a row, the second over a
shorter cache (the array keeps the first call's partials), and a plan too large for the array is
refused with nothing launched."""
import numpy as np
import pytest

from tests.util import rel_err, sdpa_random_inputs

pytestmark = pytest.mark.gpu


def _decode_both_ways(c, layer, q, g):
    from moeflux_amd import ffi
    from moeflux_amd.hip import DeviceArray
    dq, dg = DeviceArray.from_host(q), DeviceArray.from_host(g)
    outs = []
    for fn in (c.lib.mfa_sdpa_decode_dev, c.lib.mfa_sdpa_decode_static_dev):
        do = DeviceArray.from_host(np.full(q.shape, np.nan, np.float32))
        rc = fn(c.h, layer, dq.ptr, dg.ptr, do.ptr)
        assert rc == 0, ffi.last_error()
        c.sync()
        outs.append(do.to_host())
    return outs


@pytest.mark.parametrize("bf16", [True, False])
def test_static_scratch_decode_equals_the_workspace_decode(mfa, oracle, bf16):
    from moeflux_amd import Config
    Hq, Hkv, d = 32, 2, 256
    L_long, L_short = 5000, 700
    cfg = Config(num_layers=2, full_attn_interval=1, num_attn_heads=Hq, num_kv_heads=Hkv, head_dim=d,
                 kv_capacity=L_long, kv_dtype=1 if bf16 else 0)
    a = sdpa_random_inputs(41, Hq, Hkv, d, L_long, bf16=bf16)
    b = sdpa_random_inputs(42, Hq, Hkv, d, L_short, bf16=bf16)
    with mfa.Ctx(cfg) as c:
        for layer, (q, g, k, v) in enumerate((a, b)):
            c.kv_import(layer, oracle.bf16_to_f32(k) if bf16 else k, oracle.bf16_to_f32(v) if bf16 else v)
        # two calls in a row, the second with the smaller input
        for layer, (q, g, k, v), L in ((0, a, L_long), (1, b, L_short)):
            ws, st = _decode_both_ways(c, layer, q, g)
            assert np.array_equal(ws, st), layer
            assert rel_err(st, oracle.sdpa(L, Hq, Hkv, d, q, g, k, v)) <= (1e-4 if bf16 else 1e-5)
        # and with a forced split count (an empty tail split among them)
        c.set_num_splits(7)
        ws, st = _decode_both_ways(c, 1, b[0], b[1])
        assert np.array_equal(ws, st)


def test_static_scratch_decode_leaves_the_free_device_memory_as_it_was(mfa):
    """What the entry point is for: no allocation.  Free device memory (hipMemGetInfo) is read before
    and after calls over cache lengths that change the split plan from 1 workgroup per row group to
    128 and back; not a byte may have moved, where the same sweep through a fresh context's first
    ordinary decode may grow its workspace."""
    from moeflux_amd import Config, ffi
    from moeflux_amd.hip import DeviceArray, mem_free
    Hq, Hkv, d, L = 32, 2, 256, 33000
    cfg = Config(num_layers=1, full_attn_interval=1, num_attn_heads=Hq, num_kv_heads=Hkv, head_dim=d,
                 kv_capacity=L, kv_dtype=1)
    rng = np.random.default_rng(8)
    k = rng.standard_normal((L, Hkv * d), dtype=np.float32)
    q = rng.standard_normal(Hq * d, dtype=np.float32)
    with mfa.Ctx(cfg) as c:
        c.kv_import(0, k, k[::-1].copy())
        dq = DeviceArray.from_host(q)
        do = DeviceArray.from_host(np.zeros(q.shape, np.float32))
        c.sync()
        plans = set()
        free0 = mem_free()
        for n in (33000, 8192, 700, 64, 1):
            c.memory_seq_rm(n)
            assert c.kv_len(0) == n
            plans.add(c.lib.mfa_debug_num_splits(1, Hq, Hkv, d, n, 256, 0))
            assert c.lib.mfa_sdpa_decode_static_dev(c.h, 0, dq.ptr, dq.ptr, do.ptr) == 0, ffi.last_error()
            c.sync()
            assert mem_free() == free0, n
        assert len(plans) >= 3 and max(plans) >= 64 and min(plans) == 1
        assert np.isfinite(do.to_host()).all()


def test_static_scratch_refuses_a_plan_that_does_not_fit(mfa):
    """The automatic split plans stay within the array (a partial per workgroup, one or two
    workgroups per CU); a forced count of 375 splits of 2 kv heads (the cache is long enough to give
    each 64 positions) is 12 MiB of partial rows and is refused with nothing launched."""
    from moeflux_amd import Config, ffi
    from moeflux_amd.hip import DeviceArray
    Hq, Hkv, d, L = 32, 2, 256, 24000
    cfg = Config(num_layers=1, full_attn_interval=1, num_attn_heads=Hq, num_kv_heads=Hkv, head_dim=d,
                 kv_capacity=L, kv_dtype=0)
    rng = np.random.default_rng(3)
    k = rng.standard_normal((L, Hkv * d), dtype=np.float32)
    with mfa.Ctx(cfg) as c:
        c.kv_import(0, k, k)
        q = rng.standard_normal(Hq * d, dtype=np.float32)
        dq = DeviceArray.from_host(q)
        do = DeviceArray.from_host(np.full(q.shape, 7.0, np.float32))
        c.set_num_splits(375)
        assert c.lib.mfa_debug_num_splits(0, Hq, Hkv, d, L, 256, 375) * Hkv * 16 * d * 4 > 8 << 20
        assert c.lib.mfa_sdpa_decode_static_dev(c.h, 0, dq.ptr, dq.ptr, do.ptr) == ffi.ERR_INVALID
        assert "static scratch" in ffi.last_error()
        c.sync()
        assert (do.to_host() == 7.0).all()          # nothing was launched
        ref = DeviceArray.from_host(np.zeros(q.shape, np.float32))
        assert c.lib.mfa_sdpa_decode_dev(c.h, 0, dq.ptr, dq.ptr, ref.ptr) == 0   # the context is still usable
        c.set_num_splits(0)
        assert c.lib.mfa_sdpa_decode_static_dev(c.h, 0, dq.ptr, dq.ptr, do.ptr) == 0
        c.sync()
        assert rel_err(do.to_host(), ref.to_host()) <= 1e-5
