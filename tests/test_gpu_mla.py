"""GPU parity of attention over a latent cache (the folded form of multi-head latent
attention) against the CPU oracle, through the C ABI."""
import ctypes as C

import numpy as np
import pytest

from tests.util import TOL_F32, rel_err

pytestmark = pytest.mark.gpu

R, P = 512, 64


def _random(seed, H, L, spread=1.0):
    rng = np.random.default_rng(seed)
    return (rng.standard_normal((H, R)).astype(np.float32) * 0.1 * spread,
            rng.standard_normal((H, P)).astype(np.float32) * 0.1 * spread,
            rng.standard_normal((L, R)).astype(np.float32), rng.standard_normal((L, P)).astype(np.float32))


def _pattern(H, L):
    """tests/mla_sdpa_tiled.rs:84-116: the reference's deterministic test inputs."""
    i = lambda n: np.arange(n, dtype=np.float32)
    return (np.sin(i(H * R) * np.float32(0.0007)).astype(np.float32) * np.float32(0.1),
            np.sin(i(H * P) * np.float32(0.0011)).astype(np.float32) * np.float32(0.1),
            np.sin(i(L * R) * np.float32(0.00013)).astype(np.float32) * np.float32(0.05),
            np.sin(i(L * P) * np.float32(0.00017)).astype(np.float32) * np.float32(0.05))


@pytest.mark.parametrize("H,L", [(1, 1), (16, 15), (16, 16), (20, 17), (64, 100), (128, 1000), (5, 4097), (128, 2500),
                                 (72, 333)])
def test_mla_matches_oracle(mfa, oracle, H, L):
    """Head counts that do not fill a 16-head group or a 64-head workgroup, cache lengths
    around the 16-position block and the split boundaries."""
    qp, qe, lat, rk = _random(H * 7 + L, H, L)
    scale = 1.0 / np.sqrt(192.0)
    ref = oracle.mla_sdpa_folded(H, R, P, L, scale, qp, qe, lat, rk)
    out = mfa.mla_sdpa_folded(H, R, P, L, scale, qp, qe, lat, rk)
    assert rel_err(out, ref) <= TOL_F32


def test_mla_peaked_weights(mfa, oracle):
    """Large queries: scores of tens of units, a softmax close to one-hot, a running maximum
    that moves by tens of units between blocks.  The kernel forms every product from bf16
    parts (x = hi + lo to 2^-18 x, three partial products), so a score of magnitude |s|
    carries an error of about 1e-5 |s|, which the exponential turns into that relative
    error of a weight: at |s| ~ 10 the bar for this case is 1e-4, not 1e-5."""
    H, L = 32, 700
    qp, qe, lat, rk = _random(9, H, L, spread=12.0)
    ref = oracle.mla_sdpa_folded(H, R, P, L, 0.3, qp, qe, lat, rk)
    out = mfa.mla_sdpa_folded(H, R, P, L, 0.3, qp, qe, lat, rk)
    assert np.all(np.isfinite(out))
    assert rel_err(out, ref) <= 1e-4


@pytest.mark.parametrize("L", [4096, 8192, 16384])
def test_mla_reference_test_inputs(mfa, oracle, L):
    """tests/mla_sdpa_tiled.rs:143-185 (its cache lengths, 128 heads, its bar of cosine
    similarity >= 0.9999 between the single-pass and the tiled kernel) with the oracle as
    the single-pass side, and this build's own tolerance on top."""
    H = 128
    qp, qe, lat, rk = _pattern(H, L)
    scale = np.float32(1.0 / np.sqrt(128.0 + 64.0))
    ref = oracle.mla_sdpa_folded(H, R, P, L, scale, qp, qe, lat, rk)
    out = mfa.mla_sdpa_folded(H, R, P, L, scale, qp, qe, lat, rk)
    cos = float(np.dot(out.astype(np.float64), ref.astype(np.float64)) /
                (np.linalg.norm(out.astype(np.float64)) * np.linalg.norm(ref.astype(np.float64))))
    assert cos >= 0.9999
    assert rel_err(out, ref) <= TOL_F32


def test_mla_device_entry_reuses_the_workspace(mfa, oracle):
    """The device entry on the context's stream: a long cache, then a short one (fewer
    splits, same workspace), then the long one again."""
    from moeflux_amd import Config, ffi
    from moeflux_amd.hip import DeviceArray
    H = 128
    with mfa.Ctx(Config(num_layers=1, full_attn_interval=1, num_attn_heads=8, num_kv_heads=2, head_dim=64,
                        kv_capacity=4)) as c:
        for L in (3000, 40, 3000):
            qp, qe, lat, rk = _random(L, H, L)
            d = [DeviceArray.from_host(a) for a in (qp, qe, lat, rk)]
            do = DeviceArray((H * R,), np.float32, zero=True)
            rc = c.lib.mfa_mla_sdpa_folded_dev(c.h, H, R, P, L, C.c_float(0.07), d[0].ptr, d[1].ptr, d[2].ptr,
                                               d[3].ptr, do.ptr)
            assert rc == 0, ffi.last_error()
            c.sync()
            assert rel_err(do.to_host(), oracle.mla_sdpa_folded(H, R, P, L, 0.07, qp, qe, lat, rk)) <= TOL_F32


def test_mla_split_count_invariance(mfa, oracle):
    """tests/mla_sdpa_tiled.rs:143-185 compares the tiled kernel with the single-pass one; here the
    number of partitions of the cache is forced to 1, 3, 16 and 64 and every result is held to
    the oracle."""
    from moeflux_amd import Config, ffi
    from moeflux_amd.hip import DeviceArray
    H, L = 48, 1500
    qp, qe, lat, rk = _random(21, H, L)
    ref = oracle.mla_sdpa_folded(H, R, P, L, 0.09, qp, qe, lat, rk)
    d = [DeviceArray.from_host(a) for a in (qp, qe, lat, rk)]
    do = DeviceArray((H * R,), np.float32, zero=True)
    with mfa.Ctx(Config(num_layers=1, full_attn_interval=1, num_attn_heads=8, num_kv_heads=2, head_dim=64,
                        kv_capacity=4)) as c:
        for splits in (1, 3, 16, 64):
            assert c.lib.mfa_set_num_splits(c.h, splits) == 0
            rc = c.lib.mfa_mla_sdpa_folded_dev(c.h, H, R, P, L, C.c_float(0.09), d[0].ptr, d[1].ptr, d[2].ptr,
                                               d[3].ptr, do.ptr)
            assert rc == 0, ffi.last_error()
            c.sync()
            assert rel_err(do.to_host(), ref) <= TOL_F32, splits


def test_mla_size_independent_properties(mfa):
    """At the full length (32768 positions, 128 heads), where the oracle would take minutes:
    a zero query gives the mean latent row; equal latent rows come back whatever the weights;
    a cache made of two copies of a shorter one gives the shorter one's result."""
    H, L = 128, 32768
    qp, qe, lat, rk = _random(3, H, L)
    z = mfa.mla_sdpa_folded(H, R, P, L, 0.07, qp * 0, qe * 0, lat, rk).reshape(H, R)
    mean = lat.astype(np.float64).mean(axis=0)
    assert np.max(np.abs(z - mean)) <= 1e-6
    same = np.broadcast_to(lat[0], (L, R)).copy()
    s = mfa.mla_sdpa_folded(H, R, P, L, 0.07, qp, qe, same, rk).reshape(H, R)
    assert np.max(np.abs(s - lat[0])) <= 1e-5 * np.max(np.abs(lat[0]))
    half = mfa.mla_sdpa_folded(H, R, P, L // 2, 0.07, qp, qe, lat[:L // 2], rk[:L // 2])
    twice = mfa.mla_sdpa_folded(H, R, P, L, 0.07, qp, qe, np.concatenate([lat[:L // 2]] * 2),
                                np.concatenate([rk[:L // 2]] * 2))
    assert rel_err(twice, half) <= TOL_F32


def test_mla_errors(mfa):
    from moeflux_amd import ffi
    lib = ffi.load()
    a = np.zeros(1024, np.float32)
    p = a.ctypes.data_as(C.c_void_p)
    f = lambda H, r, pe, L: lib.mfa_mla_sdpa_folded(H, r, pe, L, C.c_float(1.0), p, p, p, p, p)
    assert f(1, 512, 64, 0) == ffi.ERR_INVALID
    assert f(0, 512, 64, 1) == ffi.ERR_INVALID
    assert f(1, 256, 64, 1) == ffi.ERR_SHAPE
    assert lib.mfa_mla_sdpa_folded(1, 512, 64, 1, C.c_float(1.0), None, p, p, p, p) == ffi.ERR_INVALID
