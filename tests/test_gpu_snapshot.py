"""The context's state in the reference's 'MFLX' snapshot wire format
(crates/moeflux/src/riir/state_snapshot.rs:1-73), through the C ABI."""
import struct

import numpy as np
import pytest

from tests.util import GdnCase, sdpa_random_inputs

pytestmark = pytest.mark.gpu

Hq, Hkv, D = 8, 2, 64
MAGIC = 0x4D464C58


def _cfg(bf16=False, cap=64):
    from moeflux_amd import Config
    return Config(num_layers=4, full_attn_interval=2, num_attn_heads=Hq, num_kv_heads=Hkv, head_dim=D,
                  kv_capacity=cap, kv_dtype=1 if bf16 else 0, linear_num_k_heads=2, linear_num_v_heads=4,
                  linear_key_dim=64, linear_value_dim=64)


def _fill(c, case, oracle, bf16):
    """Layers 0, 2 linear (some steps), layers 1, 3 full attention (17 and 40 rows)."""
    rows = {}
    for layer, n in ((1, 17), (3, 40)):
        _, _, k, v = sdpa_random_inputs(layer, Hq, Hkv, D, n, bf16=bf16)
        c.kv_import(layer, k, v)
        rows[layer] = (oracle.bf16_to_f32(k), oracle.bf16_to_f32(v)) if bf16 else (k, v)
    for layer in (0, 2):
        c.set_linear_weights(layer, case.conv_w, case.a_log, case.dt_bias, case.norm_w)
        c.linear_state_import(layer, case.conv_state * (layer + 1), case.ssm_state)
        for t in range(layer + 1):
            c.gdn_step(layer, case.qkv[t], case.z[t], case.alpha[t], case.beta[t])
    return rows


@pytest.mark.parametrize("bf16", [False, True])
def test_snapshot_layout_and_round_trip(mfa, oracle, bf16):
    case = GdnCase(3, 2, 4, 64, 64, T=4)
    cfg = _cfg(bf16)
    conv_b, ssm_b, row_b = 3 * case.C * 4, 4 * 64 * 64 * 4, Hkv * D * 4
    with mfa.Ctx(cfg) as c:
        rows = _fill(c, case, oracle, bf16)
        blob = c.state_save()
        assert len(blob) == c.state_size() == 40 + 2 * (conv_b + ssm_b) + 2 * 4 + 2 * (17 + 40) * row_b
        # header, field by field (state_snapshot.rs:6-16, 236-247)
        assert struct.unpack("<10I", blob[:40]) == (MAGIC, 2, 4, 2, Hkv, D, conv_b, ssm_b, 0, 0)
        # body, rebuilt from the per-layer exports in layer order (state_snapshot.rs:17-22)
        want = bytearray(blob[:40])
        for layer in range(4):
            if cfg.is_full(layer):
                k, v = c.kv_export(layer)
                want += struct.pack("<i", k.shape[0]) + k.tobytes() + v.tobytes()
                assert np.array_equal(k, rows[layer][0]) and np.array_equal(v, rows[layer][1])
            else:
                cs, ss = c.linear_state_export(layer)
                want += cs.astype("<f4").tobytes() + ss.astype("<f4").tobytes()
        assert bytes(want) == blob
        q, g, _, _ = sdpa_random_inputs(9, Hq, Hkv, D, 1)
        x = GdnCase(11, 2, 4, 64, 64, T=1)
        ref_a = c.sdpa_decode(3, q, g)
        ref_l = c.gdn_step(2, x.qkv[0], x.z[0], x.alpha[0], x.beta[0])
    # a fresh context continues exactly where the saved one stood
    with mfa.Ctx(cfg) as c2:
        for layer in (0, 2):
            c2.set_linear_weights(layer, case.conv_w, case.a_log, case.dt_bias, case.norm_w)
        c2.state_load(blob)
        assert c2.kv_len(1) == 17 and c2.kv_len(3) == 40 and c2.memory_seq_pos_max() == 40
        assert c2.state_save() == blob
        assert np.array_equal(c2.sdpa_decode(3, q, g), ref_a)
        assert np.array_equal(c2.gdn_step(2, x.qkv[0], x.z[0], x.alpha[0], x.beta[0]), ref_l)
        # version 1: the first eight header words only (state_snapshot.rs:64-73, 383-390)
        v1 = struct.pack("<8I", MAGIC, 1, 4, 2, Hkv, D, conv_b, ssm_b) + blob[40:]
        c2.memory_clear()
        c2.state_load(v1)
        assert c2.state_save() == blob


def test_snapshot_through_a_page_locked_buffer_and_with_an_empty_cache(mfa, oracle):
    """mfa_host_alloc gives the buffer the copies run fastest with; the bytes are those of a save
    into ordinary memory.  One full-attention layer holds no positions: its record is the length
    word alone, and loading it empties that layer's cache."""
    import ctypes as C
    from moeflux_amd import ffi
    lib = ffi.load()
    case = GdnCase(3, 2, 4, 64, 64, T=4)
    cfg = _cfg(True)
    with mfa.Ctx(cfg) as c:
        _fill(c, case, oracle, True)
        c.kv_import(1, np.zeros((0, Hkv * D), np.float32), np.zeros((0, Hkv * D), np.float32))
        assert c.kv_len(1) == 0 and c.kv_len(3) == 40
        blob = c.state_save()
        size = c.state_size()
        assert size == len(blob)
        pin = lib.mfa_host_alloc(size)
        assert pin
        try:
            assert lib.mfa_state_save(c.h, pin, size) == size
            assert C.string_at(pin, size) == blob
            c.memory_clear()
            assert lib.mfa_state_load(c.h, pin, size) == 0
            assert c.kv_len(1) == 0 and c.kv_len(3) == 40
            assert c.state_save() == blob
        finally:
            lib.mfa_host_free(pin)
        assert lib.mfa_host_alloc(0) is None and lib.mfa_host_alloc(-5) is None
        lib.mfa_host_free(None)


def test_snapshot_rejections_leave_the_context_untouched(mfa, oracle):
    from moeflux_amd import MfaError
    case = GdnCase(3, 2, 4, 64, 64, T=4)
    with mfa.Ctx(_cfg()) as c:
        _fill(c, case, oracle, False)
        blob = c.state_save()

        def patched(off, fmt, val):
            b = bytearray(blob)
            b[off:off + struct.calcsize(fmt)] = struct.pack(fmt, val)
            return bytes(b)

        first_len_off = 40 + 3 * case.C * 4 + 4 * 64 * 64 * 4   # layer 1's `i32 len`
        assert struct.unpack("<i", blob[first_len_off:first_len_off + 4])[0] == 17
        bad = {
            "magic": patched(0, "<I", 0x4D464C59),
            "version": patched(4, "<I", 3),
            "num_layers": patched(8, "<I", 5),
            "head_dim": patched(20, "<I", 128),
            "conv bytes": patched(24, "<I", 1),
            "truncated body": blob[:-5],
            "truncated header": blob[:20],
            "negative len": patched(first_len_off, "<i", -1),
            "len beyond capacity": patched(first_len_off, "<i", 65),
        }
        c.memory_seq_rm(10)           # so that a successful (wrong) load would be visible
        before = c.state_save()
        for name, b in bad.items():
            with pytest.raises(MfaError):
                c.state_load(b)
            assert c.state_save() == before, name
        c.state_load(blob)
        assert c.state_save() == blob


def test_snapshot_larger_than_the_staging_buffer(mfa, oracle):
    """The device image of a snapshot is built in runs of layers of at most 256 MiB (a larger layer
    alone), so the staging memory does not grow with the state: four full-attention layers of
    82/164/328/41 MiB with linear layers between them (runs of three layers, an oversize layer alone,
    the rest) give the bytes the per-layer exports give, load back to the same bytes, and once the
    oversize run's buffer is released the calls hold no more than the 256 MiB they may keep."""
    from moeflux_amd import Config
    from moeflux_amd.hip import mem_free
    hkv, d = 2, 256
    lens = {1: 21000, 3: 42000, 5: 84000, 7: 10500}
    cfg = Config(num_layers=8, full_attn_interval=2, num_attn_heads=8, num_kv_heads=hkv, head_dim=d,
                 kv_capacity=84032, kv_dtype=1, linear_num_k_heads=2, linear_num_v_heads=4,
                 linear_key_dim=64, linear_value_dim=64)
    case = GdnCase(3, 2, 4, 64, 64, T=2)
    rng = np.random.default_rng(5)
    with mfa.Ctx(cfg) as c:
        for layer, n in lens.items():
            k = oracle.bf16_to_f32(oracle.f32_to_bf16(rng.standard_normal((n, hkv * d), dtype=np.float32)))
            c.kv_import(layer, k, k[::-1].copy())
        for layer in (0, 2, 4, 6):
            c.set_linear_weights(layer, case.conv_w, case.a_log, case.dt_bias, case.norm_w)
            c.linear_state_import(layer, case.conv_state * (layer + 1), case.ssm_state)
        probe = rng.standard_normal(8 * d, dtype=np.float32)

        def settled_free():
            # the runtime returns a freed buffer some commands after the last one that used it
            best = 0
            for _ in range(8):
                c.sdpa_decode(7, probe, probe)
                c.sync()
                best = max(best, mem_free())
            return best

        free0 = settled_free()
        blob = c.state_save()
        assert settled_free() >= free0 - (8 << 20)
        want = bytearray(blob[:40])
        for layer in range(8):
            if layer in lens:
                k, v = c.kv_export(layer)
                want += struct.pack("<i", k.shape[0]) + k.tobytes() + v.tobytes()
            else:
                cs, ss = c.linear_state_export(layer)
                want += cs.astype("<f4").tobytes() + ss.astype("<f4").tobytes()
        assert bytes(want) == blob
        del want
        c.memory_clear()
        c.state_load(blob)
        assert [c.kv_len(layer) for layer in (1, 3, 5, 7)] == [21000, 42000, 84000, 10500]
        assert settled_free() >= free0 - (256 << 20) - (8 << 20)
        assert c.state_save() == blob
