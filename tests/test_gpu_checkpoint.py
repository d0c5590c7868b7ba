"""Checkpoints by sequence position (RsCtx::checkpoint_pos / restore_to,
crates/moeflux/src/riir/mod.rs:2015-2100), through the C ABI.  The cases are those of the
reference's tests/checkpoint_restore.rs, with the model's logits replaced by what this
library owns: the snapshot bytes and the next step's outputs, which must come back bit for bit."""
import numpy as np
import pytest

from tests.util import GdnCase, sdpa_random_inputs

pytestmark = pytest.mark.gpu

Hq, Hkv, D = 8, 2, 64


def _cfg(bf16=False, cap=200):
    from moeflux_amd import Config
    return Config(num_layers=4, full_attn_interval=2, num_attn_heads=Hq, num_kv_heads=Hkv, head_dim=D,
                  kv_capacity=cap, kv_dtype=1 if bf16 else 0, linear_num_k_heads=2, linear_num_v_heads=4,
                  linear_key_dim=64, linear_value_dim=64)


class _Stack:
    """Layers 0, 2 linear, 1, 3 full attention; `advance(n)` feeds n tokens to every layer."""

    def __init__(self, c, seed=5, tokens=400):
        self.c, self.t = c, 0
        self.case = GdnCase(seed, 2, 4, 64, 64, T=tokens)
        _, _, self.k, self.v = sdpa_random_inputs(seed, Hq, Hkv, D, tokens)
        for layer in (0, 2):
            c.set_linear_weights(layer, self.case.conv_w, self.case.a_log, self.case.dt_bias, self.case.norm_w)

    def advance(self, n):
        g = self.case
        for _ in range(n):
            t = self.t
            for layer in (1, 3):
                self.c.kv_append(layer, self.k[t] * layer, self.v[t])
            for layer in (0, 2):
                self.c.gdn_step(layer, g.qkv[t] * (layer + 1), g.z[t], g.alpha[t], g.beta[t])
            self.t += 1

    def probe(self):
        """One more token's outputs on every layer, from the current state (which it advances)."""
        q, gate, _, _ = sdpa_random_inputs(77, Hq, Hkv, D, 1)
        x = GdnCase(78, 2, 4, 64, 64, T=1)
        outs = []
        for layer in (1, 3):
            self.c.kv_append(layer, self.k[399], self.v[399])
            outs.append(self.c.sdpa_decode(layer, q, gate))
        for layer in (0, 2):
            outs.append(self.c.gdn_step(layer, x.qkv[0], x.z[0], x.alpha[0], x.beta[0]))
        return outs


@pytest.mark.parametrize("bf16", [False, True])
def test_checkpoint_then_restore_round_trips(mfa, bf16):
    """checkpoint_restore.rs:71-113: state at P, a checkpoint, more tokens, restore_to(P); the
    probe token then gives what it gave right after the checkpoint.  Here also the snapshot
    bytes, and with lengths on either side of a cache block edge."""
    with mfa.Ctx(_cfg(bf16)) as c:
        s = _Stack(c)
        for P, more in ((6, 3), (33, 40), (64, 1), (100, 0)):
            s.advance(P - s.t)
            assert c.memory_seq_pos_max() == P
            c.checkpoint_pos(P)
            blob = c.state_save()
            first = s.probe()
            s.advance(more)                      # tokens P+1 .. overwrite what the probe appended
            assert c.state_save() != blob
            c.restore_to(P)
            assert c.memory_seq_pos_max() == P and c.state_save() == blob
            again = s.probe()
            for a, b in zip(first, again):
                assert np.array_equal(a, b)
            c.restore_to(P)                      # the checkpoint at P itself survives a restore
            s.t = P
            assert c.state_save() == blob


@pytest.mark.parametrize("bf16", [False, True])
def test_restore_to_a_shorter_state_zeroes_the_dropped_rows(mfa, bf16):
    """Rows past the restored length must read as zero afterwards, as after a truncation: the
    kernels give masked positions the weight 0, and 0 times a stale NaN would be NaN as soon as
    the cache grows into the block that holds it."""
    q, gate, _, _ = sdpa_random_inputs(3, Hq, Hkv, D, 1)
    with mfa.Ctx(_cfg(bf16)) as c2:
        s2 = _Stack(c2)
        s2.advance(10)
        fresh = c2.state_save()
        s2.advance(10)
        want_state, want_out = c2.state_save(), c2.sdpa_decode(1, q, gate)
    with mfa.Ctx(_cfg(bf16)) as c:
        s = _Stack(c)
        s.advance(10)
        c.checkpoint_pos(10)
        bad = np.full(Hkv * D, np.nan, np.float32)
        for _ in range(60):
            c.kv_append(1, bad, bad)
            c.kv_append(3, bad, bad)
        c.restore_to(10)
        assert c.state_save() == fresh
        s.advance(10)                             # the same ten tokens from the restored state
        assert c.state_save() == want_state
        out = c.sdpa_decode(1, q, gate)
        assert np.isfinite(out).all() and np.array_equal(out, want_out)


def test_restore_to_unknown_pos_errors(mfa):
    """checkpoint_restore.rs:118-130; the failure changes nothing."""
    from moeflux_amd import MfaError, ffi
    with mfa.Ctx(_cfg()) as c:
        s = _Stack(c)
        s.advance(6)
        before = c.state_save()
        with pytest.raises(MfaError) as e:
            c.restore_to(9999)
        assert e.value.code == ffi.ERR_NO_CHECKPOINT and "9999" in str(e.value)
        assert c.state_save() == before and c.checkpoint_count() == 0


def test_memory_clear_drops_snapshots(mfa):
    """checkpoint_restore.rs:135-152."""
    from moeflux_amd import MfaError, ffi
    with mfa.Ctx(_cfg()) as c:
        s = _Stack(c)
        s.advance(6)
        c.checkpoint_pos(6)
        assert c.checkpoint_count() == 1
        c.memory_clear()
        assert c.checkpoint_count() == 0
        with pytest.raises(MfaError) as e:
            c.restore_to(6)
        assert e.value.code == ffi.ERR_NO_CHECKPOINT


def test_lru_eviction_keeps_last_n(mfa):
    """checkpoint_restore.rs:158-180: cap 4, five positions, the oldest goes; a failed restore
    changes nothing."""
    from moeflux_amd import MfaError
    with mfa.Ctx(_cfg()) as c:
        s = _Stack(c)
        s.advance(6)
        for pos in (50, 100, 150, 200, 250):
            c.checkpoint_pos(pos)
        assert c.checkpoint_count() == 4
        with pytest.raises(MfaError):
            c.restore_to(50)
        assert c.checkpoint_count() == 4
        c.restore_to(250)


def test_lru_protects_pos_zero(mfa):
    """checkpoint_restore.rs:185-198."""
    from moeflux_amd import MfaError
    with mfa.Ctx(_cfg()) as c:
        s = _Stack(c)
        s.advance(6)
        for pos in (0, 50, 100, 150, 200):
            c.checkpoint_pos(pos)
        assert c.checkpoint_count() == 4
        with pytest.raises(MfaError):
            c.restore_to(50)                     # the oldest unprotected one went
        c.restore_to(0)                          # position 0 stays, and restoring it voids the later ones
        assert c.checkpoint_count() == 1


def test_overwrite_restore_order_and_cap_changes(mfa):
    """riir/mod.rs:2023-2033: storing at a position again replaces the state and makes it the
    newest; :2083-2084: a restore drops the later positions only; :2094-2096: a lower cap acts at
    the next store, and with a cap below 2 the protected entries stay (:2052-2058)."""
    from moeflux_amd import MfaError
    with mfa.Ctx(_cfg()) as c:
        s = _Stack(c)
        s.advance(5)
        c.checkpoint_pos(5)
        old = c.state_save()
        s.advance(4)
        c.checkpoint_pos(9)
        s.advance(3)
        c.checkpoint_pos(5)                       # same key, the state of 12 tokens
        now = c.state_save()
        assert c.checkpoint_count() == 2
        c.restore_to(5)                           # drops 9 (> 5), brings back the 12-token state
        assert c.state_save() == now != old and c.checkpoint_count() == 1
        for pos in (20, 30, 40):
            c.checkpoint_pos(pos)                 # order now 5, 20, 30, 40
        c.checkpoint_pos(5)                       # 5 becomes the newest: 20, 30, 40, 5
        c.checkpoint_pos(60)                      # evicts 20, not 5
        assert c.checkpoint_count() == 4
        with pytest.raises(MfaError):
            c.restore_to(20)
        c.set_max_checkpoints(2)
        assert c.checkpoint_count() == 4          # not retroactive
        c.checkpoint_pos(70)                      # 30, 40 and 5 go, oldest first, until two are left
        assert c.checkpoint_count() == 2
        c.restore_to(70)
        c.restore_to(60)                          # drops 70
        assert c.checkpoint_count() == 1
        c.set_max_checkpoints(0)
        c.checkpoint_pos(0)                       # 60 goes; position 0 is never evicted
        c.checkpoint_pos(80)                      # nothing evictable: 0 and the one just stored stay
        assert c.checkpoint_count() == 2
        c.restore_to(0)
        with pytest.raises(MfaError):
            c.set_max_checkpoints(-1)


def test_checkpoint_of_an_empty_context_and_of_one_kind_only(mfa):
    """Nothing appended yet (zero-length caches, zero states), and stacks with only one kind of layer."""
    from moeflux_amd import Config
    with mfa.Ctx(_cfg()) as c:
        s = _Stack(c)
        empty = c.state_save()
        c.checkpoint_pos(0)
        s.advance(7)
        c.restore_to(0)
        assert c.state_save() == empty and c.memory_seq_pos_max() == 0
    with mfa.Ctx(Config(num_layers=2, full_attn_interval=1, num_attn_heads=Hq, num_kv_heads=Hkv, head_dim=D,
                        kv_capacity=64, kv_dtype=1)) as c:
        _, _, k, v = sdpa_random_inputs(1, Hq, Hkv, D, 40, bf16=True)
        c.kv_import(0, k[:33], v[:33])
        c.checkpoint_pos(33)
        blob = c.state_save()
        c.kv_import(0, k, v)
        c.kv_import(1, k[:5], v[:5])
        c.restore_to(33)
        assert c.state_save() == blob and c.kv_len(1) == 0
    case = GdnCase(2, 2, 4, 64, 64, T=6)
    with mfa.Ctx(Config(num_layers=2, full_attn_interval=3, linear_num_k_heads=2, linear_num_v_heads=4,
                        linear_key_dim=64, linear_value_dim=64)) as c:
        for layer in (0, 1):
            c.set_linear_weights(layer, case.conv_w, case.a_log, case.dt_bias, case.norm_w)
        for t in range(3):
            c.gdn_step(0, case.qkv[t], case.z[t], case.alpha[t], case.beta[t])
        c.checkpoint_pos(3)
        blob = c.state_save()
        a = c.gdn_step(0, case.qkv[3], case.z[3], case.alpha[3], case.beta[3])
        c.gdn_step(1, case.qkv[4], case.z[4], case.alpha[4], case.beta[4])
        c.restore_to(3)
        assert c.state_save() == blob
        assert np.array_equal(c.gdn_step(0, case.qkv[3], case.z[3], case.alpha[3], case.beta[3]), a)
