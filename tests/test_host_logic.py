"""Host-side arithmetic of the library that needs no GPU: the tiled KV-cache
addressing and the split-K partitioning."""
import numpy as np
import pytest

from moeflux_amd import ffi


@pytest.mark.parametrize("dtype,vblk", [(ffi.KV_BF16, 32), (ffi.KV_F32, 16)])
@pytest.mark.parametrize("D", [64, 128, 256])
@pytest.mark.parametrize("is_v", [0, 1])
def test_tiling_is_a_bijection_on_every_block(dtype, vblk, D, is_v):
    """K lies in chunks of 64 positions, V in blocks of 32 (bf16) or 16 (f32); a chunk / block of a
    plane is one contiguous run, and the addressing is one-to-one without holes."""
    lib = ffi.load()
    blk = vblk if is_v else 64
    npos = 3 * 64
    off = np.array([[lib.mfa_debug_kv_offset(dtype, is_v, p, x, D) for x in range(D)]
                    for p in range(npos)])
    assert sorted(off.reshape(-1).tolist()) == list(range(npos * D))        # one-to-one, no holes
    for b in range(npos // blk):                                             # a chunk / block is contiguous
        o = off[b * blk:(b + 1) * blk]
        assert o.min() == b * blk * D and o.max() == (b + 1) * blk * D - 1


def test_tiling_matches_the_kernels_operand_order():
    """bf16: lane (row m = lane%16, group g = lane/16) of a 1 KiB piece reads 8 consecutive elements
    at piece*512 + lane*8.  K piece s*4 + sub of a chunk must be channels 8*(4s+g)..+7 of position
    16*sub + m (k-step s, sub-tile sub: the four waves of a decode workgroup read the four sub-tiles
    of a k-step side by side); V piece dt of a block the 8 positions {4g..4g+3, 16+4g..16+4g+3} of
    channel 16*dt + m."""
    lib = ffi.load()
    D = 256
    for chunk in (0, 2):
        for s in (0, 3, 7):
            for sub in range(4):
                for lane in (0, 17, 38, 63):
                    m, g = lane % 16, lane // 16
                    base = chunk * 64 * D + (s * 4 + sub) * 512 + lane * 8
                    for e in range(8):
                        assert lib.mfa_debug_kv_offset(ffi.KV_BF16, 0, chunk * 64 + 16 * sub + m, 8 * (4 * s + g) + e, D) == base + e
    for li in (0, 5, 9, 15):
        for lane in (0, 17, 38, 63):
            m, g = lane % 16, lane // 16
            base = li * 512 + lane * 8
            for e in range(8):
                pos = 16 * (e // 4) + 4 * g + e % 4
                assert lib.mfa_debug_kv_offset(ffi.KV_BF16, 1, pos, 16 * li + m, D) == base + e
    # f32: K piece s*4 + sub holds channels 4*(4s+g)..+3 of position 16*sub + m; V piece dt of a
    # 16-position block holds positions 4g .. 4g+3 of channel 16 dt + m
    D = 128
    for s in (0, 3, 7):
        for sub in range(4):
            for lane in (0, 21, 63):
                m, g = lane % 16, lane // 16
                base = 64 * D + (s * 4 + sub) * 256 + lane * 4
                for j in range(4):
                    assert lib.mfa_debug_kv_offset(ffi.KV_F32, 0, 64 + 16 * sub + m, 4 * (4 * s + g) + j, D) == base + j
    for li in (0, 3, 7):
        for lane in (0, 21, 63):
            m, g = lane % 16, lane // 16
            base = li * 256 + lane * 4
            for j in range(4):
                assert lib.mfa_debug_kv_offset(ffi.KV_F32, 1, 4 * g + j, 16 * li + m, D) == base + j


def test_tiling_rejects_bad_arguments():
    lib = ffi.load()
    assert lib.mfa_debug_kv_offset(ffi.KV_BF16, 0, -1, 0, 256) == -1
    assert lib.mfa_debug_kv_offset(ffi.KV_BF16, 0, 0, 256, 256) == -1
    assert lib.mfa_debug_kv_offset(ffi.KV_BF16, 0, 0, 0, 100) == -1
    assert lib.mfa_debug_kv_offset(9, 0, 0, 0, 256) == -1


def test_workspace_bound_covers_every_length_up_to_the_capacity():
    """A context sizes its split-K workspace by the most splits any length up to its capacity gets."""
    lib = ffi.load()
    ns, mx = lib.mfa_debug_num_splits, lib.mfa_debug_max_splits
    rng = np.random.default_rng(5)
    shapes = [(ffi.KV_BF16, 32, 2, 256), (ffi.KV_F32, 32, 4, 128), (ffi.KV_BF16, 64, 2, 128), (ffi.KV_BF16, 8, 8, 64),
              (ffi.KV_F32, 40, 2, 256), (ffi.KV_BF16, 32 * 12, 2 * 12, 256), (ffi.KV_BF16, 16, 1, 128)]
    for kv, Hq, Hkv, d in shapes:
        for cap in (1, 100, 4096, 8191, 32800, 65536, 131072):
            for forced in (0, 3, 129, 300):
                bound = mx(kv, Hq, Hkv, d, cap, 256, forced)
                assert bound >= 1
                lens = {1, cap, max(1, cap - 1), max(1, cap // 2)} | {int(x) for x in rng.integers(1, cap + 1, 40)}
                for L in sorted(lens):
                    got = ns(kv, Hq, Hkv, d, L, 256, forced)
                    assert 1 <= got <= bound, (kv, Hq, Hkv, d, cap, forced, L, got, bound)
    assert mx(ffi.KV_BF16, 30, 4, 128, 64, 256, 0) == -1


def test_split_partitioning():
    """The cache is handed out in units of 64 positions (128 at head_dim 64 of a bf16 cache), one
    workgroup per CU where there are that many units; the shares differ by at most one unit, so the
    split count never falls as the cache grows."""
    lib = ffi.load()
    ns = lib.mfa_debug_num_splits
    # the 32K decode shape: 512 units per kv head, 256 CUs / 2 kv heads -> 128 splits of 4
    assert ns(ffi.KV_BF16, 32, 2, 256, 32768, 256, 0) == 128
    assert ns(ffi.KV_BF16, 32, 2, 256, 32800, 256, 0) == 128      # one split of 5 units, 127 of 4
    assert ns(ffi.KV_BF16, 32, 2, 256, 49152, 256, 0) == 128      # 6 units each
    # the 4K f32 decode shape: 64 units per kv head, 4 kv heads -> 64 splits of one unit
    assert ns(ffi.KV_F32, 32, 4, 128, 4096, 256, 0) == 64
    assert ns(ffi.KV_BF16, 32, 2, 256, 1, 256, 0) == 1
    assert ns(ffi.KV_F32, 32, 4, 128, 64, 256, 0) == 1
    assert ns(ffi.KV_F32, 32, 4, 128, 65, 256, 0) == 2
    # no automatic share below the kernel's smallest pass (2 chunks at head_dim 256 of a bf16 cache)
    assert ns(ffi.KV_BF16, 32, 2, 256, 192, 256, 0) == 1
    assert ns(ffi.KV_BF16, 32, 2, 256, 193, 256, 0) == 2
    assert ns(ffi.KV_BF16, 32, 2, 256, 8192, 256, 0) == 64
    for forced in (1, 2, 7, 64):
        got = ns(ffi.KV_BF16, 32, 2, 256, 8192, 256, forced)
        assert 1 <= got <= forced
    assert ns(ffi.KV_BF16, 32, 2, 256, 100, 256, 64) == 2          # never more splits than units
    # more than 16 query heads per kv head: the head groups share the CUs
    assert ns(ffi.KV_BF16, 64, 2, 128, 32768, 256, 0) == 64
    # 12 layers x 2 kv heads in one launch: 256 / 24 = 10 splits of 12 or 13 units
    assert ns(ffi.KV_BF16, 32 * 12, 2 * 12, 256, 8192, 256, 0) == 10
    prev = 0
    for L in range(1, 70000, 61):
        got = ns(ffi.KV_BF16, 32, 2, 256, L, 256, 0)
        assert got >= prev
        prev = got
    assert ns(ffi.KV_BF16, 30, 4, 128, 64, 256, 0) == -1          # 30 % 4 != 0
    assert ns(ffi.KV_BF16, 32, 2, 256, 0, 256, 0) == -1
