"""Host-side arithmetic of the library that needs no GPU: the tiled KV-cache
addressing and the split-K partitioning."""
import numpy as np
import pytest

from moeflux_amd import ffi


@pytest.mark.parametrize("dtype,blk", [(ffi.KV_BF16, 32), (ffi.KV_F32, 16)])
@pytest.mark.parametrize("D", [64, 128, 256])
@pytest.mark.parametrize("is_v", [0, 1])
def test_tiling_is_a_bijection_on_every_block(dtype, blk, D, is_v):
    lib = ffi.load()
    npos = 3 * blk
    off = np.array([[lib.mfa_debug_kv_offset(dtype, is_v, p, x, D) for x in range(D)]
                    for p in range(npos)])
    assert sorted(off.reshape(-1).tolist()) == list(range(npos * D))        # one-to-one, no holes
    for b in range(3):                                                       # a block is contiguous
        o = off[b * blk:(b + 1) * blk]
        assert o.min() == b * blk * D and o.max() == (b + 1) * blk * D - 1


def test_tiling_matches_the_decode_kernels_operand_order():
    """bf16: lane (row m = lane%16, group g = lane/16) of load `li` in a block reads 8
    consecutive elements at li*512 + lane*8; they must be channels 8*(4s+g)..+7 of position
    16*sub + m for K (li = 2*s + sub), and for V the 8 positions
    {4g..4g+3, 16+4g..16+4g+3} of channel 16*dt + m (li = dt)."""
    lib = ffi.load()
    D = 256
    for li in (0, 5, 9, 15):
        for lane in (0, 17, 38, 63):
            m, g = lane % 16, lane // 16
            base = li * 512 + lane * 8
            s, sub = li // 2, li % 2
            for e in range(8):
                assert lib.mfa_debug_kv_offset(ffi.KV_BF16, 0, 16 * sub + m, 8 * (4 * s + g) + e, D) == base + e
                pos = 16 * (e // 4) + 4 * g + e % 4
                assert lib.mfa_debug_kv_offset(ffi.KV_BF16, 1, pos, 16 * li + m, D) == base + e
    # f32: K load s holds channels 4*(4s+g)..+3 of position m; V load dt holds positions
    # 4g .. 4g+3 of channel 16 dt + m
    D = 128
    for li in (0, 3, 7):
        for lane in (0, 21, 63):
            m, g = lane % 16, lane // 16
            base = li * 256 + lane * 4
            for j in range(4):
                assert lib.mfa_debug_kv_offset(ffi.KV_F32, 0, m, 4 * (4 * li + g) + j, D) == base + j
                assert lib.mfa_debug_kv_offset(ffi.KV_F32, 1, 4 * g + j, 16 * li + m, D) == base + j


def test_tiling_rejects_bad_arguments():
    lib = ffi.load()
    assert lib.mfa_debug_kv_offset(ffi.KV_BF16, 0, -1, 0, 256) == -1
    assert lib.mfa_debug_kv_offset(ffi.KV_BF16, 0, 0, 256, 256) == -1
    assert lib.mfa_debug_kv_offset(ffi.KV_BF16, 0, 0, 0, 100) == -1
    assert lib.mfa_debug_kv_offset(9, 0, 0, 0, 256) == -1


def test_workspace_bound_covers_every_length_up_to_the_capacity():
    """The split count falls and rises with the length (1024 blocks: 128 splits of one pass; 1025
    blocks: 65 splits of two), so a context sizes its split-K workspace by a bound over all lengths
    up to its capacity, not by the count at the capacity."""
    lib = ffi.load()
    ns, mx = lib.mfa_debug_num_splits, lib.mfa_debug_max_splits
    assert ns(ffi.KV_BF16, 32, 2, 256, 32768, 256, 0) == 128
    assert ns(ffi.KV_BF16, 32, 2, 256, 32800, 256, 0) == 65
    assert mx(ffi.KV_BF16, 32, 2, 256, 32800, 256, 0) >= 128
    rng = np.random.default_rng(5)
    shapes = [(ffi.KV_BF16, 32, 2, 256), (ffi.KV_F32, 32, 4, 128), (ffi.KV_BF16, 64, 2, 128), (ffi.KV_BF16, 8, 8, 64),
              (ffi.KV_F32, 40, 2, 256), (ffi.KV_BF16, 32 * 12, 2 * 12, 256)]
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
    lib = ffi.load()
    ns = lib.mfa_debug_num_splits
    # config 3: 1024 blocks of 32 positions per kv head, 256 CUs / 2 kv heads -> 128 splits
    assert ns(ffi.KV_BF16, 32, 2, 256, 32768, 256, 0) == 128
    # config 1: 256 blocks of 16 positions per kv head, 4 kv heads -> 64 splits of 4 blocks
    assert ns(ffi.KV_F32, 32, 4, 128, 4096, 256, 0) == 64
    assert ns(ffi.KV_BF16, 32, 2, 256, 1, 256, 0) == 1
    assert ns(ffi.KV_BF16, 32, 2, 256, 33, 256, 0) == 1          # 2 blocks, one split
    for forced in (1, 2, 7, 64):
        got = ns(ffi.KV_BF16, 32, 2, 256, 8192, 256, forced)
        assert 1 <= got <= forced
    # more than 16 query heads per kv head: head groups share the CUs; up to head_dim 128 two
    # workgroups fit a CU, so 2 * 256 / 4 splits where each still gets a whole pass of 8 blocks
    assert ns(ffi.KV_BF16, 64, 2, 128, 32768, 256, 0) == 128
    assert ns(ffi.KV_F32, 32, 4, 128, 32768, 256, 0) == 128       # 2048 blocks of 16, 16 per split
    assert ns(ffi.KV_F32, 32, 4, 128, 8192, 256, 0) == 64         # 512 blocks: one pass of 8 each, not doubled
    # whole passes only: 12 layers x 2 kv heads of 256 blocks -> 256 / 24 = 10 splits of 26 blocks
    # would leave a ragged fourth pass; 8 splits of 32
    assert ns(ffi.KV_BF16, 32 * 12, 2 * 12, 256, 8192, 256, 0) == 8
    assert ns(ffi.KV_BF16, 32, 2, 256, 49152, 256, 0) == 96       # 1536 blocks: 16 per split, not 12
    assert ns(ffi.KV_BF16, 30, 4, 128, 64, 256, 0) == -1          # 30 % 4 != 0
    assert ns(ffi.KV_BF16, 32, 2, 256, 0, 256, 0) == -1
