"""GPU parity of the 4-bit dequantising matrix-vector product (the projections either side
of the attention core) against the CPU oracle, through the C ABI."""
import ctypes as C

import numpy as np
import pytest

from tests.util import TOL_F32, rel_err

pytestmark = pytest.mark.gpu


def _weights(rng, out_dim, in_dim, oracle):
    packed = rng.integers(0, 2 ** 32, size=(out_dim, in_dim // 8), dtype=np.uint64).astype(np.uint32)
    # MLX affine 4-bit: scale = (max - min) / 15, bias = min of a group of 64 weights
    sc = oracle.f32_to_bf16(np.abs(rng.standard_normal((out_dim, in_dim // 64))) * 0.01 + 0.002)
    bi = oracle.f32_to_bf16(-7.5 * oracle.bf16_to_f32(sc) + rng.standard_normal((out_dim, in_dim // 64)) * 0.003)
    return packed, sc, bi


def test_reference_unit_vectors(mfa):
    """cpu_matvec.rs:366-417: the reference's known answers, bit for bit."""
    ones = np.ones(64, np.float32)
    f = mfa.dequant_matvec_4bit_cpu
    assert f(np.full(8, 0x11111111, np.uint32), [0x3F80], [0x0000], 64, 1, ones)[0] == 64.0
    assert np.array_equal(f(np.full(16, 0xFFFFFFFF, np.uint32), [0x3F80] * 2, [0x3F80] * 2, 64, 2, np.zeros(64, np.float32)),
                          np.zeros(2, np.float32))
    assert f(np.zeros(8, np.uint32), [0x40A0], [0x4000], 64, 1, ones)[0] == 128.0


@pytest.mark.parametrize("out_dim,in_dim", [(1, 64), (5, 192), (33, 2048), (512, 4096), (100, 4160), (4096, 8192),
                                            (16384, 4096), (37, 1024), (7168, 16384), (100, 12288), (33, 8256)])
def test_matvec_matches_oracle(mfa, oracle, out_dim, in_dim):
    """Projection shapes of the variants (q_proj 16384x4096, k/v_proj 512x4096, o_proj 4096x8192,
    expert down_proj x1024, the latent-attention variants' o_proj 7168x16384) and ragged ones:
    row counts that do not fill a workgroup, widths that do not fill the last 1024-input run."""
    rng = np.random.default_rng(out_dim + in_dim)
    packed, sc, bi = _weights(rng, out_dim, in_dim, oracle)
    x = rng.standard_normal(in_dim).astype(np.float32)
    ref = oracle.dequant_matvec_4bit(packed, sc, bi, in_dim, out_dim, x)
    out = mfa.dequant_matvec_4bit_cpu(packed, sc, bi, in_dim, out_dim, x)
    assert rel_err(out, ref) <= TOL_F32


@pytest.mark.parametrize("scale", [1e-30, 1e-6, 1e4, 1e30])
def test_matvec_input_magnitudes(mfa, oracle, scale):
    """The kernel splits x into three bf16 parts (exact for any f32 whose parts stay normal) and
    converts the nibbles exactly: the result must not depend on the magnitude of x, nor on a
    large common offset in x (group sums much larger than the signed part)."""
    rng = np.random.default_rng(11)
    out_dim, in_dim = 48, 2048
    packed, sc, bi = _weights(rng, out_dim, in_dim, oracle)
    x = (rng.standard_normal(in_dim) * scale).astype(np.float32)
    ref = oracle.dequant_matvec_4bit(packed, sc, bi, in_dim, out_dim, x)
    assert rel_err(mfa.dequant_matvec_4bit_cpu(packed, sc, bi, in_dim, out_dim, x), ref) <= TOL_F32
    xo = (x + np.float32(3.0 * scale)).astype(np.float32)
    ref = oracle.dequant_matvec_4bit(packed, sc, bi, in_dim, out_dim, xo)
    assert rel_err(mfa.dequant_matvec_4bit_cpu(packed, sc, bi, in_dim, out_dim, xo), ref) <= TOL_F32


def test_batched_products_in_one_launch(mfa, oracle):
    """q, k and v projections of one layer as one call on device pointers
    (full_attn_forward.rs:193-227 batches them into one command buffer)."""
    from moeflux_amd import Config, ffi
    from moeflux_amd.hip import DeviceArray
    rng = np.random.default_rng(4)
    in_dim = 4096
    x = rng.standard_normal(in_dim).astype(np.float32)
    shapes = [16384, 512, 512]
    dx = DeviceArray.from_host(x)
    keep, refs, outs = [dx], [], []
    specs = (ffi.mfa_matvec_spec * 3)()
    for i, od in enumerate(shapes):
        packed, sc, bi = _weights(rng, od, in_dim, oracle)
        refs.append(oracle.dequant_matvec_4bit(packed, sc, bi, in_dim, od, x))
        dw, ds, db = DeviceArray.from_host(packed), DeviceArray.from_host(sc), DeviceArray.from_host(bi)
        do = DeviceArray((od,), np.float32, zero=True)
        keep += [dw, ds, db]
        outs.append(do)
        specs[i] = ffi.mfa_matvec_spec(dw.ptr, ds.ptr, db.ptr, dx.ptr, do.ptr, od, in_dim)
    with mfa.Ctx(Config(num_layers=1, full_attn_interval=1, num_attn_heads=8, num_kv_heads=2, head_dim=64,
                        kv_capacity=4)) as c:
        rc = c.lib.mfa_dequant_matvec_4bit_dev(c.h, 3, C.byref(specs))
        assert rc == 0, ffi.last_error()
        c.sync()
        for o, r in zip(outs, refs):
            assert rel_err(o.to_host(), r) <= TOL_F32


def test_batched_products_of_different_widths(mfa, oracle):
    """Eight products in one launch whose input widths differ (the launch is shaped by the widest)
    and whose row counts do not fill their last 16-row tile."""
    from moeflux_amd import Config, ffi
    from moeflux_amd.hip import DeviceArray
    rng = np.random.default_rng(8)
    shapes = [(100, 4096), (33, 64), (512, 2048), (1, 1024), (17, 4160), (64, 192), (250, 3072), (16, 8192)]
    keep, refs, outs = [], [], []
    specs = (ffi.mfa_matvec_spec * len(shapes))()
    for i, (od, idim) in enumerate(shapes):
        packed, sc, bi = _weights(rng, od, idim, oracle)
        x = rng.standard_normal(idim).astype(np.float32)
        refs.append(oracle.dequant_matvec_4bit(packed, sc, bi, idim, od, x))
        dw, ds, db, dx = (DeviceArray.from_host(a) for a in (packed, sc, bi, x))
        do = DeviceArray((od,), np.float32, zero=True)
        keep += [dw, ds, db, dx]
        outs.append(do)
        specs[i] = ffi.mfa_matvec_spec(dw.ptr, ds.ptr, db.ptr, dx.ptr, do.ptr, od, idim)
    with mfa.Ctx(Config(num_layers=1, full_attn_interval=1, num_attn_heads=8, num_kv_heads=2, head_dim=64,
                        kv_capacity=4)) as c:
        rc = c.lib.mfa_dequant_matvec_4bit_dev(c.h, len(shapes), C.byref(specs))
        assert rc == 0, ffi.last_error()
        c.sync()
        for o, r, sh in zip(outs, refs, shapes):
            assert rel_err(o.to_host(), r) <= TOL_F32, sh


def test_scale_rows_off_a_16_byte_boundary(mfa, oracle):
    """Scales and biases that start 2 bytes past a 16-byte boundary take the element-wise loads;
    the result is the same as for aligned ones."""
    from moeflux_amd import Config, ffi
    from moeflux_amd.hip import DeviceArray
    rng = np.random.default_rng(9)
    od, idim = 100, 4096
    packed, sc, bi = _weights(rng, od, idim, oracle)
    x = rng.standard_normal(idim).astype(np.float32)
    ref = oracle.dequant_matvec_4bit(packed, sc, bi, idim, od, x)
    pad = lambda a: np.concatenate([np.zeros(1, np.uint16), np.ascontiguousarray(a).reshape(-1)])
    dw, dx = DeviceArray.from_host(packed), DeviceArray.from_host(x)
    ds, db = DeviceArray.from_host(pad(sc)), DeviceArray.from_host(pad(bi))
    das, dab = DeviceArray.from_host(np.ascontiguousarray(sc)), DeviceArray.from_host(np.ascontiguousarray(bi))
    o1, o2 = DeviceArray((od,), np.float32, zero=True), DeviceArray((od,), np.float32, zero=True)
    with mfa.Ctx(Config(num_layers=1, full_attn_interval=1, num_attn_heads=8, num_kv_heads=2, head_dim=64,
                        kv_capacity=4)) as c:
        spec = (ffi.mfa_matvec_spec * 1)(ffi.mfa_matvec_spec(dw.ptr, ds.offset(1), db.offset(1), dx.ptr, o1.ptr, od, idim))
        assert c.lib.mfa_dequant_matvec_4bit_dev(c.h, 1, C.byref(spec)) == 0, ffi.last_error()
        spec = (ffi.mfa_matvec_spec * 1)(ffi.mfa_matvec_spec(dw.ptr, das.ptr, dab.ptr, dx.ptr, o2.ptr, od, idim))
        assert c.lib.mfa_dequant_matvec_4bit_dev(c.h, 1, C.byref(spec)) == 0, ffi.last_error()
        c.sync()
        assert rel_err(o1.to_host(), ref) <= TOL_F32
        assert np.array_equal(o1.to_host(), o2.to_host())
        # weights and x are read 16 bytes at a time: other alignments are refused, not misread
        spec = (ffi.mfa_matvec_spec * 1)(ffi.mfa_matvec_spec(dw.offset(1), das.ptr, dab.ptr, dx.ptr, o2.ptr, od - 1, idim))
        assert c.lib.mfa_dequant_matvec_4bit_dev(c.h, 1, C.byref(spec)) == ffi.ERR_INVALID
        spec = (ffi.mfa_matvec_spec * 1)(ffi.mfa_matvec_spec(dw.ptr, das.ptr, dab.ptr, dx.offset(1), o2.ptr, od, idim - 64))
        assert c.lib.mfa_dequant_matvec_4bit_dev(c.h, 1, C.byref(spec)) == ffi.ERR_INVALID


def test_tiled_weights_give_the_same_products(mfa, oracle):
    """Weights, scales and biases re-ordered on the device (mfa_matvec_tile_weights_dev) and multiplied
    with mfa_dequant_matvec_4bit_tiled_dev, whose specs carry no scales or biases: the same results, bit
    for bit, as the file order gives, for ragged row counts, input widths that do not fill a run of 1024,
    and products of different widths in one launch; the re-ordered copy itself is checked against the
    layout's definition."""
    from moeflux_amd import Config, ffi
    from moeflux_amd.hip import DeviceArray
    rng = np.random.default_rng(10)
    shapes = [(100, 4096), (33, 64), (17, 9280), (1, 1024), (17, 4160), (250, 3072), (40, 16384), (1000, 4096)]
    keep, refs, outs, touts = [], [], [], []
    specs = (ffi.mfa_matvec_spec * len(shapes))()
    tspecs = (ffi.mfa_matvec_spec * len(shapes))()
    with mfa.Ctx(Config(num_layers=1, full_attn_interval=1, num_attn_heads=8, num_kv_heads=2, head_dim=64,
                        kv_capacity=4)) as c:
        lib = c.lib
        for i, (od, idim) in enumerate(shapes):
            packed, sc, bi = _weights(rng, od, idim, oracle)
            x = rng.standard_normal(idim).astype(np.float32)
            refs.append(oracle.dequant_matvec_4bit(packed, sc, bi, idim, od, x))
            dw, ds, db, dx = (DeviceArray.from_host(a) for a in (packed, sc, bi, x))
            words = int(lib.mfa_matvec_tiled_words(od, idim))
            tiles, runs = (od + 15) // 16, (idim + 1023) // 1024
            assert words == tiles * runs * 9 * 64 * 4
            dt = DeviceArray((words,), np.uint32)
            assert lib.mfa_matvec_tile_weights_dev(c.h, od, idim, dw.ptr, ds.ptr, db.ptr, dt.ptr) == 0, ffi.last_error()
            do, dto = DeviceArray((od,), np.float32, zero=True), DeviceArray((od,), np.float32, zero=True)
            keep += [dw, ds, db, dx, dt]
            outs.append(do)
            touts.append(dto)
            specs[i] = ffi.mfa_matvec_spec(dw.ptr, ds.ptr, db.ptr, dx.ptr, do.ptr, od, idim)
            tspecs[i] = ffi.mfa_matvec_spec(dt.ptr, None, None, dx.ptr, dto.ptr, od, idim)
            if i in (0, 4):   # the layout: [tile][run][scales and biases, then 8 steps][lane] x 4 words
                c.sync()
                rec = dt.to_host().reshape(tiles, runs, 9, 64, 4)
                t = rec[:, :, 1:]
                shape4 = (tiles, runs, 8, 64)
                rows = np.broadcast_to(np.minimum(16 * np.arange(tiles)[:, None, None, None] + np.arange(64)[None, None, None, :] % 16, od - 1), shape4)
                chunk = np.broadcast_to(4 * (8 * np.arange(runs)[None, :, None, None] + np.arange(8)[None, None, :, None]) + np.arange(64)[None, None, None, :] // 16, shape4)
                src = np.zeros((od, runs * 32, 4), np.uint32)
                src[:, :idim // 32] = packed.reshape(od, idim // 32, 4)
                assert np.array_equal(t, src[rows, chunk])
                # lane (n, g): row n's values for groups 16 run + 2 e + g % 2, scales for g < 2, else biases
                sb = rec[:, :, 0].copy().view(np.uint16).reshape(tiles, runs, 64, 8)
                groups = idim // 64
                both = np.zeros((2, od, runs * 16), np.uint16)
                both[0, :, :groups], both[1, :, :groups] = sc.reshape(od, groups), bi.reshape(od, groups)
                lanes = np.arange(64)
                r3 = np.minimum(16 * np.arange(tiles)[:, None, None, None] + (lanes % 16)[None, None, :, None], od - 1)
                g3 = 16 * np.arange(runs)[None, :, None, None] + 2 * np.arange(8)[None, None, None, :] + ((lanes // 16) % 2)[None, None, :, None]
                k3 = (lanes // 32)[None, None, :, None]
                assert np.array_equal(sb, both[np.broadcast_to(k3, sb.shape), np.broadcast_to(r3, sb.shape), np.broadcast_to(g3, sb.shape)])
        assert lib.mfa_dequant_matvec_4bit_dev(c.h, len(shapes), C.byref(specs)) == 0, ffi.last_error()
        assert lib.mfa_dequant_matvec_4bit_tiled_dev(c.h, len(shapes), C.byref(tspecs)) == 0, ffi.last_error()
        c.sync()
        for o, to, r, sh in zip(outs, touts, refs, shapes):
            assert rel_err(to.to_host(), r) <= TOL_F32, sh
            assert np.array_equal(o.to_host(), to.to_host()), sh
        # aligned group counts only (the 16-byte scale loads), one product
        one = (ffi.mfa_matvec_spec * 1)(tspecs[7])
        assert lib.mfa_dequant_matvec_4bit_tiled_dev(c.h, 1, C.byref(one)) == 0, ffi.last_error()
        c.sync()
        assert np.array_equal(touts[7].to_host(), outs[7].to_host())
        assert lib.mfa_matvec_tiled_words(16, 32) < 0
        assert lib.mfa_matvec_tile_weights_dev(c.h, 16, 64, None, keep[1].ptr, keep[2].ptr, keep[4].ptr) == ffi.ERR_INVALID


def test_matvec_errors(mfa):
    """cpu_matvec.rs:92-97: in_dim must be a multiple of the group size; NULL and shape checks."""
    from moeflux_amd import ffi
    lib = ffi.load()
    w, s, x, o = np.zeros(8, np.uint32), np.zeros(1, np.uint16), np.zeros(64, np.float32), np.zeros(1, np.float32)
    p = lambda a: a.ctypes.data_as(C.c_void_p)
    assert lib.mfa_dequant_matvec_4bit(1, 32, 64, p(w), p(s), p(s), p(x), p(o)) == ffi.ERR_INVALID
    assert lib.mfa_dequant_matvec_4bit(1, 64, 32, p(w), p(s), p(s), p(x), p(o)) == ffi.ERR_SHAPE
    assert lib.mfa_dequant_matvec_4bit(0, 64, 64, p(w), p(s), p(s), p(x), p(o)) == ffi.ERR_INVALID
    assert lib.mfa_dequant_matvec_4bit(1, 64, 64, None, p(s), p(s), p(x), p(o)) == ffi.ERR_INVALID
    assert lib.mfa_dequant_matvec_4bit(1, 64, 64, p(w), p(s), p(s), p(x), p(o)) == 0
    # wider than the widest supported row (16384 inputs): refused, nothing is read
    big_w, big_s, big_x = np.zeros(16448 // 8, np.uint32), np.zeros(16448 // 64, np.uint16), np.zeros(16448, np.float32)
    assert lib.mfa_dequant_matvec_4bit(1, 16448, 64, p(big_w), p(big_s), p(big_s), p(big_x), p(o)) == ffi.ERR_SHAPE
