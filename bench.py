#!/usr/bin/env python3
"""Benchmark of the MI355X attention path.

Headline (the one JSON line the driver reads): attention
microseconds per layer per token with the achieved HBM rate, on the
long-context configuration the metric is quoted on — gated GQA decode,
32 Q / 2 KV heads, head_dim 256, 32768 cached positions, bf16 K/V, batch 1
(the other workloads - 4K f32 decode, the DeltaNet step, the 512-token chunk, the 48-layer
sweep, the projections and the latent-cache attention - are reported under "extra").  A "step" is one
layer's decode attention for one token: mfa_sdpa_decode_dev over a KV cache that
already resides in HBM.  Steps rotate over `--layers` independent caches whose
total exceeds the 256 MB last-level cache, so every step streams from HBM.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Also on the line: "roofline" (the split-K partial kernel against 8 TB/s, timed
live with HIP events on the library's stream) and "cpu_baseline" (the scalar CPU
oracle on the same shape, one thread, on this host).
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published


def _c3_partial_traffic_bytes():
    """HBM bytes per launch of the split-K partial kernel on the headline workload: rocprofv3
    FETCH_SIZE + WRITE_SIZE scaled by the plain copy kernel, as recorded next to the counter summary
    (profiles/sdpa_partial_bf16_d256_c3_hbm_counters.md); None when the record is missing."""
    try:
        with open(os.path.join(ROOT, "profiles", "sdpa_partial_bf16_d256_c3_hbm_counters.json")) as f:
            return int(json.load(f)["traffic_bytes_per_dispatch"])
    except (OSError, KeyError, ValueError):
        return None


def _bf16_bits(x):
    """f32 -> bf16 bit patterns, round to nearest even (inputs here are finite)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    return ((u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))) >> np.uint32(16)).astype(np.uint16)


def _bf16_round(x):
    """f32 values rounded to the nearest bf16, as f32."""
    return (_bf16_bits(x).astype(np.uint32) << np.uint32(16)).view(np.float32)


class _GdnInputs:
    """Synthetic constants, state and T tokens of inputs of one Gated-DeltaNet layer at the step
    shape the metric names: A_log = 0, dt_bias = 0, norm weight 1, conv weights ~ N(0, 0.5) in bf16."""

    def __init__(self, seed, Hk, Hv, dk, dv, K=4, T=1, zero_state=False):
        rng = np.random.default_rng(seed)
        self.Hk, self.Hv, self.dk, self.dv, self.K, self.T = Hk, Hv, dk, dv, K, T
        self.C = C = 2 * Hk * dk + Hv * dv
        self.conv_w = _bf16_bits(rng.standard_normal(C * K) * 0.5)
        self.a_log = np.zeros(Hv, np.float32)
        self.dt_bias = _bf16_bits(np.zeros(Hv))
        self.norm_w = _bf16_bits(np.ones(dv))
        if zero_state:
            self.conv_state = np.zeros((K - 1) * C, np.float32)
            self.ssm_state = np.zeros(Hv * dv * dk, np.float32)
        else:
            self.conv_state = rng.standard_normal((K - 1) * C).astype(np.float32)
            self.ssm_state = (rng.standard_normal(Hv * dv * dk) * 0.02).astype(np.float32)
        self.qkv = rng.standard_normal((T, C)).astype(np.float32)
        self.z = rng.standard_normal((T, Hv * dv)).astype(np.float32)
        self.alpha = rng.standard_normal((T, Hv)).astype(np.float32)
        self.beta = rng.standard_normal((T, Hv)).astype(np.float32)


REPS = 11  # repetitions of the timed region; the median is reported


def _timed(ctx, lib, fn, steps, warmup, reps=REPS):
    """`warmup` untimed calls of fn(i), then `reps` repetitions of a timed region of exactly `steps`
    calls, each bracketed by a stream synchronisation on both sides.  Returns the medians over the
    repetitions of (wall ms per step, HIP-event ms per step); the events are recorded on the
    library's stream just inside the wall-clock bracket."""
    for i in range(warmup):
        fn(i)
    lib.mfa_sync(ctx.h)
    walls, evs = [], []
    ms = C.c_float(0)
    n = warmup
    for _ in range(reps):
        lib.mfa_sync(ctx.h)
        t0 = time.perf_counter()
        lib.mfa_timer_start(ctx.h)
        for i in range(n, n + steps):
            fn(i)
        rc = lib.mfa_timer_stop(ctx.h, C.byref(ms))  # records the end event and waits for it: the stream is idle
        wall = (time.perf_counter() - t0) * 1e3
        if rc != 0:
            raise RuntimeError("mfa_timer_stop failed")
        walls.append(wall / steps)
        evs.append(ms.value / steps)
        n += steps
    walls.sort()
    evs.sort()
    return walls[len(walls) // 2], evs[len(evs) // 2]


def bench_sdpa(name, Hq, Hkv, d, L, bf16, layers, steps, warmup, seed):
    from moeflux_amd import Config, Ctx, ffi
    from moeflux_amd.hip import DeviceArray
    lib = ffi.load()
    rng = np.random.default_rng(seed)
    kvd = Hkv * d
    qs = 1.0 / np.sqrt(d)
    ctx = Ctx(Config(num_layers=layers, full_attn_interval=1, num_attn_heads=Hq, num_kv_heads=Hkv,
                     head_dim=d, kv_capacity=L, kv_dtype=ffi.KV_BF16 if bf16 else ffi.KV_F32))
    # one long random sequence; layer l sees the window starting at row 8*l
    base_k = rng.standard_normal((L + 8 * layers, kvd), dtype=np.float32)
    base_v = rng.standard_normal((L + 8 * layers, kvd), dtype=np.float32)
    if bf16:
        base_k, base_v = _bf16_bits(base_k), _bf16_bits(base_v)
    else:
        base_k *= qs
        base_v *= qs
    for l in range(layers):
        ctx.kv_import(l, base_k[8 * l:8 * l + L], base_v[8 * l:8 * l + L])
    q = (rng.standard_normal((layers, Hq * d)) * qs).astype(np.float32)
    g = rng.standard_normal((layers, Hq * d)).astype(np.float32)
    dq, dg = DeviceArray.from_host(q), DeviceArray.from_host(g)
    dout = DeviceArray((layers, Hq * d), np.float32, zero=True)
    qd = Hq * d

    # argument tuples are built once: at a few microseconds per step the interpreter's own work counts
    call = lib.mfa_sdpa_decode_dev
    args = [(ctx.h, l, dq.offset(l * qd), dg.offset(l * qd), dout.offset(l * qd)) for l in range(layers)]

    def step(i):
        if call(*args[i % layers]) != 0:
            raise RuntimeError(ffi.last_error())

    wall_ms, ev_ms = _timed(ctx, lib, step, steps, warmup)
    out = dout.to_host()
    # the partial kernel alone (the kernel the roofline is stated for)
    lib.mfa_set_partial_only(ctx.h, 1)
    _, part_ms = _timed(ctx, lib, step, steps, warmup)
    lib.mfa_set_partial_only(ctx.h, 0)
    es = 2 if bf16 else 4
    alg_bytes = 2 * L * kvd * es + 3 * Hq * d * 4
    res = {
        "workload": name, "us_per_layer_token": wall_ms * 1e3, "us_event": ev_ms * 1e3,
        "us_partial_kernel_loop": part_ms * 1e3, "algorithmic_bytes": alg_bytes,
        "gbps": alg_bytes / (wall_ms * 1e-3) / 1e9,
        "gbps_partial_kernel": alg_bytes / (part_ms * 1e-3) / 1e9,
    }
    res["pct_peak"] = 100.0 * res["gbps"] / HBM_PEAK_GBPS
    sample = (q[0], g[0], base_k[:L], base_v[:L], out[0])
    ctx.close()
    for a in (dq, dg, dout):
        a.free()
    return res, sample


def bench_gdn(name, Hk, Hv, dk, dv, layers, steps, warmup, seed):
    from moeflux_amd import Config, Ctx, ffi
    from moeflux_amd.hip import DeviceArray
    lib = ffi.load()
    case = _GdnInputs(seed, Hk, Hv, dk, dv, T=1)
    ctx = Ctx(Config(num_layers=layers, full_attn_interval=layers + 1, linear_num_k_heads=Hk,
                     linear_num_v_heads=Hv, linear_key_dim=dk, linear_value_dim=dv))
    rng = np.random.default_rng(seed + 1)
    for l in range(layers):
        ctx.set_linear_weights(l, case.conv_w, case.a_log, case.dt_bias, case.norm_w)
        ctx.linear_state_import(l, case.conv_state,
                                (rng.standard_normal(Hv * dv * dk) * 0.02).astype(np.float32))
    C_, tv = case.C, Hv * dv
    dx = DeviceArray.from_host(rng.standard_normal((layers, C_)).astype(np.float32))
    dz = DeviceArray.from_host(rng.standard_normal((layers, tv)).astype(np.float32))
    da = DeviceArray.from_host(rng.standard_normal((layers, Hv)).astype(np.float32))
    db = DeviceArray.from_host(rng.standard_normal((layers, Hv)).astype(np.float32))
    dout = DeviceArray((layers, tv), np.float32, zero=True)

    call = lib.mfa_gdn_step_dev
    args = [(ctx.h, l, dx.offset(l * C_), dz.offset(l * tv), da.offset(l * Hv), db.offset(l * Hv), dout.offset(l * tv))
            for l in range(layers)]

    def step(i):
        if call(*args[i % layers]) != 0:
            raise RuntimeError(ffi.last_error())

    wall_ms, ev_ms = _timed(ctx, lib, step, steps, warmup)
    K = 4
    alg_bytes = 2 * Hv * dv * dk * 4 + 2 * (K - 1) * C_ * 4 + C_ * 4 + C_ * K * 2 + 2 * tv * 4 + 704
    res = {"workload": name, "us_per_layer_token": wall_ms * 1e3, "us_event": ev_ms * 1e3,
           "algorithmic_bytes": alg_bytes, "gbps": alg_bytes / (wall_ms * 1e-3) / 1e9}
    res["pct_peak"] = 100.0 * res["gbps"] / HBM_PEAK_GBPS
    ctx.close()
    for a in (dx, dz, da, db, dout):
        a.free()
    return res


def bench_prefill(steps, warmup, seed, T=512):
    """A 512-token prompt chunk from an empty cache / zero state —
    causal GQA attention (32 Q / 4 KV heads, d=128, bf16 cache) and the Gated-DeltaNet
    chunk (configs[1] shape).  Every timed call uses a fresh layer, so kv_len0 = 0."""
    from moeflux_amd import Config, Ctx, ffi
    from moeflux_amd.hip import DeviceArray
    lib = ffi.load()
    Hq, Hkv, d = 32, 4, 128
    n = REPS * steps + warmup
    rng = np.random.default_rng(seed)
    ctx = Ctx(Config(num_layers=n, full_attn_interval=1, num_attn_heads=Hq, num_kv_heads=Hkv,
                     head_dim=d, kv_capacity=T, kv_dtype=ffi.KV_BF16))
    dq = DeviceArray.from_host((rng.standard_normal((T, Hq * d)) / np.sqrt(d)).astype(np.float32))
    dg = DeviceArray.from_host(rng.standard_normal((T, Hq * d)).astype(np.float32))
    dk = DeviceArray.from_host(rng.standard_normal((T, Hkv * d)).astype(np.float32))
    dv = DeviceArray.from_host(rng.standard_normal((T, Hkv * d)).astype(np.float32))
    do = DeviceArray((T, Hq * d), np.float32, zero=True)
    layer = [0]

    def step(i):
        rc = lib.mfa_prefill_attn_dev(ctx.h, layer[0], T, dq.ptr, dg.ptr, dk.ptr, dv.ptr, do.ptr)
        layer[0] += 1
        if rc != 0:
            raise RuntimeError(ffi.last_error())

    wall_ms, ev_ms = _timed(ctx, lib, step, steps, warmup)
    flops = 2 * 2 * Hq * (T * (T + 1) // 2) * d
    res = {"attention_us_per_chunk": ev_ms * 1e3, "attention_causal_flop": flops,
           "attention_tflops": flops / (ev_ms * 1e-3) / 1e12,
           "attention_us_per_token_layer": ev_ms * 1e3 / T}
    ctx.close()
    # The same chunk with a query that is exact in bf16 (what a bf16 model hands over, and what
    # the configuration's "bf16" says): its low parts are zero and the kernel leaves their products out.
    dqb = DeviceArray.from_host(_bf16_round((rng.standard_normal((T, Hq * d)) / np.sqrt(d)).astype(np.float32)))
    ctx = Ctx(Config(num_layers=n, full_attn_interval=1, num_attn_heads=Hq, num_kv_heads=Hkv,
                     head_dim=d, kv_capacity=T, kv_dtype=ffi.KV_BF16))
    layer[0] = 0
    dq, dq_f32 = dqb, dq
    wall_ms, ev_ms = _timed(ctx, lib, step, steps, warmup)
    res["attention_bf16_query_us_per_chunk"] = ev_ms * 1e3
    dq = dq_f32
    ctx.close()

    # The same chunk behind a context of 32768 cached positions (a long prompt taken in chunks):
    # the rows now share 1040 cache blocks instead of at most 16, which is the size at which the
    # kernel's matrix work dominates.  Every call appends its 512 rows again after a truncation
    # (outside the timed region).
    L0 = 32768
    ctx = Ctx(Config(num_layers=1, full_attn_interval=1, num_attn_heads=Hq, num_kv_heads=Hkv,
                     head_dim=d, kv_capacity=L0 + T, kv_dtype=ffi.KV_BF16))
    kv0 = rng.standard_normal((L0, Hkv * d), dtype=np.float32)
    ctx.kv_import(0, kv0, kv0)
    cflops = 2 * 2 * Hq * (T * L0 + T * (T + 1) // 2) * d
    # the probabilities enter as two bf16 parts, and so does a query that is not exact in bf16:
    # matrix instructions per (score, value) product pair
    for key, qdev, instr in (("attention_after_32768_positions", dq, 4), ("attention_after_32768_positions_bf16_query", dqb, 3)):
        ms, times = C.c_float(0), []
        for i in range(4 + min(steps, 20)):
            ctx.memory_seq_rm(L0)
            lib.mfa_sync(ctx.h)
            lib.mfa_timer_start(ctx.h)
            if lib.mfa_prefill_attn_dev(ctx.h, 0, T, qdev.ptr, dg.ptr, dk.ptr, dv.ptr, do.ptr) != 0:
                raise RuntimeError(ffi.last_error())
            lib.mfa_timer_stop(ctx.h, C.byref(ms))
            if i >= 4:
                times.append(ms.value)
        med = sorted(times)[len(times) // 2]
        res[key] = {
            "us_per_chunk": med * 1e3, "flop": cflops, "tflops": cflops / (med * 1e-3) / 1e12,
            "matrix_tflops": instr / 2 * cflops / (med * 1e-3) / 1e12,
            "pct_of_bf16_peak": 100 * instr / 2 * cflops / (med * 1e-3) / 2.5e15}
    ctx.close()
    for a in (dq, dqb, dg, dk, dv, do):
        a.free()

    case = _GdnInputs(seed, 16, 32, 128, 128, T=T, zero_state=True)
    layers = 8
    ctx = Ctx(Config(num_layers=layers, full_attn_interval=layers + 1, linear_num_k_heads=16,
                     linear_num_v_heads=32))
    for l in range(layers):
        ctx.set_linear_weights(l, case.conv_w, case.a_log, case.dt_bias, case.norm_w)
    dx, dz = DeviceArray.from_host(case.qkv), DeviceArray.from_host(case.z)
    da, db = DeviceArray.from_host(case.alpha), DeviceArray.from_host(case.beta)
    do = DeviceArray((T, 32 * 128), np.float32, zero=True)

    def gstep(i):
        rc = lib.mfa_prefill_gdn_dev(ctx.h, i % layers, T, dx.ptr, dz.ptr, da.ptr, db.ptr, do.ptr)
        if rc != 0:
            raise RuntimeError(ffi.last_error())

    wall_ms, ev_ms = _timed(ctx, lib, gstep, steps, warmup)
    gflops = 7 * 128 * 128 * 32 * T
    res.update({"deltanet_us_per_chunk": ev_ms * 1e3, "deltanet_sequential_equivalent_flop": gflops,
                "deltanet_tflops": gflops / (ev_ms * 1e-3) / 1e12,
                "deltanet_us_per_token_layer": ev_ms * 1e3 / T})
    ctx.close()
    for a in (dx, dz, da, db, do):
        a.free()
    return res


def bench_sweep(steps, warmup, seed):
    """The attention launches of one token over a 48-layer hybrid stack,
    36 Gated-DeltaNet layers (configs[1] shape) and 12 gated full-attention layers
    (32 Q / 2 KV heads, d=256, kv_len 8192, bf16), distinct buffers per layer, in layer order
    on one stream (mfa_token_sweep_dev)."""
    from moeflux_amd import Config, Ctx, ffi
    from moeflux_amd.hip import DeviceArray
    lib = ffi.load()
    NL, Hq, Hkv, d, L = 48, 32, 2, 256, 8192
    cfg = Config(num_layers=NL, full_attn_interval=4, num_attn_heads=Hq, num_kv_heads=Hkv, head_dim=d,
                 kv_capacity=L, kv_dtype=ffi.KV_BF16, linear_num_k_heads=16, linear_num_v_heads=32)
    ctx = Ctx(cfg)
    rng = np.random.default_rng(seed)
    case = _GdnInputs(seed, 16, 32, 128, 128, T=1)
    base_k = _bf16_bits(rng.standard_normal((L + 8 * 12, Hkv * d), dtype=np.float32))
    base_v = _bf16_bits(rng.standard_normal((L + 8 * 12, Hkv * d), dtype=np.float32))
    nf = nl = 0
    for i in range(NL):
        if cfg.is_full(i):
            ctx.kv_import(i, base_k[8 * nf:8 * nf + L], base_v[8 * nf:8 * nf + L])
            nf += 1
        else:
            ctx.set_linear_weights(i, case.conv_w, case.a_log, case.dt_bias, case.norm_w)
            ctx.linear_state_import(i, case.conv_state,
                                    (rng.standard_normal(32 * 128 * 128) * 0.02).astype(np.float32))
            nl += 1
    qd, C_, tv = Hq * d, case.C, 32 * 128
    fq = DeviceArray.from_host((rng.standard_normal((nf, qd)) / 16).astype(np.float32))
    fg = DeviceArray.from_host(rng.standard_normal((nf, qd)).astype(np.float32))
    fo = DeviceArray((nf, qd), np.float32, zero=True)
    lx = DeviceArray.from_host(rng.standard_normal((nl, C_)).astype(np.float32))
    lz = DeviceArray.from_host(rng.standard_normal((nl, tv)).astype(np.float32))
    la = DeviceArray.from_host(rng.standard_normal((nl, 32)).astype(np.float32))
    lb = DeviceArray.from_host(rng.standard_normal((nl, 32)).astype(np.float32))
    lo = DeviceArray((nl, tv), np.float32, zero=True)

    def step(i):
        rc = lib.mfa_token_sweep_dev(ctx.h, fq.ptr, fg.ptr, fo.ptr, lx.ptr, lz.ptr, la.ptr, lb.ptr, lo.ptr)
        if rc != 0:
            raise RuntimeError(ffi.last_error())

    alg = 36 * 4522688 + 12 * (2 * L * Hkv * d * 2 + 3 * qd * 4)
    res = {"layers": NL, "algorithmic_bytes": alg}
    # "per_kind": the 36 DeltaNet layers in one launch and the 12 full-attention layers in
    # one split-K launch + merge (all inputs of the token are known up front);
    # "per_layer": the 48 launch chains one after another, what a caller whose layers
    # depend on each other pays.
    samples = {}
    for name, per_layer in (("per_kind", 0), ("per_layer", 1)):
        if lib.mfa_set_sweep_per_layer(ctx.h, per_layer) != 0:
            raise RuntimeError(ffi.last_error())
        wall_ms, ev_ms = _timed(ctx, lib, step, steps, warmup)
        gbps = alg / (wall_ms * 1e-3) / 1e9
        res[name] = {"us_per_token_sweep": wall_ms * 1e3, "us_event": ev_ms * 1e3,
                     "us_per_layer_token": wall_ms * 1e3 / NL, "gbps": gbps,
                     "pct_peak": 100.0 * gbps / HBM_PEAK_GBPS,
                     "pct_peak_event": 100.0 * alg / (ev_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS}
        # one more sweep from a known state of the first DeltaNet layer, kept for the check against
        # the CPU oracle (cpu_secondary): the first full-attention layer's and that layer's outputs
        s0 = (rng.standard_normal(32 * 128 * 128) * 0.02).astype(np.float32)
        for i in range(NL):   # every layer, so that all conv rings stand at the same slot again
            if not cfg.is_full(i):
                ctx.linear_state_import(i, case.conv_state, s0)
        step(0)
        ctx.sync()
        samples[name] = {"full_out": fo.to_host()[0], "lin_out": lo.to_host()[0], "ssm0": s0}
    sample = {"modes": samples, "q": fq.to_host()[0], "g": fg.to_host()[0], "k": base_k[:L], "v": base_v[:L],
              "case": case, "x": lx.to_host()[0], "z": lz.to_host()[0], "a": la.to_host()[0], "b": lb.to_host()[0],
              "shape": (Hq, Hkv, d, L)}
    ctx.close()
    for a in (fq, fg, fo, lx, lz, la, lb, lo):
        a.free()
    return res, sample


def calibrate_copy(nbytes=64 << 20, reps=20):
    """`--calibrate-copy`: launch only the plain copy kernel (nbytes read + nbytes written per
    launch), for scaling rocprofv3 FETCH_SIZE / WRITE_SIZE readings."""
    from moeflux_amd import Config, Ctx, ffi
    from moeflux_amd.hip import DeviceArray
    lib = ffi.load()
    ctx = Ctx(Config(num_layers=1, full_attn_interval=2, linear_num_k_heads=1, linear_num_v_heads=1))
    bufs = [DeviceArray((nbytes,), np.uint8, zero=True) for _ in range(8)]
    for i in range(reps):
        lib.mfa_debug_copy_dev(ctx.h, bufs[4 + i % 4].ptr, bufs[i % 4].ptr, nbytes)
    ctx.sync()
    ctx.close()
    print(json.dumps({"copy_kernel": "plain_copy_kernel", "bytes_read_per_launch": nbytes,
                      "bytes_written_per_launch": nbytes, "launches": reps}))


def calibrate_read(nbytes=64 << 20, reps=200):
    """`--calibrate-read`: launches that only read 64 MiB (mfa_debug_read_dev), rotating over 8 buffers,
    for several workgroup counts: what the memory system allows a launch of the headline kernel's size."""
    from moeflux_amd import Config, Ctx, ffi
    from moeflux_amd.hip import DeviceArray
    lib = ffi.load()
    ctx = Ctx(Config(num_layers=1, full_attn_interval=2, linear_num_k_heads=1, linear_num_v_heads=1))
    bufs = [DeviceArray((nbytes,), np.uint8, zero=True) for _ in range(8)]
    out = {"bytes_read_per_launch": nbytes, "launches_per_figure": reps, "by_workgroups": {}}
    for wgs in (256, 512, 1024, 2048, 4096):
        def step(i, wgs=wgs):
            if lib.mfa_debug_read_dev(ctx.h, bufs[i % 8].ptr, nbytes, wgs) != 0:
                raise RuntimeError(ffi.last_error())
        _, ev_ms = _timed(ctx, lib, step, reps, 20, reps=5)
        out["by_workgroups"][str(wgs)] = {"us_per_launch": ev_ms * 1e3, "gbps": nbytes / (ev_ms * 1e-3) / 1e9,
                                          "pct_peak": 100.0 * nbytes / (ev_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS}
    best = min(out["by_workgroups"].values(), key=lambda r: r["us_per_launch"])
    out["best_us_per_launch"] = best["us_per_launch"]
    out["best_pct_peak"] = best["pct_peak"]
    ctx.close()
    print(json.dumps(out))


def cpu_baseline(sample, Hq, Hkv, d, L, budget_s=12.0):
    """The CPU oracle (a port of the reference's scalar sdpa_cpu, which is what the
    reference itself runs at kv_len >= 8192), one thread, f32 cache, same inputs."""
    from oracle import cref
    q, g, k, v, gpu_out = sample
    kf = cref.bf16_to_f32(k) if k.dtype == np.uint16 else k
    vf = cref.bf16_to_f32(v) if v.dtype == np.uint16 else v
    t0 = time.perf_counter()
    ref = cref.sdpa(L, Hq, Hkv, d, q, g, kf, vf)
    first = time.perf_counter() - t0
    n = int(max(1, min(60, budget_s / max(first, 1e-3))))
    t0 = time.perf_counter()
    for _ in range(n):
        cref.sdpa(L, Hq, Hkv, d, q, g, kf, vf)
    per = (time.perf_counter() - t0) / n
    err = float(np.abs(gpu_out - ref).max() / np.abs(ref).max())
    return {"value": per * 1e6, "unit": "us/layer/token", "cores": 1, "kind": "port",
            "sample": f"{n} calls of the oracle's orc_sdpa at the full workload shape "
                      f"(kv_len {L}, f32-widened cache), single thread"}, err


def bench_matvec(steps, warmup, seed):
    """The projections either side of the attention core at the A17B variant's shapes
    (variants.rs:384-400): q, k and v projections of a full-attention layer in one launch
    ([16384 + 512 + 512, 4096] 4-bit group-64 weights) and o_proj ([4096, 8192]); weight sets
    rotated so that every launch reads its weights from HBM."""
    import ctypes as C
    from moeflux_amd import Config, Ctx, ffi
    from moeflux_amd.hip import DeviceArray
    lib = ffi.load()
    ctx = Ctx(Config(num_layers=1, full_attn_interval=1, num_attn_heads=8, num_kv_heads=2, head_dim=64, kv_capacity=4))
    rng = np.random.default_rng(seed)
    res, keep = {}, []

    def weights(od, idim):
        w = DeviceArray.from_host(rng.integers(0, 2 ** 32, size=(od, idim // 8), dtype=np.uint64).astype(np.uint32))
        sc = DeviceArray.from_host(np.full((od, idim // 64), 0x3C00, np.uint16))
        bi = DeviceArray.from_host(np.full((od, idim // 64), 0xBD00, np.uint16))
        keep.extend([w, sc, bi])
        return w, sc, bi

    for name, shapes, idim, nsets in (("qkv_proj", (16384, 512, 512), 4096, 8), ("o_proj", (4096,), 8192, 14)):
        x = DeviceArray.from_host(rng.standard_normal(idim).astype(np.float32))
        keep.append(x)
        sets = []
        for _ in range(nsets):
            specs = (ffi.mfa_matvec_spec * len(shapes))()
            for i, od in enumerate(shapes):
                w, sc, bi = weights(od, idim)
                o = DeviceArray((od,), np.float32, zero=True)
                keep.append(o)
                specs[i] = ffi.mfa_matvec_spec(w.ptr, sc.ptr, bi.ptr, x.ptr, o.ptr, od, idim)
            sets.append(specs)

        def step(i, sets=sets, n=len(shapes)):
            if lib.mfa_dequant_matvec_4bit_dev(ctx.h, n, C.byref(sets[i % len(sets)])) != 0:
                raise RuntimeError(ffi.last_error())

        wall_ms, ev_ms = _timed(ctx, lib, step, steps, warmup)
        nw = sum(shapes) * idim
        alg = nw // 2 + (nw // 64) * 4 + idim * 4 + sum(shapes) * 4
        res[name] = {"shapes": [[od, idim] for od in shapes], "us_per_launch": ev_ms * 1e3, "algorithmic_bytes": alg,
                     "gbps": alg / (ev_ms * 1e-3) / 1e9, "pct_peak": 100.0 * alg / (ev_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS}
        # the same products over weights re-ordered at load time (mfa_matvec_tile_weights_dev)
        tsets = []
        for specs in sets:
            tspecs = (ffi.mfa_matvec_spec * len(shapes))()
            for i, od in enumerate(shapes):
                tw = DeviceArray((int(lib.mfa_matvec_tiled_words(od, idim)),), np.uint32)
                keep.append(tw)
                if lib.mfa_matvec_tile_weights_dev(ctx.h, od, idim, specs[i].w_packed, specs[i].scales, specs[i].biases, tw.ptr) != 0:
                    raise RuntimeError(ffi.last_error())
                sp = specs[i]
                tspecs[i] = ffi.mfa_matvec_spec(tw.ptr, None, None, sp.x, sp.out, od, idim)
            tsets.append(tspecs)

        def tstep(i, tsets=tsets, n=len(shapes)):
            if lib.mfa_dequant_matvec_4bit_tiled_dev(ctx.h, n, C.byref(tsets[i % len(tsets)])) != 0:
                raise RuntimeError(ffi.last_error())

        wall_ms, ev_ms = _timed(ctx, lib, tstep, steps, warmup)
        res[name]["tiled_weights_us_per_launch"] = ev_ms * 1e3
        res[name]["tiled_weights_pct_peak"] = 100.0 * alg / (ev_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS
    ctx.close()
    for a in keep:
        a.free()
    return res


def bench_prologue(steps, warmup, seed):
    """What precedes the attention core in a full-attention layer, at the headline shape (32 Q /
    2 KV heads, head_dim 256, bf16 caches holding 32768 positions, 8 layers rotated over like the
    headline's caches): the prologue alone (q/gate split, per-head norms, rotation, cache append -
    one launch) and the whole layer step from the raw projections (mfa_full_attn_step_dev) in its
    two forms: two launches (the attention launch norms and rotates its own query heads and
    appends the token, the merge takes the token as one more split) and three (prologue,
    attention, merge).  Every call appends a position; the caches start short of 32768 by the
    number of calls, so that the three measurements run up to the headline's length and not past
    it.  One more measurement continues from there: just past a length at which every workgroup
    has one whole pass, the plan changes to half as many workgroups with two passes each."""
    from moeflux_amd import Config, Ctx, ffi
    from moeflux_amd.hip import DeviceArray
    lib = ffi.load()
    Hq, Hkv, d, L, NL = 32, 2, 256, 32768, 8
    per_run = (REPS * steps + warmup + NL - 1) // NL + 1     # positions a measurement adds to a layer
    L0 = L - 3 * per_run
    ctx = Ctx(Config(num_layers=NL, full_attn_interval=1, num_attn_heads=Hq, num_kv_heads=Hkv, head_dim=d,
                     kv_capacity=L + per_run, kv_dtype=ffi.KV_BF16))
    rng = np.random.default_rng(seed)
    kv = _bf16_bits(rng.standard_normal((L0, Hkv * d), dtype=np.float32))
    w = _bf16_bits(np.ones(d, np.float32))
    for l in range(NL):
        ctx.kv_import(l, kv, kv)
        ctx.set_full_weights(l, w, w)
    qp = DeviceArray.from_host(rng.standard_normal(2 * Hq * d).astype(np.float32))
    k = DeviceArray.from_host(rng.standard_normal(Hkv * d).astype(np.float32))
    v = DeviceArray.from_host(rng.standard_normal(Hkv * d).astype(np.float32))
    q, g, o = (DeviceArray((Hq * d,), np.float32, zero=True) for _ in range(3))
    pos = [L0] * NL

    def pro(i):
        l = i % NL
        if lib.mfa_attn_prologue_dev(ctx.h, l, pos[l], qp.ptr, k.ptr, v.ptr, q.ptr, g.ptr) != 0:
            raise RuntimeError(ffi.last_error())
        pos[l] += 1

    def full(i):
        l = i % NL
        if lib.mfa_full_attn_step_dev(ctx.h, l, pos[l], qp.ptr, k.ptr, v.ptr, o.ptr) != 0:
            raise RuntimeError(ffi.last_error())
        pos[l] += 1

    lib.mfa_set_step_launches(ctx.h, 3)
    _, full3_ms = _timed(ctx, lib, full, steps, warmup)
    lib.mfa_set_step_launches(ctx.h, 2)
    _, full2_ms = _timed(ctx, lib, full, steps, warmup)
    _, pro_ms = _timed(ctx, lib, pro, steps, warmup)
    if max(pos) > L:
        raise RuntimeError("the step measurements ran past %d positions" % L)
    for l in range(NL):      # on from the headline's length exactly
        while pos[l] < L:
            full(l)
    _, past_ms = _timed(ctx, lib, full, steps, warmup)
    alg = 2 * Hq * d * 4 + 2 * Hkv * d * 4 + 2 * Hq * d * 4 + 2 * Hkv * d * 2
    res = {"shape": "32 Q / 2 KV heads, head_dim 256, bf16 caches growing to 32768 positions (from %d), 8 layers rotated over" % L0,
           "prologue_us_per_call": pro_ms * 1e3, "prologue_algorithmic_bytes": alg,
           "full_attn_step_us_per_call": full2_ms * 1e3, "launches_per_full_step": 2,
           "full_attn_step_three_launches_us_per_call": full3_ms * 1e3,
           "full_attn_step_past_32768_positions_us_per_call": past_ms * 1e3}
    ctx.close()
    for a in (qp, k, v, q, g, o):
        a.free()
    return res


def bench_snapshot(seed):
    """The 'MFLX' snapshot of a 48-layer hybrid stack (36 DeltaNet layers, 12 full-attention layers
    with 2048 cached positions each): bytes, and the time to save it to and load it from host
    memory (device reads and writes, conversion from and to the tiled cache, PCIe both ways);
    beside it the same state stored and restored as a device-resident checkpoint."""
    from moeflux_amd import Config, Ctx, ffi
    lib = ffi.load()
    NL, Hq, Hkv, d, L = 48, 32, 2, 256, 2048
    ctx = Ctx(Config(num_layers=NL, full_attn_interval=4, num_attn_heads=Hq, num_kv_heads=Hkv, head_dim=d,
                     kv_capacity=L, kv_dtype=ffi.KV_BF16, linear_num_k_heads=16, linear_num_v_heads=32))
    rng = np.random.default_rng(seed)
    kv = _bf16_bits(rng.standard_normal((L, Hkv * d), dtype=np.float32))
    for i in range(NL):
        if (i + 1) % 4 == 0:
            ctx.kv_import(i, kv, kv)
    size = ctx.state_size()
    buf = np.empty(size, np.uint8)
    p = buf.ctypes.data_as(C.c_void_p)
    times = {"save": [], "load": []}
    for _ in range(3):
        t0 = time.perf_counter()
        nbytes = lib.mfa_state_save(ctx.h, p, size)
        times["save"].append(time.perf_counter() - t0)
        if nbytes != size:
            raise RuntimeError("mfa_state_save: %d of %d bytes" % (nbytes, size))
        t0 = time.perf_counter()
        if lib.mfa_state_load(ctx.h, p, size) != 0:
            raise RuntimeError(ffi.last_error())
        lib.mfa_sync(ctx.h)
        times["load"].append(time.perf_counter() - t0)
    # the same through a page-locked buffer of the library's (mfa_host_alloc)
    pin = lib.mfa_host_alloc(size)
    if not pin:
        raise RuntimeError(ffi.last_error())
    times["save_pinned"], times["load_pinned"] = [], []
    for _ in range(3):
        t0 = time.perf_counter()
        nbytes = lib.mfa_state_save(ctx.h, pin, size)
        times["save_pinned"].append(time.perf_counter() - t0)
        if nbytes != size:
            raise RuntimeError("mfa_state_save: %d of %d bytes" % (nbytes, size))
        t0 = time.perf_counter()
        if lib.mfa_state_load(ctx.h, pin, size) != 0:
            raise RuntimeError(ffi.last_error())
        lib.mfa_sync(ctx.h)
        times["load_pinned"].append(time.perf_counter() - t0)
    if C.string_at(pin, size) != buf.tobytes():
        raise RuntimeError("snapshot through the page-locked buffer differs")
    lib.mfa_host_free(pin)
    # the same state as a checkpoint kept on the device (mfa_checkpoint_pos / mfa_restore_to)
    times["checkpoint"], times["restore"] = [], []
    for _ in range(3):
        t0 = time.perf_counter()
        if lib.mfa_checkpoint_pos(ctx.h, L) != 0:
            raise RuntimeError(ffi.last_error())
        times["checkpoint"].append(time.perf_counter() - t0)
        t0 = time.perf_counter()
        if lib.mfa_restore_to(ctx.h, L) != 0:
            raise RuntimeError(ffi.last_error())
        times["restore"].append(time.perf_counter() - t0)
    ctx.close()
    return {"layers": NL, "kv_len": L, "bytes": size, "save_ms": min(times["save"]) * 1e3,
            "load_ms": min(times["load"]) * 1e3, "save_gbps": size / min(times["save"]) / 1e9,
            "load_gbps": size / min(times["load"]) / 1e9,
            "save_pinned_ms": min(times["save_pinned"]) * 1e3, "load_pinned_ms": min(times["load_pinned"]) * 1e3,
            "save_pinned_gbps": size / min(times["save_pinned"]) / 1e9,
            "load_pinned_gbps": size / min(times["load_pinned"]) / 1e9,
            "device_checkpoint_ms": min(times["checkpoint"]) * 1e3,
            "device_restore_ms": min(times["restore"]) * 1e3}


def bench_mla(steps, warmup, seed, lens=(4096, 32768)):
    """Attention of one token over a latent cache at the MLA variants' shape (128 heads,
    kv_lora_rank 512, qk_rope_head_dim 64; variants.rs), f32 caches, cache sets rotated."""
    from moeflux_amd import Config, Ctx, ffi
    from moeflux_amd.hip import DeviceArray
    lib = ffi.load()
    H, R, P = 128, 512, 64
    ctx = Ctx(Config(num_layers=1, full_attn_interval=1, num_attn_heads=8, num_kv_heads=2, head_dim=64, kv_capacity=4))
    rng = np.random.default_rng(seed)
    res = {}
    qp = DeviceArray.from_host(rng.standard_normal((H, R), dtype=np.float32) * 0.1)
    qe = DeviceArray.from_host(rng.standard_normal((H, P), dtype=np.float32) * 0.1)
    out = DeviceArray((H * R,), np.float32, zero=True)
    for L in lens:
        nsets = 4
        sets = [(DeviceArray.from_host(rng.standard_normal((L, R), dtype=np.float32)),
                 DeviceArray.from_host(rng.standard_normal((L, P), dtype=np.float32))) for _ in range(nsets)]

        def step(i, sets=sets, L=L):
            lat, rk = sets[i % len(sets)]
            if lib.mfa_mla_sdpa_folded_dev(ctx.h, H, R, P, L, C.c_float(1.0 / np.sqrt(192.0)), qp.ptr, qe.ptr,
                                           lat.ptr, rk.ptr, out.ptr) != 0:
                raise RuntimeError(ffi.last_error())

        _, ev_ms = _timed(ctx, lib, step, steps, warmup)
        flops = 2.0 * H * L * (R + P + R)        # the two products, once
        alg = L * (R + P) * 4 + 2 * H * R * 4 + H * P * 4
        sec = ev_ms * 1e-3
        res[f"L{L}"] = {"us_per_call": ev_ms * 1e3, "flops": flops, "tflops": flops / sec / 1e12,
                        # every product is three bf16 partial products on the matrix pipeline
                        "bf16_mfma_flops_issued": 3 * flops,
                        "pct_bf16_mfma_peak": 100.0 * 3 * flops / sec / 1e12 / 2500.0,
                        "algorithmic_bytes": alg, "gbps": alg / sec / 1e9,
                        "pct_hbm_peak": 100.0 * alg / sec / 1e9 / HBM_PEAK_GBPS}
        for lat, rk in sets:
            lat.free(); rk.free()
    ctx.close()
    for a in (qp, qe, out):
        a.free()
    return res


def cpu_baseline_all_cores(sample, Hq, Hkv, d, L):
    """The same oracle function with the query heads spread over the host cores this process
    may use (heads are independent; the reference's own CPU path is single-threaded)."""
    import os
    from concurrent.futures import ThreadPoolExecutor
    from oracle import cref
    q, g, k, v, _ = sample
    kf = (cref.bf16_to_f32(k) if k.dtype == np.uint16 else k).reshape(L, Hkv, d)
    vf = (cref.bf16_to_f32(v) if v.dtype == np.uint16 else v).reshape(L, Hkv, d)
    cores = max(1, min(len(os.sched_getaffinity(0)), 16, Hq))
    kh = [np.ascontiguousarray(kf[:, h]) for h in range(Hkv)]
    vh = [np.ascontiguousarray(vf[:, h]) for h in range(Hkv)]
    hpk = Hq // Hkv
    qs, gs = q.reshape(Hq, d), g.reshape(Hq, d)

    def one(h):  # ctypes drops the GIL for the duration of the call
        return cref.sdpa(L, 1, 1, d, qs[h], gs[h], kh[h // hpk], vh[h // hpk])

    with ThreadPoolExecutor(cores) as ex:
        list(ex.map(one, range(Hq)))
        t0 = time.perf_counter()
        n = 3
        for _ in range(n):
            list(ex.map(one, range(Hq)))
        per = (time.perf_counter() - t0) / n
    return {"value": per * 1e6, "unit": "us/layer/token", "cores": cores, "kind": "port",
            "sample": f"{n} calls, the {Hq} query heads of orc_sdpa spread over {cores} threads"}


def cpu_secondary(sweep_sample=None):
    """One-thread oracle timings of the secondary configurations, same shapes, bounded samples;
    with a sample of the 48-layer sweep (inputs and GPU outputs of its first full-attention and
    first DeltaNet layer), the GPU outputs' error against the oracle on those inputs."""
    from oracle import cref
    rng = np.random.default_rng(1)

    def timed(fn, n):
        fn()
        t0 = time.perf_counter()
        for _ in range(n):
            fn()
        return (time.perf_counter() - t0) / n * 1e6

    def sdpa_inputs(Hq, Hkv, d, L):
        return (rng.standard_normal(Hq * d, dtype=np.float32), rng.standard_normal(Hq * d, dtype=np.float32),
                rng.standard_normal((L, Hkv * d), dtype=np.float32), rng.standard_normal((L, Hkv * d), dtype=np.float32))

    out = {}
    q, g, k, v = sdpa_inputs(32, 4, 128, 4096)
    out["c1_us_per_layer_token"] = timed(lambda: cref.sdpa(4096, 32, 4, 128, q, g, k, v), 5)
    c = _GdnInputs(2, 16, 32, 128, 128, T=1)
    step = lambda: cref.gdn_step(16, 32, 128, 128, 4, 1e-6, c.conv_w, c.a_log, c.dt_bias, c.norm_w, c.qkv[0],
                                 c.z[0], c.alpha[0], c.beta[0], c.conv_state, c.ssm_state)
    out["c2_us_per_layer_token"] = timed(step, 20)
    T = 512
    qq = rng.standard_normal((T, 32 * 128), dtype=np.float32)
    kk = rng.standard_normal((T, 4 * 128), dtype=np.float32)
    out["c4_attention_us_per_chunk"] = timed(lambda: cref.prefill_attn(T, 0, 32, 4, 128, qq, qq, kk, kk), 1)
    out["c4_deltanet_us_per_chunk"] = out["c2_us_per_layer_token"] * T
    q, g, k, v = sdpa_inputs(32, 2, 256, 8192)
    full = timed(lambda: cref.sdpa(8192, 32, 2, 256, q, g, k, v), 3)
    out["c5_us_per_token_sweep"] = 36 * out["c2_us_per_layer_token"] + 12 * full
    if sweep_sample is not None:
        sm = sweep_sample
        Hq, Hkv, d, L = sm["shape"]
        ref_f = cref.sdpa(L, Hq, Hkv, d, sm["q"], sm["g"], cref.bf16_to_f32(sm["k"]), cref.bf16_to_f32(sm["v"]))
        cs = sm["case"]
        chk = {}
        for mode, o in sm["modes"].items():
            ref_l, _, _ = cref.gdn_step(cs.Hk, cs.Hv, cs.dk, cs.dv, cs.K, 1e-6, cs.conv_w, cs.a_log, cs.dt_bias,
                                        cs.norm_w, sm["x"], sm["z"], sm["a"], sm["b"], cs.conv_state, o["ssm0"])
            chk[mode] = {"full_layer_rel_err": float(np.abs(o["full_out"] - ref_f).max() / np.abs(ref_f).max()),
                         "deltanet_layer_rel_err": float(np.abs(o["lin_out"] - ref_l).max() / np.abs(ref_l).max())}
        out["c5_gpu_vs_oracle"] = chk
    out["cores"] = 1
    out["kind"] = "port"
    out["sample"] = ("oracle functions at the full shapes: c1 5 calls, c2 20 calls, c4 attention one 512-token "
                     "chunk, c4 DeltaNet = 512 x the c2 step, c5 = 36 x the c2 step + 12 x orc_sdpa at kv_len 8192 (3 calls)")
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--layers", type=int, default=8, help="independent KV caches rotated over")
    ap.add_argument("--no-extra", action="store_true", help="skip the secondary configurations")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="launch only the plain copy kernel (for scaling memory counters) and exit")
    ap.add_argument("--calibrate-read", action="store_true",
                    help="time launches that only read 64 MiB (the memory system's ceiling at the headline launch size) and exit")
    ap.add_argument("--tokens", type=int, default=512, help="chunk length for --only c4")
    ap.add_argument("--f4-len", type=int, default=0, help="one cache length for --only f4 (default: 4096 and 32768)")
    ap.add_argument("--only", choices=["c1", "c2", "c4", "c5", "f1", "f2", "f3", "f4"], default=None,
                    help="run one secondary configuration alone (for profiling) and print its figures")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py: this path is measured on one GPU only (batch-1 decode attention on one "
              "device); run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    if a.calibrate_copy:
        calibrate_copy()
        return
    if a.calibrate_read:
        calibrate_read()
        return

    if a.only == "c1":
        r, _ = bench_sdpa("c1", 32, 4, 128, 4096, False, 24, a.steps, a.warmup, 0xC0FFEE + 1)
        print(json.dumps({"c1_gqa_decode_f32_L4096": r}))
        return
    if a.only == "c2":
        print(json.dumps({"c2_gated_deltanet_step": bench_gdn("c2", 16, 32, 128, 128, 160, a.steps, a.warmup, 0xC0FFEE + 2)}))
        return
    if a.only == "c4":
        print(json.dumps({f"c4_prefill_chunk_{a.tokens}": bench_prefill(a.steps, a.warmup, 0xC0FFEE + 4, a.tokens)}))
        return
    if a.only == "f1":
        print(json.dumps({"f1_attention_prologue": bench_prologue(a.steps, a.warmup, 0xC0FFEE + 8)}))
        return
    if a.only == "f2":
        print(json.dumps({"f2_state_snapshot": bench_snapshot(0xC0FFEE + 9)}))
        return
    if a.only == "f3":
        print(json.dumps({"f3_projection_matvecs": bench_matvec(a.steps, a.warmup, 0xC0FFEE + 6)}))
        return
    if a.only == "f4":
        lens = (a.f4_len,) if a.f4_len else (4096, 32768)
        print(json.dumps({"f4_mla_folded_sdpa": bench_mla(a.steps, a.warmup, 0xC0FFEE + 7, lens)}))
        return
    if a.only == "c5":
        r, sm = bench_sweep(a.steps, a.warmup, 0xC0FFEE + 5)
        if not a.no_cpu:
            r["gpu_vs_oracle"] = cpu_secondary(sm)["c5_gpu_vs_oracle"]
        print(json.dumps({"c5_token_sweep_48_layers": r}))
        return

    Hq, Hkv, d, L = 32, 2, 256, 32768
    head, sample = bench_sdpa("c3", Hq, Hkv, d, L, True, a.layers, a.steps, a.warmup, 0xC0FFEE + 3)
    line = {
        "metric": "attention us/layer/token + achieved HBM GB/s (% peak) at ctx 32K, 1 GPU",
        "value": head["us_per_layer_token"], "unit": "us/layer/token", "n_gpus": 1,
        "steps": a.steps, "warmup": a.warmup, "ms_per_step": head["us_per_layer_token"] / 1e3,
        "us_event": head["us_event"], "timing": f"median of {REPS} repetitions of the {a.steps}-step region; value is wall clock "
                                                 "with a stream synchronisation on both sides, us_event the same region between HIP events",
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "bf16 K/V, f32 accumulate",
        "data": "synthetic",
        "config": {"workload": "gated GQA decode, 32 Q / 2 KV heads, head_dim 256, kv_len 32768, "
                               "bf16 K/V ~N(0,1), f32 q and gate, batch 1 (BASELINE configs[2])",
                   "kv_caches_rotated": a.layers, "timed_calls": "mfa_sdpa_decode_dev"},
        "hbm_gbps": head["gbps"], "hbm_pct_peak": head["pct_peak"],
        "roofline": {"bound": "hbm", "achieved": head["gbps_partial_kernel"], "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": head["gbps_partial_kernel"] / HBM_PEAK_GBPS,
                     "traffic": _c3_partial_traffic_bytes(), "kernel": "sdpa_partial_kernel<bf16, 256>",
                     "algorithmic_bytes_per_launch": head["algorithmic_bytes"],
                     "us_per_launch": head["us_partial_kernel_loop"]},
    }
    if not a.no_cpu:
        line["cpu_baseline"], line["gpu_vs_oracle_rel_err"] = cpu_baseline(sample, Hq, Hkv, d, L)
        line["cpu_baseline_all_cores"] = cpu_baseline_all_cores(sample, Hq, Hkv, d, L)
    else:
        line["cpu_baseline"] = None
    del sample
    if not a.no_extra:
        extra = {}
        r, _ = bench_sdpa("c1", 32, 4, 128, 4096, False, 24, a.steps, a.warmup, 0xC0FFEE + 1)
        extra["c1_gqa_decode_f32_L4096"] = r
        extra["c2_gated_deltanet_step"] = bench_gdn("c2", 16, 32, 128, 128, 160, a.steps, a.warmup,
                                                    0xC0FFEE + 2)
        extra["c4_prefill_chunk_512"] = bench_prefill(20, 5, 0xC0FFEE + 4)
        extra["c5_token_sweep_48_layers"], sweep_sample = bench_sweep(max(20, a.steps // 8), 5, 0xC0FFEE + 5)
        extra["f1_attention_prologue"] = bench_prologue(max(50, a.steps // 4), 10, 0xC0FFEE + 8)
        extra["f2_state_snapshot"] = bench_snapshot(0xC0FFEE + 9)
        extra["f3_projection_matvecs"] = bench_matvec(a.steps // 2, a.warmup, 0xC0FFEE + 6)
        extra["f4_mla_folded_sdpa"] = bench_mla(max(20, a.steps // 8), 5, 0xC0FFEE + 7)
        if not a.no_cpu:
            extra["cpu_one_thread"] = cpu_secondary(sweep_sample)
        line["extra"] = extra
    print(json.dumps(line))


if __name__ == "__main__":
    main()
