#!/usr/bin/env python3
"""Benchmark of the MI355X attention path.

Headline (the one JSON line the driver reads): BASELINE.json's metric, attention
microseconds per layer per token with the achieved HBM rate, on the
long-context configuration the metric is quoted on — gated GQA decode,
32 Q / 2 KV heads, head_dim 256, 32768 cached positions, bf16 K/V, batch 1
(configs[2]; configs[0] and [1] are reported under "extra").  A "step" is one
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


def _timed(ctx, lib, fn, steps, warmup):
    """Run fn(i) warmup+steps times; returns (wall ms per step, event ms per step)."""
    for i in range(warmup):
        fn(i)
    lib.mfa_sync(ctx.h)
    t0 = time.perf_counter()
    lib.mfa_timer_start(ctx.h)
    for i in range(steps):
        fn(i)
    ms = C.c_float(0)
    rc = lib.mfa_timer_stop(ctx.h, C.byref(ms))  # records the end event and waits for it
    lib.mfa_sync(ctx.h)
    wall = (time.perf_counter() - t0) * 1e3
    if rc != 0:
        raise RuntimeError("mfa_timer_stop failed")
    return wall / steps, ms.value / steps


def bench_sdpa(name, Hq, Hkv, d, L, bf16, layers, steps, warmup, seed):
    from moeflux_amd import Config, Ctx, ffi
    from moeflux_amd.hip import DeviceArray
    from oracle import cref
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
        base_k, base_v = cref.f32_to_bf16(base_k), cref.f32_to_bf16(base_v)
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

    def step(i):
        l = i % layers
        rc = lib.mfa_sdpa_decode_dev(ctx.h, l, dq.offset(l * qd), dg.offset(l * qd), dout.offset(l * qd))
        if rc != 0:
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
    from tests.util import GdnCase
    lib = ffi.load()
    case = GdnCase(seed, Hk, Hv, dk, dv, T=1, plain=True)
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

    def step(i):
        l = i % layers
        rc = lib.mfa_gdn_step_dev(ctx.h, l, dx.offset(l * C_), dz.offset(l * tv), da.offset(l * Hv),
                                  db.offset(l * Hv), dout.offset(l * tv))
        if rc != 0:
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
    n = int(max(1, min(20, budget_s / max(first, 1e-3))))
    t0 = time.perf_counter()
    for _ in range(n):
        cref.sdpa(L, Hq, Hkv, d, q, g, kf, vf)
    per = (time.perf_counter() - t0) / n
    err = float(np.abs(gpu_out - ref).max() / np.abs(ref).max())
    return {"value": per * 1e6, "unit": "us/layer/token", "cores": 1, "kind": "port",
            "sample": f"{n} calls of the oracle's orc_sdpa at the full workload shape "
                      f"(kv_len {L}, f32-widened cache), single thread"}, err


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--layers", type=int, default=8, help="independent KV caches rotated over")
    ap.add_argument("--no-extra", action="store_true", help="skip the secondary configurations")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py: this path is measured on one GPU only (batch-1 decode attention on one "
              "device); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    Hq, Hkv, d, L = 32, 2, 256, 32768
    head, sample = bench_sdpa("c3", Hq, Hkv, d, L, True, a.layers, a.steps, a.warmup, 0xC0FFEE + 3)
    line = {
        "metric": "attention us/layer/token + achieved HBM GB/s (% peak) at ctx 32K, 1 GPU",
        "value": head["us_per_layer_token"], "unit": "us/layer/token", "n_gpus": 1,
        "steps": a.steps, "warmup": a.warmup, "ms_per_step": head["us_per_layer_token"] / 1e3,
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "bf16 K/V, f32 accumulate",
        "data": "synthetic",
        "config": {"workload": "gated GQA decode, 32 Q / 2 KV heads, head_dim 256, kv_len 32768, "
                               "bf16 K/V ~N(0,1), f32 q and gate, batch 1 (BASELINE configs[2])",
                   "kv_caches_rotated": a.layers, "timed_calls": "mfa_sdpa_decode_dev"},
        "hbm_gbps": head["gbps"], "hbm_pct_peak": head["pct_peak"],
        "roofline": {"bound": "hbm", "achieved": head["gbps_partial_kernel"], "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": head["gbps_partial_kernel"] / HBM_PEAK_GBPS,
                     "traffic": None, "kernel": "sdpa_partial_kernel<bf16, 256>",
                     "algorithmic_bytes_per_launch": head["algorithmic_bytes"],
                     "us_per_launch": head["us_partial_kernel_loop"]},
    }
    if not a.no_cpu:
        line["cpu_baseline"], line["gpu_vs_oracle_rel_err"] = cpu_baseline(sample, Hq, Hkv, d, L)
    else:
        line["cpu_baseline"] = None
    del sample
    if not a.no_extra:
        extra = {}
        r, _ = bench_sdpa("c1", 32, 4, 128, 4096, False, 24, a.steps, a.warmup, 0xC0FFEE + 1)
        extra["c1_gqa_decode_f32_L4096"] = r
        extra["c2_gated_deltanet_step"] = bench_gdn("c2", 16, 32, 128, 128, 160, a.steps, a.warmup,
                                                    0xC0FFEE + 2)
        line["extra"] = extra
    print(json.dumps(line))


if __name__ == "__main__":
    main()
