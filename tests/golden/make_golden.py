"""Writes tests/golden/attention_f64.json, attn_prologue_f64.json and around_the_core_f64.json: small cases of every
function on the attention path and around it, inputs and float64 expected outputs.

The expected values come from oracle/f64ref.py — vectorised float64 numpy built
on library routines (einsum, scipy.special.softmax / expit), written from the
mathematics and sharing no code with the C restatement the fixtures pin.  The
reference repository holds no numeric vectors for these kernels (its tests store
input formulas and tolerances only), so these are the committed vectors.

    python tests/golden/make_golden.py
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import cref, f64ref  # noqa: E402


def r32(rng, *shape, scale=1.0):
    return (rng.standard_normal(shape) * scale).astype(np.float32)


def lst(a):
    return np.asarray(a).reshape(-1).tolist()


def prologue_cases():
    """What precedes the attention core in a full-attention layer: q/gate split, per-head
    norms, partial rotation (small positions: the f32 frequency table is itself 6e-8 from exact)."""
    rng = np.random.default_rng(20261126)
    cases = []
    for (Hq, Hkv, d, rd, theta, pos) in [(4, 2, 16, 4, 1e7, 0), (4, 2, 16, 4, 1e7, 3), (2, 1, 32, 8, 1e7, 57),
                                         (3, 3, 16, 16, 1e4, 9), (8, 2, 64, 16, 1e7, 100)]:
        qn = cref.f32_to_bf16(1.0 + 0.3 * rng.standard_normal(d))
        kn = cref.f32_to_bf16(1.0 + 0.3 * rng.standard_normal(d))
        qp, k, v = r32(rng, Hq * 2 * d), r32(rng, Hkv * d), r32(rng, Hkv * d)
        q, g, kr, vr = f64ref.attn_prologue(pos, Hq, Hkv, d, rd, theta, 1e-6, qn, kn, qp, k, v)
        cases.append(dict(Hq=Hq, Hkv=Hkv, d=d, rotary_dim=rd, theta=theta, pos=pos, eps=1e-6, q_norm=lst(qn),
                          k_norm=lst(kn), q_proj_out=lst(qp), k=lst(k), v=lst(v), q_out=lst(q), gate_out=lst(g),
                          k_row=lst(kr), v_row=lst(vr)))
    with open(os.path.join(HERE, "attn_prologue_f64.json"), "w") as f:
        json.dump({"attn_prologue": cases}, f)


def around_the_core_cases():
    """Attention over a latent cache and the 4-bit dequantising matrix-vector product."""
    rng = np.random.default_rng(20261127)
    mla, mv = [], []
    for (H, R, P, L, scale) in [(2, 8, 4, 1, 0.5), (3, 16, 4, 9, 0.29), (5, 32, 8, 40, 0.16), (16, 64, 16, 33, 0.11)]:
        qp, qe = r32(rng, H, R, scale=0.4), r32(rng, H, P, scale=0.4)
        lat, rk = r32(rng, L, R), r32(rng, L, P)
        out = f64ref.mla_sdpa_folded(H, R, P, L, scale, qp, qe, lat, rk)
        mla.append(dict(H=H, R=R, P=P, L=L, scale=scale, q_prime=lst(qp), q_pe=lst(qe), latent=lst(lat),
                        rope_k=lst(rk), out=lst(out)))
    for (od, idim) in [(1, 64), (3, 128), (7, 320), (16, 512)]:
        packed = rng.integers(0, 2 ** 32, size=(od, idim // 8), dtype=np.uint64).astype(np.uint32)
        sc = cref.f32_to_bf16(np.abs(rng.standard_normal((od, idim // 64))) * 0.02 + 0.003)
        bi = cref.f32_to_bf16(rng.standard_normal((od, idim // 64)) * 0.1)
        x = r32(rng, idim)
        out = f64ref.dequant_matvec_4bit(packed, sc, bi, idim, od, x)
        mv.append(dict(out_dim=od, in_dim=idim, packed=lst(packed), scales=lst(sc), biases=lst(bi), x=lst(x),
                       out=lst(out)))
    with open(os.path.join(HERE, "around_the_core_f64.json"), "w") as f:
        json.dump({"mla_sdpa_folded": mla, "dequant_matvec_4bit": mv}, f)


def main():
    prologue_cases()
    around_the_core_cases()
    rng = np.random.default_rng(20261125)
    cases = {"sdpa": [], "gdn_step": [], "conv1d": [], "rms_norm_qk": [], "decay_beta": [],
             "delta_net_step": [], "rms_norm_gated": [], "prefill_attn": []}

    for (Hq, Hkv, d, L) in [(4, 2, 8, 1), (4, 2, 8, 2), (4, 2, 8, 7), (4, 2, 8, 33), (6, 1, 4, 5),
                            (3, 3, 8, 9)]:
        q, g = r32(rng, Hq * d), r32(rng, Hq * d)
        k, v = r32(rng, L, Hkv * d), r32(rng, L, Hkv * d)
        cases["sdpa"].append(dict(Hq=Hq, Hkv=Hkv, d=d, L=L, q=lst(q), gate=lst(g), k=lst(k), v=lst(v),
                                  out=lst(f64ref.sdpa(L, Hq, Hkv, d, q, g, k, v))))

    for (Hk, Hv, dk, dv, K, T) in [(1, 2, 4, 4, 4, 3), (2, 4, 8, 4, 4, 2), (2, 2, 4, 8, 3, 4)]:
        C = 2 * Hk * dk + Hv * dv
        cw = cref.f32_to_bf16(r32(rng, C * K, scale=0.5))
        a_log = r32(rng, Hv, scale=0.5)
        dt = cref.f32_to_bf16(r32(rng, Hv, scale=0.5))
        nw = cref.f32_to_bf16(1.0 + r32(rng, dv, scale=0.2))
        cs = r32(rng, (K - 1) * C).astype(np.float64)
        ss = r32(rng, Hv * dv * dk, scale=0.3).astype(np.float64)
        case = dict(Hk=Hk, Hv=Hv, dk=dk, dv=dv, K=K, T=T, eps=1e-6, conv_w=lst(cw), a_log=lst(a_log),
                    dt_bias=lst(dt), norm_w=lst(nw), conv_state0=lst(cs), ssm_state0=lst(ss),
                    qkv=[], z=[], alpha=[], beta=[], out=[])
        for _ in range(T):
            x, z = r32(rng, C), r32(rng, Hv * dv)
            al, be = r32(rng, Hv), r32(rng, Hv)
            o, cs, ss = f64ref.gdn_step(Hk, Hv, dk, dv, K, 1e-6, cw, a_log, dt, nw, x, z, al, be, cs, ss)
            for key, val in (("qkv", x), ("z", z), ("alpha", al), ("beta", be), ("out", o)):
                case[key].append(lst(val))
        case["conv_state"] = lst(cs)
        case["ssm_state"] = lst(ss)
        cases["gdn_step"].append(case)

    for (C, K) in [(6, 4), (5, 2), (8, 3)]:
        st, x = r32(rng, (K - 1) * C), r32(rng, C)
        w = cref.f32_to_bf16(r32(rng, C * K, scale=0.7))
        cases["conv1d"].append(dict(C=C, K=K, state=lst(st), x=lst(x), w=lst(w),
                                    out=lst(f64ref.conv1d_step(st, x, w, C, K)),
                                    shifted=lst(f64ref.conv_state_shift(st, x, C, K))))

    for (Hk, dk) in [(2, 8), (3, 16)]:
        q, k = r32(rng, Hk * dk, scale=2.0), r32(rng, Hk * dk, scale=0.3)
        qn, kn = f64ref.rms_norm_qk(Hk, dk, q, k)
        cases["rms_norm_qk"].append(dict(Hk=Hk, dk=dk, q=lst(q), k=lst(k), qn=lst(qn), kn=lst(kn)))

    al, be, a_log = r32(rng, 6, scale=2.0), r32(rng, 6, scale=2.0), r32(rng, 6)
    dt = cref.f32_to_bf16(r32(rng, 6))
    g, b = f64ref.decay_beta(al, be, a_log, dt)
    cases["decay_beta"].append(dict(alpha=lst(al), beta=lst(be), a_log=lst(a_log), dt_bias=lst(dt),
                                    g=lst(g), b=lst(b)))

    for (Hv, Hk, dk, dv) in [(2, 1, 4, 4), (4, 2, 8, 4)]:
        g, b = rng.uniform(0.2, 1.0, Hv).astype(np.float32), rng.uniform(0.1, 0.9, Hv).astype(np.float32)
        q, k, v = r32(rng, Hk * dk, scale=0.3), r32(rng, Hk * dk, scale=0.4), r32(rng, Hv * dv)
        S = r32(rng, Hv * dv * dk, scale=0.5)
        Sn, o = f64ref.delta_net_step(Hv, Hk, dk, dv, g, b, q, k, v, S)
        cases["delta_net_step"].append(dict(Hv=Hv, Hk=Hk, dk=dk, dv=dv, g=lst(g), b=lst(b), q=lst(q),
                                            k=lst(k), v=lst(v), S=lst(S), S_new=lst(Sn), out=lst(o)))

    x, z = r32(rng, 16), r32(rng, 16)
    w = cref.f32_to_bf16(1.0 + r32(rng, 16, scale=0.3))
    cases["rms_norm_gated"].append(dict(x=lst(x), z=lst(z), w=lst(w), eps=1e-6,
                                        out=lst(f64ref.rms_norm_gated(x, z, w, 1e-6))))

    for (T, L0, Hq, Hkv, d) in [(5, 0, 4, 2, 8), (3, 4, 4, 1, 8)]:
        q, g = r32(rng, T, Hq * d), r32(rng, T, Hq * d)
        k, v = r32(rng, L0 + T, Hkv * d), r32(rng, L0 + T, Hkv * d)
        cases["prefill_attn"].append(dict(T=T, L0=L0, Hq=Hq, Hkv=Hkv, d=d, q=lst(q), gate=lst(g),
                                          k=lst(k), v=lst(v),
                                          out=lst(f64ref.prefill_attn(T, L0, Hq, Hkv, d, q, g, k, v))))

    path = os.path.join(HERE, "attention_f64.json")
    with open(path, "w") as f:
        json.dump(cases, f)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
