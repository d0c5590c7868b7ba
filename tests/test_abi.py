"""The C-ABI library: it loads, exports every symbol include/moeflux_attn.h declares,
and rejects bad arguments with the documented codes before it touches the GPU.
Runs on the CPU (no compute calls)."""
import ctypes as C
import os
import re

import numpy as np
import pytest

from moeflux_amd import ffi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = open(os.path.join(ROOT, "include", "moeflux_attn.h")).read()


def declared_symbols():
    body = re.sub(r"/\*.*?\*/", "", HEADER, flags=re.S)
    return sorted(set(re.findall(r"\b(mfa_[a-z0-9_]+)\s*\(", body)))


def test_library_is_built_in_tree_and_loads():
    assert os.path.exists(ffi.lib_path()), "run `python -m moeflux_amd.build`"
    assert ffi.lib_path().startswith(ROOT)
    ffi.load()


def test_every_declared_symbol_is_exported_and_bound():
    lib = ffi.load()
    syms = declared_symbols()
    assert len(syms) >= 40
    for name in syms:
        assert hasattr(lib, name), f"{name} declared in the header but not exported"
        assert name in ffi.SIGNATURES, f"{name} has no ctypes prototype"
    assert sorted(ffi.SIGNATURES) == syms, "ctypes table and header disagree"


def test_rust_view_declares_every_entry_point_with_the_headers_parameter_count():
    """moeflux_amd/rust/ffi.rs cannot be compiled here; names, parameter counts and the
    pointer/scalar kind of every parameter are held to the header instead."""
    plain = re.sub(r"/\*.*?\*/", "", HEADER, flags=re.S)
    plain = re.sub(r"//[^\n]*", "", plain)
    c_protos = {m.group(1): m.group(2) for m in re.finditer(r"\b(mfa_[a-z0-9_]+)\s*\(([^;{]*?)\)\s*;", plain)}
    rust = open(os.path.join(ROOT, "moeflux_amd", "rust", "ffi.rs")).read()
    r_protos = {m.group(1): m.group(2) for m in re.finditer(r"pub fn (mfa_[a-z0-9_]+)\(([^;]*?)\)\s*(?:->[^;]*)?;", rust, flags=re.S)}
    assert sorted(r_protos) == declared_symbols()
    for name, args in c_protos.items():
        c_args = [] if args.strip() in ("", "void") else [a.strip() for a in args.split(",")]
        r_args = [a.strip() for a in r_protos[name].split(",") if a.strip()]
        assert len(c_args) == len(r_args), name
        for ca, ra in zip(c_args, r_args):
            assert ("*" in ca) == ("*" in ra), (name, ca, ra)
            assert ("const" in ca.split("*")[0].split()) == ("*const" in ra) if "*" in ca else True, (name, ca, ra)


def test_header_cites_the_reference_for_every_entry_point():
    # each declaration is preceded by a comment naming a reference file or saying it has none
    for name in declared_symbols():
        idx = HEADER.index(name + "(")
        ctx = HEADER[max(0, idx - 1600):idx]
        assert re.search(r"\.(rs|h|m|metal)[:\s,)]|No counterpart|no reference counterpart|Text of the last|Block until|hipStream_t", ctx), name


def test_destroy_null_is_a_noop_and_null_ctx_is_an_error():
    lib = ffi.load()
    lib.mfa_ctx_destroy(None)                       # moeflux.h:62-64
    assert lib.mfa_sync(None) == ffi.ERR_INVALID
    assert lib.mfa_kv_len(None, 0) == ffi.ERR_INVALID
    assert lib.mfa_pos_max(None) == ffi.ERR_INVALID
    assert lib.mfa_reset(None) == ffi.ERR_INVALID
    assert lib.mfa_stream(None) is None
    assert b"NULL" in lib.mfa_last_error_string()


def _cfg(**kw):
    base = dict(num_layers=4, full_attn_interval=4, num_attn_heads=32, num_kv_heads=2, head_dim=256,
                kv_capacity=64, kv_dtype=0, linear_num_k_heads=16, linear_num_v_heads=32,
                linear_key_dim=128, linear_value_dim=128, conv_kernel_size=4, rms_norm_eps=1e-6)
    base.update(kw)
    return ffi.mfa_config(*[base[f[0]] for f in ffi.mfa_config._fields_])


@pytest.mark.parametrize("kw,needle", [
    (dict(num_layers=0), "positive"),
    (dict(num_attn_heads=30, num_kv_heads=4), "multiple"),          # gpu_attn.rs:262
    (dict(head_dim=96), "not supported"),
    (dict(kv_dtype=7), "not supported"),
    (dict(kv_capacity=0), "non-positive"),
    (dict(linear_num_v_heads=30), "multiple"),                        # linear_attn.rs:306
    (dict(linear_key_dim=100), "not supported"),
    (dict(conv_kernel_size=0), "non-positive"),
])
def test_create_rejects_bad_config_without_a_gpu(kw, needle):
    lib = ffi.load()
    cfg = _cfg(**kw)
    assert lib.mfa_ctx_create(C.byref(cfg)) is None                  # moeflux.h:52-54
    assert needle in ffi.last_error()
    assert lib.mfa_ctx_create(None) is None


def test_stateless_hooks_validate_before_touching_the_gpu():
    lib = ffi.load()
    a = np.zeros(64 * 64, np.float32)
    p = a.ctypes.data
    u = np.zeros(64 * 64, np.uint16).ctypes.data
    inv = ffi.ERR_INVALID
    assert lib.mfa_sdpa(0, 4, 2, 64, p, p, p, p, p) == inv            # kv_len <= 0 (sdpa.rs:71)
    assert "kv_len" in ffi.last_error()
    assert lib.mfa_sdpa(-3, 4, 2, 64, p, p, p, p, p) == inv
    assert lib.mfa_sdpa(4, 4, 2, 64, None, p, p, p, p) == inv         # NULL (moeflux.h:177-178)
    assert lib.mfa_sdpa(4, 6, 4, 64, p, p, p, p, p) == inv            # Hq % Hkv
    assert lib.mfa_sdpa(4, 4, 2, 48, p, p, p, p, p) == ffi.ERR_SHAPE
    assert lib.mfa_sdpa_bf16kv(0, 4, 2, 64, p, p, u, u, p) == inv
    assert lib.mfa_attn_scores_batched(4, 2, 64, 0, p, p, 0.125, p) == inv
    assert lib.mfa_attn_scores_batched(6, 4, 64, 8, p, p, 0.125, p) == inv
    assert lib.mfa_attn_softmax_batched(0, 8, p) == inv
    assert lib.mfa_attn_values_batched(4, 2, 64, 8, p, None, p) == inv
    assert lib.mfa_sigmoid_gate(0, p, p) == inv                        # moeflux.h:524-527
    assert lib.mfa_conv1d_step(0, 4, p, p, u, p) == inv                # linear_attn.rs:97
    assert lib.mfa_conv1d_step(8, 4, p, p, None, p) == inv
    assert lib.mfa_rms_norm_bare(0, 1e-6, p, p) == inv                 # linear_attn.rs:166
    assert lib.mfa_rms_norm_qk(0, 128, p, p) == inv
    assert lib.mfa_compute_decay_beta(0, p, p, p, u, p, p) == inv
    assert lib.mfa_gated_delta_net_step(3, 2, 64, 64, p, p, p, p, p, p, p) == inv   # linear_attn.rs:306
    assert lib.mfa_gated_delta_recurrence(p, u, p, p, p, p, p, 0, 1, 64, 64, p, p) == inv
    assert lib.mfa_gated_rms_norm(1, 0, 1e-6, p, p, u, p) == inv
    # the library is still usable after errors
    assert lib.mfa_sigmoid_gate(-1, p, p) == inv


def test_python_mirror_fails_loudly_without_the_library(monkeypatch, tmp_path):
    monkeypatch.setattr(ffi, "_lib", None)
    monkeypatch.setattr(ffi, "_LIB_PATH", str(tmp_path / "missing.so"))
    with pytest.raises(ImportError, match="no CPU fallback"):
        ffi.load()


def test_rust_build_script_compiles_every_hip_source():
    """moeflux_amd/rust/build.rs names its sources one by one; the list is held to csrc/*.hip
    so that a new source cannot be left out of the library the Rust crate links."""
    rs = open(os.path.join(ROOT, "moeflux_amd", "rust", "build.rs")).read()
    body = rs[rs.index("for f in ["):rs.index("] {")]
    listed = re.findall(r'"([a-z0-9_]+\.hip)"', body)
    on_disk = sorted(f for f in os.listdir(os.path.join(ROOT, "moeflux_amd", "csrc")) if f.endswith(".hip"))
    assert listed == on_disk
    # the flags that change results are the Python build's too
    from moeflux_amd import build as hip_build
    for flag in ("--offload-arch=gfx950", "-ffp-contract=off", "-packed-fp32-ops"):
        assert flag in rs and any(flag in f for f in hip_build.FLAGS), flag
