// build.rs for a `moeflux-attn-hip-sys` crate: compiles the HIP sources with hipcc
// into libmoeflux_attn_hip.so and links it, the way crates/moeflux-sys/build.rs:80-96
// compiles and links the Objective-C engine.  Not compiled in this repository's
// image (no rustc); kept next to the sources it builds.
use std::{env, path::PathBuf, process::Command};

fn main() {
    let root = PathBuf::from(env::var("CARGO_MANIFEST_DIR").unwrap());
    let csrc = root.join("csrc");
    let out = PathBuf::from(env::var("OUT_DIR").unwrap());
    let lib = out.join("libmoeflux_attn_hip.so");
    let hipcc = env::var("HIPCC").unwrap_or_else(|_| "/opt/rocm/bin/hipcc".into());
    let mut cmd = Command::new(hipcc);
    cmd.args(["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden", "-ffp-contract=off"])
        .args(["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"])
        .arg("-I").arg(root.join("include")).arg("-I").arg(&csrc);
    // every .hip file under csrc/, in sorted order (a test holds this list to the directory)
    for f in [
        "api.hip", "attn_kernels.hip", "attn_prologue.hip", "checkpoint.hip", "dequant_matvec.hip", "gdn.hip",
        "gdn_chunk.hip", "gdn_wy.hip", "kv_cache.hip", "mla_sdpa.hip", "sdpa_decode.hip", "sdpa_prefill.hip",
        "sdpa_static.hip", "snapshot.hip",
    ] {
        println!("cargo:rerun-if-changed=csrc/{f}");
        cmd.arg(csrc.join(f));
    }
    cmd.arg("-o").arg(&lib);
    assert!(cmd.status().expect("hipcc not found").success(), "hipcc failed");
    println!("cargo:rustc-link-search=native={}", out.display());
    println!("cargo:rustc-link-lib=dylib=moeflux_attn_hip");
}
