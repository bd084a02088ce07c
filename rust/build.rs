// build.rs -- builds libmk_hip.so (gfx950 code objects + the C-ABI host layer) with hipcc and links it.
//
// The reference has no build script (its Metal kernels are compiled at run time, src/metal.rs:462-593); the HIP path
// compiles its kernels offline.  MK_HIP_SRC points at the directory that holds csrc/ and include/ (a checkout of the
// library); without the `hip` feature nothing is built.  Not compiled here: the build image has no Rust toolchain.
use std::env;
use std::path::PathBuf;
use std::process::Command;

const SOURCES: &[&str] = &[
    "host.hip", "codec.hip", "gemv_mxfp4.hip", "gemv_q8.hip", "moe.hip", "mla.hip", "mla_heads.hip", "gemm_mxfp4.hip",
    "gemm_q8x.hip", "prefill.hip", "front.hip", "weights.hip", "vq1.hip", "quantize.hip",
];

fn main() {
    if env::var_os("CARGO_FEATURE_HIP").is_none() {
        return;
    }
    let root = PathBuf::from(env::var("MK_HIP_SRC").expect("MK_HIP_SRC: path of the libmk_hip sources (the directory holding microkimi_amd/csrc and include/)"));
    let csrc = root.join("microkimi_amd").join("csrc");
    let out_dir = PathBuf::from(env::var("OUT_DIR").unwrap());
    let lib = out_dir.join("libmk_hip.so");
    let hipcc = env::var("HIPCC").unwrap_or_else(|_| "/opt/rocm/bin/hipcc".to_string());
    let mut cmd = Command::new(&hipcc);
    cmd.args(["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-Wno-unused-value", "-fno-strict-aliasing"]);
    // compiler-formed packed-f32 operations are kept off on this target
    cmd.args(["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]);
    cmd.arg("-I").arg(root.join("include")).arg("-I").arg(&csrc).arg("-DMK_BUILD=1");
    for s in SOURCES {
        let p = csrc.join(s);
        println!("cargo:rerun-if-changed={}", p.display());
        cmd.arg(p);
    }
    println!("cargo:rerun-if-changed={}", root.join("include").join("mk_hip.h").display());
    cmd.arg("-o").arg(&lib);
    let status = cmd.status().unwrap_or_else(|e| panic!("cannot run {}: {}", hipcc, e));
    assert!(status.success(), "hipcc failed");
    println!("cargo:rustc-link-search=native={}", out_dir.display());
    println!("cargo:rustc-link-lib=dylib=mk_hip");
    // the HIP runtime the library itself links
    println!("cargo:rustc-link-search=native=/opt/rocm/lib");
    println!("cargo:rustc-link-lib=dylib=amdhip64");
}
