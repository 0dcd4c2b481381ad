//! Compiles the HIP sources with hipcc into libnerva_hip.a and links it, or - without hipcc, or
//! with NERVA_HIP_BUILD=stubs - builds the crate against Rust stubs that answer every call with
//! status = -1, hip_error = 100, the way nerva-cuda does without nvcc
//! (crates/nerva-cuda/build.rs:7-51, 113-148; native_stubs.rs:5-33).
use std::env;
use std::path::{Path, PathBuf};
use std::process::Command;

const SOURCES: &[&str] = &[
    "gemv_stream", "fp8_gemv", "attn_decode", "attn_prompt", "argmax", "synth_fill",
    "sampler", "gemm_rows", "gemm_block", "op_entry", "decode_session",
];

fn main() {
    println!("cargo:rustc-check-cfg=cfg(nerva_hip_native_stubs)");
    println!("cargo:rerun-if-env-changed=NERVA_HIP_BUILD");
    println!("cargo:rerun-if-env-changed=NERVA_HIP_SOURCE_DIR");
    println!("cargo:rerun-if-env-changed=NERVA_HIP_ARCH");
    println!("cargo:rerun-if-env-changed=HIPCC");
    let hipcc = PathBuf::from(env::var("HIPCC").unwrap_or_else(|_| "/opt/rocm/bin/hipcc".into()));
    let mode = env::var("NERVA_HIP_BUILD").unwrap_or_else(|_| "auto".into()).to_ascii_lowercase();
    let native = match mode.as_str() {
        "stub" | "stubs" | "off" | "none" => false,
        "native" | "hip" | "on" => {
            assert!(hipcc.exists(), "NERVA_HIP_BUILD=native requires hipcc (set HIPCC)");
            true
        }
        "auto" | "" => hipcc.exists(),
        other => panic!("unsupported NERVA_HIP_BUILD={other}; use auto, native, or stubs"),
    };
    if !native {
        println!("cargo:rustc-cfg=nerva_hip_native_stubs");
        println!("cargo:warning=nerva-hip using Rust native stubs (no hipcc): every call reports hip_error 100");
        return;
    }
    let manifest = PathBuf::from(env::var("CARGO_MANIFEST_DIR").unwrap());
    let root = env::var("NERVA_HIP_SOURCE_DIR").map(PathBuf::from).unwrap_or_else(|_| manifest.join("native/hip"));
    let (csrc, include) = if root.join("nerva_amd/csrc").exists() {
        (root.join("nerva_amd/csrc"), root.join("include")) // a checkout of the library's repository
    } else {
        (root.clone(), root.join("include")) // vendored: native/hip/*.hip, native/hip/include/*.h
    };
    let out = PathBuf::from(env::var("OUT_DIR").unwrap());
    let arch = env::var("NERVA_HIP_ARCH").unwrap_or_else(|_| "gfx950".into());
    let mut objects = Vec::new();
    for name in SOURCES {
        let src = csrc.join(format!("{name}.hip"));
        println!("cargo:rerun-if-changed={}", src.display());
        let obj = out.join(format!("{name}.o"));
        compile(&hipcc, &arch, &csrc, &include, &src, &obj);
        objects.push(obj);
    }
    let archive = out.join("libnerva_hip.a");
    let _ = std::fs::remove_file(&archive);
    let ok = Command::new("ar").arg("rcs").arg(&archive).args(&objects).status().expect("ar").success();
    assert!(ok, "ar failed");
    let rocm = hipcc.parent().and_then(Path::parent).map(|p| p.join("lib")).unwrap_or_else(|| "/opt/rocm/lib".into());
    println!("cargo:rustc-link-search=native={}", out.display());
    println!("cargo:rustc-link-lib=static=nerva_hip");
    println!("cargo:rustc-link-search=native={}", rocm.display());
    println!("cargo:rustc-link-lib=dylib=amdhip64");
    println!("cargo:rustc-link-lib=dylib=stdc++");
}

fn compile(hipcc: &Path, arch: &str, csrc: &Path, include: &Path, src: &Path, obj: &Path) {
    let ok = Command::new(hipcc)
        .args(["-c", "-O3", "-std=c++17", "-fPIC"])
        .arg(format!("--offload-arch={arch}"))
        // packed fp32 VALU ops stay off for every device function of the library
        .args(["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"])
        .arg(format!("-I{}", include.display()))
        .arg(format!("-I{}", csrc.display()))
        .arg(src)
        .arg("-o")
        .arg(obj)
        .status()
        .expect("hipcc")
        .success();
    assert!(ok, "hipcc failed on {}", src.display());
}
