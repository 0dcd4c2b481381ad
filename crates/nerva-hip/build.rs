//! Compiles the HIP sources with hipcc into libnerva_hip.a and links it, or - without hipcc, or
//! with NERVA_HIP_BUILD=stubs - builds the crate against Rust stubs that answer every call with
//! status = -1, hip_error = 100, the way nerva-cuda does without nvcc
//! (crates/nerva-cuda/build.rs:7-51, 113-148; native_stubs.rs:5-33).
use std::env;
use std::path::{Path, PathBuf};
use std::process::Command;

/// Kernels that request their data with hand-written loads and wait for it with explicit counts. The compiler
/// does not know that such a register is still being written, so a spill of it reads garbage: these kernels
/// must compile without scratch memory, which this script checks like the library's own build (build.py). What
/// the check cannot see - a register copy the compiler places between such a load and its wait - is covered by
/// the library's parity tests only, which is why the kernels are built for the one target they were checked on.
const HAND_ISSUED_LOADS: &[&str] = &["attn_step_kernel", "moe_gate_up_lean_kernel", "moe_down_lean_kernel", "fp8_gemv_lean_kernel", "gemm_deep_kernel"];
const SUPPORTED_ARCH: &str = "gfx950";

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
    let arch = env::var("NERVA_HIP_ARCH").unwrap_or_else(|_| SUPPORTED_ARCH.into());
    assert!(arch == SUPPORTED_ARCH, "NERVA_HIP_ARCH={arch}: the kernels are written and checked for {SUPPORTED_ARCH} only");
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
    let output = Command::new(hipcc)
        .args(["-c", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function"])
        .arg(format!("--offload-arch={arch}"))
        // packed fp32 VALU ops stay off for every device function of the library
        .args(["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"])
        .arg("-Rpass-analysis=kernel-resource-usage")
        .arg(format!("-I{}", include.display()))
        .arg(format!("-I{}", csrc.display()))
        .arg(src)
        .arg("-o")
        .arg(obj)
        .output()
        .expect("hipcc");
    let remarks = String::from_utf8_lossy(&output.stderr);
    assert!(output.status.success(), "hipcc failed on {}:\n{}", src.display(), remarks);
    let spilling = spilling_kernels(&remarks);
    let bad: Vec<&String> = spilling.iter().filter(|k| HAND_ISSUED_LOADS.iter().any(|name| k.contains(name))).collect();
    assert!(bad.is_empty(), "{}: kernels that issue loads by hand must not spill registers: {:?}", src.display(), bad);
}

/// Kernels whose register allocation went to scratch memory, from hipcc's resource-usage remarks.
fn spilling_kernels(remarks: &str) -> Vec<String> {
    let mut bad = Vec::new();
    let mut name: Option<String> = None;
    for line in remarks.lines() {
        if let Some(at) = line.find("Function Name:") {
            name = Some(line[at + "Function Name:".len()..].split('[').next().unwrap_or("").trim().to_string());
        } else if let Some(at) = line.find("ScratchSize [bytes/lane]:") {
            let size: u64 = line[at + "ScratchSize [bytes/lane]:".len()..].split('[').next().unwrap_or("").trim().parse().unwrap_or(0);
            if let (Some(kernel), true) = (name.take(), size != 0) {
                bad.push(format!("{kernel} ({size} bytes a lane)"));
            }
        }
    }
    bad
}
