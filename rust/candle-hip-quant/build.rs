//! Compiles the HIP sources of libcandle_hip_quant for gfx950 with hipcc and links them statically, the way
//! candle-kernels/build.rs builds its CUDA kernels with nvcc.  With the `prebuilt` feature the directory named by
//! CANDLE_HIP_QUANT_LIB_DIR is searched for libcandle_hip_quant.so instead.
use std::path::PathBuf;
use std::process::Command;

const SOURCES: [&str; 10] =
    ["cq_api", "cq_dequant", "cq_actquant", "cq_matvec", "cq_matmul", "cq_moe", "cq_quantize", "cq_nn", "cq_layer", "cq_matvec_batch"];

fn main() {
    let rocm = std::env::var("ROCM_PATH").unwrap_or_else(|_| "/opt/rocm".to_string());
    println!("cargo:rustc-link-search=native={rocm}/lib");
    println!("cargo:rustc-link-lib=dylib=amdhip64");
    if std::env::var("CARGO_FEATURE_PREBUILT").is_ok() {
        let dir = std::env::var("CANDLE_HIP_QUANT_LIB_DIR").expect("CANDLE_HIP_QUANT_LIB_DIR names the directory of libcandle_hip_quant.so");
        println!("cargo:rustc-link-search=native={dir}");
        println!("cargo:rustc-link-lib=dylib=candle_hip_quant");
        return;
    }
    // the crate sits at <repo>/rust/candle-hip-quant; the sources at <repo>/candle_amd/csrc, the headers at <repo>/include
    let manifest = PathBuf::from(std::env::var("CARGO_MANIFEST_DIR").unwrap());
    let repo = manifest.parent().unwrap().parent().unwrap().to_path_buf();
    let csrc = repo.join("candle_amd").join("csrc");
    let out = PathBuf::from(std::env::var("OUT_DIR").unwrap());
    let hipcc = std::env::var("HIPCC").unwrap_or_else(|_| format!("{rocm}/bin/hipcc"));
    println!("cargo:rerun-if-changed={}", repo.join("include").display());
    println!("cargo:rerun-if-changed={}", csrc.display());
    let mut objs = Vec::new();
    let mut children = Vec::new();
    for s in SOURCES {
        let obj = out.join(format!("{s}.o"));
        // -ffp-contract=off: the quantizers and the dequantizer must round like the scalar CPU code;
        // packed-fp32 instructions stay off for the device pass
        let child = Command::new(&hipcc)
            .args(["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off"])
            .args(["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"])
            // the first fourteen dwords of scalar kernel arguments arrive in SGPRs at wave launch
            .args(["-mllvm", "-amdgpu-kernarg-preload-count=14"])
            .arg("-c")
            .arg(csrc.join(format!("{s}.hip")))
            .arg("-o")
            .arg(&obj)
            .spawn()
            .expect("hipcc not found: set HIPCC or ROCM_PATH");
        children.push((s, child));
        objs.push(obj);
    }
    for (s, mut c) in children {
        assert!(c.wait().unwrap().success(), "hipcc failed for {s}.hip");
    }
    let lib = out.join("libcandle_hip_quant.a");
    let _ = std::fs::remove_file(&lib);
    assert!(Command::new("ar").arg("crs").arg(&lib).args(&objs).status().unwrap().success(), "ar failed");
    println!("cargo:rustc-link-search=native={}", out.display());
    println!("cargo:rustc-link-lib=static=candle_hip_quant");
    println!("cargo:rustc-link-lib=dylib=stdc++");
}
