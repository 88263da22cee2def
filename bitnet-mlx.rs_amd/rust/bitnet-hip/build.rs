// Builds the gfx950 kernels with hipcc and links them, the way bitnet-cuda/build.rs drives nvcc
// (feature-gated, fixed kernel list, one static library).  No CUDA compatibility path, one architecture.
use std::env;
use std::path::PathBuf;
use std::process::Command;

const KERNELS: &[&str] =
    &["api.hip", "act_quant.hip", "weight_prep.hip", "gemv_w2a8.hip", "gemm_w2a8.hip", "gemv_base3.hip", "diag.hip"];

fn main() {
    println!("cargo:rerun-if-changed=build.rs");
    println!("cargo:rerun-if-changed=../../csrc");
    println!("cargo:rerun-if-changed=../../../include/bitnet_hip.h");
    if env::var("CARGO_FEATURE_HIP").is_err() {
        return; // without the feature every entry point returns HipError::HipNotEnabled (see src/lib.rs)
    }
    let rocm = env::var("ROCM_PATH").unwrap_or_else(|_| "/opt/rocm".to_string());
    let hipcc = PathBuf::from(&rocm).join("bin/hipcc");
    let out = PathBuf::from(env::var("OUT_DIR").unwrap());
    let csrc = PathBuf::from(env::var("CARGO_MANIFEST_DIR").unwrap()).join("../../csrc");
    let mut objects = Vec::new();
    for k in KERNELS {
        let obj = out.join(k.replace(".hip", ".o"));
        let status = Command::new(&hipcc)
            .args(["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
                   "-fhip-fp32-correctly-rounded-divide-sqrt",
                   "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                   "-mllvm", "-amdgpu-kernarg-preload-count=10", "-c"])
            .arg(csrc.join(k))
            .arg("-o")
            .arg(&obj)
            .status()
            .expect("hipcc not found: set ROCM_PATH");
        assert!(status.success(), "hipcc failed on {k}");
        objects.push(obj);
    }
    let lib = out.join("libbitnet_hip_kernels.a");
    let status = Command::new("ar").arg("crs").arg(&lib).args(&objects).status().expect("ar");
    assert!(status.success());
    println!("cargo:rustc-link-search=native={}", out.display());
    println!("cargo:rustc-link-lib=static=bitnet_hip_kernels");
    println!("cargo:rustc-link-search=native={rocm}/lib");
    println!("cargo:rustc-link-lib=amdhip64");
    println!("cargo:rustc-link-lib=stdc++");
}
