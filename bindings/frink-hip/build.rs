// hipcc builds libfrink_hip.a from the vendored sources (csrc/ = frink_amd/csrc/, include/ = include/ of
// the library's repository), cargo links it.  `python -m frink_amd.build` produces the same archive.
fn main() {
    if std::env::var_os("CARGO_FEATURE_HIP").is_none() {
        return;
    }
    let out = std::path::PathBuf::from(std::env::var("OUT_DIR").unwrap());
    let hipcc = std::env::var("HIPCC").unwrap_or_else(|_| "/opt/rocm/bin/hipcc".into());
    let srcs = [
        "frk_runtime.cpp", "frk_quant.hip", "frk_gemv.hip", "frk_gemv_fused.hip", "frk_gemm.hip", "frk_gemm_q6.hip",
        "frk_gemm_q8.hip", "frk_moe.hip", "frk_thin.hip", "frk_gemv_direct.hip", "frk_gemv_f32dot.hip", "frk_kinds.hip", "frk_probe.hip",
    ];
    let mut objs = vec![];
    for s in srcs {
        let o = out.join(format!("{s}.o"));
        let ok = std::process::Command::new(&hipcc)
            .args(["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-Iinclude",
                   "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-x", "hip", "-c"])
            .arg(format!("csrc/{s}"))
            .arg("-o")
            .arg(&o)
            .status()
            .expect("hipcc not found: set HIPCC")
            .success();
        assert!(ok, "hipcc failed on {s}");
        objs.push(o);
        println!("cargo:rerun-if-changed=csrc/{s}");
    }
    println!("cargo:rerun-if-changed=include/frink_hip.h");
    let lib = out.join("libfrink_hip.a");
    assert!(std::process::Command::new("ar").arg("rcs").arg(&lib).args(&objs).status().unwrap().success());
    println!("cargo:rustc-link-search=native={}", out.display());
    println!("cargo:rustc-link-lib=static=frink_hip");
    println!("cargo:rustc-link-search=native=/opt/rocm/lib");
    println!("cargo:rustc-link-lib=dylib=amdhip64");
    println!("cargo:rustc-link-lib=dylib=stdc++");
}
