// rai-core/build.rs -- builds librai_hip.so with hipcc when the `hip` feature is on and links it.
//
// The reference tree has no build script (all native code lives in third-party crates); this one is the
// counterpart of what candle-core's own build does for its CUDA kernels.  RAI_HIP_SRC points at the directory
// that holds `include/` and `rai_amd/csrc/` (a checkout of the kernel repository); RAI_HIP_LIB_DIR, when set,
// names a directory with a prebuilt librai_hip.so and skips the compile.
use std::{env, path::PathBuf, process::Command};

fn main() {
    println!("cargo:rerun-if-env-changed=RAI_HIP_SRC");
    println!("cargo:rerun-if-env-changed=RAI_HIP_LIB_DIR");
    if env::var("CARGO_FEATURE_HIP").is_err() {
        return;
    }
    let rocm = env::var("ROCM_PATH").unwrap_or_else(|_| "/opt/rocm".to_string());
    if let Ok(dir) = env::var("RAI_HIP_LIB_DIR") {
        println!("cargo:rustc-link-search=native={dir}");
    } else {
        let root = PathBuf::from(env::var("RAI_HIP_SRC").expect("RAI_HIP_SRC = root of the rai_amd checkout"));
        let csrc = root.join("rai_amd").join("csrc");
        let out = PathBuf::from(env::var("OUT_DIR").unwrap());
        let mut objects = Vec::new();
        let mut sources: Vec<PathBuf> = std::fs::read_dir(&csrc)
            .expect("rai_amd/csrc")
            .filter_map(|e| e.ok().map(|e| e.path()))
            .filter(|p| matches!(p.extension().and_then(|e| e.to_str()), Some("hip") | Some("cpp")))
            .collect();
        sources.sort();
        for src in &sources {
            println!("cargo:rerun-if-changed={}", src.display());
            let obj = out.join(format!("{}.o", src.file_name().unwrap().to_string_lossy()));
            let mut cmd = Command::new(format!("{rocm}/bin/hipcc"));
            cmd.args([
                "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
                // hipcc must not form packed-f32 instructions from float code
                "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                "-Wno-unused-result",
            ]);
            if src.file_name().unwrap() == "attention.hip" {
                cmd.args(["-mllvm", "-amdgpu-mfma-vgpr-form"]);
            }
            cmd.arg(format!("-I{}", root.join("include").display()))
                .arg(format!("-I{}", csrc.display()))
                .args(["-x", "hip", "-c"])
                .arg(src)
                .arg("-o")
                .arg(&obj);
            assert!(cmd.status().expect("hipcc").success(), "hipcc failed for {}", src.display());
            objects.push(obj);
        }
        let lib = out.join("librai_hip.so");
        let mut link = Command::new(format!("{rocm}/bin/hipcc"));
        link.args(["--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", "-o"]).arg(&lib).args(&objects);
        assert!(link.status().expect("hipcc link").success(), "linking librai_hip.so failed");
        println!("cargo:rustc-link-search=native={}", out.display());
    }
    println!("cargo:rustc-link-search=native={rocm}/lib");
    println!("cargo:rustc-link-lib=dylib=rai_hip");
    println!("cargo:rustc-link-lib=dylib=amdhip64");
}
