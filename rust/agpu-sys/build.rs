//! Compiles the HIP sources of libagpu_hip.so for gfx950 and links the shared library, as
//! async-gpu_amd/csrc/build.sh does (the reference's build.rs shells out in the same way for its PTX,
//! crates/core/gpu-host/build.rs:104-160).  AGPU_CSRC points at the csrc directory (default: the one in this repository),
//! HIPCC at the compiler (default /opt/rocm/bin/hipcc).
use std::path::{Path, PathBuf};
use std::process::Command;

fn main() {
    let out = PathBuf::from(std::env::var("OUT_DIR").expect("OUT_DIR"));
    let manifest = PathBuf::from(std::env::var("CARGO_MANIFEST_DIR").expect("CARGO_MANIFEST_DIR"));
    let csrc = std::env::var("AGPU_CSRC").map(PathBuf::from).unwrap_or_else(|_| manifest.join("../../async-gpu_amd/csrc"));
    let hipcc = std::env::var("HIPCC").unwrap_or_else(|_| "/opt/rocm/bin/hipcc".to_string());
    println!("cargo:rerun-if-changed={}", csrc.display());
    println!("cargo:rerun-if-env-changed=AGPU_CSRC");
    println!("cargo:rerun-if-env-changed=HIPCC");

    let mut objects: Vec<PathBuf> = Vec::new();
    let mut sources: Vec<PathBuf> = std::fs::read_dir(&csrc)
        .expect("csrc directory")
        .filter_map(|e| e.ok().map(|e| e.path()))
        .filter(|p| p.extension().map(|x| x == "hip").unwrap_or(false))
        .collect();
    sources.sort();
    for src in &sources {
        let obj = out.join(Path::new(src.file_stem().unwrap()).with_extension("o"));
        let status = Command::new(&hipcc)
            .args(["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-ffp-contract=off"])
            // packed FP32 instructions are kept out of the generated code
            .args(["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"])
            .arg("-c")
            .arg(src)
            .arg("-o")
            .arg(&obj)
            .status()
            .expect("hipcc");
        assert!(status.success(), "hipcc failed on {}", src.display());
        objects.push(obj);
    }
    // the host-side quantizer (quantize_weight_int4 on the CPU, where the reference runs it)
    let qobj = out.join("quantize_host.o");
    let status = Command::new("g++")
        .args(["-O2", "-std=c++17", "-fPIC", "-fopenmp", "-fvisibility=hidden", "-ffp-contract=off", "-c"])
        .arg(csrc.join("quantize_host.cpp"))
        .arg("-o")
        .arg(&qobj)
        .status()
        .expect("g++");
    assert!(status.success(), "g++ failed on quantize_host.cpp");
    objects.push(qobj);

    let lib = out.join("libagpu_hip.so");
    let status = Command::new(&hipcc)
        .args(["--offload-arch=gfx950", "-shared", "-fPIC", "-o"])
        .arg(&lib)
        .args(&objects)
        .arg("-fopenmp")
        .status()
        .expect("hipcc (link)");
    assert!(status.success(), "linking libagpu_hip.so failed");

    println!("cargo:rustc-link-search=native={}", out.display());
    println!("cargo:rustc-link-lib=dylib=agpu_hip");
    println!("cargo:rustc-link-arg=-Wl,-rpath,{}", out.display());
}
