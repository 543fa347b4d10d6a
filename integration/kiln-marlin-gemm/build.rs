// Build script of the MI355X kiln-marlin-gemm crate.
//
// Takes the place of the reference's nvcc build (crates/kiln-marlin-gemm/build.rs:1-108):
// compiles the HIP sources for gfx950 with hipcc and links the HIP runtime.
// Unlike the reference it fails loudly when the toolkit is missing instead of
// skipping the kernel.
//
// What is compiled is not spelled out here: csrc/objects.list names every object of the library as
// `object:source[:extra flag]` (some kernel files are compiled twice, the second time with a define
// that adds the low-rank term), and the Makefile that builds the shared library for the C and
// Python harnesses reads the same file, so the two builds cannot drift apart.
use std::{env, fs, path::PathBuf, process::Command};

fn main() {
    let rocm = env::var("ROCM_PATH").unwrap_or_else(|_| "/opt/rocm".into());
    let hipcc = PathBuf::from(&rocm).join("bin/hipcc");
    assert!(hipcc.exists(), "kiln-marlin-gemm: hipcc not found under {rocm}; set ROCM_PATH");
    let arch = env::var("KILN_HIP_ARCHS").unwrap_or_else(|_| "gfx950".into());
    let out = PathBuf::from(env::var("OUT_DIR").unwrap());
    let crate_dir = PathBuf::from(env::var("CARGO_MANIFEST_DIR").unwrap());
    // csrc/ holds the kernel sources, include/ the two public headers (kiln_w4a16.h, kiln_marlin_proj.h)
    let (csrc, include) = (crate_dir.join("csrc"), crate_dir.join("include"));

    let manifest = csrc.join("objects.list");
    let listing = fs::read_to_string(&manifest).expect("kiln-marlin-gemm: csrc/objects.list is missing");
    println!("cargo:rerun-if-changed=csrc/objects.list");
    let mut objects = Vec::new();
    for line in listing.lines().map(str::trim).filter(|l| !l.is_empty() && !l.starts_with('#')) {
        let mut fields = line.split(':');
        let (stem, src) = (fields.next().unwrap(), fields.next().expect("object:source[:flag]"));
        let flag = fields.next();
        let obj = out.join(format!("{stem}.o"));
        let mut cmd = if src.ends_with(".cpp") {
            // host code: the quantiser and the layout writer
            let mut c = Command::new(env::var("CXX").unwrap_or_else(|_| "g++".into()));
            c.args(["-O3", "-std=c++17", "-fPIC", "-pthread", "-c"]);
            c
        } else {
            let mut c = Command::new(&hipcc);
            c.arg(format!("--offload-arch={arch}"))
                .args(["-O3", "-std=c++17", "-fPIC", "-c"])
                // packed-f32 VALU instructions are switched off for all device code
                .args(["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]);
            c
        };
        cmd.arg(format!("-I{}", include.display()));
        if let Some(f) = flag {
            cmd.arg(f);
        }
        cmd.arg(csrc.join(src)).arg("-o").arg(&obj);
        assert!(cmd.status().expect("run the compiler").success(), "compiling {src} failed");
        println!("cargo:rerun-if-changed=csrc/{src}");
        objects.push(obj);
    }
    assert!(!objects.is_empty(), "kiln-marlin-gemm: csrc/objects.list names no object");
    for entry in fs::read_dir(&csrc).unwrap().flatten() {
        if entry.path().extension().is_some_and(|e| e == "h") {
            println!("cargo:rerun-if-changed=csrc/{}", entry.file_name().to_string_lossy());
        }
    }
    let lib = out.join("libkiln_marlin_gemm.a");
    assert!(Command::new("ar").arg("crs").arg(&lib).args(&objects).status().unwrap().success());
    println!("cargo:rustc-link-search=native={}", out.display());
    println!("cargo:rustc-link-lib=static=kiln_marlin_gemm");
    println!("cargo:rustc-link-search=native={rocm}/lib");
    println!("cargo:rustc-link-lib=dylib=amdhip64");
    println!("cargo:rustc-link-lib=dylib=stdc++");
    println!("cargo:rerun-if-env-changed=ROCM_PATH");
    println!("cargo:rerun-if-env-changed=KILN_HIP_ARCHS");
}
