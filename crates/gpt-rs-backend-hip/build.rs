//! Builds `libgptrs_hip.so` with hipcc (through the repository's build script) and links it.
//! Not compiled in this repository's build image (no Rust toolchain there).
use std::{env, path::PathBuf, process::Command};

fn main() {
    // <repo>/crates/gpt-rs-backend-hip -> <repo>/gpt.rs_amd
    let root = PathBuf::from(env::var("CARGO_MANIFEST_DIR").unwrap()).join("../..");
    let pkg = root.join("gpt.rs_amd");
    // python gpt.rs_amd/build.py == hipcc --offload-arch=gfx950 -O3 -fPIC ... -shared -o libgptrs_hip.so
    let status = Command::new("python3").arg(pkg.join("build.py")).status().expect("python3 not found");
    assert!(status.success(), "hipcc build of libgptrs_hip.so failed");
    println!("cargo:rustc-link-search=native={}", pkg.display());
    println!("cargo:rustc-link-lib=dylib=gptrs_hip");
    println!("cargo:rerun-if-changed={}", pkg.join("csrc").display());
    println!("cargo:rerun-if-changed={}", root.join("include/gptrs_hip.h").display());
}
