// Links the prebuilt shared libraries (python -m pie_amd.build writes them into pie_amd/).
// PIE_HIP_LIB_DIR overrides the directory.
use std::env;
use std::path::PathBuf;

fn main() {
    let dir = env::var("PIE_HIP_LIB_DIR").map(PathBuf::from).unwrap_or_else(|_| {
        PathBuf::from(env::var("CARGO_MANIFEST_DIR").unwrap()).join("../..")
    });
    println!("cargo:rustc-link-search=native={}", dir.display());
    println!("cargo:rustc-link-lib=dylib=pie_driver_hip");
    println!("cargo:rustc-link-lib=dylib=pie_hip_kernels");
    println!("cargo:rustc-link-arg=-Wl,-rpath,{}", dir.display());
    println!("cargo:rerun-if-env-changed=PIE_HIP_LIB_DIR");
}
