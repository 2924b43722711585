// Links libperegrine_hip.so (built by `make -C peregrine_amd/csrc`, which needs hipcc).
// PEREGRINE_HIP_LIB_DIR names the directory that holds it; by default the in-tree location
// relative to this crate.
fn main() {
    let dir = std::env::var("PEREGRINE_HIP_LIB_DIR").unwrap_or_else(|_| {
        let here = std::env::var("CARGO_MANIFEST_DIR").expect("cargo sets CARGO_MANIFEST_DIR");
        format!("{here}/../../peregrine_amd/lib")
    });
    println!("cargo:rustc-link-search=native={dir}");
    println!("cargo:rustc-link-lib=dylib=peregrine_hip");
    println!("cargo:rustc-link-arg=-Wl,-rpath,{dir}");
    println!("cargo:rerun-if-env-changed=PEREGRINE_HIP_LIB_DIR");
}
