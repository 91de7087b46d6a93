// Points the linker at libferrotensor_hip.so: FERROTENSOR_HIP_LIB_DIR, or ../../ferrotensor_amd
// (where `python -m ferrotensor_amd.build` puts it), plus the HIP runtime.
fn main() {
    let dir = std::env::var("FERROTENSOR_HIP_LIB_DIR").unwrap_or_else(|_| {
        format!("{}/../../ferrotensor_amd", std::env::var("CARGO_MANIFEST_DIR").unwrap())
    });
    println!("cargo:rustc-link-search=native={dir}");
    println!("cargo:rustc-link-lib=dylib=ferrotensor_hip");
    println!("cargo:rustc-link-search=native=/opt/rocm/lib");
    println!("cargo:rustc-link-lib=dylib=amdhip64");
    println!("cargo:rerun-if-env-changed=FERROTENSOR_HIP_LIB_DIR");
}
