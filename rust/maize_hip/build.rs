// Points the linker at libmaize_hip.so (built by `make -C maize_amd/csrc` into maize_amd/lib).
fn main() {
    let dir = std::env::var("MAIZE_HIP_LIB_DIR").unwrap_or_else(|_| "../../maize_amd/lib".to_string());
    println!("cargo:rustc-link-search=native={dir}");
    println!("cargo:rustc-link-arg=-Wl,-rpath,{dir}");
    println!("cargo:rerun-if-env-changed=MAIZE_HIP_LIB_DIR");
}
