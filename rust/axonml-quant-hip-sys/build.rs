// Points the linker at libaxq.so: AXQ_LIB_DIR, or <repository>/axonml_amd where `make -C axonml_amd/csrc` puts it.
fn main() {
    let dir = std::env::var("AXQ_LIB_DIR").unwrap_or_else(|_| format!("{}/../../axonml_amd", env!("CARGO_MANIFEST_DIR")));
    println!("cargo:rustc-link-search=native={dir}");
    println!("cargo:rustc-link-lib=dylib=axq");
    println!("cargo:rerun-if-env-changed=AXQ_LIB_DIR");
}
