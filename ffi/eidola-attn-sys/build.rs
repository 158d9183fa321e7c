// Links the prebuilt HIP library.  EIDOLA_ATTN_LIB_DIR names the directory that holds
// libeidola_attn_hip.so (built by `make -C eidola_amd/csrc`); the library itself links the
// HIP runtime, so nothing else is needed on the link line.
fn main() {
    println!("cargo:rerun-if-env-changed=EIDOLA_ATTN_LIB_DIR");
    let dir = std::env::var("EIDOLA_ATTN_LIB_DIR")
        .expect("set EIDOLA_ATTN_LIB_DIR to the directory that holds libeidola_attn_hip.so");
    println!("cargo:rustc-link-search=native={dir}");
    println!("cargo:rustc-link-lib=dylib=eidola_attn_hip");
}
