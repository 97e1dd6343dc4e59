// Links libratchet_hip.so.  RATCHET_HIP_LIB_DIR names the directory that holds it (the
// `ratchet_amd/` directory of a checkout after `python -m ratchet_amd.build`).
// Not compiled in this repository's build image (no rustc there).
fn main() {
    let dir = std::env::var("RATCHET_HIP_LIB_DIR").expect("set RATCHET_HIP_LIB_DIR to the directory of libratchet_hip.so");
    println!("cargo:rustc-link-search=native={dir}");
    println!("cargo:rustc-link-lib=dylib=ratchet_hip");
    println!("cargo:rerun-if-env-changed=RATCHET_HIP_LIB_DIR");
}
