// Links against librumus_hip.so.  RUMUS_HIP_LIB_DIR points at the directory that holds it
// (rumus_amd/ in the rumus-hip repository after `make -C rumus_amd/csrc`).
fn main() {
    if let Ok(dir) = std::env::var("RUMUS_HIP_LIB_DIR") {
        println!("cargo:rustc-link-search=native={dir}");
    }
    println!("cargo:rustc-link-lib=dylib=rumus_hip");
    println!("cargo:rerun-if-env-changed=RUMUS_HIP_LIB_DIR");
}
