// libughip.so is built outside cargo (python -m ug_amd.build, or hipcc on ug_amd/csrc/ughip/*).
// UGHIP_LIB_DIR names the directory that holds it; it also becomes the binary's rpath so that
// `cargo test` finds the library without LD_LIBRARY_PATH.
fn main() {
    println!("cargo:rerun-if-env-changed=UGHIP_LIB_DIR");
    if let Ok(dir) = std::env::var("UGHIP_LIB_DIR") {
        println!("cargo:rustc-link-search=native={dir}");
        println!("cargo:rustc-link-arg=-Wl,-rpath,{dir}");
    }
    println!("cargo:rustc-link-lib=dylib=ughip");
}
