// Link against librlx_mi355x.so. RLX_MI355X_LIB_DIR points at the directory that holds it
// (the `rlx_amd/` folder of the library's source tree after `make -C rlx_amd/csrc`).
fn main() {
    if let Ok(dir) = std::env::var("RLX_MI355X_LIB_DIR") {
        println!("cargo:rustc-link-search=native={dir}");
        println!("cargo:rustc-link-arg=-Wl,-rpath,{dir}");
    }
    println!("cargo:rustc-link-lib=dylib=rlx_mi355x");
    println!("cargo:rerun-if-env-changed=RLX_MI355X_LIB_DIR");
}
