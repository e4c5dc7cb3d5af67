// Links librfq.so.  RFQ_LIB_DIR names the directory that holds it (the `rocmforge_amd/` directory of the
// library's source tree after `make -C rocmforge_amd/csrc`); without it the default search path is used.
fn main() {
    println!("cargo:rerun-if-env-changed=RFQ_LIB_DIR");
    if let Ok(dir) = std::env::var("RFQ_LIB_DIR") {
        println!("cargo:rustc-link-search=native={}", dir);
        println!("cargo:rustc-link-arg=-Wl,-rpath,{}", dir);
    }
    println!("cargo:rustc-link-lib=dylib=rfq");
}
