// Links librbmoe.so.  RBMOE_LIB_DIR names the directory that holds it (rustingbrain_amd/ of the
// library's tree after `python -m rustingbrain_amd.build`).
fn main() {
    if let Ok(dir) = std::env::var("RBMOE_LIB_DIR") {
        println!("cargo:rustc-link-search=native={dir}");
        println!("cargo:rustc-link-arg=-Wl,-rpath,{dir}");
    }
    println!("cargo:rustc-link-lib=dylib=rbmoe");
    println!("cargo:rerun-if-env-changed=RBMOE_LIB_DIR");
}
