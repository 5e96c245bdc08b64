// Points the linker at libcoeus_mi355x.so: COEUS_LIB_DIR = the directory that holds it
// (coeus_amd/ in the source tree of the library).
fn main() {
    let dir = std::env::var("COEUS_LIB_DIR").expect("set COEUS_LIB_DIR to the directory of libcoeus_mi355x.so");
    println!("cargo:rustc-link-search=native={dir}");
    println!("cargo:rustc-link-lib=dylib=coeus_mi355x");
    println!("cargo:rerun-if-env-changed=COEUS_LIB_DIR");
}
