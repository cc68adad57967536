// Tells cargo where libmgn_hip.so lives.  MGN_HIP_LIB_DIR is the directory that holds it
// (`make -C meganeura_amd/csrc` writes it to meganeura_amd/); without the variable the
// linker's default search path is used.
fn main() {
    println!("cargo:rerun-if-env-changed=MGN_HIP_LIB_DIR");
    if let Ok(dir) = std::env::var("MGN_HIP_LIB_DIR") {
        println!("cargo:rustc-link-search=native={}", dir);
        println!("cargo:rustc-link-arg=-Wl,-rpath,{}", dir);
    }
    println!("cargo:rustc-link-lib=dylib=mgn_hip");
}
