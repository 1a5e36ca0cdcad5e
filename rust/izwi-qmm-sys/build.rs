// Links libizwi_qmm.so.  IZWI_QMM_LIB_DIR names the directory that holds it (the `izwi_amd/`
// folder of this repository after `make -C izwi_amd/csrc`); without it the system's default
// library path is searched.
fn main() {
    println!("cargo:rerun-if-env-changed=IZWI_QMM_LIB_DIR");
    if let Ok(dir) = std::env::var("IZWI_QMM_LIB_DIR") {
        println!("cargo:rustc-link-search=native={dir}");
        println!("cargo:rustc-link-arg=-Wl,-rpath,{dir}");
    }
    println!("cargo:rustc-link-lib=dylib=izwi_qmm");
}
