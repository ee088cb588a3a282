//! Links libforja_hip.so.  `FORJA_HIP_LIB_DIR` names the directory that holds it (the
//! `forja_amd/` directory of the forja-hip build tree after `python -m forja_amd.build`).
fn main() {
    println!("cargo:rerun-if-env-changed=FORJA_HIP_LIB_DIR");
    if let Ok(directory) = std::env::var("FORJA_HIP_LIB_DIR") {
        println!("cargo:rustc-link-search=native={directory}");
        println!("cargo:rustc-link-arg=-Wl,-rpath,{directory}");
    }
    println!("cargo:rustc-link-lib=dylib=forja_hip");
}
