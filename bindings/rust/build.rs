// Links libsliced_hip.so.  SLICED_HIP_LIB_DIR names the directory that holds it (the
// `sliced_amd/` directory of the library's tree after `python -m sliced_amd.build`).
fn main() {
    let dir = std::env::var("SLICED_HIP_LIB_DIR")
        .expect("set SLICED_HIP_LIB_DIR to the directory that holds libsliced_hip.so");
    println!("cargo:rustc-link-search=native={dir}");
    println!("cargo:rustc-link-lib=dylib=sliced_hip");
    println!("cargo:rustc-link-arg=-Wl,-rpath,{dir}");
    println!("cargo:rerun-if-env-changed=SLICED_HIP_LIB_DIR");
}
