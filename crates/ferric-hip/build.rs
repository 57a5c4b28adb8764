fn main() {
    // Directory that holds libferric_hip.so (ferric_amd/ of the library's tree after `python -m ferric_amd.build`).
    println!("cargo:rerun-if-env-changed=FERRIC_HIP_LIB_DIR");
    if let Ok(dir) = std::env::var("FERRIC_HIP_LIB_DIR") {
        println!("cargo:rustc-link-search=native={dir}");
        println!("cargo:rustc-link-arg=-Wl,-rpath,{dir}");
    }
}
