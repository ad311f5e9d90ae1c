// Tells the linker where libhipcompute.so lives: HIPCOMPUTE_LIB_DIR (the directory that holds the
// library built by `make -C onnx-vulkan-rs_amd/csrc`), else the system's default search path.
fn main() {
    println!("cargo:rerun-if-env-changed=HIPCOMPUTE_LIB_DIR");
    if let Ok(dir) = std::env::var("HIPCOMPUTE_LIB_DIR") {
        println!("cargo:rustc-link-search=native={dir}");
        println!("cargo:rustc-link-arg=-Wl,-rpath,{dir}");
    }
    println!("cargo:rustc-link-lib=dylib=hipcompute");
}
