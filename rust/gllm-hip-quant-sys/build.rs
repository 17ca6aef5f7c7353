// Links libgllm_hip_quant.so; GLLM_HIP_QUANT_LIB_DIR names the directory that holds it.
fn main() {
    if let Ok(dir) = std::env::var("GLLM_HIP_QUANT_LIB_DIR") {
        println!("cargo:rustc-link-search=native={dir}");
        println!("cargo:rustc-link-arg=-Wl,-rpath,{dir}");
    }
    println!("cargo:rustc-link-lib=dylib=gllm_hip_quant");
    println!("cargo:rerun-if-env-changed=GLLM_HIP_QUANT_LIB_DIR");
}
