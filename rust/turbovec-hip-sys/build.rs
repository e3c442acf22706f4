// Links the hipcc-built shared library.  The library is built outside cargo
// (`python -m turbovec_amd.build`: hipcc --offload-arch=gfx950 over turbovec_amd/csrc/), so this
// script only tells rustc where it is.
//
//   TURBOVEC_HIP_LIB_DIR   directory holding libturbovec_hip.so (required)
//   ROCM_PATH              ROCm root, default /opt/rocm (the library depends on libamdhip64.so)
use std::env;
use std::path::PathBuf;

fn main() {
    println!("cargo:rerun-if-env-changed=TURBOVEC_HIP_LIB_DIR");
    println!("cargo:rerun-if-env-changed=ROCM_PATH");
    let dir = PathBuf::from(
        env::var("TURBOVEC_HIP_LIB_DIR")
            .expect("set TURBOVEC_HIP_LIB_DIR to the directory that holds libturbovec_hip.so"),
    );
    if !dir.join("libturbovec_hip.so").exists() {
        panic!("{} holds no libturbovec_hip.so (build it with `python -m turbovec_amd.build`)", dir.display());
    }
    let rocm = env::var("ROCM_PATH").unwrap_or_else(|_| "/opt/rocm".to_string());
    println!("cargo:rustc-link-search=native={}", dir.display());
    println!("cargo:rustc-link-search=native={rocm}/lib");
    println!("cargo:rustc-link-lib=dylib=turbovec_hip");
    println!("cargo:rustc-link-lib=dylib=amdhip64");
    // let binaries and tests find the library without LD_LIBRARY_PATH
    println!("cargo:rustc-link-arg=-Wl,-rpath,{}", dir.display());
    // handed to dependants as DEP_TURBOVEC_HIP_LIB_DIR
    println!("cargo:lib_dir={}", dir.display());
}
