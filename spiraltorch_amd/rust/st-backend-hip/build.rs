// Links libsthip.so (which itself links libamdhip64).  STHIP_LIB_DIR names the directory that holds it; the
// reference's build.rs compiled hip_kernels/*.cu with hipcc and archived them (build.rs:51-78) — that step is gone,
// the kernels are built by spiraltorch_amd/csrc/Makefile.
use std::env;

fn main() {
    println!("cargo:rerun-if-env-changed=STHIP_LIB_DIR");
    if let Ok(dir) = env::var("STHIP_LIB_DIR") {
        println!("cargo:rustc-link-search=native={dir}");
        println!("cargo:rustc-link-arg=-Wl,-rpath,{dir}");
    }
    println!("cargo:rustc-link-lib=dylib=sthip");
}
