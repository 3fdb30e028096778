// Locates (or builds) libferrox_hip.so and tells cargo to link it.
//   FERROX_HIP_LIB_DIR  directory that already holds libferrox_hip.so (e.g. <repo>/ferrox_amd)
//   FERROX_HIP_REPO     checkout of the library's sources; the library is built there with
//                       `python3 -m ferrox_amd.build` (hipcc --offload-arch=gfx950) when the variable above is unset
// This replaces the reference's build.rs, which compiles kernels/*.cu to PTX with nvcc.
use std::env;
use std::path::PathBuf;
use std::process::Command;

fn main() {
    println!("cargo:rerun-if-env-changed=FERROX_HIP_LIB_DIR");
    println!("cargo:rerun-if-env-changed=FERROX_HIP_REPO");
    let dir = if let Ok(dir) = env::var("FERROX_HIP_LIB_DIR") {
        PathBuf::from(dir)
    } else {
        let repo = PathBuf::from(env::var("FERROX_HIP_REPO").expect("set FERROX_HIP_LIB_DIR or FERROX_HIP_REPO"));
        let status = Command::new("python3")
            .args(["-m", "ferrox_amd.build"])
            .current_dir(&repo)
            .status()
            .expect("failed to run the library build");
        assert!(status.success(), "building libferrox_hip.so failed");
        repo.join("ferrox_amd")
    };
    println!("cargo:rustc-link-search=native={}", dir.display());
    println!("cargo:rustc-link-lib=dylib=ferrox_hip");
    println!("cargo:rustc-link-arg=-Wl,-rpath,{}", dir.display());
}
