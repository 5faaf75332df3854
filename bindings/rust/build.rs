// Builds libellm_attn.so with hipcc for gfx950 (through the library's own Makefile, which
// carries the flags: --offload-arch=gfx950 -O3, packed FP32 operations disabled) and tells
// cargo to link it.  gfx950 only: there is no second code path to select.
use std::env;
use std::path::PathBuf;
use std::process::Command;

fn main() {
    // bindings/rust/ -> repository root
    let root = PathBuf::from(env::var("CARGO_MANIFEST_DIR").unwrap()).join("../..");
    let csrc = root.join("ellm_amd/csrc");
    let lib_dir = root.join("ellm_amd/lib");
    let hipcc = env::var("HIPCC").unwrap_or_else(|_| "/opt/rocm/bin/hipcc".to_string());

    let status = Command::new("make")
        .arg("-C")
        .arg(&csrc)
        .arg(format!("HIPCC={hipcc}"))
        .arg("ARCH=gfx950")
        .arg(format!("-j{}", env::var("NUM_JOBS").unwrap_or_else(|_| "8".to_string())))
        .status()
        .expect("could not run make (is hipcc installed?)");
    assert!(status.success(), "building libellm_attn.so failed");

    println!("cargo:rustc-link-search=native={}", lib_dir.display());
    println!("cargo:rustc-link-lib=dylib=ellm_attn");
    // so that binaries find the library without LD_LIBRARY_PATH
    println!("cargo:rustc-link-arg=-Wl,-rpath,{}", lib_dir.display());
    for f in [
        "api.hip", "attn_general.hip", "noalloc.hip", "decode.hip", "decode_balanced.hip", "prefill.hip", "kv_cache.hip",
        "project.hip", "project_mid.hip", "project_small.hip", "project_api.hip", "step.hip", "handles.hpp", "common.hpp",
        "kernels.hpp", "decode_common.hpp", "decode_plan.hpp", "decode_shares.hpp", "chunk_plan.hpp", "project_common.hpp",
        "project_epilogue.hpp", "Makefile",
    ] {
        println!("cargo:rerun-if-changed={}", csrc.join(f).display());
    }
    println!("cargo:rerun-if-changed={}", root.join("include/ellm_attn.h").display());
    println!("cargo:rerun-if-env-changed=HIPCC");
}
