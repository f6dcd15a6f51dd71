// build.rs -- compile the HIP sources with hipcc for gfx950 and link them statically
use std::process::Command;
fn main() {
    let out = std::env::var("OUT_DIR").unwrap();
    let src = "vfkv/csrc";
    let mut objs = vec![];
    for f in ["api.hip", "kv_append.hip", "rope_append.hip", "gated_output.hip", "attn_decode.hip", "attn_prefill.hip"] {
        let o = format!("{out}/{}.o", f.trim_end_matches(".hip"));
        let ok = Command::new("/opt/rocm/bin/hipcc")
            .args(["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
                   "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                   "-mllvm", "-amdgpu-mfma-vgpr-form=1", "-mllvm", "-amdgpu-kernarg-preload-count=16",
                   "-c", &format!("{src}/{f}"), "-o", &o])
            .status().unwrap().success();
        assert!(ok, "hipcc failed on {f}");
        objs.push(o);
    }
    let lib = format!("{out}/libvfkv.a");
    assert!(Command::new("ar").arg("crs").arg(&lib).args(&objs).status().unwrap().success());
    println!("cargo:rustc-link-search=native={out}");
    println!("cargo:rustc-link-lib=static=vfkv");
    println!("cargo:rustc-link-search=native=/opt/rocm/lib");
    println!("cargo:rustc-link-lib=dylib=amdhip64");
    println!("cargo:rustc-link-lib=dylib=stdc++");
    println!("cargo:rerun-if-changed={src}");
}
