// build.rs of the crate that carries the optimizer (drop-in for crates/core/build.rs:1-21, which
// drives nvcc through `cc::Build::cuda(true)` with -arch=sm_80).  Here the native side is
// hand-written HIP for gfx950, compiled by hipcc; there is no CUDA path and no feature switch.
//
// Source text only: this repository's build environment has no Rust toolchain, so the file is
// exercised by the reference's maintainers, not by this repository's tests.
use std::env;
use std::path::PathBuf;
use std::process::Command;

fn main() {
    let out = PathBuf::from(env::var("OUT_DIR").unwrap());
    let src = PathBuf::from(env::var("CARGO_MANIFEST_DIR").unwrap()).join("csrc");
    let hipcc = env::var("HIPCC").unwrap_or_else(|_| "/opt/rocm/bin/hipcc".to_string());
    let arch = env::var("ERI_HIP_ARCH").unwrap_or_else(|_| "gfx950".to_string());

    let device_flags = [
        format!("--offload-arch={arch}"),
        "-O3".into(),
        "-fPIC".into(),
        "-std=c++17".into(),
        // every fp32 operation of the update rounds on its own, as the reference's chain of
        // tensor ops does (src/trainers/adam8bit_enhanced.rs:252-275)
        "-ffp-contract=off".into(),
        "-Xclang".into(),
        "-target-feature".into(),
        "-Xclang".into(),
        "-packed-fp32-ops".into(),
    ];
    let mut objects = Vec::new();
    // (source, object name, extra define, compiled as HIP?) -- the plain step kernel is built once per
    // parameter dtype
    for (file, obj_name, define, is_hip) in [
        ("eri_adam8_kernels.hip", "kernels", "", true),
        ("eri_adam8_step_split.hip", "step_split", "", true),
        ("eri_adam8_step_pipelined.hip", "step_pipelined", "-DERI_PIPE_LAYOUT=1", true),
        ("eri_adam8_step_pipelined.hip", "step_pipelined_grad_f32", "-DERI_PIPE_LAYOUT=2", true),
        ("eri_adam8_step_pipelined.hip", "step_pipelined_f32", "-DERI_PIPE_LAYOUT=0", true),
        ("eri_adam8_step_plain.hip", "step_plain_bf16", "-DERI_PLAIN_BF16=1", true),
        ("eri_adam8_step_plain.hip", "step_plain_f32", "-DERI_PLAIN_BF16=0", true),
        ("eri_optim8_api.cpp", "api", "", true),
        ("eri_adam8bit_host.cpp", "host", "", false),
    ] {
        let obj = out.join(format!("{obj_name}.o"));
        let mut cmd = Command::new(&hipcc);
        if !define.is_empty() {
            cmd.arg(define);
        }
        if is_hip {
            cmd.args(&device_flags).args(["-x", "hip"]);
        } else {
            cmd.args(["-O2", "-fPIC", "-std=c++17"]);
        }
        let status = cmd.arg("-c").arg(src.join(file)).arg("-o").arg(&obj).status().expect("hipcc not found");
        assert!(status.success(), "hipcc failed on {file}");
        objects.push(obj);
        println!("cargo:rerun-if-changed=csrc/{file}");
    }
    let lib = out.join("liberi_optim8.a");
    let status = Command::new("ar").arg("crs").arg(&lib).args(&objects).status().expect("ar not found");
    assert!(status.success());

    println!("cargo:rustc-link-search=native={}", out.display());
    println!("cargo:rustc-link-lib=static=eri_optim8");
    println!("cargo:rustc-link-search=native=/opt/rocm/lib");
    println!("cargo:rustc-link-lib=dylib=amdhip64");
    println!("cargo:rustc-link-lib=dylib=stdc++");
    for h in ["eri_adam8_device.h", "eri_adam8_inline.h", "eri_dynamic_maps.inc"] {
        println!("cargo:rerun-if-changed=csrc/{h}");
    }
}
