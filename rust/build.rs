//! Compiles the HIP units of `comfyui-backend-but-rust_amd/csrc` for gfx950 with hipcc, archives them into
//! `libgpu_kernels.a`, builds the hipBLASLt wrapper into `libgpu_blas.a`, and tells cargo to link both together with
//! the HIP runtime.  This takes the place of the reference's nvcc step (its build.rs:69-93,131-141) for the units of
//! the quantized-linear path.  The unit list and the flags are the ones of the package's build.py and Makefile; the
//! floating-point flags matter for bit-exact results.
use std::env;
use std::path::{Path, PathBuf};
use std::process::Command;

const UNITS: &[&str] = &[
    "quant_rows.hip", "prologue_rows.hip", "weight_formats.hip", "act_tables.hip", "int8_gemm.hip", "w6.hip",
    "w6_requant.hip", "w6a8_group_gemm.hip", "attn_int8.hip",
];

fn run(cmd: &mut Command) {
    let status = cmd.status().unwrap_or_else(|e| panic!("cannot start {:?}: {}", cmd, e));
    assert!(status.success(), "{:?} failed with {}", cmd, status);
}

fn main() {
    let manifest = PathBuf::from(env::var("CARGO_MANIFEST_DIR").unwrap());
    let csrc = manifest.join("..").join("comfyui-backend-but-rust_amd").join("csrc");
    let include = manifest.join("..").join("include");
    let out = PathBuf::from(env::var("OUT_DIR").unwrap());
    let arch = env::var("HIP_ARCH").unwrap_or_else(|_| "gfx950".to_string());
    let rocm = env::var("ROCM_PATH").unwrap_or_else(|_| "/opt/rocm".to_string());
    let hipcc = Path::new(&rocm).join("bin").join("hipcc");

    let mut objects = Vec::new();
    for unit in UNITS {
        let obj = out.join(unit.replace(".hip", ".o"));
        let mut cmd = Command::new(&hipcc);
        cmd.arg(format!("--offload-arch={arch}"))
            .args(["-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden"])
            // exact arithmetic: no contraction except where fmaf is written, IEEE divide, no fast-math
            .args(["-ffp-contract=off", "-fno-fast-math", "-fhip-fp32-correctly-rounded-divide-sqrt"])
            // keep the compiler from forming packed-fp32 instructions
            .args(["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"])
            .arg("-Wno-inline-asm");
        if *unit == "w6a8_group_gemm.hip" {
            // its VALU fold reads every MFMA result: keep them out of accumulator registers
            cmd.args(["-mllvm", "-amdgpu-mfma-vgpr-form"]);
        }
        cmd.arg("-I").arg(&include).arg("-c").arg(csrc.join(unit)).arg("-o").arg(&obj);
        run(&mut cmd);
        println!("cargo:rerun-if-changed={}", csrc.join(unit).display());
        objects.push(obj);
    }
    let kernels = out.join("libgpu_kernels.a");
    let _ = std::fs::remove_file(&kernels);
    run(Command::new("ar").arg("crs").arg(&kernels).args(&objects));

    // host-only C++ over hipBLASLt
    let blas_obj = out.join("blas_gemm.o");
    run(Command::new(&hipcc)
        .args(["-O2", "-std=c++17", "-fPIC", "-fvisibility=hidden"])
        .arg("-I").arg(&include)
        .arg("-c").arg(csrc.join("blas_gemm.cpp")).arg("-o").arg(&blas_obj));
    let blas = out.join("libgpu_blas.a");
    let _ = std::fs::remove_file(&blas);
    run(Command::new("ar").arg("crs").arg(&blas).arg(&blas_obj));

    for header in ["gpu_api.h", "gpu_blas_api.h"] {
        println!("cargo:rerun-if-changed={}", include.join(header).display());
    }
    println!("cargo:rerun-if-changed={}", csrc.join("blas_gemm.cpp").display());
    println!("cargo:rerun-if-env-changed=HIP_ARCH");
    println!("cargo:rerun-if-env-changed=ROCM_PATH");
    println!("cargo:rustc-link-search=native={}", out.display());
    println!("cargo:rustc-link-search=native={}/lib", rocm);
    println!("cargo:rustc-link-lib=static=gpu_kernels");
    println!("cargo:rustc-link-lib=static=gpu_blas");
    println!("cargo:rustc-link-lib=dylib=hipblaslt");
    println!("cargo:rustc-link-lib=dylib=amdhip64");
    println!("cargo:rustc-link-lib=dylib=stdc++");
}
