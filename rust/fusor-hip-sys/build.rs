//! Links `libfusor_hip.a`, the hipcc-built static library behind `include/fusor_hip.h`.
//!
//! Two ways to get the archive, chosen by environment variables:
//!   * `FUSOR_HIP_LIB_DIR=<dir>`: use the prebuilt `<dir>/libfusor_hip.a`
//!     (`python -m floneum_amd.build` leaves one in `floneum_amd/`);
//!   * otherwise compile `floneum_amd/csrc/*.hip` here with hipcc for gfx950 and archive the objects
//!     into `$OUT_DIR`.  `FUSOR_HIP_ROOT` names the checkout (default: two directories above this crate),
//!     `HIPCC` the compiler (default `/opt/rocm/bin/hipcc`), `ROCM_PATH` the ROCm prefix (default `/opt/rocm`).
use std::env;
use std::path::{Path, PathBuf};
use std::process::Command;

const SOURCES: &[&str] = &[
    "api.hip",
    "attn_generic.hip",
    "attn_decode.hip",
    "attn_prefill_mfma.hip",
    "attn_prefill_mfma_wide.hip",
    "attn_prefill_mfma_rows32.hip",
    "attn_prefill_mfma_rows64.hip",
    "attn_prefill_f32.hip",
    "kv_cache.hip",
    "mask_intervals.hip",
    "rope.hip",
    "calibration.hip",
];

// the flags floneum_amd/build.py uses; packed-f32 VALU forms are kept out of the generated code on purpose
const FLAGS: &[&str] = &[
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
];

fn run(cmd: &mut Command) {
    let status = cmd.status().unwrap_or_else(|e| panic!("cannot start {cmd:?}: {e}"));
    assert!(status.success(), "{cmd:?} failed with {status}");
}

fn compile(root: &Path, out_dir: &Path) {
    let hipcc = env::var("HIPCC").unwrap_or_else(|_| "/opt/rocm/bin/hipcc".into());
    let csrc = root.join("floneum_amd").join("csrc");
    let mut objects = Vec::new();
    for src in SOURCES {
        let path = csrc.join(src);
        println!("cargo:rerun-if-changed={}", path.display());
        let obj = out_dir.join(src.replace(".hip", ".o"));
        let mut cmd = Command::new(&hipcc);
        cmd.args(FLAGS);
        if *src == "rope.hip" {
            // the rotary embedding rounds every product and sum on its own (bit parity with fusor's CPU ops)
            cmd.arg("-ffp-contract=off");
        }
        cmd.arg("-c").arg(&path).arg("-o").arg(&obj);
        run(&mut cmd);
        objects.push(obj);
    }
    for header in ["common.h", "device_utils.h", "attn_bounds.h"] {
        println!("cargo:rerun-if-changed={}", csrc.join(header).display());
    }
    let archive = out_dir.join("libfusor_hip.a");
    let _ = std::fs::remove_file(&archive);
    run(Command::new("ar").arg("rcs").arg(&archive).args(&objects));
}

fn main() {
    println!("cargo:rerun-if-env-changed=FUSOR_HIP_LIB_DIR");
    println!("cargo:rerun-if-env-changed=FUSOR_HIP_ROOT");
    println!("cargo:rerun-if-env-changed=HIPCC");
    println!("cargo:rerun-if-env-changed=ROCM_PATH");
    let out_dir = PathBuf::from(env::var("OUT_DIR").unwrap());
    let lib_dir = match env::var("FUSOR_HIP_LIB_DIR") {
        Ok(dir) => PathBuf::from(dir),
        Err(_) => {
            let root = env::var("FUSOR_HIP_ROOT").map(PathBuf::from).unwrap_or_else(|_| {
                PathBuf::from(env::var("CARGO_MANIFEST_DIR").unwrap()).join("..").join("..")
            });
            compile(&root, &out_dir);
            out_dir
        }
    };
    let rocm = env::var("ROCM_PATH").unwrap_or_else(|_| "/opt/rocm".into());
    println!("cargo:rustc-link-search=native={}", lib_dir.display());
    println!("cargo:rustc-link-lib=static=fusor_hip");
    println!("cargo:rustc-link-search=native={rocm}/lib");
    println!("cargo:rustc-link-lib=dylib=amdhip64");
    println!("cargo:rustc-link-lib=dylib=stdc++");
}
