// Builds libhf2q_hip.so from the HIP sources of this repository with hipcc and links it.
//
// The kernels are gfx950 (MI355X) code: every translation unit under hf2q_amd/csrc is compiled with the flags of
// hf2q_amd/build.py (tests/test_bindings.py keeps the two lists in step), the objects are linked into one shared
// library in OUT_DIR, and cargo is told to link it.  HIPCC names the compiler (default /opt/rocm/bin/hipcc); with
// HF2Q_HIP_LIB_DIR set, nothing is compiled and the library already built there (python -m hf2q_amd.build) is linked
// instead.
use std::env;
use std::path::{Path, PathBuf};
use std::process::Command;

// Translation units of the library (hf2q_amd/csrc/*.hip).
const SOURCES: &[&str] = &[
    "api.hip",
    "blocks.hip",
    "dense.hip",
    "dense_ffn.hip",
    "dequant.hip",
    "gemm.hip",
    "gemm_f16.hip",
    "gemv.hip",
    "gemvm.hip",
    "gemvr32.hip",
    "gguf.hip",
    "moe.hip",
    "moe_fused.hip",
    "quantize.hip",
    "shadow.hip",
    "tq.hip",
    "tqp.hip",
];

// Libraries the shared object is linked against beside the HIP runtime (the vendor GEMM behind hq_matmul_f16_shadow).
const LINK_LIBS: &[&str] = &["-lhipblaslt"];

// Flags of every compile; -Xclang -target-feature -Xclang -packed-fp32-ops keeps the compiler from forming packed-fp32
// VALU operations.
const FLAGS: &[&str] = &[
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fvisibility=hidden",
    "-Wall",
    "-Wextra",
    "-Wno-unused-parameter",
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
];

// Translation units whose arithmetic must not be contracted (the byte-exact quantizers).
const STRICT_FP: &[(&str, &str)] = &[("quantize.hip", "-ffp-contract=off")];

fn run(cmd: &mut Command) {
    let status = cmd.status().unwrap_or_else(|e| panic!("failed to start {:?}: {}", cmd, e));
    assert!(status.success(), "{:?} failed with {}", cmd, status);
}

fn main() {
    println!("cargo:rerun-if-env-changed=HF2Q_HIP_LIB_DIR");
    println!("cargo:rerun-if-env-changed=HIPCC");
    println!("cargo:rerun-if-env-changed=ROCM_PATH");
    let manifest = PathBuf::from(env::var("CARGO_MANIFEST_DIR").unwrap());
    let root = manifest.join("../..");
    let csrc = root.join("hf2q_amd/csrc");
    println!("cargo:rerun-if-changed={}", root.join("include/hf2q_hip.h").display());
    let rocm = env::var("ROCM_PATH").unwrap_or_else(|_| "/opt/rocm".to_string());

    let lib_dir: PathBuf = if let Ok(dir) = env::var("HF2Q_HIP_LIB_DIR") {
        PathBuf::from(dir)
    } else {
        let hipcc = env::var("HIPCC").unwrap_or_else(|_| format!("{}/bin/hipcc", rocm));
        let out = PathBuf::from(env::var("OUT_DIR").unwrap());
        for entry in std::fs::read_dir(&csrc).expect("hf2q_amd/csrc") {
            let p = entry.unwrap().path();
            if p.extension().map_or(false, |e| e == "h" || e == "hip") {
                println!("cargo:rerun-if-changed={}", p.display());
            }
        }
        let mut objects = Vec::new();
        for src in SOURCES {
            let obj = out.join(Path::new(src).with_extension("o"));
            let mut cmd = Command::new(&hipcc);
            cmd.args(FLAGS);
            for (file, flag) in STRICT_FP {
                if file == src {
                    cmd.arg(flag);
                }
            }
            cmd.arg("-c").arg(csrc.join(src)).arg("-o").arg(&obj);
            run(&mut cmd);
            objects.push(obj);
        }
        let mut link = Command::new(&hipcc);
        link.args(["--offload-arch=gfx950", "-shared", "-fPIC", "-o"]).arg(out.join("libhf2q_hip.so")).args(&objects).args(LINK_LIBS);
        run(&mut link);
        out
    };
    println!("cargo:rustc-link-search=native={}", lib_dir.display());
    println!("cargo:rustc-link-lib=dylib=hf2q_hip");
    // the HIP runtime the library itself is linked against
    println!("cargo:rustc-link-search=native={}/lib", rocm);
    println!("cargo:rustc-link-arg=-Wl,-rpath,{}", lib_dir.display());
}
