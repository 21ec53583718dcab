// Builds libatenia_moe_hip.a for gfx950 with hipcc and tells rustc to link it.
//
// Same shape as the reference's build script (build.rs:201-231 declare the cfg and return early
// for a CPU-only build; :378-419 compile one object per kernel file; :438-453 archive with
// `ar rcs`; :349-375 link directives, cfg set last).  hipcc --offload-arch=gfx950 is the only
// compiler invoked: no CUDA headers, no second backend.
use std::env;
use std::path::{Path, PathBuf};
use std::process::Command;

// The translation units of the library.  Must equal SRCS of ateniaengine_amd/csrc/Makefile.
const SOURCES: &[&str] = &[
    "moe_abi.hip",
    "router.hip",
    "permute.hip",
    "ffn_stream.hip",
    "ffn_tiled.hip",
    "ffn_tiled_duo.hip",
    "ffn_f32.hip",
    "combine.hip",
    "norm.hip",
    "v3_route.hip",
    "dequant.hip",
];

// Kernels that restate f32 arithmetic of the reference with one rounding per operation: compiled
// without contraction of a * b + c into FMA (hipcc's default is -ffp-contract=fast, which would
// silently change the combine, the RMSNorm and the f32 expert path in the last bit).
const NO_CONTRACT: &[&str] = &["combine.hip", "norm.hip", "ffn_f32.hip"];

const HIPCC_FLAGS: &[&str] = &[
    "--offload-arch=gfx950",
    "-O3",
    "-fPIC",
    "-std=c++17",
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
];

// The hipcc release the kernels' generated code was validated with (HIPCC_VALIDATED of the
// Makefile): the inline-assembly wait states of ffn_tiled.hip and the checks of
// tests/test_isa_guards.py were read against this release's assembly.
const HIPCC_VALIDATED: &str = "7.2";

fn hipcc_release(hipcc: &Path) -> Option<String> {
    let out = Command::new(hipcc).arg("--version").output().ok()?;
    let text = String::from_utf8_lossy(&out.stdout).to_string();
    let v = text.lines().find_map(|l| l.strip_prefix("HIP version: "))?;
    let mut it = v.split('.');
    Some(format!("{}.{}", it.next()?, it.next()?))
}

fn find_hipcc() -> Option<PathBuf> {
    let rocm = env::var("ROCM_PATH").unwrap_or_else(|_| "/opt/rocm".to_string());
    let p = Path::new(&rocm).join("bin").join("hipcc");
    if p.exists() { Some(p) } else { None }
}

fn main() {
    // Declared on every path, also the CPU-only one, so that `#[cfg(atenia_hip)]` never trips
    // the unexpected_cfgs lint; SET only on the success path, as the last action.
    println!("cargo::rustc-check-cfg=cfg(atenia_hip)");
    println!("cargo::rerun-if-env-changed=ROCM_PATH");
    println!("cargo::rerun-if-env-changed=ATENIA_MOE_HIP_CSRC");

    let hipcc = match find_hipcc() {
        Some(p) => p,
        None => {
            eprintln!("[build.rs] hipcc not found under ROCM_PATH (/opt/rocm)");
            eprintln!("[build.rs] Skipping HIP kernel compilation (CPU-only build)");
            return;
        }
    };
    match hipcc_release(&hipcc) {
        Some(v) if v == HIPCC_VALIDATED => {}
        other => println!(
            "cargo::warning=hipcc release {:?} differs from the validated {}: run tests/test_isa_guards.py \
             against it before trusting the tiled kernels",
            other, HIPCC_VALIDATED
        ),
    }
    let manifest = PathBuf::from(env::var("CARGO_MANIFEST_DIR").unwrap());
    let csrc = env::var("ATENIA_MOE_HIP_CSRC")
        .map(PathBuf::from)
        .unwrap_or_else(|_| manifest.join("../../ateniaengine_amd/csrc"));
    let header = csrc.join("../../include/atenia_moe_hip.h");
    println!("cargo::rerun-if-changed={}", header.display());
    println!("cargo::rerun-if-changed={}", csrc.join("select_wave.h").display());
    println!("cargo::rerun-if-changed={}", csrc.join("moe_internal.h").display());

    let out = PathBuf::from(env::var("OUT_DIR").unwrap());
    let mut objects = Vec::new();
    for src in SOURCES {
        let input = csrc.join(src);
        let object = out.join(format!("{src}.o"));
        println!("cargo::rerun-if-changed={}", input.display());
        let mut cmd = Command::new(&hipcc);
        cmd.args(HIPCC_FLAGS);
        if NO_CONTRACT.contains(src) {
            cmd.arg("-ffp-contract=off");
        }
        cmd.arg("-c").arg(&input).arg("-o").arg(&object);
        let output = cmd.output().expect("failed to run hipcc");
        if !output.status.success() {
            eprintln!("---- HIPCC STDERR ----\n{}", String::from_utf8_lossy(&output.stderr));
            panic!("HIP kernel compilation failed for {src}");
        }
        objects.push(object);
    }

    let archive = out.join("libatenia_moe_hip.a");
    let _ = std::fs::remove_file(&archive);
    let status = Command::new("ar")
        .arg("rcs")
        .arg(&archive)
        .args(&objects)
        .status()
        .expect("failed to create the static library with ar");
    assert!(status.success(), "ar rcs failed");

    let rocm = env::var("ROCM_PATH").unwrap_or_else(|_| "/opt/rocm".to_string());
    println!("cargo::rustc-link-search=native={}", out.display());
    println!("cargo::rustc-link-search=native={rocm}/lib");
    println!("cargo::rustc-link-lib=static=atenia_moe_hip");
    println!("cargo::rustc-link-lib=dylib=amdhip64");
    println!("cargo::rustc-link-lib=dylib=stdc++");

    // Reached only when hipcc was found and every kernel compiled and was archived above.
    println!("cargo::rustc-cfg=atenia_hip");
}
