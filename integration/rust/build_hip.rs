// The `hip` block of `libs/rtensors/build.rs`, next to the CUDA block (build.rs:342-532): compiles the HIP sources of the backend with
// hipcc and links the result, so that `cargo build --features hip` needs nothing but a ROCm toolchain.
//
// Layout expected in the crate: `hip/csrc/*.hip`, `hip/csrc/*.h`, `hip/csrc/build_flags.txt` and `hip/include/rt_hip.h` (this
// repository's `rtensors_amd/csrc/` and `include/`, copied as they are).  `build_flags.txt` is the one description of the build:
// compile flags, source list, headers and link flags, with `{arch}` standing for the target.  The Python builder of this repository
// (`python -m rtensors_amd.build`) reads the same file, so both produce the same library.
//
// Environment:
//   HIPCC_PATH    full path of hipcc (else $ROCM_PATH/bin/hipcc, /opt/rocm/bin/hipcc, then `hipcc` on PATH)
//   RT_HIP_ARCH   offload target (default gfx950; the kernels are written for CDNA4 only)
//   RT_HIP_LIB_DIR  directory of a prebuilt librt_hip.so: skips the compilation (what CI without a ROCm toolchain uses)
//
// In `main()`:   #[cfg(feature = "hip")] build_hip();

#[cfg(feature = "hip")]
fn find_hipcc() -> Option<std::path::PathBuf> {
    use std::path::PathBuf;
    if let Ok(p) = std::env::var("HIPCC_PATH") {
        let p = PathBuf::from(p);
        if p.exists() {
            return Some(p);
        }
    }
    for root in [std::env::var("ROCM_PATH").ok(), std::env::var("ROCM_HOME").ok(), Some("/opt/rocm".to_string())].into_iter().flatten() {
        let p = PathBuf::from(root).join("bin").join("hipcc");
        if p.exists() {
            return Some(p);
        }
    }
    std::env::var_os("PATH").and_then(|paths| std::env::split_paths(&paths).map(|d| d.join("hipcc")).find(|p| p.exists()))
}

/// Sections of build_flags.txt: `[name]` headers, one entry per line, `#` comments, `{arch}` replaced by the target.
#[cfg(feature = "hip")]
fn read_build_flags(path: &std::path::Path, arch: &str) -> std::collections::HashMap<String, Vec<String>> {
    let text = std::fs::read_to_string(path).unwrap_or_else(|e| panic!("cannot read {}: {e}", path.display()));
    let mut out: std::collections::HashMap<String, Vec<String>> = std::collections::HashMap::new();
    let mut cur = String::new();
    for line in text.lines() {
        let line = line.trim();
        if line.is_empty() || line.starts_with('#') {
            continue;
        }
        if line.starts_with('[') && line.ends_with(']') {
            cur = line[1..line.len() - 1].to_string();
            out.entry(cur.clone()).or_default();
        } else {
            out.get_mut(&cur).expect("entry before the first [section]").push(line.replace("{arch}", arch));
        }
    }
    out
}

#[cfg(feature = "hip")]
fn build_hip() {
    use std::path::PathBuf;
    use std::process::Command;

    println!("cargo:rerun-if-env-changed=HIPCC_PATH");
    println!("cargo:rerun-if-env-changed=RT_HIP_ARCH");
    println!("cargo:rerun-if-env-changed=RT_HIP_LIB_DIR");

    // a prebuilt library: link it and be done
    if let Ok(dir) = std::env::var("RT_HIP_LIB_DIR") {
        println!("cargo:rustc-link-search=native={dir}");
        println!("cargo:rustc-link-lib=dylib=rt_hip");
        println!("cargo:rustc-link-arg=-Wl,-rpath,{dir}");
        return;
    }

    let hipcc = find_hipcc().expect(
        "\n\nhipcc not found.  Install ROCm (7.x) or point HIPCC_PATH at hipcc, or ROCM_PATH at the installation;\n\
         or set RT_HIP_LIB_DIR to a directory that already holds librt_hip.so.\n",
    );
    let arch = std::env::var("RT_HIP_ARCH").unwrap_or_else(|_| "gfx950".to_string());
    let csrc = PathBuf::from("hip").join("csrc");
    let flags_file = csrc.join("build_flags.txt");
    println!("cargo:rerun-if-changed={}", flags_file.display());
    let b = read_build_flags(&flags_file, &arch);
    let out_dir = PathBuf::from(std::env::var("OUT_DIR").unwrap());

    for h in &b["headers"] {
        println!("cargo:rerun-if-changed={}", csrc.join(h).display());
    }
    // one object per source file, compiled in parallel (a file takes up to two minutes: every kernel is instantiated for 13 dtypes)
    let mut children = Vec::new();
    let mut objects = Vec::new();
    for src in &b["sources"] {
        let path = csrc.join(src);
        println!("cargo:rerun-if-changed={}", path.display());
        let obj = out_dir.join(format!("{}.o", src.trim_end_matches(".hip")));
        let mut cmd = Command::new(&hipcc);
        cmd.args(&b["compile"]).arg("-c").arg(&path).arg("-o").arg(&obj);
        children.push((src.clone(), cmd.spawn().unwrap_or_else(|e| panic!("cannot run {}: {e}", hipcc.display()))));
        objects.push(obj);
    }
    for (src, mut child) in children {
        let status = child.wait().unwrap();
        assert!(status.success(), "\n\nhipcc failed on {src} (target {arch}).  The kernels are written for gfx950; set RT_HIP_ARCH to override.\n");
    }

    // a shared library, linked by hipcc itself: it embeds the device code objects and pulls in the HIP runtime
    let lib = out_dir.join("librt_hip.so");
    let (libs, opts): (Vec<&String>, Vec<&String>) = b["link"].iter().partition(|f| f.starts_with("-l"));
    let status = Command::new(&hipcc).args(opts).arg("-o").arg(&lib).args(&objects).args(libs).status().unwrap();
    assert!(status.success(), "linking librt_hip.so failed");

    println!("cargo:rustc-link-search=native={}", out_dir.display());
    println!("cargo:rustc-link-lib=dylib=rt_hip");
    println!("cargo:rustc-link-arg=-Wl,-rpath,{}", out_dir.display());
}
