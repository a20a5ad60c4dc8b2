// Locates a prebuilt libhs_attn.so the way bitsandbytes-sys locates libbitsandbytes
// (crates/bitsandbytes-sys/build.rs:85-160, 398-478): environment variable, then well-known directories.
// There is no build-from-source step here: the library is produced by `python -m hyprstream_amd.build`
// (hipcc --offload-arch=gfx950) in the kernel repository and installed beside the binary.
use std::env;
use std::path::{Path, PathBuf};

fn find_lib_dir() -> Option<PathBuf> {
    if let Ok(p) = env::var("HS_ATTN_LIB_PATH") {
        let p = PathBuf::from(p);
        // accept either the directory or the path of the .so itself
        let dir = if p.is_file() { p.parent().map(Path::to_path_buf)? } else { p };
        if dir.join("libhs_attn.so").exists() {
            return Some(dir);
        }
        println!("cargo:warning=HS_ATTN_LIB_PATH={} holds no libhs_attn.so", dir.display());
    }
    let mut candidates: Vec<PathBuf> = vec!["/usr/local/lib".into(), "/usr/lib".into(), "/opt/hs-attn/lib".into()];
    if let Ok(ld) = env::var("LD_LIBRARY_PATH") {
        candidates.extend(ld.split(':').filter(|s| !s.is_empty()).map(PathBuf::from));
    }
    candidates.into_iter().find(|d| d.join("libhs_attn.so").exists())
}

fn main() {
    println!("cargo:rerun-if-env-changed=HS_ATTN_LIB_PATH");
    println!("cargo:rerun-if-env-changed=ROCM_PATH");
    let dir = find_lib_dir().expect("libhs_attn.so not found: set HS_ATTN_LIB_PATH to its directory");
    println!("cargo:rustc-link-search=native={}", dir.display());
    println!("cargo:rustc-link-lib=dylib=hs_attn");
    if env::var("CARGO_FEATURE_KV_CACHE").is_ok() {
        assert!(dir.join("libhs_kv_cache.so").exists(), "feature kv-cache needs libhs_kv_cache.so beside libhs_attn.so");
        println!("cargo:rustc-link-lib=dylib=hs_kv_cache");
    }
    // the kernels' only dependency (bitsandbytes-sys links amdhip64 the same way in its HIP configuration)
    let rocm = env::var("ROCM_PATH").unwrap_or_else(|_| "/opt/rocm".to_string());
    println!("cargo:rustc-link-search=native={}/lib", rocm);
    println!("cargo:rustc-link-lib=dylib=amdhip64");
    println!("cargo:rustc-cfg=hs_attn_hip");
}
