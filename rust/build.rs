// Links librembrandt_hip.so (built by `python -m rembrandt_amd.build`); set REMBRANDT_HIP_LIB_DIR to
// the directory that holds it.  Takes the place of `-L /usr/local/cuda/lib64` in the reference's build.rs.
fn main() {
  let dir = std::env::var("REMBRANDT_HIP_LIB_DIR").unwrap_or("../rembrandt_amd".to_string());
  println!("cargo:rustc-link-search=native={}", dir);
  println!("cargo:rustc-link-lib=dylib=rembrandt_hip");
}
