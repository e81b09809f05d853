// Links libojas_mi355x.so. The library is built outside cargo (hipcc); OJAS_MI355X_LIB_DIR names
// the directory that holds it.
fn main() {
    println!("cargo:rerun-if-env-changed=OJAS_MI355X_LIB_DIR");
    if let Ok(dir) = std::env::var("OJAS_MI355X_LIB_DIR") {
        println!("cargo:rustc-link-search=native={dir}");
        println!("cargo:rustc-link-arg=-Wl,-rpath,{dir}");
    }
    println!("cargo:rustc-link-lib=dylib=ojas_mi355x");
}
