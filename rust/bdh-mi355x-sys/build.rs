// Links the prebuilt C-ABI library.  BDH_MI355X_LIB_DIR = directory holding libbdh_mi355x.so
// (burn_dragon_amd/ after `python -m burn_dragon_amd.build`).
fn main() {
    if let Ok(dir) = std::env::var("BDH_MI355X_LIB_DIR") {
        println!("cargo:rustc-link-search=native={dir}");
        println!("cargo:rustc-link-arg=-Wl,-rpath,{dir}");
    }
    println!("cargo:rustc-link-lib=dylib=bdh_mi355x");
    println!("cargo:rerun-if-env-changed=BDH_MI355X_LIB_DIR");
}
