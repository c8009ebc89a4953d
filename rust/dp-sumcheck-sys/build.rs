// Tells cargo where libdpsumcheck.so is.  The library is built by the repository's own recipe
// (`python deep-prove_amd/build.py`: hipcc, no GPU needed) into deep-prove_amd/lib; DPSUMCHECK_LIB_DIR overrides the
// place.  Nothing is compiled here.
use std::env;
use std::path::PathBuf;

fn main() {
    println!("cargo:rerun-if-env-changed=DPSUMCHECK_LIB_DIR");
    let dir = match env::var_os("DPSUMCHECK_LIB_DIR") {
        Some(d) => PathBuf::from(d),
        None => {
            let manifest = PathBuf::from(env::var_os("CARGO_MANIFEST_DIR").expect("cargo sets CARGO_MANIFEST_DIR"));
            manifest.join("..").join("..").join("deep-prove_amd").join("lib")
        }
    };
    let dir = dir.canonicalize().unwrap_or(dir);
    println!("cargo:rustc-link-search=native={}", dir.display());
    println!("cargo:rustc-link-lib=dylib=dpsumcheck");
    // so that a binary finds the library next to where it was linked from without LD_LIBRARY_PATH
    println!("cargo:rustc-link-arg=-Wl,-rpath,{}", dir.display());
    // the header is the contract: rebuild when it moves
    println!("cargo:rerun-if-changed=../../include/dpsumcheck.h");
}
