#!/usr/bin/env python3
"""Applies to a homura checkout the handful of edits that let its `rocm` feature run on an MI355X through this
library:

    python homura_amd/integration/apply_to_homura.py /path/to/homura          # edit in place
    python homura_amd/integration/apply_to_homura.py /path/to/homura --check  # only verify that every anchor is there

  build.rs                         gfx950 is accepted; HOMURA_ROCM_PREBUILT=<dir holding libhomura_rocm.a> links
                                   that archive instead of compiling csrc/*.hip, and gfx950 requires it
  src/backend/rocm/context.rs      gfx950 counts as tested
  src/backend/rocm/mod.rs          gfx9 reports compute units, not workgroup processors
  src/ops/mod.rs, src/ops/binary.rs, src/backend/cpu/mod.rs,
  src/backend/rocm/ffi.rs, src/backend/rocm/elementwise.rs
                                   BinaryOp::BitwiseAnd / Tensor::bitwise_and (HMR_BINARY_BITWISE_AND = 15, appended)

Every edit is anchored on one line of the file as homura has it; the script stops, changing nothing, when an anchor is
missing or not unique (a newer homura: apply the edit by hand; EDITS below holds each one in full). Afterwards:

    HOMURA_ROCM_PREBUILT=/path/to/homura_amd/lib HOMURA_OFFLOAD_ARCH=gfx950 cargo build --features rocm
"""
import os
import sys

# (file, anchor line as it stands, "replace" | "after" | "before", new text)
EDITS = [
    ("build.rs", 'const SUPPORTED: &[&str] = &["gfx1201", "gfx1200"];', "replace",
     'const SUPPORTED: &[&str] = &["gfx950", "gfx1201", "gfx1200"];'),
    ("build.rs", "    let rocm = rocm_root();", "after",
     """    // gfx950 (MI355X, wave64) is served by the prebuilt homura_amd library, which exports the same hmr_* ABI:
    // HOMURA_ROCM_PREBUILT names the directory that holds its libhomura_rocm.a.
    println!("cargo:rerun-if-env-changed=HOMURA_ROCM_PREBUILT");
    if let Some(dir) = env::var_os("HOMURA_ROCM_PREBUILT") {
        let dir = PathBuf::from(dir);
        let lib = rocm.join("lib");
        println!("cargo:rustc-link-search=native={}", dir.display());
        println!("cargo:rustc-link-lib=static=homura_rocm");
        println!("cargo:rustc-link-search=native={}", lib.display());
        println!("cargo:rustc-link-lib=dylib=amdhip64");
        println!("cargo:rustc-link-lib=dylib=stdc++");
        println!("cargo:rustc-link-arg=-Wl,-rpath,{}", lib.display());
        println!("cargo:lib={}", lib.display());
        return;
    }
    if archs.iter().any(|a| a == "gfx950") {
        fail(
            "gfx950 is not compiled from csrc/: set HOMURA_ROCM_PREBUILT to the directory that holds \\
             homura_amd's libhomura_rocm.a",
        );
    }"""),
    ("src/backend/rocm/context.rs", '    if arch != "gfx1201" && !WARNED.swap(true, Ordering::Relaxed) {', "replace",
     '    if arch != "gfx1201" && arch != "gfx950" && !WARNED.swap(true, Ordering::Relaxed) {'),
    ("src/backend/rocm/mod.rs", "        compute_units: 2 * p.multiprocessor_count as u32,", "replace",
     """        // On gfx9 (CDNA) HIP counts compute units themselves: 256 on an MI355X.
        compute_units: if text(&p.arch).starts_with("gfx9") {
            p.multiprocessor_count as u32
        } else {
            2 * p.multiprocessor_count as u32
        },"""),
    ("src/ops/mod.rs", "    LogicalOr,", "after", "    BitwiseAnd,"),
    ("src/ops/binary.rs", "    if compute == DType::Bool && op == Pow {", "before",
     """    if op == BitwiseAnd && compute.is_floating_point() {
        panic!("bitwise_and is not supported for float tensors");
    }"""),
    ("src/ops/binary.rs", "    /// In-place [`add`](Tensor::add).", "before",
     """    /// Elementwise bitwise and of integer tensors (two's complement); logical and of bool tensors.
    #[track_caller]
    pub fn bitwise_and(&self, other: impl Into<Operand>) -> Tensor {
        self.binary(BinaryOp::BitwiseAnd, other)
    }
"""),
    ("src/backend/cpu/mod.rs", "            Mul | Minimum => map2::<bool, bool, bool>(out, a, b, |x, y| x && y),", "replace",
     "            Mul | Minimum | BitwiseAnd => map2::<bool, bool, bool>(out, a, b, |x, y| x && y),"),
    ("src/backend/cpu/mod.rs", "            Minimum => map2::<T, T, T>(out, a, b, |x, y| x.min(y)),", "after",
     "            BitwiseAnd => map2::<T, T, T>(out, a, b, |x, y| x & y),"),
    ("src/backend/rocm/ffi.rs", "pub const HMR_BINARY_LOGICAL_OR: i32 = 14;", "after",
     "pub const HMR_BINARY_BITWISE_AND: i32 = 15;"),
    ("src/backend/rocm/elementwise.rs", "        LogicalOr => ffi::HMR_BINARY_LOGICAL_OR,", "after",
     "        BitwiseAnd => ffi::HMR_BINARY_BITWISE_AND,"),
]


def main(argv):
    if len(argv) < 2 or argv[1].startswith("-"):
        sys.exit(__doc__)
    root, check_only = argv[1], "--check" in argv[2:]
    texts, problems = {}, []
    for path, anchor, how, new in EDITS:
        full = os.path.join(root, path)
        if path not in texts:
            try:
                with open(full, encoding="utf-8") as f:
                    texts[path] = f.read().split("\n")
            except OSError as e:
                problems.append(f"{path}: {e}")
                texts[path] = None
        lines = texts[path]
        if lines is None:
            continue
        if new.split("\n")[0] in lines and how != "replace" or (how == "replace" and new.split("\n")[0] in lines and anchor not in lines):
            continue  # applied before
        hits = [i for i, line in enumerate(lines) if line == anchor]
        if len(hits) != 1:
            problems.append(f"{path}: the line {anchor.strip()!r} is there {len(hits)} times, not once")
            continue
        i, block = hits[0], new.split("\n")
        if how == "replace":
            lines[i:i + 1] = block
        elif how == "after":
            lines[i + 1:i + 1] = block
        else:
            lines[i:i] = block
    if problems:
        sys.exit("nothing was changed:\n  " + "\n  ".join(problems))
    if check_only:
        print(f"all {len(EDITS)} anchors are in place")
        return
    for path, lines in texts.items():
        with open(os.path.join(root, path), "w", encoding="utf-8") as f:
            f.write("\n".join(lines))
    print(f"applied {len(EDITS)} edits to {len(texts)} files under {root}")


if __name__ == "__main__":
    main(sys.argv)
