"""The script that edits a homura checkout for this library (homura_amd/integration/apply_to_homura.py) finds every
one of its anchors in the reference tree, applies its edits once, and leaves an edited tree alone. Runs only where
the reference sources are mounted; nothing is copied into the repository."""
import os
import shutil
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SCRIPT = os.path.join(ROOT, "homura_amd", "integration", "apply_to_homura.py")
REFERENCE = "/root/reference"
FILES = ["build.rs", "src/backend/rocm/context.rs", "src/backend/rocm/mod.rs", "src/ops/mod.rs", "src/ops/binary.rs",
         "src/backend/cpu/mod.rs", "src/backend/rocm/ffi.rs", "src/backend/rocm/elementwise.rs"]


@pytest.mark.skipif(not os.path.exists(os.path.join(REFERENCE, "build.rs")), reason="the reference sources are not mounted here")
def test_the_overlay_applies_to_the_reference_tree_once(tmp_path):
    for f in FILES:
        os.makedirs(os.path.dirname(tmp_path / f), exist_ok=True)
        shutil.copy(os.path.join(REFERENCE, f), tmp_path / f)
    out = subprocess.run([sys.executable, SCRIPT, str(tmp_path), "--check"], capture_output=True, text=True)
    assert out.returncode == 0 and "anchors are in place" in out.stdout, out.stdout + out.stderr
    assert (tmp_path / "build.rs").read_text() == open(os.path.join(REFERENCE, "build.rs")).read()   # --check edits nothing
    out = subprocess.run([sys.executable, SCRIPT, str(tmp_path)], capture_output=True, text=True)
    assert out.returncode == 0, out.stdout + out.stderr
    edited = {f: (tmp_path / f).read_text() for f in FILES}
    assert '"gfx950", "gfx1201"' in edited["build.rs"] and "HOMURA_ROCM_PREBUILT" in edited["build.rs"]
    assert 'arch != "gfx950"' in edited["src/backend/rocm/context.rs"]
    assert 'starts_with("gfx9")' in edited["src/backend/rocm/mod.rs"]
    assert "    BitwiseAnd,\n}" in edited["src/ops/mod.rs"]
    assert "pub fn bitwise_and(" in edited["src/ops/binary.rs"] and "bitwise_and is not supported for float tensors" in edited["src/ops/binary.rs"]
    assert edited["src/backend/cpu/mod.rs"].count("BitwiseAnd") == 2
    assert "HMR_BINARY_BITWISE_AND: i32 = 15" in edited["src/backend/rocm/ffi.rs"]
    assert "BitwiseAnd => ffi::HMR_BINARY_BITWISE_AND" in edited["src/backend/rocm/elementwise.rs"]
    # A second run finds its work done and changes nothing.
    out = subprocess.run([sys.executable, SCRIPT, str(tmp_path)], capture_output=True, text=True)
    assert out.returncode == 0, out.stdout + out.stderr
    assert {f: (tmp_path / f).read_text() for f in FILES} == edited


def test_the_overlay_refuses_a_tree_it_does_not_recognise(tmp_path):
    (tmp_path / "build.rs").write_text("fn main() {}\n")
    out = subprocess.run([sys.executable, SCRIPT, str(tmp_path)], capture_output=True, text=True)
    assert out.returncode != 0 and "nothing was changed" in out.stderr
    assert (tmp_path / "build.rs").read_text() == "fn main() {}\n"
