"""The C-ABI library as a link target (no GPU, no compute calls): it loads, exports every symbol that
include/*.h declares and every one of the 77 functions homura's Rust crate declares in
src/backend/rocm/ffi.rs, keeps everything else local, and reports the struct layouts and enum values the
Rust side asserts (ref: src/backend/rocm/tests.rs:10-59, csrc/homura_rocm.h:592-610)."""
import ctypes
import os
import re
import subprocess

import pytest

from homura_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INCLUDE = os.path.join(ROOT, "include")

# The `extern "C"` block of src/backend/rocm/ffi.rs, names only.
RUST_FFI = """
    hmr_abi_check hmr_adaptive_avg_pool2d hmr_adaptive_avg_pool2d_backward hmr_addr hmr_arg_reduce hmr_binary
    hmr_binary_constant hmr_binary_scalar hmr_built_archs hmr_context_create hmr_context_destroy
    hmr_context_synchronize hmr_copy hmr_copy_device hmr_copy_from_host hmr_copy_to_host hmr_device_count
    hmr_device_properties_get hmr_exclusive_cumprod hmr_fill hmr_flip hmr_free hmr_fused hmr_gather hmr_gemm
    hmr_gemm_fold hmr_gemm_path_name hmr_gemm_select hmr_gemm_workspace hmr_index_add hmr_index_add_workspace
    hmr_index_check hmr_index_overwrite hmr_index_overwrite_workspace hmr_index_positions hmr_index_select
    hmr_last_error hmr_malloc hmr_mask_coordinates hmr_mask_count hmr_mask_workspace hmr_max_pool2d
    hmr_max_pool2d_backward hmr_max_pool2d_backward_workspace hmr_max_pool2d_check
    hmr_max_pool2d_gather_backward hmr_mem_get_info hmr_memset hmr_random_int hmr_random_normal
    hmr_random_uniform hmr_reduce hmr_reduce_workspace hmr_scatter_add hmr_scatter_add_workspace hmr_softmax
    hmr_softmax_workspace hmr_test_current_device hmr_test_fail hmr_test_fail_after_probe hmr_test_fail_data
    hmr_test_fail_properties hmr_test_fail_stream_create hmr_test_force_gemm_path hmr_test_index_value
    hmr_test_live_streams hmr_test_pool_candidates hmr_test_reduce_plan hmr_test_set_current_device
    hmr_test_softmax_plan hmr_test_wide_pool hmr_triangle hmr_unary hmr_unfold_backward hmr_var hmr_where
    hmr_where_constant
""".split()


def declared_in_headers():
    names = set()
    for f in sorted(os.listdir(INCLUDE)):
        text = open(os.path.join(INCLUDE, f)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        text = re.sub(r"//[^\n]*", "", text)
        names.update(re.findall(r"\b(hmr_[a-z0-9_]+)\s*\(", text))
    return names


def exported():
    out = subprocess.check_output(["nm", "-D", "--defined-only", capi.LIB_PATH], text=True)
    return {line.split()[-1] for line in out.splitlines() if line.strip()}


def test_rust_ffi_list_is_complete():
    assert len(RUST_FFI) == 77 and len(set(RUST_FFI)) == 77


# Beside the Rust crate's 77: the stream accessor for harnesses and the reduction that allocates nothing.
EXTENSIONS = {"hmr_ext_stream", "hmr_reduce_static"}


def test_the_library_exports_exactly_the_declared_set():
    assert exported() == set(RUST_FFI) | EXTENSIONS
    assert declared_in_headers() == set(RUST_FFI) | EXTENSIONS


def test_every_declared_symbol_is_exported():
    declared = declared_in_headers()
    assert len(declared) == 79
    have = exported()
    assert not (declared - have), f"declared in include/*.h but not exported: {sorted(declared - have)}"
    assert not (set(RUST_FFI) - have), f"needed by the Rust crate but not exported: {sorted(set(RUST_FFI) - have)}"
    assert not (set(RUST_FFI) - declared), f"not declared in include/*.h: {sorted(set(RUST_FFI) - declared)}"


def test_only_hmr_symbols_are_global():
    """ref: build.rs:232-250 keeps only hmr_* global in the relocatable object."""
    stray = {s for s in exported() if not s.startswith("hmr_")}
    assert not stray, sorted(stray)


def test_every_symbol_binds_through_ctypes():
    lib = ctypes.CDLL(capi.LIB_PATH)
    for name in sorted(declared_in_headers()):
        assert getattr(lib, name) is not None
    assert set(capi.PROTOTYPES) | set(capi.UNBUILT) >= set(RUST_FFI)


ARCHIVE = os.path.join(os.path.dirname(capi.LIB_PATH), "libhomura_rocm.a")


def test_static_archive_is_one_object_with_only_hmr_symbols_global():
    """The Rust build links libhomura_rocm.a: one relocatable object in which only hmr_* stay global
    (ref: build.rs:231-250; linked at build.rs:60-70)."""
    assert os.path.exists(ARCHIVE)
    members = subprocess.check_output(["ar", "t", ARCHIVE], text=True).split()
    assert members == ["homura_rocm.o"], members
    out = subprocess.check_output(["nm", "--defined-only", "-g", ARCHIVE], text=True, stderr=subprocess.DEVNULL)
    have = {line.split()[-1] for line in out.splitlines() if len(line.split()) == 3}
    assert set(RUST_FFI) <= have
    stray = {s for s in have if not s.startswith("hmr_")}
    assert not stray, sorted(stray)[:20]
    # Nothing is left for the linker to find except what the Rust build links beside it: the HIP runtime,
    # the C++ runtime and libc / libm.
    out = subprocess.check_output(["nm", "--undefined-only", ARCHIVE], text=True, stderr=subprocess.DEVNULL)
    undefined = {line.split()[-1] for line in out.splitlines() if len(line.split()) == 2}
    assert not {s for s in undefined if s.startswith("hmr_")}, "an hmr_* symbol is not defined in the archive"


def test_a_c_program_links_statically_against_the_archive(tmp_path):
    """Linked here from source, so the test fails if the archive needs anything but amdhip64 and stdc++."""
    exe = tmp_path / "static_check"
    source = os.path.join(ROOT, "homura_amd", "csrc", "static_check.c")
    subprocess.check_call(["gcc", "-O1", "-I", INCLUDE, source, ARCHIVE, "-L/opt/rocm/lib", "-lamdhip64", "-lstdc++",
                           "-lm", "-lpthread", "-Wl,-rpath,/opt/rocm/lib", "-o", str(exe)])
    out = subprocess.check_output([str(exe)], text=True)
    assert out.startswith("archs gfx950, desc 424 bytes, max dims 25")


def test_abi_layout():
    """What the_abi_matches_the_library asserts on the Rust side (ref: src/backend/rocm/tests.rs:10-59)."""
    info = capi.hmr_abi_info()
    capi.lib.hmr_abi_check(ctypes.byref(info))
    D, P = capi.hmr_tensor_desc, capi.hmr_device_properties
    assert info.abi_info_size == ctypes.sizeof(capi.hmr_abi_info)
    assert (info.desc_size, info.desc_align) == (ctypes.sizeof(D), ctypes.alignment(D)) == (424, 8)
    assert list(info.desc_offsets) == [D.data.offset, D.offset.offset, D.dtype.offset, D.ndim.offset, D.sizes.offset,
                                       D.strides.offset] == [0, 8, 16, 20, 24, 224]
    assert (info.properties_size, info.properties_align) == (ctypes.sizeof(P), ctypes.alignment(P))
    assert list(info.properties_offsets) == [P.name.offset, P.arch.offset, P.multiprocessor_count.offset,
                                             P.warp_size.offset, P.total_memory.offset]
    assert list(info.status_values) == [0, 1, 2, 3, 4]
    assert list(info.dtype_values) == list(range(10))
    assert info.max_dims == 25
    assert capi.lib.hmr_built_archs().decode() == "gfx950"


def test_out_of_scope_entry_points_fail_loudly():
    """Kernel families outside this library return HMR_INVALID with a message; they never pretend."""
    lib = ctypes.CDLL(capi.LIB_PATH)
    lib.hmr_last_error.restype = ctypes.c_char_p
    lib.hmr_gemm_path_name.restype = ctypes.c_char_p
    rc = lib.hmr_max_pool2d_check(None, None, None, None, None, None, None, None)
    assert rc == 2
    assert lib.hmr_last_error() == b"hmr_max_pool2d_check: not built in this library"


def test_a_null_context_is_refused_before_anything_is_touched():
    """Every launch goes through one bracket, which refuses a null context with a message (no GPU needed: nothing is
    queued and no HIP call is made)."""
    from ctypes import byref
    d = capi.make_desc(0x1000, capi.F32, (16,), (1,))
    assert capi.lib.hmr_fill(None, byref(d), 0) == capi.HMR_INVALID
    assert b"null context" in capi.lib.hmr_last_error()
    assert capi.lib.hmr_unary(None, 0, byref(d), byref(d)) == capi.HMR_INVALID
    assert b"null context" in capi.lib.hmr_last_error()
