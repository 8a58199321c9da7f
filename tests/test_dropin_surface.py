"""The C++ host surface is call-compatible with code written against the reference's headers:
tests/cpp/dropin_surface.cpp calls every method and free function of that surface with the
reference's argument lists and default arguments, includes this library's headers only, and is
compiled and linked here against libdeusridet_memoria.so.  It is built, not run."""
import os
import shutil
import subprocess

import pytest

from deusridet_amd import host

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_dropin_surface_compiles_and_links(tmp_path):
    cxx = shutil.which("g++")
    if not cxx:
        pytest.skip("no g++")
    assert os.path.exists(host.LIB_PATH), "build the host library first"
    lib_dir = os.path.dirname(host.LIB_PATH)
    exe = tmp_path / "dropin_surface"
    cmd = [cxx, "-std=c++17", "-Wall", "-Wextra", "-Werror", "-D__HIP_PLATFORM_AMD__", "-I" + os.path.join(ROOT, "include"),
           "-I/opt/rocm/include", "-I" + os.path.join(ROOT, "deusridet_amd"), os.path.join(ROOT, "tests", "cpp", "dropin_surface.cpp"),
           "-L" + lib_dir, "-ldeusridet_memoria", "-ldrk_kv", "-Wl,-rpath," + lib_dir, "-Wl,--no-undefined", "-o", str(exe)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    assert exe.exists()


def test_wrapper_symbols_are_exported():
    """The two layer wrappers exist under the reference's names (paged_attention.h:75-106)."""
    out = subprocess.run(["nm", "-D", "--defined-only", "-C", host.LIB_PATH], capture_output=True, text=True).stdout
    for name in ("deusridet::full_attention_forward_paged(", "deusridet::full_attention_forward_paged_prefill(",
                 "deusridet::paged_kv_cache_write(", "deusridet::paged_kv_cache_write_batch(",
                 "deusridet::paged_gqa_decode_attention(", "deusridet::invoke_extract_kv_from_pages(",
                 "deusridet::invoke_inject_kv_to_pages("):
        assert name in out, name
