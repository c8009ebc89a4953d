"""The hot kernels' bodies on the CPU under the host sanitizers (tests/cpp/emu_prod_kernel.cpp, tests/cpp/emu_slice_kernel.cpp,
tests/cpp/emu_poly_kernel.cpp):
no GPU involved."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CLANG = "/opt/rocm/llvm/bin/clang++"
needs_clang = pytest.mark.skipif(not os.path.exists(CLANG), reason="needs clang (ext_vector_type, -ftrivial-auto-var-init)")


def _build_and_run(tmp_path, source, args):
    csrc = os.path.join(ROOT, "deep-prove_amd", "csrc")
    shutil.copy(os.path.join(csrc, "gl.hpp"), tmp_path / "gl.hpp")
    text = open(os.path.join(csrc, "kernels.hpp")).read()
    # dynamic LDS has no host spelling: the emulation hands every workgroup a buffer of its own
    assert "extern __shared__ u64 dyn[];" in text
    (tmp_path / "kernels.hpp").write_text(text.replace("extern __shared__ u64 dyn[];", "u64 *dyn = emu::dyn_lds();"))
    exe = tmp_path / "emu"
    subprocess.check_call([CLANG, "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined",
                           "-ftrivial-auto-var-init=pattern", "-I", str(tmp_path), "-I", os.path.join(ROOT, "tests", "cpp", "emu"),
                           "-I", os.path.join(ROOT, "include"), "-pthread", "-o", str(exe), os.path.join(ROOT, "tests", "cpp", source)])
    out = subprocess.run([str(exe)] + args, capture_output=True, text=True, timeout=900)
    assert out.returncode == 0, out.stdout[-3000:] + out.stderr[-3000:]
    assert "all cases ok" in out.stdout and "MISMATCH" not in out.stdout
    assert "runtime error" not in out.stderr and "AddressSanitizer" not in out.stderr


@needs_clang
def test_prod_kernel_body_under_host_sanitizers(tmp_path):
    _build_and_run(tmp_path, "emu_prod_kernel.cpp", ["quick"])


@needs_clang
def test_slice_kernel_body_under_host_sanitizers(tmp_path):
    # the resident rounds: trips of one and two rounds, one and several workgroups, hand-over between launches
    _build_and_run(tmp_path, "emu_slice_kernel.cpp", [])


@needs_clang
def test_poly_kernel_body_under_host_sanitizers(tmp_path):
    # sums of several terms over shared tables: term by term and as a nested program, a pair's work over 1, 4 and 16 lanes,
    # many groups, launches made ahead, a launch that stays for every remaining round
    _build_and_run(tmp_path, "emu_poly_kernel.cpp", [])
