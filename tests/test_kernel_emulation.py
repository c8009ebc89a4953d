"""The hot kernels' bodies on the CPU under the host sanitizers (tests/cpp/emu_prod_kernel.cpp, tests/cpp/emu_slice_kernel.cpp,
tests/cpp/emu_poly_kernel.cpp): no GPU involved.  The three programs are built and run side by side (a build under the
sanitizers takes over a minute), once per test session; each test then reads its program's outcome."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CLANG = "/opt/rocm/llvm/bin/clang++"
needs_clang = pytest.mark.skipif(not os.path.exists(CLANG), reason="needs clang (ext_vector_type, -ftrivial-auto-var-init)")

PROGRAMS = {"prod": ("emu_prod_kernel.cpp", ["quick"]), "slice": ("emu_slice_kernel.cpp", []), "poly": ("emu_poly_kernel.cpp", [])}


@pytest.fixture(scope="module")
def outcomes(tmp_path_factory):
    tmp_path = tmp_path_factory.mktemp("emu")
    csrc = os.path.join(ROOT, "deep-prove_amd", "csrc")
    shutil.copy(os.path.join(csrc, "gl.hpp"), tmp_path / "gl.hpp")
    text = open(os.path.join(csrc, "kernels.hpp")).read()
    # dynamic LDS has no host spelling: the emulation hands every workgroup a buffer of its own
    assert "extern __shared__ u64 dyn[];" in text
    (tmp_path / "kernels.hpp").write_text(text.replace("extern __shared__ u64 dyn[];", "u64 *dyn = emu::dyn_lds();"))
    procs = {}
    for name, (source, args) in PROGRAMS.items():
        exe = tmp_path / ("emu_" + name)
        build = " ".join([CLANG, "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined",
                          "-ftrivial-auto-var-init=pattern", "-I", str(tmp_path), "-I", os.path.join(ROOT, "tests", "cpp", "emu"),
                          "-I", os.path.join(ROOT, "include"), "-pthread", "-o", str(exe), os.path.join(ROOT, "tests", "cpp", source)])
        # build, then run, in one shell per program: the three go on side by side
        procs[name] = subprocess.Popen(["bash", "-c", build + " && exec " + " ".join([str(exe)] + args)], stdout=subprocess.PIPE,
                                       stderr=subprocess.PIPE, text=True)
    out = {}
    for name, p in procs.items():
        try:
            so, se = p.communicate(timeout=1500)
        except subprocess.TimeoutExpired:
            p.kill()
            so, se = p.communicate()
            se += "\n(timed out)"
        out[name] = (p.returncode, so, se)
    return out


def _check(outcome):
    rc, so, se = outcome
    assert rc == 0, so[-3000:] + se[-3000:]
    assert "all cases ok" in so and "MISMATCH" not in so
    assert "runtime error" not in se and "AddressSanitizer" not in se


@needs_clang
def test_prod_kernel_body_under_host_sanitizers(outcomes):
    _check(outcomes["prod"])


@needs_clang
def test_slice_kernel_body_under_host_sanitizers(outcomes):
    # the resident rounds: trips of one and two rounds, one and several workgroups, hand-over between launches
    _check(outcomes["slice"])


@needs_clang
def test_poly_kernel_body_under_host_sanitizers(outcomes):
    # sums of several terms over shared tables: term by term and as a nested program, a pair's work over 1, 4 and 16 lanes,
    # many groups, launches made ahead, factored eq weights, a launch that stays for every remaining round
    _check(outcomes["poly"])
