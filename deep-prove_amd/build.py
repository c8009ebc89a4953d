"""Build recipe of the two shared libraries (run on a machine with ROCm; no GPU needed).

    libdpsumcheck.so   HIP kernels + C ABI      hipcc --offload-arch=gfx950
    libdpsc_host.so    C++ host mirror + C API  g++
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "lib")

HIPCC_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-Wall",
               # packed FP32 instructions are kept out of every code object built here
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _run(cmd):
    print("+", " ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if out.strip():
        print(out, flush=True)
    if res.returncode != 0:
        raise RuntimeError(f"build step failed ({res.returncode}): {' '.join(cmd)}")


def build_device():
    os.makedirs(LIB, exist_ok=True)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    _run([hipcc, *HIPCC_FLAGS, "-o", os.path.join(LIB, "libdpsumcheck.so"), os.path.join(HERE, "csrc", "dpsumcheck.hip")])


def build_host():
    os.makedirs(LIB, exist_ok=True)
    _run(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wextra", "-o", os.path.join(LIB, "libdpsc_host.so"),
          os.path.join(HERE, "host", "host_capi.cpp"), "-L" + LIB, "-ldpsumcheck", "-Wl,-rpath,$ORIGIN"])


def build_all():
    build_device()
    build_host()


if __name__ == "__main__":
    build_all()
    sys.exit(0)
