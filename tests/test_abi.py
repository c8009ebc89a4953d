"""The C-ABI libraries load on a machine without a GPU and export every symbol
their headers declare; a context cannot be created without a device."""
import ctypes
import importlib
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared(header, prefix):
    text = open(os.path.join(ROOT, header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(" + prefix + r"[a-z0-9_]+)\s*\(", text)))


def test_device_library_exports_every_declared_symbol():
    names = _declared("include/dpsumcheck.h", "dps_")
    assert len(names) >= 30
    lib = ctypes.CDLL(os.path.join(ROOT, "deep-prove_amd", "lib", "libdpsumcheck.so"))
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing


def test_host_library_exports_every_declared_symbol():
    names = _declared("deep-prove_amd/host/dpsc_host.h", "dph_")
    assert len(names) >= 15
    ctypes.CDLL(os.path.join(ROOT, "deep-prove_amd", "lib", "libdpsumcheck.so"), mode=ctypes.RTLD_GLOBAL)
    lib = ctypes.CDLL(os.path.join(ROOT, "deep-prove_amd", "lib", "libdpsc_host.so"))
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing


def test_status_strings_and_kernel_names():
    dp = importlib.import_module("deep-prove_amd")
    assert dp.dev.dps_status_str(0) == b"ok"
    assert all(dp.dev.dps_status_str(i) for i in range(8))
    assert all(dp.dev.dps_kernel_name(k) != b"?" for k in range(len(dp.KERNELS)))


def test_no_silent_cpu_path():
    # without a GPU there is nothing to fall back to: creating a context fails loudly
    dp = importlib.import_module("deep-prove_amd")
    try:
        ctx = dp.Context(0)
    except dp.DpsError as e:
        assert e.status != 0
    else:
        ctx.close()  # a GPU is present (running on the GPU box)


def test_package_does_not_reference_the_checker():
    # the shipped code must not import, link or open anything under oracle/
    pkg = os.path.join(ROOT, "deep-prove_amd")
    for base, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".h", ".cpp")):
                text = open(os.path.join(base, f)).read()
                assert "dpsc_oracle" not in text and "oracle/" not in text, os.path.join(base, f)
