"""CPU tests of the C++ host mirror: hash, transcript, expression flattening and
the verifier, against the checker and published vectors."""
import importlib
import os
import subprocess

import numpy as np
import pytest

from test_oracle_field import BLAKE3_KAT
from util import rand_e2

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def dp():
    return importlib.import_module("deep-prove_amd")


def test_blake3_published_vectors(dp):
    for msg, digest in BLAKE3_KAT:
        assert dp.blake3(msg).hex() == digest


def test_blake3_incremental_against_recursive_tree(dp, orc):
    # two independent implementations (incremental with a chaining-value stack here,
    # recursive subtree split in the checker) across chunk and tree boundaries
    rng = np.random.Generator(np.random.PCG64(1))
    for n in [1, 63, 64, 65, 1023, 1024, 1025, 2047, 2048, 2049, 3072, 4096, 4097, 5000, 8192, 8193, 20000]:
        data = rng.integers(0, 256, size=n, dtype=np.uint8).tobytes()
        assert dp.blake3(data) == orc.blake3(data), n


def test_transcript_matches_checker(dp, orc):
    a, b = dp.Transcript(b"model_proving"), orc.OracleTranscript(b"model_proving")
    assert a.state() == b.state()
    xs = rand_e2(5, 2)
    a.append_u64(12345); b.append_u64(12345)
    a.append_scalars(xs); b.append_scalars(xs)
    assert (a.append_and_sample(b"batching_challenge") == b.append_and_sample(b"batching_challenge")).all()
    a.append_bytes(b"\x01" * 1500); b.append_bytes(b"\x01" * 1500)
    a.append_message(b"logup_alpha"); b.append_message(b"logup_alpha")
    assert (a.read_challenges(3) == b.read_challenges(3)).all()
    assert a.state() == b.state()
    c = a.clone()
    assert (c.challenge_scalar() == a.challenge_scalar()).all()


def test_verifier_accepts_checker_proof_and_rejects_tampering(dp, orc):
    # IOPVerifierState::verify of the host mirror on a proof made by the checker (no GPU involved)
    n = 7
    tabs = [rand_e2(1 << n, 10 + k) for k in range(3)]
    terms = [(np.array([2, 5], np.uint64), [0, 1, 2]), (np.array([1, 0], np.uint64), [0, 2])]
    otr = orc.OracleTranscript()
    proof, point, finals = orc.sc_prove(n, tabs, terms, otr)
    claim = orc.e2_add(proof[0, 0], proof[0, 1])
    ctx_free = dp.Context.__new__(dp.Context)  # the verifier needs no device
    tr = dp.Transcript()
    rc, vpoint, expected = dp.Context.sumcheck_verify(ctx_free, claim, proof, tr)
    assert rc == 0 and (vpoint == point).all() and tr.state() == otr.state()
    orc_rc, _, oexp = orc.sc_verify(claim, proof, orc.OracleTranscript())
    assert orc_rc == 0 and (expected == oexp).all()
    bad = proof.copy()
    bad[4, 2, 1] ^= np.uint64(1)
    rc, _, _ = dp.Context.sumcheck_verify(ctx_free, claim, bad, dp.Transcript())
    assert rc != 0


def test_expression_flattening_cpp(tmp_path):
    exe = tmp_path / "test_expression"
    subprocess.check_call(["g++", "-O1", "-std=c++17", "-o", str(exe), os.path.join(ROOT, "tests", "cpp", "test_expression.cpp")])
    out = subprocess.run([str(exe)], capture_output=True, text=True)
    assert out.returncode == 0, out.stdout + out.stderr


def test_blake3_vector_and_portable_compressions_agree(dp):
    """The host mirror hashes with a 512-bit-permute compression where the CPU has AVX-512 and with a portable loop
    elsewhere (DPSC_BLAKE3_PORTABLE forces the loop): same digests and the same transcript on both."""
    import sys

    script = (
        "import importlib, sys, numpy as np\n"
        "sys.path.insert(0, %r)\n"
        "dp = importlib.import_module('deep-prove_amd')\n"
        "out = [dp.blake3(bytes(range(256)) * k)[:8].hex() for k in (0, 1, 3, 5, 9)]\n"
        "t = dp.Transcript(b'paths')\n"
        "t.append_u64(7); t.append_bytes(b'x' * 100)\n"
        "t.append_scalars(np.arange(10, dtype=np.uint64).reshape(5, 2))\n"
        "out.append(t.append_and_sample(b'c').tolist()); out.append(t.state()[0].hex())\n"
        "print(out)\n" % ROOT)
    runs = []
    for portable in (False, True):
        env = dict(os.environ)
        env.pop("DPSC_BLAKE3_PORTABLE", None)
        if portable:
            env["DPSC_BLAKE3_PORTABLE"] = "1"
        res = subprocess.run([sys.executable, "-c", script], capture_output=True, text=True, env=env)
        assert res.returncode == 0, res.stderr
        runs.append(res.stdout.strip())
    assert runs[0] == runs[1] and runs[0].startswith("['")
