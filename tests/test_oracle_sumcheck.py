"""Pins the checker's sumcheck prover and verifier against the protocol's
definition (brute-force round polynomials), its invariants and special cases."""
import numpy as np
import pytest

import pyfield as pf
from pyfield import E2
from pytranscript import PyTranscript
from util import from_E2, py_rng, rand_base, rand_e2, to_E2


def _py_prove(orc, tables, nvars, n, terms, label=b"m2vec"):
    """Definition-first prover: every round message by brute force over the
    boolean suffixes, transcript from the written layout."""
    degree = max(len(f) for _, f in terms)
    tr = PyTranscript(orc.blake3, label)
    tr.append_u64(n)
    tr.append_u64(degree)
    prefix, proof = [], []
    for _ in range(n):
        msg = pf.round_poly_bruteforce(tables, nvars, n, terms, prefix, degree)
        proof.append(msg)
        tr.append_scalars([m.pair() for m in msg])
        prefix.append(E2(*tr.challenge_scalar()))
    finals = [pf.mle_eval(t, prefix[n - m:]) for t, m in zip(tables, nvars)]
    return proof, prefix, finals, tr


CASES = [
    # (n, table nvars, terms as (coeff, factors))
    (4, [4, 4], [(E2(1), [0, 1])]),                                   # plain product, degree 2
    (4, [4, 4, 4], [(E2(1), [0, 1, 2])]),                             # eq*f*g shape, degree 3
    (3, [3, 3, 3, 3], [(E2(5, 9), [0, 2]), (E2(11, 3), [1, 3])]),     # einsum-like sum of products
    (4, [4, 2, 4, 2], [(E2(3, 1), [0, 2]), (E2(2, 2), [1, 3]), (E2(7), [0, 1, 2])]),  # fewer-variable tables
    (3, [3], [(E2(1), [0])]),                                         # degree 1: reduces to evaluate
    (3, [3, 3, 3, 3, 3], [(E2(1), [0, 1, 2, 3, 4])]),                 # degree 5 (pooling-like)
]


@pytest.mark.parametrize("case", range(len(CASES)))
def test_prover_matches_bruteforce_definition(orc, case):
    n, nvars, terms = CASES[case]
    tabs_np = [rand_e2(1 << m, 100 + case * 10 + k) for k, m in enumerate(nvars)]
    tabs = [to_E2(t) for t in tabs_np]
    proof, point, finals, tr = _py_prove(orc, tabs, nvars, n, terms)
    otr = orc.OracleTranscript(b"m2vec")
    oproof, opoint, ofinal = orc.sc_prove(n, tabs_np, [(from_E2([c])[0], f) for c, f in terms], otr)
    assert [to_E2(r) for r in oproof] == proof
    assert to_E2(opoint) == point
    assert to_E2(ofinal) == finals
    assert otr.state() == (tr.state, tr.k)


def test_round_invariants_and_verifier(orc):
    n = 6
    tabs = [rand_e2(1 << n, 200 + k) for k in range(3)]
    terms = [(np.array([1, 0], np.uint64), [0, 1, 2])]
    tr = orc.OracleTranscript()
    proof, point, final = orc.sc_prove(n, tabs, terms, tr)
    # the claimed sum is the plain sum of products
    claim = E2(0)
    a, b, c = (to_E2(t) for t in tabs)
    for x, y, z in zip(a, b, c):
        claim = claim + x * y * z
    p1 = to_E2(proof[0])
    assert p1[0] + p1[1] == claim
    # p_{j+1}(0) + p_{j+1}(1) = p_j(r_j)
    for j in range(n - 1):
        nxt = to_E2(proof[j + 1])
        assert nxt[0] + nxt[1] == pf.interpolate(to_E2(proof[j]), to_E2(point[j])[0])
    # final evaluations are the MLEs at the challenge point, and close the chain
    fe = [to_E2(orc.mle_evaluate(t, point))[0] for t in tabs]
    assert to_E2(final) == fe
    assert fe[0] * fe[1] * fe[2] == pf.interpolate(to_E2(proof[-1]), to_E2(point[-1])[0])
    # verifier accepts, reproduces the point and the transcript, rejects a tampered proof
    vtr = orc.OracleTranscript()
    rc, vpoint, expected = orc.sc_verify(from_E2([claim])[0], proof, vtr)
    assert rc == 0 and (vpoint == point).all() and vtr.state() == tr.state()
    assert to_E2(expected)[0] == fe[0] * fe[1] * fe[2]
    bad = proof.copy()
    bad[2, 1, 0] ^= np.uint64(1)
    rc, _, _ = orc.sc_verify(from_E2([claim])[0], bad, orc.OracleTranscript())
    assert rc == 3
    rc, _, _ = orc.sc_verify(from_E2([claim + 1])[0], proof, orc.OracleTranscript())
    assert rc == 1


def test_degree_one_is_evaluate(orc):
    n = 5
    t = rand_e2(1 << n, 300)
    proof, point, final = orc.sc_prove(n, [t], [(np.array([1, 0], np.uint64), [0])], orc.OracleTranscript())
    assert (final[0] == orc.mle_evaluate(t, point)).all()


def test_base_field_inputs_embed(orc):
    # config-1 shape: two base-field tables, degree 2
    n = 8
    f, g = rand_base(1 << n, 400), rand_base(1 << n, 401)
    tabs = [orc.embed_base(f), orc.embed_base(g)]
    proof, point, final = orc.sc_prove(n, tabs, [(np.array([1, 0], np.uint64), [0, 1])], orc.OracleTranscript())
    s = sum(int(a) * int(b) for a, b in zip(f, g)) % pf.P
    p1 = to_E2(proof[0])
    assert p1[0] + p1[1] == E2(s)


def test_interpolate_recovers_polynomial(orc):
    rng = py_rng(9)
    coeffs = [pf.rand_e2(rng) for _ in range(5)]

    def poly(x):
        acc = E2(0)
        for c in reversed(coeffs):
            acc = acc * x + c
        return acc

    evals = [poly(E2(t)) for t in range(5)]
    r = pf.rand_e2(rng)
    assert to_E2(orc.interpolate(from_E2(evals), from_E2([r])[0]))[0] == poly(r)


def test_transcript_layout(orc):
    tr, py = orc.OracleTranscript(b"model_proving"), PyTranscript(orc.blake3, b"model_proving")
    tr.append_u64(7); py.append_u64(7)
    xs = rand_e2(3, 500)
    tr.append_scalars(xs); py.append_scalars([tuple(int(v) for v in x) for x in xs])
    a, b = tr.append_and_sample(b"batching_challenge"), py.append_and_sample(b"batching_challenge")
    assert tuple(int(v) for v in a) == b
    tr.append_bytes(b"x" * 300); py.append_bytes(b"x" * 300)
    assert tuple(int(v) for v in tr.challenge_scalar()) == py.challenge_scalar()
    assert tr.state() == (py.state, py.k)


def test_fast_build_matches_plain_build(orc):
    # the division-free build (timed as the CPU baseline) against the plain one
    n = 10
    tabs = [rand_e2(1 << n, 600 + k) for k in range(3)]
    terms = [(np.array([3, 4], np.uint64), [0, 1, 2]), (np.array([1, 0], np.uint64), [0, 2])]
    vals = [0, 1, pf.P - 1, 2**32, 2**32 - 1, 2**63, 0xFFFFFFFF00000000] + [int(x) for x in rand_base(200, 601)]
    try:
        orc.select(False)
        ref = orc.sc_prove(n, tabs, terms, orc.OracleTranscript())
        orc.select(True)
        for a in vals:
            for b in vals[:12]:
                assert orc.gl_mul(a, b) == a * b % pf.P
        fast = orc.sc_prove(n, tabs, terms, orc.OracleTranscript())
    finally:
        orc.select(False)
    for x, y in zip(ref, fast):
        assert (x == y).all()
