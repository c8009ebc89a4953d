"""CPU checks of the checker's claims-batching sumcheck (zkml/src/poly_commit):
what pins it without the reference's engine are the protocol's own identities."""
import numpy as np
import pytest

from opening_cases import make_instance
from pyfield import E2
from util import from_E2, rand_e2, to_E2


def test_chunk_coefficients_rebuild_the_claim(orc):
    # mod.rs:38-45: P(r) = sum_c C_c P_c(r_1..r_m) with C_c = eq(bits(c), r_{m+1..n})
    for nv, m in [(6, 6), (6, 4), (7, 2), (5, 0)]:
        full = rand_e2(1 << nv, 40 + nv + m)
        point = rand_e2(nv, 90 + nv)
        nch = 1 << (nv - m)
        coeffs = orc.chunk_batching_coefficients(nch, point)
        acc = E2(0)
        for c in range(nch):
            v = to_E2(orc.mle_evaluate(full[c << m:(c + 1) << m], point[:m]))[0]
            acc = acc + to_E2(coeffs[c])[0] * v
        assert (from_E2([acc])[0] == orc.mle_evaluate(full, point)).all()


@pytest.mark.parametrize("chunk_vars", [None, 4])
def test_claims_batching_round_trip(orc, chunk_vars):
    polys, claims, shapes = make_instance(orc, 7, chunk_vars, small=True)
    tr = orc.OracleTranscript(b"commit test")
    proof, point, evals = orc.claims_batching_prove(polys, claims, tr)
    n = max(len(c[0]).bit_length() - 1 for c in polys)
    assert proof.shape == (n, 3, 2) and evals.shape[0] == sum(len(c) for c in polys)
    # the evaluations handed on are those of the zero-padded chunk tables at the common point
    k = 0
    for chunks in polys:
        for ch in chunks:
            m = len(ch).bit_length() - 1
            v = to_E2(orc.mle_evaluate(ch, point[:m]))[0]
            for r in to_E2(point[m:]):
                v = v * (E2(1) - r)
            assert (evals[k] == from_E2([v])[0]).all()
            k += 1
    vt = orc.OracleTranscript(b"commit test")
    ok, vpoint = orc.claims_batching_verify(shapes, claims, proof, evals, vt)
    assert ok and (vpoint == point).all() and vt.state() == tr.state()
    # a wrong claim, a wrong evaluation and a wrong message are each rejected
    bad_claims = [list(c) for c in claims]
    p0, e0 = bad_claims[2][0]
    bad_claims[2][0] = (p0, orc.e2_add(e0, orc.e2(1)))
    assert not orc.claims_batching_verify(shapes, bad_claims, proof, evals, orc.OracleTranscript(b"commit test"))[0]
    bad_evals = evals.copy()
    bad_evals[1, 0] ^= np.uint64(1)
    assert not orc.claims_batching_verify(shapes, claims, proof, bad_evals, orc.OracleTranscript(b"commit test"))[0]
    bad_proof = proof.copy()
    bad_proof[n - 1, 2, 1] ^= np.uint64(2)
    assert not orc.claims_batching_verify(shapes, claims, bad_proof, evals, orc.OracleTranscript(b"commit test"))[0]


def test_same_poly_round_trip(orc):
    # zkml/src/iop/same_poly.rs:190-229 (test_same_poly_proof): 14 claims on a 10-variable polynomial; the merged
    # claim must be a true evaluation of the polynomial
    n, k = 10, 14
    poly = rand_e2(1 << n, 321)
    claims = []
    for i in range(k):
        pt = rand_e2(n, 400 + i)
        claims.append((pt, orc.mle_evaluate(poly, pt)))
    tr = orc.OracleTranscript()
    proof, point, ev = orc.same_poly_prove(poly, claims, tr)
    assert (ev == orc.mle_evaluate(poly, point)).all()
    vt = orc.OracleTranscript()
    ok, vpoint = orc.same_poly_verify(n, claims, proof, ev, vt)
    assert ok and (vpoint == point).all() and vt.state() == tr.state()
    bad = [(p, e) for p, e in claims]
    bad[5] = (bad[5][0], orc.e2_add(bad[5][1], orc.e2(1)))
    assert not orc.same_poly_verify(n, bad, proof, ev, orc.OracleTranscript())[0]
    assert not orc.same_poly_verify(n, claims, proof, orc.e2_add(ev, orc.e2(0, 1)), orc.OracleTranscript())[0]
