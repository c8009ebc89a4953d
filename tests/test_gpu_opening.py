"""GPU parity of the claims-batching sumcheck of the opening proof
(zkml/src/poly_commit/prover.rs:140-255) against the CPU checker."""
import importlib

import numpy as np
import pytest

from opening_cases import make_instance

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dp():
    return importlib.import_module("deep-prove_amd")


@pytest.fixture(scope="module")
def ctx(dp):
    c = dp.Context(0)
    yield c
    c.close()


@pytest.mark.parametrize("chunk_vars,small", [(None, True), (4, True), (None, False), (10, False)])
def test_claims_batching_matches_checker_and_verifies(dp, ctx, orc, chunk_vars, small):
    polys, claims, shapes = make_instance(orc, 11, chunk_vars, small)
    # every polynomial is uploaded once; its chunks are borrowed windows of that upload
    gpu_polys = []
    for chunks in polys:
        whole = ctx.mle_from_ext2(np.concatenate(chunks))
        m = len(chunks[0]).bit_length() - 1
        gpu_polys.append([whole.view(c << m, m) for c in range(len(chunks))])
    tr, otr = dp.Transcript(b"commit test"), orc.OracleTranscript(b"commit test")
    proof, point, evals = dp.claims_batching_prove(ctx, gpu_polys, claims, tr)
    oproof, opoint, oevals = orc.claims_batching_prove(polys, claims, otr)
    assert (proof == oproof).all() and (point == opoint).all() and (evals == oevals).all()
    assert tr.state() == otr.state()
    rc, vpoint = dp.claims_batching_verify(shapes, claims, proof, evals, dp.Transcript(b"commit test"))
    assert rc == 0 and (vpoint == point).all()
    bad = evals.copy()
    bad[0, 1] ^= np.uint64(1)
    rc, _ = dp.claims_batching_verify(shapes, claims, proof, bad, dp.Transcript(b"commit test"))
    assert rc != 0


@pytest.mark.parametrize("n,k", [(10, 14), (4, 1), (13, 3)])
def test_same_poly_matches_checker_and_verifies(dp, ctx, orc, n, k):
    # zkml/src/iop/same_poly.rs:190-229
    from util import rand_e2

    poly = rand_e2(1 << n, 700 + n)
    claims = []
    for i in range(k):
        pt = rand_e2(n, 800 + 7 * n + i)
        claims.append((pt, orc.mle_evaluate(poly, pt)))
    tr, otr = dp.Transcript(), orc.OracleTranscript()
    h = ctx.mle_from_ext2(poly)
    proof, point, ev = dp.same_poly_prove(ctx, h, claims, tr)
    oproof, opoint, oev = orc.same_poly_prove(poly, claims, otr)
    assert (proof == oproof).all() and (point == opoint).all() and (ev == oev).all() and tr.state() == otr.state()
    assert (h.evaluate(point) == ev).all()
    rc, vpoint = dp.same_poly_verify(n, claims, proof, ev, dp.Transcript())
    assert rc == 0 and (vpoint == point).all()
    bad = proof.copy()
    bad[0, 0, 0] ^= np.uint64(1)
    assert dp.same_poly_verify(n, claims, bad, ev, dp.Transcript())[0] != 0
