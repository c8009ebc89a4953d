"""GPU parity of the sumcheck that links a lookup argument to its layer
(zkml/src/lookup/operation/inputs/proving.rs:26-114, every variant of
variant.rs:222-348) against the CPU checker, and the verifier's round trip."""
import importlib

import numpy as np
import pytest

from linking_cases import CASES, chunk_vars, make_instance

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dp():
    return importlib.import_module("deep-prove_amd")


@pytest.fixture(scope="module")
def ctx(dp):
    c = dp.Context(0)
    yield c
    c.close()


def _run(dp, ctx, orc, cfg, seed, big=None):
    tabs, weight, lcp, lp = make_instance(cfg, seed)
    nv = chunk_vars(cfg)
    gpu = [ctx.mle_from_i64(t, nv) for t in tabs]
    gw = None if weight is None else ctx.mle_from_i64(weight, nv)
    tr, otr = dp.Transcript(b"linking"), orc.OracleTranscript(b"linking")
    proof, point, evals, weight_eval, ch = dp.linking_prove(ctx, cfg, gpu, tr, lcp, lp, gw)
    omles = [orc.embed_i64(t) for t in tabs]
    ow = None if weight is None else orc.embed_i64(weight)
    oproof, opoint, oevals, oweight_eval, och = orc.linking_prove(cfg, omles, otr, lcp, lp, ow)
    assert proof.shape == oproof.shape and (proof == oproof).all()
    assert (point == opoint).all() and (evals == oevals).all()
    assert (weight_eval is None) == (oweight_eval is None)
    if weight_eval is not None:
        assert (weight_eval == oweight_eval).all()
    assert len(ch) == len(och) and all((a == b).all() for a, b in zip(ch, och))
    assert tr.state() == otr.state()
    return proof, point, evals, weight_eval, lcp, lp, tr


@pytest.mark.parametrize("case", range(len(CASES)))
def test_linking_sumcheck_matches_checker_and_verifies(dp, ctx, orc, case):
    cfg = CASES[case]
    proof, point, evals, weight_eval, lcp, lp, tr = _run(dp, ctx, orc, cfg, 50 + case)
    claim = orc.e2_add(proof[0][0], proof[0][1])
    vt = dp.Transcript(b"linking")
    rc, vpoint = dp.linking_verify(cfg, claim, proof, evals, weight_eval, vt, lcp, lp)
    assert rc == 0 and (vpoint == point).all() and vt.state() == tr.state()
    bad = evals.copy()
    bad[0, 0] ^= np.uint64(1)
    assert dp.linking_verify(cfg, claim, proof, bad, weight_eval, dp.Transcript(b"linking"), lcp, lp)[0] != 0
    assert dp.linking_verify(cfg, orc.e2_add(claim, orc.e2(1)), proof, evals, weight_eval, dp.Transcript(b"linking"), lcp, lp)[0] != 0


def test_linking_sumcheck_layer_sized(dp, ctx, orc):
    # a GPT-2 sized activation: 12 heads of 256 x 64 through a signed table with one zeroing chunk
    cfg = dict(variant="standard", shape=[12, 256, 64], value_chunks=1, zero_chunks=1, bit_size=8, signed=True, min_out=-128, max_out=127,
               input_sign="positive", norm_sum=False, has_weight=False)
    proof, *_ = _run(dp, ctx, orc, cfg, 7)
    assert proof.shape == (14, 5, 2)


def test_linking_sumcheck_argument_errors(dp, ctx):
    cfg = CASES[1]
    tabs, weight, lcp, lp = make_instance(cfg, 3)
    nv = chunk_vars(cfg)
    gpu = [ctx.mle_from_i64(t, nv) for t in tabs]
    with pytest.raises(dp.DpsError):   # a table short
        dp.linking_prove(ctx, cfg, gpu[:-1], dp.Transcript(b"x"), lcp, lp)
    with pytest.raises(dp.DpsError):   # claim point of the wrong length
        dp.linking_prove(ctx, cfg, gpu, dp.Transcript(b"x"), lcp[:-1], lp)
    with pytest.raises(dp.DpsError):   # a weight table where the variant has none
        dp.linking_prove(ctx, cfg, gpu, dp.Transcript(b"x"), lcp, lp, gpu[0])
    with pytest.raises(dp.DpsError):   # a table with fewer variables than the chunk
        dp.linking_prove(ctx, cfg, [ctx.mle_from_i64(tabs[0][: 1 << (nv - 1)], nv - 1)] + gpu[1:], dp.Transcript(b"x"), lcp, lp)
