"""Sums that are worked out on the host from their first round: the small layers of a fraction tree.

The last launch of a tree's build leaves the layers of at most 256 entries per array in host memory as well, and a sum
of at most 7 variables over such tables (every layer sumcheck of the LogUp-GKR prover near the root of the tree,
zkml/src/lookup/logup_gkr/prover.rs:205-296) then runs without any launch: the entries are there, the eq factor is taken
from its point, and a few hundred field products take the host less time than a launch takes to start.  Checked here:
such a session's messages, challenges' effect and final evaluations are the checker's, it holds no place on the device,
and it falls back to launches when the host's copies are no longer those of its tree."""
import importlib

import numpy as np
import pytest

from util import rand_base, rand_e2

pytestmark = pytest.mark.gpu

ONE = np.array([1, 0], dtype=np.uint64)


@pytest.fixture(scope="module")
def dp():
    return importlib.import_module("deep-prove_amd")


def _tree(ctx, n, seed, table=False):
    cols = [ctx.mle_from_base(rand_base(1 << n, seed + k)) for k in range(2)]
    numer = ctx.mle_from_base(rand_base(1 << n, seed + 9)) if table else None
    c, beta = rand_e2(1, seed + 10)[0], rand_e2(1, seed + 11)[0]
    return ctx.logup_build(cols, numer, c, beta), cols, numer


def _layer_sum(ctx, orc, lg, k, seed):
    """the sumcheck the prover runs over layer k of a tree: eq * (n_lo d_hi + n_hi d_lo + lambda d_lo d_hi) over the
    layer's halves.  Returns (n_vars, device tables, host tables, terms)."""
    num, den = lg.layer(k)
    m = int(num.info()[1]).bit_length() - 2  # variables of a half
    half = 1 << m
    views = [num.view(0, m), num.view(half, m), den.view(0, m), den.view(half, m)]
    host = [v.download() for v in views]
    r = rand_e2(m, seed)
    lam = rand_e2(1, seed + 1)[0]
    terms = [(ONE, [4, 0, 3]), (ONE, [4, 1, 2]), (lam, [4, 2, 3])]
    return m, views + [ctx.eq_build(r)], host + [orc.eq_evals(r)], terms


def _run_rounds(dp, orc, ctx, m, dev_tabs, host_tabs, terms, label, with_claim, expect_on_host):
    ref_proof, ref_point, ref_finals = orc.sc_prove(m, host_tabs, terms, orc.OracleTranscript(label))
    s = ctx.session(m, dev_tabs, terms)
    if with_claim:
        p0, p1 = [int(x) for x in ref_proof[0][0]], [int(x) for x in ref_proof[0][1]]
        s.set_claim(np.array([(p0[0] + p1[0]) % dp.P, (p0[1] + p1[1]) % dp.P], dtype=np.uint64))
    for j in range(m):
        got = s.round(None if j == 0 else ref_point[j - 1])
        assert (got == ref_proof[j]).all(), (m, j)
        if j == 0 and m >= 6:
            # a sum of this size is otherwise resident on the GPU from its first round, and its launch holds a place there
            assert (dp.resident_budget(0)[0] == 0) == expect_on_host, (m, dp.resident_budget(0))
    finals = s.finish(ref_point[m - 1])
    assert (finals == ref_finals).all()
    assert dp.resident_budget(0)[0] == 0


@pytest.mark.parametrize("table", [False, True])
def test_layer_sums_near_the_root_run_on_the_host(dp, orc, table):
    ctx = dp.Context(0)
    lg, _, _ = _tree(ctx, 11, 51000, table)
    top = lg.num_layers()
    # layers of 2^10 .. 2 entries per array: the sums have 9 .. 0 variables; those of at most 7 are the host's
    for k in range(1, top):
        m, dev_tabs, host_tabs, terms = _layer_sum(ctx, orc, lg, k, 51100 + k)
        if m < 1:
            continue
        for with_claim in (True, False):
            _run_rounds(dp, orc, ctx, m, dev_tabs, host_tabs, terms, b"host rounds", with_claim, expect_on_host=m <= 7)
    ctx.close()


def test_product_over_two_small_layer_tables(dp, orc):
    """one product of two tables (with and without an eq factor) instead of a sum of several terms"""
    ctx = dp.Context(0)
    lg, _, _ = _tree(ctx, 9, 52000)
    num, den = lg.layer(3)  # 2^6 entries each
    m = 6
    host = [num.download(), den.download()]
    r = rand_e2(m, 52010)
    for terms, dev_tabs, host_tabs in (
        ([(rand_e2(1, 52011)[0], [0, 1])], [num, den], host),
        ([(ONE, [2, 0, 1])], [num, den, ctx.eq_build(r)], host + [orc.eq_evals(r)]),
    ):
        ref = orc.sc_prove(m, host_tabs, terms, orc.OracleTranscript(b"small product"))
        got = ctx.sumcheck_prove(m, dev_tabs, terms, dp.Transcript(b"small product"))
        assert all((np.asarray(a) == np.asarray(b)).all() for a, b in zip(got, ref))
    ctx.close()


def test_host_copies_of_an_older_tree_are_not_used(dp, orc):
    """The copies rotate through a few areas of host memory: once the context has built that many more trees, a sum over
    an older tree's small layer runs as launches again -- same proof."""
    ctx = dp.Context(0)
    lg, _, _ = _tree(ctx, 10, 53000)
    m, dev_tabs, host_tabs, terms = _layer_sum(ctx, orc, lg, 2, 53100)
    assert m == 7  # (as launches: two trips and three rounds on the host, so the launch still waits after round 1)
    _run_rounds(dp, orc, ctx, m, dev_tabs, host_tabs, terms, b"older tree", True, expect_on_host=True)
    later = [_tree(ctx, 9, 53200 + 20 * i)[0] for i in range(8)]
    _run_rounds(dp, orc, ctx, m, dev_tabs, host_tabs, terms, b"older tree", True, expect_on_host=False)
    # ... while the newest tree's layers are the host's
    m2, dev2, host2, terms2 = _layer_sum(ctx, orc, later[-1], 2, 53400)  # (layer 1 is the first launch's, the others the last one's)
    assert m2 == 6
    _run_rounds(dp, orc, ctx, m2, dev2, host2, terms2, b"newest tree", False, expect_on_host=True)
    ctx.close()


def test_small_eq_table_is_built_when_its_entries_are_read(dp, orc):
    """An eq table of few variables is not built when it is made (a sum on the host reads its point): whoever reads
    entries gets them all the same."""
    ctx = dp.Context(0)
    for m in (0, 1, 3, 7):
        r = rand_e2(m, 54000 + m)
        e = ctx.eq_build(r)
        want = orc.eq_evals(r)
        if m >= 1:
            # first as a factor of a sum over ordinary tables (launches), then as entries
            f = rand_e2(1 << m, 54100 + m)
            ref = orc.sc_prove(m, [f, want], [(ONE, [0, 1])], orc.OracleTranscript(b"eq"))
            got = ctx.sumcheck_prove(m, [ctx.mle_from_ext2(f), e], [(ONE, [0, 1])], dp.Transcript(b"eq"))
            assert all((np.asarray(a) == np.asarray(b)).all() for a, b in zip(got, ref))
        assert (e.download() == want).all()
        if m >= 1:
            assert (e.view(0, m - 1).download() == want[: 1 << (m - 1)]).all()
            pt = rand_e2(m, 54200 + m)
            assert (e.evaluate(pt) == orc.mle_evaluate(want, pt)).all()
    ctx.close()
