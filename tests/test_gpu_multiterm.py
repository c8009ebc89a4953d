"""GPU parity of sums of several product terms over shared tables (the fused multi-term kernels) against
the CPU checker, on seeded random expressions that reach every way such a session can run: rounds of more
than 2^16 pairs and of few pairs, resident rounds and the finish inside the resident launch, a common eq
factor or none, more than one group of tables, more terms than are staged on chip, repeated factors,
tables with fewer variables, tables no term uses, and a round whose claim cannot replace the evaluation at 1."""
import importlib

import numpy as np
import pytest

from util import py_rng, rand_base, rand_e2

P = 0xFFFFFFFF00000001

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dp():
    return importlib.import_module("deep-prove_amd")


@pytest.fixture(scope="module")
def ctx(dp):
    c = dp.Context(0)
    yield c
    c.close()


def _instance(ctx, orc, seed, n, table_vars, base, n_terms, max_deg, with_eq, unused=0, eq_point=None):
    """table_vars: variables of each table (n = full size, fewer = constant in the low variables);
    base: indices of base-field tables.  Returns (gpu tables, checker tables, terms)."""
    rng = py_rng(seed)
    gpu, host = [], []
    for k, m in enumerate(table_vars):
        if k in base:
            v = rand_base(1 << m, seed * 50 + k)
            gpu.append(ctx.mle_from_base(v))
            host.append(orc.embed_base(v))
        else:
            v = rand_e2(1 << m, seed * 50 + k)
            gpu.append(ctx.mle_from_ext2(v))
            host.append(v)
    used = len(table_vars) - unused
    terms = []
    for _ in range(n_terms):
        deg = rng.randint(1, max_deg)
        fs = [rng.randrange(used) for _ in range(deg)]
        coeff = np.array([rng.randrange(1, 1 << 62), rng.randrange(0, 1 << 62)], dtype=np.uint64)
        terms.append((coeff, fs))
    if with_eq:
        pt = rand_e2(n, seed * 50 + 49) if eq_point is None else eq_point
        gpu.append(ctx.eq_build(pt))
        host.append(orc.eq_evals(pt))
        e = len(gpu) - 1
        terms = [(c, fs + [e]) for c, fs in terms]
    return gpu, host, terms


def _check(dp, ctx, orc, n, gpu, host, terms):
    tr, otr = dp.Transcript(b"multi"), orc.OracleTranscript(b"multi")
    proof, point, finals = ctx.sumcheck_prove(n, gpu, terms, tr)
    oproof, opoint, ofinals = orc.sc_prove(n, host, terms, otr)
    assert (proof == oproof).all() and (point == opoint).all() and (finals == ofinals).all()
    assert tr.state() == otr.state()


CASES = [
    # n, table_vars, base, n_terms, max_deg, with_eq, unused
    dict(n=18, table_vars=[18] * 5, base=[], n_terms=12, max_deg=4, with_eq=True),          # large rounds, nested form, resident finish
    dict(n=18, table_vars=[18] * 6, base=[0, 1], n_terms=70, max_deg=3, with_eq=False),     # more terms than are staged on chip
    dict(n=17, table_vars=[17] * 12, base=[3], n_terms=20, max_deg=3, with_eq=True),        # two groups of tables
    dict(n=12, table_vars=[12] * 8, base=[], n_terms=10, max_deg=3, with_eq=True, unused=1),  # a table no term uses: finish outside
    dict(n=19, table_vars=[19, 19, 19, 10, 0, 19], base=[0, 1, 2], n_terms=9, max_deg=5, with_eq=False),  # fewer-variable tables, repeats
    dict(n=9, table_vars=[9] * 4, base=[], n_terms=6, max_deg=3, with_eq=True),             # resident from the first launch
    dict(n=10, table_vars=[10] * 3, base=[1], n_terms=5, max_deg=6, with_eq=False),          # degree 6
    dict(n=13, table_vars=[13] * 7, base=[], n_terms=48, max_deg=2, with_eq=True),          # a full group, as many terms as fit
    dict(n=1, table_vars=[1, 1], base=[], n_terms=3, max_deg=2, with_eq=True),
    dict(n=2, table_vars=[2, 2, 0], base=[], n_terms=4, max_deg=3, with_eq=False),
]


@pytest.mark.parametrize("case", range(len(CASES)))
def test_random_expressions_match_checker(dp, ctx, orc, case):
    c = dict(CASES[case])
    n = c.pop("n")
    gpu, host, terms = _instance(ctx, orc, 300 + case, n, **c)
    _check(dp, ctx, orc, n, gpu, host, terms)
    # a second proof from the same tables: nothing in a session may change them
    _check(dp, ctx, orc, n, gpu, host, terms)


@pytest.mark.parametrize("n_terms,with_eq", [(40, False), (12, True), (33, True)])
def test_many_groups(dp, ctx, orc, n_terms, with_eq):
    """every term over tables of its own: as many groups as terms -- up to 32 of them stay resident side by side
    (one workgroup each, the host adds their sums), more run a launch per round"""
    n, per_term = 8, 5
    tabs = [rand_e2(1 << n, 6000 + k) for k in range(n_terms * per_term)]
    gpu = [ctx.mle_from_ext2(t) for t in tabs]
    host = list(tabs)
    rng = py_rng(n_terms)
    terms = []
    for t in range(n_terms):
        coeff = np.array([rng.randrange(1, 1 << 62), rng.randrange(0, 1 << 62)], dtype=np.uint64)
        terms.append((coeff, [t * per_term + f for f in range(per_term)]))
    if with_eq:
        pt = rand_e2(n, 6500 + n_terms)
        gpu.append(ctx.eq_build(pt))
        host.append(orc.eq_evals(pt))
        terms = [(c, fs + [len(gpu) - 1]) for c, fs in terms]
    _check(dp, ctx, orc, n, gpu, host, terms)


@pytest.mark.parametrize("n,zero_at", [(10, 0), (10, 4), (12, 9), (12, 11), (6, 2)])
def test_eq_point_with_a_zero_coordinate(dp, ctx, orc, n, zero_at):
    """eq(rho, .) with rho_v = 0 makes the message of round v + 1 vanish at 1: that round must evaluate t = 1
    itself instead of deriving it from the claim, also when it falls among the resident rounds."""
    pt = rand_e2(n, 777 + n + zero_at)
    pt[zero_at] = 0
    gpu, host, terms = _instance(ctx, orc, 400 + n + zero_at, n, [n] * 4, [], 6, 3, True, eq_point=pt)
    _check(dp, ctx, orc, n, gpu, host, terms)
    # the same with more tables than one group holds
    gpu, host, terms = _instance(ctx, orc, 500 + n + zero_at, n, [n] * 11, [], 9, 2, True, eq_point=pt)
    _check(dp, ctx, orc, n, gpu, host, terms)
    # the single-product path with the same point
    f, g = rand_base(1 << n, 5), rand_base(1 << n, 6)
    one = np.array([1, 0], dtype=np.uint64)
    _check(dp, ctx, orc, n, [ctx.mle_from_base(f), ctx.mle_from_base(g), ctx.eq_build(pt)],
           [orc.embed_base(f), orc.embed_base(g), orc.eq_evals(pt)], [(one, [2, 0, 1])])


@pytest.mark.parametrize("n,zeros", [(6, (5,)), (9, (8, 6)), (11, (10, 9, 7, 6)), (12, (11, 3))])
@pytest.mark.parametrize("kind", ["product", "terms"])
def test_last_rounds_on_the_host_with_zero_coordinates(dp, ctx, orc, n, zeros, kind):
    """The rounds the host works out after the resident launch has left (and the last trips before them): with an eq
    point that has zero coordinates there, p(1) cannot come from the claim in those rounds and is evaluated; with the
    sum stated by the caller; round by round and through the callback entry."""
    pt = rand_e2(n, 4100 + n)
    for z in zeros:
        pt[z] = 0
    if kind == "product":
        f, g = rand_base(1 << n, 4200 + n), rand_e2(1 << n, 4201 + n)
        gpu, host = [ctx.mle_from_base(f), ctx.mle_from_ext2(g), ctx.eq_build(pt)], [orc.embed_base(f), g, orc.eq_evals(pt)]
        terms = [(np.array([7, 9], dtype=np.uint64), [2, 0, 1])]
    else:
        gpu, host, terms = _instance(ctx, orc, 4300 + n, n, [n] * 5, [1], 6, 3, True, eq_point=pt)
        terms.append((np.array([11, 0], dtype=np.uint64), []))  # and a constant term
    _check(dp, ctx, orc, n, gpu, host, terms)
    ref_proof, ref_point, ref_finals = orc.sc_prove(n, host, terms, orc.OracleTranscript(b"multi"))
    # the same with the sum stated, round by round
    claim = np.array([(int(ref_proof[0][0][k]) + int(ref_proof[0][1][k])) % P for k in range(2)], dtype=np.uint64)
    s = ctx.session(n, gpu, terms)
    s.set_claim(claim)
    chal = None
    for j in range(n):
        assert (s.round(chal) == ref_proof[j]).all(), j
        chal = ref_point[j]
    assert (s.finish(chal) == ref_finals).all()


@pytest.mark.parametrize("n,n_tabs,n_terms,with_eq", [(7, 16, 8, False), (8, 16, 8, False), (8, 16, 24, True), (9, 16, 8, False),
                                                      (12, 13, 10, True), (16, 16, 8, False), (16, 9, 12, True), (17, 16, 8, False)])
def test_more_tables_than_a_group_all_rounds_resident(dp, ctx, orc, n, n_tabs, n_terms, with_eq):
    """Up to 16 full-size tables whose first round fits the resident launches (2^15 pairs) run there from round 1,
    as the stacked products of an einsum do; the last rounds (one or two with so many tables and terms) are worked out
    on the host from the entries the launch hands over.  n = 17 is the first size that does not fit and runs the
    groups' launches."""
    gpu, host, terms = _instance(ctx, orc, 1300 + n + n_tabs, n, [n] * n_tabs, [], n_terms, 2, with_eq)
    # every table in some term: the stacked products first
    one = np.array([1, 0], dtype=np.uint64)
    e = [len(gpu) - 1] if with_eq else []
    terms = [(one, [2 * i, min(2 * i + 1, n_tabs - 1)] + e) for i in range((n_tabs + 1) // 2)] + terms[(n_tabs + 1) // 2:]
    _check(dp, ctx, orc, n, gpu, host, terms)
    _check(dp, ctx, orc, n, gpu, host, terms)


@pytest.mark.parametrize("n_tabs", [4, 11, 18])
def test_resident_groups_give_way(dp, ctx, orc, n_tabs):
    """A multi-term session stays on the GPU from the round of 256 pairs on (one workgroup, or one per group of
    tables), or from round 1 (up to 16 tables).  Another call on the context makes the resident launch exit through its mailbox, the interrupted
    session reports it, an unfinished session can simply be dropped, and the context keeps working."""
    n = 11
    gpu, host, terms = _instance(ctx, orc, 700 + n_tabs, n, [n] * n_tabs, [], 2 * n_tabs, 2, True)
    ref_proof, ref_point, ref_finals = orc.sc_prove(n, host, terms, orc.OracleTranscript(b"multi"))
    for how in ("other call", "abort", "dropped", "finish by hand"):
        s = ctx.session(n, gpu, terms)
        chal = None
        rounds = n if how == "finish by hand" else 6  # rounds 3 and later run inside the resident launch
        for j in range(rounds):
            assert (s.round(chal) == ref_proof[j]).all()
            chal = ref_point[j]
        if how == "other call":
            assert (ctx.eq_build(ref_point[:3]).download() == orc.eq_evals(ref_point[:3])).all()
            with pytest.raises(dp.DpsError):
                s.round(chal)
        elif how == "abort":
            s.abort()
            with pytest.raises(dp.DpsError):
                s.round(chal)
        elif how == "finish by hand":
            assert (s.finish(chal) == ref_finals).all()
        del s
        _check(dp, ctx, orc, n, gpu, host, terms)


@pytest.mark.parametrize("n_tabs", [4, 18])
def test_launch_made_ahead_steps_aside(dp, ctx, orc, n_tabs):
    """Rounds of few workgroups are launched during the round before and wait for their challenge.  Such a launch
    has changed nothing yet: when another call needs the context, or the caller is slow, it ends, and the session
    carries on with ordinary launches and the same messages."""
    import time
    # 18 tables are several groups: launches of their own up to round 5 (a launch stays for the later rounds from
    # n - j + 1 <= 9 on).  4 tables are one group, whose rounds are resident from the first that fits 256 workgroups of 512
    # pairs (round 3 of 20): rounds 1 and 2 are launches, and the resident launches are queued during round 2.
    n, afters = (14, (1, 3, 4, 5)) if n_tabs > 7 else (20, (1, 2))
    gpu, host, terms = _instance(ctx, orc, 900 + n_tabs, n, [n] * n_tabs, [], 2 * n_tabs, 2, True)
    ref_proof, ref_point, ref_finals = orc.sc_prove(n, host, terms, orc.OracleTranscript(b"multi"))
    for after in afters:
        for how in ("other call", "slow caller"):
            s = ctx.session(n, gpu, terms)
            chal = None
            for j in range(n):
                assert (s.round(chal) == ref_proof[j]).all(), (after, how, j)
                chal = ref_point[j]
                if j + 1 == after:
                    if how == "other call":
                        assert (ctx.eq_build(ref_point[:3]).download() == orc.eq_evals(ref_point[:3])).all()
                    else:
                        # longer than the host trusts the launch to wait; the first time, longer than the launch waits
                        time.sleep(0.3 if after == 1 else 0.05)
            assert (s.finish(chal) == ref_finals).all()
            del s
    _check(dp, ctx, orc, n, gpu, host, terms)


@pytest.mark.parametrize("with_eq,n", [(True, 21), (False, 21), (True, 22)])
def test_product_launch_made_ahead_steps_aside(dp, ctx, orc, with_eq, n):
    """The same for a single product of full-size tables.  Its rounds are resident from the first that fits 256
    workgroups of 1024 pairs (round 3 of 21, round 4 of 22); the rounds before are launches, each made during the round
    before it, and so are the resident launches (several workgroups, then one).  In a launch of more than 64
    workgroups only the first workgroup looks for the mail and passes it on to the others; the resident launch of
    several workgroups always does so.  Once a resident launch has had its first mail another call on the context ends
    the session (test_resident_kernel_gives_way)."""
    import time
    f, g = rand_base(1 << n, 31), rand_e2(1 << n, 32)
    gpu, host, fs = [ctx.mle_from_base(f), ctx.mle_from_ext2(g)], [orc.embed_base(f), g], [0, 1]
    if with_eq:
        pt = rand_e2(n, 33)
        gpu.append(ctx.eq_build(pt))
        host.append(orc.eq_evals(pt))
        fs = [2, 0, 1]
    terms = [(np.array([3, 5], dtype=np.uint64), fs)]
    ref_proof, ref_point, ref_finals = orc.sc_prove(n, host, terms, orc.OracleTranscript(b"multi"))
    for after in (1, 2):
        for how in ("other call", "slow caller"):
            s = ctx.session(n, gpu, terms)
            chal = None
            for j in range(n):
                assert (s.round(chal) == ref_proof[j]).all(), (after, how, j)
                chal = ref_point[j]
                if j + 1 == after:
                    if how == "other call":
                        assert (ctx.eq_build(ref_point[:3]).download() == orc.eq_evals(ref_point[:3])).all()
                    else:
                        # longer than the host trusts the launch to wait; the first time, longer than the launch waits
                        time.sleep(0.3 if after == 1 else 0.05)
            assert (s.finish(chal) == ref_finals).all()
            del s
    # a slow caller in the resident rounds is waited for (the resident launches poll for seconds, not milliseconds)
    s = ctx.session(n, gpu, terms)
    chal = None
    for j in range(n):
        assert (s.round(chal) == ref_proof[j]).all(), j
        chal = ref_point[j]
        if j + 1 in (4, 5, n - 1):
            time.sleep(0.05)
    assert (s.finish(chal) == ref_finals).all()
    del s
    _check(dp, ctx, orc, n, gpu, host, terms)


def _fadd(a, b):
    """sum of two extension elements given as limb pairs"""
    P = 0xFFFFFFFF00000001
    return np.array([(int(a[0]) + int(b[0])) % P, (int(a[1]) + int(b[1])) % P], dtype=np.uint64)


@pytest.mark.parametrize("shape", ["product n=6", "product n=14", "product n=19", "product n=12 no eq", "terms n=8", "terms n=13", "terms n=18"])
def test_claim_known_before_round_one(dp, ctx, orc, shape):
    """With the value of the whole sum given (dps_sc_set_claim) round 1 takes p(1) from it like every later round;
    the messages and final evaluations are the same bits.  Covers the single-product kernels (small, with the resident
    last rounds, with factored eq weights) and the multi-term ones (resident from round 1, launched, large rounds)."""
    kind, rest = shape.split(" ", 1)
    n = int(rest.split("=")[1].split()[0])
    if kind == "product":
        f, g = rand_base(1 << n, 41), rand_e2(1 << n, 42)
        gpu, host, fs = [ctx.mle_from_base(f), ctx.mle_from_ext2(g)], [orc.embed_base(f), g], [0, 1]
        if "no eq" not in shape:
            pt = rand_e2(n, 43)
            gpu.append(ctx.eq_build(pt))
            host.append(orc.eq_evals(pt))
            fs = [2, 0, 1]
        terms = [(np.array([3, 5], dtype=np.uint64), fs)]
    else:
        gpu, host, terms = _instance(ctx, orc, 1200 + n, n, [n] * 5, [1], 9, 3, True)
    ref_proof, ref_point, ref_finals = orc.sc_prove(n, host, terms, orc.OracleTranscript(b"multi"))
    s = ctx.session(n, gpu, terms)
    s.set_claim(_fadd(ref_proof[0][0], ref_proof[0][1]))
    chal = None
    for j in range(n):
        assert (s.round(chal) == ref_proof[j]).all(), (shape, j)
        chal = ref_point[j]
    assert (s.finish(chal) == ref_finals).all()
    # too late once the session has started
    with pytest.raises(dp.DpsError):
        s.set_claim(ref_proof[0][0])
    del s
    # a wrong claim gives a first message that sums to it (and no longer the true one)
    s = ctx.session(n, gpu, terms)
    wrong = _fadd(_fadd(ref_proof[0][0], ref_proof[0][1]), np.array([1, 0], dtype=np.uint64))
    s.set_claim(wrong)
    m = s.round(None)
    assert (m[0] == ref_proof[0][0]).all() and (_fadd(m[0], m[1]) == wrong).all()
    del s
    _check(dp, ctx, orc, n, gpu, host, terms)
