"""GPU parity: field arithmetic, table routines and the sumcheck engine through
the C ABI, bit for bit against the CPU checker on the same seeded inputs."""
import importlib

import numpy as np
import pytest

import pyfield as pf
from pyfield import E2, P
from util import from_E2, py_rng, rand_base, rand_e2, rand_i64, to_E2

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dp():
    return importlib.import_module("deep-prove_amd")


@pytest.fixture(scope="module")
def ctx(dp):
    c = dp.Context(0)
    yield c
    c.close()


ONE = np.array([1, 0], dtype=np.uint64)
EDGE = [0, 1, 2, 7, P - 1, P - 2, 2**32, 2**32 - 1, 2**32 + 1, 2**63, 2**63 - 1, (P - 1) // 2, (P + 1) // 2, 0xFFFFFFFF,
        0xFFFFFFFF00000000, 0xFFFFFFFE00000001, 0xFFFFFFFEFFFFFFFF,
        # products whose top limb exceeds the low word while the third limb is zero, one, or large (borrow alone, borrow
        # and carry together in the reduction)
        2**48, 2**48 + 2**16, 2**48 + 2**47 + 1]


def test_device_field_arithmetic(ctx):
    rng = py_rng(11)
    vals = EDGE + [rng.randrange(P) for _ in range(2000)]
    # all edge pairs, then random pairs
    a0 = [x for x in EDGE for _ in EDGE] + vals
    b0 = [y for _ in EDGE for y in EDGE] + list(reversed(vals))
    a1 = list(reversed(a0))
    b1 = [b0[(i * 7 + 3) % len(b0)] for i in range(len(b0))]
    A = np.array(list(zip(a0, a1)), dtype=np.uint64)
    B = np.array(list(zip(b0, b1)), dtype=np.uint64)
    got = {op: ctx.field_op(op, A, B) for op in (0, 1, 2, 3, 4, 6, 7, 8)}
    for i in range(len(a0)):
        x, y = E2(a0[i], a1[i]), E2(b0[i], b1[i])
        assert tuple(int(v) for v in got[0][i]) == (x + y).pair()
        assert tuple(int(v) for v in got[1][i]) == (x - y).pair()
        assert tuple(int(v) for v in got[2][i]) == (x * y).pair()
        assert tuple(int(v) for v in got[3][i]) == (a0[i] * b0[i] % P, a1[i] * b1[i] % P)
        assert tuple(int(v) for v in got[4][i]) == (x * E2(b0[i])).pair()
        # products gathered without a reduction per product: one product pair plus a term, and a long sum
        assert tuple(int(v) for v in got[6][i]) == (x * y + x).pair()
        assert tuple(int(v) for v in got[7][i]) == ((a0[i] * b0[i] + a1[i]) % P, (a0[i] * b0[i] + a1[i] * b1[i] + b0[i]) % P)
        long_sum = E2(40) * (x * y + y * E2(a1[i]) + x) + E2(0, 40 * b0[i] % P)
        assert tuple(int(v) for v in got[8][i]) == long_sum.pair()
    # int64 embedding and multiplication by a 32-bit constant
    ints = [0, 1, -1, 2047, -2048, 2**40, -(2**40), 2**62, -(2**62), -(2**63), 2**63 - 1]
    A = np.array([[x % 2**64, vals[i]] for i, x in enumerate(ints)], dtype=np.uint64)
    B = np.array([[0, c] for c in [7, 1, 0, 2**32 - 1, 12345, 7, 7, 7, 7, 7, 7]], dtype=np.uint64)
    got = ctx.field_op(5, A, B)
    for i, x in enumerate(ints):
        assert int(got[i][0]) == x % P
        assert int(got[i][1]) == vals[i] * int(B[i][1]) % P


@pytest.mark.parametrize("m", [0, 1, 2, 5, 8, 9, 11, 16, 17])
def test_eq_table(ctx, orc, m):
    point = rand_e2(m, 20 + m)
    got = ctx.eq_build(point).download()
    assert (got == orc.eq_evals(point)).all()


@pytest.mark.parametrize("m", [19, 21])
def test_eq_table_read_as_entries_after_a_session(dp, ctx, orc, m):
    """An eq table of more than 17 variables is built piecewise: the small suffix levels with the table, the rest when
    something reads them.  A product session (which reads levels, not entries), then the table's own entries through a
    view, an evaluation and a download: each finds what it needs, whatever was built before."""
    point = rand_e2(m, 70 + m)
    f = rand_base(1 << m, 71 + m)
    eq, mf = ctx.eq_build(point), ctx.mle_from_base(f)
    terms = [(np.array([1, 0], dtype=np.uint64), [0, 1])]
    want_eq = orc.eq_evals(point)
    ref = orc.sc_prove(m, [want_eq, orc.embed_base(f)], terms, orc.OracleTranscript(b"lazy"))
    got = ctx.sumcheck_prover(m, [eq, mf], terms)(dp.Transcript(b"lazy"))
    assert all((a == b).all() for a, b in zip(got, ref))
    half = eq.view(1 << (m - 1), m - 1).download()
    assert (half == want_eq[1 << (m - 1):]).all()
    z = rand_e2(m, 72 + m)
    assert (eq.evaluate(z) == orc.mle_evaluate(want_eq, z)).all()
    assert (eq.download() == want_eq).all()
    # and in the other order: entries first, a session afterwards
    eq2 = ctx.eq_build(point)
    assert (eq2.download() == want_eq).all()
    got2 = ctx.sumcheck_prover(m, [eq2, mf], terms)(dp.Transcript(b"lazy"))
    assert all((a == b).all() for a, b in zip(got2, ref))


def test_i64_embedding_and_padding(ctx, orc):
    v = rand_i64(300, 31, lo=-2**40, hi=2**40)
    v[:4] = [0, -1, 2**62, -(2**62)]
    got = ctx.mle_from_i64(v).download()
    assert got.shape[0] == 512
    assert (got[:300] == orc.embed_i64(v)).all() and (got[300:] == 0).all()


@pytest.mark.parametrize("n", [1, 4, 9, 14])
def test_evaluate_fix_low_fix_high(ctx, orc, n):
    tab = rand_e2(1 << n, 40 + n)
    base = rand_base(1 << n, 50 + n)
    point = rand_e2(n, 60 + n)
    m, mb = ctx.mle_from_ext2(tab), ctx.mle_from_base(base)
    assert (m.evaluate(point) == orc.mle_evaluate(tab, point)).all()
    assert (mb.evaluate(point) == orc.mle_evaluate(orc.embed_base(base), point)).all()
    for k in sorted({0, 1, n // 2, n}):
        assert (m.fix_low(point[:k]).download() == orc.mle_fix_low(tab, point[:k])).all()
        assert (mb.fix_low(point[:k]).download() == orc.mle_fix_low(orc.embed_base(base), point[:k])).all()
        assert (m.fix_high(point[n - k:]).download() == orc.mle_fix_high(tab, point[n - k:])).all()


def test_vector_and_tensor_mle_layout(ctx):
    # zkml/src/lib.rs:357-369 and zkml/src/tensor/mod.rs:1874-1897 restated on the GPU tables
    n = 6
    v = rand_e2(1 << n, 70)
    m = ctx.mle_from_ext2(v)
    for i in [0, 5, 37, 63]:
        assert (m.evaluate(from_E2([E2((i >> j) & 1) for j in range(n)])) == v[i]).all()
    rows, cols = 8, 8
    for r in [0, 3, 7]:
        row = m.fix_high(from_E2([E2((r >> j) & 1) for j in range(3)]))
        assert (row.download() == v[r * cols:(r + 1) * cols]).all()


def _check_prove(dp, ctx, orc, n, gpu_tabs, orc_tabs, terms, label=b"m2vec"):
    tr, otr = dp.Transcript(label), orc.OracleTranscript(label)
    proof, point, finals = ctx.sumcheck_prove(n, gpu_tabs, terms, tr)
    oproof, opoint, ofinals = orc.sc_prove(n, orc_tabs, terms, otr)
    assert (proof == oproof).all()
    assert (point == opoint).all()
    assert (finals == ofinals).all()
    assert tr.state() == otr.state()
    return proof, point, finals


SHAPES = [
    (4, [4, 4], [((1, 0), [0, 1])]),
    (4, [4, 4, 4], [((1, 0), [0, 1, 2])]),
    (3, [3, 3, 3, 3], [((5, 9), [0, 2]), ((11, 3), [1, 3])]),
    (4, [4, 2, 4, 2], [((3, 1), [0, 2]), ((2, 2), [1, 3]), ((7, 0), [0, 1, 2])]),
    (3, [3], [((1, 0), [0])]),
    (3, [3, 3, 3, 3, 3], [((1, 0), [0, 1, 2, 3, 4])]),
    (6, [6, 6, 6, 6, 6, 6], [((1, 0), [0, 1, 2, 3, 4, 5])]),
    (9, [9, 9, 0, 4], [((2, 3), [0, 1]), ((4, 5), [2, 3, 0]), ((9, 9), [])]),
    (1, [1, 1], [((1, 0), [0, 1])]),
    (5, [5, 5], [((1, 0), [0, 0, 1])]),
    (10, [10, 10, 10, 7, 7, 7], [((1, 1), [0, 1, 2]), ((2, 5), [3, 4, 5]), ((3, 0), [0, 5])]),
]


@pytest.mark.parametrize("case", range(len(SHAPES)))
def test_sumcheck_matches_checker_small_shapes(dp, ctx, orc, case):
    n, nvars, terms = SHAPES[case]
    terms = [(np.array(c, dtype=np.uint64), f) for c, f in terms]
    tabs = [rand_e2(1 << m, 1000 + 17 * case + k) for k, m in enumerate(nvars)]
    gpu = [ctx.mle_from_ext2(t) for t in tabs]
    _check_prove(dp, ctx, orc, n, gpu, tabs, terms)


@pytest.mark.parametrize("n", [2, 7, 16])
def test_config1_plain_product_base_field(dp, ctx, orc, n):
    # two base-field tables, degree 2 (configuration 1 at n = 16)
    f, g = rand_base(1 << n, 2000 + n), rand_base(1 << n, 2100 + n)
    gpu = [ctx.mle_from_base(f), ctx.mle_from_base(g)]
    proof, _, _ = _check_prove(dp, ctx, orc, n, gpu, [orc.embed_base(f), orc.embed_base(g)], [(ONE, [0, 1])])
    s = sum(int(a) * int(b) for a, b in zip(f, g)) % P
    p1 = to_E2(proof[0])
    assert p1[0] + p1[1] == E2(s)


@pytest.mark.parametrize("n,mix", [(3, "bbe"), (8, "bbe"), (15, "bbe"), (9, "bee"), (9, "eee"), (9, "bbb"), (9, "ebe"), (8, "be"), (8, "ee")])
def test_hadamard_shape_mixed_fields(dp, ctx, orc, n, mix):
    # eq(r, x) * f(x) * g(x) (zkml/src/layers/hadamard.rs:93-131) with base and extension inputs in every order
    gpu, ref = [], []
    for k, kind in enumerate(mix):
        if kind == "b":
            v = rand_base(1 << n, 3000 + 31 * n + k)
            gpu.append(ctx.mle_from_base(v))
            ref.append(orc.embed_base(v))
        else:
            v = rand_e2(1 << n, 3500 + 31 * n + k)
            gpu.append(ctx.mle_from_ext2(v))
            ref.append(v)
    _check_prove(dp, ctx, orc, n, gpu, ref, [(ONE, list(range(len(mix))))])


def test_hadamard_proving_roundtrip(dp, ctx, orc):
    # test_hadamard_proving (zkml/src/layers/hadamard.rs:173-209): prove, verify, check the input claim
    n = 10
    v1, v2 = rand_i64(1 << n, 4000), rand_i64(1 << n, 4001)
    r = rand_e2(n, 4002)
    out = ctx.mle_from_i64(v1 * v2)
    claim = out.evaluate(r)
    m1, m2, beta = ctx.mle_from_i64(v1), ctx.mle_from_i64(v2), ctx.eq_build(r)
    tr = dp.Transcript()
    proof, point, finals = ctx.sumcheck_prove(n, [m1, m2, beta], [(ONE, [0, 1, 2])], tr)
    p1 = to_E2(proof[0])
    assert p1[0] + p1[1] == to_E2(claim)[0]  # extract_sum == claim
    rc, vpoint, expected = ctx.sumcheck_verify(claim, proof, dp.Transcript())
    assert rc == 0 and (vpoint == point).all()
    beta_eval = orc.identity_eval(r, point)
    e = to_E2(finals)
    assert to_E2(beta_eval)[0] == e[2]
    assert e[0] * e[1] * e[2] == to_E2(expected)[0]
    assert (m1.evaluate(point) == finals[0]).all() and (m2.evaluate(point) == finals[1]).all()
    # a tampered proof is rejected
    bad = proof.copy()
    bad[3, 0, 0] ^= np.uint64(1)
    rc, _, _ = ctx.sumcheck_verify(claim, bad, dp.Transcript())
    assert rc != 0


def test_same_poly_shape(dp, ctx, orc):
    # zkml/src/iop/same_poly.rs:84-114: poly * sum_i a_i * eq_i, challenges as coefficients
    n, k = 10, 14
    poly = rand_e2(1 << n, 5000)
    points = [rand_e2(n, 5001 + i) for i in range(k)]
    tr, otr = dp.Transcript(), orc.OracleTranscript()
    a = tr.read_challenges(k)
    assert (a == otr.read_challenges(k)).all()
    gpu = [ctx.mle_from_ext2(poly)] + [ctx.eq_build(p) for p in points]
    ref = [poly] + [orc.eq_evals(p) for p in points]
    terms = [(a[i], [0, 1 + i]) for i in range(k)]
    proof, point, finals = ctx.sumcheck_prove(n, gpu, terms, tr)
    oproof, opoint, ofinals = orc.sc_prove(n, ref, terms, otr)
    assert (proof == oproof).all() and (point == opoint).all() and (finals == ofinals).all()
    assert tr.state() == otr.state()


def test_round_by_round_session_and_errors(dp, ctx, orc):
    n = 5
    tabs = [rand_e2(1 << n, 6000 + k) for k in range(2)]
    gpu = [ctx.mle_from_ext2(t) for t in tabs]
    terms = [(ONE, [0, 1])]
    s = ctx.session(n, gpu, terms)
    with pytest.raises(dp.DpsError):
        s.round(ONE)  # round 1 takes no challenge
    msgs, chal = [], None
    otr = orc.OracleTranscript()
    oproof, opoint, ofinals = orc.sc_prove(n, tabs, terms, otr)
    for j in range(n):
        msgs.append(s.round(chal))
        chal = opoint[j]
    with pytest.raises(dp.DpsError):
        s.round(chal)  # no round n+1
    finals = s.finish(chal)
    with pytest.raises(dp.DpsError):
        s.finish(chal)
    assert (np.stack(msgs) == oproof).all() and (finals == ofinals).all()
    # the borrowed tables are untouched
    assert (gpu[0].download() == tabs[0]).all()
    # misuse is reported, not executed
    with pytest.raises(dp.DpsError):
        ctx.session(3, gpu, terms)  # tables larger than the sum
    with pytest.raises(dp.DpsError):
        ctx.session(n, gpu, [(ONE, [0, 2])])  # unknown table
    with pytest.raises(dp.DpsError):
        ctx.session(n, gpu, [(np.array([P, 0], dtype=np.uint64), [0, 1])])  # non-canonical coefficient
    with pytest.raises(dp.DpsError):
        ctx.session(n, gpu, [(ONE, [0] * 7)])  # degree above the compiled kernels


def test_resident_kernel_gives_way(dp, ctx, orc):
    # A product session of 12 variables runs its last 8 rounds in one kernel that stays on the GPU between rounds.
    # Another call on the context makes that kernel exit (through its mailbox; nothing is killed), the interrupted
    # session reports the failure, and the context keeps working.  dps_sc_abort does the same on request.
    n = 12
    f, g = rand_base(1 << n, 8100), rand_base(1 << n, 8101)
    mf, mg = ctx.mle_from_base(f), ctx.mle_from_base(g)
    terms = [(ONE, [0, 1])]
    ref_proof, ref_point, _ = orc.sc_prove(n, [orc.embed_base(f), orc.embed_base(g)], terms, orc.OracleTranscript())
    for how in ("other call", "abort"):
        s = ctx.session(n, [mf, mg], terms)
        chal = None
        for j in range(6):  # rounds 4 to 6 are already inside the resident kernel
            assert (s.round(chal) == ref_proof[j]).all()
            chal = ref_point[j]
        if how == "other call":
            assert (ctx.mle_from_base(f).download()[:, 0] == f).all()  # an upload on the same context
        else:
            s.abort()
        with pytest.raises(dp.DpsError):
            s.round(chal)
        del s
        # the context is fine: the same proof from scratch
        proof, point, _ = ctx.sumcheck_prove(n, [mf, mg], terms, dp.Transcript())
        assert (proof == ref_proof).all() and (point == ref_point).all()


@pytest.mark.parametrize("n,with_eq", [(12, False), (13, True), (9, True)])
def test_last_rounds_are_the_hosts(dp, ctx, orc, n, with_eq):
    """The resident launch leaves before the last rounds: the tables' entries come to the host with its last trip, and
    the rounds that are left (and the final evaluations) are worked out there.  From then on the session needs nothing
    of the GPU: other calls on the context, whole proofs included, between its last rounds do not disturb it."""
    f, g = rand_base(1 << n, 8200 + n), rand_e2(1 << n, 8201 + n)
    gpu, host, fs = [ctx.mle_from_base(f), ctx.mle_from_ext2(g)], [orc.embed_base(f), g], [0, 1]
    if with_eq:
        pt = rand_e2(n, 8202 + n)
        gpu.append(ctx.eq_build(pt))
        host.append(orc.eq_evals(pt))
        fs = [2, 0, 1]
    terms = [(np.array([3, 5], dtype=np.uint64), fs)]
    ref_proof, ref_point, ref_finals = orc.sc_prove(n, host, terms, orc.OracleTranscript(b"host tail"))
    for first_other in (n - 2, n - 1, n):  # rounds completed before the first other call
        s = ctx.session(n, gpu, terms)
        chal = None
        for j in range(n):
            assert (s.round(chal) == ref_proof[j]).all(), (first_other, j)
            chal = ref_point[j]
            if j + 1 >= first_other:
                proof, point, finals = ctx.sumcheck_prove(n, gpu, terms, dp.Transcript(b"host tail"))
                assert (proof == ref_proof).all() and (point == ref_point).all() and (finals == ref_finals).all()
        assert (s.finish(chal) == ref_finals).all()
        del s


def test_views_are_borrowed_halves(dp, ctx, orc):
    # SmartSlice::Borrowed halves as used by the LogUp layers (circuit.rs:260-271)
    n = 8
    tab = rand_e2(1 << n, 7000)
    m = ctx.mle_from_ext2(tab)
    lo, hi = m.view(0, n - 1), m.view(1 << (n - 1), n - 1)
    assert (lo.download() == tab[:1 << (n - 1)]).all() and (hi.download() == tab[1 << (n - 1):]).all()
    _check_prove(dp, ctx, orc, n - 1, [lo, hi], [tab[:1 << (n - 1)], tab[1 << (n - 1):]], [(ONE, [0, 1])])
    with pytest.raises(dp.DpsError):
        m.view(1, 3)  # pair loads need an even offset
    with pytest.raises(dp.DpsError):
        m.view(1 << n, 1)


def test_config3_shape_mid_size(dp, ctx, orc):
    # eq * f * g with base f, g and extension eq at a size that spans many workgroups
    n = 20
    f, g = rand_base(1 << n, 8000), rand_base(1 << n, 8001)
    r = rand_e2(n, 8002)
    gpu = [ctx.mle_from_base(f), ctx.mle_from_base(g), ctx.eq_build(r)]
    ref = [orc.embed_base(f), orc.embed_base(g), orc.eq_evals(r)]
    _check_prove(dp, ctx, orc, n, gpu, ref, [(ONE, [2, 0, 1])])


@pytest.mark.parametrize("n,kinds,zero_at", [(17, "ee", None), (18, "be", 1), (17, "e", None), (18, "b", 0), (19, "bb", 2)])
def test_large_rounds_take_eq_weights_from_two_small_tables(dp, ctx, orc, n, kinds, zero_at):
    """In rounds of at least 2^16 pairs a product with an eq factor does not stream the eq weights: they are the
    product of an entry of a 2^16-entry table (per thread) and one of a later level (per workgroup and step).
    One and two tables, base-field and extension sources, and an eq point with a zero coordinate in such a round
    (then the evaluation at 1 cannot come from the claim)."""
    tabs_gpu, tabs_ref = [], []
    for k, kind in enumerate(kinds):
        if kind == "b":
            v = rand_base(1 << n, 8100 + k)
            tabs_gpu.append(ctx.mle_from_base(v))
            tabs_ref.append(orc.embed_base(v))
        else:
            v = rand_e2(1 << n, 8100 + k)
            tabs_gpu.append(ctx.mle_from_ext2(v))
            tabs_ref.append(v)
    r = rand_e2(n, 8110)
    if zero_at is not None:
        r[zero_at] = 0
    tabs_gpu.append(ctx.eq_build(r))
    tabs_ref.append(orc.eq_evals(r))
    e = len(kinds)
    _check_prove(dp, ctx, orc, n, tabs_gpu, tabs_ref, [(np.array([7, 3], dtype=np.uint64), [e] + list(range(e)))])


@pytest.mark.parametrize("n,zero_at", [(21, None), (21, 0), (21, 1), (21, 2), (22, 3), (20, None)])
def test_first_two_rounds_in_one_launch(dp, ctx, orc, n, zero_at):
    """eq * f * g over base-field tables of 21 variables and more (with fewer, round 3 is already one of the resident
    rounds): one launch reads the tables once for rounds 1 and 2 (round 2's sums as a polynomial in round 1's challenge)
    and writes nothing, round 3 folds the tables twice on its way in.  An eq point with a zero coordinate in round 1, in
    round 2 (then the ordinary launches take the session: round 2's value at 1 cannot come from the claim), in round 3
    (which then evaluates at 1 itself) and in a later round; the same proof when the caller states the sum, and when the
    session is driven round by round with another call on the context after round 2."""
    f, g = rand_base(1 << n, 8300 + n), rand_base(1 << n, 8301 + n)
    r = rand_e2(n, 8302 + n)
    if zero_at is not None:
        r[zero_at] = 0
    gpu = [ctx.mle_from_base(f), ctx.mle_from_base(g), ctx.eq_build(r)]
    ref = [orc.embed_base(f), orc.embed_base(g), orc.eq_evals(r)]
    terms = [(np.array([5, 11], dtype=np.uint64), [0, 2, 1])]
    want = orc.sc_prove(n, ref, terms, orc.OracleTranscript(b"two"))
    got = ctx.sumcheck_prove(n, gpu, terms, dp.Transcript(b"two"))
    assert all((a == b).all() for a, b in zip(got, want))
    # the sum stated by the caller
    p1 = to_E2(want[0][0])
    again = ctx.sumcheck_prover(n, gpu, terms, claim=from_E2([p1[0] + p1[1]])[0])(dp.Transcript(b"two"))
    assert all((a == b).all() for a, b in zip(again, want))
    # round by round; after round 2 another call ends the launch made ahead for round 3, which is then launched again
    s = ctx.session(n, gpu, terms)
    chal = None
    for j in range(n):
        assert (s.round(chal) == want[0][j]).all(), j
        chal = want[1][j]
        if j == 1 and n >= 21:
            assert (ctx.eq_build(want[1][:3]).download() == orc.eq_evals(want[1][:3])).all()
    assert (s.finish(chal) == want[2]).all()


def test_prepared_prover_gives_the_same_proofs(dp, ctx, orc):
    """sumcheck_prover marshals handles and terms once; each call is the proof sumcheck_prove gives."""
    n = 11
    f, g = rand_base(1 << n, 8200), rand_e2(1 << n, 8201)
    r = rand_e2(n, 8202)
    gpu = [ctx.mle_from_base(f), ctx.mle_from_ext2(g), ctx.eq_build(r)]
    terms = [(ONE, [2, 0, 1])]
    want = ctx.sumcheck_prove(n, gpu, terms, dp.Transcript(b"p"))
    prover = ctx.sumcheck_prover(n, gpu, terms)
    for _ in range(3):
        got = prover(dp.Transcript(b"p"))
        assert all((a == b).all() for a, b in zip(got, want))


def _materialise_zero_pad(tab, n):
    out = np.zeros((1 << n, 2), dtype=np.uint64)
    out[: tab.shape[0]] = tab
    return out


ZPAD_SHAPES = [
    # (n, [(vars, zero-padded?)...], terms)
    (5, [(5, False), (3, True)], [((1, 0), [0, 1])]),
    (6, [(6, False), (0, True), (2, True)], [((3, 1), [0, 1]), ((2, 2), [0, 2]), ((5, 0), [1, 2])]),
    (7, [(4, True), (4, True), (7, False), (3, False)], [((1, 0), [0, 1]), ((9, 4), [0, 2, 3]), ((1, 1), [2])]),
    (9, [(9, True), (5, True), (1, True), (9, False)], [((1, 0), [0, 3]), ((7, 7), [1, 3]), ((2, 0), [2, 3]), ((3, 3), [1, 2])]),
    (11, [(11, False), (10, True), (8, True), (11, False), (6, True)], [((1, 0), [0, 1]), ((1, 2), [2, 3]), ((4, 0), [4, 0])]),
]


@pytest.mark.parametrize("case", range(len(ZPAD_SHAPES)))
def test_zero_padded_views_match_materialised_padding(dp, ctx, orc, case):
    # DensePolynomial::zero_pad_num_vars (zkml/src/poly_commit/prover.rs:214-226): the GPU reads the short tables in
    # place; the checker is handed the padded tables written out in full
    n, tabs_spec, terms = ZPAD_SHAPES[case]
    terms = [(np.array(c, dtype=np.uint64), f) for c, f in terms]
    tabs = [rand_e2(1 << m, 9000 + 31 * case + k) for k, (m, _) in enumerate(tabs_spec)]
    gpu, ref = [], []
    for t, (m, z) in zip(tabs, tabs_spec):
        h = ctx.mle_from_ext2(t)
        gpu.append(h.zero_pad(n) if z else h)
        ref.append(_materialise_zero_pad(t, n) if z else t)
    _, point, finals = _check_prove(dp, ctx, orc, n, gpu, ref, terms)
    # the final evaluation of a padded table is that of the short one times prod (1 - r_high)
    for k, (m, z) in enumerate(tabs_spec):
        if z:
            v = to_E2(orc.mle_evaluate(tabs[k], point[:m]))[0]
            for r in to_E2(point[m:]):
                v = v * (E2(1) - r)
            assert (finals[k] == from_E2([v])[0]).all()


def test_zero_pad_errors(dp, ctx):
    t = ctx.mle_from_ext2(rand_e2(8, 77))
    with pytest.raises(dp.DpsError):
        t.zero_pad(2)
    z = t.zero_pad(5)
    with pytest.raises(dp.DpsError):
        z.evaluate(rand_e2(3, 1))
    with pytest.raises(dp.DpsError):
        z.view(0, 2)
    one = np.array([1, 0], dtype=np.uint64)
    with pytest.raises(dp.DpsError):
        dp.Session(ctx, 6, [z], [(one, [0])])


def test_eq_tables_built_together(dp, ctx, orc):
    """dps_eq_build_many: every table equals the one built alone, including the suffix levels a sumcheck reads
    when the table is a factor of every term; sizes on both sides of the one-launch limit, the empty point"""
    ms = [0, 1, 5, 10, 16, 17, 3, 10]
    points = [rand_e2(m, 900 + i) for i, m in enumerate(ms)]
    tabs = ctx.eq_build_many(points)
    assert len(tabs) == len(ms)
    for t, p, m in zip(tabs, points, ms):
        assert t.info() == (dp.KIND_EXT2, 1 << m)
        assert (t.download() == orc.eq_evals(p)).all()
    assert ctx.eq_build_many([]) == []
    # as the common eq factor of a product (closed form over the suffix tables)
    n = 10
    f, g = rand_base(1 << n, 950), rand_base(1 << n, 951)
    one = np.array([1, 0], dtype=np.uint64)
    for k in (3, 7):
        _check_prove(dp, ctx, orc, n, [ctx.mle_from_base(f), ctx.mle_from_base(g), tabs[k]],
                     [orc.embed_base(f), orc.embed_base(g), orc.eq_evals(points[k])], [(one, [2, 0, 1])])
    # many tables: more than one launch's worth of staging is split, not refused
    many = [rand_e2(12, 2000 + i) for i in range(80)]
    got = ctx.eq_build_many(many)
    for t, p in zip(got[::13], many[::13]):
        assert (t.download() == orc.eq_evals(p)).all()
    with pytest.raises(dp.DpsError):
        ctx.eq_build_many([np.array([[dp.P, 0]], dtype=np.uint64)])
