"""Pins the checker's einsum partial evaluation and LogUp-GKR restatements
against closed forms (plain integer matrix products, sums of fractions) and
their prover/verifier round trips."""
import numpy as np
import pytest

import pyfield as pf
from pyfield import E2, P
from util import from_E2, py_rng, rand_base, rand_e2, rand_i64, to_E2

C_, O_, S_ = 0, 1, 2  # contracted, outer, stacked


def _pad(shape):
    return [1 << max(0, (d - 1).bit_length()) for d in shape]


def _padded(t):
    out = np.zeros(_pad(t.shape), dtype=np.int64)
    out[tuple(slice(0, d) for d in t.shape)] = t
    return out


def test_partial_eval_is_matrix_vector_product(orc):
    # A(ik): fixing the outer axis i at r gives sum_i eq(r, i) A[i, k]   (non power-of-two sizes)
    m, k = 5, 6
    A = rand_i64((m, k), 1)
    r = rand_e2(3, 2)
    got = orc.partial_eval(_padded(A), _pad(A.shape), list(A.shape), [O_, C_], [r, None])
    assert got.shape == (1, 8, 2)
    eq = to_E2(orc.eq_evals(r))
    for col in range(8):
        expect = E2(0)
        if col < k:
            for i in range(m):
                expect = expect + eq[i] * int(A[i, col])
        assert to_E2(got[0, col])[0] == expect
    # W(kj): fixing the trailing outer axis j
    W = rand_i64((k, 7), 3)
    rj = rand_e2(3, 4)
    got = orc.partial_eval(_padded(W), _pad(W.shape), list(W.shape), [C_, O_], [None, rj])
    eqj = to_E2(orc.eq_evals(rj))
    for row in range(8):
        expect = E2(0)
        if row < k:
            for j in range(7):
                expect = expect + eqj[j] * int(W[row, j])
        assert to_E2(got[0, row])[0] == expect


def test_partial_eval_matches_full_mle_at_reconstructed_point(orc):
    # MLE_fixed(s) == MLE_full(point with the fixed coordinates put back) (einsum/prove.rs:337-361)
    A = rand_i64((4, 8, 2), 5)  # power-of-two so the padded tensor is the tensor
    r0, r2 = rand_e2(2, 6), rand_e2(1, 7)
    fixed = orc.partial_eval(A, list(A.shape), list(A.shape), [O_, C_, O_], [r0, None, r2])[0]
    s = rand_e2(3, 8)
    full = orc.embed_i64(A.reshape(-1))
    # last dimension lowest: point = (axis2 vars, axis1 vars, axis0 vars)
    point = np.concatenate([r2, s, r0])
    assert (orc.mle_evaluate(fixed, s) == orc.mle_evaluate(full, point)).all()


def test_stacked_axes_split_and_coefficients(orc):
    # Q(hqd): h stacked, q outer, d contracted -> one table per head
    Q = rand_i64((3, 4, 5), 9)
    rh, rq = rand_e2(2, 10), rand_e2(2, 11)
    tabs = orc.partial_eval(_padded(Q), _pad(Q.shape), list(Q.shape), [S_, O_, C_], [rh, rq, None])
    assert tabs.shape == (3, 8, 2)
    eq = to_E2(orc.eq_evals(rq))
    for h in range(3):
        for d in range(5):
            expect = E2(0)
            for q in range(4):
                expect = expect + eq[q] * int(Q[h, q, d])
            assert to_E2(tabs[h, d])[0] == expect
    coeffs = orc.stacking_coeffs(_pad(Q.shape), list(Q.shape), [S_, O_, C_], [rh, rq, None])
    assert (coeffs == orc.eq_evals(rh)[:3]).all()


def test_matmul_claim_identity(orc):
    # sum_k A(r_i, k) B(k, r_j) == C(r_i, r_j) with C = A @ B over the integers
    A, B = rand_i64((4, 6), 12), rand_i64((6, 8), 13)
    Cm = A @ B
    ri, rj = rand_e2(2, 14), rand_e2(3, 15)
    a = orc.partial_eval(_padded(A), _pad(A.shape), list(A.shape), [O_, C_], [ri, None])[0]
    b = orc.partial_eval(_padded(B), _pad(B.shape), list(B.shape), [C_, O_], [None, rj])[0]
    lhs = E2(0)
    for x, y in zip(to_E2(a), to_E2(b)):
        lhs = lhs + x * y
    claim = orc.mle_evaluate(orc.embed_i64(Cm.reshape(-1)), np.concatenate([rj, ri]))
    assert to_E2(claim)[0] == lhs


def test_logup_circuit_construction(orc):
    # test_circuit_construction (circuit.rs:603-624): sum_i -1/v_i == N/D at the root
    col = rand_base(1 << 10, 20)
    layers = orc.logup_build([col], None, (0, 0), (1, 0))
    n, d = layers[-1]
    assert n.shape[0] == 2
    out = to_E2(np.concatenate([n, d]))
    num = out[0] * out[3] + out[1] * out[2]
    den = out[2] * out[3]
    expect = 0
    for v in col:
        expect = (expect - pow(int(v), P - 2, P)) % P
    assert num * den.inv() == E2(expect)


def test_logup_table_balances_lookups(orc):
    # sum_i m_i/(c + t_i) - sum_j 1/(c + l_j) == 0 when the multiplicities are exact counts
    table = np.arange(16, dtype=np.uint64) * np.uint64(3) + np.uint64(1)
    rng = np.random.Generator(np.random.PCG64(21))
    idx = rng.integers(0, 16, size=64)
    lookups = table[idx]
    mult = np.bincount(idx, minlength=16).astype(np.uint64)
    c, beta = rand_e2(1, 22)[0], rand_e2(1, 23)[0]
    lt = orc.logup_build([table], mult, c, beta)[-1]
    ll = orc.logup_build([lookups], None, c, beta)[-1]

    def frac(layer):
        o = to_E2(np.concatenate(layer))
        return o[0] * o[3] + o[1] * o[2], o[2] * o[3]

    (nt, dt), (nl, dl) = frac(lt), frac(ll)
    assert nt * dl + nl * dt == E2(0)


@pytest.mark.parametrize("is_table", [False, True])
def test_logup_batch_prove_verify_roundtrip(orc, is_table):
    # test_logup_batch_prove (logup_gkr/mod.rs:24-79): several sizes, two instances each,
    # verifier accepts and the output claims are the column MLEs at the final point
    instances, meta, columns = [], [], []
    for n in (7, 6, 5):
        for rep in range(2):
            ncols = 1 if not is_table else 2
            cols = [rand_base(1 << n, 100 * n + 10 * rep + k) for k in range(ncols)]
            c, beta = rand_e2(1, 30 + n + rep)[0], rand_e2(1, 40 + n + rep)[0]
            numer = rand_base(1 << n, 7 * n + rep) if is_table else None
            instances.append(dict(cols=cols, numer=numer, c=c, beta=beta))
            meta.append((ncols, n - 1, c, beta))
            columns += ([numer] if is_table else []) + cols
    stream = orc.logup_batch_prove(instances, orc.OracleTranscript())
    vtr = orc.OracleTranscript()
    rc, claims, point = orc.logup_batch_verify(meta, is_table, stream, vtr)
    assert rc == 0
    k = 0
    for (ncols, nv, _, _), ins in zip(meta, instances):
        sub = point[len(point) - (nv + 1):]
        for col in ([ins["numer"]] if is_table else []) + ins["cols"]:
            assert (orc.mle_evaluate(orc.embed_base(col), sub) == claims[k]).all()
            k += 1
    # the prover's own claim evaluations sit in the stream and agree
    total = 6
    pos = sum(v * 4 for v in range(1, total + 1))
    # a flipped round evaluation is rejected
    bad = stream.copy()
    bad[5, 0] ^= np.uint64(1)
    rc, _, _ = orc.logup_batch_verify(meta, is_table, bad, orc.OracleTranscript())
    assert rc != 0


def test_logup_smaller_instances_roll_in(orc):
    # a single-size batch and a mixed batch both verify; fewer-variable tables depend on the last variables
    cols = rand_base(1 << 4, 50)
    c, beta = rand_e2(1, 51)[0], rand_e2(1, 52)[0]
    stream = orc.logup_batch_prove([dict(cols=[cols], numer=None, c=c, beta=beta)], orc.OracleTranscript())
    rc, claims, point = orc.logup_batch_verify([(1, 3, c, beta)], False, stream, orc.OracleTranscript())
    assert rc == 0 and (orc.mle_evaluate(orc.embed_base(cols), point) == claims[0]).all()
