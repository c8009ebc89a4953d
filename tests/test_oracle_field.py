"""Pins the checker's field arithmetic, hash and table routines against
big-integer arithmetic, published hash vectors and definitions."""
import numpy as np
import pytest

import pyfield as pf
from pyfield import E2, P
from util import from_E2, py_rng, rand_e2, to_E2

EDGE = [0, 1, 2, 7, P - 1, P - 2, 2**32, 2**32 - 1, 2**32 + 1, 2**63, 2**63 - 1, (P - 1) // 2, (P + 1) // 2,
        0xFFFFFFFF, 0xFFFFFFFF00000000]


def test_base_field_edges_and_random(orc):
    rng = py_rng(1)
    vals = EDGE + [rng.randrange(P) for _ in range(300)]
    for a in vals[:40]:
        for b in vals[:40]:
            assert orc.gl_mul(a, b) == a * b % P
            assert orc.gl_add(a, b) == (a + b) % P
            assert orc.gl_sub(a, b) == (a - b) % P
    for a, b in zip(vals, reversed(vals)):
        assert orc.gl_mul(a, b) == a * b % P
    # (p-1)^2 = 1, 2^96 = -1, 2^64 = 2^32 - 1
    assert orc.gl_mul(P - 1, P - 1) == 1
    assert orc.lib().orc_gl_pow(2, 96) == P - 1
    assert orc.lib().orc_gl_pow(2, 64) == 2**32 - 1
    for a in vals:
        if a:
            assert orc.gl_mul(a, orc.gl_inv(a)) == 1
            assert orc.lib().orc_gl_pow(a, P - 1) == 1  # Fermat


def test_i64_embedding_roundtrip(orc):
    # negatives map to p - |x|; the inverse map recovers the integer
    for x in [0, 1, -1, 2047, -2048, 2**40, -(2**40), 2**62, -(2**62), -(2**63), 2**63 - 1]:
        f = orc.gl_from_i64(x)
        assert f == x % P
        if abs(x) < 2**62:
            assert orc.gl_to_i64(f) == x
    assert orc.gl_from_i64(-5) == P - 5


def test_ext2_against_bigint(orc):
    rng = py_rng(2)
    xs = [pf.rand_e2(rng) for _ in range(100)] + [E2(0, 0), E2(1, 0), E2(0, 1), E2(P - 1, P - 1)]
    for a, b in zip(xs, reversed(xs)):
        assert tuple(int(v) for v in orc.e2_mul(a.pair(), b.pair())) == (a * b).pair()
        assert tuple(int(v) for v in orc.e2_add(a.pair(), b.pair())) == (a + b).pair()
        assert tuple(int(v) for v in orc.e2_sub(a.pair(), b.pair())) == (a - b).pair()
    # X * X = 7
    assert tuple(int(v) for v in orc.e2_mul((0, 1), (0, 1))) == (7, 0)
    for a in xs[:50]:
        inv = orc.e2_inv(a.pair())
        assert tuple(int(v) for v in orc.e2_mul(a.pair(), inv)) == (1, 0)


def test_nonresidue_is_not_a_square():
    # X^2 - 7 is irreducible iff 7 is a non-residue: Euler's criterion
    assert pow(7, (P - 1) // 2, P) == P - 1


BLAKE3_KAT = [
    (b"", "af1349b9f5f9a1a6a0404dea36dcc9499bcb25c9adc112b7cc9a93cae41f3262"),
    (b"abc", "6437b3ac38465133ffb63b75273a8db548c558465d79db03fd359c6cd5bd9d85"),
    (bytes([0]), "2d3adedff11b61f14c886e35afa036736dcd87a74d27b5c1510225d0f592e213"),
]


def test_blake3_published_vectors(orc):
    for msg, digest in BLAKE3_KAT:
        assert orc.blake3(msg).hex() == digest


def test_eq_table_definition_and_invariants(orc):
    rng = py_rng(3)
    for m in range(0, 7):
        point = [pf.rand_e2(rng) for _ in range(m)]
        tab = to_E2(orc.eq_evals(from_E2(point)) if m else orc.eq_evals(np.zeros((0, 2), np.uint64)))
        assert len(tab) == 1 << m
        for i, v in enumerate(tab):
            assert v == pf.eq_at(point, i)
        total = E2(0)
        for v in tab:
            total = total + v
        assert total == E2(1)
    # at a boolean point the table is an indicator
    bits = [1, 0, 1, 1]
    tab = to_E2(orc.eq_evals(from_E2([E2(b) for b in bits])))
    idx = sum(b << j for j, b in enumerate(bits))
    assert [v == E2(1) for v in tab] == [i == idx for i in range(16)]


def test_identity_eval_matches_table_evaluation(orc):
    rng = py_rng(4)
    r1 = [pf.rand_e2(rng) for _ in range(5)]
    r2 = [pf.rand_e2(rng) for _ in range(5)]
    expect = pf.mle_eval([pf.eq_at(r1, i) for i in range(32)], r2)
    got = to_E2(orc.identity_eval(from_E2(r1), from_E2(r2)))[0]
    assert got == expect


def test_vector_mle_little_endian(orc):
    # evaluating at the little-endian bits of i returns v[i]
    n = 5
    v = rand_e2(1 << n, 5)
    for i in [0, 1, 6, 19, 31]:
        pt = from_E2([E2((i >> j) & 1) for j in range(n)])
        assert (orc.mle_evaluate(v, pt) == v[i]).all()


def test_mle_evaluate_definition(orc):
    rng = py_rng(6)
    n = 6
    v = rand_e2(1 << n, 6)
    point = [pf.rand_e2(rng) for _ in range(n)]
    expect = pf.mle_eval(to_E2(v), point)
    assert to_E2(orc.mle_evaluate(v, from_E2(point)))[0] == expect


def test_tensor_mle_fix_high_binds_rows(orc):
    # row-major matrix: the last dimension takes the low variables, so binding
    # the high variables to the bits of r selects row r
    rows, cols = 8, 4
    m = rand_e2(rows * cols, 7)
    for r in [0, 3, 7]:
        pt = from_E2([E2((r >> j) & 1) for j in range(3)])
        row = orc.mle_fix_high(m, pt)
        assert (row == m[r * cols:(r + 1) * cols]).all()
        for c in range(cols):
            cpt = from_E2([E2((c >> j) & 1) for j in range(2)])
            assert (orc.mle_evaluate(row, cpt) == m[r * cols + c]).all()


def test_fix_low_then_high_equals_evaluate(orc):
    rng = py_rng(8)
    n = 7
    v = rand_e2(1 << n, 8)
    point = [pf.rand_e2(rng) for _ in range(n)]
    full = orc.mle_evaluate(v, from_E2(point))
    lo = orc.mle_fix_low(v, from_E2(point[:3]))
    assert (orc.mle_evaluate(lo, from_E2(point[3:])) == full).all()
    hi = orc.mle_fix_high(v, from_E2(point[4:]))
    assert (orc.mle_evaluate(hi, from_E2(point[:4])) == full).all()
    # fix_low agrees with the definition entry by entry
    for i in range(1 << (n - 3)):
        bits = [E2((i >> j) & 1) for j in range(n - 3)]
        assert to_E2(lo[i])[0] == pf.mle_eval(to_E2(v), point[:3] + bits)
