#!/usr/bin/env python3
"""Writes the fixtures in this directory.  Run from the repository root:

    python tests/golden/make_golden.py

field_vectors.json comes from Python's big integers alone (tests/pyfield.py);
protocol_vectors.json from the CPU checker under oracle/, whose functions are
pinned by the definition-level tests in tests/test_oracle_*.py.  No file of the
reference is read or run: its engine crate is not in the reference checkout, and
it holds no vectors for this path.  The fixtures freeze today's bits so that the
checker, the host mirror and the GPU library cannot drift together unnoticed.
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
for p in (os.path.join(ROOT, "tests"), os.path.join(ROOT, "oracle")):
    sys.path.insert(0, p)

from pyfield import E2, P  # noqa: E402
from util import SplitMix64, rand_base, rand_e2, rand_i64  # noqa: E402


def hx(a):
    return [format(int(x), "016x") for x in np.asarray(a, dtype=np.uint64).reshape(-1)]


def st(t):
    state, rounds = t.state()
    return dict(state=state.hex(), absorbed=rounds)


def field_vectors():
    g = SplitMix64(2024)
    edge = [0, 1, 2, 7, P - 1, P - 2, 2**32, 2**32 - 1, 2**32 + 1, 2**63, P - 2**32, 2**64 - 2**32]
    edge = [e % P for e in edge]
    vals = edge + [g.field() for _ in range(20)]
    base = []
    for i, a in enumerate(vals):
        b = vals[(7 * i + 3) % len(vals)]
        base.append(dict(a=format(a, "016x"), b=format(b, "016x"), add=format((a + b) % P, "016x"), sub=format((a - b) % P, "016x"),
                         mul=format(a * b % P, "016x"), inv=format(pow(a, P - 2, P), "016x")))
    ext = []
    for i in range(24):
        x = E2(vals[i % len(vals)], vals[(5 * i + 1) % len(vals)])
        y = E2(vals[(3 * i + 2) % len(vals)], vals[(11 * i + 4) % len(vals)])
        m, s = x * y, x + y
        inv = x.inv() if x != E2(0) else E2(0)
        ext.append(dict(x=[format(x.a, "016x"), format(x.b, "016x")], y=[format(y.a, "016x"), format(y.b, "016x")],
                        mul=[format(m.a, "016x"), format(m.b, "016x")], add=[format(s.a, "016x"), format(s.b, "016x")],
                        inv=[format(inv.a, "016x"), format(inv.b, "016x")]))
    emb = [dict(x=v, f=format(v % P, "016x")) for v in [0, 1, -1, 2047, -2048, 2**62, -(2**62), -(2**63)]]
    return dict(p=format(P, "016x"), nonresidue=7, base=base, ext=ext, i64_embedding=emb)


def protocol_vectors():
    import dpsc_oracle as orc

    orc.build()
    out = {}
    out["blake3"] = {"": orc.blake3(b"").hex(), "abc": orc.blake3(b"abc").hex(), "00": orc.blake3(b"\x00").hex(),
                     "1025 bytes i%251": orc.blake3(bytes(i % 251 for i in range(1025))).hex()}
    tr = orc.OracleTranscript(b"golden")
    tr.append_u64(5)
    tr.append_scalars(rand_e2(3, 1))
    c1 = tr.challenge_scalar()
    c2 = tr.append_and_sample(b"label")
    out["transcript"] = dict(label="golden", ops="append_u64(5); append_scalars(rand_e2(3,1)); challenge; append_and_sample('label')",
                             challenges=hx(np.stack([c1, c2])), state=st(tr))
    pt = rand_e2(4, 2)
    out["eq_evals"] = dict(point=hx(pt), table=hx(orc.eq_evals(pt)))
    # degree-3 product with an eq table, n = 5 (the benchmark's shape in small)
    n = 5
    f, g, r = rand_base(1 << n, 3), rand_base(1 << n, 4), rand_e2(n, 5)
    one = np.array([1, 0], dtype=np.uint64)
    t = orc.OracleTranscript(b"golden")
    proof, point, finals = orc.sc_prove(n, [orc.embed_base(f), orc.embed_base(g), orc.eq_evals(r)], [(one, [2, 0, 1])], t)
    out["sumcheck_eq_f_g"] = dict(n=n, f_seed=3, g_seed=4, r_seed=5, proof=hx(proof), point=hx(point), finals=hx(finals), state=st(t))
    # several terms, tables with fewer variables, a constant
    n = 6
    tabs = [rand_e2(1 << m, 10 + k) for k, m in enumerate([6, 6, 3, 0])]
    terms = [(np.array([3, 1], np.uint64), [0, 1]), (np.array([2, 2], np.uint64), [0, 2, 3]), (np.array([9, 9], np.uint64), [])]
    t = orc.OracleTranscript(b"golden")
    proof, point, finals = orc.sc_prove(n, tabs, terms, t)
    out["sumcheck_mixed"] = dict(n=n, table_vars=[6, 6, 3, 0], seeds=[10, 11, 12, 13], terms=[[[3, 1], [0, 1]], [[2, 2], [0, 2, 3]], [[9, 9], []]],
                                 proof=hx(proof), point=hx(point), finals=hx(finals), state=st(t))
    # partial evaluation of a small stacked tensor
    shape, kinds = (3, 4, 5), [2, 1, 0]
    ten = rand_i64(shape, 20)
    pd = [4, 4, 8]
    padded = np.zeros(pd, dtype=np.int64)
    padded[:3, :4, :5] = ten
    pts = [None, rand_e2(2, 21), None]
    out["partial_eval"] = dict(shape=list(shape), kinds=kinds, tensor_seed=20, point_seed=21, tables=hx(orc.partial_eval(padded, pd, list(shape), kinds, pts)))
    # LogUp: a 2-column lookup instance of 2^5 rows
    cols = [rand_base(32, 30), rand_base(32, 31)]
    c, beta = rand_e2(1, 32)[0], rand_e2(1, 33)[0]
    t = orc.OracleTranscript(b"golden")
    stream = orc.logup_batch_prove([dict(cols=cols, numer=None, c=c, beta=beta)], t)
    out["logup_lookup"] = dict(col_seeds=[30, 31], c_seed=32, beta_seed=33, stream=hx(stream), state=st(t))
    # claims batching and same_poly
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    from opening_cases import make_instance

    polys, claims, shapes = make_instance(orc, 5, 4, small=True)
    t = orc.OracleTranscript(b"golden")
    proof, point, evals = orc.claims_batching_prove(polys, claims, t)
    out["claims_batching"] = dict(instance="opening_cases.make_instance(orc, 5, 4, small=True)", proof=hx(proof), point=hx(point), evals=hx(evals),
                                  state=st(t))
    poly = rand_e2(1 << 6, 40)
    cl = [(rand_e2(6, 41 + i), None) for i in range(3)]
    cl = [(p_, orc.mle_evaluate(poly, p_)) for p_, _ in cl]
    t = orc.OracleTranscript(b"golden")
    proof, point, ev = orc.same_poly_prove(poly, cl, t)
    out["same_poly"] = dict(poly_seed=40, point_seeds=[41, 42, 43], proof=hx(proof), point=hx(point), eval=hx(ev), state=st(t))
    # the lookup-linking sumcheck: a signed table with one zeroing chunk (3 chunks), and the weighted normalisation variant
    from linking_cases import CASES, make_instance as linking_instance

    out["linking"] = []
    for case, seed in ((1, 60), (9, 61)):
        tabs, weight, lcp, lp = linking_instance(CASES[case], seed)
        t = orc.OracleTranscript(b"golden")
        proof, point, evals, weight_eval, ch = orc.linking_prove(CASES[case], [orc.embed_i64(x) for x in tabs], t, lcp, lp,
                                                                 None if weight is None else orc.embed_i64(weight))
        out["linking"].append(dict(instance=f"linking_cases.make_instance(CASES[{case}], {seed})", case=case, seed=seed, proof=hx(proof), point=hx(point),
                                   evals=hx(evals), weight_eval=None if weight_eval is None else hx(weight_eval), challenges=hx(np.stack(ch)),
                                   state=st(t)))
    return out


if __name__ == "__main__":
    with open(os.path.join(HERE, "field_vectors.json"), "w") as fh:
        json.dump(field_vectors(), fh, indent=1)
    with open(os.path.join(HERE, "protocol_vectors.json"), "w") as fh:
        json.dump(protocol_vectors(), fh, indent=1)
    print("wrote", os.listdir(HERE))
