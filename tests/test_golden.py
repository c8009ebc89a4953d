"""The committed fixtures under tests/golden/ against the checker (CPU) and the
GPU library.  field_vectors.json was written from Python big integers alone;
protocol_vectors.json freezes the checker's output (see golden/make_golden.py)."""
import importlib
import importlib.util
import json
import os

import numpy as np
import pytest

from util import rand_base, rand_e2, rand_i64

HERE = os.path.dirname(os.path.abspath(__file__))


def _load(name):
    with open(os.path.join(HERE, "golden", name)) as fh:
        return json.load(fh)


def _u(hexes, shape=None):
    a = np.array([int(h, 16) for h in hexes], dtype=np.uint64)
    return a if shape is None else a.reshape(shape)


def test_checker_matches_field_vectors(orc):
    fv = _load("field_vectors.json")
    for row in fv["base"]:
        a, b = int(row["a"], 16), int(row["b"], 16)
        assert orc.gl_add(a, b) == int(row["add"], 16) and orc.gl_sub(a, b) == int(row["sub"], 16)
        assert orc.gl_mul(a, b) == int(row["mul"], 16)
        if a:
            assert orc.gl_inv(a) == int(row["inv"], 16)
    for row in fv["ext"]:
        x, y = _u(row["x"]), _u(row["y"])
        assert (orc.e2_mul(x, y) == _u(row["mul"])).all() and (orc.e2_add(x, y) == _u(row["add"])).all()
        if x.any():
            assert (orc.e2_inv(x) == _u(row["inv"])).all()
    for row in fv["i64_embedding"]:
        assert orc.gl_from_i64(row["x"]) == int(row["f"], 16)


def test_checker_reproduces_protocol_vectors(orc):
    spec = importlib.util.spec_from_file_location("make_golden", os.path.join(HERE, "golden", "make_golden.py"))
    mg = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mg)
    assert json.loads(json.dumps(mg.protocol_vectors())) == _load("protocol_vectors.json")
    assert json.loads(json.dumps(mg.field_vectors())) == _load("field_vectors.json")


@pytest.fixture(scope="module")
def dp():
    return importlib.import_module("deep-prove_amd")


@pytest.fixture(scope="module")
def ctx(dp):
    c = dp.Context(0)
    yield c
    c.close()


@pytest.mark.gpu
def test_gpu_matches_field_vectors(ctx):
    fv = _load("field_vectors.json")
    x = np.array([[int(r["x"][0], 16), int(r["x"][1], 16)] for r in fv["ext"]], dtype=np.uint64)
    y = np.array([[int(r["y"][0], 16), int(r["y"][1], 16)] for r in fv["ext"]], dtype=np.uint64)
    mul = np.array([[int(r["mul"][0], 16), int(r["mul"][1], 16)] for r in fv["ext"]], dtype=np.uint64)
    add = np.array([[int(r["add"][0], 16), int(r["add"][1], 16)] for r in fv["ext"]], dtype=np.uint64)
    assert (ctx.field_op(2, x, y) == mul).all() and (ctx.field_op(0, x, y) == add).all()
    a = np.array([[int(r["a"], 16), int(r["b"], 16)] for r in fv["base"]], dtype=np.uint64)
    b = np.array([[int(r["b"], 16), int(r["a"], 16)] for r in fv["base"]], dtype=np.uint64)
    want = np.array([[int(r["mul"], 16)] * 2 for r in fv["base"]], dtype=np.uint64)
    assert (ctx.field_op(3, a, b) == want).all()  # two independent base products per row


@pytest.mark.gpu
def test_gpu_matches_protocol_vectors(dp, ctx, orc):
    pv = _load("protocol_vectors.json")
    assert dp.blake3(b"abc").hex() == pv["blake3"]["abc"]
    assert dp.blake3(bytes(i % 251 for i in range(1025))).hex() == pv["blake3"]["1025 bytes i%251"]
    tr = dp.Transcript(b"golden")
    tr.append_u64(5)
    tr.append_scalars(rand_e2(3, 1))
    c1 = tr.challenge_scalar()
    c2 = tr.append_and_sample(b"label")
    assert (np.stack([c1, c2]).reshape(-1) == _u(pv["transcript"]["challenges"])).all()
    assert tr.state()[0].hex() == pv["transcript"]["state"]["state"]
    e = pv["eq_evals"]
    assert (ctx.eq_build(_u(e["point"], (-1, 2))).download().reshape(-1) == _u(e["table"])).all()

    one = np.array([1, 0], dtype=np.uint64)
    g = pv["sumcheck_eq_f_g"]
    n = g["n"]
    f, gg, r = rand_base(1 << n, 3), rand_base(1 << n, 4), rand_e2(n, 5)
    t = dp.Transcript(b"golden")
    proof, point, finals = ctx.sumcheck_prove(n, [ctx.mle_from_base(f), ctx.mle_from_base(gg), ctx.eq_build(r)], [(one, [2, 0, 1])], t)
    assert (proof.reshape(-1) == _u(g["proof"])).all() and (point.reshape(-1) == _u(g["point"])).all()
    assert (finals.reshape(-1) == _u(g["finals"])).all() and t.state()[0].hex() == g["state"]["state"]

    m = pv["sumcheck_mixed"]
    tabs = [ctx.mle_from_ext2(rand_e2(1 << v, s)) for v, s in zip(m["table_vars"], m["seeds"])]
    terms = [(np.array(c, dtype=np.uint64), fs) for c, fs in m["terms"]]
    t = dp.Transcript(b"golden")
    proof, point, finals = ctx.sumcheck_prove(m["n"], tabs, terms, t)
    assert (proof.reshape(-1) == _u(m["proof"])).all() and (finals.reshape(-1) == _u(m["finals"])).all()
    assert t.state()[0].hex() == m["state"]["state"]

    pe = pv["partial_eval"]
    ten = rand_i64(tuple(pe["shape"]), pe["tensor_seed"])
    got = ctx.partial_eval(ctx.tensor_from_i64(ten), [4, 4, 8], pe["shape"], pe["kinds"], [None, rand_e2(2, pe["point_seed"]), None])
    assert (np.concatenate([x.download().reshape(-1) for x in got]) == _u(pe["tables"])).all()

    lg = pv["logup_lookup"]
    cols = [ctx.mle_from_base(rand_base(32, s)) for s in lg["col_seeds"]]
    t = dp.Transcript(b"golden")
    stream = dp.logup_batch_prove(ctx, [dict(cols=cols, numer=None, c=rand_e2(1, lg["c_seed"])[0], beta=rand_e2(1, lg["beta_seed"])[0])], t)
    assert (stream.reshape(-1) == _u(lg["stream"])).all() and t.state()[0].hex() == lg["state"]["state"]

    from opening_cases import make_instance

    cb = pv["claims_batching"]
    polys, claims, _ = make_instance(orc, 5, 4, small=True)
    t = dp.Transcript(b"golden")
    proof, point, evals = dp.claims_batching_prove(ctx, [[ctx.mle_from_ext2(c) for c in chunks] for chunks in polys], claims, t)
    assert (proof.reshape(-1) == _u(cb["proof"])).all() and (evals.reshape(-1) == _u(cb["evals"])).all()
    assert t.state()[0].hex() == cb["state"]["state"]

    sp = pv["same_poly"]
    poly = rand_e2(1 << 6, sp["poly_seed"])
    cl = [(p_, orc.mle_evaluate(poly, p_)) for p_ in (rand_e2(6, s) for s in sp["point_seeds"])]
    t = dp.Transcript(b"golden")
    proof, point, ev = dp.same_poly_prove(ctx, ctx.mle_from_ext2(poly), cl, t)
    assert (proof.reshape(-1) == _u(sp["proof"])).all() and (ev == _u(sp["eval"])).all() and t.state()[0].hex() == sp["state"]["state"]

    from linking_cases import CASES, chunk_vars, make_instance as linking_instance

    for lk in pv["linking"]:
        cfg = CASES[lk["case"]]
        tabs, weight, lcp, lp = linking_instance(cfg, lk["seed"])
        nv = chunk_vars(cfg)
        t = dp.Transcript(b"golden")
        proof, point, evals, weight_eval, ch = dp.linking_prove(ctx, cfg, [ctx.mle_from_i64(x, nv) for x in tabs], t, lcp, lp,
                                                                None if weight is None else ctx.mle_from_i64(weight, nv))
        assert (proof.reshape(-1) == _u(lk["proof"])).all() and (evals.reshape(-1) == _u(lk["evals"])).all()
        assert (ch.reshape(-1) == _u(lk["challenges"])).all() and t.state()[0].hex() == lk["state"]["state"]
        assert (weight_eval is None) == (lk["weight_eval"] is None)
        if weight_eval is not None:
            assert (weight_eval == _u(lk["weight_eval"])).all()
