"""CPU checks of the checker's lookup-linking sumcheck (zkml/src/lookup/operation).
What pins it without the reference's engine: the sum the proof opens with must be
what the protocol says it is -- the chunk outputs rebuilt entry by entry from the
looked-up pieces, evaluated as a multilinear extension of the WHOLE padded tensor at
the layer's claim point, plus the random linear combination of the pieces evaluated
at the LogUp point -- computed here with Python integers, without expressions,
monomials, eq tables or per-chunk coefficients."""
import numpy as np
import pytest

from linking_cases import CASES, ceil_log2, chunk_vars, chunks_of, make_instance
from pyfield import E2, P
from util import from_E2, to_E2


def _fe(x):
    return int(x) % P


def _pow(x, k):
    out = E2(1)
    for _ in range(k):
        out = out * x
    return out


def _entrywise(cfg, tabs, weight, ch):
    """Per chunk: the output entries (and their squares), the linear combination's (power, table) list."""
    nvc, nz, bits, C = cfg["value_chunks"], cfg["zero_chunks"], cfg["bit_size"], chunks_of(cfg)
    inv2 = pow(2, P - 2, P)
    out, out_sq, lin = [], [], []
    for c in range(C):
        w = [[_fe(v) for v in t] for t in tabs[c * (nvc + nz):(c + 1) * (nvc + nz)]]
        n = len(w[0])
        P_c, Psq_c = [], []
        for x in range(n):
            if nvc == 1:
                value = w[0][x]
            else:
                value = -(1 << (nvc * bits - 1)) + sum((1 << (bits * i)) * (w[i][x] + (1 << (bits - 1))) for i in range(nvc))
            z = [w[nvc + i][x] for i in range(nz)]
            if cfg["signed"]:
                if nz == 0:
                    prod, clamp, sq = 1, 0, 0
                else:
                    cmin, cmax = (cfg["min_out"], cfg["max_out"]) if nvc == 1 else (-(1 << (nvc * bits - 1)), (1 << (nvc * bits - 1)) - 1)
                    lower = 1
                    for v in z[:-1]:
                        lower = lower * v % P
                    top = z[-1]
                    keep = (1 - top * top) % P
                    prod = lower * keep % P
                    up = (top * (top + 1) * inv2 + keep * (1 - lower)) % P   # 1 when the value overflowed upwards
                    down = top * (top - 1) * inv2 % P                         # 1 when it overflowed downwards
                    clamp = (cmax * up + cmin * down) % P
                    sq = (cmax * cmax * up + cmin * cmin * down) % P
            else:
                prod = 1
                for v in z:
                    prod = prod * v % P
                clamp = (cfg["max_out"] if cfg["input_sign"] == "positive" else cfg["min_out"]) if nz else 1
                sq = 0
            P_c.append((clamp + prod * value) % P)
            Psq_c.append((sq + prod * value * value) % P)
        out.append(P_c)
        out_sq.append(Psq_c)
        lin.append([(i + 1, c * (nvc + nz) + i) for i in range(nvc + nz)])
    return out, out_sq, lin


def _mle(orc, values, point):
    arr = np.array([v % P for v in values], dtype=np.uint64)
    return to_E2(orc.mle_evaluate(orc.embed_base(arr), point))[0]


def _expected_sum(orc, cfg, tabs, weight, ch, last_claim_point, logup_point):
    shape = cfg["shape"]
    C, nv = chunks_of(cfg), chunk_vars(cfg)
    rows, cols = (1 << ceil_log2(shape[-2]) if len(shape) >= 2 else 1), 1 << ceil_log2(shape[-1])
    fd = ceil_log2(shape[-1])
    out, out_sq, lin = _entrywise(cfg, tabs, weight, ch)
    s = to_E2(ch[0])[0]
    v = cfg["variant"]
    extra0 = C * (cfg["value_chunks"] + cfg["zero_chunks"])
    # output side: what multiplies the output eq table, per chunk, placed into the whole padded tensor
    lead = shape[:max(0, len(shape) - 2)]
    lead_pad = [1 << ceil_log2(d) for d in lead]
    whole = [0] * (int(np.prod(lead_pad, dtype=np.int64)) * rows * cols if lead else rows * cols)
    for c in range(C):
        idx, rem = 0, c
        coords = []
        for d in reversed(lead):
            coords.append(rem % d)
            rem //= d
        coords.reverse()
        for a, co in enumerate(coords):
            idx = idx * lead_pad[a] + co
        vals = out[c]
        if v == "glu":
            vals = [a * _fe(b) % P for a, b in zip(vals, tabs[extra0 + c])]
        if v == "normalisation" and cfg["has_weight"]:
            vals = [a * _fe(b) % P for a, b in zip(vals, weight)]
        whole[idx * rows * cols:(idx + 1) * rows * cols] = vals
    total = _mle(orc, whole, last_claim_point)
    # per-chunk coefficients for everything else: the multilinear extension of the indicator of chunk c
    coeffs = []
    lead_point = last_claim_point[nv:]
    for c in range(C):
        ind = [0] * max(1, int(np.prod(lead_pad, dtype=np.int64)) if lead else 1)
        idx, rem, coords = 0, c, []
        for d in reversed(lead):
            coords.append(rem % d)
            rem //= d
        coords.reverse()
        for a, co in enumerate(coords):
            idx = idx * lead_pad[a] + co
        ind[idx] = 1
        coeffs.append(_mle(orc, ind, lead_point) if lead else E2(1))
    row_point = logup_point[fd:]
    for c in range(C):
        acc = E2(0)
        for power, t in lin[c]:
            acc = acc + _pow(s, power) * _mle(orc, [_fe(x) for x in tabs[t]], logup_point)
        if v in ("softmax", "normalisation"):
            nch = to_E2(ch[1 + C])[0]
            rowsum = lambda vals: [sum(vals[r * cols:(r + 1) * cols]) % P for r in range(rows)]
            if v == "softmax":
                acc = acc + nch * _mle(orc, rowsum(out[c]), row_point)
            else:
                acc = acc + nch * _mle(orc, rowsum(out_sq[c]), row_point)
                if cfg["norm_sum"]:
                    acc = acc + nch * nch * _mle(orc, rowsum(out[c]), row_point)
                inp = to_E2(ch[2 + C])[0]
                both = [_fe(a) * _fe(b) % P for a, b in zip(tabs[extra0 + c], tabs[extra0 + C + c])]
                acc = acc + inp * _mle(orc, both, logup_point)
        total = total + coeffs[c] * acc
    return total


def _tables(orc, tabs, weight):
    return [orc.embed_i64(t) for t in tabs], (None if weight is None else orc.embed_i64(weight))


@pytest.mark.parametrize("case", range(len(CASES)))
def test_linking_sum_is_the_protocols_statement(orc, case):
    cfg = CASES[case]
    tabs, weight, lcp, lp = make_instance(cfg, 50 + case)
    mles, w = _tables(orc, tabs, weight)
    tr = orc.OracleTranscript(b"linking")
    proof, point, evals, weight_eval, ch = orc.linking_prove(cfg, mles, tr, lcp, lp, w)
    assert proof.shape[0] == chunk_vars(cfg) and evals.shape[0] == len(tabs)
    assert len(ch) == 1 + chunks_of(cfg) + {"standard": 0, "glu": 0, "softmax": 1, "normalisation": 2}[cfg["variant"]]
    opened = to_E2(proof[0][0])[0] + to_E2(proof[0][1])[0] if chunk_vars(cfg) else None
    want = _expected_sum(orc, cfg, tabs, weight, ch, lcp, lp)
    if opened is not None:
        assert opened == want
    # the evaluations handed on are the tables' at the sumcheck point
    for t, e in zip(mles, evals):
        assert (orc.mle_evaluate(t, point) == e).all()
    if w is not None:
        assert (orc.mle_evaluate(w, point) == weight_eval).all()
    else:
        assert weight_eval is None
    # and the verifier accepts from that sum on, ending in the same transcript state
    vt = orc.OracleTranscript(b"linking")
    ok, vpoint, vch = orc.linking_verify(cfg, from_E2([want])[0], proof, evals, weight_eval, vt, lcp, lp)
    assert ok and (vpoint == point).all() and vt.state() == tr.state()
    assert all((a == b).all() for a, b in zip(ch, vch))


def test_linking_verifier_rejects(orc):
    cfg = CASES[1]
    tabs, weight, lcp, lp = make_instance(cfg, 99)
    mles, w = _tables(orc, tabs, weight)
    proof, point, evals, weight_eval, ch = orc.linking_prove(cfg, mles, orc.OracleTranscript(b"linking"), lcp, lp, w)
    claim = orc.e2_add(proof[0][0], proof[0][1])
    fresh = lambda: orc.OracleTranscript(b"linking")
    assert orc.linking_verify(cfg, claim, proof, evals, weight_eval, fresh(), lcp, lp)[0]
    assert not orc.linking_verify(cfg, orc.e2_add(claim, orc.e2(1)), proof, evals, weight_eval, fresh(), lcp, lp)[0]
    bad = evals.copy()
    bad[2, 0] ^= np.uint64(1)
    assert not orc.linking_verify(cfg, claim, proof, bad, weight_eval, fresh(), lcp, lp)[0]
    badp = proof.copy()
    badp[1, 2, 1] ^= np.uint64(4)
    assert not orc.linking_verify(cfg, claim, badp, evals, weight_eval, fresh(), lcp, lp)[0]
    lp2 = lp.copy()
    lp2[0, 0] ^= np.uint64(1)
    assert not orc.linking_verify(cfg, claim, proof, evals, weight_eval, fresh(), lcp, lp2)[0]
    assert not orc.linking_verify(cfg, claim, proof, evals, weight_eval, orc.OracleTranscript(b"other"), lcp, lp)[0]
