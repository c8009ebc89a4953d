"""GPU parity for the callers of the engine: einsum partial evaluation and
proof (configurations 2 and 4), LogUp-GKR layer build and batched proof
(configuration 5), each against the CPU checker on the same seeded inputs."""
import importlib

import numpy as np
import pytest

from pyfield import E2, P
from util import from_E2, rand_base, rand_e2, rand_i64, to_E2

pytestmark = pytest.mark.gpu
C_, O_, S_ = 0, 1, 2


@pytest.fixture(scope="module")
def dp():
    return importlib.import_module("deep-prove_amd")


@pytest.fixture(scope="module")
def ctx(dp):
    c = dp.Context(0)
    yield c
    c.close()


def _pad(shape):
    return [1 << max(0, (d - 1).bit_length()) for d in shape]


def _padded(t):
    out = np.zeros(_pad(t.shape), dtype=np.int64)
    out[tuple(slice(0, d) for d in t.shape)] = t
    return out


PE_CASES = [
    # shape, kinds
    ((5, 6), [O_, C_]),            # strided column contraction
    ((6, 7), [C_, O_]),            # contiguous row contraction
    ((300, 350), [O_, C_]),        # the reference's matmul test sizes (einsum/mod.rs:700-722)
    ((350, 256), [C_, O_]),
    ((3, 4, 5), [S_, O_, C_]),     # heads stacked
    ((4, 8, 2), [O_, C_, O_]),     # two outer axes around the contraction
    ((2, 3, 4, 5), [S_, O_, C_, C_]),
    ((8, 16), [C_, C_]),           # nothing to fix: copy and pad
    ((1, 9), [O_, C_]),
    ((512, 768), [O_, C_]),        # configuration 2, X
    ((768, 3072), [C_, O_]),       # configuration 2, W
    ((8, 512, 256), [S_, O_, C_]), # configuration 4, Q / K
    ((5, 6), [O_, O_]),            # every axis fixed: Tensor::evaluate of the quantised tensor at a claim point
    ((3, 4, 5), [O_, O_, O_]),
    ((300, 350), [O_, O_]),
]


def test_int16_tensor_edges(dp, ctx, orc):
    """extreme 16-bit values embed like their int64 counterparts; odd lengths; what int16 tensors refuse"""
    v = np.array([-32768, 32767, -1, 0, 1, -12345, 777], dtype=np.int64)
    t16 = ctx.tensor_from_i16(v)
    assert t16.info() == (dp.KIND_I16, 7)
    assert (t16.download() == v).all()
    point = [rand_e2(3, 5)]
    want = orc.partial_eval(_padded(v), [8], [7], [O_], point)
    got = ctx.partial_eval(t16, [8], [7], [O_], point)
    assert (got[0].download() == want[0]).all()
    p8 = np.concatenate([v, [0]])
    assert (ctx.tensor_from_i16(p8).evaluate(point[0]) == orc.mle_evaluate(orc.embed_i64(p8), point[0])).all()
    with pytest.raises(ValueError):
        ctx.tensor_from_i16(np.array([40000]))
    with pytest.raises(dp.DpsError):
        ctx.tensor_from_i16(p8).view(0, 2)
    with pytest.raises(dp.DpsError):
        ctx.tensor_from_i16(p8).zero_pad(4)
    with pytest.raises(dp.DpsError):
        ctx.session(3, [ctx.tensor_from_i16(p8)], [((1, 0), [0])])


@pytest.mark.parametrize("shape", [(5,), (3, 5), (4, 8), (2, 3, 7), (300, 350)])
def test_padded_table_from_resident_tensor(dp, ctx, orc, shape):
    """dps_mle_from_tensor: the padded tensor's base-field table from compact or padded storage, 64- and 16-bit"""
    t = rand_i64(shape, 77)
    want = orc.embed_i64(_padded(t).reshape(-1))
    for make in (ctx.tensor_from_i64, ctx.tensor_from_i16):
        for stored in (t, _padded(t)):
            got = ctx.mle_from_tensor(make(stored), _pad(shape), list(shape))
            assert got.info() == (dp.KIND_BASE, want.shape[0])
            assert (got.download() == want).all()
    with pytest.raises(dp.DpsError):
        ctx.mle_from_tensor(ctx.tensor_from_i64(t.reshape(-1)[:-1]), _pad(shape), list(shape))
    with pytest.raises(dp.DpsError):
        ctx.mle_from_tensor(ctx.tensor_from_i64(t), [d + 1 for d in _pad(shape)], list(shape))


@pytest.mark.parametrize("case", range(len(PE_CASES)))
def test_partial_eval_matches_checker(ctx, orc, case):
    shape, kinds = PE_CASES[case]
    t = rand_i64(shape, 100 + case)
    pd = _pad(shape)
    points = [rand_e2(max(0, (p - 1).bit_length()), 200 + 10 * case + a) if k != C_ else None for a, (p, k) in enumerate(zip(pd, kinds))]
    ref = orc.partial_eval(_padded(t), pd, list(shape), kinds, points)
    dev_t = ctx.tensor_from_i64(_padded(t))
    got = ctx.partial_eval(dev_t, pd, list(shape), kinds, points)
    assert len(got) == ref.shape[0]
    for g, r in zip(got, ref):
        assert (g.download() == r).all()
    # the same tensor stored compactly (unpadded, as the model holds it): padding happens in the kernels' indexing
    got2 = ctx.partial_eval(ctx.tensor_from_i64(t), pd, list(shape), kinds, points)
    assert len(got2) == ref.shape[0]
    for g, r in zip(got2, ref):
        assert (g.download() == r).all()
    # the same values in 16-bit storage, padded and compact
    for stored in (_padded(t), t):
        t16 = ctx.tensor_from_i16(stored)
        assert (t16.download() == stored.reshape(-1)).all()
        got3 = ctx.partial_eval(t16, pd, list(shape), kinds, points)
        assert len(got3) == ref.shape[0]
        for g, r in zip(got3, ref):
            assert (g.download() == r).all()
    if all(k == O_ for k in kinds):
        # ... which is the padded tensor's multilinear extension at the point (last axis = lowest variables)
        full_point = np.concatenate([points[a] for a in reversed(range(len(shape)))])
        want = orc.mle_evaluate(orc.embed_i64(_padded(t).reshape(-1)), full_point)
        assert len(got2) == 1 and (got2[0].download()[0] == want).all()


def _oracle_einsum(orc, ops, lhs, rhs, claims, label=b"m2vec", biases=None):
    return orc.einsum_prove(ops, lhs, rhs, claims, label, biases)


def _check_einsum(dp, ctx, orc, ops, lhs, rhs, seed, biases=None):
    # output claims: the true MLE evaluations of the integer results (with the bias added where there is one)
    claims, bias_parts = [], []
    for r, op in enumerate(ops):
        out = np.einsum(f"{op[0]},{op[1]}->{op[2]}", lhs, rhs[r])
        added = np.zeros_like(out)
        if biases is not None and biases[r] is not None:
            # broadcast over the output axes the bias does not have
            added = np.broadcast_to(biases[r].reshape([out.shape[op[2].index(c)] if c in op[3] else 1 for c in op[2]]), out.shape).copy()
            assert [c for c in op[2] if c in op[3]] == list(op[3])  # (the reshape above takes the bias axes in output order)
        nvars = sum(max(0, (d - 1).bit_length()) for d in _pad(out.shape))
        pt = rand_e2(nvars, seed + r)
        ev = orc.mle_evaluate(orc.embed_i64(_padded(out + added).reshape(-1)), pt)
        claims.append((pt, ev))
        # what the verifier takes off the claim: the broadcast bias (zero in the padding) at the claim's point
        bias_parts.append(orc.mle_evaluate(orc.embed_i64(_padded(added).reshape(-1)), pt))
    tr = dp.Transcript()
    got = dp.einsum_prove(ctx, ops, lhs, rhs, claims, tr, biases)
    ref, otr = _oracle_einsum(orc, ops, lhs, rhs, claims, biases=biases)
    assert len(got["bias_claims"]) == len(ref["bias_claims"])
    for (go, gp, ge), (ro, rp, re) in zip(got["bias_claims"], ref["bias_claims"]):
        assert go == ro and (gp == rp).all() and (ge == re).all()
    assert (got["proof"] == ref["proof"]).all()
    assert (got["evaluations"] == ref["evaluations"]).all()
    if ref["aggregation_proof"] is None:
        assert got["aggregation_proof"] is None
    else:
        assert (got["aggregation_proof"] == ref["aggregation_proof"]).all()
    assert len(got["claims"]) == len(ref["claims"])
    for (gp, ge), (rp, re) in zip(got["claims"], ref["claims"]):
        assert (gp == rp).all() and (ge == re).all()
    assert tr.state() == otr.state()
    # the same proof from tensors that stay on the device, in 64-bit and in 16-bit storage, proved twice from
    # the same handles (nothing in a proof may change them)
    for bits in (64, 16):
        dl, dr = dp.Tensor(ctx, lhs, bits), [dp.Tensor(ctx, x, bits) for x in rhs]
        db = None if biases is None else [None if b is None else dp.Tensor(ctx, b, bits) for b in biases]
        for _ in range(2):
            rt = dp.Transcript()
            again = dp.einsum_prove(ctx, ops, dl, dr, claims, rt, db)
            for (go, gp, ge), (ro, rp, re) in zip(again["bias_claims"], got["bias_claims"]):
                assert go == ro and (gp == rp).all() and (ge == re).all()
            assert (again["proof"] == got["proof"]).all() and (again["evaluations"] == got["evaluations"]).all()
            assert (again["aggregation_proof"] is None) == (got["aggregation_proof"] is None)
            if got["aggregation_proof"] is not None:
                assert (again["aggregation_proof"] == got["aggregation_proof"]).all()
            for (gp, ge), (rp, re) in zip(again["claims"], got["claims"]):
                assert (gp == rp).all() and (ge == re).all()
            assert rt.state() == tr.state()
    # the proof proves the output claim: p_1(0) + p_1(1) = sum_r gamma^r claim_r
    vt = orc.OracleTranscript()
    gamma = vt.append_and_sample(b"batching_challenge")
    acc, gp = E2(0), E2(1)
    for (_, ev), part in zip(claims, bias_parts):
        acc = acc + gp * (to_E2(ev)[0] - to_E2(part)[0])
        gp = gp * to_E2(gamma)[0]
    p1 = to_E2(got["proof"][0])
    assert p1[0] + p1[1] == acc
    # every input claim is the input tensor's MLE at the claim point
    tensors = [lhs] + list(rhs)
    for (pt, ev), t in zip(got["claims"], tensors):
        assert (orc.mle_evaluate(orc.embed_i64(_padded(t).reshape(-1)), pt) == ev).all()
    return got


def test_einsum_matmul_small(dp, ctx, orc):
    _check_einsum(dp, ctx, orc, [("ik", "kj", "ij")], rand_i64((5, 6), 1), [rand_i64((6, 7), 2)], 300)


def test_einsum_matmul_reference_test_sizes(dp, ctx, orc):
    # zkml/src/layers/einsum/mod.rs:700-722: 300 x 350 x 256
    _check_einsum(dp, ctx, orc, [("ik", "kj", "ij")], rand_i64((300, 350), 3), [rand_i64((350, 256), 4)], 310)


def test_einsum_transposed_matmul_with_bias(dp, ctx, orc):
    # zkml/src/layers/einsum/mod.rs:699-722: "A(ij)@B(kj)->C(ik)+BIAS(k)", 300 x 350 times the transpose of 256 x 350
    _check_einsum(dp, ctx, orc, [("ij", "kj", "ik", "k")], rand_i64((300, 350), 21), [rand_i64((256, 350), 22)], 360,
                  biases=[rand_i64((256,), 23)])


def test_einsum_bias_on_some_outputs(dp, ctx, orc):
    # three weights against one input, a bias over both output axes on the first, over the rows on the last, none in
    # between (unpadded sizes: the padding of a broadcast bias is zero, which the statement check below relies on)
    x = rand_i64((6, 7), 24)
    ws = [rand_i64((7, 5), 25 + k) for k in range(3)]
    _check_einsum(dp, ctx, orc, [("ik", "kj", "ij", "ij"), ("ik", "kj", "ij"), ("ik", "kj", "ij", "i")], x, ws, 370,
                  biases=[rand_i64((6, 5), 28), None, rand_i64((6,), 29)])


def test_einsum_stacked(dp, ctx, orc):
    # A(ijk) @ B(ikl): i stacked
    _check_einsum(dp, ctx, orc, [("ijk", "ikl", "ijl")], rand_i64((3, 5, 6), 5), [rand_i64((3, 6, 4), 6)], 320)


def test_einsum_three_rhs_with_aggregation(dp, ctx, orc):
    # QKV-like: one LHS against three weights, then the input aggregation sumcheck (prove.rs:260-302)
    x = rand_i64((6, 8), 7)
    ws = [rand_i64((8, 5), 8 + k) for k in range(3)]
    got = _check_einsum(dp, ctx, orc, [("ik", "kj", "ij")] * 3, x, ws, 330)
    assert got["aggregation_proof"] is not None


def test_config2_gpt2_mlp_up_projection(dp, ctx, orc):
    # X [512 x 768] @ W [768 x 3072], 12-bit entries; 10-variable degree-2 sumcheck over the contraction
    X, W = rand_i64((512, 768), 11), rand_i64((768, 3072), 12)
    got = _check_einsum(dp, ctx, orc, [("ik", "kj", "ij")], X, [W], 340)
    assert got["proof"].shape == (10, 3, 2)


def test_config4_attention_scores(dp, ctx, orc):
    # 'hsd,htd->hst': Q, K [8 x 512 x 256]; 8-variable sumcheck over head_dim with the heads stacked
    Q, K = rand_i64((8, 512, 256), 13), rand_i64((8, 512, 256), 14)
    got = _check_einsum(dp, ctx, orc, [("hsd", "htd", "hst")], Q, [K], 350)
    assert got["proof"].shape == (8, 3, 2) and got["evaluations"].shape[0] == 16


def _download_layers(lg):
    out = []
    for k in range(1, lg.num_layers()):
        n, d = lg.layer(k)
        out.append((n.download(), d.download()))
    return out


@pytest.mark.parametrize("n,ncols,table", [(2, 1, False), (5, 1, False), (10, 2, False), (10, 2, True), (14, 1, True), (16, 3, False)])
def test_logup_layers_match_checker(ctx, orc, n, ncols, table):
    cols = [rand_base(1 << n, 400 + 10 * n + k) for k in range(ncols)]
    numer = rand_base(1 << n, 450 + n) if table else None
    c, beta = rand_e2(1, 460 + n)[0], rand_e2(1, 470 + n)[0]
    ref = orc.logup_build(cols, numer, c, beta)
    lg = ctx.logup_build([ctx.mle_from_base(x) for x in cols], None if numer is None else ctx.mle_from_base(numer), c, beta)
    got = _download_layers(lg)
    assert len(got) == len(ref) == n - 1
    for (gn, gd), (rn, rd) in zip(got, ref):
        assert (gn == rn).all() and (gd == rd).all()
    assert (lg.outputs() == np.concatenate(ref[-1])).all()


def test_logup_circuit_construction_identity(ctx):
    # test_circuit_construction (circuit.rs:603-624) on the GPU circuit
    col = rand_base(1 << 10, 480)
    lg = ctx.logup_build([ctx.mle_from_base(col)], None, (0, 0), (1, 0))
    o = to_E2(lg.outputs())
    expect = 0
    for v in col:
        expect = (expect - pow(int(v), P - 2, P)) % P
    assert (o[0] * o[3] + o[1] * o[2]) * (o[2] * o[3]).inv() == E2(expect)


def _logup_case(ctx, sizes, reps, ncols, table, seed):
    host, dev, meta = [], [], []
    for n in sizes:
        for rep in range(reps):
            cols = [rand_base(1 << n, seed + 100 * n + 10 * rep + k) for k in range(ncols)]
            numer = rand_base(1 << n, seed + 7 * n + rep) if table else None
            c, beta = rand_e2(1, seed + 30 + n + rep)[0], rand_e2(1, seed + 40 + n + rep)[0]
            host.append(dict(cols=cols, numer=numer, c=c, beta=beta))
            dev.append(dict(cols=[ctx.mle_from_base(x) for x in cols], numer=None if numer is None else ctx.mle_from_base(numer), c=c, beta=beta))
            meta.append((ncols, n - 1, c, beta))
    return host, dev, meta


@pytest.mark.parametrize("sizes,reps,ncols,table", [((4,), 1, 1, False), ((7, 6, 5), 2, 1, False), ((8, 6), 1, 2, True), ((11, 10, 9, 8, 7), 2, 1, False)])
def test_logup_batch_prove_matches_checker_and_verifies(dp, ctx, orc, sizes, reps, ncols, table):
    # the last case is test_logup_batch_prove (logup_gkr/mod.rs:24-79): sizes 2^7..2^11, two instances each
    host, dev, meta = _logup_case(ctx, sizes, reps, ncols, table, 500)
    tr, otr = dp.Transcript(), orc.OracleTranscript()
    got = dp.logup_batch_prove(ctx, dev, tr)
    ref = orc.logup_batch_prove(host, otr)
    assert got.shape == ref.shape and (got == ref).all()
    assert tr.state() == otr.state()
    # the host mirror's verifier accepts, the checker's verifier accepts, both return the same claims
    rc, claims, point = dp.logup_batch_verify(meta, table, got, dp.Transcript())
    orc_rc, oclaims, opoint = orc.logup_batch_verify(meta, table, got, orc.OracleTranscript())
    assert rc == 0 and orc_rc == 0
    assert (claims == oclaims).all() and (point == opoint).all()
    # output claims are the column MLEs at the final point (logup_gkr/mod.rs:70-78)
    k = 0
    for (nc, nv, _, _), ins in zip(meta, dev):
        sub = point[len(point) - (nv + 1):]
        for col in ([ins["numer"]] if table else []) + ins["cols"]:
            assert (col.evaluate(sub) == claims[k]).all()
            k += 1
    bad = got.copy()
    bad[3, 1] ^= np.uint64(1)
    rc, _, _ = dp.logup_batch_verify(meta, table, bad, dp.Transcript())
    assert rc != 0


def test_config5_lookup_argument_reduced(dp, ctx, orc):
    # configuration 5 at 2^16 lookups into a 2^10-entry table of 16-bit values (full size runs in the benchmark):
    # multiplicities are exact counts, so the two fraction sums cancel
    rng = np.random.Generator(np.random.PCG64(600))
    t_in = np.arange(1 << 10, dtype=np.uint64)
    t_out = (t_in * np.uint64(40503) + np.uint64(17)) & np.uint64(0xFFFF)
    idx = rng.integers(0, 1 << 10, size=1 << 16)
    mult = np.bincount(idx, minlength=1 << 10).astype(np.uint64)
    tr, otr = dp.Transcript(), orc.OracleTranscript()
    c, beta = tr.append_and_sample(b"c"), tr.append_and_sample(b"beta")
    otr.append_and_sample(b"c"), otr.append_and_sample(b"beta")
    look_h = [dict(cols=[t_in[idx], t_out[idx]], numer=None, c=c, beta=beta)]
    tab_h = [dict(cols=[t_in, t_out], numer=mult, c=c, beta=beta)]
    look_d = [dict(cols=[ctx.mle_from_base(x) for x in look_h[0]["cols"]], numer=None, c=c, beta=beta)]
    tab_d = [dict(cols=[ctx.mle_from_base(x) for x in tab_h[0]["cols"]], numer=ctx.mle_from_base(mult), c=c, beta=beta)]
    gl, gt = dp.logup_batch_prove(ctx, look_d, tr), dp.logup_batch_prove(ctx, tab_d, tr)
    rl, rt = orc.logup_batch_prove(look_h, otr), orc.logup_batch_prove(tab_h, otr)
    assert (gl == rl).all() and (gt == rt).all() and tr.state() == otr.state()

    def frac(stream, total):
        o = to_E2(stream[-(total + 1) - 4:-(total + 1)])
        return o[0] * o[3] + o[1] * o[2], o[2] * o[3]

    (nl, dl), (nt, dt) = frac(gl, 15), frac(gt, 9)
    assert nl * dt + nt * dl == E2(0)
