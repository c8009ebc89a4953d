"""GPU parity at the benchmark's full sizes and in the corners of the C ABI that the smaller cases do not reach:
configuration 3 at n = 24, configuration 5 at 2^22 lookups into a 2^16-entry table, tables in device memory the
caller owns (dps_mle_wrap_device), and two contexts driven from two threads at once."""
import importlib
import threading

import numpy as np
import pytest

from pyfield import E2
from util import rand_base, rand_e2, to_E2

pytestmark = pytest.mark.gpu

ONE = np.array([1, 0], dtype=np.uint64)


@pytest.fixture(scope="module")
def dp():
    return importlib.import_module("deep-prove_amd")


@pytest.fixture(scope="module")
def ctx(dp):
    c = dp.Context(0)
    yield c
    c.close()


def test_config3_full_size(dp, ctx, orc):
    """eq(r, x) * f(x) * g(x) at n = 24 (zkml/src/layers/hadamard.rs:93-131 at the benchmark's size): the 768-workgroup
    grid, the eq weights taken from two small tables in rounds 1..8, the challenge relayed through device memory to the
    large launches made ahead, and the resident last rounds, all in one proof.  Messages, point, final evaluations and
    transcript state against the CPU checker."""
    n = 24
    f, g = rand_base(1 << n, 24001), rand_base(1 << n, 24002)
    r = rand_e2(n, 24003)
    gpu = [ctx.mle_from_base(f), ctx.mle_from_base(g), ctx.eq_build(r)]
    ref = [orc.embed_base(f), orc.embed_base(g), orc.eq_evals(r)]
    terms = [(ONE, [2, 0, 1])]
    tr, otr = dp.Transcript(b"cfg3"), orc.OracleTranscript(b"cfg3")
    proof, point, finals = ctx.sumcheck_prove(n, gpu, terms, tr)
    oproof, opoint, ofinals = orc.sc_prove(n, ref, terms, otr)
    assert (proof == oproof).all()
    assert (point == opoint).all() and (finals == ofinals).all()
    assert tr.state() == otr.state()
    # a second proof over the same handles (the eq table's low tables are now there from the start): same bits
    proof2, _, finals2 = ctx.sumcheck_prove(n, gpu, terms, dp.Transcript(b"cfg3"))
    assert (proof2 == oproof).all() and (finals2 == ofinals).all()
    # the caller states the sum (hadamard.rs:117-121 knows it): round 1 then takes p(1) from it, same messages
    s = dp.Session(ctx, n, gpu, terms)
    p1 = to_E2(oproof[0])
    claim = p1[0] + p1[1]
    s.set_claim(np.array([claim.a, claim.b], dtype=np.uint64))
    chal = None
    for j in range(n):
        assert (s.round(chal) == oproof[j]).all(), "round %d" % (j + 1)
        chal = opoint[j]
    assert (s.finish(chal) == ofinals).all()


def test_config5_full_size(dp, ctx, orc):
    """configuration 5 as the benchmark runs it: 2^22 lookups (two columns) into a 2^16-entry table with exact
    multiplicities (zkml/src/lookup/logup_gkr/prover.rs:91-344).  The bottom layers' sumchecks have rounds of more than
    2^16 pairs, which only this size sends through the large multi-term kernel and its nested program."""
    log_l, log_t = 22, 16
    rng = np.random.Generator(np.random.PCG64(600))
    t_in = np.arange(1 << log_t, dtype=np.uint64)
    t_out = (t_in * np.uint64(40503) + np.uint64(17)) & np.uint64(0xFFFF)
    idx = rng.integers(0, 1 << log_t, size=1 << log_l)
    mult = np.bincount(idx, minlength=1 << log_t).astype(np.uint64)
    tr, otr = dp.Transcript(b"cfg5"), orc.OracleTranscript(b"cfg5")
    c, beta = tr.append_and_sample(b"c"), tr.append_and_sample(b"beta")
    otr.append_and_sample(b"c"), otr.append_and_sample(b"beta")
    look_cols = [t_in[idx], t_out[idx]]
    look_h = [dict(cols=look_cols, numer=None, c=c, beta=beta)]
    tab_h = [dict(cols=[t_in, t_out], numer=mult, c=c, beta=beta)]
    look_d = [dict(cols=[ctx.mle_from_base(x) for x in look_cols], numer=None, c=c, beta=beta)]
    tab_d = [dict(cols=[ctx.mle_from_base(t_in), ctx.mle_from_base(t_out)], numer=ctx.mle_from_base(mult), c=c, beta=beta)]
    gl, gt = dp.logup_batch_prove(ctx, look_d, tr), dp.logup_batch_prove(ctx, tab_d, tr)
    rl, rt = orc.logup_batch_prove(look_h, otr), orc.logup_batch_prove(tab_h, otr)
    assert gl.shape == rl.shape and (gl == rl).all()
    assert gt.shape == rt.shape and (gt == rt).all()
    assert tr.state() == otr.state()

    # the two fraction sums cancel (exact multiplicities): sum_j -1/(c + l_j) + sum_i m_i/(c + t_i) = 0
    def frac(stream, total):
        o = to_E2(stream[-(total + 1) - 4:-(total + 1)])
        return o[0] * o[3] + o[1] * o[2], o[2] * o[3]

    (nl, dl), (nt, dt) = frac(gl, log_l - 1), frac(gt, log_t - 1)
    assert nl * dt + nt * dl == E2(0)


def test_wrapped_device_memory(dp, ctx, orc):
    """dps_mle_wrap_device: tables in device memory the caller owns (here torch's allocator stands for the caller).
    Download round trip, a proof over wrapped tables, an evaluation, and dps_mle_free handing the memory back only
    after the context's queued work is done."""
    torch = pytest.importorskip("torch")
    n = 13
    f, g = rand_base(1 << n, 7101), rand_e2(1 << n, 7102)
    dev = torch.device("cuda:0")
    # int64 carries the bits; the library reads them as uint64
    tf = torch.from_numpy(f.view(np.int64)).to(dev)
    tg0 = torch.from_numpy(np.ascontiguousarray(g[:, 0]).view(np.int64)).to(dev)
    tg1 = torch.from_numpy(np.ascontiguousarray(g[:, 1]).view(np.int64)).to(dev)
    torch.cuda.synchronize()
    wf = ctx.wrap_device(dp.KIND_BASE, tf.data_ptr(), None, 1 << n)
    wg = ctx.wrap_device(dp.KIND_EXT2, tg0.data_ptr(), tg1.data_ptr(), 1 << n)
    assert wf.info() == (dp.KIND_BASE, 1 << n) and wg.info() == (dp.KIND_EXT2, 1 << n)
    assert (wf.download()[:, 0] == f).all() and (wg.download() == g).all()
    r = rand_e2(n, 7103)
    eq = ctx.eq_build(r)
    terms = [(np.array([3, 5], dtype=np.uint64), [2, 0, 1]), (ONE, [0, 1])]
    tr, otr = dp.Transcript(b"wrap"), orc.OracleTranscript(b"wrap")
    proof, point, finals = ctx.sumcheck_prove(n, [wf, wg, eq], terms, tr)
    oproof, opoint, ofinals = orc.sc_prove(n, [orc.embed_base(f), g, orc.eq_evals(r)], terms, otr)
    assert (proof == oproof).all() and (point == opoint).all() and (finals == ofinals).all()
    assert tr.state() == otr.state()
    assert (wg.evaluate(point) == orc.mle_evaluate(g, point)).all()
    # the proof read the tables in place and wrote nothing to them
    torch.cuda.synchronize()
    assert (tf.cpu().numpy().view(np.uint64) == f).all()
    assert (tg1.cpu().numpy().view(np.uint64) == g[:, 1]).all()
    # a session is given up part-way (its next launch is already queued and waits on the GPU for a challenge), then the
    # handles are freed: dps_mle_free of caller-owned memory ends that launch and waits for the context's queued work,
    # after which the caller may overwrite the memory
    s = dp.Session(ctx, n, [wf, wg], [(ONE, [0, 1])])
    s.round(None)
    s.abort()
    wf.free()
    wg.free()
    del s
    tf.zero_()
    tg0.zero_()
    torch.cuda.synchronize()
    assert int(tf.abs().sum().item()) == 0
    # misuse: an extension table needs both limb arrays, pointers must be 16-byte aligned
    with pytest.raises(dp.DpsError):
        ctx.wrap_device(dp.KIND_EXT2, tg0.data_ptr(), None, 1 << n)
    with pytest.raises(dp.DpsError):
        ctx.wrap_device(dp.KIND_BASE, tf.data_ptr() + 8, None, 4)
    # the context still works
    v = rand_e2(1 << 6, 7104)
    assert (ctx.mle_from_ext2(v).download() == v).all()


def test_two_contexts_from_two_threads(dp, orc):
    """Several engine sessions live at once from different threads (the reference's ThreadPoolExecutor proves chunks
    concurrently: zkml/src/graph/executor.rs:148, zkml/src/iop/mod.rs:268-279).  Two contexts on the one GPU, one
    thread each, every thread proving its own multi-term statement 20 times while the other does the same: resident
    kernels and launches made ahead of both contexts share the GPU.  Every proof equals the checker's; a thread stops
    at its first mismatch or error."""
    cases = []
    for t, (n, seed) in enumerate([(14, 9100), (13, 9200)]):
        tabs = [rand_e2(1 << n, seed + k) for k in range(4)]
        r = rand_e2(n, seed + 9)
        lam = np.array([5 + t, 7], dtype=np.uint64)
        terms = [(ONE, [4, 0, 3]), (ONE, [4, 1, 2]), (lam, [4, 2, 3])] if t == 0 else [(lam, [0, 1]), (ONE, [2, 3, 4]), (ONE, [1, 4])]
        label = b"thread%d" % t
        ref = orc.sc_prove(n, tabs + [orc.eq_evals(r)], terms, orc.OracleTranscript(label))
        cases.append((n, tabs, r, terms, label, ref))
    failures = [None, None]
    start = threading.Barrier(2)

    def work(t):
        n, tabs, r, terms, label, ref = cases[t]
        try:
            c = dp.Context(0)
            gpu = [c.mle_from_ext2(x) for x in tabs] + [c.eq_build(r)]
            start.wait(timeout=60)
            for it in range(20):
                got = c.sumcheck_prove(n, gpu, terms, dp.Transcript(label))
                if not all((a == b).all() for a, b in zip(got, ref)):
                    failures[t] = "thread %d: proof %d differs from the checker" % (t, it)
                    return
            del gpu
            c.close()
        except Exception as e:  # noqa: BLE001 (reported by the main thread)
            failures[t] = "thread %d: %r" % (t, e)

    threads = [threading.Thread(target=work, args=(t,)) for t in range(2)]
    for th in threads:
        th.start()
    for th in threads:
        th.join(timeout=100)
    assert not any(th.is_alive() for th in threads), "a thread did not finish"
    assert failures == [None, None], failures
