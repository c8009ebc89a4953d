"""The entry point that allocates nothing (dps_mle_evaluate_noalloc) against the existing dps_mle_evaluate: same bits,
on calls in a row that share the library's one work area per GPU, the later ones with smaller inputs."""
import importlib

import numpy as np
import pytest

from util import rand_base, rand_e2, rand_i64

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dp():
    return importlib.import_module("deep-prove_amd")


@pytest.fixture(scope="module")
def ctx(dp):
    c = dp.Context(0)
    yield c
    c.close()


def test_evaluate_noalloc_matches_evaluate(dp, ctx, orc):
    # two calls in a row through the C ABI, the second with a smaller input: the work area keeps the first call's
    # contents (longer eq tables, more partial sums) and the second must not be disturbed by them
    big, small = 16, 9
    tb, ts = rand_e2(1 << big, 31001), rand_base(1 << small, 31002)
    pb, ps = rand_e2(big, 31003), rand_e2(small, 31004)
    mb, ms = ctx.mle_from_ext2(tb), ctx.mle_from_base(ts)
    got_b = mb.evaluate_noalloc(pb)
    got_s = ms.evaluate_noalloc(ps)
    assert (got_b == mb.evaluate(pb)).all() and (got_s == ms.evaluate(ps)).all()
    # and against the CPU checker's evaluation
    assert (got_b == orc.mle_evaluate(tb, pb)).all()
    assert (got_s == orc.mle_evaluate(orc.embed_base(ts), ps)).all()
    # again in the other order, and repeated: same bits every time
    assert (ms.evaluate_noalloc(ps) == got_s).all() and (mb.evaluate_noalloc(pb) == got_b).all()
    assert (mb.evaluate_noalloc(pb) == got_b).all()


@pytest.mark.parametrize("n", [0, 1, 5, 11, 12, 13, 14, 20])
def test_evaluate_noalloc_sizes_and_kinds(dp, ctx, n):
    # every storage kind on both sides of the row length (2^12) at which the kernel changes its loop
    pt = rand_e2(n, 32000 + n)
    ext = ctx.mle_from_ext2(rand_e2(1 << n, 32100 + n))
    base = ctx.mle_from_base(rand_base(1 << n, 32200 + n))
    assert (ext.evaluate_noalloc(pt) == ext.evaluate(pt)).all()
    assert (base.evaluate_noalloc(pt) == base.evaluate(pt)).all()
    if n <= 14:
        v = rand_i64(1 << n, 32300 + n)
        t64, t16 = ctx.tensor_from_i64(v), ctx.tensor_from_i16(v)
        want = t64.evaluate(pt)
        assert (t64.evaluate_noalloc(pt) == want).all() and (t16.evaluate_noalloc(pt) == want).all()


def test_evaluate_noalloc_full_size_and_limits(dp, ctx):
    # the largest table the work area serves, then one beyond it
    n = 24
    base = ctx.mle_from_base(rand_base(1 << n, 33001))
    pt = rand_e2(n, 33002)
    assert (base.evaluate_noalloc(pt) == base.evaluate(pt)).all()
    # a smaller call right after the largest
    small = ctx.mle_from_ext2(rand_e2(1 << 3, 33003))
    ps = rand_e2(3, 33004)
    assert (small.evaluate_noalloc(ps) == small.evaluate(ps)).all()
    del base
    too_big = ctx.mle_from_base(rand_base(1 << 25, 33005))
    with pytest.raises(dp.DpsError) as e:
        too_big.evaluate_noalloc(rand_e2(25, 33006))
    assert e.value.status == 5 and "24" in str(e.value)
    with pytest.raises(dp.DpsError):
        small.evaluate_noalloc(rand_e2(4, 1))  # point length does not match
    bad = rand_e2(3, 2)
    bad[1, 0] = np.uint64(dp.P)
    with pytest.raises(dp.DpsError):
        small.evaluate_noalloc(bad)  # not canonical
    with pytest.raises(dp.DpsError):
        small.zero_pad(5).evaluate_noalloc(rand_e2(5, 3))
    # the context is still usable
    assert (small.evaluate_noalloc(ps) == small.evaluate(ps)).all()


def _device_free_bytes():
    import torch

    return torch.cuda.mem_get_info(0)[0]


def test_evaluate_noalloc_takes_nothing_from_the_driver(dp, ctx, orc):
    # neither the context's pool nor the device's free memory moves across the calls, whatever the table is --
    # including an eq table of 20 variables whose entries have never been read (dps_eq_build keeps them
    # unmaterialised: that one is evaluated in closed form, prod eq1(rho_i, z_i))
    n = 20
    rho, z = rand_e2(n, 34001), rand_e2(n, 34002)
    eq = ctx.eq_build(rho)
    base = ctx.mle_from_base(rand_base(1 << 18, 34003))
    zb = rand_e2(18, 34004)
    small_eq = ctx.eq_build(rand_e2(11, 34005))
    zs = rand_e2(11, 34006)
    ctx.sync()

    def taken():
        # blocks the context holds from the driver, handed out or cached (tables of earlier tests may go back to the
        # cache at any time: that moves a block from one count to the other), and their bytes
        in_use, cached, nbytes = ctx.pool_info()
        return in_use + cached, nbytes

    pool0, free0 = taken(), _device_free_bytes()
    got_eq = eq.evaluate_noalloc(z)
    got_base = base.evaluate_noalloc(zb)
    got_small = small_eq.evaluate_noalloc(zs)
    assert taken() == pool0 and _device_free_bytes() == free0
    assert (got_eq == orc.identity_eval(rho, z)).all()
    # the allocating call builds the table's entries and evaluates them: the same element
    assert (eq.evaluate(z) == got_eq).all()
    # ... and once they are there the entry point reads them like any table's
    pool1 = taken()
    assert (eq.evaluate_noalloc(z) == got_eq).all() and taken() == pool1
    assert (got_base == base.evaluate(zb)).all() and (got_small == small_eq.evaluate(zs)).all()


def test_evaluate_noalloc_refuses_while_a_launch_waits(dp, ctx, orc):
    # between the rounds of a small product session its resident launch waits on the GPU for the next challenge: ending
    # it would take a stream wait, so the entry point says so instead, and the session goes on undisturbed
    n = 12
    f, g = rand_base(1 << n, 35001), rand_base(1 << n, 35002)
    terms = [(np.array([1, 0], np.uint64), [0, 1])]
    mf, mg = ctx.mle_from_base(f), ctx.mle_from_base(g)
    other = ctx.mle_from_base(rand_base(1 << 6, 35003))
    zo = rand_e2(6, 35004)
    want_other = other.evaluate(zo)
    tr = dp.Transcript(b"busy")
    tr.append_u64(n)
    tr.append_u64(2)
    s = ctx.session(n, [mf, mg], terms)
    msgs, point = [], []
    ch = None
    for j in range(1, n + 1):
        msgs.append(s.round(ch))
        if j == 2:
            with pytest.raises(dp.DpsError) as e:
                other.evaluate_noalloc(zo)
            assert e.value.status == 4
        tr.append_scalars(msgs[-1])
        ch = tr.challenge_scalar()
        point.append(ch)
    finals = s.finish(ch)
    otr = orc.OracleTranscript(b"busy")
    oproof, opoint, ofinals = orc.sc_prove(n, [orc.embed_base(f), orc.embed_base(g)], terms, otr)
    assert (np.array(msgs) == oproof).all() and (np.array(point) == opoint).all() and (finals == ofinals).all()
    assert (other.evaluate_noalloc(zo) == want_other).all()


def test_evaluate_noalloc_from_two_threads(dp, orc):
    # two contexts on two threads share the GPU's one work area: the library lets one call at a time use it
    import threading

    errors = []

    def worker(seed):
        try:
            c = dp.Context(0)
            tabs = [(c.mle_from_ext2(rand_e2(1 << k, seed + k)), rand_e2(k, seed + 100 + k)) for k in (7, 13, 16)]
            want = [t.evaluate(z) for t, z in tabs]
            for it in range(50):
                t, z = tabs[it % 3]
                got = t.evaluate_noalloc(z)
                if not (got == want[it % 3]).all():
                    errors.append("thread %d call %d: %r != %r" % (seed, it, got, want[it % 3]))
                    return
            del tabs
            c.close()
        except Exception as ex:  # noqa: BLE001 -- reported by the main thread
            errors.append("thread %d: %r" % (seed, ex))

    ts = [threading.Thread(target=worker, args=(36000 + 1000 * i,)) for i in range(2)]
    for t in ts:
        t.start()
    for t in ts:
        t.join(120)
    assert not any(t.is_alive() for t in ts), "a thread did not finish"
    assert not errors, errors
