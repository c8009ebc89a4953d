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
