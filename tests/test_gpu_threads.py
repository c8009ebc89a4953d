"""Several contexts on one GPU, and the device's ledger of launches that wait on it.

The reference proves the chunks of a model concurrently from a thread pool (zkml/src/graph/executor.rs:148,
zkml/src/iop/mod.rs:268-279), so several sessions are live at once from different threads.  Launches that stay on the
GPU between the host's turns (resident launches, launches made ahead) take their place in a process-wide ledger of the
device first; one that finds no place is not made and its rounds run as ordinary launches.  Checked here: the proofs
are the checker's bits whatever the ledger allows, from one thread with the budget cut down and from four threads
that contend for the whole device."""
import importlib
import threading

import numpy as np
import pytest

from util import rand_base, rand_e2

pytestmark = pytest.mark.gpu

ONE = np.array([1, 0], dtype=np.uint64)


@pytest.fixture(scope="module")
def dp():
    return importlib.import_module("deep-prove_amd")


def _product(orc, n, seed):
    """eq(r, .) * f * g over base-field f, g: (uploads for a context, checker tables, terms)"""
    f, g, r = rand_base(1 << n, seed), rand_base(1 << n, seed + 1), rand_e2(n, seed + 2)
    up = lambda c: [c.mle_from_base(f), c.mle_from_base(g), c.eq_build(r)]  # noqa: E731
    return up, lambda: [orc.embed_base(f), orc.embed_base(g), orc.eq_evals(r)], [(ONE, [0, 1, 2])]


def _layer(orc, n, seed):
    """a fraction-sum layer's shape: eq * (t0 t3 + t1 t2 + lambda t2 t3) over four extension tables"""
    tabs, r = [rand_e2(1 << n, seed + k) for k in range(4)], rand_e2(n, seed + 9)
    lam = np.array([seed % 1000 + 5, 7], dtype=np.uint64)
    up = lambda c: [c.mle_from_ext2(t) for t in tabs] + [c.eq_build(r)]  # noqa: E731
    return up, lambda: tabs + [orc.eq_evals(r)], [(ONE, [4, 0, 3]), (ONE, [4, 1, 2]), (lam, [4, 2, 3])]


def _stacked(orc, n, seed, pairs=8):
    """sum_h c_h A_h B_h over 2 * pairs extension tables (an einsum's stacked operands: several groups of tables)"""
    tabs = [rand_e2(1 << n, seed + k) for k in range(2 * pairs)]
    terms = [(np.array([seed % 97 + h + 1, h], dtype=np.uint64), [h, pairs + h]) for h in range(pairs)]
    up = lambda c: [c.mle_from_ext2(t) for t in tabs]  # noqa: E731
    return up, lambda: list(tabs), terms


def _reference(orc, n, host_tables, terms, label):
    return orc.sc_prove(n, host_tables(), terms, orc.OracleTranscript(label))


def _same(got, ref):
    return all((np.asarray(a) == np.asarray(b)).all() for a, b in zip(got, ref))


@pytest.mark.parametrize("budget", [0, 1, 64, 200])
def test_rounds_without_a_place_on_the_device(dp, orc, budget):
    """With the budget cut down, resident launches wider than it and launches made ahead find no place: the same rounds
    run as launches of their own (budget 0: every round of every session), and every proof is still the checker's."""
    shapes = [
        ("product", 18, _product(orc, 18, 41000)),   # resident from round 1 in 256 workgroups
        ("product", 21, _product(orc, 21, 41100)),   # first two rounds in one launch, rounds 3.. ahead, resident from round 4
        ("product", 13, _product(orc, 13, 41200)),   # a narrow resident launch (fits the larger budgets)
        ("product", 22, _product(orc, 22, 41700)),   # rounds 3 and 4 one launch; without the resident launch behind it, a catch-up fold
        ("layer", 17, _layer(orc, 17, 41300)),       # several terms: a launch of its own, then resident
        ("layer", 11, _layer(orc, 11, 41400)),
        ("stacked", 8, _stacked(orc, 8, 41500)),     # three groups of tables, every round resident when admitted
        ("stacked", 17, _stacked(orc, 17, 41600, pairs=5)),  # two groups: the groups' launches, resident side by side at the end
    ]
    ctx = dp.Context(0)
    try:
        dp.set_resident_budget(0, budget)
        assert dp.resident_budget(0) == (0, budget)
        for kind, n, (up, host_tables, terms) in shapes:
            label = b"budget"
            ref = _reference(orc, n, host_tables, terms, label)
            gpu = up(ctx)
            for _ in range(2):
                tr = dp.Transcript(label)
                got = ctx.sumcheck_prove(n, gpu, terms, tr)
                assert _same(got, ref), (kind, n, budget)
                assert dp.resident_budget(0)[0] == 0, "a finished session still holds its place"
    finally:
        dp.set_resident_budget(0, -1)
        ctx.close()
    used, cap = dp.resident_budget(0)
    assert used == 0 and cap > 0


def test_a_session_left_midway_gives_its_place_back(dp, orc):
    ctx = dp.Context(0)
    up, _, terms = _product(orc, 16, 42000)
    gpu = up(ctx)
    s = ctx.session(16, gpu, terms)
    s.round(None)
    assert dp.resident_budget(0)[0] > 0  # its resident launch waits on the GPU
    s.abort()
    assert dp.resident_budget(0)[0] == 0
    del s
    # ... and so does a context that is closed while a launch of it waits
    s2 = ctx.session(16, gpu, terms)
    s2.round(None)
    assert dp.resident_budget(0)[0] > 0
    del s2, gpu
    ctx.close()
    assert dp.resident_budget(0)[0] == 0


def test_four_contexts_from_four_threads(dp, orc):
    """Four contexts on the one GPU, one thread each; every thread proves its own 18-variable eq * f * g (a resident
    launch of 256 workgroups: the whole device) and its own 17-variable three-term sum, five times each, while the
    others do the same.  Only one of the wide launches can hold the device at a time; the others' rounds run as
    ordinary launches.  Every proof equals the checker's and no call fails; a thread stops at its first mismatch."""
    n_threads, reps = 4, 5
    cases = []
    for t in range(n_threads):
        prod, layer = _product(orc, 18, 43000 + 100 * t), _layer(orc, 17, 44000 + 100 * t)
        label = b"thread%d" % t
        cases.append([(18, prod, _reference(orc, 18, prod[1], prod[2], label)), (17, layer, _reference(orc, 17, layer[1], layer[2], label))])
    failures = [None] * n_threads
    start = threading.Barrier(n_threads)

    def work(t):
        try:
            c = dp.Context(0)
            live = [(n, up(c), terms, ref) for n, (up, _, terms), ref in cases[t]]
            start.wait(timeout=120)
            for it in range(reps):
                for n, gpu, terms, ref in live:
                    got = c.sumcheck_prove(n, gpu, terms, dp.Transcript(b"thread%d" % t))
                    if not _same(got, ref):
                        failures[t] = "thread %d: proof %d of the %d-variable sum differs from the checker" % (t, it, n)
                        return
            del live
            c.close()
        except Exception as e:  # noqa: BLE001 (reported by the main thread)
            failures[t] = "thread %d: %r" % (t, e)

    threads = [threading.Thread(target=work, args=(t,)) for t in range(n_threads)]
    for th in threads:
        th.start()
    for th in threads:
        th.join(timeout=110)
    assert not any(th.is_alive() for th in threads), "a thread did not finish"
    assert failures == [None] * n_threads, failures
    assert dp.resident_budget(0)[0] == 0
