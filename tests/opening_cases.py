"""Seeded instances of the claims-batching sumcheck, shaped like the reference's
test_poly_commit (zkml/src/poly_commit/mod.rs:224-409): five model polynomials of
10..15 variables (every second one with two claims), one table polynomial, eight
witness polynomials of 10..13 variables; with the chunked variant every polynomial
of more than `chunk_vars` variables is held as chunks of 2^chunk_vars entries."""
import numpy as np

from util import py_rng, rand_e2


def make_instance(orc, seed, chunk_vars=None, small=False):
    rng = py_rng(seed)
    lo, hi = (3, 7) if small else (10, 15)
    sizes = [rng.randint(lo, hi) for _ in range(5)] + [rng.randint(lo, hi - 2)] + [rng.randint(lo, hi - 2) for _ in range(8)]
    polys, claims = [], []
    for i, nv in enumerate(sizes):
        full = rand_e2(1 << nv, seed * 100 + i)
        n_claims = 2 if (i < 5 and i % 2 == 1) else 1
        cls = []
        for k in range(n_claims):
            point = rand_e2(nv, seed * 1000 + 10 * i + k)
            cls.append((point, orc.mle_evaluate(full, point)))
        m = nv if chunk_vars is None else min(nv, chunk_vars)
        chunks = [full[c << m:(c + 1) << m] for c in range(1 << (nv - m))]
        polys.append(chunks)
        claims.append(cls)
    shapes = [(len(c), nv) for c, nv in zip(polys, sizes)]
    return polys, claims, shapes
