"""Seeded instances of the sumcheck that links a lookup argument to its layer
(zkml/src/lookup/operation/inputs/proving.rs:26-114): one per variant and per
shape of the chunking (one or several value chunks; none, one or two zeroing
chunks; signed and unsigned tables; rank 1 to 4 inputs)."""
import numpy as np

from util import rand_e2, rand_i64

CASES = [
    dict(variant="standard", shape=[5, 6], value_chunks=1, zero_chunks=0, bit_size=8, signed=True, min_out=-128, max_out=127),
    dict(variant="standard", shape=[3, 4, 5], value_chunks=1, zero_chunks=1, bit_size=8, signed=True, min_out=-100, max_out=90),
    dict(variant="standard", shape=[2, 3, 4, 5], value_chunks=2, zero_chunks=2, bit_size=4, signed=True, min_out=-7, max_out=7),
    dict(variant="standard", shape=[2, 4, 4], value_chunks=1, zero_chunks=2, bit_size=8, signed=False, min_out=0, max_out=255, input_sign="positive"),
    dict(variant="standard", shape=[7], value_chunks=1, zero_chunks=0, bit_size=8, signed=False, min_out=0, max_out=255, input_sign="positive"),
    dict(variant="standard", shape=[3, 3, 2], value_chunks=3, zero_chunks=1, bit_size=4, signed=False, min_out=-9, max_out=0, input_sign="negative"),
    dict(variant="glu", shape=[2, 4, 8], value_chunks=1, zero_chunks=1, bit_size=8, signed=True, min_out=-128, max_out=127),
    dict(variant="softmax", shape=[3, 4, 6], value_chunks=1, zero_chunks=1, bit_size=8, signed=False, min_out=0, max_out=200, input_sign="negative"),
    dict(variant="softmax", shape=[4, 8], value_chunks=1, zero_chunks=0, bit_size=8, signed=True, min_out=-128, max_out=127),
    dict(variant="normalisation", shape=[2, 4, 8], value_chunks=1, zero_chunks=1, bit_size=8, signed=True, min_out=-128, max_out=127, norm_sum=True,
         has_weight=True),
    dict(variant="normalisation", shape=[3, 2, 5], value_chunks=2, zero_chunks=0, bit_size=4, signed=True, min_out=-8, max_out=7, norm_sum=False,
         has_weight=False),
    dict(variant="normalisation", shape=[2, 2, 4], value_chunks=1, zero_chunks=2, bit_size=8, signed=True, min_out=-50, max_out=60, norm_sum=False,
         has_weight=True),
]
for _c in CASES:
    _c.setdefault("input_sign", "positive")
    _c.setdefault("norm_sum", False)
    _c.setdefault("has_weight", False)


def ceil_log2(n):
    return max(0, (n - 1).bit_length())


def chunks_of(cfg):
    n = 1
    for d in cfg["shape"][:max(0, len(cfg["shape"]) - 2)]:
        n *= d
    return n


def chunk_vars(cfg):
    return sum(ceil_log2(d) for d in cfg["shape"][-2:])


def make_instance(cfg, seed):
    """Witness tables as int64 arrays (values small enough for a lookup table's columns), in the expression's
    order, the optional weight table, and the two points.  The sumcheck is an identity in the tables, so they
    need not come from a real layer."""
    n = 1 << chunk_vars(cfg)
    nvc, nz, C = cfg["value_chunks"], cfg["zero_chunks"], chunks_of(cfg)
    half = 1 << (cfg["bit_size"] - 1)
    tabs, k = [], 0
    for c in range(C):
        for i in range(nvc):
            tabs.append(rand_i64(n, seed * 1000 + k, -half, half - 1))
            k += 1
        for i in range(nz):
            top_signed = cfg["signed"] and i == nz - 1
            tabs.append(rand_i64(n, seed * 1000 + k, -1 if top_signed else 0, 1))
            k += 1
    extra = {"standard": 0, "softmax": 0, "glu": 1, "normalisation": 2}[cfg["variant"]]
    for e in range(extra * C):
        tabs.append(rand_i64(n, seed * 1000 + k, -300, 300))
        k += 1
    weight = rand_i64(n, seed * 1000 + k, -64, 64) if cfg["has_weight"] else None
    total_vars = sum(ceil_log2(d) for d in cfg["shape"])
    last_claim_point = rand_e2(total_vars, seed * 7 + 1)
    logup_point = rand_e2(chunk_vars(cfg), seed * 7 + 2)
    return tabs, weight, last_claim_point, logup_point
