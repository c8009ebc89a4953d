"""ctypes bindings of the CPU checker (test infrastructure only).

Only tests/, the smoke check and the benchmark's cpu_baseline leg import this
module.  Extension elements cross as numpy uint64 arrays of shape (..., 2)
holding (c0, c1).
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libdpsc_oracle.so")

P = 0xFFFFFFFF00000001
MAX_FACTORS = 8
AXIS_CONTRACTED, AXIS_OUTER, AXIS_STACKED = 0, 1, 2


def build(force=False):
    """Compile the checker with the Makefile beside this file."""
    if force or not os.path.exists(_LIB_PATH) or not os.path.exists(os.path.join(_HERE, "libdpsc_oracle_fast.so")):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s"])
    return _LIB_PATH


class Term(C.Structure):
    _fields_ = [("coeff", C.c_uint64 * 2), ("n_factors", C.c_uint32), ("factors", C.c_uint32 * MAX_FACTORS)]


class Transcript(C.Structure):
    _fields_ = [("state", C.c_uint8 * 32), ("n_rounds", C.c_uint32)]


class LogupInstance(C.Structure):
    _fields_ = [
        ("n_cols", C.c_uint32),
        ("len", C.c_uint64),
        ("cols", C.POINTER(C.c_void_p)),
        ("numer", C.c_void_p),
        ("c", C.c_uint64 * 2),
        ("beta", C.c_uint64 * 2),
    ]


_lib = None
_FAST_PATH = os.path.join(_HERE, "libdpsc_oracle_fast.so")
_use_fast = False


def select(fast: bool):
    """Switch between the plain checker and its division-free build (the timed
    CPU baseline).  Both come from the same source; tests compare them."""
    global _lib, _use_fast
    if fast != _use_fast:
        _use_fast, _lib = fast, None


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(_FAST_PATH if _use_fast else _LIB_PATH)
        u64, i64, vp = C.c_uint64, C.c_int64, C.c_void_p
        for name in ("add", "sub", "mul", "pow"):
            f = getattr(_lib, "orc_gl_" + name)
            f.restype, f.argtypes = u64, [u64, u64]
        for name in ("neg", "inv"):
            f = getattr(_lib, "orc_gl_" + name)
            f.restype, f.argtypes = u64, [u64]
        _lib.orc_gl_from_i64.restype, _lib.orc_gl_from_i64.argtypes = u64, [i64]
        _lib.orc_gl_to_i64.restype, _lib.orc_gl_to_i64.argtypes = i64, [u64]
        _lib.orc_logup_arena_len.restype, _lib.orc_logup_arena_len.argtypes = u64, [u64]
        _lib.orc_logup_layer_offset.restype, _lib.orc_logup_layer_offset.argtypes = u64, [u64, C.c_uint32]
        _lib.orc_partial_eval.restype = i64
        _lib.orc_stacking_coeffs.restype = i64
        _lib.orc_logup_batch_prove.restype = i64
        _lib.orc_sc_prove.restype = C.c_int
        _lib.orc_sc_verify.restype = C.c_int
        _lib.orc_logup_batch_verify.restype = C.c_int
        _lib.orc_num_threads.restype = C.c_int
    return _lib


def _e2arr(x):
    a = np.ascontiguousarray(x, dtype=np.uint64)
    assert a.shape[-1] == 2, a.shape
    return a


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def e2(c0, c1=0):
    return np.array([c0 % P, c1 % P], dtype=np.uint64)


# ---- field ----
def gl_mul(a, b):
    return lib().orc_gl_mul(int(a), int(b))


def gl_add(a, b):
    return lib().orc_gl_add(int(a), int(b))


def gl_sub(a, b):
    return lib().orc_gl_sub(int(a), int(b))


def gl_inv(a):
    return lib().orc_gl_inv(int(a))


def gl_from_i64(x):
    return lib().orc_gl_from_i64(int(x))


def gl_to_i64(x):
    return lib().orc_gl_to_i64(int(x))


def _bin(name, a, b):
    a, b = _e2arr(a), _e2arr(b)
    out = np.zeros(2, dtype=np.uint64)
    getattr(lib(), name)(_p(a), _p(b), _p(out))
    return out


def e2_add(a, b):
    return _bin("orc_e2_add", a, b)


def e2_sub(a, b):
    return _bin("orc_e2_sub", a, b)


def e2_mul(a, b):
    return _bin("orc_e2_mul", a, b)


def e2_inv(a):
    a = _e2arr(a)
    out = np.zeros(2, dtype=np.uint64)
    lib().orc_e2_inv(_p(a), _p(out))
    return out


# ---- tables ----
def eq_evals(point):
    point = _e2arr(point).reshape(-1, 2)
    m = point.shape[0]
    out = np.zeros((1 << m, 2), dtype=np.uint64)
    lib().orc_eq_evals(_p(point), C.c_uint32(m), _p(out))
    return out


def identity_eval(r1, r2):
    r1, r2 = _e2arr(r1).reshape(-1, 2), _e2arr(r2).reshape(-1, 2)
    n = min(len(r1), len(r2))
    out = np.zeros(2, dtype=np.uint64)
    lib().orc_identity_eval(_p(r1), _p(r2), C.c_uint32(n), _p(out))
    return out


def embed_base(v):
    v = np.ascontiguousarray(v, dtype=np.uint64)
    out = np.zeros((v.size, 2), dtype=np.uint64)
    lib().orc_embed_base(_p(v), C.c_uint64(v.size), _p(out))
    return out


def embed_i64(v):
    v = np.ascontiguousarray(v, dtype=np.int64)
    out = np.zeros((v.size, 2), dtype=np.uint64)
    lib().orc_embed_i64(_p(v), C.c_uint64(v.size), _p(out))
    return out


def _nvars(tbl):
    n = int(tbl.shape[0]).bit_length() - 1
    assert 1 << n == tbl.shape[0]
    return n


def mle_evaluate(tbl, point):
    tbl, point = _e2arr(tbl), _e2arr(point).reshape(-1, 2)
    n = _nvars(tbl)
    assert point.shape[0] == n
    out = np.zeros(2, dtype=np.uint64)
    lib().orc_mle_evaluate(_p(tbl), C.c_uint32(n), _p(point), _p(out))
    return out


def mle_fix_low(tbl, point):
    tbl, point = _e2arr(tbl), _e2arr(point).reshape(-1, 2)
    n, k = _nvars(tbl), point.shape[0]
    out = np.zeros((1 << (n - k), 2), dtype=np.uint64)
    lib().orc_mle_fix_low(_p(tbl), C.c_uint32(n), _p(point), C.c_uint32(k), _p(out))
    return out


def mle_fix_high(tbl, point):
    tbl, point = _e2arr(tbl), _e2arr(point).reshape(-1, 2)
    n, k = _nvars(tbl), point.shape[0]
    out = np.zeros((1 << (n - k), 2), dtype=np.uint64)
    lib().orc_mle_fix_high(_p(tbl), C.c_uint32(n), _p(point), C.c_uint32(k), _p(out))
    return out


# ---- hash / transcript ----
def blake3(data: bytes) -> bytes:
    out = (C.c_uint8 * 32)()
    buf = (C.c_uint8 * max(1, len(data))).from_buffer_copy(data or b"\0")
    lib().orc_blake3(buf, C.c_size_t(len(data)), out)
    return bytes(out)


class OracleTranscript:
    def __init__(self, label: bytes = b"m2vec"):
        self.t = Transcript()
        lib().orc_tr_new(C.byref(self.t), label, C.c_size_t(len(label)))

    def state(self):
        return bytes(self.t.state), int(self.t.n_rounds)

    def append_message(self, label: bytes):
        lib().orc_tr_append_message(C.byref(self.t), label, C.c_size_t(len(label)))

    def append_bytes(self, data: bytes):
        lib().orc_tr_append_bytes(C.byref(self.t), data, C.c_size_t(len(data)))

    def append_u64(self, x):
        lib().orc_tr_append_u64(C.byref(self.t), C.c_uint64(x))

    def append_scalars(self, xs):
        xs = _e2arr(xs).reshape(-1, 2)
        lib().orc_tr_append_scalars(C.byref(self.t), _p(xs), C.c_size_t(xs.shape[0]))

    def challenge_scalar(self):
        out = np.zeros(2, dtype=np.uint64)
        lib().orc_tr_challenge_scalar(C.byref(self.t), _p(out))
        return out

    def append_and_sample(self, label: bytes):
        out = np.zeros(2, dtype=np.uint64)
        lib().orc_tr_append_and_sample(C.byref(self.t), label, C.c_size_t(len(label)), _p(out))
        return out

    def read_challenges(self, n):
        return np.stack([self.challenge_scalar() for _ in range(n)]) if n else np.zeros((0, 2), np.uint64)


# ---- sumcheck ----
def make_terms(terms):
    """terms: list of (coeff e2, [mle indices])"""
    arr = (Term * max(1, len(terms)))()
    for i, (coeff, factors) in enumerate(terms):
        c = _e2arr(coeff)
        arr[i].coeff[0], arr[i].coeff[1] = int(c[0]), int(c[1])
        arr[i].n_factors = len(factors)
        for k, f in enumerate(factors):
            arr[i].factors[k] = f
    return arr


def _table_ptrs(tables):
    tabs = [_e2arr(t) for t in tables]
    ptrs = (C.c_void_p * max(1, len(tabs)))(*[t.ctypes.data for t in tabs])
    nvs = (C.c_uint32 * max(1, len(tabs)))(*[_nvars(t) for t in tabs])
    return tabs, ptrs, nvs


def sc_round_poly(live, tables, cur_nvars, terms):
    tabs, ptrs, _ = _table_ptrs(tables)
    nvs = (C.c_uint32 * len(tabs))(*cur_nvars)
    tarr = make_terms(terms)
    degree = max((len(f) for _, f in terms), default=0)
    out = np.zeros((degree + 1, 2), dtype=np.uint64)
    lib().orc_sc_round_poly(C.c_uint32(live), C.c_uint32(len(tabs)), ptrs, nvs, tarr, C.c_uint32(len(terms)),
                            C.c_uint32(degree), _p(out))
    return out


def sc_prove(n_vars, tables, terms, transcript):
    """Returns (proof[n_vars, d+1, 2], point[n_vars, 2], final_evals[n_mles, 2])."""
    tabs, ptrs, nvs = _table_ptrs(tables)
    tarr = make_terms(terms)
    degree = max((len(f) for _, f in terms), default=0)
    proof = np.zeros((n_vars, degree + 1, 2), dtype=np.uint64)
    point = np.zeros((n_vars, 2), dtype=np.uint64)
    final = np.zeros((len(tabs), 2), dtype=np.uint64)
    rc = lib().orc_sc_prove(C.c_uint32(n_vars), C.c_uint32(len(tabs)), ptrs, nvs, tarr, C.c_uint32(len(terms)),
                            C.byref(transcript.t), _p(proof), _p(point), _p(final))
    if rc != 0:
        raise ValueError(f"orc_sc_prove failed: {rc}")
    return proof, point, final


def sc_verify(claimed_sum, proof, transcript):
    """Returns (bad_round (0 = ok), point, expected_evaluation)."""
    proof = _e2arr(proof)
    n_vars, npts = proof.shape[0], proof.shape[1]
    claimed = _e2arr(claimed_sum)
    point = np.zeros((n_vars, 2), dtype=np.uint64)
    expected = np.zeros(2, dtype=np.uint64)
    rc = lib().orc_sc_verify(_p(claimed), _p(proof), C.c_uint32(n_vars), C.c_uint32(npts - 1),
                             C.byref(transcript.t), _p(point), _p(expected))
    return rc, point, expected


def interpolate(evals, r):
    evals, r = _e2arr(evals).reshape(-1, 2), _e2arr(r)
    out = np.zeros(2, dtype=np.uint64)
    lib().orc_interpolate(_p(evals), C.c_uint32(evals.shape[0] - 1), _p(r), _p(out))
    return out


# ---- einsum partial evaluation ----
def _points_ptrs(points):
    keep = [None if p is None else _e2arr(p).reshape(-1, 2) for p in points]
    ptrs = (C.c_void_p * len(keep))(*[None if p is None else p.ctypes.data for p in keep])
    return keep, ptrs


def partial_eval(tensor, padded_dims, unpadded_dims, kinds, points):
    tensor = np.ascontiguousarray(tensor, dtype=np.int64)
    nd = len(padded_dims)
    pd = (C.c_uint64 * nd)(*padded_dims)
    ud = (C.c_uint64 * nd)(*unpadded_dims)
    kd = (C.c_int32 * nd)(*kinds)
    keep, ptrs = _points_ptrs(points)
    cap = 1
    for d in unpadded_dims:
        cap *= d
    cap = 2 * cap + 2
    out = np.zeros((cap, 2), dtype=np.uint64)
    tl = C.c_uint64(0)
    n = lib().orc_partial_eval(_p(tensor), pd, ud, C.c_uint32(nd), kd, ptrs, _p(out), C.c_uint64(cap), C.byref(tl))
    if n < 0:
        raise ValueError(f"orc_partial_eval failed: {n}")
    return out[: n * tl.value].reshape(n, tl.value, 2).copy()


def stacking_coeffs(padded_dims, unpadded_dims, kinds, points):
    nd = len(padded_dims)
    pd = (C.c_uint64 * nd)(*padded_dims)
    ud = (C.c_uint64 * nd)(*unpadded_dims)
    kd = (C.c_int32 * nd)(*kinds)
    keep, ptrs = _points_ptrs(points)
    cap = 1
    for d, k in zip(unpadded_dims, kinds):
        if k == AXIS_STACKED:
            cap *= d
    out = np.zeros((cap, 2), dtype=np.uint64)
    n = lib().orc_stacking_coeffs(pd, ud, C.c_uint32(nd), kd, ptrs, _p(out), C.c_uint64(cap))
    if n < 0:
        raise ValueError(f"orc_stacking_coeffs failed: {n}")
    return out[:n].copy()


# ---- LogUp ----
def logup_build(cols, numer, c, beta):
    cols = [np.ascontiguousarray(x, dtype=np.uint64) for x in cols]
    ln = cols[0].size
    ptrs = (C.c_void_p * len(cols))(*[x.ctypes.data for x in cols])
    nm = None if numer is None else np.ascontiguousarray(numer, dtype=np.uint64)
    alen = lib().orc_logup_arena_len(C.c_uint64(ln))
    arena = np.zeros((alen + 1, 2), dtype=np.uint64)
    cc, bb = _e2arr(c), _e2arr(beta)
    lib().orc_logup_build(ptrs, C.c_uint32(len(cols)), None if nm is None else _p(nm), C.c_uint64(ln), _p(cc), _p(bb),
                          _p(arena))
    layers = []
    top = ln.bit_length() - 1
    for k in range(1, top):
        off = lib().orc_logup_layer_offset(C.c_uint64(ln), C.c_uint32(k))
        sz = ln >> k
        layers.append((arena[off:off + sz].copy(), arena[off + sz:off + 2 * sz].copy()))
    return layers


def _instances(instances):
    """instances: list of dicts {cols: [u64 arrays], numer: array|None, c: e2, beta: e2}"""
    arr = (LogupInstance * len(instances))()
    keep = []
    for i, ins in enumerate(instances):
        cols = [np.ascontiguousarray(x, dtype=np.uint64) for x in ins["cols"]]
        ptrs = (C.c_void_p * len(cols))(*[x.ctypes.data for x in cols])
        nm = None if ins.get("numer") is None else np.ascontiguousarray(ins["numer"], dtype=np.uint64)
        keep.append((cols, ptrs, nm))
        arr[i].n_cols = len(cols)
        arr[i].len = cols[0].size
        arr[i].cols = C.cast(ptrs, C.POINTER(C.c_void_p))
        arr[i].numer = None if nm is None else nm.ctypes.data
        c, b = _e2arr(ins["c"]), _e2arr(ins["beta"])
        arr[i].c[0], arr[i].c[1] = int(c[0]), int(c[1])
        arr[i].beta[0], arr[i].beta[1] = int(b[0]), int(b[1])
    return arr, keep


def logup_batch_prove(instances, transcript):
    """Returns the flat proof stream (see orc_logup_batch_prove)."""
    arr, keep = _instances(instances)
    total = max(int(i["cols"][0].size).bit_length() - 2 for i in instances)
    cap = sum(v * 4 for v in range(1, total + 1))
    cap += (total + 2) * sum(2 * len(i["cols"]) + 6 for i in instances) + total + 8
    out = np.zeros((cap, 2), dtype=np.uint64)
    n = lib().orc_logup_batch_prove(arr, C.c_uint32(len(instances)), C.byref(transcript.t), _p(out), C.c_uint64(cap))
    if n < 0:
        raise ValueError(f"orc_logup_batch_prove failed: {n}")
    return out[:n].copy()


def logup_batch_verify(instances_meta, is_table, stream, transcript):
    """instances_meta: list of (n_cols, num_vars, c, beta).  Returns (rc, claims, point)."""
    n = len(instances_meta)
    ncols = (C.c_uint32 * n)(*[m[0] for m in instances_meta])
    nvars = (C.c_uint32 * n)(*[m[1] for m in instances_meta])
    cs = np.stack([_e2arr(m[2]) for m in instances_meta])
    bs = np.stack([_e2arr(m[3]) for m in instances_meta])
    stream = _e2arr(stream)
    total = max(m[1] for m in instances_meta)
    n_claims = sum(m[0] + (1 if is_table else 0) for m in instances_meta)
    claims = np.zeros((n_claims, 2), dtype=np.uint64)
    point = np.zeros((total + 1, 2), dtype=np.uint64)
    rc = lib().orc_logup_batch_verify(ncols, nvars, _p(cs), _p(bs), C.c_int(1 if is_table else 0), C.c_uint32(n),
                                      _p(stream), C.c_uint64(stream.shape[0]), C.byref(transcript.t), _p(claims),
                                      _p(point))
    return rc, claims, point


# ---- claims-batching sumcheck of the opening proof ----
# Follows zkml/src/poly_commit/prover.rs:140-255 (prover), mod.rs:46-68,95-159 (chunk
# coefficients, eq point, expression) and verifier.rs:203-340 (verifier).  The
# zero-padded views the reference takes (prover.rs:214-226) are written out in full
# here, straight from their definition: entries beyond the table's length are 0.
def _pow_e2(x, k):
    out = e2(1)
    for _ in range(k):
        out = e2_mul(out, x)
    return out


def chunk_batching_coefficients(num_chunks, point):
    """mod.rs:46-58: C_c = identity_eval(point[-b:], bits_le(c)), b = log2(num_chunks)."""
    point = _e2arr(point).reshape(-1, 2)
    b = num_chunks.bit_length() - 1
    assert 1 << b == num_chunks
    coords = point[len(point) - b:]
    out = []
    for c in range(num_chunks):
        bits = np.array([[(c >> j) & 1, 0] for j in range(b)], dtype=np.uint64).reshape(-1, 2)
        out.append(identity_eval(coords, bits) if b else e2(1))
    return out


def _claims_batching_terms(polys_chunks, claims, challenge):
    """mod.rs:95-159 flattened: one product chal^k * C_c * chunk_c * eq_k per (claim, chunk)."""
    eq_offset = sum(polys_chunks)
    terms, k, base = [], 0, 0
    for nch, cls in zip(polys_chunks, claims):
        for point, _ in cls:
            ck = _pow_e2(challenge, k)
            for c, coeff in enumerate(chunk_batching_coefficients(nch, point)):
                terms.append((e2_mul(ck, coeff), [base + c, eq_offset + k]))
            k += 1
        base += nch
    return terms


def claims_batching_prove(polys, claims, transcript):
    """polys: per committed polynomial, the list of its chunk tables ((2^m, 2) arrays);
    claims: per polynomial, a list of (point, eval).  Returns (proof, point, chunk_evals)."""
    chunk_tabs, eq_tabs = [], []
    max_vars = 0
    for chunks, cls in zip(polys, claims):
        nch = len(chunks)
        b = nch.bit_length() - 1
        for point, ev in cls:
            point = _e2arr(point).reshape(-1, 2)
            transcript.append_scalars(_e2arr(ev).reshape(1, 2))
            eq_tabs.append(eq_evals(point[: len(point) - b]))
        chunk_tabs.extend(_e2arr(c).reshape(-1, 2) for c in chunks)
        max_vars = max(max_vars, _nvars(_e2arr(chunks[0]).reshape(-1, 2)))

    def padded(t):
        out = np.zeros((1 << max_vars, 2), dtype=np.uint64)
        out[: t.shape[0]] = t
        return out

    tables = [padded(t) for t in chunk_tabs + eq_tabs]
    challenge = transcript.append_and_sample(b"model_batching")
    terms = _claims_batching_terms([len(c) for c in polys], claims, challenge)
    proof, point, finals = sc_prove(max_vars, tables, terms, transcript)
    return proof, point, finals[: len(chunk_tabs)]


def claims_batching_verify(shapes, claims, proof, chunk_evals, transcript):
    """shapes: per polynomial (num_chunks, num_vars of the whole polynomial).
    Returns (ok, point)."""
    eq_points, evals = [], []
    max_vars = 0
    for (nch, nv), cls in zip(shapes, claims):
        b = nch.bit_length() - 1
        for point, ev in cls:
            point = _e2arr(point).reshape(-1, 2)
            transcript.append_scalars(_e2arr(ev).reshape(1, 2))
            eq_points.append(point[: len(point) - b])
            evals.append(_e2arr(ev))
        max_vars = max(max_vars, nv - b)
    challenge = transcript.append_and_sample(b"model_batching")
    claimed, acc = e2(0), e2(1)
    for ev in evals:
        claimed = e2_add(claimed, e2_mul(acc, ev))
        acc = e2_mul(acc, challenge)
    proof = _e2arr(proof)
    if proof.shape[0] != max_vars or proof.shape[1] != 3:
        return False, None
    bad, point, expected = sc_verify(claimed, proof, transcript)
    if bad:
        return False, point
    wit = [_e2arr(v) for v in _e2arr(chunk_evals).reshape(-1, 2)]
    for ep in eq_points:
        v = identity_eval(point[: len(ep)], ep) if len(ep) else e2(1)
        for r in point[len(ep):]:
            v = e2_mul(v, e2_sub(e2(1), r))
        wit.append(v)
    total = e2(0)
    for coeff, (a, b_) in _claims_batching_terms([s[0] for s in shapes], claims, challenge):
        total = e2_add(total, e2_mul(coeff, e2_mul(wit[a], wit[b_])))
    return bool((total == expected).all()), point


# ---- merging claims on one polynomial (zkml/src/iop/same_poly.rs:84-169) ----
def same_poly_prove(poly, claims, transcript):
    """claims: list of (point, eval).  Returns (proof, point, eval)."""
    poly = _e2arr(poly).reshape(-1, 2)
    a = transcript.read_challenges(len(claims))
    tables = [poly] + [eq_evals(p) for p, _ in claims]
    terms = [(a[i], [0, 1 + i]) for i in range(len(claims))]
    proof, point, finals = sc_prove(_nvars(poly), tables, terms, transcript)
    return proof, point, finals[0]


def same_poly_verify(num_vars, claims, proof, eval_, transcript):
    """Returns (ok, point)."""
    a = transcript.read_challenges(len(claims))
    y = e2(0)
    for (_, ev), ai in zip(claims, a):
        y = e2_add(y, e2_mul(_e2arr(ev), ai))
    proof = _e2arr(proof)
    if proof.shape[0] != num_vars or proof.shape[1] != 3:
        return False, None
    bad, point, expected = sc_verify(y, proof, transcript)
    if bad:
        return False, point
    computed = e2(0)
    for (pt, _), ai in zip(claims, a):
        computed = e2_add(computed, e2_mul(ai, identity_eval(pt, point)))
    return bool((e2_mul(_e2arr(eval_), computed) == expected).all()), point


# ---- sumcheck linking a lookup argument to its layer (zkml/src/lookup/operation) ----
# The expression is built as a polynomial in the witness tables with the challenges
# already substituted: a dict {sorted tuple of table indices: coefficient}.
# Pinned by tests/test_oracle_linking.py: the sum the proof opens with equals the
# protocol's statement recomputed entry by entry with Python integers.  Parity unpinned:
# the degree the prover declares when the top-degree monomials' coefficients are zero
# (here: the degree of the surviving monomials), and everything the sumcheck engine
# itself leaves unpinned (message layout, transcript bytes, binding order).
class _Poly:
    def __init__(self, terms=None):
        self.t = terms or {}

    @staticmethod
    def const(c):
        return _Poly({(): _e2arr(c)})

    @staticmethod
    def const_i64(x):
        return _Poly({(): e2(gl_from_i64(x))})

    @staticmethod
    def wit(i):
        return _Poly({(i,): e2(1)})

    def __add__(self, o):
        out = dict(self.t)
        for k, v in o.t.items():
            out[k] = e2_add(out[k], v) if k in out else v
        return _Poly(out)

    def __neg__(self):
        return _Poly({k: e2_sub(e2(0), v) for k, v in self.t.items()})

    def __sub__(self, o):
        return self + (-o)

    def __mul__(self, o):
        out = {}
        for ka, va in self.t.items():
            for kb, vb in o.t.items():
                k = tuple(sorted(ka + kb))
                v = e2_mul(va, vb)
                out[k] = e2_add(out[k], v) if k in out else v
        return _Poly(out)

    def terms(self):
        return [(v, list(k)) for k, v in sorted(self.t.items()) if v.any()]


def split_point(padded_shape, point):
    """Shape::split_point (zkml/src/shape.rs:475-496): the last dimension takes the lowest variables."""
    point = _e2arr(point).reshape(-1, 2)
    out, start = [None] * len(padded_shape), 0
    for a in reversed(range(len(padded_shape))):
        ln = max(0, (padded_shape[a] - 1).bit_length())
        out[a] = point[start:start + ln]
        start += ln
    assert start == len(point)
    return out


def eq_point_and_batching_challenges(shape, point):
    """Shape::compute_eq_point_and_batching_challenges (zkml/src/shape.rs:565-610): the variables of the last
    two dimensions form the eq point; the leading dimensions turn into one coefficient per 2-D chunk."""
    padded = [1 << max(0, (d - 1).bit_length()) for d in shape]
    skip = max(0, len(shape) - 2)
    eq_pt, bc = np.zeros((0, 2), dtype=np.uint64), [e2(1)]
    for i, (dp, size) in enumerate(zip(split_point(padded, point), shape)):
        if i < skip:
            ev = eq_evals(dp)[:size]
            bc = [e2_mul(c, e) for c in bc for e in ev]
        else:
            eq_pt = np.concatenate([dp, eq_pt])
    return eq_pt, bc


def _linking_chunks(cfg):
    n = 1
    for d in cfg["shape"][:max(0, len(cfg["shape"]) - 2)]:
        n *= d
    return n


def _linking_extra_per_chunk(cfg):
    return {"standard": 0, "softmax": 0, "glu": 1, "normalisation": 2}[cfg["variant"]]


def linking_expression(cfg, ch):
    """LookupVariant::build_full_sumcheck_expression with the challenges `ch` substituted
    (zkml/src/lookup/operation/variant.rs:55-348, 475-522).  cfg: variant ('standard', 'glu', 'softmax',
    'normalisation'), shape (unpadded input shape), value_chunks, zero_chunks, bit_size, signed, min_out,
    max_out, input_sign ('positive' / 'negative', unsigned tables), norm_sum, has_weight."""
    nvc, nz, bits = cfg["value_chunks"], cfg["zero_chunks"], cfg["bit_size"]
    chunks = _linking_chunks(cfg)
    per_chunk = nvc + nz
    total_out = chunks * per_chunk
    total_wit = chunks * _linking_extra_per_chunk(cfg) + total_out
    one, W, K = _Poly.const(e2(1)), _Poly.wit, _Poly.const_i64
    spow = lambda k: _Poly.const(_pow_e2(ch[0], k))
    out_eq, logup_eq, norm_eq = W(total_wit), W(total_wit + 1), W(total_wit + 2)
    final_dim_log = max(0, (cfg["shape"][-1] - 1).bit_length())
    pow_two = K(1 << final_dim_log)
    full = _Poly()
    for c in range(chunks):
        off = c * per_chunk
        # the value the chunk's lookups stand for, and the start of the linear combination (variant.rs:475-522)
        if nvc == 1:
            value, total, wo, sco = W(off), W(off) * spow(1), off + 1, 2
        else:
            value, total = K(-(1 << (nvc * bits - 1))), _Poly()
            for i in range(nvc):
                value = value + K(1 << (bits * i)) * (W(off + i) + K(1 << (bits - 1)))
                total = total + W(off + i) * spow(i + 1)
            wo, sco = off + nvc, 1 + nvc
        # zeroing chunks (variant.rs:95-220)
        sq_clamp = _Poly()
        if cfg["signed"]:
            prod = one
            for i in range(max(0, nz - 1)):
                prod = prod * W(wo + i)
                total = total + W(wo + i) * spow(sco + i)
            if nz:
                if nvc == 1:
                    cmin, cmax = cfg["min_out"], cfg["max_out"]
                else:
                    cmin, cmax = -(1 << (nvc * bits - 1)), (1 << (nvc * bits - 1)) - 1
                last, lower = W(wo - 1 + nz), prod
                omt = one - last * last
                prod = prod * omt
                total = total + last * spow(sco - 1 + nz)
                half = _Poly.const(e2_inv(e2(2)))
                first = last * (last + one) * half + (omt - lower * omt)
                second = last * (last - one) * half
                clamp = first * K(cmax) + second * K(cmin)
                if cfg["variant"] == "normalisation":
                    sq_clamp = first * K(cmax) * K(cmax) + second * K(cmin) * K(cmin)
            else:
                clamp = _Poly()
        else:
            prod = one
            for i in range(nz):
                prod = prod * W(wo + i)
                total = total + W(wo + i) * spow(sco + i)
            # without zeroing chunks the reference's clamping term is the constant one (variant.rs:200-203)
            clamp = K(cfg["max_out"] if cfg["input_sign"] == "positive" else cfg["min_out"]) if nz else one
        prod_expr = clamp + prod * value
        cc = _Poly.const(ch[1 + c])
        v = cfg["variant"]
        if v == "standard":
            e = cc * (out_eq * prod_expr + logup_eq * total)
        elif v == "glu":
            e = cc * (out_eq * prod_expr * W(total_out + c) + logup_eq * total)
        elif v == "softmax":
            nc = _Poly.const(ch[1 + chunks]) * pow_two
            e = cc * (out_eq * prod_expr + nc * (norm_eq * prod_expr) + logup_eq * total)
        else:
            sq_expr = sq_clamp + prod * value * value
            sumsq_c = _Poly.const(ch[1 + chunks]) * pow_two
            oeq = out_eq * W(total_wit + 3) if cfg["has_weight"] else out_eq
            part = oeq * prod_expr
            if cfg["norm_sum"]:
                part = part + _Poly.const(_pow_e2(ch[1 + chunks], 2)) * pow_two * (norm_eq * prod_expr)
            e = cc * (part + sumsq_c * (norm_eq * sq_expr)
                      + logup_eq * (total + _Poly.const(ch[2 + chunks]) * (W(total_out + c) * W(total_out + chunks + c))))
        full = full + e
    return full.terms()


def _linking_setup(cfg, last_claim_point, logup_point, transcript):
    eq_pt, bc = eq_point_and_batching_challenges(cfg["shape"], last_claim_point)
    ch = [transcript.append_and_sample(b"sum")] + bc
    if cfg["variant"] in ("softmax", "normalisation"):
        ch.append(transcript.append_and_sample(b"normalisation"))
    if cfg["variant"] == "normalisation":
        ch.append(transcript.append_and_sample(b"input"))
    logup_point = _e2arr(logup_point).reshape(-1, 2)
    eq_points = [eq_pt, logup_point]
    if cfg["variant"] in ("softmax", "normalisation"):
        fd = max(0, (cfg["shape"][-1] - 1).bit_length())
        half = e2_inv(e2(2))
        eq_points.append(np.concatenate([np.tile(half, (fd, 1)), logup_point[fd:]]))
    return eq_pt, ch, eq_points


def linking_prove(cfg, mles, transcript, last_claim_point, logup_point, weight=None):
    """LookupInputConfig::prove_linking_sumcheck (zkml/src/lookup/operation/inputs/proving.rs:26-114).
    Returns (proof, point, evaluations of `mles`, weight evaluation or None, batching challenges)."""
    eq_pt, ch, eq_points = _linking_setup(cfg, last_claim_point, logup_point, transcript)
    tables = [_e2arr(m).reshape(-1, 2) for m in mles] + [eq_evals(p) for p in eq_points]
    if weight is not None:
        tables.append(_e2arr(weight).reshape(-1, 2))
    terms = linking_expression(cfg, ch)
    proof, point, finals = sc_prove(len(eq_pt), tables, terms, transcript)
    return proof, point, finals[:len(mles)], (finals[-1] if weight is not None else None), ch


def linking_verify(cfg, initial_claim, proof, evaluations, weight_eval, transcript, last_claim_point, logup_point):
    """LookupInputConfig::verify_linking_sumcheck (inputs/verifying.rs:236-330) from the initial claim on
    (prepare_sumcheck_verification is the caller's).  Returns (ok, point, batching challenges)."""
    eq_pt, ch, eq_points = _linking_setup(cfg, last_claim_point, logup_point, transcript)
    terms = linking_expression(cfg, ch)
    degree = max(len(f) for _, f in terms)
    proof = _e2arr(proof)
    if proof.shape[0] != len(eq_pt) or proof.shape[1] != degree + 1:
        return False, None, ch
    bad, point, expected = sc_verify(initial_claim, proof, transcript)
    if bad:
        return False, point, ch
    wit = [_e2arr(v) for v in _e2arr(evaluations).reshape(-1, 2)] + [identity_eval(p, point) if len(p) else e2(1) for p in eq_points]
    if weight_eval is not None:
        wit.append(_e2arr(weight_eval))
    total = e2(0)
    for coeff, fs in terms:
        v = coeff
        for f in fs:
            v = e2_mul(v, wit[f])
        total = e2_add(total, v)
    return bool((total == expected).all()), point, ch

# ---------------------------------------------------------------------------
# EinSum::prove_internal (zkml/src/layers/einsum/prove.rs:138-316) restated with the pieces above: axis
# classification, partial evaluation of both sides, the batched sumcheck over the contracted axes, the
# input claims, the aggregation sumcheck when several operations share the left-hand side, and the bias
# claims (prove.rs:191-214, axis.rs:582-637).  ops: (lhs axes, rhs axes, output axes[, bias axes]) as strings.
# ---------------------------------------------------------------------------
AXIS_CONTRACTED, AXIS_OUTER, AXIS_STACKED = 0, 1, 2


def _pad_shape(shape):
    return [1 << max(0, (int(d) - 1).bit_length()) for d in shape]


def _pad_tensor(t):
    out = np.zeros(_pad_shape(t.shape), dtype=np.int64)
    out[tuple(slice(0, d) for d in t.shape)] = t
    return out


def einsum_prove(ops, lhs, rhs, claims, label=b"m2vec", biases=None):
    """prove_internal restated with the checker's pieces (einsum/prove.rs:138-316), one or more RHS; a bias gives a
    claim of its own, its padded tensor's MLE at the slices of the output claim's point that its axes name
    (prove.rs:191-214, axis.rs:582-637)."""
    R = len(ops)
    tr = OracleTranscript(label)
    lp, lpad = _pad_tensor(lhs), _pad_shape(lhs.shape)

    def classify(op, ch):
        l, r, o = ch in op[0], ch in op[1], ch in op[2]
        return AXIS_STACKED if (l and r and o) else AXIS_CONTRACTED if (l and r) else AXIS_OUTER

    def split(shape, point):
        out, start = [None] * len(shape), 0
        for a in reversed(range(len(shape))):
            ln = max(0, (shape[a] - 1).bit_length())
            out[a] = point[start:start + ln]
            start += ln
        return out

    def reconstruct(fixes, pts, sc_point, shape):
        out, skip = [], 0
        for a in reversed(range(len(fixes))):
            if fixes[a] == AXIS_CONTRACTED:
                ln = max(0, (shape[a] - 1).bit_length())
                out.append(sc_point[skip:skip + ln])
                skip += ln
            else:
                out.append(pts[a])
        return np.concatenate(out) if out else np.zeros((0, 2), np.uint64)

    lfix, rfix, lpts, rpts, ltabs, rtabs, coeffs, bias_claims = [], [], [], [], [], [], [], []
    for r, op in enumerate(ops):
        rpad = _pad_shape(rhs[r].shape)
        out_shape = [lpad[op[0].index(c)] if c in op[0] else rpad[op[1].index(c)] for c in op[2]]
        sl = split(out_shape, claims[r][0])
        if biases is not None and biases[r] is not None:
            bpt = [sl[op[2].index(c)] for c in reversed(op[3])]
            bpt = np.concatenate(bpt) if bpt else np.zeros((0, 2), np.uint64)
            bias_claims.append((r, bpt, mle_evaluate(embed_i64(_pad_tensor(biases[r]).reshape(-1)), bpt)))
        lk = [classify(op, c) for c in op[0]]
        rk = [classify(op, c) for c in op[1]]
        lpt = [None if k == AXIS_CONTRACTED else sl[op[2].index(c)] for c, k in zip(op[0], lk)]
        rpt = [None if k == AXIS_CONTRACTED else sl[op[2].index(c)] for c, k in zip(op[1], rk)]
        lfix.append(lk); rfix.append(rk); lpts.append(lpt); rpts.append(rpt)
        ltabs.append(partial_eval(lp, lpad, list(lhs.shape), lk, lpt))
        rtabs.append(partial_eval(_pad_tensor(rhs[r]), rpad, list(rhs[r].shape), rk, rpt))
        coeffs.append(stacking_coeffs(lpad, list(lhs.shape), lk, lpt))
    S = ltabs[0].shape[0]
    gamma = tr.append_and_sample(b"batching_challenge")
    tabs = [t for v in ltabs for t in v] + [t for v in rtabs for t in v]
    nv = int(tabs[0].shape[0]).bit_length() - 1
    terms, gpow = [], np.array([1, 0], np.uint64)
    for r in range(R):
        for j in range(S):
            terms.append((e2_mul(gpow, coeffs[r][j]), [r * S + j, R * S + r * S + j]))
        gpow = e2_mul(gpow, gamma)
    proof, point, finals = sc_prove(nv, tabs, terms, tr)
    half = len(finals) // 2
    out_claims = []
    for r in range(R):
        ev = np.zeros(2, np.uint64)
        for j in range(S):
            ev = e2_add(ev, e2_mul(coeffs[r][j], finals[half + r * S + j]))
        out_claims.append((reconstruct(rfix[r], rpts[r], point, _pad_shape(rhs[r].shape)), ev))
    agg = None
    if R > 1:
        eqs = [eq_evals(reconstruct(lfix[r], lpts[r], point, lpad)) for r in range(R)]
        g2 = tr.append_and_sample(b"input_batching_challenge")
        aterms, gp = [], np.array([1, 0], np.uint64)
        for r in range(R):
            aterms.append((gp, [0, 1 + r]))
            gp = e2_mul(gp, g2)
        full = embed_i64(lp.reshape(-1))
        agg, apoint, afinals = sc_prove(int(full.shape[0]).bit_length() - 1, [full] + eqs, aterms, tr)
        lhs_claim = (apoint, afinals[0])
    else:
        ev = np.zeros(2, np.uint64)
        for j in range(S):
            ev = e2_add(ev, e2_mul(coeffs[0][j], finals[j]))
        lhs_claim = (reconstruct(lfix[0], lpts[0], point, lpad), ev)
    return dict(proof=proof, evaluations=finals, aggregation_proof=agg, claims=[lhs_claim] + out_claims, bias_claims=bias_claims), tr


def num_threads():
    return lib().orc_num_threads()
