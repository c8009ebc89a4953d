"""MI355X sumcheck prover: Python bindings of the C ABI (libdpsumcheck.so, the
HIP library) and of the C++ host mirror (libdpsc_host.so: transcript,
prove/verify loops, einsum and LogUp drivers).

The directory name carries a hyphen, so load it with
``importlib.import_module("deep-prove_amd")``.

There is no CPU implementation behind these calls: if the HIP library has not
been built, importing this package fails; on a machine without a GPU
``Context()`` fails.  Extension-field values cross as numpy uint64 arrays whose
last axis is (c0, c1).
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_DIR = os.path.join(_HERE, "lib")
P = 0xFFFFFFFF00000001
MAX_FACTORS = 8
AXIS_CONTRACTED, AXIS_OUTER, AXIS_STACKED = 0, 1, 2
KIND_BASE, KIND_EXT2, KIND_I64, KIND_I16 = 0, 1, 2, 3
KERNELS = ["eval_first", "fold_eval", "eval_terms", "fold", "eq", "axis_dot", "logup", "finalize", "tail"]


class DpsError(RuntimeError):
    def __init__(self, status, msg):
        super().__init__(f"[status {status}] {msg}")
        self.status = status


def _load(name):
    path = os.path.join(LIB_DIR, name)
    if not os.path.exists(path):
        raise ImportError(f"{path} is missing: build it first (python -c 'import __graft_entry__ as g; g.build()')")
    return C.CDLL(path, mode=C.RTLD_GLOBAL)


dev = _load("libdpsumcheck.so")
host = _load("libdpsc_host.so")


class Term(C.Structure):
    _fields_ = [("coeff", C.c_uint64 * 2), ("n_factors", C.c_uint32), ("factors", C.c_uint32 * MAX_FACTORS)]


_vp, _u32, _u64, _i32 = C.c_void_p, C.c_uint32, C.c_uint64, C.c_int32
dev.dps_last_error.restype = C.c_char_p
dev.dps_last_error.argtypes = [_vp]
dev.dps_status_str.restype = C.c_char_p
dev.dps_kernel_name.restype = C.c_char_p
host.dph_last_error.restype = C.c_char_p
host.dph_tr_new.restype = _vp
host.dph_tr_new.argtypes = [C.c_char_p]
host.dph_tr_clone.restype = _vp
host.dph_tr_clone.argtypes = [_vp]
for _f, _a in [("dph_tr_free", [_vp]), ("dph_tr_append_message", [_vp, C.c_char_p]),
               ("dph_tr_append_bytes", [_vp, C.c_char_p, C.c_size_t]), ("dph_tr_append_u64", [_vp, _u64]),
               ("dph_tr_append_scalars", [_vp, _vp, C.c_size_t]), ("dph_tr_challenge_scalar", [_vp, _vp]),
               ("dph_tr_append_and_sample", [_vp, C.c_char_p, _vp]), ("dph_tr_state", [_vp, _vp, _vp]),
               ("dph_blake3", [C.c_char_p, C.c_size_t, _vp])]:
    getattr(host, _f).restype = None
    getattr(host, _f).argtypes = _a

# every dps_* entry point takes pointers and integers; declare the ones whose
# integer arguments are 64-bit so that ctypes does not truncate them
dev.dps_mle_from_i64.argtypes = [_vp, _vp, _u64, _u32, _vp]
dev.dps_tensor_from_i64.argtypes = [_vp, _vp, _u64, _vp]
dev.dps_tensor_from_i16.argtypes = [_vp, _vp, _u64, _vp]
dev.dps_mle_from_tensor.restype = _i32
dev.dps_mle_from_tensor.argtypes = [_vp, _vp, _vp, _vp, _u32, _vp]
dev.dps_mle_wrap_device.argtypes = [_vp, _i32, _vp, _vp, _u64, _vp]
dev.dps_mle_view.argtypes = [_vp, _u64, _u32, _vp]
dev.dps_eq_build_many.restype = _i32
dev.dps_eq_build_many.argtypes = [_vp, _vp, _vp, _u32, _vp]
dev.dps_mle_zero_pad.restype = _i32
dev.dps_mle_zero_pad.argtypes = [_vp, _u32, _vp]
dev.dps_debug_field_op.argtypes = [_vp, _i32, _vp, _vp, _u64, _vp]
dev.dps_debug_copy.restype = _i32
dev.dps_debug_copy.argtypes = [_vp, _u64, _u32, _vp]
dev.dps_debug_read.restype = _i32
dev.dps_debug_read.argtypes = [_vp, _u64, _u32, _vp]
for _f in ["dps_ctx_create", "dps_ctx_destroy", "dps_ctx_sync", "dps_mle_from_base", "dps_mle_from_ext2", "dps_mle_info",
           "dps_mle_download", "dps_mle_free", "dps_eq_build", "dps_mle_evaluate", "dps_mle_fix_low", "dps_mle_fix_high",
           "dps_partial_eval", "dps_sc_begin", "dps_sc_set_claim", "dps_sc_degree", "dps_sc_round", "dps_sc_finish", "dps_sc_abort", "dps_sc_free",
           "dps_sc_prove", "dps_logup_build", "dps_logup_num_layers", "dps_logup_layer", "dps_logup_outputs",
           "dps_logup_free", "dps_profile_enable", "dps_profile_reset", "dps_profile_read"]:
    getattr(dev, _f).restype = _i32
dev.dps_ctx_create.argtypes = [_i32, _vp]
dev.dps_ctx_destroy.argtypes = [_vp]
dev.dps_ctx_sync.argtypes = [_vp]
dev.dps_mle_from_base.argtypes = [_vp, _vp, _u32, _vp]
dev.dps_mle_from_ext2.argtypes = [_vp, _vp, _vp, _u32, _vp]
dev.dps_mle_info.argtypes = [_vp, _vp, _vp]
dev.dps_mle_download.argtypes = [_vp, _vp, _vp]
dev.dps_mle_free.argtypes = [_vp]
dev.dps_eq_build.argtypes = [_vp, _vp, _u32, _vp]
dev.dps_mle_evaluate.argtypes = [_vp, _vp, _vp, _u32, _vp]
dev.dps_mle_evaluate_noalloc.restype = _i32
dev.dps_mle_evaluate_noalloc.argtypes = [_vp, _vp, _vp, _u32, _vp]
dev.dps_mle_fix_low.argtypes = [_vp, _vp, _vp, _u32, _vp]
dev.dps_mle_fix_high.argtypes = [_vp, _vp, _vp, _u32, _vp]
dev.dps_partial_eval.argtypes = [_vp, _vp, _vp, _vp, _u32, _vp, _vp, _vp, _u32, _vp]
dev.dps_sc_begin.argtypes = [_vp, _u32, _vp, _u32, _vp, _u32, _vp]
dev.dps_sc_degree.argtypes = [_vp, _vp]
dev.dps_sc_set_claim.argtypes = [_vp, _vp]
dev.dps_sc_round.argtypes = [_vp, _vp, _vp]
dev.dps_sc_finish.argtypes = [_vp, _vp, _vp]
dev.dps_sc_free.argtypes = [_vp]
dev.dps_sc_prove.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp]
dev.dps_logup_build.argtypes = [_vp, _vp, _u32, _vp, _vp, _vp, _vp]
dev.dps_logup_num_layers.argtypes = [_vp, _vp]
dev.dps_logup_layer.argtypes = [_vp, _u32, _vp, _vp]
dev.dps_logup_outputs.argtypes = [_vp, _vp]
dev.dps_logup_free.argtypes = [_vp]
dev.dps_profile_enable.argtypes = [_vp, _i32]
dev.dps_profile_reset.argtypes = [_vp]
dev.dps_profile_read.argtypes = [_vp, _i32, _vp, _vp, _vp, _vp, _vp, _vp]
dev.dps_ctx_pool_info.restype = _i32
dev.dps_ctx_pool_info.argtypes = [_vp, _vp, _vp, _vp]
dev.dps_device_set_resident_budget.restype = _i32
dev.dps_device_set_resident_budget.argtypes = [_i32, _i32]
dev.dps_device_resident_budget.restype = _i32
dev.dps_device_resident_budget.argtypes = [_i32, _vp, _vp]
host.dph_sumcheck_prove.restype = _i32
host.dph_sumcheck_prove.argtypes = [_vp, _u32, _vp, _u32, _vp, _u32, _vp, _vp, _vp, _vp, _vp]
host.dph_sumcheck_prove_claimed.restype = _i32
host.dph_sumcheck_prove_claimed.argtypes = [_vp, _u32, _vp, _u32, _vp, _u32, _vp, _vp, _vp, _vp, _vp, _vp]
host.dph_sumcheck_verify.restype = _i32
host.dph_sumcheck_verify.argtypes = [_vp, _vp, _u32, _u32, _vp, _vp, _vp]


def set_resident_budget(device, compute_units):
    """Cap, in compute units, on what the launches that wait on the GPU (resident launches, launches made ahead) of all
    contexts of this process may hold on `device` together; -1: the whole device (the default), 0: none ever waits
    (dps_device_set_resident_budget)."""
    rc = dev.dps_device_set_resident_budget(device, compute_units)
    if rc != 0:
        raise DpsError(rc, "dps_device_set_resident_budget")


def resident_budget(device):
    """(compute units held now by waiting launches, cap in force) on `device` (dps_device_resident_budget)"""
    used, cap = C.c_int32(0), C.c_int32(0)
    rc = dev.dps_device_resident_budget(device, C.byref(used), C.byref(cap))
    if rc != 0:
        raise DpsError(rc, "dps_device_resident_budget")
    return used.value, cap.value


def _ptr(a):
    return a.ctypes.data_as(_vp)


def _e2(x):
    a = np.ascontiguousarray(x, dtype=np.uint64)
    assert a.shape[-1] == 2, a.shape
    return a


def make_terms(terms):
    """terms: iterable of (coeff (c0, c1), [table indices])."""
    terms = list(terms)
    arr = (Term * max(1, len(terms)))()
    for i, (coeff, factors) in enumerate(terms):
        c = _e2(coeff)
        arr[i].coeff[0], arr[i].coeff[1] = int(c[0]), int(c[1])
        arr[i].n_factors = len(factors)
        for k, f in enumerate(factors):
            arr[i].factors[k] = f
    return arr, len(terms)


class Transcript:
    """Blake3Transcript of the host mirror."""

    def __init__(self, label=b"m2vec", _raw=None):
        self._t = _raw if _raw is not None else host.dph_tr_new(label)

    def __del__(self):
        if getattr(self, "_t", None):
            host.dph_tr_free(self._t)
            self._t = None

    def clone(self):
        return Transcript(_raw=host.dph_tr_clone(self._t))

    def append_message(self, label: bytes):
        host.dph_tr_append_message(self._t, label)

    def append_bytes(self, data: bytes):
        host.dph_tr_append_bytes(self._t, data, len(data))

    def append_u64(self, x):
        host.dph_tr_append_u64(self._t, x)

    def append_scalars(self, xs):
        xs = _e2(xs).reshape(-1, 2)
        host.dph_tr_append_scalars(self._t, _ptr(xs), xs.shape[0])

    def challenge_scalar(self):
        out = np.zeros(2, dtype=np.uint64)
        host.dph_tr_challenge_scalar(self._t, _ptr(out))
        return out

    def append_and_sample(self, label: bytes):
        out = np.zeros(2, dtype=np.uint64)
        host.dph_tr_append_and_sample(self._t, label, _ptr(out))
        return out

    def read_challenges(self, n):
        return np.stack([self.challenge_scalar() for _ in range(n)]) if n else np.zeros((0, 2), np.uint64)

    def state(self):
        st = (C.c_uint8 * 32)()
        n = C.c_uint32(0)
        host.dph_tr_state(self._t, st, C.byref(n))
        return bytes(st), int(n.value)


def blake3(data: bytes) -> bytes:
    out = (C.c_uint8 * 32)()
    host.dph_blake3(data, len(data), out)
    return bytes(out)


class Mle:
    """A table in HBM (owned, borrowed or a view)."""

    def __init__(self, ctx, handle):
        self.ctx, self._h = ctx, handle

    def __del__(self):
        self.free()

    def free(self):
        if getattr(self, "_h", None) and self.ctx._c:
            dev.dps_mle_free(self._h)
        self._h = None

    @property
    def handle(self):
        return self._h

    def info(self):
        k, n = _i32(0), _u64(0)
        self.ctx._chk(dev.dps_mle_info(self._h, C.byref(k), C.byref(n)), "dps_mle_info")
        return int(k.value), int(n.value)

    def __len__(self):
        return self.info()[1]

    @property
    def kind(self):
        return self.info()[0]

    def download(self):
        """(len, 2) uint64 for field tables; int64 vector for raw tensors."""
        kind, n = self.info()
        c0 = np.zeros(n, dtype=np.uint64)
        c1 = np.zeros(n, dtype=np.uint64)
        self.ctx._chk(dev.dps_mle_download(self._h, _ptr(c0), _ptr(c1)), "dps_mle_download")
        if kind in (KIND_I64, KIND_I16):
            return c0.view(np.int64)
        return np.stack([c0, c1], axis=-1)

    def view(self, offset, n_vars):
        h = _vp()
        self.ctx._chk(dev.dps_mle_view(self._h, offset, n_vars, C.byref(h)), "dps_mle_view")
        return Mle(self.ctx, h)

    def zero_pad(self, n_vars):
        """the table as a sumcheck over n_vars variables reads it: 0 wherever an added variable is 1"""
        h = _vp()
        self.ctx._chk(dev.dps_mle_zero_pad(self._h, n_vars, C.byref(h)), "dps_mle_zero_pad")
        return Mle(self.ctx, h)

    def evaluate(self, point):
        point = _e2(point).reshape(-1, 2)
        out = np.zeros(2, dtype=np.uint64)
        self.ctx._chk(dev.dps_mle_evaluate(self.ctx._c, self._h, _ptr(point), point.shape[0], _ptr(out)), "dps_mle_evaluate")
        return out

    def evaluate_noalloc(self, point):
        """the same value through the entry point that allocates nothing (dps_mle_evaluate_noalloc)"""
        point = _e2(point).reshape(-1, 2)
        out = np.zeros(2, dtype=np.uint64)
        self.ctx._chk(dev.dps_mle_evaluate_noalloc(self.ctx._c, self._h, _ptr(point), point.shape[0], _ptr(out)), "dps_mle_evaluate_noalloc")
        return out

    def fix_low(self, point):
        point = _e2(point).reshape(-1, 2)
        h = _vp()
        self.ctx._chk(dev.dps_mle_fix_low(self.ctx._c, self._h, _ptr(point), point.shape[0], C.byref(h)), "dps_mle_fix_low")
        return Mle(self.ctx, h)

    def fix_high(self, point):
        point = _e2(point).reshape(-1, 2)
        h = _vp()
        self.ctx._chk(dev.dps_mle_fix_high(self.ctx._c, self._h, _ptr(point), point.shape[0], C.byref(h)), "dps_mle_fix_high")
        return Mle(self.ctx, h)


class Logup:
    def __init__(self, ctx, handle):
        self.ctx, self._h = ctx, handle

    def __del__(self):
        if getattr(self, "_h", None) and self.ctx._c:
            dev.dps_logup_free(self._h)
        self._h = None

    def num_layers(self):
        n = _u32(0)
        self.ctx._chk(dev.dps_logup_num_layers(self._h, C.byref(n)), "dps_logup_num_layers")
        return int(n.value)

    def layer(self, k):
        a, b = _vp(), _vp()
        self.ctx._chk(dev.dps_logup_layer(self._h, k, C.byref(a), C.byref(b)), "dps_logup_layer")
        return Mle(self.ctx, a), Mle(self.ctx, b)

    def outputs(self):
        out = np.zeros((4, 2), dtype=np.uint64)
        self.ctx._chk(dev.dps_logup_outputs(self._h, _ptr(out)), "dps_logup_outputs")
        return out


class Session:
    """Round-by-round access to a sumcheck (dps_sc_begin / round / finish)."""

    def __init__(self, ctx, n_vars, mles, terms):
        self.ctx, self.n_vars, self.n_mles = ctx, n_vars, len(mles)
        self._keep = list(mles)
        hs = (_vp * max(1, len(mles)))(*[m.handle for m in mles])
        tarr, nt = make_terms(terms)
        h = _vp()
        ctx._chk(dev.dps_sc_begin(ctx._c, n_vars, hs, len(mles), tarr, nt, C.byref(h)), "dps_sc_begin")
        self._h = h
        d = _u32(0)
        dev.dps_sc_degree(h, C.byref(d))
        self.degree = int(d.value)

    def __del__(self):
        if getattr(self, "_h", None) and self.ctx._c:
            dev.dps_sc_free(self._h)
        self._h = None

    def set_claim(self, claim):
        """The value of the whole sum, if known: round 1 then takes p(1) from it (dps_sc_set_claim)."""
        c = _e2(claim)
        self.ctx._chk(dev.dps_sc_set_claim(self._h, _ptr(c)), "dps_sc_set_claim")

    def abort(self):
        self.ctx._chk(dev.dps_sc_abort(self._h), "dps_sc_abort")

    def round(self, challenge=None):
        out = np.zeros((self.degree + 1, 2), dtype=np.uint64)
        ch = None if challenge is None else _e2(challenge)
        self.ctx._chk(dev.dps_sc_round(self._h, None if ch is None else _ptr(ch), _ptr(out)), "dps_sc_round")
        return out

    def finish(self, challenge=None):
        out = np.zeros((max(1, self.n_mles), 2), dtype=np.uint64)
        ch = None if challenge is None else _e2(challenge)
        self.ctx._chk(dev.dps_sc_finish(self._h, None if ch is None else _ptr(ch), _ptr(out)), "dps_sc_finish")
        return out[: self.n_mles]


class Context:
    """One GPU context: a HIP stream plus a device memory pool."""

    def __init__(self, device=0):
        self._c = None
        c = _vp()
        rc = dev.dps_ctx_create(device, C.byref(c))
        if rc != 0:
            raise DpsError(rc, "dps_ctx_create failed (no usable GPU?): " + dev.dps_status_str(rc).decode())
        self._c = c

    def __del__(self):
        self.close()

    def close(self):
        if getattr(self, "_c", None):
            dev.dps_ctx_destroy(self._c)
        self._c = None

    def _chk(self, rc, what):
        if rc != 0:
            raise DpsError(rc, f"{what}: {dev.dps_status_str(rc).decode()}: {dev.dps_last_error(self._c).decode()}")

    def _chk_host(self, rc, what):
        if rc != 0:
            raise DpsError(rc, f"{what}: {host.dph_last_error().decode()}")

    def pool_info(self):
        """(device blocks handed out, blocks cached for reuse, bytes of both) (dps_ctx_pool_info)"""
        a, b, c = C.c_uint64(0), C.c_uint64(0), C.c_uint64(0)
        self._chk(dev.dps_ctx_pool_info(self._c, C.byref(a), C.byref(b), C.byref(c)), "dps_ctx_pool_info")
        return a.value, b.value, c.value

    def sync(self):
        self._chk(dev.dps_ctx_sync(self._c), "dps_ctx_sync")

    # ---- tables ----
    def mle_from_base(self, v):
        v = np.ascontiguousarray(v, dtype=np.uint64)
        nv = int(v.size).bit_length() - 1
        assert 1 << nv == v.size, "length must be a power of two"
        h = _vp()
        self._chk(dev.dps_mle_from_base(self._c, _ptr(v), nv, C.byref(h)), "dps_mle_from_base")
        return Mle(self, h)

    def mle_from_ext2(self, v):
        v = _e2(v).reshape(-1, 2)
        nv = int(v.shape[0]).bit_length() - 1
        assert 1 << nv == v.shape[0], "length must be a power of two"
        c0, c1 = np.ascontiguousarray(v[:, 0]), np.ascontiguousarray(v[:, 1])
        h = _vp()
        self._chk(dev.dps_mle_from_ext2(self._c, _ptr(c0), _ptr(c1), nv, C.byref(h)), "dps_mle_from_ext2")
        return Mle(self, h)

    def mle_from_i64(self, v, n_vars=None):
        v = np.ascontiguousarray(v, dtype=np.int64).reshape(-1)
        if n_vars is None:
            n_vars = max(0, int(v.size - 1).bit_length())
        h = _vp()
        self._chk(dev.dps_mle_from_i64(self._c, _ptr(v), v.size, n_vars, C.byref(h)), "dps_mle_from_i64")
        return Mle(self, h)

    def tensor_from_i64(self, v):
        v = np.ascontiguousarray(v, dtype=np.int64).reshape(-1)
        h = _vp()
        self._chk(dev.dps_tensor_from_i64(self._c, _ptr(v), v.size, C.byref(h)), "dps_tensor_from_i64")
        return Mle(self, h)

    def tensor_from_i16(self, v):
        """the quantised tensor in 16-bit storage (values must fit int16)"""
        v = np.ascontiguousarray(v)
        if v.dtype != np.int16:
            if v.size and (v.min() < -32768 or v.max() > 32767):
                raise ValueError("tensor_from_i16: values do not fit 16 bits")
            v = v.astype(np.int16)
        v = v.reshape(-1)
        h = _vp()
        self._chk(dev.dps_tensor_from_i16(self._c, _ptr(v), v.size, C.byref(h)), "dps_tensor_from_i16")
        return Mle(self, h)

    def mle_from_tensor(self, tensor, padded_dims, unpadded_dims):
        """the padded tensor as a base-field table (zero outside the unpadded region), built on the device"""
        nd = len(padded_dims)
        pd, ud = (_u64 * nd)(*padded_dims), (_u64 * nd)(*unpadded_dims)
        h = _vp()
        self._chk(dev.dps_mle_from_tensor(self._c, tensor.handle, pd, ud, nd, C.byref(h)), "dps_mle_from_tensor")
        return Mle(self, h)

    def wrap_device(self, kind, ptr_c0, ptr_c1, length):
        h = _vp()
        self._chk(dev.dps_mle_wrap_device(self._c, kind, ptr_c0, ptr_c1, length, C.byref(h)), "dps_mle_wrap_device")
        return Mle(self, h)

    def eq_build(self, point):
        point = _e2(point).reshape(-1, 2)
        h = _vp()
        self._chk(dev.dps_eq_build(self._c, _ptr(point), point.shape[0], C.byref(h)), "dps_eq_build")
        return Mle(self, h)

    def eq_build_many(self, points):
        """one eq table per point; the small ones come out of a single launch"""
        pts = [np.ascontiguousarray(_e2(p).reshape(-1, 2)) for p in points]
        n = len(pts)
        ptrs = (_vp * max(1, n))(*[p.ctypes.data for p in pts])
        ms = (_u32 * max(1, n))(*[p.shape[0] for p in pts])
        hs = (_vp * max(1, n))()
        self._chk(dev.dps_eq_build_many(self._c, ptrs, ms, n, hs), "dps_eq_build_many")
        return [Mle(self, _vp(hs[i])) for i in range(n)]

    def partial_eval(self, tensor, padded_dims, unpadded_dims, kinds, points):
        nd = len(padded_dims)
        pd = (_u64 * nd)(*padded_dims)
        ud = (_u64 * nd)(*unpadded_dims)
        kd = (_i32 * nd)(*kinds)
        keep = [None if p is None else _e2(p).reshape(-1, 2) for p in points]
        pts = (_vp * nd)(*[None if p is None else p.ctypes.data for p in keep])
        cap = 1
        for d, k in zip(unpadded_dims, kinds):
            if k == AXIS_STACKED:
                cap *= d
        out = (_vp * cap)()
        n = _u32(0)
        self._chk(dev.dps_partial_eval(self._c, tensor.handle, pd, ud, nd, kd, pts, out, cap, C.byref(n)), "dps_partial_eval")
        return [Mle(self, _vp(out[i])) for i in range(n.value)]

    # ---- sumcheck ----
    def session(self, n_vars, mles, terms):
        return Session(self, n_vars, mles, terms)

    def sumcheck_prove(self, n_vars, mles, terms, transcript):
        """IOPProverState::prove with the native transcript.
        Returns (proof[n_vars, d+1, 2], point[n_vars, 2], final_evals[n_mles, 2])."""
        hs = (_vp * max(1, len(mles)))(*[m.handle for m in mles])
        tarr, nt = make_terms(terms)
        degree = max((len(f) for _, f in terms), default=0)
        proof = np.zeros((n_vars, degree + 1, 2), dtype=np.uint64)
        point = np.zeros((n_vars, 2), dtype=np.uint64)
        finals = np.zeros((max(1, len(mles)), 2), dtype=np.uint64)
        d = _u32(0)
        self._chk_host(host.dph_sumcheck_prove(self._c, n_vars, hs, len(mles), tarr, nt, transcript._t, _ptr(proof), _ptr(point),
                                               _ptr(finals), C.byref(d)), "dph_sumcheck_prove")
        return proof, point, finals[: len(mles)]

    def sumcheck_prover(self, n_vars, mles, terms, claim=None):
        """The same proof called repeatedly: returns prove(transcript) with the handles and terms already marshalled
        (a caller in a compiled language has no such per-call cost; from Python it is 10 us a proof).
        `claim`: the value of the whole sum when the caller holds it (the claim a layer prover is reducing)."""
        hs = (_vp * max(1, len(mles)))(*[m.handle for m in mles])
        tarr, nt = make_terms(terms)
        degree = max((len(f) for _, f in terms), default=0)
        n_mles = len(mles)
        keep = list(mles)
        d = _u32(0)
        dref = C.byref(d)
        cl = None if claim is None else np.ascontiguousarray(_e2(claim))
        clp = None if cl is None else cl.ctypes.data

        # (the three results share one buffer: taking an array's address costs more than making the array)
        n_proof, n_point = n_vars * (degree + 1) * 2, n_vars * 2
        n_words = n_proof + n_point + max(1, n_mles) * 2
        call, ctx_c = host.dph_sumcheck_prove_claimed, self._c

        def prove(transcript):
            buf = np.zeros(n_words, dtype=np.uint64)
            base = buf.ctypes.data
            rc = call(ctx_c, n_vars, hs, n_mles, tarr, nt, clp, transcript._t, base, base + 8 * n_proof, base + 8 * (n_proof + n_point), dref)
            if rc != 0:
                self._chk_host(rc, "dph_sumcheck_prove")
            return (buf[:n_proof].reshape(n_vars, degree + 1, 2), buf[n_proof:n_proof + n_point].reshape(n_vars, 2),
                    buf[n_proof + n_point:n_proof + n_point + 2 * n_mles].reshape(n_mles, 2))

        prove.keep = (keep, cl)
        return prove

    def sumcheck_verify(self, claimed_sum, proof, transcript):
        proof = _e2(proof)
        n_vars, npts = proof.shape[0], proof.shape[1]
        cs = _e2(claimed_sum)
        point = np.zeros((n_vars, 2), dtype=np.uint64)
        expected = np.zeros(2, dtype=np.uint64)
        rc = host.dph_sumcheck_verify(_ptr(cs), _ptr(proof), n_vars, npts - 1, transcript._t, _ptr(point), _ptr(expected))
        return rc, point, expected

    # ---- LogUp ----
    def logup_build(self, cols, numer, c, beta):
        hs = (_vp * len(cols))(*[m.handle for m in cols])
        cc, bb = _e2(c), _e2(beta)
        h = _vp()
        self._chk(dev.dps_logup_build(self._c, hs, len(cols), None if numer is None else numer.handle, _ptr(cc), _ptr(bb), C.byref(h)),
                  "dps_logup_build")
        return Logup(self, h)

    # ---- measurement ----
    def profile(self, on=True):
        self._chk(dev.dps_profile_enable(self._c, 1 if on else 0), "dps_profile_enable")

    def profile_reset(self):
        self._chk(dev.dps_profile_reset(self._c), "dps_profile_reset")

    def profile_read(self):
        out = {}
        for k, name in enumerate(KERNELS):
            n, mn = _u64(0), _u64(0)
            ms, by, mms, mby = C.c_double(0), C.c_double(0), C.c_double(0), C.c_double(0)
            self._chk(dev.dps_profile_read(self._c, k, C.byref(n), C.byref(ms), C.byref(by), C.byref(mn), C.byref(mms), C.byref(mby)),
                      "dps_profile_read")
            out[name] = dict(launches=n.value, ms=ms.value, bytes=by.value, max_launches=mn.value, max_ms=mms.value, max_bytes=mby.value,
                             symbol=dev.dps_kernel_name(k).decode())
        return out

    def field_op(self, op, a, b):
        a, b = _e2(a).reshape(-1, 2), _e2(b).reshape(-1, 2)
        n = a.shape[0]
        aa = np.ascontiguousarray(np.concatenate([a[:, 0], a[:, 1]]))
        bb = np.ascontiguousarray(np.concatenate([b[:, 0], b[:, 1]]))
        out = np.zeros(2 * n, dtype=np.uint64)
        self._chk(dev.dps_debug_field_op(self._c, op, _ptr(aa), _ptr(bb), n, _ptr(out)), "dps_debug_field_op")
        return np.stack([out[:n], out[n:]], axis=-1)

    def copy_ms(self, n_bytes, reps=10):
        """average duration of a plain device copy of n_bytes (the bandwidth yardstick)"""
        ms = C.c_double(0)
        self._chk(dev.dps_debug_copy(self._c, n_bytes, reps, C.byref(ms)), "dps_debug_copy")
        return ms.value


def _read_ms(self, n_bytes, reps=10):
    """average duration of a launch that only streams n_bytes in (the yardstick of read-only launches)"""
    ms = C.c_double(0)
    self._chk(dev.dps_debug_read(self._c, n_bytes, reps, C.byref(ms)), "dps_debug_read")
    return ms.value


Context.read_ms = _read_ms


# ---- einsum and LogUp drivers of the host mirror ----
host.dph_einsum_prove.restype = _i32
host.dph_einsum_prove.argtypes = [_vp, _u32, _vp, _vp, _vp, _u32, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _u64, _vp]
host.dph_einsum_prove_resident.restype = _i32
host.dph_einsum_prove_resident.argtypes = host.dph_einsum_prove.argtypes
host.dph_logup_batch_prove.restype = _i32
host.dph_logup_batch_prove.argtypes = [_vp, _u32, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _u64, _vp]
host.dph_logup_batch_verify.restype = _i32
host.dph_logup_batch_verify.argtypes = [_u32, _vp, _vp, _vp, _vp, _i32, _vp, _u64, _vp, _vp, _vp]


def _parse_proof(words, pos):
    rounds, npts = int(words[pos]), int(words[pos + 1])
    pos += 2
    proof = words[pos:pos + 2 * rounds * npts].reshape(rounds, npts, 2).copy()
    return proof, pos + 2 * rounds * npts


class Tensor:
    """A quantised tensor kept on the device (unpadded, row-major): weights across
    proofs, activations across the layers that read them.  bits: 64 or 16."""

    def __init__(self, ctx, values, bits=64):
        values = np.asarray(values)
        self.shape = tuple(values.shape)
        if bits == 64:
            self.mle = ctx.tensor_from_i64(values)
        elif bits == 16:
            self.mle = ctx.tensor_from_i16(values)
        else:
            raise ValueError("Tensor: bits must be 64 or 16")

    @property
    def ndim(self):
        return len(self.shape)


def einsum_prove(ctx, ops, lhs, rhs, claims, transcript, biases=None):
    """EinSum::prove_internal.  ops: list of (lhs_labels, rhs_labels, out_labels) or, for an
    output with a bias, (lhs_labels, rhs_labels, out_labels, bias_labels);
    lhs: int64 ndarray (unpadded); rhs: list of int64 ndarrays; claims: list of
    (point[k, 2], eval[2]) on the outputs; biases: None, or one entry per op (None where
    the op has no bias).  lhs, every rhs and every bias may instead be `Tensor`s already on
    the device (nothing is uploaded then).  Returns a dict with the sumcheck proof, the
    final evaluations, the optional aggregation proof, the input claims and the bias
    claims (output index, point, evaluation)."""
    R = len(ops)
    lab = []
    for o in ops:
        lab += [s.encode() for s in o] + ([b""] if len(o) == 3 else [])
    labels = (C.c_char_p * (4 * R))(*lab)
    resident = isinstance(lhs, Tensor)
    bk = list(biases) if biases is not None else None
    if bk is not None:
        if len(bk) != R or any((b is None) != (len(o) == 3 or not o[3]) for b, o in zip(bk, ops)):
            raise ValueError("einsum_prove: one bias per op that names bias labels")
        if any(b is not None and isinstance(b, Tensor) != resident for b in bk):
            raise ValueError("einsum_prove: either every tensor is on the device or none is")
    if resident != all(isinstance(x, Tensor) for x in rhs) or (not resident and any(isinstance(x, Tensor) for x in rhs)):
        raise ValueError("einsum_prove: either every tensor is on the device or none is")
    if resident:
        rk = list(rhs)
        rptr = (_vp * R)(*[x.mle.handle for x in rk])
        lhs_arg = lhs.mle.handle
        fn, fn_name = host.dph_einsum_prove_resident, "dph_einsum_prove_resident"
    else:
        lhs = np.ascontiguousarray(lhs, dtype=np.int64)
        rk = [np.ascontiguousarray(x, dtype=np.int64) for x in rhs]
        rptr = (_vp * R)(*[x.ctypes.data for x in rk])
        lhs_arg = _ptr(lhs)
        fn, fn_name = host.dph_einsum_prove, "dph_einsum_prove"
    lshape = (_u64 * lhs.ndim)(*lhs.shape)
    rshapes_keep = [(_u64 * x.ndim)(*x.shape) for x in rk]
    rshapes = (_vp * R)(*[C.cast(s, _vp).value for s in rshapes_keep])
    rranks = (_u32 * R)(*[x.ndim for x in rk])
    bptr = bshapes = branks = None
    if bk is not None:
        if not resident:
            bk = [None if b is None else np.ascontiguousarray(b, dtype=np.int64) for b in bk]
            bptr = (_vp * R)(*[None if b is None else b.ctypes.data for b in bk])
        else:
            bptr = (_vp * R)(*[None if b is None else b.mle.handle for b in bk])
        bshapes_keep = [None if b is None else (_u64 * b.ndim)(*b.shape) for b in bk]
        bshapes = (_vp * R)(*[None if s_ is None else C.cast(s_, _vp).value for s_ in bshapes_keep])
        branks = (_u32 * R)(*[0 if b is None else b.ndim for b in bk])
    pts_keep = [_e2(p).reshape(-1, 2) for p, _ in claims]
    pts = (_vp * R)(*[p.ctypes.data for p in pts_keep])
    plens = (_u32 * R)(*[p.shape[0] for p in pts_keep])
    evals = np.ascontiguousarray(np.stack([_e2(e) for _, e in claims]))
    cap = 1 << 16
    out = np.zeros(cap, dtype=np.uint64)
    n = _u64(0)
    ctx._chk_host(fn(ctx._c, R, labels, lhs_arg, lshape, lhs.ndim, rptr, rshapes, rranks, bptr, bshapes, branks, pts, plens, _ptr(evals),
                     transcript._t, _ptr(out), cap, C.byref(n)), fn_name)
    w = out[: n.value]
    res = {}
    res["proof"], pos = _parse_proof(w, 0)
    ne = int(w[pos])
    pos += 1
    res["evaluations"] = w[pos:pos + 2 * ne].reshape(ne, 2).copy()
    pos += 2 * ne
    if int(w[pos]) == 0:
        res["aggregation_proof"] = None
        pos += 1
    else:
        res["aggregation_proof"], pos = _parse_proof(w, pos)
    nc = int(w[pos])
    pos += 1
    res["claims"] = []
    for _ in range(nc):
        pl = int(w[pos])
        pos += 1
        point = w[pos:pos + 2 * pl].reshape(pl, 2).copy()
        pos += 2 * pl
        res["claims"].append((point, w[pos:pos + 2].copy()))
        pos += 2
    nb = int(w[pos])
    pos += 1
    res["bias_claims"] = []
    for _ in range(nb):
        output, pl = int(w[pos]), int(w[pos + 1])
        pos += 2
        point = w[pos:pos + 2 * pl].reshape(pl, 2).copy()
        pos += 2 * pl
        res["bias_claims"].append((output, point, w[pos:pos + 2].copy()))
        pos += 2
    return res


def logup_batch_prove(ctx, instances, transcript):
    """new_batch_multiple_sizes_prove.  instances: list of dicts with keys cols
    (list of Mle), numer (Mle or None), c, beta.  Returns the flat proof stream
    (elements, shape (k, 2)); see dph_logup_batch_prove for the layout."""
    n = len(instances)
    ncols = (_u32 * n)(*[len(i["cols"]) for i in instances])
    flat = [m.handle for i in instances for m in i["cols"]]
    cols = (_vp * len(flat))(*flat)
    is_table = instances[0].get("numer") is not None
    numer = (_vp * n)(*[i["numer"].handle for i in instances]) if is_table else None
    cs = np.ascontiguousarray(np.stack([_e2(i["c"]) for i in instances]))
    bs = np.ascontiguousarray(np.stack([_e2(i["beta"]) for i in instances]))
    total = max(len(i["cols"][0]).bit_length() - 2 for i in instances)
    cap = sum(v * 4 for v in range(1, total + 1)) + (total + 2) * sum(2 * len(i["cols"]) + 6 for i in instances) + total + 8
    out = np.zeros((cap, 2), dtype=np.uint64)
    ne = _u64(0)
    ctx._chk_host(host.dph_logup_batch_prove(ctx._c, n, ncols, cols, numer, _ptr(cs), _ptr(bs), transcript._t, _ptr(out), cap, C.byref(ne)),
                  "dph_logup_batch_prove")
    return out[: ne.value].copy()


def logup_batch_verify(instances_meta, is_table, stream, transcript):
    """new_verify_logup_proof_multiple_sizes.  instances_meta: list of (n_cols,
    num_vars, c, beta).  Returns (status, claims, point); status 0 = accepted."""
    n = len(instances_meta)
    ncols = (_u32 * n)(*[m[0] for m in instances_meta])
    nvars = (_u32 * n)(*[m[1] for m in instances_meta])
    cs = np.ascontiguousarray(np.stack([_e2(m[2]) for m in instances_meta]))
    bs = np.ascontiguousarray(np.stack([_e2(m[3]) for m in instances_meta]))
    stream = _e2(stream)
    total = max(m[1] for m in instances_meta)
    n_claims = sum(m[0] + (1 if is_table else 0) for m in instances_meta)
    claims = np.zeros((n_claims, 2), dtype=np.uint64)
    point = np.zeros((total + 1, 2), dtype=np.uint64)
    rc = host.dph_logup_batch_verify(n, ncols, nvars, _ptr(cs), _ptr(bs), 1 if is_table else 0, _ptr(stream), stream.shape[0], transcript._t,
                                     _ptr(claims), _ptr(point))
    return rc, claims, point


host.dph_claims_batching_prove.restype = _i32
host.dph_claims_batching_prove.argtypes = [_vp, _u32, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp]
host.dph_claims_batching_verify.restype = _i32
host.dph_claims_batching_verify.argtypes = [_u32, _vp, _vp, _vp, _vp, _vp, _vp, _u32, _vp, _vp, _vp]


def _flat_claims(claims):
    pts = [np.ascontiguousarray(_e2(p).reshape(-1, 2)) for cls in claims for p, _ in cls]
    points = np.ascontiguousarray(np.concatenate(pts)) if pts else np.zeros((0, 2), dtype=np.uint64)
    evals = np.ascontiguousarray(np.stack([_e2(e) for cls in claims for _, e in cls]))
    return points, evals


def claims_batching_prover(ctx, polys, claims):
    """The same statement as claims_batching_prove with the call's arguments marshalled once: returns run(transcript) ->
    (proof[n, 3, 2], point[n, 2], chunk_evals[total_chunks, 2]), for callers that prove over the same tables repeatedly."""
    n = len(polys)
    cpp = (_u32 * n)(*[len(c) for c in polys])
    flat = [m.handle for c in polys for m in c]
    chunks = (_vp * len(flat))(*flat)
    npc = (_u32 * n)(*[len(c) for c in claims])
    points, evals = _flat_claims(claims)
    n_vars = max((len(c[0]).bit_length() - 1) for c in polys)
    keep = (polys, cpp, chunks, npc, points, evals)  # what the pointers below point into

    def run(transcript):
        proof = np.zeros((n_vars, 3, 2), dtype=np.uint64)
        point = np.zeros((n_vars, 2), dtype=np.uint64)
        out = np.zeros((len(flat), 2), dtype=np.uint64)
        nv = _u32(0)
        ctx._chk_host(host.dph_claims_batching_prove(ctx._c, n, keep[1], keep[2], keep[3], _ptr(keep[4]), _ptr(keep[5]), transcript._t, _ptr(proof),
                                                     _ptr(point), _ptr(out), C.byref(nv)), "dph_claims_batching_prove")
        assert nv.value == n_vars
        return proof, point, out

    return run


def claims_batching_prove(ctx, polys, claims, transcript):
    """Claims-batching sumcheck of the opening proof.  polys: per committed polynomial
    the list of its chunk tables (Mle); claims: per polynomial a list of (point, eval).
    Returns (proof[n, 3, 2], point[n, 2], chunk_evals[total_chunks, 2])."""
    return claims_batching_prover(ctx, polys, claims)(transcript)


def claims_batching_verify(shapes, claims, proof, chunk_evals, transcript):
    """shapes: per polynomial (num_chunks, num_vars of the whole polynomial).
    Returns (status, point); status 0 = accepted."""
    n = len(shapes)
    cpp = (_u32 * n)(*[s[0] for s in shapes])
    pv = (_u32 * n)(*[s[1] for s in shapes])
    npc = (_u32 * n)(*[len(c) for c in claims])
    points, evals = _flat_claims(claims)
    proof = np.ascontiguousarray(_e2(proof))
    ce = np.ascontiguousarray(_e2(chunk_evals))
    n_vars = proof.shape[0]
    point = np.zeros((n_vars, 2), dtype=np.uint64)
    rc = host.dph_claims_batching_verify(n, cpp, pv, npc, _ptr(points), _ptr(evals), _ptr(proof), n_vars, _ptr(ce), transcript._t, _ptr(point))
    return rc, point


host.dph_same_poly_prove.restype = _i32
host.dph_same_poly_prove.argtypes = [_vp, _vp, _u32, _vp, _vp, _vp, _vp, _vp, _vp]
host.dph_same_poly_verify.restype = _i32
host.dph_same_poly_verify.argtypes = [_u32, _u32, _vp, _vp, _vp, _vp, _vp, _vp]


def same_poly_prove(ctx, poly, claims, transcript):
    """same_poly::Prover: claims is a list of (point, eval) on the table `poly`.
    Returns (proof[n, 3, 2], point[n, 2], eval[2])."""
    n_vars = len(poly).bit_length() - 1
    points = np.ascontiguousarray(np.stack([_e2(p).reshape(n_vars, 2) for p, _ in claims]))
    evals = np.ascontiguousarray(np.stack([_e2(e) for _, e in claims]))
    proof = np.zeros((n_vars, 3, 2), dtype=np.uint64)
    point = np.zeros((n_vars, 2), dtype=np.uint64)
    ev = np.zeros(2, dtype=np.uint64)
    ctx._chk_host(host.dph_same_poly_prove(ctx._c, poly.handle, len(claims), _ptr(points), _ptr(evals), transcript._t, _ptr(proof), _ptr(point),
                                           _ptr(ev)), "dph_same_poly_prove")
    return proof, point, ev


def same_poly_verify(n_vars, claims, proof, ev, transcript):
    """same_poly::Verifier.  Returns (status, point); status 0 = accepted."""
    points = np.ascontiguousarray(np.stack([_e2(p).reshape(n_vars, 2) for p, _ in claims]))
    evals = np.ascontiguousarray(np.stack([_e2(e) for _, e in claims]))
    proof = np.ascontiguousarray(_e2(proof))
    ev = np.ascontiguousarray(_e2(ev))
    point = np.zeros((n_vars, 2), dtype=np.uint64)
    rc = host.dph_same_poly_verify(n_vars, len(claims), _ptr(points), _ptr(evals), _ptr(proof), _ptr(ev), transcript._t, _ptr(point))
    return rc, point


# ---- the sumcheck linking a lookup argument to its layer ----
class _LinkingConfig(C.Structure):
    _fields_ = [("variant", _i32), ("normalised_sum", _i32), ("has_weight", _i32), ("number_of_value_chunks", _u32),
                ("number_of_zeroing_chunks", _u32), ("table_bit_size", _u32), ("table_is_signed", _i32), ("input_sign_negative", _i32),
                ("min_output_value", C.c_int64), ("max_output_value", C.c_int64), ("rank", _u32), ("unpadded_input_shape", _vp)]


host.dph_linking_prove.restype = _i32
host.dph_linking_prove.argtypes = [_vp, _vp, _vp, _u32, _vp, _vp, _u32, _vp, _u32, _vp, _vp, _u64, _vp]
host.dph_linking_verify.restype = _i32
host.dph_linking_verify.argtypes = [_vp, _vp, _vp, _u32, _u32, _vp, _u32, _vp, _vp, _u32, _vp, _u32, _vp, _vp]
LINKING_VARIANTS = {"standard": 0, "glu": 1, "softmax": 2, "normalisation": 3}


def _linking_config(cfg):
    shape = (_u64 * len(cfg["shape"]))(*cfg["shape"])
    c = _LinkingConfig(LINKING_VARIANTS[cfg["variant"]], int(cfg.get("norm_sum", False)), int(cfg.get("has_weight", False)),
                       cfg["value_chunks"], cfg["zero_chunks"], cfg["bit_size"], int(cfg["signed"]),
                       int(cfg.get("input_sign", "positive") == "negative"), cfg.get("min_out", 0), cfg.get("max_out", 0), len(cfg["shape"]),
                       C.cast(shape, _vp))
    return c, shape


def linking_prove(ctx, cfg, mles, transcript, last_claim_point, logup_point, weight=None):
    """LookupInputConfig::prove_linking_sumcheck.  cfg: dict with variant ('standard', 'glu', 'softmax',
    'normalisation'), shape (unpadded input shape), value_chunks, zero_chunks, bit_size, signed, min_out,
    max_out, input_sign, norm_sum, has_weight.  mles: the witness tables in the expression's order.
    Returns (proof[n, d+1, 2], point[n, 2], evaluations[len(mles), 2], weight evaluation or None, challenges)."""
    c, keep = _linking_config(cfg)
    hs = (_vp * max(1, len(mles)))(*[m.handle for m in mles])
    lcp, lp = _e2(last_claim_point).reshape(-1, 2), _e2(logup_point).reshape(-1, 2)
    cap = 1 << 16
    out = np.zeros(cap, dtype=np.uint64)
    n = _u64(0)
    ctx._chk_host(host.dph_linking_prove(ctx._c, C.byref(c), hs, len(mles), None if weight is None else weight.handle, _ptr(lcp), lcp.shape[0],
                                         _ptr(lp), lp.shape[0], transcript._t, _ptr(out), cap, C.byref(n)), "dph_linking_prove")
    w = out[: n.value]
    proof, pos = _parse_proof(w, 0)
    ne = int(w[pos])
    pos += 1
    evals = w[pos:pos + 2 * ne].reshape(ne, 2).copy()
    pos += 2 * ne
    weight_eval = None
    if int(w[pos]):
        weight_eval = w[pos + 1:pos + 3].copy()
        pos += 2
    pos += 1
    rounds = proof.shape[0]
    point = w[pos:pos + 2 * rounds].reshape(rounds, 2).copy()
    pos += 2 * rounds
    nc = int(w[pos])
    challenges = w[pos + 1:pos + 1 + 2 * nc].reshape(nc, 2).copy()
    return proof, point, evals, weight_eval, challenges


def linking_verify(cfg, initial_claim, proof, evaluations, weight_eval, transcript, last_claim_point, logup_point):
    """LookupInputConfig::verify_linking_sumcheck from the claimed sum on.  Returns (status, point); status 0 = accepted."""
    c, keep = _linking_config(cfg)
    proof = np.ascontiguousarray(_e2(proof))
    evaluations = np.ascontiguousarray(_e2(evaluations)).reshape(-1, 2)
    lcp, lp = _e2(last_claim_point).reshape(-1, 2), _e2(logup_point).reshape(-1, 2)
    claim = np.ascontiguousarray(_e2(initial_claim))
    we = None if weight_eval is None else np.ascontiguousarray(_e2(weight_eval))
    point = np.zeros((proof.shape[0], 2), dtype=np.uint64)
    rc = host.dph_linking_verify(C.byref(c), _ptr(claim), _ptr(proof), proof.shape[0], proof.shape[1], _ptr(evaluations), evaluations.shape[0],
                                 None if we is None else _ptr(we), _ptr(lcp), lcp.shape[0], _ptr(lp), lp.shape[0], transcript._t, _ptr(point))
    return rc, point
