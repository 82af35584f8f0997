"""ctypes/numpy front end of the CPU oracle -- TEST INFRASTRUCTURE, NOT PRODUCT.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg import this
module.  The shipped package never does and has no CPU fallback.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "librs_oracle.so")


def build(force=False):
    """Compile oracle/librs_oracle.so with gcc (seconds)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-s", "-C", _HERE] + (["-B"] if force else []))
    return _LIB_PATH


class Diag(C.Structure):
    _fields_ = [
        ("xmax", C.c_float), ("emin_bits", C.c_uint32),
        ("D", C.c_uint64 * 2), ("P", C.c_uint64 * 2),
        ("left_bits", C.c_uint32), ("thr_bits", C.c_uint32),
        ("rounds", C.c_uint32), ("n_gt", C.c_uint32),
        ("n_eq", C.c_uint32), ("index", C.c_int32),
        ("G", C.c_uint64 * 2), ("w_tie", C.c_uint64),
        ("S", C.c_uint64 * 2), ("r", C.c_uint64 * 2),
    ]

    def asdict(self):
        """128-bit fields come back as Python integers."""
        out = {}
        for n, t in self._fields_:
            v = getattr(self, n)
            out[n] = (int(v[0]) | (int(v[1]) << 64)) if t is C.c_uint64 * 2 else v
        return out


# numpy view of the same record; 128-bit quantities are (low, high) uint64 pairs
DIAG_DTYPE = np.dtype([
    ("xmax", "<f4"), ("emin_bits", "<u4"), ("D", "<u8", (2,)), ("P", "<u8", (2,)),
    ("left_bits", "<u4"), ("thr_bits", "<u4"), ("rounds", "<u4"), ("n_gt", "<u4"),
    ("n_eq", "<u4"), ("index", "<i4"), ("G", "<u8", (2,)), ("w_tie", "<u8"),
    ("S", "<u8", (2,)), ("r", "<u8", (2,)),
])
assert DIAG_DTYPE.itemsize == C.sizeof(Diag) == 120


def u128(pair):
    """(low, high) uint64 pair -> Python int."""
    return int(pair[0]) | (int(pair[1]) << 64)


class LiteralDiag(C.Structure):
    _fields_ = [
        ("threshold", C.c_float), ("comp", C.c_float), ("pmax", C.c_float),
        ("pmin", C.c_float), ("denom", C.c_float), ("xmax", C.c_float),
        ("kept", C.c_uint32), ("n_eq", C.c_uint32), ("n_gt", C.c_uint32),
        ("rounds", C.c_uint32), ("idxt", C.c_int32), ("index", C.c_int32),
    ]

    def asdict(self):
        return {n: getattr(self, n) for n, _ in self._fields_}


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(_LIB_PATH)
        fp, u32p, u64 = C.POINTER(C.c_float), C.POINTER(C.c_uint32), C.c_uint64
        L.rs_oracle_sf.restype = C.c_float
        L.rs_oracle_sf.argtypes = [C.c_float]
        L.rs_oracle_scale.restype = C.c_float
        L.rs_oracle_scale.argtypes = [C.c_float, C.c_float, C.c_int, C.c_float]
        L.rs_oracle_e_bits.restype = C.c_uint32
        L.rs_oracle_e_bits.argtypes = [C.c_float, C.c_float]
        L.rs_oracle_w.restype = u64
        L.rs_oracle_w.argtypes = [C.c_uint32]
        L.rs_oracle_ceil_mul.restype = None
        L.rs_oracle_ceil_mul.argtypes = [C.c_float, u64, u64, C.POINTER(u64)]
        L.rs_oracle_r_from_bits.restype = None
        L.rs_oracle_r_from_bits.argtypes = [u64, u64, u64, C.POINTER(u64)]
        L.rs_oracle_normalize.restype = C.c_int
        L.rs_oracle_normalize.argtypes = [C.c_double, C.c_int64, C.c_double, C.c_int64, C.c_int64,
                                          C.c_int64, fp, C.POINTER(C.c_int32), fp]
        L.rs_oracle_philox.restype = None
        L.rs_oracle_philox.argtypes = [u32p, u32p, u32p]
        L.rs_oracle_philox_draw.restype = None
        L.rs_oracle_philox_draw.argtypes = [u64, u64, u64, u32p]
        L.rs_oracle_rng_init.restype = None
        L.rs_oracle_rng_init.argtypes = [C.c_void_p, u64, C.c_int32]
        L.rs_oracle_thr_by_sort.restype = C.c_uint32
        L.rs_oracle_thr_by_sort.argtypes = [C.c_void_p, C.c_int32, C.c_int32, u64, u64]
        L.rs_oracle_row.restype = None
        L.rs_oracle_row.argtypes = [C.c_void_p, C.c_void_p, C.c_int32, C.c_float, C.c_int32, C.c_float,
                                    C.c_int, C.c_float, u64, C.c_float, C.c_float, C.c_float,
                                    C.c_void_p, C.POINTER(Diag)]
        L.rs_oracle_batch.restype = None
        L.rs_oracle_batch.argtypes = [C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                      C.c_int32, C.c_int32, C.c_float, C.c_int32, C.c_float,
                                      C.c_float, C.c_float, C.c_float, C.c_void_p]
        L.rs_oracle_batch_e.restype = None
        L.rs_oracle_batch_e.argtypes = L.rs_oracle_batch.argtypes + [C.c_void_p]
        L.ref_literal_row.restype = None
        L.ref_literal_row.argtypes = [C.c_void_p, C.c_void_p, C.c_int32, C.c_float, C.c_int32, C.c_float,
                                      C.c_int, C.c_float, C.c_float, C.c_float, C.c_float, C.c_float,
                                      C.c_void_p, C.POINTER(LiteralDiag)]
        L.ref_literal_block_scan_f32.restype = None
        L.ref_literal_block_scan_f32.argtypes = [C.c_void_p, C.c_void_p, fp, C.c_int]
        L.ref_literal_wave64_scan_f32.restype = None
        L.ref_literal_wave64_scan_f32.argtypes = [C.c_void_p, C.c_void_p, C.c_int]
        _lib = L
    return _lib


def _ptr(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def normalize(temperature, top_k, top_p, V, B=1, T=1):
    """Returns (c, k, p) after the host wrapper's normalisation, or raises ValueError."""
    c, k, p = C.c_float(), C.c_int32(), C.c_float()
    rc = lib().rs_oracle_normalize(temperature, top_k, top_p, B, T, V, C.byref(c), C.byref(k), C.byref(p))
    if rc:
        raise ValueError({-1: "vocabulary", -2: "B/T", -3: "temperature"}[rc])
    return c.value, k.value, p.value


def e_bits(x, M):
    """Bit patterns of e = 2^(x - M) for scaled logits x (array) and M = floor(max x)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    f = lib().rs_oracle_e_bits
    return np.array([f(float(v), float(M)) for v in x.ravel()], dtype=np.uint32).reshape(x.shape)


def w_of(bits):
    """Exact integer weights W = e * 2^63 of bit patterns (array) as uint64; 0 for dead tokens (e = 0)."""
    bits = np.ascontiguousarray(bits, dtype=np.uint32)
    live = bits >= np.uint32(0x2B800000)
    m = (bits & np.uint32(0x7FFFFF)).astype(np.uint64) | np.uint64(0x800000)
    ex = np.where(live, bits >> np.uint32(23), np.uint32(87)).astype(np.uint64)
    return np.where(live, m << (ex - np.uint64(87)), np.uint64(0))


def ceil_mul(f, s):
    out = (C.c_uint64 * 2)()
    lib().rs_oracle_ceil_mul(f, s & (2 ** 64 - 1), s >> 64, out)
    return int(out[0]) | (int(out[1]) << 64)


def r_from_bits(u64, s):
    out = (C.c_uint64 * 2)()
    lib().rs_oracle_r_from_bits(u64, s & (2 ** 64 - 1), s >> 64, out)
    return int(out[0]) | (int(out[1]) << 64)


def philox(ctr, key):
    c = (C.c_uint32 * 4)(*ctr)
    k = (C.c_uint32 * 2)(*key)
    o = (C.c_uint32 * 4)()
    lib().rs_oracle_philox(c, k, o)
    return list(o)


def philox_draw(seed, row, n):
    o = (C.c_uint32 * 4)()
    lib().rs_oracle_philox_draw(seed, row, n, o)
    return list(o)


def rng_init(seed, B):
    rng = np.zeros((B, 16), dtype=np.uint32)
    lib().rs_oracle_rng_init(_ptr(rng), seed, B)
    return rng


def sample_row(logits, c, top_k, top_p, u=None, u64=0, penalties=None,
               presence=0.0, repetition=0.0, decay=1.0, want_e=False):
    """One row through the canonical oracle.  penalties (if given) is updated in place."""
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    V = logits.shape[0]
    if penalties is not None:
        assert penalties.dtype == np.float32 and penalties.flags.c_contiguous and penalties.shape == (V,)
    e = np.empty(V, dtype=np.uint32) if want_e else None
    d = Diag()
    lib().rs_oracle_row(_ptr(logits), _ptr(penalties), V, c, top_k, top_p,
                        int(u is not None), float(u) if u is not None else 0.0, int(u64),
                        presence, repetition, decay, _ptr(e), C.byref(d))
    out = d.asdict()
    if want_e:
        out["e_bits"] = e
    return out


def sample_batch(logits, c, top_k, top_p, rng=None, injected_u=None, penalties=None,
                 presence=0.0, repetition=0.0, decay=1.0, want_e=False):
    """A batch through the canonical oracle.

    logits: (V,), (B, V) or (B, T, V) float32; for (B, T, V) only logits[:, T-1, :] is read
    (sampling.cu:176,202).  Returns (out int32 (B,), diag structured array (B,)), and with want_e
    also the bit patterns of e of every token, uint32 (B, V).
    """
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    if logits.ndim == 1:
        logits = logits[None, :]
    if logits.ndim == 3:
        B, T, V = logits.shape
        row_stride, offset = T * V, (T - 1) * V
    else:
        B, V = logits.shape
        row_stride, offset = V, 0
    base = logits.ctypes.data + 4 * offset
    out = np.empty(B, dtype=np.int32)
    diag = np.zeros(B, dtype=DIAG_DTYPE)
    if injected_u is not None:
        injected_u = np.ascontiguousarray(injected_u, dtype=np.float32)
        assert injected_u.shape == (B,)
    else:
        assert rng is not None and rng.dtype == np.uint32 and rng.shape == (B, 16)
    if penalties is not None:
        assert penalties.dtype == np.float32 and penalties.flags.c_contiguous and penalties.shape == (B, V)
    e = np.empty((B, V), dtype=np.uint32) if want_e else None
    lib().rs_oracle_batch_e(C.c_void_p(base), row_stride, _ptr(penalties), _ptr(out), _ptr(rng),
                            _ptr(injected_u), B, V, c, top_k, top_p, presence, repetition, decay,
                            _ptr(diag), _ptr(e))
    return (out, diag, e) if want_e else (out, diag)


def thr_by_sort(e_bits, top_k, P):
    e_bits = np.ascontiguousarray(e_bits, dtype=np.uint32)
    return lib().rs_oracle_thr_by_sort(_ptr(e_bits), e_bits.shape[0], top_k, P & (2 ** 64 - 1), P >> 64)


def literal_row(logits, c, top_k, top_p, u1, u2, variant=0, penalties=None,
                presence=0.0, repetition=0.0, decay=1.0, want_probs=False):
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    V = logits.shape[0]
    probs = np.empty(V, dtype=np.float32) if want_probs else None
    d = LiteralDiag()
    lib().ref_literal_row(_ptr(logits), _ptr(penalties), V, c, top_k, top_p, variant, u1, u2,
                          presence, repetition, decay, _ptr(probs), C.byref(d))
    out = d.asdict()
    if want_probs:
        out["probs"] = probs
    return out


def literal_block_scan(x, descending=True):
    x = np.ascontiguousarray(x, dtype=np.float32)
    assert x.shape == (1024,)
    out = np.empty(1024, dtype=np.float32)
    tot = C.c_float()
    lib().ref_literal_block_scan_f32(_ptr(x), _ptr(out), C.byref(tot), int(descending))
    return out, tot.value


def literal_wave64_scan(x, descending=True):
    x = np.ascontiguousarray(x, dtype=np.float32)
    assert x.shape == (64,)
    out = np.empty(64, dtype=np.float32)
    lib().ref_literal_wave64_scan_f32(_ptr(x), _ptr(out), int(descending))
    return out
