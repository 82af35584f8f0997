"""ctypes binding of the C ABI in include/rapid_sampling.h, used by the tests to
call the HIP library directly (torch only provides device memory)."""
import ctypes as C
import os

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB_PATH = os.path.join(ROOT, "rapid_sampling_amd", "librapid_sampling_hip.so")
HEADER = os.path.join(ROOT, "include", "rapid_sampling.h")

# 128-bit quantities are (low, high) uint64 pairs
DIAG_DTYPE = np.dtype([
    ("xmax", "<f4"), ("emin_bits", "<u4"), ("D", "<u8", (2,)), ("P", "<u8", (2,)),
    ("left_bits", "<u4"), ("thr_bits", "<u4"), ("rounds", "<u4"), ("n_gt", "<u4"),
    ("n_eq", "<u4"), ("index", "<i4"), ("G", "<u8", (2,)), ("w_tie", "<u8"),
    ("S", "<u8", (2,)), ("r", "<u8", (2,)),
])

PATHS = {None: 0, "auto": 0, "cluster": 1, "stream": 2, "optimistic": 3, "attempt": 3, "fused": 4, "wide": 5, "wide1": 6, "row": 7}


class Options(C.Structure):
    """rs_options of include/rapid_sampling.h"""
    _fields_ = [("path", C.c_int32), ("slice_r", C.c_int32), ("policy", C.c_void_p)]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("HIP library not built: run python rapid_sampling_amd/build.py")
        L = C.CDLL(LIB_PATH)
        vp, i32, i64, f32, sz = C.c_void_p, C.c_int32, C.c_int64, C.c_float, C.c_size_t
        L.rs_version.restype = C.c_int
        L.rs_error_string.restype = C.c_char_p
        L.rs_error_string.argtypes = [C.c_int]
        L.rs_normalize_args.restype = C.c_int
        L.rs_normalize_args.argtypes = [C.c_double, i64, C.c_double, i64, i64, i64,
                                        C.POINTER(f32), C.POINTER(i32), C.POINTER(f32)]
        L.rs_workspace_bytes.restype = C.c_int
        L.rs_workspace_bytes.argtypes = [i32, i32, C.POINTER(sz)]
        L.rs_workspace_set_wait_limit.restype = C.c_int
        L.rs_workspace_set_wait_limit.argtypes = [vp, C.c_uint32, vp]
        L.rs_policy_create.restype = C.c_int
        L.rs_policy_create.argtypes = [C.POINTER(vp)]
        L.rs_policy_destroy.restype = None
        L.rs_policy_destroy.argtypes = [vp]
        L.rs_policy_state.restype = C.c_int
        L.rs_policy_state.argtypes = [vp, C.POINTER(i32)]
        L.rs_policy_error.restype = C.c_int
        L.rs_policy_error.argtypes = [vp, C.POINTER(i32), i32]
        L.rs_sample_ex.restype = C.c_int
        L.rs_sample_ex.argtypes = [vp, i32, i64, vp, vp, vp, vp, i32, i32, f32, f32, f32, f32, i32, f32,
                                   vp, sz, vp, vp, C.POINTER(Options), vp]
        L.rs_workspace_init.restype = C.c_int
        L.rs_workspace_init.argtypes = [vp, sz, vp]
        L.rs_workspace_status.restype = C.c_int
        L.rs_workspace_status.argtypes = [vp, C.POINTER(i32), vp]
        L.rs_workspace_where.restype = C.c_int
        L.rs_workspace_where.argtypes = [vp, C.POINTER(C.c_uint32), vp]
        L.rs_philox_init.restype = C.c_int
        L.rs_philox_init.argtypes = [vp, C.c_uint64, i32, vp]
        L.rs_sample.restype = C.c_int
        L.rs_sample.argtypes = [vp, i64, vp, vp, vp, vp, i32, i32, f32, f32, f32, f32, i32, f32,
                                vp, sz, vp, vp, vp]
        L.rs_sample_dtype.restype = C.c_int
        L.rs_sample_dtype.argtypes = [vp, i32, i64, vp, vp, vp, vp, i32, i32, f32, f32, f32, f32, i32, f32,
                                      vp, sz, vp, vp, vp]
        L.rs_sample_static.restype = C.c_int
        L.rs_sample_static.argtypes = [vp, i32, i64, vp, vp, vp, vp, i32, i32, f32, f32, f32, f32, i32, f32,
                                       vp, vp, C.POINTER(Options), vp]
        L.rs_static_prepare.restype = C.c_int
        L.rs_static_prepare.argtypes = []
        L.rs_static_workspace.restype = C.c_void_p
        L.rs_static_workspace.argtypes = []
        L.rs_static_status.restype = C.c_int
        L.rs_static_status.argtypes = [C.POINTER(i32), C.POINTER(C.c_uint32), i32, vp]
        L.rs_floor_read.restype = C.c_int
        L.rs_floor_read.argtypes = [vp, i64, vp, i32, i32, i32, vp]
        _lib = L
    return _lib


def normalize(temperature, top_k, top_p, V, B=1, T=1):
    c, k, p = C.c_float(), C.c_int32(), C.c_float()
    rc = lib().rs_normalize_args(temperature, top_k, top_p, B, T, V, C.byref(c), C.byref(k), C.byref(p))
    return rc, c.value, k.value, p.value


HEADER_BYTES = 2304          # the workspace's launch header (sizeof(rs::WsHeader)); tests that spoil a workspace leave it alone


def workspace_bytes(B, V):
    n = C.c_size_t()
    rc = lib().rs_workspace_bytes(B, V, C.byref(n))
    return rc, n.value


class Sampler:
    """Holds a workspace on the current torch device and calls rs_sample on the
    current torch stream."""

    def __init__(self, B, V, with_policy=False, init=False):
        """with_policy: own an rs_policy (routing reports, asynchronous error word) and pass it with
        every call.  init: clear the workspace with rs_workspace_init instead of torch.zeros."""
        import torch
        self.torch = torch
        rc, n = workspace_bytes(B, V)
        assert rc == 0
        if init:
            self.ws = torch.empty(n, dtype=torch.int8, device="cuda")
            assert lib().rs_workspace_init(self.ws.data_ptr(), n, self.stream()) == 0
        else:
            self.ws = torch.zeros(n, dtype=torch.int8, device="cuda")
        self.B, self.V = B, V
        self.policy = None
        if with_policy:
            h = C.c_void_p()
            assert lib().rs_policy_create(C.byref(h)) == 0 and h.value
            self.policy = h

    def close(self):
        """Frees the policy; only after the device has finished every call that was given it."""
        if self.policy is not None:
            self.torch.cuda.synchronize()
            lib().rs_policy_destroy(self.policy)
            self.policy = None

    def policy_state(self):
        st = C.c_int32(-100)
        assert lib().rs_policy_state(self.policy, C.byref(st)) == 0
        return st.value

    def policy_error(self, clear=False):
        e = C.c_int32(-100)
        assert lib().rs_policy_error(self.policy, C.byref(e), 1 if clear else 0) == 0
        return e.value

    def reinit(self):
        assert lib().rs_workspace_init(self.ws.data_ptr(), self.ws.numel(), self.stream()) == 0

    def set_wait_limit(self, ms):
        assert lib().rs_workspace_set_wait_limit(self.ws.data_ptr(), ms, self.stream()) == 0

    def stream(self):
        return C.c_void_p(self.torch.cuda.current_stream().cuda_stream)

    def status(self):
        st = C.c_int32(-100)
        rc = lib().rs_workspace_status(self.ws.data_ptr(), C.byref(st), self.stream())
        assert rc == 0
        return st.value

    def where(self):
        """(wait, row, slice, seen, wanted) of the first wait that gave up; wait 0 = none."""
        w = (C.c_uint32 * 4)()
        rc = lib().rs_workspace_where(self.ws.data_ptr(), w, self.stream())
        assert rc == 0
        return int(w[0]), int(w[1]) >> 16, int(w[1]) & 0xffff, int(w[2]), int(w[3])

    def sample(self, logits, c, top_k, top_p, *, rng=None, uniforms=None, penalties=None,
               presence=0.0, repetition=0.0, decay=1.0, want_diag=True, want_e=False, path=None, force_r=None,
               sync=True):
        """logits: (B,V) or (B,T,V) cuda tensor, float32 (rs_sample) or bfloat16 / float16
        (rs_sample_dtype); with path / force_r / a policy the call goes through rs_sample_ex.
        Returns dict of cpu numpy results."""
        torch = self.torch
        dtype = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}[logits.dtype]
        if logits.dim() == 3:
            B, T, V = logits.shape
            ptr = logits.data_ptr() + logits.element_size() * (T - 1) * logits.stride(1)
            stride = logits.stride(0)
        else:
            B, V = logits.shape
            ptr, stride = logits.data_ptr(), logits.stride(0)
        if penalties is not None:
            B = penalties.shape[0]
        out = torch.full((B,), -7, dtype=torch.int32, device="cuda")
        diag = torch.zeros((B, DIAG_DTYPE.itemsize), dtype=torch.uint8, device="cuda") if want_diag else None
        eb = torch.empty((B, V), dtype=torch.int32, device="cuda") if want_e else None
        tail = (penalties.data_ptr() if penalties is not None else None,
                out.data_ptr(), rng.data_ptr() if rng is not None else None,
                uniforms.data_ptr() if uniforms is not None else None,
                B, V, presence, repetition, decay, c, top_k, top_p,
                self.ws.data_ptr(), self.ws.numel(),
                diag.data_ptr() if diag is not None else None,
                eb.data_ptr() if eb is not None else None, self.stream())
        if path is not None or force_r is not None or self.policy is not None:
            opt = Options(PATHS[path], force_r or 0, self.policy)
            rc = lib().rs_sample_ex(ptr, dtype, stride, *tail[:-1], C.byref(opt), tail[-1])
        elif dtype == 0:
            rc = lib().rs_sample(ptr, stride, *tail)
        else:
            rc = lib().rs_sample_dtype(ptr, dtype, stride, *tail)
        res = {"rc": rc}
        if rc != 0:
            return res
        if not sync:
            res["out_dev"] = out
            res["diag_dev"] = diag
            return res
        torch.cuda.synchronize()
        res["out"] = out.cpu().numpy()
        if want_diag:
            res["diag"] = diag.cpu().numpy().view(DIAG_DTYPE).reshape(B)
        if want_e:
            res["e_bits"] = eb.cpu().numpy().view(np.uint32)
        return res
