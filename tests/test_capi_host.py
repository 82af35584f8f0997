"""CPU-side checks of the boundary (no GPU, no compute calls): the C-ABI library loads and exports every
symbol include/rapid_sampling.h declares, the host logic of the reference wrappers (normalisation,
limits, error codes) behaves as sampling.cu:452-486 / :976-1011, and the PyTorch extension raises the
reference's exceptions for the reference's conditions."""
import ctypes as C
import os
import re

import numpy as np
import pytest

from tests import capi

F32 = np.float32


def _declared_functions():
    text = open(capi.HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = re.findall(r"\b(rs_[a-z_]+)\s*\(", text)
    return sorted(set(names))


def test_library_exports_every_declared_symbol():
    L = capi.lib()
    names = _declared_functions()
    assert {"rs_sample", "rs_philox_init", "rs_workspace_bytes", "rs_workspace_init", "rs_normalize_args",
            "rs_workspace_status", "rs_workspace_where", "rs_error_string", "rs_version", "rs_floor_read"} <= set(names)
    for n in names:
        assert hasattr(L, n), n
    assert L.rs_version() >= 100


def test_error_strings_cover_every_code():
    L = capi.lib()
    text = open(capi.HEADER).read()
    codes = [int(v) for v in re.findall(r"#define\s+RS_ERR_[A-Z_]+\s+(-\d+)", text)]
    assert len(codes) >= 9
    for c in codes + [0]:
        s = L.rs_error_string(c)
        assert s and s != b"unknown error"
    assert L.rs_error_string(-1000) == b"unknown error"


def test_diag_struct_layout_matches_header():
    text = open(capi.HEADER).read()
    body = re.search(r"typedef struct rs_row_diag \{(.*?)\} rs_row_diag;", text, flags=re.S).group(1)
    fields = re.findall(r"\b(float|uint32_t|int32_t|uint64_t)\s+(\w+)(?:\[(\d+)\])?;", body)
    assert [f[1] for f in fields] == list(capi.DIAG_DTYPE.names)
    size = {"float": 4, "uint32_t": 4, "int32_t": 4, "uint64_t": 8}
    assert sum(size[t] * int(n or 1) for t, _, n in fields) == capi.DIAG_DTYPE.itemsize == 120
    from oracle import oracle as O
    assert O.DIAG_DTYPE == capi.DIAG_DTYPE


@pytest.mark.parametrize("temp,k,p,V,exp_k,exp_p", [
    (1.0, -1, 0.5, 131072, 131072, 0.5), (1.0, 0, 0.5, 1024, 1024, 0.5), (1.0, 5000, 0.5, 1024, 1024, 0.5),
    (2.0, 50, 1.5, 1024, 50, 1.0), (0.5, 50, -1.0, 1024, 50, 1.0), (1.0, 50, 0.0, 1024, 1, 1.0),
])
def test_normalize_args_matches_reference_rules(oracle, temp, k, p, V, exp_k, exp_p):
    rc, c, kk, pp = capi.normalize(temp, k, p, V)
    assert rc == 0 and kk == exp_k and pp == exp_p
    assert (c, kk, pp) == oracle.normalize(temp, k, p, V)      # same host logic as the oracle's restatement
    assert c == float(F32(1.4426950408889634 / temp))


@pytest.mark.parametrize("temp,V,B,T,code", [
    (1.0, 0, 1, 1, -1), (1.0, 10, 1, 1, -1), (1.0, 1048580, 1, 1, -1), (1.0, 8, 0, 1, -2), (1.0, 8, 2, 0, -2),
    (0.0005, 8, 1, 1, -3), (1000.5, 8, 1, 1, -3), (float("nan"), 8, 1, 1, -3),
])
def test_normalize_args_error_codes(temp, V, B, T, code):
    rc, _, _, _ = capi.normalize(temp, -1, 0.5, V, B, T)
    assert rc == code


def test_limits_accept_the_extremes():
    assert capi.normalize(0.001, -1, 1.0, 1048576)[0] == 0
    assert capi.normalize(1000.0, 1, 1.0, 4)[0] == 0


def test_workspace_size_is_independent_of_t_monotone_and_bounded():
    """rs_workspace_bytes takes (B, V) only -- T never enters.  It grows with B and with V (so that a
    workspace for the largest B and the largest V serves every smaller call), and stays well below the
    reference's per-call scratch of B*V floats (sampling.cu:488,1014) apart from a fixed reserve of 12 MB
    and a record per row."""
    Bs, Vs = (1, 2, 3, 7, 64, 128, 1000), (4, 4096, 32768, 131072, 152064, 1048576)
    sizes = {}
    for B in Bs:
        for V in Vs:
            rc, n = capi.workspace_bytes(B, V)
            assert rc == 0 and n % 256 == 0
            assert n <= 12 * 2 ** 20 + B * (65536 + 0.4 * 4 * V)
            sizes[B, V] = n
    for i, B in enumerate(Bs):
        for j, V in enumerate(Vs):
            if i:
                assert sizes[Bs[i - 1], V] < sizes[B, V]
            if j:
                assert sizes[B, Vs[j - 1]] <= sizes[B, V]
    assert capi.workspace_bytes(0, 8)[0] == -2 and capi.workspace_bytes(1, 6)[0] == -1


def test_sample_rejects_bad_arguments_before_touching_the_device():
    """Argument screening of rs_sample runs on the host; none of these reaches a launch."""
    L = capi.lib()
    ok = dict(logits=256, stride=1024, pen=None, out=256, rng=256, u=None, B=1, V=1024,
              c=1.0, k=10, p=0.5, ws=256, wsb=1 << 26)

    def call(**kw):
        a = dict(ok); a.update(kw)
        return L.rs_sample(a["logits"], a["stride"], a["pen"], a["out"], a["rng"], a["u"], a["B"], a["V"],
                           0.0, 0.0, 1.0, a["c"], a["k"], a["p"], a["ws"], a["wsb"], None, None, None)

    assert call(logits=None) == -4 and call(out=None) == -4 and call(ws=None) == -4
    assert call(rng=None, u=None) == -4
    assert call(V=1022) == -1 and call(V=0) == -1 and call(V=1048580) == -1
    assert call(B=0) == -2
    assert call(k=0) == -7 and call(k=2000) == -7 and call(p=0.0) == -7 and call(p=1.5) == -7 and call(c=0.0) == -7
    assert call(logits=260) == -6 and call(B=2, stride=1023) == -6 and call(pen=8) == -6
    assert call(wsb=16) == -5 and call(ws=264) == -5


# ---------------------------------------------------------------- the PyTorch extension, host side only
@pytest.fixture(scope="module")
def sample():
    import rapid_sampling_amd
    return rapid_sampling_amd


def test_extension_exposes_reference_api(sample):
    """Same three names as /root/reference/sampling.cpp:6-8, positional order preserved."""
    for n in ("setup_rand", "batch_sampling_temperature_topk_topp", "batch_sampling_repetition_temperature_topk_topp"):
        assert callable(getattr(sample, n))
    assert sample.STATE_BYTES_PER_ROW == 64
    doc = sample.batch_sampling_repetition_temperature_topk_topp.__doc__
    order = ["logits", "penalties", "states", "presence_penalty", "repetition_penalty", "penalty_decay",
             "temperature", "top_k", "top_p"]
    pos = [doc.index(n + ":") for n in order]
    assert pos == sorted(pos)
    doc = sample.batch_sampling_temperature_topk_topp.__doc__
    pos = [doc.index(n + ":") for n in ["logits", "states", "temperature", "top_k", "top_p"]]
    assert pos == sorted(pos)


def test_extension_raises_reference_errors_in_reference_order(sample):
    import torch
    st = torch.zeros(64, dtype=torch.int8)
    f = sample.batch_sampling_temperature_topk_topp
    with pytest.raises(ValueError, match=r"Logits tensor must be of type float32 \(FP32\), got"):
        f(torch.zeros(2, 6, dtype=torch.float16), st, 0.0, -1, 0.5)       # dtype is checked first
    with pytest.raises(ValueError, match=r"Vocabulary size must be multiple of 4, and no larger than 1048576, got 6"):
        f(torch.zeros(2, 6), st, 0.0, -1, 0.5)                             # then V
    with pytest.raises(ValueError, match=r"Vocabulary size .* got 1048580"):
        f(torch.zeros(1, 1048580), st, 1.0, -1, 0.5)
    with pytest.raises(ValueError, match=r"B and T must be positive, got B=0, T=1"):
        f(torch.zeros(0, 8), st, 0.0, -1, 0.5)                             # then B, T
    with pytest.raises(ValueError, match=r"Temperature outside range, got 0.000000, expect \[0.001, 1000\]"):
        f(torch.zeros(2, 8), st, 0.0, -1, 0.5)                             # then temperature
    with pytest.raises(ValueError, match=r"Temperature outside range, got 2000"):
        f(torch.zeros(2, 3, 8), st, 2000.0, -1, 0.5)
    with pytest.raises(ValueError, match="must live on the GPU"):
        f(torch.zeros(2, 8), st, 1.0, -1, 0.5)                             # only then our own checks
    g = sample.batch_sampling_repetition_temperature_topk_topp
    with pytest.raises(ValueError, match=r"Logits tensor must be of type float32"):
        g(torch.zeros(2, 8, dtype=torch.float64), torch.zeros(2, 8), st, 0.1, 0.1, 0.9, 1.0, -1, 0.5)
    with pytest.raises(ValueError, match=r"Temperature outside range"):
        g(torch.zeros(2, 8), torch.zeros(2, 8), st, 0.1, 0.1, 0.9, 1e-4, -1, 0.5)
    with pytest.raises(ValueError, match=r"B must be positive"):
        sample.setup_rand(0, 0)
    # half-precision logits are an opt-in: bfloat16 and float16 pass the first check with
    # accept_half=True (and fail the next one here), other types never do
    with pytest.raises(ValueError, match=r"type float32 \(FP32\), got"):
        f(torch.zeros(2, 8, dtype=torch.bfloat16), st, 1.0, -1, 0.5)
    with pytest.raises(ValueError, match=r"type float32 \(FP32\), got"):
        f(torch.zeros(2, 8, dtype=torch.float64), st, 1.0, -1, 0.5, accept_half=True)
    for dt in (torch.bfloat16, torch.float16):
        with pytest.raises(ValueError, match="must live on the GPU"):
            f(torch.zeros(2, 8, dtype=dt), st, 1.0, -1, 0.5, accept_half=True)
        with pytest.raises(ValueError, match="must live on the GPU"):
            g(torch.zeros(2, 8, dtype=dt), torch.zeros(2, 8), st, 0.1, 0.1, 0.9, 1.0, -1, 0.5, accept_half=True)


def test_extension_accepts_keywords_like_the_readme(sample):
    """The reference README calls the penalty entry point with keywords (README.md:100-110); its own
    binding has no argument names, ours does.  Checked up to the first device touch."""
    import torch
    with pytest.raises(ValueError, match="must live on the GPU"):
        sample.batch_sampling_repetition_temperature_topk_topp(
            torch.zeros(2, 8), torch.zeros(2, 8), torch.zeros(128, dtype=torch.int8),
            presence_penalty=0.1, repetition_penalty=0.1, penalty_decay=0.95, temperature=0.8, top_k=50, top_p=0.9)


def test_product_does_not_import_the_oracle():
    """The shipped package must not reach into oracle/ (no CPU fallback)."""
    root = os.path.join(capi.ROOT, "rapid_sampling_amd")
    for dirpath, _, files in os.walk(root):
        for fn in files:
            if fn.endswith((".py", ".cpp", ".hip", ".h")):
                text = open(os.path.join(dirpath, fn), errors="ignore").read()
                for pat in (r"^\s*(import|from)\s+oracle", r"oracle/", r"rs_oracle", r"ref_literal"):
                    assert not re.search(pat, text, flags=re.M), (os.path.join(dirpath, fn), pat)
    libs = os.popen("ldd %s 2>/dev/null" % capi.LIB_PATH).read()
    assert "rs_oracle" not in libs


def test_library_reads_no_environment_and_takes_no_locks():
    """The C ABI is stateless: what a call needs lives in its arguments, the workspace and the caller's
    rs_policy.  The library imports neither getenv nor any mutex / once primitive."""
    import subprocess
    out = subprocess.run(["nm", "-D", "--undefined-only", capi.LIB_PATH], capture_output=True, text=True, check=True).stdout
    for sym in ("getenv", "pthread_mutex_lock", "pthread_once", "__cxa_guard_acquire"):
        assert sym not in out, sym


def test_options_and_policy_arguments_are_checked():
    L = capi.lib()
    assert L.rs_policy_state(None, C.byref(C.c_int32())) == -4
    assert L.rs_policy_error(None, C.byref(C.c_int32()), 0) == -4
    assert L.rs_policy_create(None) == -4
    L.rs_policy_destroy(None)                              # a no-op
    assert L.rs_workspace_set_wait_limit(None, 5, None) == -4
    assert L.rs_workspace_set_wait_limit(C.c_void_p(256), 50000, None) == -7
    # options out of range are refused before anything is launched (pointers are never dereferenced:
    # the checks come first)
    bad = capi.Options(9, 0, None)
    args = [C.c_void_p(4096), 0, 1024, None, C.c_void_p(4096), C.c_void_p(4096), None, 1, 1024,
            0.0, 0.0, 1.0, 1.0, 10, 0.5, C.c_void_p(4096), 1 << 30, None, None, C.byref(bad), None]
    assert L.rs_sample_ex(*args) == -7
