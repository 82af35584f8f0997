"""GPU parity: the HIP library, called through its C ABI, against the CPU oracle
on the same seeded inputs.  Bar: everything here is integer / bit-pattern work,
so every compared field must be EQUAL (sampled index, threshold, kept set as
{e >= thr} from bit-identical e, counts, integer masses); updated penalties are
compared bit for bit as well (the stated bar is 1e-6 relative)."""
import os
from ctypes import byref as C_byref, c_void_p as C_void_p

import numpy as np
import pytest

from tests import helpers as H

pytestmark = pytest.mark.gpu

# every diagnostic both sides define (emin_bits, left_bits and rounds describe the oracle's
# literal search loop; the GPU selects the same threshold by radix and does not produce them)
FIELDS = ["xmax", "D", "P", "thr_bits", "n_gt", "n_eq", "index", "G", "w_tie", "S", "r"]


@pytest.fixture(scope="module")
def torch_cuda():
    import torch
    assert torch.cuda.is_available(), "these tests need the GPU"
    return torch


def _check(res, ref_out, ref_diag, what, ref_e=None):
    assert res["rc"] == 0, what
    for f in FIELDS:
        got, exp = res["diag"][f], ref_diag[f]
        assert np.array_equal(got, exp), "%s: field %s differs, rows %s" % (what, f, np.nonzero(got != exp)[0][:8])
    assert np.array_equal(res["out"], ref_out), what
    if ref_e is not None:
        # e of every token bit for bit (0 for dead tokens): with the threshold above, the kept set {e >= thr}
        bad = np.nonzero((res["e_bits"] != ref_e).any(axis=1))[0]
        assert bad.size == 0, "%s: e differs in rows %s" % (what, bad[:8])


def _run_case(torch, oracle, capi, logits_np, temperature, top_k, top_p, *, pen_np=None, u_np=None,
              presence=0.0, repetition=0.0, decay=1.0, force_r=None, what="", dtype=None):
    """dtype: torch.bfloat16 / torch.float16 to hand the logits over in that format (logits_np must
    then hold values that format represents exactly)."""
    if logits_np.ndim == 3:
        B, T, V = logits_np.shape
    else:
        (B, V), T = logits_np.shape, 1
    rc, c, k, p = capi.normalize(temperature, top_k, top_p, V, B, T)
    assert rc == 0
    oc, ok, op = oracle.normalize(temperature, top_k, top_p, V, B, T)
    assert (c, k, p) == (oc, ok, op)
    pen_ref = None if pen_np is None else pen_np.copy()
    ref_out, ref_diag, ref_e = oracle.sample_batch(logits_np, c, k, p, injected_u=u_np, penalties=pen_ref,
                                                   presence=presence, repetition=repetition, decay=decay, want_e=True)
    smp = capi.Sampler(B, V)
    lg = torch.from_numpy(logits_np).cuda()
    if dtype is not None:
        lg = lg.to(dtype)
        assert torch.equal(lg.float().cpu(), torch.from_numpy(logits_np)) or np.isnan(logits_np).any()
    pen = None if pen_np is None else torch.from_numpy(pen_np.copy()).cuda()
    u = torch.from_numpy(u_np).cuda()
    print("case", what, "B", B, "T", T, "V", V, "k", k, "p", p, "R", force_r, flush=True)
    res = smp.sample(lg, c, k, p, uniforms=u, penalties=pen, presence=presence, repetition=repetition,
                     decay=decay, want_e=True, force_r=force_r)
    _check(res, ref_out, ref_diag, what, ref_e)
    assert smp.status() == 0
    if pen is not None:
        assert np.array_equal(pen.cpu().numpy().view(np.uint32), pen_ref.view(np.uint32)), what + ": penalties"
    # second call on the same workspace: it must have been left clean
    pen2 = None if pen_np is None else torch.from_numpy(pen_np.copy()).cuda()
    res2 = smp.sample(lg, c, k, p, uniforms=u, penalties=pen2, presence=presence, repetition=repetition,
                      decay=decay, force_r=force_r)
    _check(res2, ref_out, ref_diag, what + " (second call)")
    # Every way through the library on this one workspace: the general kernel alone, the wait-free
    # streaming path (taken for top_k <= 1024; rows it cannot finish go on to the general kernel), the
    # same attempted whatever top_k is, the one-launch path (streaming pass and finish in one kernel,
    # falling back inside the kernel), the wide paths (two passes over the logits and a finish, for kept
    # sets of any size; one pass behind a sample of the row), the row kernel (one workgroup per row, rows of
    # up to 65536 tokens; longer ones take the general kernel), then the general kernel again on the workspace
    # these leave behind.  All but the general kernel also return the e of every token: the kept set on that path.
    # With penalties: the one-launch path and the general kernel.
    paths = ("cluster", "stream", "optimistic", "fused", "wide", "wide1", "row", "cluster") if pen_np is None else ("fused", "stream", "cluster", "fused")
    for path in paths:
        pen3 = None if pen_np is None else torch.from_numpy(pen_np.copy()).cuda()
        with_e = path != "cluster" and not (path == "row" and V > 65536)
        res3 = smp.sample(lg, c, k, p, uniforms=u, penalties=pen3, presence=presence, repetition=repetition, decay=decay,
                          path=path, force_r=force_r, want_e=with_e)
        _check(res3, ref_out, ref_diag, what + " (path %s)" % path, ref_e if with_e else None)
        if path == "row" and V <= 65536:
            # (0: a row that is one tie of all its tokens, finished from the row's bins)
            assert np.isin(res3["diag"]["rounds"], (0, 10)).all(), what + ": the row kernel finishes every row itself"
        assert smp.status() == 0
        if pen3 is not None:
            assert np.array_equal(pen3.cpu().numpy().view(np.uint32), pen_ref.view(np.uint32)), what + ": penalties, path " + path
    return res, ref_diag


def test_c1_uniform_logits_top_p(torch_cuda, oracle):
    """BASELINE config 1: B=1, V=131072, U[0,1), T=1, top_k=-1, top_p=0.5, one uniform per row."""
    from tests import capi
    lg = H.logits_uniform(1, 131072, seed=0)
    res, ref = _run_case(torch_cuda, oracle, capi, lg, 1.0, -1, 0.5, u_np=H.uniforms(1), what="C1")
    # kept set = {e >= thr}: e bit-identical and thr identical => identical set
    row = oracle.sample_row(lg[0], *oracle.normalize(1.0, -1, 0.5, 131072), u=float(H.uniforms(1)[0]), want_e=True)
    assert np.array_equal(res["e_bits"][0], row["e_bits"])
    kept_gpu = np.nonzero(res["e_bits"][0] >= res["diag"]["thr_bits"][0])[0]
    kept_ref = np.nonzero(row["e_bits"] >= row["thr_bits"])[0]
    assert np.array_equal(kept_gpu, kept_ref) and len(kept_ref) == ref["n_gt"][0] + ref["n_eq"][0]


def test_c2_single_row_split(torch_cuda, oracle):
    """BASELINE config 2: B=1, V=262144, N(0,1)*3, top_p=0.3."""
    from tests import capi
    _run_case(torch_cuda, oracle, capi, H.logits_normal(1, 262144, 3.0, seed=3), 1.0, -1, 0.3,
              u_np=H.uniforms(1, 5), what="C2")


def test_c3_mixed_topk_topp(torch_cuda, oracle):
    """BASELINE config 3: B=64, V=152064, N(0,2) + 10 on 16 ids, T=0.8, top_k=50, top_p=0.9."""
    from tests import capi
    _run_case(torch_cuda, oracle, capi, H.logits_spiked(64, 152064, seed=4), 0.8, 50, 0.9,
              u_np=H.uniforms(64, 6), what="C3")


def test_c5_shape_btv_reduced(torch_cuda, oracle):
    """BASELINE config 5 at reduced B: (B,T,V)=(6,4,1048576), top_k=1024, top_p=0.95; only t=T-1 is read."""
    from tests import capi
    lg = H.logits_normal(6 * 4, 1048576, 1.5, seed=7).reshape(6, 4, 1048576)
    _run_case(torch_cuda, oracle, capi, lg, 1.0, 1024, 0.95, u_np=H.uniforms(6, 8), what="C5r")


@pytest.mark.parametrize("R", [1, 2, 4, 8, 16, 32])
def test_every_slice_length(torch_cuda, oracle, R):
    """Same rows through every tokens-per-thread variant: identical results."""
    from tests import capi
    V = 50304                      # not a multiple of the slice: ragged last workgroup
    lg = H.logits_normal(5, V, 2.0, seed=10 + R)
    _run_case(torch_cuda, oracle, capi, lg, 0.7, 100, 0.8, u_np=H.uniforms(5, 11), force_r=R, what="R%d" % R)


@pytest.mark.parametrize("V,top_k,top_p,temp", [
    (4, -1, 1.0, 1.0), (4, 1, 1.0, 1.0), (256, 10, 0.3, 1.0), (1028, -1, 0.999, 2.0),
    (32768, 1000, 1.0, 0.5), (65536, -1, 0.1, 1.0), (100256, 10000, 0.7, 1.3), (151936, -1, 0.0, 1.0),
    (1048576, -1, 0.9, 1.0), (1048576, 1048576, 1.0, 1.0),
])
def test_grid_of_shapes(torch_cuda, oracle, V, top_k, top_p, temp):
    from tests import capi
    B = 3
    lg = H.logits_normal(B, V, 2.5, seed=V % 97)
    _run_case(torch_cuda, oracle, capi, lg, temp, top_k, top_p, u_np=H.uniforms(B, V % 13),
              what="grid V=%d" % V)


def test_degenerate_rows(torch_cuda, oracle):
    """All-equal logits (every token ties), NaN/Inf entries, one dominant token."""
    from tests import capi
    V = 4096
    lg = np.zeros((6, V), dtype=np.float32)
    lg[1] = 1.5
    lg[2] = H.logits_normal(1, V, 1.0, seed=1)[0]; lg[2, 7] = np.inf; lg[2, 9] = -np.inf; lg[2, 11] = np.nan
    lg[3] = H.logits_normal(1, V, 1.0, seed=2)[0]; lg[3, 100] = 300.0
    lg[4] = -np.inf
    lg[5] = H.logits_normal(1, V, 1.0, seed=3)[0]; lg[5, :2000] = lg[5, 2000]
    for (k, p) in [(10, 0.5), (-1, 1.0), (1, 1.0), (-1, 1e-30), (V, 0.9)]:
        _run_case(torch_cuda, oracle, capi, lg, 1.0, k, p, u_np=H.uniforms(6, 17), what="degenerate k=%s p=%s" % (k, p))
    # infinities times a factor below one (temperature above log2 e) stay infinities before the clean-up
    # (sampling.cu:553); on the streaming path as well (forced: the call is smaller than it would take)
    big = np.tile(lg, (1, 40))
    _run_case(torch_cuda, oracle, capi, big, 4.0, 10, 0.9, u_np=H.uniforms(6, 18), what="degenerate T=4")


def test_masked_tokens_are_never_returned(torch_cuda, oracle):
    """Logits at -inf (or merely 41 octaves and more below the maximum) are dead: probability 0,
    as exp2f underflows in the reference (sampling.cu:235).  With nothing trimming the tail
    (top_k = -1, top_p = 1) and the uniform at its upper end they must still never come back."""
    from tests import capi
    torch = torch_cuda
    rng = np.random.default_rng(77)
    for V in (1 << 16, 1 << 18):
        B = 6
        lg = np.full((B, V), -np.inf, dtype=np.float32)
        live = []
        for b in range(B):
            n_live = [4, 4, 100, V // 2, 1, 4][b]
            ids = np.sort(rng.choice(V, size=n_live, replace=False))
            lg[b, ids] = rng.standard_normal(n_live).astype(np.float32) * 2
            if b == 1:
                lg[b, lg[b] == -np.inf] = -200.0                     # finite, but far below 2^-40 of the maximum
            if b == 5:
                lg[b, ids[-1] + 1:] = np.nan                         # cleaned to 0 by sf: live
                ids = np.concatenate([ids, np.arange(ids[-1] + 1, V)])
            live.append(set(ids.tolist()))
        for top_k, top_p in [(-1, 1.0), (1000, 1.0), (-1, 0.999999)]:
            for u in (1.0, float(np.nextafter(np.float32(1.0), np.float32(0.0))), 0.9999999):
                u_np = np.full(B, u, dtype=np.float32)
                res, ref = _run_case(torch, oracle, capi, lg, 1.0, top_k, top_p, u_np=u_np,
                                     what="masked V=%d k=%d p=%g u=%r" % (V, top_k, top_p, u))
                for b in range(B):
                    assert int(res["out"][b]) in live[b], (b, int(res["out"][b]))
                    assert res["diag"]["thr_bits"][b] >= 0x2B800000
                    dead = res["e_bits"][b] == 0
                    assert dead.sum() == V - len(live[b])


@pytest.mark.parametrize("B,V,top_k,top_p,gen", [(512, 256, 10, 0.9, 3), (512, 256, -1, 1.0, 0), (512, 256, 1, 0.1, 4),
                                                  (512, 262144, 10000, 0.7, 3), (512, 262144, -1, 0.1, 1)])
def test_corners_of_the_reference_benchmark_grid(torch_cuda, oracle, B, V, top_k, top_p, gen):
    """The extremes of the reference's benchmark sweep (/root/reference/bench.py:32-35: B up to 512, V from
    256 to 262144, top_k up to 10000, top_p down to 0.1) with its logit generators (bench.py:66-72:
    zeros, U[0,1), N(0,1)/2, N(0,1)*3, U[0,1)*4): 512 rows of one workgroup each, and 512 rows of a quarter
    million tokens with a kept set of thousands."""
    from tests import capi
    rng = np.random.default_rng(1000 * gen + V % 1000 + B)
    if gen == 0:
        lg = np.zeros((B, V), dtype=np.float32)
    elif gen == 1:
        lg = rng.random((B, V), dtype=np.float32)
    elif gen == 3:
        lg = rng.standard_normal((B, V), dtype=np.float32) * np.float32(3.0)
    else:
        lg = rng.random((B, V), dtype=np.float32) * np.float32(4.0)
    _run_case(torch_cuda, oracle, capi, lg, 1.0, top_k, top_p, u_np=H.uniforms(B, 55),
              what="sweep corner B=%d V=%d k=%d p=%g gen=%d" % (B, V, top_k, top_p, gen))


def test_uniform_extremes(torch_cuda, oracle):
    """u -> 0+ picks the first kept token, u = 1 the last one."""
    from tests import capi
    V = 8192
    lg = H.logits_normal(4, V, 2.0, seed=21)
    u = np.array([1.0, np.nextafter(np.float32(0), np.float32(1)), 1e-30, 0.5], dtype=np.float32)
    res, ref = _run_case(torch_cuda, oracle, capi, lg, 1.0, 20, 0.9, u_np=u, what="u extremes")
    e, thr = res["e_bits"], res["diag"]["thr_bits"]
    kept0 = np.nonzero(e[0] >= thr[0])[0]
    kept1 = np.nonzero(e[1] >= thr[1])[0]
    assert res["out"][0] == kept0[-1] and res["out"][1] == kept1[0]


def test_streaming_path_mixed_rows(torch_cuda, oracle):
    """Rows of one batch that end differently on the streaming path: top_k-bound rows finished from the
    stashes, rows where top_p cuts inside the stashes, peaked rows, masked (-inf) stretches that put whole
    slices in another frame, a row of ties too large to gather, NaN/Inf entries."""
    from tests import capi
    V = 65536 + 4096                 # 5 slices of 16384 tokens, the last one short
    rng = np.random.default_rng(77)
    lg = (rng.standard_normal((10, V)) * 2.0).astype(np.float32)
    lg[1, 1000] = 40.0                                   # one dominant token
    lg[2, 16384:49152] = -np.inf                         # two slices fully masked
    lg[3, :] = -np.inf; lg[3, 60000:60010] = 1.0         # almost everything masked, small tie
    lg[4, :] = 0.25                                      # all equal
    lg[5, 5] = np.nan; lg[5, 6] = np.inf; lg[5, 7] = -np.inf
    lg[6, 16384:32768] -= 200.0                          # a slice 288 octaves down: clamped in the row's frame
    lg[7, :32768] = lg[7, 32768]                         # a tie of 32768 tokens at a middling value
    lg[8, 20000:20600] = 9.0                             # a tie of 600 tokens at the top
    for (k, p) in [(50, 0.9), (1024, 0.95), (1, 1.0), (1000, 0.2), (7, 1.0), (1024, 1.0)]:
        _run_case(torch_cuda, oracle, capi, lg, 0.9, k, p, u_np=H.uniforms(10, 91), what="stream mixed k=%s p=%s" % (k, p))
    # which rows the streaming path finished from the stashes (diag.rounds == 0) and which the slow way
    rc, c, k, p = capi.normalize(0.9, 50, 0.9, V, 10, 1)
    res = capi.Sampler(10, V).sample(torch_cuda.from_numpy(lg).cuda(), c, k, p, path="stream",
                                     uniforms=torch_cuda.from_numpy(H.uniforms(10, 91)).cuda())
    rounds = res["diag"]["rounds"]
    assert rounds[0] == 0 and rounds[1] == 0 and rounds[8] == 0 and rounds[9] == 0, rounds
    # slices whose maxima are more than 87 octaves apart (rows 2, 3, 5, 6): what the far ones put
    # into the row's bins is taken out again, and the row is finished all the same
    assert all(rounds[i] == 0 for i in (2, 3, 5, 6)), rounds
    # a tie of all 69632 tokens needs no stash: recognised from the row's bins and finished as well
    assert rounds[4] == 0, rounds


def test_c5_full_size_paths_agree(torch_cuda, oracle):
    """BASELINE config 5 at its full size, (B,T,V) = (128,4,1048576) fp32 = 2 GiB, top_k 1024, top_p 0.95.
    Too large for the oracle in a test; checked through what does not depend on size: the streaming path
    and the cluster path are different decompositions of the same integer arithmetic, so every diagnostic
    and every index must be equal; and all 128 sampled rows are run through the oracle as well."""
    torch = torch_cuda
    from tests import capi
    B, T, V = 128, 4, 1048576
    g = torch.Generator(device="cuda")
    g.manual_seed(5)
    lg = torch.randn((B, T, V), generator=g, device="cuda", dtype=torch.float32) * 1.5
    rc, c, k, p = capi.normalize(1.0, 1024, 0.95, V, B, T)
    u = torch.from_numpy(H.uniforms(B, 123)).cuda()
    smp = capi.Sampler(B, V)
    res = {}
    for path in ("stream", "cluster", "stream"):
        print("full C5", path, flush=True)
        r = smp.sample(lg, c, k, p, uniforms=u, path=path)
        assert r["rc"] == 0 and smp.status() == 0
        if path in res:
            for f in FIELDS:
                assert np.array_equal(res[path]["diag"][f], r["diag"][f]), "repeat differs: " + f
        res[path] = r
    for f in FIELDS:
        assert np.array_equal(res["stream"]["diag"][f], res["cluster"]["diag"][f]), f
    assert np.array_equal(res["stream"]["out"], res["cluster"]["out"])
    assert (res["stream"]["diag"]["rounds"] == 0).all()            # every row finished by the streaming path
    d = res["stream"]["diag"]
    assert (d["n_gt"] < 1024).all() and (d["n_gt"] + d["n_eq"] >= 1).all()
    for lo in range(0, B, 32):                                       # 32 rows (128 MiB) at a time
        sub = lg[lo:lo + 32, T - 1, :].cpu().numpy()
        ref_out, ref_diag = oracle.sample_batch(sub, c, k, p, injected_u=H.uniforms(B, 123)[lo:lo + 32])
        for f in FIELDS:
            assert np.array_equal(d[f][lo:lo + 32], ref_diag[f]), (f, lo)
        assert np.array_equal(res["stream"]["out"][lo:lo + 32], ref_out), lo


@pytest.mark.parametrize("B,T,V,top_k,top_p,gen", [(512, 1, 262144, -1, 0.9, "u1"), (128, 4, 1048576, 10000, 0.95, "n15"),
                                                    (768, 1, 50304, 10000, 1.0, "u1"), (128, 1, 100256, 10000, 0.9, "u1"),
                                                    (30, 1, 1048576, 10000, 1.0, "n15")])
def test_wide_path_at_scale(torch_cuda, oracle, B, T, V, top_k, top_p, gen):
    """Kept sets of thousands of tokens at scale (the reference's benchmark grid has top_k 10000 and top_p
    0.9 on flat generators, /root/reference/bench.py:34-35, :66-72; its search costs the same whatever the
    kept set, sampling.cu:261-329): 512 flat rows of 262144 tokens under top_p 0.9, the bandwidth
    configuration's 128 rows of a million tokens with top_k 10000, 768 flat rows of 50304 tokens.  The
    library takes a wide path for the long rows by itself -- the one-pass one from 2^26 tokens per call on
    and, in rows of up to 262144 tokens, which it cuts into slices of 8192 tokens, from 12 million
    (diag.rounds == 9: 128 rows of 100256 tokens), the two-pass one below that in longer rows (7: 30 rows of a
    million), every row: none done the slow way -- and the row kernel
    for the rows of 50304 tokens (10); every row goes through the oracle, and the general kernel, both wide
    paths and, where the rows fit it, the row kernel must agree in every field."""
    torch = torch_cuda
    from tests import capi
    g = torch.Generator(device="cuda")
    g.manual_seed(50 + B)
    shape = (B, T, V) if T > 1 else (B, V)
    lg = torch.rand(shape, generator=g, device="cuda") if gen == "u1" else torch.randn(shape, generator=g, device="cuda") * 1.5
    rc, c, k, p = capi.normalize(1.0, top_k, top_p, V, B, T)
    u_np = H.uniforms(B, 321)
    u = torch.from_numpy(u_np).cuda()
    smp = capi.Sampler(B, V)
    res = {}
    for path in ("auto", "cluster", "wide", "wide1") + (("row",) if V <= 65536 else ()):
        print("wide at scale", B, T, V, path, flush=True)
        r = smp.sample(lg, c, k, p, uniforms=u, path=path)
        assert r["rc"] == 0 and smp.status() == 0
        res[path] = r
    auto_rounds = 10 if V <= 65536 else 9 if B * V >= (12000000 if V <= 262144 else 2 ** 26) else 7
    assert (res["auto"]["diag"]["rounds"] == auto_rounds).all(), np.unique(res["auto"]["diag"]["rounds"], return_counts=True)
    assert (res["wide"]["diag"]["rounds"] == 7).all()
    assert (res["wide1"]["diag"]["rounds"] == 9).all(), np.unique(res["wide1"]["diag"]["rounds"], return_counts=True)
    assert (res["cluster"]["diag"]["rounds"] < 7).all()
    for f in FIELDS:
        assert np.array_equal(res["auto"]["diag"][f], res["cluster"]["diag"][f]), f
        assert np.array_equal(res["auto"]["diag"][f], res["wide"]["diag"][f]), f
        assert np.array_equal(res["auto"]["diag"][f], res["wide1"]["diag"][f]), f
        if "row" in res:
            assert np.array_equal(res["auto"]["diag"][f], res["row"]["diag"][f]), f
    assert np.array_equal(res["auto"]["out"], res["cluster"]["out"])
    d = res["auto"]["diag"]
    step = 64 if V <= 262144 else 32
    for lo in range(0, B, step):
        sub = (lg[lo:lo + step, T - 1, :] if T > 1 else lg[lo:lo + step]).cpu().numpy()
        ref_out, ref_diag = oracle.sample_batch(sub, c, k, p, injected_u=u_np[lo:lo + step])
        for f in FIELDS:
            assert np.array_equal(d[f][lo:lo + step], ref_diag[f]), (f, lo)
        assert np.array_equal(res["auto"]["out"][lo:lo + step], ref_out), lo


def test_wide_path_unusual_rows(torch_cuda, oracle):
    """Rows the wide path's second pass cannot serve the usual way, each against the oracle on every path:
    a boundary bin that holds more than a quarter of a slice (flat rows at a temperature of 2: the waves'
    queues overflow and the slice is gone through again from memory); sorted rows, whose slices are no
    samples of the row at all, so that no slice's window covers the row's threshold (done the slow way,
    diag.rounds == 8); rows of a few distinct values (ties of thousands of tokens in one sub-bin); rows
    with masked stretches that put whole slices far below the row's frame; a tie of all tokens."""
    torch = torch_cuda
    from tests import capi
    V = 131072 + 8192
    rng = np.random.default_rng(123)
    lg = rng.random((8, V), dtype=np.float32)
    lg[1] = np.sort(lg[1])[::-1]                                      # descending: slice 0 holds the whole kept set
    lg[2] = np.sort(lg[2])                                            # ascending
    lg[3] = np.round(lg[3] * 16) / 16                                 # 17 distinct values
    lg[4, 16384:81920] = -np.inf                                      # four slices fully masked
    lg[5] = 0.5                                                       # one tie of all tokens
    lg[6] = (rng.standard_normal(V) * 1.5).astype(np.float32)
    lg[7, ::3] += 0.5                                                 # two populations
    for (temp, k, p) in [(2.0, -1, 0.9), (1.0, 10000, 1.0), (1.0, -1, 0.5), (0.7, 3000, 0.8)]:
        _run_case(torch, oracle, capi, lg, temp, k, p, u_np=H.uniforms(8, 61), what="wide unusual T=%g k=%d p=%g" % (temp, k, p))
    rc, c, k, p = capi.normalize(1.0, -1, 0.5, V, 8, 1)
    res = capi.Sampler(8, V).sample(torch.from_numpy(lg).cuda(), c, k, p, path="wide", uniforms=torch.from_numpy(H.uniforms(8, 61)).cuda())
    rounds = res["diag"]["rounds"]
    assert rounds[0] == 7 and rounds[4] == 7 and rounds[6] == 7 and rounds[7] == 7, rounds
    assert rounds[1] == 8 and rounds[2] == 8, rounds                # sorted rows: the slow way
    assert rounds[5] == 0, rounds                                   # one tie of all tokens: finished from the row's bins
    # The one-pass wide path: its sample is taken from all over the row and its window is a range of values,
    # so a sorted row is finished there when the one slice that holds the tokens around the threshold
    # can set all of them aside; rows of a few distinct values put thousands of ties into one sub-bin.
    res = capi.Sampler(8, V).sample(torch.from_numpy(lg).cuda(), c, k, p, path="wide1", uniforms=torch.from_numpy(H.uniforms(8, 61)).cuda())
    rounds = res["diag"]["rounds"]
    assert rounds[0] == 9 and rounds[4] == 9 and rounds[6] == 9 and rounds[7] == 9, rounds
    assert rounds[1] in (8, 9) and rounds[2] in (8, 9) and rounds[3] == 8 and rounds[5] == 0, rounds


def test_one_pass_wide_path_on_slices_of_8192_tokens_unusual_rows(torch_cuda, oracle):
    """From 12 million tokens per call on, rows of up to 262144 tokens take the one-pass wide path on slices
    of 8192 tokens (diag.rounds == 9) when the workspace has the room rs_workspace_bytes asks for.  The rows
    of test_wide_path_unusual_rows twelve times over, 96 rows of 139264 tokens (17 slices each): sorted rows,
    few distinct values, masked slices, one tie of all tokens, two populations; every row against the oracle,
    the general kernel and the two-pass path equal in every field; rows the sample misjudges may go the slow
    way (8), a tie of all tokens is finished from the row's bins (0)."""
    torch = torch_cuda
    from tests import capi
    V, reps = 131072 + 8192, 12
    rng = np.random.default_rng(124)
    lg8 = rng.random((8, V), dtype=np.float32)
    lg8[1] = np.sort(lg8[1])[::-1]
    lg8[2] = np.sort(lg8[2])
    lg8[3] = np.round(lg8[3] * 16) / 16
    lg8[4, 16384:81920] = -np.inf
    lg8[5] = 0.5
    lg8[6] = (rng.standard_normal(V) * 1.5).astype(np.float32)
    lg8[7, ::3] += 0.5
    lg_np = np.tile(lg8, (reps, 1))
    B = 8 * reps
    lg = torch.from_numpy(lg_np).cuda()
    u_np = H.uniforms(B, 66)
    u = torch.from_numpy(u_np).cuda()
    for (temp, k, p) in [(1.0, 10000, 1.0), (2.0, -1, 0.9)]:
        rc, c, kk, pp = capi.normalize(temp, k, p, V, B, 1)
        ref_out, ref_diag = oracle.sample_batch(lg_np, c, kk, pp, injected_u=u_np)
        smp = capi.Sampler(B, V)
        res = {}
        for path in ("auto", "wide1", "wide", "cluster"):
            print("short slices, unusual rows", temp, k, p, path, flush=True)
            res[path] = smp.sample(lg, c, kk, pp, uniforms=u, path=path)
            assert res[path]["rc"] == 0 and smp.status() == 0
            _check(res[path], ref_out, ref_diag, "short slices T=%g k=%d p=%g path %s" % (temp, k, p, path))
        rounds = res["auto"]["diag"]["rounds"]
        assert np.isin(rounds, (0, 8, 9)).all() and (rounds == 9).sum() >= 4 * reps, np.unique(rounds, return_counts=True)
        assert np.array_equal(rounds, res["wide1"]["diag"]["rounds"])
        smp.close()


def test_row_kernel_unusual_rows(torch_cuda, oracle):
    """The row kernel (one workgroup per row, the row in its registers) on rows that take each of its ways:
    a boundary bin of more tokens than its list holds (flat rows at a temperature of 2: every level counted
    from the registers), sorted rows (a stretch per wave: the whole kept set in one wave's), rows of a few
    distinct values (ties of thousands), masked stretches, a tie of all tokens, a row with one live token,
    NaNs, few kept tokens (groups without one skipped); against the oracle on every path, in rows of every
    length class the kernel is built for, float32, bfloat16 and half."""
    torch = torch_cuda
    from tests import capi
    rng = np.random.default_rng(321)
    for V in (65536, 50304, 20480, 12288, 4100, 64):
        lg = rng.random((10, V), dtype=np.float32)
        lg[1] = np.sort(lg[1])[::-1]
        lg[2] = np.sort(lg[2])
        lg[3] = np.round(lg[3] * 16) / 16
        lg[4, V // 8:V // 8 * 5] = -np.inf
        lg[5] = 0.5
        lg[6] = (rng.standard_normal(V) * 1.5).astype(np.float32)
        lg[7, ::3] += 0.5
        lg[8] = -np.inf
        lg[8, V - 3] = 1.0
        lg[9, :V // 16] = np.nan
        cases = [(2.0, -1, 0.9), (1.0, 10000, 1.0), (1.0, 40, 0.95)] if V >= 20480 else [(2.0, -1, 0.9), (1.0, 40, 0.95)]
        for (temp, k, p) in cases:
            _run_case(torch, oracle, capi, lg, temp, k, p, u_np=H.uniforms(10, 62), what="row kernel V=%d T=%g k=%d p=%g" % (V, temp, k, p))
    for fmt in (torch.bfloat16, torch.float16):
        lg = torch.from_numpy((rng.standard_normal((6, 50304)) * 3).astype(np.float32)).to(fmt).float().numpy()
        _run_case(torch, oracle, capi, lg, 1.0, -1, 0.9, u_np=H.uniforms(6, 63), dtype=fmt, what="row kernel %s" % fmt)


def test_row_kernel_takes_the_wide_kept_sets_of_calls_of_many_short_rows(torch_cuda, oracle):
    """Calls of 128 rows and more (64 in rows of fewer than 32768 tokens) of 8192 to 65536 tokens whose kept
    sets the stashes cannot hold go to the row kernel by themselves (diag.rounds == 10): a top_k of
    thousands at once, a nucleus once the probe has reported its long lists; fewer rows, longer rows, 257
    to 511 rows of fewer than 40000 tokens, more than 256 rows of fewer than 32768 and calls with a bounding
    top_k do not.  Every call against the general kernel in every field, 64 rows of each against the oracle."""
    torch = torch_cuda
    from tests import capi
    for (B, V, k, p, row) in [(128, 50304, 10000, 1.0, True), (300, 16384, 5000, 1.0, False), (200, 16384, 5000, 1.0, True),
                              (127, 50304, 10000, 1.0, False), (160, 65540, 10000, 1.0, False), (256, 32768, 50, 0.9, False),
                              (300, 32768, 5000, 1.0, False), (520, 32768, -1, 0.9, True), (64, 8192, 2000, 1.0, True)]:
        lg_np = H.logits_uniform(B, V, seed=B)
        lg = torch.from_numpy(lg_np).cuda()
        rc, c, kk, pp = capi.normalize(1.0, k, p, V, B, 1)
        u_np = H.uniforms(B, 64)
        u = torch.from_numpy(u_np).cuda()
        smp = capi.Sampler(B, V, with_policy=True, init=True)
        print("row kernel routing", B, V, k, p, flush=True)
        res = None
        for call in range(3 if k == -1 else 1):                  # a nucleus: a probe first, then calls that know
            res = smp.sample(lg, c, kk, pp, uniforms=u)
            assert res["rc"] == 0 and smp.status() == 0
        rounds = res["diag"]["rounds"]
        assert ((rounds == 10).all() if row else (rounds != 10).all()), (B, V, k, p, np.unique(rounds, return_counts=True))
        ref = smp.sample(lg, c, kk, pp, uniforms=u, path="cluster")
        for f in FIELDS:
            assert np.array_equal(res["diag"][f], ref["diag"][f]), f
        assert np.array_equal(res["out"], ref["out"])
        ref_out, ref_diag = oracle.sample_batch(lg_np[B - 64:], c, kk, pp, injected_u=u_np[B - 64:])
        for f in FIELDS:
            assert np.array_equal(res["diag"][f][B - 64:], ref_diag[f]), f
        assert np.array_equal(res["out"][B - 64:], ref_out)
        smp.close()
    # A bounding top_k whose rows have long lists all the same (flat rows, top_k 1000): the streaming finish
    # says so to the policy in every call the row kernel suits, whatever its size (elsewhere only in calls of
    # fewer than 2^24 tokens), and the calls after it go to the row kernel
    B, V = 520, 50304
    lg_np = H.logits_uniform(B, V, seed=77)
    lg = torch.from_numpy(lg_np).cuda()
    rc, c, kk, pp = capi.normalize(1.0, 1000, 1.0, V, B, 1)
    u_np = H.uniforms(B, 65)
    u = torch.from_numpy(u_np).cuda()
    smp = capi.Sampler(B, V, with_policy=True, init=True)
    first = smp.sample(lg, c, kk, pp, uniforms=u)
    assert first["rc"] == 0 and (first["diag"]["rounds"] != 10).all() and smp.policy_state() == 2
    res = smp.sample(lg, c, kk, pp, uniforms=u)
    assert res["rc"] == 0 and (res["diag"]["rounds"] == 10).all() and smp.policy_state() == 2 and smp.status() == 0
    ref_out, ref_diag = oracle.sample_batch(lg_np[:64], c, kk, pp, injected_u=u_np[:64])
    for f in FIELDS:
        assert np.array_equal(res["diag"][f], first["diag"][f]), f
        assert np.array_equal(res["diag"][f][:64], ref_diag[f]), f
    assert np.array_equal(res["out"], first["out"]) and np.array_equal(res["out"][:64], ref_out)
    smp.close()
    # the library's own random numbers: drawn as on every other path, the state left as the oracle leaves it
    B, V = 130, 12288
    lg_np = H.logits_normal(B, V, 0.5, seed=51)
    rc, c, k, p = capi.normalize(1.0, 3000, 1.0, V, B, 1)
    smp = capi.Sampler(B, V)
    lg = torch.from_numpy(lg_np).cuda()
    st = torch.empty(B * 64, dtype=torch.int8, device="cuda")
    assert capi.lib().rs_philox_init(st.data_ptr(), 987654321, B, smp.stream()) == 0
    rng_ref = oracle.rng_init(987654321, B)
    for call in range(3):
        ref_out, ref_diag = oracle.sample_batch(lg_np, c, k, p, rng=rng_ref)
        res = smp.sample(lg, c, k, p, rng=st)
        _check(res, ref_out, ref_diag, "row kernel, philox call %d" % call)
        assert (res["diag"]["rounds"] == 10).all()
    assert np.array_equal(st.cpu().numpy().view(np.uint32).reshape(B, 16), rng_ref)


def test_wide_path_reports_slow_rows(torch_cuda, oracle):
    """Calls on the two-pass wide path that are given a policy report rows done the slow way in a word of
    their own (rs_policy_state bit 3): the next calls of that kind take the general kernel, the wide path is
    tried again after 64 of them, and a call that goes well clears the word through the call after it."""
    torch = torch_cuda
    from tests import capi
    B, V = 30, 1048576                                   # (the two-pass path by itself: long rows, fewer than 2^26 tokens)
    good = H.logits_uniform(B, V, seed=71)
    bad = good.copy()
    bad[11] = np.sort(bad[11])
    # top_k 20000 of a sorted row: the boundary bin's tokens lie in two slices, the upper part in one and the
    # lower part in the other, so neither slice's share says where in the bin the row's threshold is
    rc, c, k, p = capi.normalize(1.0, 20000, 1.0, V, B, 1)
    u_np = H.uniforms(B, 72)
    u = torch.from_numpy(u_np).cuda()
    ref_good = oracle.sample_batch(good, c, k, p, injected_u=u_np)
    ref_bad = oracle.sample_batch(bad, c, k, p, injected_u=u_np)
    lg_good, lg_bad = torch.from_numpy(good).cuda(), torch.from_numpy(bad).cuda()
    smp = capi.Sampler(B, V, with_policy=True, init=True)
    res = smp.sample(lg_good, c, k, p, uniforms=u)
    _check(res, *ref_good, "wide, fair rows")
    assert (res["diag"]["rounds"] == 7).all() and smp.policy_state() == 0
    res = smp.sample(lg_bad, c, k, p, uniforms=u)
    _check(res, *ref_bad, "wide, one sorted row")
    assert res["diag"]["rounds"][11] == 8 and (np.delete(res["diag"]["rounds"], 11) == 7).all() and smp.policy_state() == 8
    for i in range(3):
        res = smp.sample(lg_good, c, k, p, uniforms=u)
        _check(res, *ref_good, "after a slow row %d" % i)
        assert (res["diag"]["rounds"] < 7).all() and smp.policy_state() == 8       # general kernel
    for i in range(64):
        res = smp.sample(lg_good, c, k, p, uniforms=u, want_diag=False)
        assert res["rc"] == 0 and np.array_equal(res["out"], ref_good[0])
    assert smp.policy_state() == 0
    res = smp.sample(lg_good, c, k, p, uniforms=u)
    assert (res["diag"]["rounds"] == 7).all() and smp.policy_state() == 0 and smp.status() == 0
    smp.close()


def test_one_pass_wide_path_hands_over_to_the_two_pass_one(torch_cuda, oracle):
    """From 2^26 tokens per call on, kept sets of thousands of tokens take the one-pass wide path (a sample of
    each row decides what the one pass over it counts finely and sets aside; diag.rounds == 9).  A row of
    which the sample is no fair picture (its 30000 largest tokens all lie in stretches the sample does not
    look at, so the threshold is nowhere near where the sample expects it) is done the slow way (8) and
    reported in a word of that path's own (rs_policy_state bit 2); the next calls take the two-pass wide
    path (7), which counts everything, the one-pass path is tried again after 64 of them, and a call
    that goes well clears the word through the call after it.  Every result equals the oracle's."""
    torch = torch_cuda
    from tests import capi
    B, V = 72, 1048576
    rng = np.random.default_rng(171)
    good = (rng.standard_normal((B, V), dtype=np.float32) * np.float32(1.5)).astype(np.float32)
    rc, c, k, p = capi.normalize(1.0, 20000, 1.0, V, B, 1)
    u_np = H.uniforms(B, 172)
    u = torch.from_numpy(u_np).cuda()
    ref_good = oracle.sample_batch(good, c, k, p, injected_u=u_np)
    # the sample of a row of 2^20 tokens: 256 tokens out of every 8192, from the middle of the stretch
    odd_row = good[11].copy()
    odd_row.reshape(-1, 8192)[:, :256] += np.float32(8.0)
    ref_odd = oracle.sample_batch(odd_row[None, :], c, k, p, injected_u=u_np[11:12])
    ref_bad = (ref_good[0].copy(), ref_good[1].copy())
    ref_bad[0][11] = ref_odd[0][0]
    ref_bad[1][11] = ref_odd[1][0]
    lg_good = torch.from_numpy(good).cuda()
    lg_bad = lg_good.clone()
    lg_bad[11] = torch.from_numpy(odd_row).cuda()
    smp = capi.Sampler(B, V, with_policy=True, init=True)
    res = smp.sample(lg_good, c, k, p, uniforms=u)
    _check(res, *ref_good, "one pass, fair rows")
    assert (res["diag"]["rounds"] == 9).all() and smp.policy_state() == 0
    res = smp.sample(lg_bad, c, k, p, uniforms=u)
    _check(res, *ref_bad, "one pass, one row the sample misjudges")
    assert res["diag"]["rounds"][11] == 8 and (np.delete(res["diag"]["rounds"], 11) == 9).all() and smp.policy_state() == 4
    for i in range(3):
        res = smp.sample(lg_good, c, k, p, uniforms=u)
        _check(res, *ref_good, "after a slow row %d" % i)
        assert (res["diag"]["rounds"] == 7).all() and smp.policy_state() == 4      # the two-pass wide path
    for i in range(64):
        res = smp.sample(lg_good, c, k, p, uniforms=u, want_diag=False)
        assert res["rc"] == 0 and np.array_equal(res["out"], ref_good[0])
    assert smp.policy_state() == 0
    res = smp.sample(lg_good, c, k, p, uniforms=u)
    assert (res["diag"]["rounds"] == 9).all() and smp.policy_state() == 0 and smp.status() == 0
    smp.close()


def test_streaming_path_flat_distributions(torch_cuda, oracle):
    """Flat rows with a small top_k: the bin in which the count reaches top_k holds thousands of tokens, so
    a slice refines its cut inside that bin and the finish works on the whole stashes (the reference's
    benchmark generators, /root/reference/bench.py:66-72: zeros, U[0,1), N(0,1)/2, N(0,1)*3, U[0,1)*4)."""
    from tests import capi
    V = 65536 + 8192
    rng = np.random.default_rng(5)
    lg = np.zeros((7, V), dtype=np.float32)
    lg[1] = rng.random(V, dtype=np.float32)
    lg[2] = rng.standard_normal(V, dtype=np.float32) / 2
    lg[3] = rng.standard_normal(V, dtype=np.float32) * 3
    lg[4] = rng.random(V, dtype=np.float32) * 4
    lg[5] = rng.random(V, dtype=np.float32) * 1e-3                      # everything within a thousandth of an octave
    lg[6] = np.round(rng.random(V, dtype=np.float32) * 64) / 64         # 65 distinct values: ties of a thousand tokens
    for (k, p) in [(100, 0.9), (10, 1.0), (1000, 0.3), (1, 1.0), (1024, 1.0)]:
        _run_case(torch_cuda, oracle, capi, lg, 1.0, k, p, u_np=H.uniforms(7, 41), what="flat k=%s p=%s" % (k, p))
    rc, c, k, p = capi.normalize(1.0, 100, 0.9, V, 7, 1)
    res = capi.Sampler(7, V).sample(torch_cuda.from_numpy(lg).cuda(), c, k, p, path="stream",
                                    uniforms=torch_cuda.from_numpy(H.uniforms(7, 41)).cuda())
    rounds = res["diag"]["rounds"]
    assert all(rounds[i] == 0 for i in (1, 2, 3, 4, 6)), rounds     # finished from the stashes
    assert rounds[0] == 0, rounds                                   # all equal: one tie, recognised as such
    # the slow way: a row so flat that even a level-2 sub-bin holds more tokens than a stash
    assert rounds[5] >= 1, rounds


@pytest.mark.parametrize("B,V", [(6, 65536 + 4096), (20, 262144 + 4096)])
def test_streaming_path_peaked_and_masked_rows(torch_cuda, oracle, B, V):
    """Rows whose tokens mostly lie below 2^-40 of the maximum (wide or cold distributions, masked
    vocabulary): the streaming kernel counts such tokens by their own exponents and folds them into
    the lowest bin, refines a cut inside that bin with their number added analytically, and the
    finishing kernel takes slices far below the row's frame out of the row's bins again.  Short slices
    (first shape) and long slices (second).  Every row must equal the oracle's on every path, and all
    (the row of ties too) must be finished by the streaming path itself."""
    from tests import capi
    rng = np.random.default_rng(123)
    lg = np.empty((B, V), dtype=np.float32)
    sig = [6.0, 15.0, 40.0, 100.0, 1000.0]
    for b in range(B):
        lg[b] = rng.standard_normal(V, dtype=np.float32) * np.float32(sig[b % len(sig)])
    lg[1, : V // 2] = -np.inf                            # half the vocabulary masked, slices and all
    lg[2, 1::2] = -1e9                                   # every other token masked: no slice is empty
    lg[3, :] = -np.inf; lg[3, V - 7:] = rng.standard_normal(7)   # seven live tokens in the last, short slice
    lg[4, 4096:8192] += 500.0                            # one short slice (a quarter of a long one) far above the rest
    lg[5, :] = 1.0                                       # one tie
    u = H.uniforms(B, 17)
    for (k, p, t) in [(50, 0.9, 1.0), (1024, 1.0, 0.7), (3, 0.5, 0.05), (1000, 0.999, 4.0)]:
        _run_case(torch_cuda, oracle, capi, lg, t, k, p, u_np=u, what="peaked k=%s p=%s T=%s" % (k, p, t))
    rc, c, k, p = capi.normalize(1.0, 50, 0.9, V, B, 1)
    res = capi.Sampler(B, V).sample(torch_cuda.from_numpy(lg).cuda(), c, k, p, path="stream",
                                    uniforms=torch_cuda.from_numpy(u).cuda())
    rounds = res["diag"]["rounds"]
    assert all(rounds[i] == 0 for i in range(B)), rounds


def test_streaming_path_whole_slice_stash_beside_partial_ones(torch_cuda, oracle):
    """A wide row whose largest token sits in the short last slice: that slice's stash takes all of
    the slice, tokens at 2^-40 included, while the other slices' stashes stop above 2^-40 of their
    own, lower frames.  In the row's frame those slices' tokens all weigh 2^-40 and are not in any
    stash, so the stashes are complete only above 2^-40 and a threshold at 2^-40 (top_k larger than the
    handful of tokens above it) must not be decided from them."""
    from tests import capi
    rng = np.random.default_rng(2024)
    B, V = 6, 13 * 4096 + 648
    lg = (rng.standard_normal((B, V)) * 60.0).astype(np.float32)
    for b in range(3):
        lg[b, V - 5 - b] = lg[b].max() + np.float32(3.0 * b)        # the row's maximum in the last slice
    lg[3, 7] = lg[3].max() + np.float32(1.0)                        # and in the first, for comparison
    lg[4] = (rng.standard_normal(V) * 3.0).astype(np.float32); lg[4, V - 1] = lg[4].max() + np.float32(0.5)
    u = H.uniforms(B, 23)
    for (k, p, t) in [(100, 1.0, 0.8), (10, 0.9, 1.0), (1024, 1.0, 0.8), (1000, 0.999, 0.05)]:
        _run_case(torch_cuda, oracle, capi, lg, t, k, p, u_np=u, what="last-slice maximum k=%s p=%s T=%s" % (k, p, t))


def test_cluster_levels_with_slices_that_hold_no_boundary_tokens(torch_cuda, oracle):
    """Many rows whose threshold is a tie of thousands of tokens lying in one contiguous range (a
    masked range with everything kept: the tie at 2^-40; a range of equal largest logits): the
    cluster kernel goes through every histogram level, and the slices outside the range add nothing
    to the deeper levels, so their workgroups are not needed for those levels to complete.  A
    histogram may therefore be cleared only after an exchange every workgroup takes part in; clearing
    it after the next level left a slower workgroup polling zeros until its wait gave up.  More
    workgroups than the GPU holds at once, several calls: every result equals the oracle's and no
    wait gives up."""
    from tests import capi
    rng = np.random.default_rng(77)
    B, V = 100, 78712
    lg = (rng.standard_normal((B, V)) * 2.0).astype(np.float32)
    for b in range(B):
        lo = int(rng.integers(0, V - 1)); n = int(rng.integers(1100, V // 3))
        if b % 2 == 0:
            lg[b, lo: lo + n] = -np.inf
        else:
            lg[b, lo: lo + n] = lg[b].max() + np.float32(0.25)
    u = H.uniforms(B, 31)
    for (k, p, t) in [(-1, 1.0, 0.8), (-1, 0.999, 1.0), (5000, 1.0, 1.3)]:
        for rep in range(2):
            _run_case(torch_cuda, oracle, capi, lg, t, k, p, u_np=u, what="contiguous ties k=%s p=%s T=%s #%d" % (k, p, t, rep))


def test_cluster_rows_whose_slices_lie_in_frames_far_apart_beside_flat_ones(torch_cuda, oracle):
    """General kernel, a dozen calls on one workspace: rows whose slices lie in frames too far apart for
    the shared octave positions (whole slices masked), which redo level 1 in the row's frame and clear
    the first histogram early, beside flat rows, whose boundary bin takes a further level over the
    cluster, and sorted rows, whose slices hold different bins.  Every call against the oracle; the
    workspace must stay clean from call to call."""
    torch = torch_cuda
    from tests import capi
    B, V = 12, 266240
    rng = np.random.default_rng(321)
    lg = (rng.standard_normal((B, V)) * 15).astype(np.float32)
    lg[1, : V // 2] = -np.inf
    lg[3, :] = -np.inf; lg[3, V - 7:] = rng.standard_normal(7)
    lg[5] = rng.random(V, dtype=np.float32)
    lg[6] = np.sort(rng.random(V, dtype=np.float32))
    lg[7, 40000:200000] = -np.inf
    lg[8] = rng.random(V, dtype=np.float32) * 4
    u_np = H.uniforms(B, 322)
    smp = capi.Sampler(B, V)
    L, U = torch.from_numpy(lg).cuda(), torch.from_numpy(u_np).cuda()
    for (t, k, p) in [(1.0, -1, 0.5), (0.7, 3000, 1.0), (1.0, 50, 0.9)]:
        rc, c, kk, pp = capi.normalize(t, k, p, V, B, 1)
        ref_out, ref_diag = oracle.sample_batch(lg, c, kk, pp, injected_u=u_np)
        for it in range(4):
            res = smp.sample(L, c, kk, pp, uniforms=U, path="cluster")
            _check(res, ref_out, ref_diag, "frames far apart, T=%g k=%d p=%g call %d" % (t, k, p, it))
            assert smp.status() == 0


@pytest.mark.parametrize("fmt", ["float32", "bfloat16", "float16"])
def test_streaming_path_middle_slices(torch_cuda, oracle, fmt):
    """Calls whose 4096-token slices no longer fit the device at once but whose 8192-token slices do
    (here 52 rows of 150 000 tokens: 1924 short slices, 988 middle ones) take the streaming pass with
    slices of 8192 tokens: rows of every kind the seeded generator makes, the last slice ragged, in
    all three logit formats, through every path."""
    torch = torch_cuda
    from tests import capi
    dtype = None if fmt == "float32" else getattr(torch, fmt)
    rng = np.random.default_rng(8192)
    B, V = 52, 150000
    lg = np.stack([_random_row(rng, b % 11, V) for b in range(B)])
    if dtype is not None:
        lg = torch.from_numpy(lg).to(dtype).float().numpy()
    for (k, p, t) in [(50, 0.9, 0.8), (-1, 0.3, 1.0), (1024, 0.95, 1.5)]:
        _run_case(torch, oracle, capi, lg, t, k, p, u_np=H.uniforms(B, 8192), dtype=dtype,
                  what="middle slices %s k=%s p=%s T=%s" % (fmt, k, p, t))


@pytest.mark.parametrize("B,V", [(2, 1048576), (2, 524288), (3, 528384), (1, 1000000)])
def test_streaming_path_few_long_rows(torch_cuda, oracle, B, V):
    """A few rows of more than 262144 tokens are cut into up to 128 slices of 4096 or 8192 tokens
    (instead of 16384): rows of several kinds, a ragged last slice, a nucleus, a bounding top_k and
    both, through every path."""
    from tests import capi
    rng = np.random.default_rng(V + B)
    lg = np.stack([_random_row(rng, (2, 6, 4, 8)[b % 4], V) for b in range(B)])
    for (k, p, t) in [(50, 0.9, 0.8), (-1, 0.3, 1.0), (1000, 1.0, 1.2)]:
        _run_case(torch_cuda, oracle, capi, lg, t, k, p, u_np=H.uniforms(B, 77),
                  what="few long rows B=%d V=%d k=%s p=%s T=%s" % (B, V, k, p, t))


@pytest.mark.parametrize("B,V,k", [(4, 262144, 1000), (3, 262144, 1024), (24, 100256, 1000), (2, 1048576, 600), (6, 152064, 700)])
def test_streaming_path_flat_rows_more_stashed_than_listed(torch_cuda, oracle, B, V, k):
    """Flat rows (the reference's benchmark generators U[0,1), U[0,1)*4, N(0,1)/2) with a top_k of
    several hundred, cut into many slices: the boundary bin holds tens of thousands of tokens, every
    slice stashes several times its share of top_k, and the stashes together hold more tokens than
    the finishing workgroup's list.  It then counts the stashed tokens in steps of 1/512 octave below
    the row's largest, takes those down to the step at which there are top_k of them, and goes on from
    there: such rows finish on the streaming path (diag.rounds == 0), with a nucleus or without."""
    from tests import capi
    torch = torch_cuda
    rng = np.random.default_rng(V + k)
    gens = [lambda: rng.random(V, dtype=np.float32), lambda: rng.random(V, dtype=np.float32) * np.float32(4),
            lambda: rng.standard_normal(V, dtype=np.float32) * np.float32(0.5)]
    lg = np.stack([gens[b % 3]() for b in range(B)])
    for (p, t) in [(1.0, 1.0), (0.9, 1.0), (0.3, 0.7)]:
        _run_case(torch, oracle, capi, lg, t, k, p, u_np=H.uniforms(B, k + int(p * 10)),
                  what="flat rows B=%d V=%d k=%d p=%s T=%s" % (B, V, k, p, t))
    rc, c, kk, pp = capi.normalize(1.0, k, 1.0, V, B, 1)
    smp = capi.Sampler(B, V)
    res = smp.sample(torch.from_numpy(lg).cuda(), c, kk, pp, uniforms=torch.from_numpy(H.uniforms(B, 1)).cuda(), path="stream")
    assert (res["diag"]["rounds"] == 0).all(), res["diag"]["rounds"]
    # a call of this size (fewer than 2^24 tokens) says so to a caller's policy all the same: the general
    # kernel does such a call faster, and the next one goes there
    pol = capi.Sampler(B, V, with_policy=True, init=True)
    u = torch.from_numpy(H.uniforms(B, 1)).cuda()
    first = pol.sample(torch.from_numpy(lg).cuda(), c, kk, pp, uniforms=u)
    assert (first["diag"]["rounds"] == 0).all() and np.array_equal(first["out"], res["out"])
    if V * B < (1 << 24) and V != 152064:                # (6, 152064, 700): the stashes fit the list, nothing to report
        assert pol.policy_state() == 2
        second = pol.sample(torch.from_numpy(lg).cuda(), c, kk, pp, uniforms=u)
        assert (second["diag"]["rounds"] >= 1).all() and np.array_equal(second["out"], res["out"])
    pol.close()


@pytest.mark.parametrize("B,V", [(11, 50304), (4, 262144), (40, 152064), (2, 1048576), (3, 528384), (1, 4096)])
def test_streaming_path_keeps_everything(torch_cuda, oracle, B, V):
    """Plain temperature sampling (top_k = V, top_p = 1): every live token is kept, so there is no
    kept set to stash.  The streaming pass only counts; the finishing workgroup takes each slice's mass
    from the slice's bins (moved into the row's frame), finds the slice that holds the target and looks
    at that slice's logits once more.  Rows of every kind (ties, masks, slices whose maxima lie
    hundreds of octaves apart, most of the row dead, NaN and Inf), ragged last slices, every slice
    length, several temperatures; _run_case forces the path (twice) next to the general kernel and
    compares the token, every diagnostic (the threshold is the smallest live token, its ties counted)
    and the e of every token.  Then the same calls the way a caller makes them (no diagnostics, random
    numbers from the Philox state): the tokens and the advanced states must equal the general kernel's."""
    from tests import capi
    torch = torch_cuda
    rng = np.random.default_rng(V * 31 + B)
    lg = np.stack([_random_row(rng, (2, 9, 6, 4, 0, 8, 10, 1, 7, 5, 3)[b % 11], V) for b in range(B)])
    for t in (1.0, 0.7, 3.0):
        _run_case(torch, oracle, capi, lg, t, -1, 1.0, u_np=H.uniforms(B, int(t * 10) + V % 97),
                  what="keep all B=%d V=%d T=%s" % (B, V, t))
    rc, c, k, p = capi.normalize(1.0, -1, 1.0, V, B, 1)
    assert rc == 0 and k == V
    lgd = torch.from_numpy(lg).cuda()
    smp = capi.Sampler(B, V)
    rounds = smp.sample(lgd, c, k, p, uniforms=torch.from_numpy(H.uniforms(B, 3)).cuda(), path="stream")["diag"]["rounds"]
    assert ((rounds == 9) | (rounds == 0)).all() and (rounds == 9).any(), rounds    # 0: a row of equal logits, by division
    rng_ref = oracle.rng_init(1234 + V, B)
    ref = np.stack([oracle.sample_batch(lg, c, k, p, rng=rng_ref)[0] for _ in range(3)])
    for path in ("cluster", "stream", None):
        st = torch.empty(B * 64, dtype=torch.int8, device="cuda")
        assert capi.lib().rs_philox_init(st.data_ptr(), 1234 + V, B, smp.stream()) == 0
        res = [smp.sample(lgd, c, k, p, rng=st, want_diag=False, path=path)["out"] for _ in range(3)]
        assert smp.status() == 0
        assert np.array_equal(np.stack(res), ref), path
        assert np.array_equal(st.cpu().numpy().view(np.uint32).reshape(B, 16), rng_ref), path


@pytest.mark.parametrize("fmt", ["bfloat16", "float16"])
def test_half_precision_logits(torch_cuda, oracle, fmt):
    """Logits handed over as bfloat16 or float16 (rs_sample_dtype; an extension, the reference takes
    float32 only): both widen to float32 exactly, so every result must equal the oracle's on the widened
    values -- cluster path with the e bit patterns, streaming path with short and long slices, (B,T,V)
    addressing, masked and infinite entries, the penalty kernel."""
    torch = torch_cuda
    from tests import capi
    dtype = getattr(torch, fmt)
    rng = np.random.default_rng(321)

    def rounded(a):
        return torch.from_numpy(a).to(dtype).float().numpy()

    for (B, V, sigma) in [(5, 65536 + 4096, 3.0), (20, 262144 + 4096, 2.0)]:
        lg = rounded((rng.standard_normal((B, V)) * sigma).astype(np.float32))
        lg[1, : V // 3] = -np.inf
        lg[2, 17] = np.inf
        lg[3, 1::2] = rounded(np.full(1, -30000.0, dtype=np.float32))[0]
        for (k, p, t) in [(50, 0.9, 1.0), (-1, 0.3, 0.7), (1024, 1.0, 2.0)]:
            _run_case(torch, oracle, capi, lg, t, k, p, u_np=H.uniforms(B, 5), dtype=dtype,
                      what="%s B=%d V=%d k=%s p=%s T=%s" % (fmt, B, V, k, p, t))
    lg3 = rounded(rng.standard_normal((3, 4, 32768)).astype(np.float32) * 2)
    _run_case(torch, oracle, capi, lg3, 0.8, 40, 0.95, u_np=H.uniforms(3, 6), dtype=dtype, what=fmt + " (B,T,V)")
    lgp = rounded(rng.standard_normal((4, 131072)).astype(np.float32) * 1.5)
    pen = (rng.random((4, 131072)) < 0.02).astype(np.float32) * rng.exponential(1.0, (4, 131072)).astype(np.float32)
    _run_case(torch, oracle, capi, lgp, 0.8, 50, 0.9, pen_np=pen, u_np=H.uniforms(4, 7), presence=0.1, repetition=0.1,
              decay=0.95, dtype=dtype, what=fmt + " penalties")


def test_seeded_random_shapes_and_parameters(torch_cuda, oracle):
    """A hundred seeded random cases -- batch, vocabulary (any multiple of 4, so most slices end ragged),
    temperature, top_k, top_p and the kind of logits (the reference's five generators of bench.py:66-72,
    plus rows with masked stretches and rows of few distinct values) -- each through every path."""
    from tests import capi
    rng = np.random.default_rng(20250101)
    for case in range(100):
        B = int(rng.integers(1, 24))
        V = 4 * int(rng.integers(1, 50000)) if case % 3 else 4 * int(rng.integers(1, 2000))
        if case % 10 == 9:
            B, V = int(rng.integers(1, 8)), 4 * int(rng.integers(65537, 100000))      # long slices on the streaming path
        kind = int(rng.integers(0, 7))
        if kind == 0:
            lg = np.zeros((B, V), dtype=np.float32)
        elif kind == 1:
            lg = rng.random((B, V), dtype=np.float32)
        elif kind == 2:
            lg = rng.standard_normal((B, V), dtype=np.float32) / np.float32(2)
        elif kind == 3:
            lg = rng.standard_normal((B, V), dtype=np.float32) * np.float32(3)
        elif kind == 4:
            lg = rng.random((B, V), dtype=np.float32) * np.float32(4)
        elif kind == 5:
            lg = rng.standard_normal((B, V), dtype=np.float32) * np.float32(2)
            lo = int(rng.integers(0, V))
            lg[:, lo: lo + int(rng.integers(1, V))] = -np.inf
        else:
            lg = np.round(rng.standard_normal((B, V), dtype=np.float32) * 3).astype(np.float32)
        temp = float(rng.choice([0.05, 0.5, 0.8, 1.0, 1.3, 4.0, 100.0]))
        top_k = int(rng.choice([-1, 1, 2, 10, 50, 100, 1000, 1024, 1025, 10000]))
        top_p = float(rng.choice([0.0, 0.01, 0.1, 0.3, 0.5, 0.7, 0.9, 0.99, 1.0]))
        _run_case(torch_cuda, oracle, capi, lg, temp, top_k, top_p, u_np=H.uniforms(B, 1000 + case),
                  what="random case %d kind %d" % (case, kind))


def _random_row(rng, kind, V):
    """One row of logits of the given kind (see test_seeded_random_batches_of_mixed_rows)."""
    if kind == 0:
        return np.full(V, float(rng.choice([0.0, 1.5, -3.0, 1e30, -1e30])), dtype=np.float32)
    if kind == 1:
        return rng.random(V, dtype=np.float32)
    if kind == 2:
        return rng.standard_normal(V, dtype=np.float32) * np.float32(rng.choice([0.5, 3.0]))
    if kind == 3:
        return rng.random(V, dtype=np.float32) * np.float32(4)
    if kind == 4:                                                       # a masked stretch
        r = rng.standard_normal(V, dtype=np.float32) * np.float32(2)
        lo = int(rng.integers(0, V))
        r[lo: lo + int(rng.integers(1, V))] = -np.inf
        return r
    if kind == 5:                                                       # few distinct values
        return np.round(rng.standard_normal(V, dtype=np.float32) * 3).astype(np.float32)
    if kind == 6:                                                       # most tokens below 2^-40 of the largest
        r = rng.standard_normal(V, dtype=np.float32) * np.float32(rng.choice([6.0, 15.0, 60.0, 300.0]))
        if rng.random() < 0.5:                                          # the largest near the end of the row
            r[int(rng.integers(max(0, V - 600), V))] = r.max() + np.float32(rng.choice([0.0, 1.0, 50.0]))
        return r
    if kind == 7:                                                       # scattered masks
        r = rng.standard_normal(V, dtype=np.float32)
        r[rng.random(V) < float(rng.choice([0.5, 0.9, 0.99, 0.9999]))] = -np.inf
        r[int(rng.integers(0, V))] = 0.5
        return r
    if kind == 8:                                                       # a stretch of equal largest logits, NaN, Inf
        r = rng.standard_normal(V, dtype=np.float32)
        lo = int(rng.integers(0, V))
        r[lo: lo + int(rng.integers(1, max(2, V // 2)))] = float(r.max()) + float(rng.choice([0.0, 0.25, 2.0]))
        if rng.random() < 0.1:
            r[int(rng.integers(0, V))] = np.nan
        if rng.random() < 0.1:
            r[int(rng.integers(0, V))] = np.inf
        return r
    if kind == 9:                                                       # stretches at very different levels
        r = rng.standard_normal(V, dtype=np.float32)
        step = int(rng.choice([1024, 4096, 16384]))
        for lo in range(0, V, step):
            r[lo: lo + step] += np.float32(rng.choice([0.0, -30.0, -60.0, -100.0, -500.0, 20.0]))
        return r
    vals = (rng.standard_normal(int(rng.integers(2, 40))) * float(rng.choice([1.0, 5.0, 40.0]))).astype(np.float32)
    return vals[rng.integers(0, len(vals), V)]                          # ties at every level


def test_seeded_random_batches_of_mixed_rows(torch_cuda, oracle):
    """Seeded random cases in which every row of a batch is of its own kind (eleven kinds: constant,
    uniform, normal, masked stretches, few distinct values, very wide, scattered masks, stretches of
    equal largest logits with NaN / Inf, stretches at levels hundreds of octaves apart, a handful of
    values repeated), over the shapes that take the different routes: short and long slices of the
    streaming path, one row of up to a million tokens, and batches of 40-140 rows of 32-80 thousand
    tokens, which give the cluster kernel more workgroups than the GPU holds at once.  Some cases carry
    penalties, some hand the logits over as bfloat16 / float16.  Each case goes through every path
    (the cases of this generator found both a wrong tie count on the streaming path and a lost
    workgroup in the cluster kernel, each at a rate of about one call in a hundred of one shape)."""
    torch = torch_cuda
    from tests import capi
    rng = np.random.default_rng(4242)
    for case in range(160):
        mode = case % 8
        if mode == 0:
            B, V = int(rng.integers(1, 4)), 4 * int(rng.integers(150000, 262145))
        elif mode in (1, 5):
            B, V = int(rng.integers(40, 140)), 4 * int(rng.integers(8000, 20000))
        elif mode == 2:
            B, V = int(rng.integers(1, 24)), 4 * int(rng.integers(1, 2000))
        elif mode == 3:
            B, V = int(rng.integers(1, 8)), 4 * int(rng.integers(65537, 110000))
        elif mode == 4:
            B, V = int(rng.integers(5, 12)), 4 * int(rng.integers(100000, 140000))
        else:
            B, V = int(rng.integers(1, 24)), 4 * int(rng.integers(1, 60000))
        same = rng.random() < 0.3
        k0 = int(rng.integers(0, 11))
        lg = np.stack([_random_row(rng, k0 if same else int(rng.integers(0, 11)), V) for _ in range(B)])
        temp = float(rng.choice([0.05, 0.5, 0.8, 1.0, 1.3, 4.0, 100.0]))
        top_k = int(rng.choice([-1, 1, 2, 10, 50, 100, 1000, 1024, 1025, 10000]))
        top_p = float(rng.choice([0.0, 0.01, 0.1, 0.3, 0.5, 0.7, 0.9, 0.99, 1.0]))
        kw = {}
        pick = rng.random()
        if pick < 0.15:
            kw = dict(pen_np=(rng.random((B, V)) < 0.02).astype(np.float32) * rng.exponential(1.0, (B, V)).astype(np.float32),
                      presence=float(rng.choice([0.0, 0.1, 1.0])), repetition=float(rng.choice([0.0, 0.1, 0.5])),
                      decay=float(rng.choice([1.0, 0.95])))
        elif pick < 0.3:
            dt = torch.bfloat16 if rng.random() < 0.5 else torch.float16
            lg = torch.from_numpy(np.nan_to_num(lg, nan=0.0)).to(dt).float().numpy()
            kw = dict(dtype=dt)
        _run_case(torch, oracle, capi, lg, temp, top_k, top_p, u_np=H.uniforms(B, 7000 + case),
                  what="mixed batch %d shape %d" % (case, mode), **kw)


def test_one_workspace_many_shapes(torch_cuda, oracle):
    """Calls of different (B, V, top_k) -- and so of different paths and layouts -- on one workspace sized
    for the largest B and the largest V: what one call leaves behind must not disturb the next."""
    torch = torch_cuda
    from tests import capi
    smp = capi.Sampler(64, 151936)
    seq = [(8, 151936, 100, 1.0, "n"), (64, 151936, -1, 0.3, "u"), (3, 32768, 50, 0.9, "n"), (64, 151936, 100, 0.9, "n"),
           (1, 151936, -1, 0.5, "u"), (40, 65536, 1000, 1.0, "n"), (64, 4096, -1, 0.9, "u"), (8, 151936, 100, 1.0, "n")]
    for i, (B, V, k_in, p_in, kind) in enumerate(seq):
        lg_np = H.logits_uniform(B, V, seed=200 + i) if kind == "u" else H.logits_normal(B, V, 2.0, seed=200 + i)
        rc, c, k, p = capi.normalize(1.0, k_in, p_in, V, B, 1)
        u_np = H.uniforms(B, 300 + i)
        ref_out, ref_diag = oracle.sample_batch(lg_np, c, k, p, injected_u=u_np)
        print("shape", i, B, V, k, p, flush=True)
        res = smp.sample(torch.from_numpy(lg_np).cuda(), c, k, p, uniforms=torch.from_numpy(u_np).cuda())
        _check(res, ref_out, ref_diag, "shape %d" % i)
        assert smp.status() == 0


def test_penalty_path_single_step(torch_cuda, oracle):
    from tests import capi
    B, V = 8, 32768
    lg = H.logits_normal(B, V, 1.5, seed=30)
    pen = H.penalties_sparse(B, V, seed=31)
    pen[0, :64] = np.inf            # masked tokens (penalty +inf)
    _run_case(torch_cuda, oracle, capi, lg, 0.8, 50, 0.9, pen_np=pen, u_np=H.uniforms(B, 32),
              presence=0.1, repetition=0.1, decay=0.95, what="penalty step")
    for R in (1, 4, 16):
        _run_case(torch_cuda, oracle, capi, lg, 0.8, 50, 0.9, pen_np=pen, u_np=H.uniforms(B, 32),
                  presence=0.25, repetition=0.1, decay=0.95, force_r=R, what="penalty step R%d" % R)


@pytest.mark.parametrize("steps", [24, 256])
def test_c4_penalty_chain(torch_cuda, oracle, steps):
    """BASELINE config 4 (B=32, V=131072, 2 % Exp(1) penalties, presence=repetition=0.1, decay=0.95,
    T=0.8, top_k=50, top_p=0.9): chained decode steps on fixed logits, penalties evolving in place on both
    sides -- the 256 steps the configuration states, and a quick 24-step case."""
    torch = torch_cuda
    from tests import capi
    B, V = 32, 131072
    lg_np = H.logits_normal(B, V, 1.5, seed=40)
    pen_ref = H.penalties_sparse(B, V, seed=41)
    rc, c, k, p = capi.normalize(0.8, 50, 0.9, V, B, 1)
    smp = capi.Sampler(B, V)
    lg = torch.from_numpy(lg_np).cuda()
    pen = torch.from_numpy(pen_ref.copy()).cuda()
    for step in range(steps):
        u_np = H.uniforms(B, 100 + step)
        ref_out, ref_diag = oracle.sample_batch(lg_np, c, k, p, injected_u=u_np, penalties=pen_ref,
                                                presence=0.1, repetition=0.1, decay=0.95)
        print("chain step", step, flush=True)
        res = smp.sample(lg, c, k, p, uniforms=torch.from_numpy(u_np).cuda(), penalties=pen,
                         presence=0.1, repetition=0.1, decay=0.95)
        _check(res, ref_out, ref_diag, "chain step %d" % step)
    got = pen.cpu().numpy()
    assert np.array_equal(got.view(np.uint32), pen_ref.view(np.uint32))
    rel = np.abs(got - pen_ref) / np.maximum(np.abs(pen_ref), 1e-30)
    assert rel.max() <= 1e-6
    assert smp.status() == 0



@pytest.mark.parametrize("B", [11, 21])
def test_one_launch_path_rows_of_more_slices_than_an_xcd_has_compute_units(torch_cuda, oracle, B):
    """The workgroups of the one-launch path wait for each other, and the hardware binds workgroup b to
    XCD b mod 8 before it starts.  With its token list in dynamic LDS the kernel ran one workgroup per
    compute unit, 32 per XCD, and a row of 47 slices whose last workgroups all belonged to one XCD could
    starve until its waits gave up (one call in some hundred, always the last row).  The list now always
    lives in static LDS.  The shape and the sequence of calls that showed it (11 rows: 517 workgroups,
    which the device holds at once, so they keep the hardware's ids), and the same with 21 rows (987
    workgroups: more than it holds, so they draw tickets), 300 times over, with a wait limit of 50 ms
    so that a starved row would show at once."""
    torch = torch_cuda
    from tests import capi
    V = 191104
    rng = np.random.default_rng(5)
    rows = []
    for _ in range(B):
        r = rng.standard_normal(V, dtype=np.float32)
        lo = int(rng.integers(0, V))
        n = int(rng.integers(1, V // 2))
        r[lo: lo + n] = float(r.max()) + float(rng.choice([0.0, 0.25, 2.0]))     # a run of ties at the top
        rows.append(r)
    lg = np.stack(rows)
    rc, c, k, p = capi.normalize(0.5, 1000, 0.0, V, B, 1)                        # top_p 0: greedy
    u_np = H.uniforms(B, 77)
    ref_out, ref_diag = oracle.sample_batch(lg, c, k, p, injected_u=u_np)
    smp = capi.Sampler(B, V)
    smp.set_wait_limit(50)
    lgt, u = torch.from_numpy(lg).cuda(), torch.from_numpy(u_np).cuda()
    for it in range(300):
        for path in ("cluster", "stream", "optimistic", "fused"):
            res = smp.sample(lgt, c, k, p, uniforms=u, path=path, want_diag=(it % 50 == 0))
            assert res["rc"] == 0 and np.array_equal(res["out"], ref_out), "iteration %d path %s" % (it, path)
            if it % 50 == 0:
                _check(res, ref_out, ref_diag, "iteration %d path %s" % (it, path))
        assert smp.status() == 0, "iteration %d" % it

@pytest.mark.parametrize("B,V,steps", [(96, 152064, 3), (128, 1048576, 2)])
def test_penalties_at_scale_streaming_pass(torch_cuda, oracle, B, V, steps):
    """Calls with penalties too large for the one-launch path (more workgroups than the GPU holds at once)
    take the streaming pass over logits and penalties, which also writes the decayed penalties, and the
    finish, which patches the sampled tokens: chained steps, tokens, diagnostics and penalties bit for bit
    against the oracle; the general kernel on the same inputs beside it."""
    torch = torch_cuda
    from tests import capi
    lg_np = H.logits_normal(B, V, 1.5, seed=140)
    pen_ref = H.penalties_sparse(B, V, seed=141)
    rc, c, k, p = capi.normalize(0.8, 50, 0.9, V, B, 1)
    smp = capi.Sampler(B, V)
    lg = torch.from_numpy(lg_np).cuda()
    pen = torch.from_numpy(pen_ref.copy()).cuda()
    for step in range(steps):
        u_np = H.uniforms(B, 500 + step)
        u = torch.from_numpy(u_np).cuda()
        pen_c = pen.clone()
        ref_out, ref_diag = oracle.sample_batch(lg_np, c, k, p, injected_u=u_np, penalties=pen_ref,
                                                presence=0.1, repetition=0.2, decay=0.95)
        print("penalties at scale: step", step, B, V, flush=True)
        res = smp.sample(lg, c, k, p, uniforms=u, penalties=pen, presence=0.1, repetition=0.2, decay=0.95)
        _check(res, ref_out, ref_diag, "streaming with penalties, step %d" % step)
        assert (res["diag"]["rounds"] == 0).all()                      # finished by the streaming path
        assert np.array_equal(pen.cpu().numpy().view(np.uint32), pen_ref.view(np.uint32)), step
        res_c = smp.sample(lg, c, k, p, uniforms=u, penalties=pen_c, presence=0.1, repetition=0.2, decay=0.95, path="cluster")
        _check(res_c, ref_out, ref_diag, "general kernel, step %d" % step)
        assert torch.equal(pen_c.view(torch.int32), pen.view(torch.int32))
        assert smp.status() == 0


def test_penalties_at_scale_unusual_rows_and_slices(torch_cuda, oracle):
    """The single pass over the penalties at scale where it cannot simply write decayed values and patch
    one token (reference: sampling.cu:427-437 on every kind of row): a row that has to be done the slow way
    (half its tokens tie at the top, so the old penalties of the whole row are needed again: the slices'
    notes are played back and the row rewritten at the end), a row of a million tokens among them, slices
    with more non-zero penalties than they can note (left alone by the pass, rewritten at the end),
    penalties of -0.0 (not +0.0: written, and 'zero' for the presence / repetition switch), a sampled token
    whose old penalty was non-zero, and a decay that is not finite (nothing can be skipped).  Three chained
    steps each, everything bit for bit against the oracle."""
    torch = torch_cuda
    from tests import capi
    B, V = 10, 1048576
    rng = np.random.default_rng(150)
    lg_np = (rng.standard_normal((B, V)) * 1.5).astype(np.float32)
    pen0 = H.penalties_sparse(B, V, seed=151)
    lg_np[1, ::2] = 9.0                                               # a tie of half the row at the top: the slow way
    pen0[1, ::2] = 0.0
    pen0[1, 4::64] = 0.25                                             # ... some of the tied tokens penalised
    pen0[2, 100000:140000] = rng.exponential(1.0, 40000).astype(np.float32)      # dense stretch: slices that cannot note all
    pen0[3, ::7] = -0.0
    top = np.argsort(lg_np[4])[-3:]
    lg_np[4, top] += 6.0                                              # three dominant tokens, already penalised
    pen0[4, top] = 0.5
    pen0[5] = 0.0                                                     # nothing penalised yet
    pen0[6] = rng.exponential(0.1, V).astype(np.float32)              # everything penalised
    rc, c, k, p = capi.normalize(0.8, 50, 0.9, V, B, 1)
    lg = torch.from_numpy(lg_np).cuda()
    for decay in (0.95, float("inf")):
        pen_ref = pen0.copy()
        if decay != 0.95:
            pen_ref[:] = 0.0                                          # 0 * inf: every entry becomes NaN, zeros too
        smp = capi.Sampler(B, V)
        pen = torch.from_numpy(pen_ref.copy()).cuda()
        for step in range(3):
            u_np = H.uniforms(B, 600 + step)
            u = torch.from_numpy(u_np).cuda()
            ref_out, ref_diag = oracle.sample_batch(lg_np, c, k, p, injected_u=u_np, penalties=pen_ref,
                                                    presence=0.1, repetition=0.2, decay=decay)
            print("penalties at scale, unusual: decay", decay, "step", step, flush=True)
            res = smp.sample(lg, c, k, p, uniforms=u, penalties=pen, presence=0.1, repetition=0.2, decay=decay)
            _check(res, ref_out, ref_diag, "unusual penalties, decay %r step %d" % (decay, step))
            got = pen.cpu().numpy().view(np.uint32)
            bad = np.nonzero((got != pen_ref.view(np.uint32)).any(axis=1))[0]
            assert bad.size == 0, (decay, step, bad)
            if decay == 0.95 and step == 0:
                assert res["diag"]["rounds"][1] == 8 and (np.delete(res["diag"]["rounds"], 1) == 0).all(), res["diag"]["rounds"]
            assert smp.status() == 0


def test_philox_stream_matches_oracle(torch_cuda, oracle):
    """Without injected uniforms: rs_philox_init + the in-kernel Philox draw give the oracle's indices,
    call after call (the draw counter advances by one per call)."""
    torch = torch_cuda
    from tests import capi
    import ctypes as C
    B, V = 16, 16384
    lg_np = H.logits_normal(B, V, 2.0, seed=50)
    rc, c, k, p = capi.normalize(1.0, -1, 0.9, V, B, 1)
    smp = capi.Sampler(B, V)
    lg = torch.from_numpy(lg_np).cuda()
    st = torch.empty(B * 64, dtype=torch.int8, device="cuda")
    assert capi.lib().rs_philox_init(st.data_ptr(), 1234567890123, B, smp.stream()) == 0
    rng_ref = oracle.rng_init(1234567890123, B)
    torch.cuda.synchronize()
    assert np.array_equal(st.cpu().numpy().view(np.uint32).reshape(B, 16), rng_ref)
    for call in range(4):
        ref_out, ref_diag = oracle.sample_batch(lg_np, c, k, p, rng=rng_ref)
        res = smp.sample(lg, c, k, p, rng=st)
        _check(res, ref_out, ref_diag, "philox call %d" % call)
    assert np.array_equal(st.cpu().numpy().view(np.uint32).reshape(B, 16), rng_ref)


@pytest.mark.parametrize("path,pen_on", [("cluster", False), ("cluster", True), ("stream", False), ("row", False)])
def test_hip_graph_decode_loop(torch_cuda, oracle, path, pen_on):
    """A sampling call captured into a HIP graph (rs_sample records only kernel launches: no memset,
    no allocation, no synchronisation) and replayed as a decode loop: every replay draws the next Philox
    number and, with penalties, continues from the penalties the previous replay left.  Each replay is
    checked against the oracle, with eager work and synchronisations between replays."""
    torch = torch_cuda
    from tests import capi
    B, V, replays = 6, 65536 + 4096 if path != "row" else 40960, 6      # (the row kernel holds rows of up to 65536 tokens)
    lg_np = H.logits_normal(B, V, 2.0, seed=70)
    pen_ref = H.penalties_sparse(B, V, seed=71) if pen_on else None
    rc, c, k, p = capi.normalize(0.9, 40, 0.9, V, B, 1)
    smp = capi.Sampler(B, V)
    lg = torch.from_numpy(lg_np).cuda()
    pen = torch.from_numpy(pen_ref.copy()).cuda() if pen_on else None
    out = torch.full((B,), -1, dtype=torch.int32, device="cuda")
    hist = torch.zeros((B,), dtype=torch.int64, device="cuda")
    st = torch.empty(B * 64, dtype=torch.int8, device="cuda")
    assert capi.lib().rs_philox_init(st.data_ptr(), 99, B, smp.stream()) == 0
    rng_ref = oracle.rng_init(99, B)
    torch.cuda.synchronize()
    opt = capi.Options(capi.PATHS[path], 0, None)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        rc = capi.lib().rs_sample_ex(lg.data_ptr(), 0, V, pen.data_ptr() if pen_on else None, out.data_ptr(),
                                     st.data_ptr(), None, B, V, 0.1, 0.2, 0.9, c, k, p,
                                     smp.ws.data_ptr(), smp.ws.numel(), None, None, C_byref(opt), smp.stream())
        hist += out                                   # a consumer of the sampled ids inside the graph
    assert rc == 0
    total = np.zeros(B, dtype=np.int64)
    for i in range(replays):
        ref_out, _ = oracle.sample_batch(lg_np, c, k, p, rng=rng_ref, penalties=pen_ref,
                                         presence=0.1, repetition=0.2, decay=0.9)
        print("graph replay", i, path, pen_on, flush=True)
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(out.cpu().numpy(), ref_out), "replay %d" % i
        total += ref_out
        scratch = torch.randn(1 << 20, device="cuda").sum().item()      # eager work between replays
        assert scratch == scratch
    assert np.array_equal(hist.cpu().numpy(), total)
    assert np.array_equal(st.cpu().numpy().view(np.uint32).reshape(B, 16), rng_ref)
    if pen_on:
        assert np.array_equal(pen.cpu().numpy().view(np.uint32), pen_ref.view(np.uint32))
    assert smp.status() == 0


def test_python_module_drop_in_calls(torch_cuda, oracle):
    """The reference's three functions through the PyTorch extension (the drop-in surface), not the C ABI:
    setup_rand + both sampling calls, (V,), (B,V) and (B,T,V) logits, penalties in place, shapes changing
    from call to call (the module's workspace cache grows), all against the oracle's Philox stream."""
    torch = torch_cuda
    import rapid_sampling_amd as sample
    seed = 20240607
    for (shape, k_in, p_in, temp) in [((5, 32768), 50, 0.9, 0.8), ((3, 4, 65536), -1, 0.7, 1.0), ((131072,), 20, 1.0, 1.3),
                                      ((70, 8192), 1000, 0.95, 1.0), ((5, 32768), 50, 0.9, 0.8)]:
        V = shape[-1]
        B = shape[0] if len(shape) > 1 else 1
        T = shape[1] if len(shape) == 3 else 1
        lg_np = H.logits_normal(B * T, V, 2.0, seed=V % 1000 + B).reshape(shape)
        c, k, p = oracle.normalize(temp, k_in, p_in, V, B, T)
        states = sample.setup_rand(seed, B)
        rng_ref = oracle.rng_init(seed, B)
        lg = torch.from_numpy(lg_np).cuda()
        for call in range(3):
            ref_out, _ = oracle.sample_batch(lg_np, c, k, p, rng=rng_ref)
            out = sample.batch_sampling_temperature_topk_topp(lg, states, temp, k_in, p_in)
            assert out.dtype == torch.int32 and tuple(out.shape) == (B,)
            assert np.array_equal(out.cpu().numpy(), ref_out), (shape, call)
        # the penalty call continues the same Philox stream and updates penalties in place
        pen_ref = H.penalties_sparse(B, V, seed=7)
        pen = torch.from_numpy(pen_ref.copy()).cuda()
        for call in range(2):
            ref_out, _ = oracle.sample_batch(lg_np, c, k, p, rng=rng_ref, penalties=pen_ref,
                                             presence=0.3, repetition=0.1, decay=0.99)
            out = sample.batch_sampling_repetition_temperature_topk_topp(lg, pen, states, 0.3, 0.1, 0.99,
                                                                         temp, k_in, p_in)
            assert np.array_equal(out.cpu().numpy(), ref_out), (shape, "pen", call)
        assert np.array_equal(pen.cpu().numpy().view(np.uint32), pen_ref.view(np.uint32))
        # keyword call with injected uniforms
        u_np = H.uniforms(B, 5)
        ref_out, _ = oracle.sample_batch(lg_np, c, k, p, injected_u=u_np)
        out = sample.batch_sampling_temperature_topk_topp(logits=lg, states=states, temperature=temp, top_k=k_in,
                                                          top_p=p_in, uniforms=torch.from_numpy(u_np).cuda())
        assert np.array_equal(out.cpu().numpy(), ref_out)
    # half-precision logits, opted into: the result of the float32 call on the widened values
    for dt in (torch.bfloat16, torch.float16):
        lgh = torch.from_numpy(H.logits_normal(6, 4 * 65536, 2.0, seed=3).reshape(6, 4, 65536)).cuda().to(dt)
        u = torch.from_numpy(H.uniforms(6, 9)).cuda()
        st = sample.setup_rand(1, 6)
        a = sample.batch_sampling_temperature_topk_topp(lgh, st, 0.9, 100, 0.95, uniforms=u, accept_half=True)
        b = sample.batch_sampling_temperature_topk_topp(lgh.float(), st, 0.9, 100, 0.95, uniforms=u)
        assert torch.equal(a, b)
        with pytest.raises(ValueError, match="float32"):
            sample.batch_sampling_temperature_topk_topp(lgh, st, 0.9, 100, 0.95, uniforms=u)


def test_streaming_calls_are_routed_by_reports(torch_cuda, oracle):
    """top_k disabled, top_p < 1: the wait-free path is an attempt.  With a policy it is made, after one call
    on the wide path that probes whether the rows' kept sets fit the stashes; peaked rows
    finish on it from the stashes (diag.rounds == 0).  A call with a row that had to be done the slow
    way (a flat row: the finishing workgroup goes through the logits again, diag.rounds == 8) says so in
    the policy's report word at once, and the next calls go to the general kernel (or, as these 600 rows of
    65536 tokens once all of them are flat, to the row kernel, diag.rounds == 10); streaming is tried
    again after 64 of them, then 128, 256, ...; that a call went well is reported by the call after it,
    whichever kernel that is.  Without a policy no attempts are made.  Every result equals the
    oracle's whatever the route."""
    torch = torch_cuda
    import ctypes as C
    from tests import capi
    B, V = 600, 65536
    peaked = H.logits_normal(B, V, 3.0, seed=90)
    flat = H.logits_uniform(B, V, seed=91)
    mixed = peaked.copy()
    mixed[7] = flat[7]                                   # one flat row among 600
    rc, c, k, p = capi.normalize(1.0, -1, 0.3, V, B, 1)
    assert k == V
    u_np = H.uniforms(B, 92)
    u = torch.from_numpy(u_np).cuda()
    ref_peaked = oracle.sample_batch(peaked, c, k, p, injected_u=u_np)
    ref_flat = oracle.sample_batch(flat, c, k, p, injected_u=u_np)
    ref_mixed = (ref_peaked[0].copy(), ref_peaked[1].copy())
    ref_mixed[0][7] = ref_flat[0][7]
    ref_mixed[1][7] = ref_flat[1][7]
    lg_peaked, lg_flat, lg_mixed = (torch.from_numpy(a).cuda() for a in (peaked, flat, mixed))

    def policy(smp):
        return smp.policy_state()

    plain = capi.Sampler(B, V)                           # no policy: no report words
    res = plain.sample(lg_peaked, c, k, p, uniforms=u)
    _check(res, *ref_peaked, "no policy")
    assert (res["diag"]["rounds"] >= 1).all()            # no attempts without a policy: the row kernel for these 600 rows

    smp = capi.Sampler(B, V, with_policy=True, init=True)
    assert policy(smp) == 0
    res = smp.sample(lg_peaked, c, k, p, uniforms=u)     # the first call of its kind on a policy is a probe: the wide path
    _check(res, *ref_peaked, "probe on peaked rows")
    assert (res["diag"]["rounds"] == 7).all() and policy(smp) == 0
    res = smp.sample(lg_peaked, c, k, p, uniforms=u)
    _check(res, *ref_peaked, "attempt on peaked rows")
    assert (res["diag"]["rounds"] == 0).all() and policy(smp) == 0
    res = smp.sample(lg_mixed, c, k, p, uniforms=u)      # attempted, one row done the slow way
    _check(res, *ref_mixed, "attempt with one flat row")
    assert res["diag"]["rounds"][7] == 8 and (np.delete(res["diag"]["rounds"], 7) == 0).all() and policy(smp) == 1
    for i in range(3):                                   # no further attempts for now, peaked or not
        res = smp.sample(lg_peaked, c, k, p, uniforms=u)
        _check(res, *ref_peaked, "after a failed attempt %d" % i)
        assert (res["diag"]["rounds"] >= 1).all() and policy(smp) == 1
    for i in range(64):                                  # 64 calls away, a try that goes well, the call after it says so
        res = smp.sample(lg_peaked, c, k, p, uniforms=u, want_diag=False)
        assert res["rc"] == 0 and np.array_equal(res["out"], ref_peaked[0])
    assert policy(smp) == 0
    res = smp.sample(lg_peaked, c, k, p, uniforms=u)
    assert (res["diag"]["rounds"] == 0).all() and policy(smp) == 0
    # rows that are always too flat: the next try after 128 calls away (a failed try doubles the stay)
    streamed = []
    for i in range(135):
        res = smp.sample(lg_flat, c, k, p, uniforms=u)
        assert res["rc"] == 0 and np.array_equal(res["out"], ref_flat[0])
        if (res["diag"]["rounds"] == 8).all():
            streamed.append(i)
        else:
            # 600 rows of 65536 tokens: the row kernel; the try after 128 calls away (call 129 here): a probe on the wide path
            assert (res["diag"]["rounds"] == 10).all() or (i == 129 and (res["diag"]["rounds"] == 7).all()), (i, res["diag"]["rounds"][:4])
        assert policy(smp) == 1
    # (the try after 128 calls is a probe on the wide path, which says no without doing any row the slow way)
    assert streamed == [0], streamed
    assert smp.status() == 0
    smp.close()
    smp = capi.Sampler(B, V, with_policy=True, init=True)

    # The same for calls WITH a bounding top_k, which stream unless told otherwise: rows whose every
    # other token ties at the top cannot be finished from the stashes (the tie is larger than any
    # stash, and it is not the whole row) and are done the slow way, the report says so (bit 1), the
    # next calls skip the streaming pass, and after 64 of them streaming is tried again.
    ties = np.zeros((B, V), dtype=np.float32)
    ties[:, ::2] = 1.0
    rc, c, k, p = capi.normalize(1.0, 10, 1.0, V, B, 1)
    ref_ties = oracle.sample_batch(ties, c, k, p, injected_u=u_np)
    ref_peaked = oracle.sample_batch(peaked, c, k, p, injected_u=u_np)
    lg_ties = torch.from_numpy(ties).cuda()
    res = smp.sample(lg_peaked, c, k, p, uniforms=u)
    _check(res, *ref_peaked, "bounded, peaked rows")
    assert (res["diag"]["rounds"] == 0).all() and policy(smp) == 0
    res = smp.sample(lg_ties, c, k, p, uniforms=u)       # streamed, every row done the slow way
    _check(res, *ref_ties, "bounded, rows of ties")
    assert (res["diag"]["rounds"] >= 1).all() and policy(smp) == 2
    res = smp.sample(lg_peaked, c, k, p, uniforms=u)     # not streamed
    _check(res, *ref_peaked, "bounded, after rows of ties")
    assert (res["diag"]["rounds"] >= 1).all() and policy(smp) == 2
    for i in range(66):
        res = smp.sample(lg_peaked, c, k, p, uniforms=u, want_diag=False)
        assert res["rc"] == 0 and np.array_equal(res["out"], ref_peaked[0])
    assert policy(smp) == 0
    res = plain.sample(lg_ties, c, k, p, uniforms=u)     # no report words: streams whatever happened before
    _check(res, *ref_ties, "bounded, no policy")
    assert plain.status() == 0 and smp.status() == 0 and smp.policy_error() == 0
    smp.close()


def test_routing_is_kept_per_kind_and_size_of_call(torch_cuda, oracle):
    """Two workloads interleaved on one workspace and one policy, both without a bounding top_k: a lone
    flat row (its kept set never fits the stashes) and a batch of peaked rows (always does).  The report
    words are kept per kind and size class of call, so the flat row's reports do not send the batch to the
    general kernel, and the batch's good reports do not send the flat row back to the streaming path: after
    its probe, every call of the batch is finished from the stashes (diag.rounds == 0), and no call of the
    flat row is ever done the slow way (diag.rounds == 8)."""
    torch = torch_cuda
    from tests import capi
    Vf, Bp, Vp = 262144, 48, 152064
    flat = (np.random.default_rng(95).random((1, Vf), dtype=np.float32) * np.float32(4.0)).astype(np.float32)
    peaked = H.logits_normal(Bp, Vp, 3.0, seed=96)
    uf_np, up_np = H.uniforms(1, 97), H.uniforms(Bp, 98)
    rc, cf, kf, pf = capi.normalize(1.0, -1, 0.3, Vf, 1, 1)
    rc, cp, kp, pp = capi.normalize(1.0, -1, 0.3, Vp, Bp, 1)
    ref_f = oracle.sample_batch(flat, cf, kf, pf, injected_u=uf_np)
    ref_p = oracle.sample_batch(peaked, cp, kp, pp, injected_u=up_np)
    lg_f, lg_p = torch.from_numpy(flat).cuda(), torch.from_numpy(peaked).cuda()
    uf, up = torch.from_numpy(uf_np).cuda(), torch.from_numpy(up_np).cuda()
    smp = capi.Sampler(Bp, Vf, with_policy=True, init=True)           # one workspace large enough for both shapes
    flat_rounds, peaked_rounds = [], []
    for i in range(150):
        res = smp.sample(lg_f, cf, kf, pf, uniforms=uf)
        _check(res, *ref_f, "interleaved, flat row, call %d" % i)
        flat_rounds.append(int(res["diag"]["rounds"][0]))
        res = smp.sample(lg_p, cp, kp, pp, uniforms=up)
        _check(res, *ref_p, "interleaved, peaked batch, call %d" % i)
        peaked_rounds.append(sorted(set(res["diag"]["rounds"].tolist())))
    assert peaked_rounds[0] == [7] and all(r == [0] for r in peaked_rounds[1:]), peaked_rounds[:5]
    assert flat_rounds[0] == 7 and 8 not in flat_rounds, flat_rounds[:10]
    assert sum(1 for r in flat_rounds if r == 7) <= 3                  # the probe, and one or two retries (64, 128 calls later)
    assert smp.policy_state() == 1 and smp.status() == 0
    smp.close()


def test_calls_issued_behind_a_probe_that_has_not_run_yet_are_probes_too(torch_cuda, oracle):
    """A caller that does not synchronise between calls issues many before the first has run.  The first
    call without a bounding top_k on a policy is a probe, and its report word is pending until it has run:
    the calls issued in the meantime are probes as well (diag.rounds == 7), not attempts that would do
    their flat rows the slow way (diag.rounds == 8).  Once the probe has run, its verdict routes the
    calls: flat rows to the general kernel, peaked rows to the streaming path.  A dozen calls queued
    behind a kernel that keeps the GPU busy while they are issued, flat rows and peaked ones."""
    torch = torch_cuda
    from tests import capi
    B, V = 8, 131072
    flat = H.logits_uniform(B, V, seed=190)
    peaked = H.logits_normal(B, V, 3.0, seed=191)
    u_np = H.uniforms(B, 192)
    rc, c, k, p = capi.normalize(1.0, -1, 0.4, V, B, 1)
    u = torch.from_numpy(u_np).cuda()
    for name, rows in (("flat", flat), ("peaked", peaked)):
        ref_out, ref_diag = oracle.sample_batch(rows, c, k, p, injected_u=u_np)
        lg = torch.from_numpy(rows).cuda()
        smp = capi.Sampler(B, V, with_policy=True, init=True)
        torch.cuda.synchronize()
        torch.cuda._sleep(40_000_000)                    # some 20 ms: the calls below are all issued before the first runs
        calls = [smp.sample(lg, c, k, p, uniforms=u, sync=False) for _ in range(12)]
        torch.cuda.synchronize()
        rounds = []
        for i, res in enumerate(calls):
            assert res["rc"] == 0
            out = res["out_dev"].cpu().numpy()
            diag = res["diag_dev"].cpu().numpy().view(capi.DIAG_DTYPE).reshape(B)
            _check({"rc": 0, "out": out, "diag": diag}, ref_out, ref_diag, "%s rows, queued call %d" % (name, i))
            rounds.append(sorted(set(diag["rounds"].tolist())))
        assert rounds[0] == [7] and all(r != [8] and 8 not in r for r in rounds), (name, rounds)
        # the probe has run: its verdict stands
        res = smp.sample(lg, c, k, p, uniforms=u)
        _check(res, ref_out, ref_diag, "%s rows, after the queue" % name)
        if name == "flat":
            assert smp.policy_state() == 1 and (res["diag"]["rounds"] >= 1).all() and (res["diag"]["rounds"] < 7).all()
        else:
            assert smp.policy_state() == 0 and (res["diag"]["rounds"] == 0).all()
        assert smp.status() == 0
        smp.close()


def test_two_streams_two_workspaces_concurrently(torch_cuda, oracle):
    """Calls on two streams, each with its own workspace, state and outputs, issued alternately
    without any synchronisation in between, so that their kernels share the GPU: a cluster-path
    workload (64 rows, nucleus sampling, several workgroups per row waiting for each other) beside a
    streaming-path one and a penalty chain.  Every call's result equals the oracle's and no wait
    gives up."""
    torch = torch_cuda
    from tests import capi
    L = capi.lib()
    N = 10
    jobs = []
    for (B, V, k_in, p_in, temp, sigma, pen_on, seed) in [(64, 152064, -1, 0.9, 0.8, 2.0, False, 1),
                                                        (48, 131072, 50, 0.95, 1.0, 1.5, False, 2),
                                                        (32, 131072, 40, 0.9, 1.0, 2.0, True, 3)]:
        lg_np = H.logits_normal(B, V, sigma, seed=seed)
        rc, c, k, p = capi.normalize(temp, k_in, p_in, V, B, 1)
        us = [H.uniforms(B, 100 * seed + i) for i in range(N)]
        pen_ref = H.penalties_sparse(B, V, seed=seed) if pen_on else None
        refs = []
        for i in range(N):
            kw = dict(penalties=pen_ref, presence=0.2, repetition=0.1, decay=0.97) if pen_on else {}
            refs.append(oracle.sample_batch(lg_np, c, k, p, injected_u=us[i], **kw)[0])
        jobs.append(dict(B=B, V=V, c=c, k=k, p=p, lg=torch.from_numpy(lg_np).cuda(), smp=capi.Sampler(B, V),
                         u=[torch.from_numpy(u).cuda() for u in us], refs=refs, pen_ref=pen_ref,
                         pen=torch.from_numpy(H.penalties_sparse(B, V, seed=seed)).cuda() if pen_on else None,
                         out=[torch.full((B,), -7, dtype=torch.int32, device="cuda") for _ in range(N)]))
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream(), torch.cuda.Stream()]
    for i in range(N):
        for j, st in zip(jobs, streams):
            rc = L.rs_sample(j["lg"].data_ptr(), j["V"], j["pen"].data_ptr() if j["pen"] is not None else None,
                             j["out"][i].data_ptr(), None, j["u"][i].data_ptr(), j["B"], j["V"], 0.2, 0.1, 0.97,
                             j["c"], j["k"], j["p"], j["smp"].ws.data_ptr(), j["smp"].ws.numel(), None, None,
                             C_void_p(st.cuda_stream))
            assert rc == 0
    torch.cuda.synchronize()
    for n, j in enumerate(jobs):
        assert j["smp"].status() == 0, n
        for i in range(N):
            assert np.array_equal(j["out"][i].cpu().numpy(), j["refs"][i]), (n, i)
        if j["pen"] is not None:
            assert np.array_equal(j["pen"].cpu().numpy().view(np.uint32), j["pen_ref"].view(np.uint32))


def test_bounded_wait_reports_error_and_recovers(torch_cuda, oracle):
    """A workspace that was never cleaned (here: filled with ones behind its header) holds histograms that
    never add up.  The workgroups must give up after the bound of their waits (shortened to 20 ms with
    rs_workspace_set_wait_limit), leave a sticky RS_ERR_DEVICE -- also in the pinned host word of the
    caller's rs_policy, readable without synchronising -- and end normally; after rs_workspace_init the
    same workspace works again."""
    torch = torch_cuda
    from tests import capi
    B, V = 2, 65536
    lg_np = H.logits_normal(B, V, 2.0, seed=80)
    rc, c, k, p = capi.normalize(1.0, -1, 0.9, V, B, 1)
    u_np = H.uniforms(B, 81)
    ref_out, ref_diag = oracle.sample_batch(lg_np, c, k, p, injected_u=u_np)
    smp = capi.Sampler(B, V, with_policy=True, init=True)
    lg, u = torch.from_numpy(lg_np).cuda(), torch.from_numpy(u_np).cuda()
    smp.set_wait_limit(20)
    smp.ws[capi.HEADER_BYTES:] = 1
    torch.cuda.synchronize()
    assert smp.policy_error() == 0
    print("poisoned workspace, expecting a bounded wait to give up", flush=True)
    res = smp.sample(lg, c, k, p, uniforms=u, want_diag=False, path="cluster")
    assert res["rc"] == 0                       # the launch itself is fine
    assert smp.policy_error() == -9             # reported to the host without a device read
    assert smp.status() == -9                   # RS_ERR_DEVICE, sticky
    wait, row, slc, seen, want = smp.where()    # the first wait that gave up: a histogram that never added up
    assert wait in (1, 2) and row < B and seen != want, (wait, row, slc, seen, want)
    smp.reinit()
    assert smp.policy_error(clear=True) == -9 and smp.policy_error() == 0
    assert smp.status() == 0 and smp.where()[0] == 0
    res = smp.sample(lg, c, k, p, uniforms=u)
    _check(res, ref_out, ref_diag, "after re-initialisation")
    assert smp.status() == 0 and smp.policy_error() == 0
    smp.close()


def test_python_module_raises_after_a_failed_call_and_recovers(torch_cuda, oracle):
    """The same failure through the drop-in module, whose workspace is private: the call whose kernel gave
    up returns (its result is garbage), the next call on that stream raises RuntimeError and sets the
    workspace up again, and the call after that is correct.  workspace_status() tells at once."""
    torch = torch_cuda
    import rapid_sampling_amd as sample
    from tests import capi
    B, V = 2, 32768                                  # small enough to take the general kernel, several workgroups per row
    lg_np = H.logits_normal(B, V, 2.0, seed=82)
    c, k, p = oracle.normalize(1.0, -1, 0.9, V, B, 1)
    u_np = H.uniforms(B, 83)
    ref_out, _ = oracle.sample_batch(lg_np, c, k, p, injected_u=u_np)
    lg, u = torch.from_numpy(lg_np).cuda(), torch.from_numpy(u_np).cuda()
    st = sample.setup_rand(1, B)
    side = torch.cuda.Stream()                       # a stream of its own: its workspace is this test's alone
    sample._sample.force_path("cluster")             # the kernel whose workgroups wait for counts that add up
    try:
      with torch.cuda.stream(side):
        out = sample.batch_sampling_temperature_topk_topp(lg, st, 1.0, -1, 0.9, uniforms=u)
        assert np.array_equal(out.cpu().numpy(), ref_out) and sample.workspace_status() == 0
        for check in ("next call", "status"):
            sample.set_wait_limit(20)
            ws = sample._sample.debug_workspace()
            ws[capi.HEADER_BYTES:] = 1
            side.synchronize()
            print("poisoned module workspace:", check, flush=True)
            sample.batch_sampling_temperature_topk_topp(lg, st, 1.0, -1, 0.9, uniforms=u)      # gives up; no exception yet
            if check == "next call":
                side.synchronize()
                with pytest.raises(RuntimeError, match="earlier sampling call"):
                    sample.batch_sampling_temperature_topk_topp(lg, st, 1.0, -1, 0.9, uniforms=u)
            else:
                assert sample.workspace_status() == -9
            out = sample.batch_sampling_temperature_topk_topp(lg, st, 1.0, -1, 0.9, uniforms=u)
            assert np.array_equal(out.cpu().numpy(), ref_out), check
            assert sample.workspace_status() == 0
    finally:
        sample._sample.force_path("auto")
    side.synchronize()


def test_python_module_calls_captured_into_a_graph(torch_cuda, oracle):
    """The drop-in module under torch.cuda.graph: the workspace is reserved before the capture (growing it
    while capturing raises a clear error), the captured calls replay as a decode loop that continues the
    Philox stream and the penalties, and an eager call on the capture stream between replays works."""
    torch = torch_cuda
    import rapid_sampling_amd as sample
    B, V, replays = 4, 65536, 4
    lg_np = H.logits_normal(B, V, 2.0, seed=84)
    pen_ref = H.penalties_sparse(B, V, seed=85)
    c, k, p = oracle.normalize(0.9, 40, 0.9, V, B, 1)
    rng_ref = oracle.rng_init(5, B)
    lg = torch.from_numpy(lg_np).cuda()
    pen = torch.from_numpy(pen_ref.copy()).cuda()
    st = sample.setup_rand(5, B)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        sample.reserve_workspace(B, V)
        with torch.cuda.graph(graph, stream=side):
            a = sample.batch_sampling_temperature_topk_topp(lg, st, 0.9, 40, 0.9)
            b = sample.batch_sampling_repetition_temperature_topk_topp(lg, pen, st, 0.1, 0.2, 0.9, 0.9, 40, 0.9)
    side.synchronize()
    for i in range(replays):
        ref_a, _ = oracle.sample_batch(lg_np, c, k, p, rng=rng_ref)
        ref_b, _ = oracle.sample_batch(lg_np, c, k, p, rng=rng_ref, penalties=pen_ref, presence=0.1, repetition=0.2, decay=0.9)
        print("module graph replay", i, flush=True)
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(a.cpu().numpy(), ref_a) and np.array_equal(b.cpu().numpy(), ref_b), i
        with torch.cuda.stream(side):                    # an eager call on the same stream and workspace
            ref_c, _ = oracle.sample_batch(lg_np, c, k, p, rng=rng_ref)
            cc = sample.batch_sampling_temperature_topk_topp(lg, st, 0.9, 40, 0.9)
            assert np.array_equal(cc.cpu().numpy(), ref_c), i
    assert np.array_equal(pen.cpu().numpy().view(np.uint32), pen_ref.view(np.uint32))
    with torch.cuda.stream(side):
        assert sample.workspace_status() == 0
        # reset_routing replaces the policy object; the graph's kernels still hold the old one's pinned
        # words, which therefore must stay allocated: replays after the reset work as before
        sample._sample.reset_routing()
    for i in range(2):
        ref_a, _ = oracle.sample_batch(lg_np, c, k, p, rng=rng_ref)
        ref_b, _ = oracle.sample_batch(lg_np, c, k, p, rng=rng_ref, penalties=pen_ref, presence=0.1, repetition=0.2, decay=0.9)
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(a.cpu().numpy(), ref_a) and np.array_equal(b.cpu().numpy(), ref_b), ("after reset_routing", i)
    # a stream without a workspace: the first call would have to allocate while capturing
    other = torch.cuda.Stream()
    with torch.cuda.stream(other):
        with pytest.raises(RuntimeError, match="reserve_workspace"):
            with torch.cuda.graph(torch.cuda.CUDAGraph(), stream=other):
                sample.batch_sampling_temperature_topk_topp(lg, st, 0.9, 40, 0.9)
    torch.cuda.synchronize()


def test_chi_square_one_million_draws(torch_cuda, oracle):
    """1,048,576 Philox-driven draws of one row against the exact renormalised weights w_i / S."""
    torch = torch_cuda
    from scipy import stats
    from tests import capi
    B, V, calls = 8192, 1024, 128
    row = H.logits_normal(1, V, 1.5, seed=60)
    rc, c, k, p = capi.normalize(1.0, 40, 0.9, V, B, 1)
    d = oracle.sample_row(row[0], c, k, p, u=0.5, want_e=True)
    e, thr = d["e_bits"], d["thr_bits"]
    w = np.where(e > thr, oracle.w_of(e).astype(np.float64), 0.0)
    w[e == thr] = float(d["w_tie"])
    assert abs(w.sum() - float(d["S"])) <= 1e-6 * float(d["S"])
    lg = torch.from_numpy(np.repeat(row, B, axis=0)).cuda()
    smp = capi.Sampler(B, V)
    st = torch.empty(B * 64, dtype=torch.int8, device="cuda")
    assert capi.lib().rs_philox_init(st.data_ptr(), 7, B, smp.stream()) == 0
    counts = np.zeros(V, dtype=np.int64)
    for _ in range(calls):
        res = smp.sample(lg, c, k, p, rng=st, want_diag=False)
        assert res["rc"] == 0
        counts += np.bincount(res["out"], minlength=V)
    n = B * calls
    assert counts[w == 0].sum() == 0, "a dropped token was sampled"
    keep = w > 0
    chi2, pval = stats.chisquare(counts[keep], n * w[keep] / w.sum())
    print("chi2", chi2, "dof", keep.sum() - 1, "p", pval)
    assert pval > 0.01
