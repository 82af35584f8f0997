"""rs_sample_static, the entry point that allocates nothing (its workspace is a static array inside the
library): called through the C ABI and compared with rs_sample_ex on the same inputs, field by field and
bit for bit, on calls in a row whose shapes shrink and grow again; the oracle is run beside them."""
import ctypes as C

import numpy as np
import pytest

from tests import helpers as H

pytestmark = pytest.mark.gpu

FIELDS = ["xmax", "D", "P", "thr_bits", "n_gt", "n_eq", "index", "G", "w_tie", "S", "r", "rounds"]


def _static_call(torch, capi, lg, c, k, p, u, pen=None, path=None, policy=None):
    B, V = lg.shape
    out = torch.full((B,), -7, dtype=torch.int32, device="cuda")
    diag = torch.zeros((B, capi.DIAG_DTYPE.itemsize), dtype=torch.uint8, device="cuda")
    opt = capi.Options(capi.PATHS[path], 0, policy)
    rc = capi.lib().rs_sample_static(lg.data_ptr(), 0, V, pen.data_ptr() if pen is not None else None, out.data_ptr(),
                                     None, u.data_ptr(), B, V, 0.1, 0.2, 0.9, c, k, p, diag.data_ptr(), None,
                                     C.byref(opt), C.c_void_p(torch.cuda.current_stream().cuda_stream))
    if rc != 0:
        return {"rc": rc}
    torch.cuda.synchronize()
    return {"rc": rc, "out": out.cpu().numpy(), "diag": diag.cpu().numpy().view(capi.DIAG_DTYPE).reshape(B)}


def test_static_scratch_entry_point_matches_the_workspace_one():
    import torch
    from oracle import oracle as O
    from tests import capi
    assert torch.cuda.is_available()
    # two calls in a row, the second smaller; then larger again, with penalties, and on the other paths
    shapes = [(8, 65536 + 4096, 50, 0.9, None, False), (3, 32768, 20, 0.8, None, False),
              (8, 65536 + 4096, 50, 0.9, None, False), (5, 131072, -1, 0.3, "attempt", False),
              (6, 40960, 40, 0.95, None, True), (2, 8192, 5, 1.0, "cluster", False), (1, 262144, -1, 0.3, None, False),
              # the one-pass wide path: in the static array, which has no room for this call's slices of 8192
              # tokens, on slices of 16384; in a workspace of rs_workspace_bytes on the shorter ones -- same integers
              (190, 100256, 10000, 1.0, None, False)]
    for n, (B, V, k_in, p_in, path, pen_on) in enumerate(shapes):
        lg_np = H.logits_normal(B, V, 2.5, seed=100 + n)
        u_np = H.uniforms(B, 200 + n)
        rc, c, k, p = capi.normalize(0.9, k_in, p_in, V, B, 1)
        assert rc == 0
        lg, u = torch.from_numpy(lg_np).cuda(), torch.from_numpy(u_np).cuda()
        pen_np = H.penalties_sparse(B, V, seed=300 + n) if pen_on else None
        pen_a = torch.from_numpy(pen_np.copy()).cuda() if pen_on else None
        pen_b = torch.from_numpy(pen_np.copy()).cuda() if pen_on else None
        print("static call", n, B, V, k, p, path, pen_on, flush=True)
        got = _static_call(torch, capi, lg, c, k, p, u, pen=pen_a, path=path)
        assert got["rc"] == 0
        exp = capi.Sampler(B, V).sample(lg, c, k, p, uniforms=u, penalties=pen_b, presence=0.1, repetition=0.2,
                                        decay=0.9, path=path or "auto")
        assert exp["rc"] == 0
        for f in FIELDS:
            assert np.array_equal(got["diag"][f], exp["diag"][f]), (n, f)
        assert np.array_equal(got["out"], exp["out"]), n
        if pen_on:
            assert torch.equal(pen_a.view(torch.int32), pen_b.view(torch.int32))
        pen_ref = pen_np.copy() if pen_on else None
        ref_out, _ = O.sample_batch(lg_np, c, k, p, injected_u=u_np, penalties=pen_ref, presence=0.1, repetition=0.2, decay=0.9)
        assert np.array_equal(got["out"], ref_out), n
    # beyond the static scratch: refused before anything is launched
    need = capi.workspace_bytes(128, 1048576)[1]
    assert need > (32 << 20)
    dummy = torch.zeros(16, dtype=torch.float32, device="cuda")
    opt = capi.Options(0, 0, None)
    rc = capi.lib().rs_sample_static(dummy.data_ptr(), 0, 1048576, None, dummy.data_ptr(), None, dummy.data_ptr(),
                                     128, 1048576, 0.0, 0.0, 1.0, 1.0, 10, 0.5, None, None, C.byref(opt), None)
    assert rc == -10
    assert b"static scratch" in capi.lib().rs_error_string(-10)


def test_static_entry_point_under_graph_capture_allocates_nothing():
    """What the entry point exists for: after rs_static_prepare (the array's address is looked up outside
    capture) a call is recorded into a HIP graph, replayed with changing uniforms and penalties carried from
    replay to replay, every replay checked against the oracle; device memory in use does not change
    across the calls."""
    import torch
    from oracle import oracle as O
    from tests import capi
    B, V = 6, 40960
    assert capi.lib().rs_static_prepare() == 0
    lg_np = H.logits_normal(B, V, 2.0, seed=400)
    pen_ref = H.penalties_sparse(B, V, seed=401)
    rc, c, k, p = capi.normalize(0.9, 40, 0.95, V, B, 1)
    lg = torch.from_numpy(lg_np).cuda()
    pen = torch.from_numpy(pen_ref.copy()).cuda()
    u = torch.zeros(B, dtype=torch.float32, device="cuda")
    out = torch.full((B,), -7, dtype=torch.int32, device="cuda")
    opt = capi.Options(0, 0, None)

    def call():
        rc = capi.lib().rs_sample_static(lg.data_ptr(), 0, V, pen.data_ptr(), out.data_ptr(), None, u.data_ptr(), B, V,
                                         0.1, 0.2, 0.9, c, k, p, None, None, C.byref(opt),
                                         C.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert rc == 0

    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        u.copy_(torch.from_numpy(H.uniforms(B, 410)))
        call()                                                         # eager, also warms the kernels up
        side.synchronize()
        ref_out, _ = O.sample_batch(lg_np, c, k, p, injected_u=H.uniforms(B, 410), penalties=pen_ref, presence=0.1, repetition=0.2, decay=0.9)
        assert np.array_equal(out.cpu().numpy(), ref_out)
        # three more calls with nothing of torch's in between: device memory in use does not move
        pen_keep = pen.clone()
        side.synchronize()
        free0 = torch.cuda.mem_get_info()[0]
        for _ in range(3):
            call()
        side.synchronize()
        assert torch.cuda.mem_get_info()[0] == free0
        pen.copy_(pen_keep)
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            call()
        for step in range(4):
            u_np = H.uniforms(B, 420 + step)
            u.copy_(torch.from_numpy(u_np))
            side.synchronize()
            g.replay()
            side.synchronize()
            ref_out, _ = O.sample_batch(lg_np, c, k, p, injected_u=u_np, penalties=pen_ref, presence=0.1, repetition=0.2, decay=0.9)
            assert np.array_equal(out.cpu().numpy(), ref_out), step
            assert np.array_equal(pen.cpu().numpy().view(np.uint32), pen_ref.view(np.uint32)), step
    st = C.c_int32(-100)
    assert capi.lib().rs_static_status(C.byref(st), None, 0, None) == 0 and st.value == 0


def test_static_entry_point_keeps_error_and_routing_words():
    """The small kernel that clears the launch counters and the call's row records before every call leaves
    the sticky words alone: an error word (set here from the host, at the address rs_static_workspace
    returns) is still there after the next call -- which itself runs correctly -- until rs_static_status
    clears it; and with a policy the routing reports work as with a workspace of the caller's own: a call
    whose rows go the slow way is reported, the next calls take the general kernel, a later good call puts
    the report back."""
    import torch
    from oracle import oracle as O
    from tests import capi
    hip = C.CDLL("libamdhip64.so")
    base = capi.lib().rs_static_workspace()
    assert base
    B, V = 3, 32768
    lg_np = H.logits_normal(B, V, 2.0, seed=430)
    u_np = H.uniforms(B, 431)
    rc, c, k, p = capi.normalize(1.0, 20, 0.9, V, B, 1)
    lg, u = torch.from_numpy(lg_np).cuda(), torch.from_numpy(u_np).cuda()
    ref_out, _ = O.sample_batch(lg_np, c, k, p, injected_u=u_np)
    torch.cuda.synchronize()
    words = (C.c_uint32 * 5)(0xFFFFFFF7, 0, 0, 0, 0)                  # error = -9 (RS_ERR_DEVICE) at byte 8
    assert hip.hipMemcpy(C.c_void_p(base + 8), words, 4, 1) == 0
    where = (C.c_uint32 * 4)(3, 5 << 16 | 2, 7, 9)                     # gave_up[4] at byte 24
    assert hip.hipMemcpy(C.c_void_p(base + 24), where, 16, 1) == 0
    got = _static_call(torch, capi, lg, c, k, p, u)
    assert got["rc"] == 0 and np.array_equal(got["out"], ref_out)      # the call itself starts from clean records
    st, w = C.c_int32(-100), (C.c_uint32 * 4)()
    assert capi.lib().rs_static_status(C.byref(st), w, 1, None) == 0
    assert st.value == -9 and list(w) == [3, 5 << 16 | 2, 7, 9]        # still there, and now cleared
    assert capi.lib().rs_static_status(C.byref(st), w, 0, None) == 0 and st.value == 0 and w[0] == 0

    # routing through a policy: rows whose every other token ties at the top go the slow way on the streaming path
    B, V = 40, 65536
    h = C.c_void_p()
    assert capi.lib().rs_policy_create(C.byref(h)) == 0

    def state():
        s_ = C.c_int32(-1)
        assert capi.lib().rs_policy_state(h, C.byref(s_)) == 0
        return s_.value

    peaked = H.logits_normal(B, V, 3.0, seed=440)
    ties = np.zeros((B, V), dtype=np.float32)
    ties[:, ::2] = 1.0
    u_np = H.uniforms(B, 441)
    rc, c, k, p = capi.normalize(1.0, 10, 1.0, V, B, 1)
    ref_p, _ = O.sample_batch(peaked, c, k, p, injected_u=u_np)
    ref_t, _ = O.sample_batch(ties, c, k, p, injected_u=u_np)
    lg_p, lg_t, u = torch.from_numpy(peaked).cuda(), torch.from_numpy(ties).cuda(), torch.from_numpy(u_np).cuda()
    got = _static_call(torch, capi, lg_p, c, k, p, u, policy=h)
    assert np.array_equal(got["out"], ref_p) and (got["diag"]["rounds"] == 0).all() and state() == 0
    got = _static_call(torch, capi, lg_t, c, k, p, u, policy=h)
    assert np.array_equal(got["out"], ref_t) and state() == 2          # reported at once
    got = _static_call(torch, capi, lg_p, c, k, p, u, policy=h)
    assert np.array_equal(got["out"], ref_p) and (got["diag"]["rounds"] >= 1).all() and state() == 2   # general kernel
    for i in range(66):
        got = _static_call(torch, capi, lg_p, c, k, p, u, policy=h)
        assert np.array_equal(got["out"], ref_p)
    assert state() == 0                                                # a good streaming call, reported by the call after it
    torch.cuda.synchronize()
    capi.lib().rs_policy_destroy(h)
