"""rs_sample_static, the entry point that allocates nothing (its workspace is a static array inside the
library): called through the C ABI and compared with rs_sample_ex on the same inputs, field by field and
bit for bit, on calls in a row whose shapes shrink and grow again; the oracle is run beside them."""
import ctypes as C

import numpy as np
import pytest

from tests import helpers as H

pytestmark = pytest.mark.gpu

FIELDS = ["xmax", "D", "P", "thr_bits", "n_gt", "n_eq", "index", "G", "w_tie", "S", "r", "rounds"]


def _static_call(torch, capi, lg, c, k, p, u, pen=None, path=None):
    B, V = lg.shape
    out = torch.full((B,), -7, dtype=torch.int32, device="cuda")
    diag = torch.zeros((B, capi.DIAG_DTYPE.itemsize), dtype=torch.uint8, device="cuda")
    opt = capi.Options(capi.PATHS[path], 0, None)
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
              (6, 40960, 40, 0.95, None, True), (2, 8192, 5, 1.0, "cluster", False), (1, 262144, -1, 0.3, None, False)]
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
