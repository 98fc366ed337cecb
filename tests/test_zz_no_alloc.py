"""The allocation-free virial entry point (a2p_fvt_virial_fwd_noalloc_f32) against the ordinary one
(a2p_fvt_virial_fwd_f32): bit-identical results through the C ABI on two calls in a row, the second
on a smaller input (the built-in buffer still holds the first call's partial sums), and a clear error
beyond its row limit."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _call(fn, B, P, U, nn, rcs, dei, stream):
    import torch
    out = torch.full((B, 9), float("nan"), dtype=torch.float32, device=rcs.device)
    vp = lambda t: ctypes.c_void_p(t.data_ptr())
    rc = fn(ctypes.c_int(B), ctypes.c_int(P), ctypes.c_int(U), vp(nn), vp(rcs), vp(dei), vp(out), stream)
    return rc, out


def test_noalloc_virial_matches_and_reuses_its_buffer():
    import torch
    from ai2pot_amd import _lib
    L = _lib.lib()
    fn_ref, fn_new = L.a2p_fvt_virial_fwd_f32, L.a2p_fvt_virial_fwd_noalloc_f32
    for f in (fn_ref, fn_new):
        f.restype = ctypes.c_int
    L.a2p_workspace_bytes.restype = ctypes.c_size_t
    dev = torch.device("cuda:0")
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    g = torch.Generator(device="cpu").manual_seed(7)
    for B, P, U in ((5, 700, 48), (2, 33, 12)):          # the second call is the smaller one
        nn = torch.randint(0, U + 1, (B, P), generator=g, dtype=torch.int32).to(dev)
        rcs = torch.randn((B, P, U, 3), generator=g, dtype=torch.float32).to(dev)
        dei = torch.randn((B, P, U, 3), generator=g, dtype=torch.float32).to(dev)
        rc0, want = _call(fn_ref, B, P, U, nn, rcs, dei, stream)
        held = L.a2p_workspace_bytes()
        rc1, got = _call(fn_new, B, P, U, nn, rcs, dei, stream)
        torch.cuda.synchronize()
        assert rc0 == 0 and rc1 == 0, L.a2p_last_error().decode()
        assert L.a2p_workspace_bytes() == held                      # the workspace was not touched
        assert torch.isfinite(want).all()
        assert torch.equal(got.view(torch.int32), want.view(torch.int32))
        # closed form in double
        mask = (torch.arange(U, device=dev)[None, None, :] < nn[:, :, None]).double()
        ref = -torch.einsum("bpua,bpuc,bpu->bac", dei.double(), rcs.double(), mask).reshape(B, 9)
        assert torch.allclose(got.double(), ref, rtol=1e-5, atol=1e-3)


def test_noalloc_virial_rejects_sizes_beyond_its_buffer():
    import torch
    from ai2pot_amd import _lib
    L = _lib.lib()
    fn = L.a2p_fvt_virial_fwd_noalloc_f32
    fn.restype = ctypes.c_int
    dev = torch.device("cuda:0")
    B, P, U = 1, 65537, 1
    nn = torch.zeros((B, P), dtype=torch.int32, device=dev)
    x = torch.zeros((B, P, U, 3), dtype=torch.float32, device=dev)
    rc, _ = _call(fn, B, P, U, nn, x, x, ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream))
    assert rc == 1                                                   # A2P_ERR_INVALID
    assert "65536" in L.a2p_last_error().decode()
