"""The drop-in libraries a reference installation would load in place of its own
(ai2pot/fromcc/__init__.py:53-134): torch.ops.nep / mtpr / fvt registered by
ai2pot_amd/_lib/lib*_bind.so and the CPython module `nblist`.  They must give the same
results as the Python mirror of the operators (which the oracle parity tests cover) and be
callable from TorchScript by name, as the exported models do (ai2pot/models/nep/nep.py:297-324)."""
import os
import sys

import numpy as np
import pytest

from ai2pot_amd import mtp_param, synth
from conftest import to_device

pytestmark = pytest.mark.gpu

LIBDIR = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "ai2pot_amd", "_lib")


@pytest.fixture(scope="module")
def dropin():
    import torch
    for name in ("libnep_bind.so", "libmtpr_bind.so", "libnnmtp_bind.so", "libfvt_sr_op_bind.so", "libnblist_bind.so"):
        path = os.path.join(LIBDIR, name)
        assert os.path.exists(path), "%s missing: run python -m ai2pot_amd.build --bind" % path
        torch.ops.load_library(path)
    if LIBDIR not in sys.path:
        sys.path.append(LIBDIR)
    import nblist
    return nblist


def small(oracle, n=120, nt=3, rcut=7.0, seed=11, dtype=np.float32):
    lat, pos = synth.random_packed(n, [14.0, 15.0, 13.0], 2.2, seed)
    ty = synth.rng_randint(seed + 1, n, nt)
    return lat, pos, ty, oracle.nblist(lat.astype(dtype), ty, pos.astype(dtype), rcut, 200)


def test_nblist_module(oracle, dropin):
    lat, pos, ty, ref = small(oracle)
    out = dropin.find_info4mlff(lat.astype(np.float32), ty, pos.astype(np.float32), 7.0, 200, True,
                                [True, True, True], False)
    assert out[0] == ref[0] and out[6] == 0
    for a, b in zip(out[1:6], ref[1:6]):
        assert np.array_equal(a.view(np.uint8), b.view(np.uint8))
    out64 = dropin.find_info4mlff(lat, ty.astype(np.int64), pos, 7.0, 200, True, [True, True, True], True)
    ref64 = oracle.nblist(lat, ty, pos, 7.0, 200, sort=True)
    for a, b in zip(out64[1:6], ref64[1:6]):
        assert np.array_equal(a.view(np.uint8), b.view(np.uint8))
    with pytest.raises(TypeError):
        dropin.find_info4mlff(lat, ty, pos, 7, 200, True, [True, True, True], False)
    with pytest.raises(RuntimeError):
        dropin.find_info4mlff(lat, ty, pos, 7.0, 10, True, [True, True, True], False)


@pytest.mark.parametrize("np_dtype", [np.float32, np.float64])
def test_nblist_op_on_device_tensors(oracle, dropin, np_dtype):
    """torch.ops.nblist.find_info4mlff: the arguments and seven results of the reference's
    nblist.find_info4mlff (source/nblist/bind/nblist_bind.cc:35-189) as device tensors, bit-identical
    to the oracle in both sort modes; the in-place form rewrites an earlier result."""
    import torch
    lat, pos, ty, ref = small(oracle, dtype=np_dtype)
    dev = "cuda:0"
    tlat = torch.from_numpy(lat.astype(np_dtype))
    tty = torch.from_numpy(ty.astype(np.int32)).to(dev)
    tpos = torch.from_numpy(pos.astype(np_dtype)).to(dev)
    for sort in (False, True):
        want = oracle.nblist(lat.astype(np_dtype), ty, pos.astype(np_dtype), 7.0, 200, sort=sort)
        out = torch.ops.nblist.find_info4mlff(tlat, tty, tpos, 7.0, 200, True, [True, True, True], sort)
        assert len(out) == 7 and all(t.is_cuda for t in out)
        assert int(out[0]) == want[0] and int(out[6]) == 0
        for a, b in zip(out[1:6], want[1:6]):
            assert a.shape == b.shape
            assert np.array_equal(a.cpu().numpy().view(np.uint8), b.view(np.uint8))
    # the lattice may live on the device too
    out_d = torch.ops.nblist.find_info4mlff(tlat.to(dev), tty, tpos, 7.0, 200, True, [True, True, True], False)
    assert all(torch.equal(a, b) for a, b in zip(out_d, torch.ops.nblist.find_info4mlff(
        tlat, tty, tpos, 7.0, 200, True, [True, True, True], False)))
    # in place over an earlier list of other positions
    lat2, pos2 = synth.random_packed(120, [14.0, 15.0, 13.0], 2.2, 29)
    bufs = [t.clone() for t in torch.ops.nblist.find_info4mlff(
        tlat, tty, torch.from_numpy(pos2.astype(np_dtype)).to(dev), 7.0, 200, True, [True, True, True], False)[1:6]]
    torch.ops.nblist.find_info4mlff_(tlat, tty, tpos, 7.0, 200, True, [True, True, True], False, *bufs, True)
    nn = ref[2]
    for a, b in zip(bufs[:2] + bufs[4:], (ref[1], ref[2], ref[5])):
        assert np.array_equal(a.cpu().numpy(), b)
    fn, rc = bufs[2].cpu().numpy(), bufs[3].cpu().numpy()
    for i in range(120):                                   # beyond a row's length the old entries may remain
        assert np.array_equal(fn[i, :nn[i]], ref[3][i, :nn[i]])
        assert np.array_equal(rc[i, :nn[i]].view(np.uint8), ref[4][i, :nn[i]].view(np.uint8))
    with pytest.raises(RuntimeError):                      # umax too small: an error with validation on
        torch.ops.nblist.find_info4mlff(tlat, tty, tpos, 7.0, 10, True, [True, True, True], False)
    with pytest.raises(RuntimeError):                      # host coordinates: no CPU path
        torch.ops.nblist.find_info4mlff(tlat, tty.cpu(), tpos.cpu(), 7.0, 200, True, [True, True, True], False)
    with pytest.raises(RuntimeError):
        torch.ops.nblist.find_info4mlff(tlat.double() if np_dtype == np.float32 else tlat.float(), tty, tpos, 7.0,
                                        200, True, [True, True, True], False)


@pytest.mark.parametrize("np_dtype", [np.float32, np.float64])
def test_compact_ops_match_the_calculator_and_the_oracle(oracle, dropin, np_dtype):
    """torch.ops.nblist.find_info4mlff_compact_ + torch.ops.nep.nepToEFVCompactOp: the device-resident
    step through registered operators only.  Same kernels as NepCalculator(path="gather"), so the
    results are bitwise the calculator's; and within the gather path's bars of the oracle."""
    import torch
    from ai2pot_amd.calculator import NepCalculator
    from test_gpu_nep import _model_to_device
    from test_gpu_nep_gather import _check
    dev = "cuda:0"
    dtype = torch.float32 if np_dtype == np.float32 else torch.float64
    lat, pos, ty, nb = small(oracle, dtype=np_dtype)
    m = synth.nep_model()
    md = _model_to_device(m, dtype)
    n, U = 120, 200
    tlat = torch.from_numpy(lat.astype(np_dtype))
    tty = torch.from_numpy(ty.astype(np.int32)).to(dev)
    tpos = torch.from_numpy(pos.astype(np_dtype)).to(dev)
    nbytes = torch.ops.nblist.compact_bytes(n, U, 4 if np_dtype == np.float32 else 8)
    assert nbytes > 0 and torch.ops.nblist.compact_bytes(n, 13, 4) == 0
    compact = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    i32 = dict(dtype=torch.int32, device=dev)
    rows = [torch.empty(n, **i32), torch.empty(n, **i32), torch.empty((n, U), **i32),
            torch.empty((n, U, 3), dtype=dtype, device=dev), torch.empty(n, **i32)]
    model_args = (8, 6, 4, 4, md["coeffs"], md["w0"], md["b0"], md["w1"], md["type_bias"])
    tail = (md["type_map"], float(m["rmax_radial"]), float(m["rmax_angular"]), md["q_scaler"])
    calc = NepCalculator(m, n, lat, ty, umax=U, dtype=dtype, device=dev, path="gather")
    for with_rows in (True, False):
        torch.ops.nblist.find_info4mlff_compact_(tlat, tty, tpos, 7.0, U, True, [True, True, True],
                                                 float(m["rmax_radial"]), float(m["rmax_angular"]), 0,
                                                 *(rows if with_rows else [None] * 5), compact)
        e, f, v = torch.ops.nep.nepToEFVCompactOp(*model_args, tty, compact, U, *tail)
        assert e.shape == (1,) and f.shape == (1, n, 3) and v.shape == (1, 9)
        ce, cf, cv = calc.step(tpos)
        calc.check()
        assert torch.equal(e, ce) and torch.equal(f[0], cf) and torch.equal(v[0], cv)
    for a, b in zip(rows, nb[1:6]):                        # the padded tensors, bit for bit
        assert np.array_equal(a.cpu().numpy().view(np.uint8), b.view(np.uint8))
    ref = oracle.nep_efv(m, synth.pack_batch([nb]), dtype=np_dtype)
    _check((e.cpu().numpy(), f.cpu().numpy(), v.cpu().numpy()), ref, np_dtype)
    # validation off: no per-call synchronisation, a flagged call surfaces at check_status
    torch.ops.nblist.set_validate(False)
    try:
        small_compact = torch.empty(torch.ops.nblist.compact_bytes(n, 8, 4 if np_dtype == np.float32 else 8),
                                    dtype=torch.uint8, device=dev)
        torch.ops.nblist.find_info4mlff_compact_(tlat, tty, tpos, 7.0, 8, True, [True, True, True], 7.0, 4.0, 0,
                                                 None, None, None, None, None, small_compact)
        with pytest.raises(RuntimeError):
            torch.ops.nblist.check_status(tpos)
    finally:
        torch.ops.nblist.set_validate(True)
    with pytest.raises(RuntimeError):                      # a buffer that is too small is refused on the host
        torch.ops.nep.nepToEFVCompactOp(*model_args, tty, compact[:1024], U, *tail)
    with pytest.raises(RuntimeError):                      # padded outputs: all or none
        torch.ops.nblist.find_info4mlff_compact_(tlat, tty, tpos, 7.0, U, True, [True, True, True], 7.0, 4.0, 0,
                                                 rows[0], None, None, None, None, compact)


def nep_args(oracle, dtype):
    import torch
    from test_gpu_nep import _model_to_device
    _, _, _, o = small(oracle)
    nb = synth.pack_batch([o])
    m = synth.nep_model()
    md = _model_to_device(m, dtype)
    d = to_device(nb, dtype)
    return (8, 6, 4, 4, md["coeffs"], md["w0"], md["b0"], md["w1"], md["type_bias"], d["binum"], d["bilist"],
            d["bnumneigh"], d["bfirstneigh"], d["brcs"], d["btypes"], md["type_map"], 0, 7.0, 4.0, md["q_scaler"],
            0.0, 0.0, torch.zeros(36, dtype=dtype, device="cuda:0"), torch.zeros(36, dtype=dtype, device="cuda:0"))


def test_nep_ops_and_torchscript(oracle, dropin):
    import torch
    from ai2pot_amd import ops
    args = nep_args(oracle, torch.float32)
    got = torch.ops.nep.nepToEFVOp(*args)
    want = ops.nepToEFVOp(*args)
    assert len(got) == 3
    for a, b in zip(got, want):
        assert torch.equal(a, b)
    ef = torch.ops.nep.nepToEFOp(*args)
    assert len(ef) == 2 and torch.equal(ef[0], want[0]) and torch.equal(ef[1], want[1])
    # with the ZBL correction switched on the registered operator and the Python mirror agree
    ck = torch.tensor([0.18175, 0.50986, 0.28022, 0.02817], device="cuda:0").repeat(9)
    dk = torch.tensor([3.1998, 0.94229, 0.4029, 0.20162], device="cuda:0").repeat(9)
    zgot = torch.ops.nep.nepToEFVOp(*(args[:20] + (2.4, 1.2, ck, dk)))
    zwant = ops.nepToEFVOp(*(args[:20] + (2.4, 1.2, ck, dk)))
    assert all(torch.equal(a, b) for a, b in zip(zgot, zwant)) and not torch.equal(zgot[0], want[0])
    d = torch.ops.nep.nepToDescriptorsOp(*(args[:5] + args[9:19]))
    assert d[0].shape == (1, 120, 22)
    assert torch.equal(d[0], ops.nepToDescriptorsOp(*(args[:5] + args[9:19]))[0])

    class Wrapper(torch.nn.Module):
        def __init__(self, consts):
            super().__init__()
            self.coeffs, self.w0, self.b0, self.w1, self.bias, self.type_map, self.qs, self.z = consts

        @torch.jit.export
        def predict_efv(self, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes):
            return torch.ops.nep.nepToEFVOp(8, 6, 4, 4, self.coeffs, self.w0, self.b0, self.w1, self.bias, binum,
                                            bilist, bnumneigh, bfirstneigh, brcs, btypes, self.type_map, 0, 7.0, 4.0,
                                            self.qs, 0.0, 0.0, self.z, self.z)

        def forward(self, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes):
            return self.predict_efv(binum, bilist, bnumneigh, bfirstneigh, brcs, btypes)

    mod = torch.jit.script(Wrapper((args[4], args[5], args[6], args[7], args[8], args[15], args[19], args[22])))
    out = mod.predict_efv(*args[9:15])
    for a, b in zip(out, want):
        assert torch.equal(a, b)
    with pytest.raises(RuntimeError):                      # wrong dtype is an error, not a crash
        torch.ops.nep.nepToEFVOp(*(args[:13] + (args[13].double(),) + args[14:]))
    with pytest.raises(RuntimeError):
        torch.ops.nep.nepToLossOp(1.0, 1.0, 1.0, args[4], args[4], args[4], *args)


def test_mtpr_ops(oracle, dropin, tmp_path):
    import torch
    from ai2pot_amd import ops
    from test_gpu_mtp import model_to_device
    # template directory materialised from the packaged tables; the library parses the text file
    d = tmp_path / "_data" / "MTP_templates"
    d.mkdir(parents=True)
    mtp_param.write_almtp(str(d / "10.almtp"), mtp_param.mtp_param(10))
    os.environ.pop("AI2POT_PATH", None)
    torch.ops.mtpr.set_ai2pot_path(str(tmp_path))
    p = torch.ops.mtpr.mtpParamOp(10)
    want = ops.mtpParamOp(10)
    assert len(p) == 7
    for a, b in zip(p, want):
        assert a.dtype == torch.int32 and torch.equal(a, b)
    with pytest.raises(RuntimeError):
        torch.ops.mtpr.mtpParamOp(12)                      # no such template file in that directory

    lat, pos, ty, o = small(oracle, n=60, nt=2, rcut=5.0, dtype=np.float64)
    nb = synth.pack_batch([o, o])
    nb["brcs"][1] *= 1.02
    m = synth.mtp_model(mtp_param.mtp_param(10), 2, 8, 5.0, 1.0, 77)
    md = model_to_device(m, torch.float64)
    dv = to_device(nb, torch.float64)
    z = torch.zeros(16, dtype=torch.float64, device="cuda:0")
    efv_args = (8, 1.0, md["coeffs"], md["linear_coeffs"], md["type_bias"], int(p[0]), p[1].cuda(), p[2].cuda(),
                p[3].cuda(), int(p[6]), dv["binum"], dv["bilist"], dv["bnumneigh"], dv["bfirstneigh"], dv["brcs"],
                dv["btypes"], md["type_map"], 0, 5.0, 1.0, md["q_scaler"], 0.0, 0.0, z, z)
    got = torch.ops.mtpr.linearMtpToEFVOp(*efv_args)
    ref = oracle.mtp_efv(m, nb)
    for a, b in zip(got, ref):
        assert np.abs(a.cpu().numpy() - b).max() <= 1e-10 * np.abs(b).max()
    assert len(torch.ops.mtpr.linearMtpToEFOp(*efv_args)) == 2

    B, P = nb["bilist"].shape
    lab = dict(energy=synth.rng_normal(1, B, -200, 3), force=synth.rng_normal(2, B * P * 3).reshape(B, P, 3),
               virial=synth.rng_normal(3, B * 9).reshape(B, 9))
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    params = [md[k].clone().requires_grad_(True) for k in ("coeffs", "linear_coeffs", "type_bias")]
    out = torch.ops.mtpr.linearMtpToLossOp(1.0, 0.7, 0.3, t(lab["energy"]), t(lab["force"]), t(lab["virial"]), 8, 1.0,
                                           params[0], params[1], params[2], *efv_args[5:])
    assert len(out) == 4 and out[0].shape == (B,)
    out[0].sum().backward()
    r = oracle.mtp_loss_step(m, nb, (1.0, 0.7, 0.3), lab)
    close = lambda a, b: np.abs(a - b).max() <= 1e-10 * np.abs(b).max()
    assert close(out[0].detach().cpu().numpy(), r["bloss"])
    assert close(torch.cat(out[1:]).detach().cpu().numpy(), r["rmse"])
    assert close(params[0].grad.cpu().numpy(), r["dcoeffs"].sum(0))
    assert close(params[1].grad.cpu().numpy(), r["dlinear"].sum(0))
    assert close(params[2].grad.cpu().numpy(), r["dbias"].sum(0))
    # energy + force loss: the same with the virial weight switched off
    params2 = [md[k].clone().requires_grad_(True) for k in ("coeffs", "linear_coeffs", "type_bias")]
    out2 = torch.ops.mtpr.linearMtpToEFLossOp(1.0, 0.7, t(lab["energy"]), t(lab["force"]), 8, 1.0, params2[0],
                                              params2[1], params2[2], *efv_args[5:])
    assert len(out2) == 3
    out2[0].sum().backward()
    r2 = oracle.mtp_loss_step(m, nb, (1.0, 0.7, 0.0), lab)
    assert close(out2[0].detach().cpu().numpy(), r2["bloss"]) and close(params2[0].grad.cpu().numpy(), r2["dcoeffs"].sum(0))
    # linear-solver operators
    A, bvec = torch.ops.mtpr.LinMatrixLinVectorOp(1.0, 0.7, 0.3, t(lab["energy"]), t(lab["force"]), t(lab["virial"]),
                                                  *efv_args)
    Ar, br = oracle.mtp_lin_system(m, nb, (1.0, 0.7, 0.3), lab)
    assert close(A.cpu().numpy(), Ar) and close(bvec.cpu().numpy(), br)
    oc = torch.ops.mtpr.CoeffsSchmidtOrthOp(2, int(p[6]), 8, md["coeffs"])
    assert len(oc) == 1 and close(oc[0].cpu().numpy(), oracle.mtp_schmidt_orth(m["coeffs"], 2, int(p[6]), 8))
    # site energies (autograd) and descriptors
    params3 = [md[k].clone().requires_grad_(True) for k in ("coeffs", "linear_coeffs", "type_bias")]
    es = torch.ops.mtpr.linearMtpToEsitesOp(8, 1.0, params3[0], params3[1], params3[2], *efv_args[5:])
    desc = torch.ops.mtpr.linearMtpToDescriptorsOp(8, 1.0, md["coeffs"], *efv_args[5:20])
    es_ref, desc_ref = oracle.mtp_esites(m, nb)
    assert len(es) == 1 and len(desc) == 1
    assert close(es[0].detach().cpu().numpy(), es_ref) and close(desc[0].cpu().numpy(), desc_ref)
    gout = synth.rng_normal(4, B * P).reshape(B, P)
    (es[0] * t(gout)).sum().backward()
    rc, rl, rb = oracle.mtp_esites_bwd(m, nb, gout)
    assert close(params3[0].grad.cpu().numpy(), rc.sum(0)) and close(params3[1].grad.cpu().numpy(), rl.sum(0))
    assert close(params3[2].grad.cpu().numpy(), rb.sum(0))
    # the legacy basis operator: the scalar moments, differentiable w.r.t. coeffs and brcs
    S = int(p[3].numel())
    w = synth.rng_normal(5, B * P * S).reshape(B, P, S)
    cb = md["coeffs"].clone().requires_grad_(True)
    rb_ = dv["brcs"].clone().requires_grad_(True)
    val = torch.ops.mtpr.mtpBasisOp(p[1].cuda(), p[2].cuda(), p[3].cuda(), p[4].cuda(), p[5].cuda(), p[6], 2, 8, 1.0, cb,
                                    dv["binum"], dv["bilist"], dv["bnumneigh"], dv["bfirstneigh"], rb_, dv["btypes"],
                                    int(rb_.shape[2]), 5.0, 1.0)
    assert len(val) == 1 and close(val[0].detach().cpu().numpy(), desc_ref)
    (val[0] * t(w)).sum().backward()
    dr_ref, dc_ref = oracle.mtp_basis_bwd(m, nb, w)
    assert close(rb_.grad.cpu().numpy(), dr_ref) and close(cb.grad.cpu().numpy().ravel(), dc_ref.sum(0))


def test_nnmtp_ops(oracle, dropin, tmp_path):    assert close(params3[2].grad.cpu().numpy(), rb.sum(0))


def test_nnmtp_ops(oracle, dropin, tmp_path):
    import torch
    from ai2pot_amd import ops
    from test_gpu_nnmtp import model_to_device, op_args
    d = tmp_path / "_data" / "MTP_templates"
    d.mkdir(parents=True)
    mtp_param.write_almtp(str(d / "10.almtp"), mtp_param.mtp_param(10))
    os.environ.pop("AI2POT_PATH", None)
    torch.ops.nnmtp.set_ai2pot_path(str(tmp_path))
    p = torch.ops.nnmtp.mtpParamOp(10)
    assert len(p) == 7 and int(p[0]) == mtp_param.mtp_param(10)["alpha_moments_count"]
    lat, pos, ty, o = small(oracle, n=60, nt=2, rcut=5.0, dtype=np.float64)
    nb = synth.pack_batch([o, o])
    nb["brcs"][1] *= 1.02
    m = synth.nnmtp_model(mtp_param.mtp_param(10), 2, 8, 12, 5.0, 1.0, 77)
    md = model_to_device(m, torch.float64)
    z = torch.zeros(16, dtype=torch.float64, device="cuda:0")
    args = op_args(m, md, to_device(nb, torch.float64)) + (0.0, 0.0, z, z)
    close = lambda a, b: np.abs(a.cpu().numpy() - b).max() <= 1e-10 * np.abs(b).max()
    er, fr, vr, esr = oracle.nnmtp_efv(m, nb)
    e, f, v = torch.ops.nnmtp.nnMtpToEFVOp(*args)
    assert close(e, er) and close(f, fr) and close(v, vr)
    assert len(torch.ops.nnmtp.nnMtpToEFOp(*args)) == 2
    assert close(torch.ops.nnmtp.nnMtpToEsitesOp(*args)[0], esr)
    desc = torch.ops.nnmtp.nnMtpToDescriptorsOp(*(args[:2] + args[5:20]))[0]
    lin = dict(m); lin["scaling"] = 1.0; lin["linear_coeffs"] = np.zeros(m["q_scaler"].size)
    assert close(desc, oracle.mtp_esites(lin, nb)[1])
    # training operators: the reference's formulas by default, as committed from its own backward
    B, P = nb["bilist"].shape
    lab = dict(energy=synth.rng_normal(1, B, -200, 3), force=synth.rng_normal(2, B * P * 3).reshape(B, P, 3),
               virial=synth.rng_normal(3, B * 9).reshape(B, 9))
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    params = [md[k].clone().requires_grad_(True) for k in ("coeffs", "w0", "w1", "type_bias")]
    pargs = args[:1] + tuple(params) + args[5:]
    out = torch.ops.nnmtp.nnMtpToLossOp(1.0, 0.7, 0.3, t(lab["energy"]), t(lab["force"]), t(lab["virial"]), *pargs)
    assert len(out) == 1 and out[0].shape == (B,)
    out[0].sum().backward()
    r = ops.nnmtp_loss_step(1.0, 0.7, 0.3, t(lab["energy"]), t(lab["force"]), t(lab["virial"]), *args[:22],
                            exact_gradient=False)
    assert torch.equal(out[0].detach(), r["bloss"])
    for prm, key in zip(params, ("dcoeffs", "dw0", "dw1", "dbias")):
        assert close(prm.grad, r[key].sum(0).cpu().numpy()), key
    rr = oracle.nnmtp_loss_step(m, nb, (1.0, 0.7, 0.3), lab)
    assert close(out[0].detach(), rr["bloss"]) and close(params[2].grad, rr["dw1"].sum(0))
    out2 = torch.ops.nnmtp.nnMtpToEFLossOp(1.0, 0.7, t(lab["energy"]), t(lab["force"]), *args)
    assert len(out2) == 1 and close(out2[0], oracle.nnmtp_loss_step(m, nb, (1.0, 0.7, 0.0), lab)["bloss"])
    w0g = md["w0"].clone().requires_grad_(True)
    es_g = torch.ops.nnmtp.nnMtpToEsitesOp(*(args[:2] + (w0g,) + args[3:]))[0]
    gout = synth.rng_normal(4, B * P).reshape(B, P)
    (es_g * t(gout)).sum().backward()
    assert close(w0g.grad, oracle.nnmtp_esites_bwd(m, nb, gout)[1].sum(0))


def test_fvt_ops(oracle, dropin):
    import torch
    from test_gpu_fvt import dev, random_case
    binum, bilist, nn, fn, dei, rcs = random_case(B=2, P=5, U=4, nghost=2, seed=3)
    U = fn.shape[2]
    lists = (dev(binum), dev(bilist), dev(nn), dev(fn))
    d = dev(dei).requires_grad_(True)
    r = dev(rcs).requires_grad_(True)
    force = lambda x: torch.ops.fvt.ForceSrOp(lists[0], lists[1], lists[2], lists[3], 2, U, x)[0]
    virial = lambda rr, x: torch.ops.fvt.VirialSrOp(lists[2], rr, U, x)[0]
    f = force(d)
    for b in range(2):
        n = binum[b]
        fr, _ = oracle.fvt_force(bilist[b, :n], nn[b, :n], fn[b, :n], 2 + 5 - n, dei[b, :n])
        assert np.abs(f[b].detach().cpu().numpy() - fr).max() < 1e-12
    assert virial(r, d).shape == (2, 3, 3)
    assert torch.autograd.gradcheck(force, (d,), eps=1e-6, atol=1e-7)
    assert torch.autograd.gradgradcheck(force, (d,), eps=1e-6, atol=1e-7)
    assert torch.autograd.gradcheck(virial, (r, d), eps=1e-6, atol=1e-7)
    assert torch.autograd.gradgradcheck(virial, (r, d), eps=1e-6, atol=1e-7)


def test_nep_loss_ops(dropin):
    """torch.ops.nep.nepToLossOp / nepToEFLossOp against the reference's own output."""
    import torch
    from test_gpu_nep_loss import GRADS, PARAMS, close, golden_case
    g, m, nb, labels = golden_case()
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a, np.float64)).to("cuda:0")
    d = to_device(nb, torch.float64)
    params = [t(m[k]).requires_grad_(True) for k in PARAMS]
    z = torch.zeros(16, dtype=torch.float64, device="cuda:0")
    tail = (d["binum"], d["bilist"], d["bnumneigh"], d["bfirstneigh"], d["brcs"], d["btypes"],
            torch.from_numpy(np.asarray(m["type_map"], np.int32)).to("cuda:0"), 0, m["rmax_radial"], m["rmax_angular"],
            t(m["q_scaler"]), 0.0, 0.0, z, z)
    sizes = (m["chebyshev_size"], m["n_radial_basis"], m["n_angular_basis"], m["l_max"])
    out = torch.ops.nep.nepToLossOp(1.0, 0.7, 0.3, t(labels["energy"]), t(labels["force"]), t(labels["virial"]),
                                    *sizes, *params, *tail)
    assert len(out) == 4 and close(out[0].detach().cpu().numpy(), g["efv/bloss"])
    assert close(torch.cat(out[1:]).detach().cpu().numpy(), g["efv/rmse"])
    gl = torch.tensor([1.5, -0.5], dtype=torch.float64, device="cuda:0")
    (out[0] * gl).sum().backward()
    for p, k in zip(params, GRADS):
        assert close(p.grad.cpu().numpy().ravel(), gl.cpu().numpy() @ g["efv/" + k]), k
    out2 = torch.ops.nep.nepToEFLossOp(1.0, 0.7, t(labels["energy"]), t(labels["force"]), *sizes,
                                       *[p.detach() for p in params], *tail)
    assert len(out2) == 3 and close(out2[0].cpu().numpy(), g["ef/bloss"])


def test_asymmetric_list_names_an_atom_more_often_than_a_row_is_long(oracle, dropin):
    """A list in which one atom is named by more pairs than umax (here every row names atom 0 in all of
    its slots, as a half list or a ghost shared by several rows can): the fixed reduction segments of
    the fast kernels overflow, the status says so, and both operator layers repeat the call with larger
    segments.  Results equal the oracle's scatter; with validation off the overflow is reported by an
    explicit status check and by nothing else."""
    import torch
    from ai2pot_amd import _lib, ops
    from test_gpu_nep import _model_to_device, check
    _, _, _, o = small(oracle, n=120, dtype=np.float64)
    o = list(o)
    umax = int(np.asarray(o[2]).max())
    umax += (-umax) % 4
    rows = np.asarray(o[3])[:, :umax].copy()
    rows[rows >= 0] = 0                                    # every pair names atom 0: 120 rows x ~50 pairs > umax
    o[3] = rows
    o[4] = np.asarray(o[4])[:, :umax].copy()
    nb = synth.pack_batch([tuple(o)])
    assert int((rows == 0).sum()) > umax
    m = synth.nep_model()
    md = _model_to_device(m, torch.float64)
    d = to_device(nb, torch.float64)
    z = torch.zeros(36, dtype=torch.float64, device="cuda:0")
    args = (8, 6, 4, 4, md["coeffs"], md["w0"], md["b0"], md["w1"], md["type_bias"], d["binum"], d["bilist"],
            d["bnumneigh"], d["bfirstneigh"], d["brcs"], d["btypes"], md["type_map"], 0, 7.0, 4.0, md["q_scaler"],
            0.0, 0.0, z, z)
    ref = oracle.nep_efv(m, nb, np.float64)
    for fn in (ops.nepToEFVOp, torch.ops.nep.nepToEFVOp):
        out = [t.cpu().numpy() for t in fn(*args)]
        check(out, ref, np.float64)
    # validation off: no exception from the call, the explicit check reports the overflow
    ops.nepToEFVOp(*args, validate=False)
    with pytest.raises(_lib.A2PError) as ei:
        _lib.check_status(torch.cuda.current_stream().cuda_stream)
    assert ei.value.code == _lib.A2P_ERR_SEGMENT
    torch.ops.nep.set_validate(False)
    try:
        torch.ops.nep.nepToEFVOp(*args)
        with pytest.raises(RuntimeError):
            torch.ops.nep.check_status(d["brcs"])
    finally:
        torch.ops.nep.set_validate(True)
    # linear MTP through the same segments
    tables = mtp_param.mtp_param(10)
    mm = synth.mtp_model(tables, 3, 8, 7.0, 0.5, 77)
    f64 = lambda a: torch.from_numpy(np.ascontiguousarray(a, np.float64)).to("cuda:0")
    i32 = lambda a: torch.from_numpy(np.ascontiguousarray(a, np.int32)).to("cuda:0")
    margs = (mm["chebyshev_size"], 1.0, f64(mm["coeffs"]), f64(mm["linear_coeffs"]), f64(mm["type_bias"]),
             mm["alpha_moments_count"], i32(mm["alpha_index_basic"]), i32(mm["alpha_index_times"]),
             i32(mm["alpha_moment_mapping"]), mm["nmus"], d["binum"], d["bilist"], d["bnumneigh"], d["bfirstneigh"],
             d["brcs"], d["btypes"], i32(mm["type_map"]), 0, mm["rmax"], mm["rmin"], f64(mm["q_scaler"]), 0.0, 0.0, z, z)
    mref = oracle.mtp_efv(mm, nb)
    for fn in (ops.linearMtpToEFVOp, torch.ops.mtpr.linearMtpToEFVOp):
        out = [t.cpu().numpy() for t in fn(*margs)]
        check(out, mref, np.float64)


def test_bind_libraries_against_the_oracle_at_working_sizes(oracle, dropin):
    """The registered operators compared with the oracle directly (not through the Python mirror) at sizes where
    every kernel variant behind them is in play: NEP fp32 at 2,000 atoms (the 8-lanes-per-atom kernel), linear MTP
    fp64 at level 20 with 4 species (256 threads per atom, monomial walk)."""
    import torch
    from test_gpu_nep import _model_to_device
    from test_gpu_nep_gather import _check
    from test_gpu_mtp import model_to_device
    dev = "cuda:0"
    # NEP through torch.ops.nblist + torch.ops.nep on device tensors
    n = 2000
    Lc = (n / 0.033) ** (1.0 / 3.0)
    lat, pos = synth.random_packed(n, [Lc, Lc, Lc], 2.2, 411)
    ty = synth.rng_randint(412, n, 3)
    m = synth.nep_model(seed=413)
    md = _model_to_device(m, torch.float32)
    out = torch.ops.nblist.find_info4mlff(torch.from_numpy(lat.astype(np.float32)),
                                          torch.from_numpy(ty.astype(np.int32)).to(dev),
                                          torch.from_numpy(pos.astype(np.float32)).to(dev), 7.0, 200, True,
                                          [True, True, True], False)
    ref_list = oracle.nblist(lat.astype(np.float32), ty, pos.astype(np.float32), 7.0, 200)
    for a, b in zip(out[1:6], ref_list[1:6]):
        assert np.array_equal(a.cpu().numpy().view(np.uint8), b.view(np.uint8))
    z = torch.zeros(36, dtype=torch.float32, device=dev)
    got = torch.ops.nep.nepToEFVOp(8, 6, 4, 4, md["coeffs"], md["w0"], md["b0"], md["w1"], md["type_bias"],
                                   out[0], out[1].unsqueeze(0), out[2].unsqueeze(0), out[3].unsqueeze(0),
                                   out[4].unsqueeze(0), out[5].unsqueeze(0), md["type_map"], 0, 7.0, 4.0,
                                   md["q_scaler"], 0.0, 0.0, z, z)
    ref = oracle.nep_efv(m, synth.pack_batch([ref_list]), np.float32)
    _check(tuple(t.cpu().numpy() for t in got), ref, np.float32)
    # linear MTP, level 20
    n = 300
    lat, pos = synth.random_packed(n, [20.0, 18.0, 16.7], 2.0, 421)
    ty = synth.rng_randint(422, n, 4)
    nbl = oracle.nblist(lat, ty, pos, 5.5, 200)
    nb = synth.pack_batch([nbl])
    tables = mtp_param.mtp_param(20)
    mm = synth.mtp_model(tables, 4, 10, 5.5, 1.8, 423, lo=-0.05, hi=0.05)
    mmd = model_to_device(mm, torch.float64)
    dv = to_device(nb, torch.float64)
    z = torch.zeros(64, dtype=torch.float64, device=dev)
    got = torch.ops.mtpr.linearMtpToEFVOp(10, 1.0, mmd["coeffs"], mmd["linear_coeffs"], mmd["type_bias"],
                                          int(mm["alpha_moments_count"]), mmd["alpha_index_basic"],
                                          mmd["alpha_index_times"], mmd["alpha_moment_mapping"], int(mm["nmus"]),
                                          dv["binum"], dv["bilist"], dv["bnumneigh"], dv["bfirstneigh"], dv["brcs"],
                                          dv["btypes"], mmd["type_map"], 0, 5.5, 1.8, mmd["q_scaler"], 0.0, 0.0, z, z)
    ref = oracle.mtp_efv(mm, nb)
    for a, b in zip(got, ref):
        assert np.abs(a.cpu().numpy() - b).max() <= 1e-10 * np.abs(b).max()
