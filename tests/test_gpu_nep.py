"""GPU parity of the NEP energy / force / virial path against the CPU oracle.

Bars: fp64 results within 1e-10 relative of the oracle; fp32 energies and virials within
1e-5 relative, fp32 forces within 1e-4 eV/A absolute + 1e-5 relative (the oracle evaluates
the fp32 inputs in double, i.e. it is the exactly rounded answer)."""
import numpy as np
import pytest

from ai2pot_amd import synth
from conftest import to_device

pytestmark = pytest.mark.gpu


def _model_to_device(m, dtype, device="cuda:0"):
    import torch
    out = dict(m)
    for k in ("coeffs", "w0", "b0", "w1", "type_bias", "q_scaler"):
        out[k] = torch.from_numpy(np.ascontiguousarray(m[k], np.float64)).to(dtype).to(device)
    out["type_map"] = torch.from_numpy(np.ascontiguousarray(m["type_map"], np.int32)).to(device)
    return out


def run_gpu(m, nb, np_dtype, virial=True):
    import torch
    from ai2pot_amd import ops
    dtype = torch.float32 if np_dtype == np.float32 else torch.float64
    md = _model_to_device(m, dtype)
    d = to_device(nb, dtype)
    fn = ops.nepToEFVOp if virial else ops.nepToEFOp
    out = fn(m["chebyshev_size"], m["n_radial_basis"], m["n_angular_basis"], m["l_max"], md["coeffs"],
             md["w0"], md["b0"], md["w1"], md["type_bias"], d["binum"], d["bilist"], d["bnumneigh"],
             d["bfirstneigh"], d["brcs"], d["btypes"], md["type_map"], d["nghost"], m["rmax_radial"],
             m["rmax_angular"], md["q_scaler"], 0.0, 0.0, None, None)
    torch.cuda.synchronize()
    return [o.cpu().numpy() for o in out]


def check(out, ref, np_dtype):
    e, f, v = out
    er, fr, vr = ref
    if np_dtype == np.float64:
        assert np.allclose(e, er, rtol=1e-10, atol=0)
        assert np.abs(f - fr).max() <= 1e-10 * max(np.abs(fr).max(), 1e-30)
        assert np.abs(v - vr).max() <= 1e-10 * max(np.abs(vr).max(), 1e-30)
    else:
        assert np.allclose(e, er, rtol=1e-5, atol=0)
        assert np.all(np.abs(f - fr) <= 1e-4 + 1e-5 * np.abs(fr))
        assert np.abs(v - vr).max() <= 1e-5 * np.abs(vr).max()


def small_structure(oracle, n=300, box=(18.0, 19.0, 20.0), ntypes=3, seed=11, dtype=np.float64,
                    rcut=7.0, umax=200, sort=False):
    lat, pos = synth.random_packed(n, list(box), 2.2, seed)
    types = synth.rng_randint(seed + 1, n, ntypes)
    return oracle.nblist(lat.astype(dtype), types, pos.astype(dtype), rcut, umax, sort=sort)


@pytest.mark.parametrize("np_dtype", [np.float64, np.float32])
def test_mos2_known_answer(oracle, np_dtype):
    """Set-up of the reference's own unit test (tests/test_nep.cc:100-255): l_max = 3,
    30 neurons, sorted list, umax 20.  Known answer E = 46.363417549065026."""
    lat, types, frac = synth.mos2_fixture()
    out = oracle.nblist(lat.astype(np_dtype), types, frac.astype(np_dtype), 5.0, 20, is_cart=False, sort=True)
    nb = synth.pack_batch([out])
    m = synth.nep_model_closed_form()
    e, f, v = run_gpu(m, nb, np_dtype)
    tol = 1e-10 if np_dtype == np.float64 else 1e-5
    assert abs(e[0] - 46.363417549065026) <= tol * 46.4
    check((e, f, v), oracle.nep_efv(m, nb, np_dtype), np_dtype)


@pytest.mark.parametrize("np_dtype", [np.float64, np.float32])
def test_random_cell_fast_path(oracle, np_dtype):
    nb = synth.pack_batch([small_structure(oracle, dtype=np_dtype)])
    m = synth.nep_model()
    check(run_gpu(m, nb, np_dtype), oracle.nep_efv(m, nb, np_dtype), np_dtype)
    # energy + force operator gives the same E and F
    e2, f2 = run_gpu(m, nb, np_dtype, virial=False)
    er, fr, _ = oracle.nep_efv(m, nb, np_dtype)
    check((e2, f2, np.ones(9)), (er, fr, np.ones(9)), np_dtype)


def test_batch_padding_permuted_ilist(oracle):
    """Three structures of different size in one padded batch, rows listed in a permuted
    order through ilist (row ii describes atom ilist[ii])."""
    a = small_structure(oracle, 120, (14.0, 15.0, 13.0), seed=31)
    b = small_structure(oracle, 200, (17.0, 15.0, 16.0), seed=32)
    c = small_structure(oracle, 37, (11.0, 15.0, 9.0), seed=33)
    nb = synth.pack_batch([a, b, c])
    rng = np.random.default_rng(5)
    for s, inum in enumerate(nb["binum"]):
        perm = rng.permutation(inum)
        for key in ("bnumneigh", "bfirstneigh", "brcs"):
            nb[key][s, :inum] = nb[key][s, perm]
        nb["bilist"][s, :inum] = perm
    m = synth.nep_model()
    check(run_gpu(m, nb, np.float64), oracle.nep_efv(m, nb, np.float64), np.float64)
    check(run_gpu(m, nb, np.float32), oracle.nep_efv(m, nb, np.float32), np.float32)


@pytest.mark.parametrize("reps", [4, 21])
def test_angular_cutoff_beyond_radial(oracle, reps):
    """A neighbour beyond the radial cutoff is skipped altogether, also when it lies inside a larger
    angular cutoff (nepBasis.h:106, 135).  256 atoms take the kernel with 8 lanes per atom, 37044
    atoms the one with a thread per atom."""
    lat, pos = synth.fcc_cell(reps, 4.6, 0.15, 61)
    ty = synth.rng_randint(62, pos.shape[0], 3)
    nb = synth.pack_batch([oracle.nblist(lat, ty, pos, 6.0, 100)])
    m = synth.nep_model(rmax_radial=4.5, rmax_angular=5.5)
    for dt in (np.float64, np.float32):
        nbt = dict(nb, brcs=nb["brcs"].astype(dt))
        check(run_gpu(m, nbt, dt), oracle.nep_efv(m, nbt, dt), dt)


@pytest.mark.parametrize("reps", [4, 21])
def test_reference_default_model(oracle, reps):
    """The hyperparameters ai2pot/models/nep/nep.py:32-46 defaults to (n_radial_basis 4, 30 neurons)
    take the same fast kernels as the benchmark model (n_radial_basis 6): 256 atoms the one with
    8 lanes per atom, 37044 atoms the staging + model pair."""
    lat, pos = synth.fcc_cell(reps, 4.6, 0.15, 63)
    ty = synth.rng_randint(64, pos.shape[0], 2)
    nb = synth.pack_batch([oracle.nblist(lat, ty, pos, 6.0, 100)])
    m = synth.nep_model(ntypes=2, n_radial_basis=4, num_neurons=30, rmax_radial=6.0, rmax_angular=4.0,
                        seed=3063, type_map=(14, 8))
    for dt in (np.float64, np.float32):
        nbt = dict(nb, brcs=nb["brcs"].astype(dt))
        check(run_gpu(m, nbt, dt), oracle.nep_efv(m, nbt, dt), dt)


def test_ghost_atoms(oracle):
    """The LAMMPS contract: neighbour indices point into [0, P + nghost); ghosts have a type
    and receive forces but own no row (interface/lammps/AI2POT/pair_ai2pot.cpp:175-249)."""
    full = small_structure(oracle, 150, (15.0, 15.0, 14.0), seed=41)
    inum, ilist, numneigh, firstneigh, rcs, types, _ = full
    nlocal = 100                       # atoms >= nlocal become ghosts of a smaller "rank"
    nb = dict(binum=np.array([nlocal], np.int32), bilist=ilist[None, :nlocal].copy(),
              bnumneigh=numneigh[None, :nlocal].copy(), bfirstneigh=firstneigh[None, :nlocal].copy(),
              brcs=rcs[None, :nlocal].copy(), btypes=types[None, :].copy(), nghost=inum - nlocal)
    nb["bfirstneigh"][nb["bfirstneigh"] < 0] = 0
    m = synth.nep_model()
    out = run_gpu(m, nb, np.float64)
    assert out[1].shape == (1, inum, 3)
    check(out, oracle.nep_efv(m, nb, np.float64), np.float64)


@pytest.mark.parametrize("cfg", [dict(K=10, n_r=7, n_a=5, l_max=2, H=17, ntypes=2),
                                 dict(K=6, n_r=4, n_a=3, l_max=0, H=8, ntypes=1),
                                 dict(K=14, n_r=10, n_a=7, l_max=4, H=5, ntypes=2),
                                 dict(K=8, n_r=6, n_a=4, l_max=4, H=200, ntypes=4)])
def test_general_shapes(oracle, cfg):
    """Sizes that do not hit the compile-time fast path, including l_max = 0 (radial only,
    nep_utilities.h:43-44) and a network too large for LDS."""
    nb = synth.pack_batch([small_structure(oracle, 90, (12.0, 13.0, 12.5), ntypes=cfg["ntypes"], seed=51,
                                           rcut=6.0)])
    m = synth.nep_model(ntypes=cfg["ntypes"], n_radial_basis=cfg["n_r"], n_angular_basis=cfg["n_a"],
                        l_max=cfg["l_max"], chebyshev_size=cfg["K"], num_neurons=cfg["H"],
                        rmax_radial=6.0, rmax_angular=4.5, seed=77, type_map=(1, 2, 3, 4))
    if cfg["l_max"] == 0:
        D = cfg["n_r"]
        m["w0"] = m["w0"][:cfg["ntypes"] * cfg["H"] * D]
        m["q_scaler"] = np.linspace(0.5, 1.5, D)
    else:
        m["q_scaler"] = np.linspace(0.5, 1.5, m["q_scaler"].size)
    check(run_gpu(m, nb, np.float64), oracle.nep_efv(m, nb, np.float64), np.float64)


def test_descriptors(oracle):
    import torch
    from ai2pot_amd import ops
    nb = synth.pack_batch([small_structure(oracle, 80, (12.0, 13.0, 12.5), seed=61)])
    m = synth.nep_model()
    md = _model_to_device(m, torch.float64)
    d = to_device(nb, torch.float64)
    out = ops.nepToDescriptorsOp(8, 6, 4, 4, md["coeffs"], d["binum"], d["bilist"], d["bnumneigh"],
                                 d["bfirstneigh"], d["brcs"], d["btypes"], md["type_map"], 0, 7.0, 4.0)
    ref = oracle.nep_descriptors(m, nb, np.float64)
    assert np.abs(out[0].cpu().numpy() - ref).max() <= 1e-10 * np.abs(ref).max()


def test_config2_full_size(oracle):
    """Benchmark configuration 2 at full size: 4096 atoms, 3 species, fp32, list cutoff 7 A."""
    lat, pos = synth.random_packed(4096, [49.8848] * 3, 2.2, 1003)
    types = synth.rng_randint(2003, 4096, 3)
    nb = synth.pack_batch([oracle.nblist(lat.astype(np.float32), types, pos.astype(np.float32), 7.0, 200)])
    m = synth.nep_model(seed=3003)
    out = run_gpu(m, nb, np.float32)
    check(out, oracle.nep_efv(m, nb, np.float32), np.float32)
    # size-independent properties: a symmetric full list gives zero net force and a
    # symmetric virial up to rounding
    f, v = out[1][0].astype(np.float64), out[2][0].reshape(3, 3)
    assert np.abs(f.sum(0)).max() < 1e-3
    assert np.abs(v - v.T).max() <= 2e-5 * np.abs(v).max()


def test_config5_full_size(oracle):
    """Benchmark configuration 5 at full size (1,048,576 atoms, list rebuilt and E/F/V on the device)
    through a size-independent property: the cell is a 16^3 block of 16,384 atoms repeated 4 x 4 x 4,
    so the energy and the virial are 64 times the block's and every replica carries the block's
    forces; the block itself is checked against the oracle.  Also: the list is symmetric (every atom
    is named as a neighbour as often as it has neighbours) and the net force vanishes."""
    import ctypes as c
    import torch
    from ai2pot_amd.calculator import NepCalculator
    # coordinates on a 2^-14 A grid: block and replicas are then exactly representable in fp32, every
    # relative vector of a replica equals the block's bit for bit, and so do the lists
    q = 2.0 ** -14
    a = np.round(316.7 / 64.0 / q) * q
    lat16, pos16 = synth.fcc_cell(16, a, 0.15, 1006)
    pos16 = np.mod(np.round(pos16 / q) * q, 16 * a)
    n16 = pos16.shape[0]
    ty16 = synth.rng_randint(2006, n16, 3)
    m = synth.nep_model(seed=3006)
    r = np.arange(4, dtype=np.float64)
    sx, sy, sz = np.meshgrid(r, r, r, indexing="ij")
    shifts = np.stack([sx.ravel(), sy.ravel(), sz.ravel()], axis=1) * (16 * a)
    pos = (shifts[:, None, :] + pos16[None, :, :]).reshape(-1, 3)
    types = np.tile(ty16, 64)
    n = pos.shape[0]
    assert n == 1048576
    calc = NepCalculator(m, n, lat16 * 4, types, umax=200, dtype=torch.float32, device="cuda:0")
    e, f, v = calc.step(torch.from_numpy(pos.astype(np.float32)).to("cuda:0"))
    torch.cuda.synchronize()
    calc.check()
    e, f, v = e.cpu().numpy().astype(np.float64), f.cpu().numpy(), v.cpu().numpy().astype(np.float64)
    ref = oracle.nblist(lat16.astype(np.float32), ty16, pos16.astype(np.float32), 7.0, 200)
    er, fr, vr = oracle.nep_efv(m, synth.pack_batch([ref]), np.float32)
    er, fr, vr = float(np.asarray(er).ravel()[0]), np.asarray(fr)[0], np.asarray(vr).reshape(9)
    assert abs(e[0] - 64 * er) <= 1e-5 * abs(64 * er)
    assert np.abs(v - 64 * vr).max() <= 1e-5 * np.abs(64 * vr).max()
    fb = f.reshape(64, n16, 3)
    assert np.all(np.abs(fb - fr[None]) <= 1e-4 + 1e-5 * np.abs(fr[None]))
    assert np.abs(f.astype(np.float64).sum(0)).max() < 0.05
    nn = calc.numneigh.cpu().numpy()
    assert np.array_equal(nn.reshape(64, n16), np.broadcast_to(np.asarray(ref[2])[None, :], (64, n16)))
    live = torch.arange(200, device="cuda:0", dtype=torch.int32)[None, :] < calc.numneigh[:, None]
    incoming = torch.bincount(calc.firstneigh[live].long(), minlength=n)
    assert torch.equal(incoming.int(), calc.numneigh)
    # first and last replica: the rows name the block's neighbours with the block's relative vectors
    # (as sets: the order within a row follows the bins, which differ between the two cells)
    ref_rows = np.asarray(ref[3]).reshape(n16, 200)
    ref_rcs = np.asarray(ref[4]).reshape(n16, 200, 3)
    want_order = np.lexsort((ref_rcs[..., 2], ref_rcs[..., 1], ref_rcs[..., 0], np.where(ref_rows >= 0, ref_rows, n16)), axis=1)
    for rep in (0, 63):
        rows = calc.firstneigh[rep * n16:(rep + 1) * n16].cpu().numpy()
        rcs = calc.rcs[rep * n16:(rep + 1) * n16].cpu().numpy()
        key = np.where(rows >= 0, rows % n16, n16)
        order = np.lexsort((rcs[..., 2], rcs[..., 1], rcs[..., 0], key), axis=1)
        assert np.array_equal(np.take_along_axis(key, order, 1),
                              np.take_along_axis(np.where(ref_rows >= 0, ref_rows, n16), want_order, 1))
        assert np.array_equal(np.take_along_axis(rcs, order[..., None], 1).view(np.uint32),
                              np.take_along_axis(ref_rcs, want_order[..., None], 1).view(np.uint32))


def test_reproducible(oracle):
    """Two runs give bit-identical forces (no floating-point atomics anywhere)."""
    nb = synth.pack_batch([small_structure(oracle, 300, dtype=np.float32)])
    m = synth.nep_model()
    a = run_gpu(m, nb, np.float32)
    b = run_gpu(m, nb, np.float32)
    for x, y in zip(a, b):
        assert np.array_equal(x.view(np.uint32), y.view(np.uint32))


def test_reproducible_staged_pair(oracle):
    """The same for a system large enough for the staging + model kernel pair (40,000 atoms)."""
    lat, pos = synth.fcc_cell(22, 4.6, 0.15, 67)
    ty = synth.rng_randint(68, pos.shape[0], 3)
    nb = synth.pack_batch([oracle.nblist(lat.astype(np.float32), ty, pos.astype(np.float32), 6.0, 100)])
    m = synth.nep_model(rmax_radial=6.0, rmax_angular=4.0)
    a = run_gpu(m, nb, np.float32)
    b = run_gpu(m, nb, np.float32)
    for x, y in zip(a, b):
        assert np.array_equal(x.view(np.uint32), y.view(np.uint32))


def test_ranked_call_equals_plain_call(oracle):
    """a2p_nep_efv_ranked_f32: the places of the pairs in the reduction segments are recorded by the
    first call on a list (or computed by a2p_pair_ranks) and used by the following calls instead of
    being claimed again; E, F and V are bit-identical to the plain call (40,000 atoms: the staging +
    model kernel pair, which is the path that uses ranks)."""
    import ctypes as c
    import torch
    from ai2pot_amd import _lib
    L = _lib.lib()
    lat, pos = synth.fcc_cell(22, 4.6, 0.15, 67)
    ty = synth.rng_randint(68, pos.shape[0], 3)
    nb = synth.pack_batch([oracle.nblist(lat.astype(np.float32), ty, pos.astype(np.float32), 6.0, 100)])
    m = synth.nep_model(rmax_radial=6.0, rmax_angular=4.0)
    plain = run_gpu(m, nb, np.float32)
    md = _model_to_device(m, torch.float32)
    d = to_device(nb, torch.float32)
    B, P, U = d["bfirstneigh"].shape
    dev = d["brcs"].device
    rank = torch.empty((B, P, U), dtype=torch.int32, device=dev)
    incoming = torch.empty((B, P), dtype=torch.int32, device=dev)
    vp = lambda t: c.c_void_p(t.data_ptr())
    stream = c.c_void_p(torch.cuda.current_stream().cuda_stream)
    _lib.check(L.a2p_pair_ranks(c.c_int(B), c.c_int(P), c.c_int(U), c.c_int(0), vp(d["binum"]),
                                vp(d["bnumneigh"]), vp(d["bfirstneigh"]), vp(rank), vp(incoming), stream))
    e = torch.empty(B, dtype=torch.float32, device=dev)
    f = torch.empty((B, P, 3), dtype=torch.float32, device=dev)
    v = torch.empty((B, 9), dtype=torch.float32, device=dev)
    H = md["w1"].numel() // 3

    def ranked(valid):
        _lib.check(L.a2p_nep_efv_ranked_f32(
            c.c_int(m["chebyshev_size"]), c.c_int(m["n_radial_basis"]), c.c_int(m["n_angular_basis"]),
            c.c_int(m["l_max"]), c.c_int(H), c.c_int(3), vp(md["coeffs"]), vp(md["w0"]), vp(md["b0"]),
            vp(md["w1"]), vp(md["type_bias"]), vp(md["q_scaler"]), c.c_double(m["rmax_radial"]),
            c.c_double(m["rmax_angular"]), c.c_int(B), c.c_int(P), c.c_int(U), c.c_int(0), vp(d["binum"]),
            vp(d["bilist"]), vp(d["bnumneigh"]), vp(d["bfirstneigh"]), vp(d["brcs"]), vp(d["btypes"]),
            vp(rank), vp(incoming), c.c_int(valid), vp(e), vp(f), vp(v), None, stream))
        torch.cuda.synchronize()
        _lib.check_status(torch.cuda.current_stream().cuda_stream)
        assert np.array_equal(e.cpu().numpy().view(np.uint32), plain[0].view(np.uint32))
        assert np.array_equal(f.cpu().numpy().view(np.uint32), plain[1].view(np.uint32))
        assert np.array_equal(v.cpu().numpy().view(np.uint32), plain[2].reshape(B, 9).view(np.uint32))

    ranked(1)                   # ranks from a2p_pair_ranks
    ranked(1)                   # ... serve any number of calls
    rank.fill_(-7)
    incoming.fill_(-7)
    ranked(0)                   # this call claims the places and records them
    live = np.arange(U)[None, None, :] < nb["bnumneigh"][:, :, None]
    assert rank.cpu().numpy()[live].min() >= 0 and np.array_equal(incoming.cpu().numpy(), nb["bnumneigh"])
    ranked(1)                   # ... for the following ones
    # every atom is named by as many pairs as it has neighbours (a full list is symmetric)
    assert np.array_equal(incoming.cpu().numpy(), nb["bnumneigh"])


@pytest.mark.parametrize("from_list", [False, True])
def test_calculator_kept_list(oracle, from_list):
    """NepCalculator: evaluations on a kept list (plain, recording the pairs' places, using them; or
    with the places the list build made) give the same bits, and a rebuild starts over."""
    import ctypes as c
    import torch
    from ai2pot_amd.calculator import NepCalculator
    lat, pos = synth.fcc_cell(22, 4.6, 0.15, 69)
    ty = synth.rng_randint(70, pos.shape[0], 3)
    m = synth.nep_model(rmax_radial=6.0, rmax_angular=4.0)
    calc = NepCalculator(m, pos.shape[0], lat, ty, umax=100, dtype=torch.float32, device="cuda:0",
                         places_from_list=from_list)
    coords = torch.from_numpy(pos.astype(np.float32)).to("cuda:0")
    stream = c.c_void_p(torch.cuda.current_stream().cuda_stream)
    outs = []
    for cycle in range(2):
        calc.rebuild(coords, stream)
        for _ in range(4):
            calc.evaluate(stream)
            torch.cuda.synchronize()
            outs.append((calc.etot.cpu().numpy().copy(), calc.force.cpu().numpy().copy(),
                         calc.virial.cpu().numpy().copy()))
    calc.check()
    for o in outs[1:]:
        for x, y in zip(outs[0], o):
            assert np.array_equal(x.view(np.uint32), y.view(np.uint32))
    ref = oracle.nblist(lat.astype(np.float32), ty, pos.astype(np.float32), 6.0, 100)
    er, fr, vr = oracle.nep_efv(m, synth.pack_batch([ref]), np.float32)
    check((outs[0][0], outs[0][1][None], outs[0][2][None]), (er, fr, vr.reshape(1, 9)), np.float32)


def test_errors(oracle):
    import torch
    from ai2pot_amd import ops, _lib
    nb = synth.pack_batch([small_structure(oracle, 60, (11.0, 11.0, 11.0), seed=71, umax=100)])
    m = synth.nep_model()
    md = _model_to_device(m, torch.float32)
    d = to_device(nb, torch.float32)

    def call(**over):
        a = dict(d)
        a.update(over)
        return ops.nepToEFVOp(8, 6, 4, 4, md["coeffs"], md["w0"], md["b0"], md["w1"], md["type_bias"],
                              a["binum"], a["bilist"], a["bnumneigh"], a["bfirstneigh"], a["brcs"],
                              a["btypes"], md["type_map"], 0, 7.0, 4.0, md["q_scaler"], 0.0, 0.0, None, None)

    call()
    with pytest.raises(RuntimeError):                       # wrong dtype
        call(brcs=d["brcs"].double())
    with pytest.raises(RuntimeError):                       # non-contiguous
        call(bfirstneigh=d["bfirstneigh"].transpose(1, 2).contiguous().transpose(1, 2))
    with pytest.raises(RuntimeError):                       # host tensor: no CPU path
        call(brcs=d["brcs"].cpu())
    with pytest.raises(RuntimeError):                       # neighbour count beyond the row
        call(bnumneigh=d["bnumneigh"] + 1000)
    bad = d["bfirstneigh"].clone()
    bad[0, 0, 0] = 10 ** 6
    with pytest.raises(_lib.A2PError):                      # neighbour index out of range
        call(bfirstneigh=bad)
    with pytest.raises(_lib.A2PError):                      # type index out of range
        call(btypes=d["btypes"] + 7)
    with pytest.raises(RuntimeError):                       # ZBL switched on without its parameter tensors
        ops.nepToEFVOp(8, 6, 4, 4, md["coeffs"], md["w0"], md["b0"], md["w1"], md["type_bias"],
                       d["binum"], d["bilist"], d["bnumneigh"], d["bfirstneigh"], d["brcs"], d["btypes"],
                       md["type_map"], 0, 7.0, 4.0, md["q_scaler"], 1.0, 0.5, None, None)
    call()                                                  # the library is still usable


def test_workspace_release(oracle):
    """a2p_workspace_bytes / a2p_workspace_release: the library holds scratch after a call, frees
    it on request, and the next call (which allocates again) returns the same bits."""
    import ctypes
    from ai2pot_amd import _lib
    L = _lib.lib()
    L.a2p_workspace_bytes.restype = ctypes.c_size_t
    m = synth.nep_model(seed=71)
    nb = synth.pack_batch([small_structure(oracle, dtype=np.float32)])
    first = run_gpu(m, nb, np.float32)
    held = L.a2p_workspace_bytes()
    assert held > 0
    _lib.check(L.a2p_workspace_release())
    assert L.a2p_workspace_bytes() == 0
    again = run_gpu(m, nb, np.float32)
    assert L.a2p_workspace_bytes() > 0
    for a, b in zip(first, again):
        assert np.array_equal(a, b)
