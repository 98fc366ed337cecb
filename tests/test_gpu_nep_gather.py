"""GPU parity of the device-resident step (compact neighbour lists + NEP E/F/V on them,
a2p_nblist_build_compact_* / a2p_nep_efv_compact_*) against the CPU oracle.

Bars as for the scatter path: fp64 within 1e-10 relative, fp32 energies and virials within 1e-5
relative, fp32 forces within 1e-4 eV/A absolute + 1e-5 relative; padded lists bit-exact; the compact
lists hold exactly the oracle's pairs with bit-identical relative vectors."""
import ctypes as c

import numpy as np
import pytest

from ai2pot_amd import synth

pytestmark = pytest.mark.gpu


def _check(out, ref, np_dtype):
    e, f, v = out
    er, fr, vr = ref
    er, fr, vr = np.asarray(er).ravel(), np.asarray(fr).reshape(-1, 3), np.asarray(vr).reshape(9)
    e, f, v = e.ravel(), f.reshape(-1, 3), v.reshape(9)
    if np_dtype == np.float64:
        assert np.allclose(e, er, rtol=1e-10, atol=0)
        assert np.abs(f - fr).max() <= 1e-10 * max(np.abs(fr).max(), 1e-30)
        assert np.abs(v - vr).max() <= 1e-10 * max(np.abs(vr).max(), 1e-30)
    else:
        assert np.allclose(e, er, rtol=1e-5, atol=0)
        assert np.all(np.abs(f - fr) <= 1e-4 + 1e-5 * np.abs(fr))
        assert np.abs(v - vr).max() <= 1e-5 * np.abs(vr).max()


def _calc(m, lat, ty, n, np_dtype, umax=200, **kw):
    import torch
    from ai2pot_amd.calculator import NepCalculator
    dtype = torch.float32 if np_dtype == np.float32 else torch.float64
    return NepCalculator(m, n, lat, ty, umax=umax, dtype=dtype, device="cuda:0", **kw)


def _step(calc, pos, np_dtype):
    import torch
    e, f, v = calc.step(torch.from_numpy(pos.astype(np_dtype)).to("cuda:0"))
    torch.cuda.synchronize()
    calc.check()
    return e.cpu().numpy().copy(), f.cpu().numpy().copy(), v.cpu().numpy().copy()


def _decode_compact(calc, np_dtype):
    """Host view of the compact buffer (layout of csrc/compact_list.h): per atom the set of
    (index, species, x, y, z) of the two classes."""
    n, U = calc.n, calc.umax
    elem = 4 if np_dtype == np.float32 else 8
    npad = (n + 63) // 64 * 64
    nch = U // 8
    raw = calc.compact.cpu().numpy()
    ints = raw[:3 * npad * 4].view(np.int32)
    order, n_outer, n_inner = ints[:npad], ints[npad:2 * npad], ints[2 * npad:3 * npad]
    off = (3 * npad * 4 + 255) // 256 * 256
    ent = raw[off:off + npad * U * 4 * elem].view(np_dtype).reshape(npad // 64, nch, 64, 8, 4)
    ent = ent.transpose(0, 2, 1, 3, 4).reshape(npad, U, 4)          # [position][slot][4]
    bits = ent[..., 3].copy().view(np.int32 if elem == 4 else np.int64).astype(np.int64)
    assert sorted(order[:n].tolist()) == list(range(n))             # a permutation of the atoms
    outer, inner = {}, {}
    for p in range(n):
        a = int(order[p])
        so = slice(0, n_outer[p])
        si = slice(U - n_inner[p], U)
        # an entry names its neighbour by position in the processing order
        pack = lambda s: sorted(zip(order[bits[p, s] & ((1 << 28) - 1)].tolist(), (bits[p, s] >> 28).tolist(),
                                    ent[p, s, 0].tolist(), ent[p, s, 1].tolist(), ent[p, s, 2].tolist()))
        outer[a], inner[a] = pack(so), pack(si)
    return outer, inner


@pytest.mark.parametrize("np_dtype", [np.float64, np.float32])
def test_random_cell_against_oracle(oracle, np_dtype):
    """Random packing, 3 species: padded lists bit-exact, compact lists = the oracle's pairs cut at the
    two cutoffs, E/F/V within the bars."""
    n = 350
    lat, pos = synth.random_packed(n, [20.0, 21.0, 22.0], 2.2, 311)
    ty = synth.rng_randint(312, n, 3)
    m = synth.nep_model(seed=3301)
    calc = _calc(m, lat, ty, n, np_dtype, path="gather")
    assert calc.path == "gather"
    out = _step(calc, pos, np_dtype)
    ref = oracle.nblist(lat.astype(np_dtype), ty, pos.astype(np_dtype), 7.0, 200)
    assert np.array_equal(calc.numneigh.cpu().numpy(), ref[2])
    assert np.array_equal(calc.firstneigh.cpu().numpy(), ref[3])
    u = np.uint32 if np_dtype == np.float32 else np.uint64
    assert np.array_equal(calc.rcs.cpu().numpy().view(u), ref[4].view(u))
    assert np.array_equal(calc.ilist.cpu().numpy(), np.arange(n)) and np.array_equal(calc.types_out.cpu().numpy(), ty)
    _check(out, oracle.nep_efv(m, synth.pack_batch([ref]), np_dtype), np_dtype)
    # compact lists against the oracle's rows
    outer, inner = _decode_compact(calc, np_dtype)
    rows, rcs, nn = np.asarray(ref[3]), np.asarray(ref[4]), np.asarray(ref[2])
    for a in range(n):
        r = np.sqrt((rcs[a, :nn[a]].astype(np_dtype) ** 2).sum(1))
        want_in = sorted((int(rows[a, s]), int(ty[rows[a, s]]), *rcs[a, s].tolist()) for s in range(nn[a]) if r[s] <= 4.0 - 1e-6)
        want_out = sorted((int(rows[a, s]), int(ty[rows[a, s]]), *rcs[a, s].tolist()) for s in range(nn[a]) if r[s] > 4.0 + 1e-6)
        border = sum(1 for s in range(nn[a]) if abs(r[s] - 4.0) <= 1e-6)
        assert len(inner[a]) + len(outer[a]) == nn[a]
        assert set(want_in) <= set(inner[a]) and set(want_out) <= set(outer[a])
        assert len(inner[a]) - len(want_in) + len(outer[a]) - len(want_out) == border


@pytest.mark.parametrize("np_dtype", [np.float64, np.float32])
def test_cell_smaller_than_cutoff(oracle, np_dtype):
    """A cell of 9 A with a 7 A cutoff: atoms meet their own images and the same neighbour through several
    images; the gather still pairs every entry with its mirror."""
    n = 24
    lat, pos = synth.random_packed(n, [9.0, 9.5, 10.0], 2.2, 321)
    lat = lat.copy()
    lat[1, 0] = 1.3                                       # triclinic
    ty = synth.rng_randint(322, n, 2)
    m = synth.nep_model(ntypes=2, seed=3302, type_map=(32, 51))
    calc = _calc(m, lat, ty, n, np_dtype, umax=200, path="gather")
    out = _step(calc, pos, np_dtype)
    ref = oracle.nblist(lat.astype(np_dtype), ty, pos.astype(np_dtype), 7.0, 200)
    assert np.array_equal(calc.firstneigh.cpu().numpy(), ref[3])
    _check(out, oracle.nep_efv(m, synth.pack_batch([ref]), np_dtype), np_dtype)


@pytest.mark.parametrize("cfg", [dict(ntypes=1, n_r=4, H=30), dict(ntypes=2, n_r=6, H=50), dict(ntypes=4, n_r=4, H=17),
                                 dict(ntypes=4, n_r=6, H=60)])
def test_model_shapes(oracle, cfg):
    """The shapes the gather kernels are instantiated for (n_radial 4 / 6, one to four species), fp64."""
    n = 160
    lat, pos = synth.random_packed(n, [15.0, 16.0, 17.0], 2.2, 331)
    ty = synth.rng_randint(332, n, cfg["ntypes"])
    m = synth.nep_model(ntypes=cfg["ntypes"], n_radial_basis=cfg["n_r"], num_neurons=cfg["H"], rmax_radial=6.0,
                        rmax_angular=4.5, seed=3303, type_map=tuple(range(30, 30 + cfg["ntypes"])))
    calc = _calc(m, lat, ty, n, np.float64, umax=160, path="gather")
    out = _step(calc, pos, np.float64)
    ref = oracle.nblist(lat, ty, pos, 6.0, 160)
    _check(out, oracle.nep_efv(m, synth.pack_batch([ref]), np.float64), np.float64)


@pytest.mark.parametrize("cfg", [dict(ntypes=3, n_r=6, H=50, n=700), dict(ntypes=1, n_r=4, H=30, n=300),
                                 dict(ntypes=4, n_r=6, H=64, n=521), dict(ntypes=2, n_r=4, H=7, n=130),
                                 dict(ntypes=3, n_r=6, H=100, n=200)])
def test_hidden_layer_on_the_matrix_cores(oracle, cfg):
    """a2p_nep_hidden_layer_unit(1): the per-species network of the workgroup's atoms as matrix products (fp32,
    species grouped in LDS, neuron counts that fill the 16-wide tiles unevenly, wavefronts with fewer than 64
    atoms, a scaled q_scaler; 100 neurons and four species stay on the vector ALUs).  Bars as for every fp32 result; the two units
    agree far inside them."""
    from ai2pot_amd import _lib
    n = cfg["n"]
    side = (n / 0.035) ** (1.0 / 3.0)
    lat, pos = synth.random_packed(n, [side, side * 1.05, side * 0.95], 2.2, 341)
    ty = synth.rng_randint(342, n, cfg["ntypes"])
    m = synth.nep_model(ntypes=cfg["ntypes"], n_radial_basis=cfg["n_r"], num_neurons=cfg["H"], seed=3304,
                        type_map=tuple(range(30, 30 + cfg["ntypes"])))
    D = cfg["n_r"] + 16
    m["q_scaler"] = 0.6 + 0.07 * np.arange(D)
    ref = oracle.nblist(lat.astype(np.float32), ty, pos.astype(np.float32), 7.0, 96)
    want = oracle.nep_efv(m, synth.pack_batch([ref]), np.float32)
    L = _lib.lib()
    before = L.a2p_nep_hidden_layer_unit(c.c_int(-1))
    outs = {}
    try:
        for unit in (1, 0):
            L.a2p_nep_hidden_layer_unit(c.c_int(unit))
            assert L.a2p_nep_hidden_layer_unit(c.c_int(-1)) == unit
            calc = _calc(m, lat, ty, n, np.float32, umax=96, path="gather")
            outs[unit] = _step(calc, pos, np.float32)
            _check(outs[unit], want, np.float32)
    finally:
        L.a2p_nep_hidden_layer_unit(c.c_int(before))
    assert np.abs(outs[0][1] - outs[1][1]).max() <= 2e-5 * max(1.0, np.abs(outs[0][1]).max())
    assert abs(outs[0][0][0] - outs[1][0][0]) <= 2e-6 * abs(outs[0][0][0])


@pytest.mark.parametrize("np_dtype", [np.float64, np.float32])
def test_more_pairs_inside_the_angular_cutoff_than_slots(oracle, np_dtype):
    """Equal cutoffs of 7 A at 0.04 atoms / A^3: every atom is named by about 57 pairs inside the angular cutoff,
    more than the 32 hand-over slots, so the rest reaches it through the spare rows (integer atomics in the fixed
    point of the slot sums): values against the oracle, and three evaluations bit for bit equal (which pair gets
    which place, and the order of the atomic additions, differ from run to run).  Also a structure whose atoms
    have no pair between the cutoffs at all."""
    n = 300
    lat, pos = synth.random_packed(n, [19.0, 20.0, 19.5], 2.0, 351)
    ty = synth.rng_randint(352, n, 3)
    m = synth.nep_model(rmax_radial=7.0, rmax_angular=7.0, seed=3305)
    calc = _calc(m, lat, ty, n, np_dtype, umax=136, path="gather")
    out = _step(calc, pos, np_dtype)
    ref = oracle.nblist(lat, ty, pos, 7.0, 136)
    assert ref[2].min() > 32 and ref[2].max() <= 136
    _check(out, oracle.nep_efv(m, synth.pack_batch([ref]), np_dtype), np_dtype)
    assert np.abs(out[1].astype(np.float64).sum(0)).max() < (1e-9 if np_dtype == np.float64 else 1e-2)
    for _ in range(2):
        again = _step(calc, pos, np_dtype)
        for x, y in zip(out, again):
            assert np.array_equal(np.ascontiguousarray(x).view(np.uint8), np.ascontiguousarray(y).view(np.uint8))
    # a smaller structure next, on the same workspace: the counters and spare rows it finds must be clean
    n2 = 120
    lat2, pos2 = synth.random_packed(n2, [14.5, 14.0, 15.0], 2.0, 353)
    ty2 = synth.rng_randint(354, n2, 3)
    calc2 = _calc(m, lat2, ty2, n2, np_dtype, umax=136, path="gather")
    out2 = _step(calc2, pos2, np_dtype)
    ref2 = oracle.nblist(lat2, ty2, pos2, 7.0, 136)
    _check(out2, oracle.nep_efv(m, synth.pack_batch([ref2]), np_dtype), np_dtype)


def test_atoms_processed_in_the_callers_order(oracle):
    """reorder_every=0: the processing order is the caller's (here a random one, the worst case for locality):
    same lists, same results within the bars, across rebuilds."""
    n = 500
    lat, pos = synth.random_packed(n, [23.0, 22.0, 24.0], 2.1, 361)
    ty = synth.rng_randint(362, n, 3)
    m = synth.nep_model(seed=3306)
    calc = _calc(m, lat, ty, n, np.float32, umax=96, path="gather", reorder_every=0)
    for k in range(3):
        p = pos + 0.02 * k * np.sin(np.arange(3 * n).reshape(n, 3))
        out = _step(calc, p, np.float32)
        ref = oracle.nblist(lat.astype(np.float32), ty, p.astype(np.float32), 7.0, 96)
        assert np.array_equal(calc.numneigh.cpu().numpy(), ref[2])
        assert np.array_equal(calc.firstneigh.cpu().numpy(), ref[3])
        assert np.array_equal(calc.compact[:4 * n].cpu().numpy().view(np.int32), np.arange(n))
        _check(out, oracle.nep_efv(m, synth.pack_batch([ref]), np.float32), np.float32)


@pytest.mark.parametrize("np_dtype", [np.float32, np.float64])
def test_pairs_across_the_cell_boundary_at_the_angular_cutoff(oracle, np_dtype):
    """A 300 A cell: 240 isolated pairs that reach across the periodic boundary at distances within a few
    roundings of the coordinates of the angular cutoff.  The two ends of such a pair see distance vectors that differ in the last bits
    (their images are rounded at the size of the coordinates), so each end alone could put the pair on a different
    side of the cutoff; the lists must put both entries in the same class, and the forces must match the oracle."""
    L, ra = 300.0, 4.0
    k = np.arange(240)
    ya = 10.0 + 18.0 * (k % 16)
    za = 10.0 + 18.0 * (k // 16)
    xa = 0.25 + 0.01 * (k % 7)
    delta = (k - 120) * (4.0e-6 if np_dtype == np.float32 else 8.0e-15)
    pos = np.zeros((480, 3))
    pos[0::2] = np.stack([xa, ya, za], 1)
    pos[1::2] = np.stack([L - (ra - xa) + delta, ya + 0.0, za + 0.0], 1)
    n = pos.shape[0]
    lat = np.diag([L, L, L]).astype(np.float64)
    ty = synth.rng_randint(372, n, 3)
    m = synth.nep_model(seed=3307)
    calc = _calc(m, lat, ty, n, np_dtype, umax=16, path="gather")
    out = _step(calc, pos, np_dtype)
    ref = oracle.nblist(lat.astype(np_dtype), ty, pos.astype(np_dtype), 7.0, 16)
    assert np.array_equal(calc.numneigh.cpu().numpy(), ref[2]) and ref[2].max() == 1
    outer, inner = _decode_compact(calc, np_dtype)
    n_in = sum(len(inner[a]) for a in range(n))
    assert 0 < n_in < n                                       # the pairs straddle the cutoff
    for a in range(n):
        for (j, _, _, _, _) in inner[a]:
            assert any(e[0] == a for e in inner[j]), (a, j)
        for (j, _, _, _, _) in outer[a]:
            assert any(e[0] == a for e in outer[j]), (a, j)
    _check(out, oracle.nep_efv(m, synth.pack_batch([ref]), np_dtype), np_dtype)
    assert np.abs(out[1].astype(np.float64).sum(0)).max() < (1e-4 if np_dtype == np.float32 else 1e-12)


def test_gather_equals_segments_and_is_reproducible(oracle):
    """fp32, 42,592 atoms (not a multiple of 256): the gather and the segment path agree within the fp32
    bars, each run of the gather gives the same bits, and skipping the padded arrays changes nothing."""
    lat, pos = synth.fcc_cell(22, 4.6, 0.15, 341)
    n = pos.shape[0]
    ty = synth.rng_randint(342, n, 3)
    m = synth.nep_model(rmax_radial=6.0, rmax_angular=4.0, seed=3304)
    a = _step(_calc(m, lat, ty, n, np.float32, umax=104, path="gather"), pos, np.float32)
    b = _step(_calc(m, lat, ty, n, np.float32, umax=104, path="gather"), pos, np.float32)
    s = _step(_calc(m, lat, ty, n, np.float32, umax=104, path="segments"), pos, np.float32)
    lean = _calc(m, lat, ty, n, np.float32, umax=104, path="gather", padded=False)
    assert lean.firstneigh is None
    d = _step(lean, pos, np.float32)
    for x, y, z in zip(a, b, d):
        assert np.array_equal(x.view(np.uint32), y.view(np.uint32))
        assert np.array_equal(x.view(np.uint32), z.view(np.uint32))
    assert np.allclose(a[0], s[0], rtol=2e-6)
    assert np.all(np.abs(a[1] - s[1]) <= 2e-4 + 2e-5 * np.abs(s[1]))
    assert np.abs(a[2] - s[2]).max() <= 2e-5 * np.abs(s[2]).max()
    assert np.abs(a[1].astype(np.float64).sum(0)).max() < 1e-2          # Newton's third law
    v = a[2].reshape(3, 3)
    assert np.abs(v - v.T).max() <= 2e-5 * np.abs(v).max()


def test_headline_size_properties_and_sampled_atoms(oracle):
    """The benchmark's configuration itself: 1,048,576 atoms (perturbed fcc, 3 species), fp32, umax 200.  The oracle
    would need minutes for the whole cell, so the whole-cell checks are properties: two runs give the same bits,
    the forces sum to zero, the virial is symmetric, and the segment path (another formulation: scatter into
    reduction segments from the padded rows) agrees within the fp32 bars.  Then the oracle itself on sampled atoms,
    among them those nearest to the faces of the cell: the rows of the atom and of all its neighbours, taken from
    the padded arrays of the step, form a small LAMMPS-style domain (the neighbours' other neighbours are ghosts),
    on which the oracle's force on the atom is complete."""
    import torch
    lat, pos = synth.fcc_cell(64, 316.7 / 64.0, 0.15, 1006)
    n = pos.shape[0]
    assert n == 1048576
    ty = synth.rng_randint(2006, n, 3)
    m = synth.nep_model(seed=3006)
    calc = _calc(m, lat, ty, n, np.float32, umax=200, path="gather")
    a = _step(calc, pos, np.float32)
    b = _step(calc, pos, np.float32)                        # rebuild in place, same coordinates
    for x, y in zip(a, b):
        assert np.array_equal(x.view(np.uint32), y.view(np.uint32))
    f64 = a[1].astype(np.float64)
    assert np.abs(f64.sum(0)).max() < 5e-2 and np.isfinite(f64).all()
    v = a[2].reshape(3, 3)
    assert np.abs(v - v.T).max() <= 2e-5 * np.abs(v).max()
    # sampled atoms against the oracle, from the rows of this step
    rng = np.random.RandomState(7)
    picks = set(int(i) for i in rng.randint(0, n, 6))
    for ax in range(3):
        picks.add(int(np.argmin(pos[:, ax])))
        picks.add(int(np.argmax(pos[:, ax])))
    U = calc.umax
    first_d, rcs_d, nn_d = calc.firstneigh.view(n, U), calc.rcs.view(n, U, 3), calc.numneigh
    for i in sorted(picks):
        ni = int(nn_d[i])
        local = [i] + sorted(set(first_d[i, :ni].cpu().numpy().tolist()) - {i})
        idx = torch.tensor(local, device="cuda:0", dtype=torch.long)
        nn = nn_d[idx].cpu().numpy()
        fn = first_d[idx].cpu().numpy()
        rc = rcs_d[idx].cpu().numpy().astype(np.float64)
        P = len(local)
        ids = {g: k for k, g in enumerate(local)}
        for r in range(P):
            for g in fn[r, :nn[r]].tolist():
                if g not in ids:
                    ids[g] = len(ids)
        firstm = np.zeros((P, U), np.int32)
        for r in range(P):
            firstm[r, :nn[r]] = [ids[g] for g in fn[r, :nn[r]].tolist()]
        glob = np.array(sorted(ids, key=ids.get))
        nb = dict(binum=np.array([P], np.int32), bilist=np.arange(P, dtype=np.int32)[None],
                  bnumneigh=nn.astype(np.int32)[None], bfirstneigh=firstm[None], brcs=rc[None],
                  btypes=ty[glob].astype(np.int32)[None], nghost=len(ids) - P)
        _, fr, _ = oracle.nep_efv(m, nb, np.float64)
        got, want = a[1][i].astype(np.float64), np.asarray(fr).reshape(-1, 3)[0]
        assert np.all(np.abs(got - want) <= 1e-4 + 1e-5 * np.abs(want)), (i, got, want)
    del calc
    torch.cuda.empty_cache()
    s = _step(_calc(m, lat, ty, n, np.float32, umax=200, path="segments"), pos, np.float32)
    assert np.allclose(a[0], s[0], rtol=2e-6)
    assert np.all(np.abs(a[1] - s[1]) <= 2e-4 + 2e-5 * np.abs(s[1]))
    assert np.abs(a[2] - s[2]).max() <= 2e-5 * np.abs(s[2]).max()


def test_rebuild_in_place(oracle):
    """Steps on moving coordinates reuse the calculator's buffers (rows updated in place, compact lists
    rewritten): every step equals a fresh calculator's."""
    lat, pos = synth.fcc_cell(8, 4.9, 0.15, 351)
    n = pos.shape[0]
    ty = synth.rng_randint(352, n, 3)
    m = synth.nep_model(seed=3305)
    disp = synth.rng_normal(353, pos.size, 0.0, 0.2).reshape(-1, 3)
    calc = _calc(m, lat, ty, n, np.float32, path="gather")
    for k in range(3):
        p = pos + disp * np.sin(1.3 * k)
        got = _step(calc, p, np.float32)
        want = _step(_calc(m, lat, ty, n, np.float32, path="gather"), p, np.float32)
        for x, y in zip(got, want):
            assert np.array_equal(x.view(np.uint32), y.view(np.uint32))
        ref = oracle.nblist(lat.astype(np.float32), ty, p.astype(np.float32), 7.0, 200)
        assert np.array_equal(calc.firstneigh.cpu().numpy(), ref[3])
        assert np.array_equal(calc.rcs.cpu().numpy().view(np.uint32), ref[4].view(np.uint32))
        _check(got, oracle.nep_efv(m, synth.pack_batch([ref]), np.float32), np.float32)


def test_gather_errors(oracle):
    import torch
    from ai2pot_amd import _lib
    from ai2pot_amd.calculator import NepCalculator
    lat, pos = synth.random_packed(100, [14.0, 14.0, 14.0], 2.2, 361)
    m = synth.nep_model(seed=3306)
    with pytest.raises(ValueError):                                   # model shape outside the gather kernels
        NepCalculator(synth.nep_model(l_max=3), 100, lat, np.zeros(100, np.int32), path="gather")
    with pytest.raises(ValueError):                                   # fp64 tables of 4 x 100 neurons exceed LDS
        NepCalculator(synth.nep_model(ntypes=4, num_neurons=100, type_map=(1, 2, 3, 4)), 100, lat, np.zeros(100, np.int32),
                      dtype=torch.float64, path="gather")
    with pytest.raises(ValueError):                                   # umax not a multiple of 8
        NepCalculator(m, 100, lat, np.zeros(100, np.int32), umax=100, path="gather")
    calc = _calc(m, lat, np.full(100, 5, np.int32), 100, np.float32, path="gather")   # species outside the model
    calc.step(torch.from_numpy(pos.astype(np.float32)).to("cuda:0"))
    with pytest.raises(_lib.A2PError):
        calc.check()
    L = _lib.lib()
    L.a2p_nblist_compact_bytes.restype = c.c_size_t
    assert L.a2p_nblist_compact_bytes(c.c_int(100), c.c_int(100), c.c_int(4)) == 0    # umax % 8 != 0
    assert L.a2p_nblist_compact_bytes(c.c_int(100), c.c_int(104), c.c_int(4)) == 3 * 128 * 4 + 128 * 104 * 16
    ok = _calc(m, lat, synth.rng_randint(362, 100, 3), 100, np.float32, umax=8, path="gather")   # rows overflow
    ok.step(torch.from_numpy(pos.astype(np.float32)).to("cuda:0"))
    with pytest.raises(_lib.A2PError):
        ok.check()


def test_order_written_by_the_caller_is_checked(oracle):
    """The processing order at the head of the compact buffer may be written by the caller.  An index outside the
    structure, or an atom named twice, is reported by the status check (the index is clamped where it is used,
    so no kernel touches memory outside the buffers); a valid order written afterwards works again."""
    import torch
    from ai2pot_amd import _lib
    n = 200
    lat, pos = synth.random_packed(n, [17.0, 16.0, 18.0], 2.2, 381)
    ty = synth.rng_randint(382, n, 3)
    m = synth.nep_model(seed=3308)
    x = torch.from_numpy(pos.astype(np.float32)).to("cuda:0")
    ref = oracle.nblist(lat.astype(np.float32), ty, pos.astype(np.float32), 7.0, 96)
    want = oracle.nep_efv(m, synth.pack_batch([ref]), np.float32)
    for bad in ([n + 5, 3], [-7, 3], [1 << 30, 3], [11, 11], None):
        calc = _calc(m, lat, ty, n, np.float32, umax=96, path="gather", reorder_every=0)
        order = calc.compact[:4 * n].view(torch.int32)
        if bad is not None:
            order[7] = bad[0]
            order[9] = bad[1]
        e, f, v = calc.step(x)
        torch.cuda.synchronize()
        if bad is None:
            calc.check()
            _check((e.cpu().numpy(), f.cpu().numpy(), v.cpu().numpy()), want, np.float32)
        else:
            with pytest.raises(_lib.A2PError):
                calc.check()


@pytest.mark.parametrize("np_dtype", [np.float32, np.float64])
def test_trajectory_across_reorders_without_host_synchronisation(oracle, np_dtype):
    """Seven steps of drifting atoms in a slab (one axis not periodic): the processing order is refreshed every third
    rebuild and kept in between, the rebuilds after the first do not synchronise with the host.  Every step's padded
    rows are the oracle's bit for bit and E/F/V stay within the bars."""
    import torch
    from ai2pot_amd.calculator import NepCalculator
    lat, pos = synth.fcc_cell(7, 4.7, 0.12, 371)
    n = pos.shape[0]
    ty = synth.rng_randint(372, n, 3)
    m = synth.nep_model(rmax_radial=6.0, rmax_angular=4.0, seed=3307)
    disp = synth.rng_normal(373, pos.size, 0.0, 0.05).reshape(-1, 3)
    dtype = torch.float32 if np_dtype == np.float32 else torch.float64
    calc = NepCalculator(m, n, lat, ty, umax=96, dtype=dtype, device="cuda:0", path="gather", pbc=(True, True, False),
                         reorder_every=3, sync_free=True)
    for k in range(7):
        p = pos + k * disp
        got = _step(calc, p, np_dtype)
        ref = oracle.nblist(lat.astype(np_dtype), ty, p.astype(np_dtype), 6.0, 96, pbc=(True, True, False))
        nn = ref[2]
        assert np.array_equal(calc.numneigh.cpu().numpy(), nn)
        fn, rc = calc.firstneigh.cpu().numpy(), calc.rcs.cpu().numpy()
        for i in range(0, n, 11):
            assert np.array_equal(fn[i, :nn[i]], ref[3][i, :nn[i]]), (k, i)
            assert np.array_equal(rc[i, :nn[i]].view(np.uint8), ref[4][i, :nn[i]].view(np.uint8)), (k, i)
            assert (fn[i, nn[i]:] == -1).all() and not rc[i, nn[i]:].any()
        _check(got, oracle.nep_efv(m, synth.pack_batch([ref]), np_dtype), np_dtype)
