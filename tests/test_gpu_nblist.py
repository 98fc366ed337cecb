"""GPU neighbour list against the CPU oracle: numneigh, firstneigh bit-exact and rcs bitwise
identical in the same precision, in both sort modes (the sorted mode includes the tie order
of libstdc++'s std::sort, which perfect lattices exercise heavily)."""
import numpy as np
import pytest

from ai2pot_amd import synth

pytestmark = pytest.mark.gpu


def gpu_list(lattice, types, coords, rcut, umax, is_cart=True, pbc=(True, True, True), sort=False):
    from ai2pot_amd import nblist
    return nblist.find_info4mlff(np.ascontiguousarray(lattice), np.ascontiguousarray(types),
                                 np.ascontiguousarray(coords), float(rcut), int(umax), bool(is_cart),
                                 [bool(x) for x in pbc], bool(sort))


def assert_same(a, b):
    assert a[0] == b[0] and a[6] == b[6]
    names = ("inum", "ilist", "numneigh", "firstneigh", "rcs", "types")
    for i in (1, 2, 5):
        assert np.array_equal(a[i], b[i]), names[i]
    bad = np.nonzero((a[3] != b[3]).any(axis=1))[0]
    assert bad.size == 0, "firstneigh differs in rows %s" % bad[:10]
    assert a[4].dtype == b[4].dtype
    assert np.array_equal(a[4].view(np.uint8), b[4].view(np.uint8)), "rcs not bitwise identical"


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("sort", [False, True])
@pytest.mark.parametrize("rcut", [3.2, 5.0, 7.0])
def test_mos2(oracle, dt, sort, rcut):
    lat, types, frac = synth.mos2_fixture()
    a = gpu_list(lat.astype(dt), types, frac.astype(dt), rcut, 200, is_cart=False, sort=sort)
    b = oracle.nblist(lat.astype(dt), types, frac.astype(dt), rcut, 200, is_cart=False, sort=sort)
    assert_same(a, b)
    if rcut == 3.2:     # the reference's own assertion, source/nblist/tests/test_neighborList.cc:244
        assert a[2].max() == 12


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("sort", [False, True])
@pytest.mark.parametrize("pbc", [(True, True, True), (True, False, True), (False, False, False)])
def test_triclinic(oracle, dt, sort, pbc):
    L = np.array([[9.0, 0.3, -0.2], [1.1, 8.2, 0.4], [-0.7, 0.9, 10.1]])
    fr = synth.rng_uniform(7, 3 * 60).reshape(60, 3)
    ty = synth.rng_randint(8, 60, 3)
    a = gpu_list(L.astype(dt), ty, fr.astype(dt), 5.5, 250, is_cart=False, pbc=pbc, sort=sort)
    b = oracle.nblist(L.astype(dt), ty, fr.astype(dt), 5.5, 250, is_cart=False, pbc=pbc, sort=sort)
    assert_same(a, b)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_unwrapped_coordinates_small_cell(oracle, dt):
    """Atoms outside the cell (the reference never wraps) and a cell smaller than the cutoff,
    so several images of the same atom are neighbours."""
    L = np.array([[4.1, 0.0, 0.0], [0.5, 3.9, 0.0], [0.2, -0.3, 4.4]])
    fr = synth.rng_uniform(17, 3 * 7).reshape(7, 3) * 3.0 - 1.0
    ty = synth.rng_randint(18, 7, 2).astype(np.int64)      # int64 types are accepted
    a = gpu_list(L.astype(dt), ty, fr.astype(dt), 6.0, 400, is_cart=False, sort=True)
    b = oracle.nblist(L.astype(dt), ty, fr.astype(dt), 6.0, 400, is_cart=False, sort=True)
    assert_same(a, b)
    assert a[5].dtype == np.int32


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("umax", [56, 54, 2000])
def test_row_capacities(oracle, dt, umax):
    """Capacities that take the LDS row buffer (multiple of 4, small), the direct stores (not a
    multiple of 4) and a row too large for the buffer."""
    lat, pos = synth.random_packed(200, [14.0, 15.0, 16.0], 2.2, 91)
    types = synth.rng_randint(92, 200, 2)
    a = gpu_list(lat.astype(dt), types, pos.astype(dt), 5.0, umax)
    b = oracle.nblist(lat.astype(dt), types, pos.astype(dt), 5.0, umax)
    assert_same(a, b)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("umax,sort", [(56, False), (54, False), (2000, False), (56, True)])
def test_update_in_place(oracle, dt, umax, sort):
    """a2p_nblist_update_* into buffers that hold an earlier list: after every step the whole
    arrays, padding included, are those of a fresh build.  The atoms move far enough between the
    steps for rows to grow and to shrink; the three capacities take the LDS row buffer, the
    direct stores and the rows too large for the buffer; the sorted list is rebuilt in full."""
    import ctypes as c
    import torch
    from ai2pot_amd import _lib
    L = _lib.lib()
    f32 = dt == np.float32
    build = L.a2p_nblist_build_f32 if f32 else L.a2p_nblist_build_f64
    update = L.a2p_nblist_update_f32 if f32 else L.a2p_nblist_update_f64
    n = 200
    lat, pos = synth.random_packed(n, [14.0, 15.0, 16.0], 2.2, 91)
    types = synth.rng_randint(92, n, 2)
    dev = "cuda:0"
    tdt = torch.float32 if f32 else torch.float64
    i32 = dict(dtype=torch.int32, device=dev)
    t_types = torch.from_numpy(types.astype(np.int32)).to(dev)
    ilist, numneigh, types_out = torch.empty(n, **i32), torch.empty(n, **i32), torch.empty(n, **i32)
    first = torch.empty((n, umax), **i32)
    rcs = torch.empty((n, umax, 3), dtype=tdt, device=dev)
    lat_h = np.ascontiguousarray(lat, dt).reshape(9)
    pbc = np.ones(3, np.int32)
    vp = lambda t: c.c_void_p(t.data_ptr())
    lengths = []
    for step in range(4):
        p = (pos + synth.rng_normal(300 + step, pos.size, 0.0, 0.35 * step).reshape(-1, 3)).astype(dt)
        coords = torch.from_numpy(p).to(dev)
        fn = build if step == 0 else update
        rc = fn(lat_h.ctypes.data_as(c.c_void_p), vp(t_types), vp(coords), c.c_int(n), c.c_double(5.0),
                c.c_int(umax), c.c_int(1), pbc.ctypes.data_as(c.c_void_p), c.c_int(1 if sort else 0), vp(ilist),
                vp(numneigh), vp(first), vp(rcs), vp(types_out), None,
                c.c_void_p(torch.cuda.current_stream().cuda_stream))
        _lib.check(rc)
        torch.cuda.synchronize()
        _lib.check_status(torch.cuda.current_stream().cuda_stream)
        b = oracle.nblist(lat.astype(dt), types, p, 5.0, umax, sort=sort)
        a = (n, ilist.cpu().numpy(), numneigh.cpu().numpy(), first.cpu().numpy(), rcs.cpu().numpy(),
             types_out.cpu().numpy(), 0)
        assert_same(a, b)
        lengths.append(a[2].copy())
    grew = sum(int((lengths[k + 1] > lengths[k]).sum()) for k in range(3))
    shrank = sum(int((lengths[k + 1] < lengths[k]).sum()) for k in range(3))
    assert grew > 20 and shrank > 20        # the sequence exercises both directions


@pytest.mark.parametrize("sort", [False, True])
def test_config2_size(oracle, sort):
    lat, pos = synth.random_packed(4096, [49.8848] * 3, 2.2, 1003)
    types = synth.rng_randint(2003, 4096, 3)
    a = gpu_list(lat.astype(np.float32), types, pos.astype(np.float32), 7.0, 200, sort=sort)
    b = oracle.nblist(lat.astype(np.float32), types, pos.astype(np.float32), 7.0, 200, sort=sort)
    assert_same(a, b)


def test_fcc_lattice_ties(oracle):
    """A perfect FCC crystal: every shell is a set of exactly tied distances."""
    lat, pos = synth.fcc_cell(6, 4.949, 0.0, 1)
    types = synth.rng_randint(3, pos.shape[0], 3)
    for dt in (np.float32, np.float64):
        a = gpu_list(lat.astype(dt), types, pos.astype(dt), 7.0, 200, sort=True)
        b = oracle.nblist(lat.astype(dt), types, pos.astype(dt), 7.0, 200, sort=True)
        assert_same(a, b)


def test_config5_recipe_reduced(oracle):
    """Configuration 5's recipe (jittered FCC, 0.033 atoms/A^3, rcut 7) at 32^3 x 4 atoms."""
    lat, pos = synth.fcc_cell(32, 316.7 / 64, 0.15, 1006)
    types = synth.rng_randint(2006, pos.shape[0], 3)
    a = gpu_list(lat.astype(np.float32), types, pos.astype(np.float32), 7.0, 200)
    b = oracle.nblist(lat.astype(np.float32), types, pos.astype(np.float32), 7.0, 200)
    assert_same(a, b)
    # symmetry of a full list: j in N(i) <=> i in N(j), as a checksum of pair counts
    inum, _, numneigh, first, rcs, _, _ = a
    assert numneigh.sum() % 2 == 0
    counts = np.bincount(first[first >= 0], minlength=inum)
    assert np.array_equal(counts, numneigh)


def test_config5_full_size_bit_exact(oracle):
    """The benchmark's own structure (1,048,576 atoms, L = 316.7 A, fp32, umax 200, unsorted) against the oracle on
    the host, every row: numneigh, firstneigh with its order, rcs bit for bit, the -1 / 0 padding included -- through
    the NumPy entry point (a fresh build) and through the device-resident step the benchmark times (compact build
    with padded rows, processing order along the space-filling curve; an in-place rebuild on top of the first)."""
    import torch
    from ai2pot_amd.calculator import NepCalculator
    lat, pos = synth.fcc_cell(64, 316.7 / 64.0, 0.15, 1006)
    n = pos.shape[0]
    assert n == 1048576
    types = synth.rng_randint(2006, n, 3)
    lat32, pos32 = lat.astype(np.float32), pos.astype(np.float32)
    b = oracle.nblist(lat32, types, pos32, 7.0, 200)
    a = gpu_list(lat32, types, pos32, 7.0, 200)
    assert_same(a, b)
    del a
    calc = NepCalculator(synth.nep_model(seed=3006), n, lat, types, umax=200, dtype=torch.float32, device="cuda:0",
                         path="gather")
    x = torch.from_numpy(pos32).to("cuda:0")
    calc.firstneigh.fill_(-7)
    calc.rcs.fill_(float("nan"))
    for build in range(2):                  # a build into buffers full of garbage, then a rebuild in place
        calc.step(x)
        torch.cuda.synchronize()
        calc.check()
        assert np.array_equal(calc.numneigh.cpu().numpy(), b[2])
        first = calc.firstneigh.cpu().numpy()
        bad = np.nonzero((first != b[3]).any(axis=1))[0]
        assert bad.size == 0, "build %d: firstneigh (order, padding) differs in rows %s" % (build, bad[:10])
        del first
        assert np.array_equal(calc.rcs.cpu().numpy().view(np.uint32), b[4].view(np.uint32)), "rcs not bitwise identical"
        assert np.array_equal(calc.ilist.cpu().numpy(), b[1]) and np.array_equal(calc.types_out.cpu().numpy(), b[5])


def test_overflow_and_type_errors(oracle):
    lat, types, frac = synth.mos2_fixture()
    with pytest.raises(RuntimeError):
        gpu_list(lat, types, frac, 7.0, 20, is_cart=False)      # 54 neighbours > umax 20
    from ai2pot_amd import nblist
    with pytest.raises(TypeError):
        nblist.find_info4mlff(lat, types, frac, 5, 20, False, [True] * 3, False)       # rcut not float
    with pytest.raises(TypeError):
        nblist.find_info4mlff(lat, types, frac, 5.0, 20, False, (True, True, True), False)  # pbc not list
    with pytest.raises(TypeError):
        nblist.find_info4mlff(lat.tolist(), types, frac, 5.0, 20, False, [True] * 3, False)
    a = gpu_list(lat, types, frac, 5.0, 20, is_cart=False, sort=True)               # still usable
    assert_same(a, oracle.nblist(lat, types, frac, 5.0, 20, is_cart=False, sort=True))


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("umax", [56, 54, 2000])
def test_build_with_places(oracle, dt, umax):
    """a2p_nblist_build_ranked_*: the list is the unsorted build's bit for bit (first call fresh,
    later calls into the kept buffers); the places of the pairs that name one neighbour are a
    permutation of 0 .. incoming - 1 and incoming is the histogram of the neighbour column."""
    import ctypes as c
    import torch
    from ai2pot_amd import _lib
    L = _lib.lib()
    f32 = dt == np.float32
    fn = L.a2p_nblist_build_ranked_f32 if f32 else L.a2p_nblist_build_ranked_f64
    n = 200
    lat, pos = synth.random_packed(n, [14.0, 15.0, 16.0], 2.2, 93)
    types = synth.rng_randint(94, n, 2)
    dev = "cuda:0"
    tdt = torch.float32 if f32 else torch.float64
    i32 = dict(dtype=torch.int32, device=dev)
    t_types = torch.from_numpy(types.astype(np.int32)).to(dev)
    ilist, numneigh, types_out = torch.empty(n, **i32), torch.empty(n, **i32), torch.empty(n, **i32)
    first = torch.empty((n, umax), **i32)
    rcs = torch.empty((n, umax, 3), dtype=tdt, device=dev)
    rank = torch.full((n, umax), -7, **i32)
    incoming = torch.full((n,), -7, **i32)
    lat_h = np.ascontiguousarray(lat, dt).reshape(9)
    pbc = np.ones(3, np.int32)
    vp = lambda t: c.c_void_p(t.data_ptr())
    for step in range(3):
        p = (pos + synth.rng_normal(310 + step, pos.size, 0.0, 0.35 * step).reshape(-1, 3)).astype(dt)
        coords = torch.from_numpy(p).to(dev)
        rc = fn(lat_h.ctypes.data_as(c.c_void_p), vp(t_types), vp(coords), c.c_int(n), c.c_double(5.0),
                c.c_int(umax), c.c_int(1), pbc.ctypes.data_as(c.c_void_p), c.c_int(0 if step == 0 else 1),
                vp(ilist), vp(numneigh), vp(first), vp(rcs), vp(types_out), vp(rank), vp(incoming), None,
                c.c_void_p(torch.cuda.current_stream().cuda_stream))
        _lib.check(rc)
        torch.cuda.synchronize()
        _lib.check_status(torch.cuda.current_stream().cuda_stream)
        b = oracle.nblist(lat.astype(dt), types, p, 5.0, umax, sort=False)
        nn, fi = numneigh.cpu().numpy(), first.cpu().numpy()
        assert_same((n, ilist.cpu().numpy(), nn, fi, rcs.cpu().numpy(), types_out.cpu().numpy(), 0), b)
        rk, inc = rank.cpu().numpy(), incoming.cpu().numpy()
        live = np.arange(umax)[None, :] < nn[:, None]
        assert np.array_equal(inc, np.bincount(fi[live], minlength=n))
        seen = np.zeros((n, int(inc.max()) + 1), np.int32)
        assert rk[live].min() >= 0 and np.all(rk[live] < inc[fi[live]])
        np.add.at(seen, (fi[live], rk[live]), 1)
        assert np.array_equal(seen.sum(1), inc) and seen.max() == 1



@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("sort", [False, True])
@pytest.mark.parametrize("pbc", [(True, True, True), (True, False, True)])
def test_builds_without_host_synchronisation(oracle, dt, sort, pbc):
    """a2p_nblist_sync_free: after one synchronised build of a structure, later builds derive the bin grid on the
    device.  Triclinic cell, fractional coordinates, atoms drifting (also out of the cell): every build is
    bitwise the oracle's, through the C ABI (NumPy front end) and through torch.ops.nblist on device tensors."""
    import os
    import torch
    from ai2pot_amd import _lib
    L = np.array([[9.0, 0.3, -0.2], [1.1, 8.2, 0.4], [-0.7, 0.9, 10.1]])
    fr = synth.rng_uniform(27, 3 * 80).reshape(80, 3)
    ty = synth.rng_randint(28, 80, 3)
    drift = synth.rng_normal(29, 3 * 80, 0.0, 0.01).reshape(80, 3)
    lib = _lib.lib()
    a = gpu_list(L.astype(dt), ty, fr.astype(dt), 5.5, 250, is_cart=False, pbc=pbc, sort=sort)   # sets the bound
    assert_same(a, oracle.nblist(L.astype(dt), ty, fr.astype(dt), 5.5, 250, is_cart=False, pbc=pbc, sort=sort))
    from ai2pot_amd import nblist
    tt0 = torch.from_numpy(ty.astype(np.int32)).to("cuda:0")
    before = lib.a2p_nblist_sync_free(1)
    try:
        for step in range(1, 4):
            f = (fr + step * drift).astype(dt)
            # check=False: a build that asks for the largest neighbour count synchronises anyway
            out = nblist.find_info4mlff_device(L.astype(dt), tt0, torch.from_numpy(f).to("cuda:0"), 5.5, 250, False,
                                               pbc, sort, check=False)
            _lib.check_status(torch.cuda.current_stream().cuda_stream)
            got = tuple(o.cpu().numpy() if hasattr(o, "cpu") else o for o in out)
            assert_same(got, oracle.nblist(L.astype(dt), ty, f, 5.5, 250, is_cart=False, pbc=pbc, sort=sort))
    finally:
        lib.a2p_nblist_sync_free(before)
    # the same through the registered operator
    libdir = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "ai2pot_amd", "_lib")
    torch.ops.load_library(os.path.join(libdir, "libnblist_bind.so"))
    tl = torch.from_numpy(L.astype(dt))
    tt = torch.from_numpy(ty.astype(np.int32)).to("cuda:0")
    args = (5.5, 250, False, [bool(x) for x in pbc], sort)
    torch.ops.nblist.find_info4mlff(tl, tt, torch.from_numpy(fr.astype(dt)).to("cuda:0"), *args)
    was = torch.ops.nblist.set_sync_free(True)
    try:
        f = (fr + 2.5 * drift).astype(dt)
        out = torch.ops.nblist.find_info4mlff(tl, tt, torch.from_numpy(f).to("cuda:0"), *args)
        want = oracle.nblist(L.astype(dt), ty, f, 5.5, 250, is_cart=False, pbc=pbc, sort=sort)
        for x, y in zip(out[1:6], want[1:6]):
            assert np.array_equal(x.cpu().numpy().view(np.uint8), y.view(np.uint8))
    finally:
        torch.ops.nblist.set_sync_free(was)
