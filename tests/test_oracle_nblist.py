"""Pins the CPU oracle's neighbour list: against the committed outputs of the reference's own
code (tests/golden/nblist.npz), against the compiled reference when oracle/_ref is present,
against the reference's own test assertions, and against a brute force over images."""
import os

import numpy as np
import pytest

from ai2pot_amd import synth

GOLD = os.path.join(os.path.dirname(__file__), "golden", "nblist.npz")


def cases():
    with np.load(GOLD) as z:
        names = sorted({k.split("/")[0] for k in z.files})
    return names


@pytest.mark.parametrize("name", cases())
def test_against_golden(oracle, name):
    with np.load(GOLD) as z:
        g = {k.split("/", 1)[1]: z[k] for k in z.files if k.startswith(name + "/")}
    rc, umax, cart, p0, p1, p2, sort = g["in_params"]
    out = oracle.nblist(g["in_lattice"], g["in_types"], g["in_coords"], rc, int(umax), is_cart=bool(cart),
                        pbc=(p0, p1, p2), sort=bool(sort))
    inum, ilist, numneigh, first, rcs, types, nghost = out
    w = g["firstneigh"].shape[1]
    assert inum == g["in_coords"].shape[0] and nghost == 0
    assert np.array_equal(ilist, g["ilist"]) and np.array_equal(numneigh, g["numneigh"])
    assert np.array_equal(types, g["types"])
    assert np.array_equal(first[:, :w], g["firstneigh"])
    assert (first[:, w:] == -1).all() and (rcs[:, w:] == 0).all()
    assert rcs.dtype == g["rcs"].dtype
    assert np.array_equal(rcs[:, :w].view(np.uint8), g["rcs"].view(np.uint8))


def brute_force(lattice, coords, rcut, pbc, nimg=3):
    """All (j, image) within rcut of every i, by exhaustive search in double."""
    n = coords.shape[0]
    rng = [range(-nimg, nimg + 1) if p else range(0, 1) for p in pbc]
    res = []
    for i in range(n):
        found = []
        for a in rng[0]:
            for b in rng[1]:
                for c in rng[2]:
                    d = coords + a * lattice[0] + b * lattice[1] + c * lattice[2] - coords[i]
                    r2 = (d * d).sum(1)
                    for j in np.nonzero((r2 < rcut * rcut) & (r2 > 1e-3))[0]:
                        found.append((int(j), tuple(np.round(d[j], 6))))
        res.append(sorted(found))
    return res


@pytest.mark.parametrize("pbc", [(True, True, True), (True, False, True), (False, False, False)])
def test_brute_force(oracle, pbc):
    L = np.array([[6.0, 0.3, -0.2], [1.1, 5.2, 0.4], [-0.7, 0.9, 6.1]])
    fr = synth.rng_uniform(77, 3 * 20).reshape(20, 3)
    ty = synth.rng_randint(78, 20, 2)
    coords = fr @ L
    inum, _, numneigh, first, rcs, _, _ = oracle.nblist(L, ty, coords, 4.0, 200, pbc=pbc)
    want = brute_force(L, coords, 4.0, pbc)
    for i in range(inum):
        got = sorted((int(first[i, s]), tuple(np.round(rcs[i, s], 6))) for s in range(numneigh[i]))
        assert got == want[i]


def test_reference_assertions(oracle):
    """source/nblist/tests/test_neighborList.cc:215, 244: 12 centre atoms, at most 12
    neighbours at rcut 3.2 on the MoS2 cell."""
    lat, types, frac = synth.mos2_fixture()
    out = oracle.nblist(lat, types, frac, 3.2, 20, is_cart=False, sort=True)
    assert out[0] == 12 and out[2].max() == 12
    # sorted rows are in non-decreasing distance
    r = np.linalg.norm(out[4], axis=2)
    for i in range(12):
        assert np.all(np.diff(r[i, :out[2][i]]) >= -1e-12)


def test_symmetry_and_overflow(oracle):
    lat, pos = synth.random_packed(200, [15.0, 16.0, 17.0], 2.0, 5)
    ty = synth.rng_randint(6, 200, 3)
    inum, _, numneigh, first, rcs, _, _ = oracle.nblist(lat.astype(np.float32), ty, pos.astype(np.float32),
                                                        6.0, 150)
    counts = np.bincount(first[first >= 0], minlength=inum)
    assert np.array_equal(counts, numneigh)               # j in N(i) <=> i in N(j)
    with pytest.raises(RuntimeError):
        oracle.nblist(lat, ty, pos, 6.0, 10)


@pytest.mark.skipif(not os.path.exists(os.path.join(os.path.dirname(__file__), "..", "oracle", "_ref",
                                                    "libref_nblist.so")), reason="oracle/_ref not built")
@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("sort", [False, True])
def test_against_compiled_reference(oracle, dt, sort):
    lat, pos = synth.fcc_cell(5, 4.949, 0.15, 9)
    ty = synth.rng_randint(10, pos.shape[0], 3)
    a = oracle.nblist(lat.astype(dt), ty, pos.astype(dt), 7.0, 200, sort=sort)
    b = oracle.ref_nblist(lat.astype(dt), ty, pos.astype(dt), 7.0, 200, sort=sort)
    for x, y in zip(a[1:6], b[1:6]):
        assert np.array_equal(x.view(np.uint8), y.view(np.uint8))
