"""Writes tests/golden/*.npz: inputs and the outputs of the reference's own C++ code
(compiled from /root/reference by oracle/Makefile into oracle/_ref) for small cases.

    make -C oracle ref && python tests/golden/make_golden.py

The fixtures are data only (arrays); they let the CPU test-suite pin this repository's
oracle, and the GPU tests pin the HIP path, where the reference tree is absent.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "..", ".."))
import oracle  # noqa: E402
from ai2pot_amd import mtp_param, synth  # noqa: E402


def trim(out):
    """Drop the padding columns beyond the longest row to keep the files small."""
    inum, ilist, numneigh, first, rcs, types, nghost = out
    w = max(int(numneigh.max()), 1)
    return dict(ilist=ilist, numneigh=numneigh, firstneigh=first[:, :w], rcs=rcs[:, :w], types=types)


def nblist_cases():
    cases = {}
    lat, types, frac = synth.mos2_fixture()
    L = np.array([[9.0, 0.3, -0.2], [1.1, 8.2, 0.4], [-0.7, 0.9, 10.1]])
    fr = synth.rng_uniform(7, 3 * 60).reshape(60, 3)
    ty = synth.rng_randint(8, 60, 3)
    for dt in (np.float32, np.float64):
        for sort in (0, 1):
            for rc in (3.2, 5.0):
                cases["mos2_%s_s%d_rc%.1f" % (dt.__name__, sort, rc)] = (
                    lat.astype(dt), types, frac.astype(dt), rc, 64, False, (1, 1, 1), sort)
            for pbc in ((1, 1, 1), (1, 0, 1), (0, 0, 0)):
                cases["tri_%s_s%d_p%d%d%d" % ((dt.__name__, sort) + pbc)] = (
                    L.astype(dt), ty, fr.astype(dt), 5.5, 80, False, pbc, sort)
    out = {}
    for name, (la, t, c, rc, umax, cart, pbc, sort) in cases.items():
        res = oracle.ref_nblist(la, t, c, rc, umax, is_cart=cart, pbc=pbc, sort=bool(sort))
        out[name + "/in_lattice"] = la
        out[name + "/in_types"] = t
        out[name + "/in_coords"] = c
        out[name + "/in_params"] = np.array([rc, umax, int(cart), pbc[0], pbc[1], pbc[2], sort], np.float64)
        for k, v in trim(res).items():
            out[name + "/" + k] = v
    np.savez_compressed(os.path.join(HERE, "nblist.npz"), **out)
    print("nblist.npz", len(cases), "cases")


def nep_cases():
    out = {}
    lat, types, frac = synth.mos2_fixture()
    nb = synth.pack_batch([oracle.ref_nblist(lat, types, frac, 5.0, 20, is_cart=False, sort=True)])
    m = synth.nep_model_closed_form()
    e, f, v = oracle.ref_nep_efv(m, nb, np.float64)
    d = oracle.ref_nep_descriptors(m, nb, np.float64)
    out.update({"mos2/E": e, "mos2/F": f, "mos2/V": v, "mos2/D": d})
    lat2, pos2 = synth.random_packed(96, [12.0, 13.0, 12.5], 2.2, 11)
    ty2 = synth.rng_randint(12, 96, 3)
    m2 = synth.nep_model()
    for dt in (np.float64, np.float32):
        o = oracle.ref_nblist(lat2.astype(dt), ty2, pos2.astype(dt), 7.0, 160)
        nb2 = synth.pack_batch([o])
        e, f, v = oracle.ref_nep_efv(m2, nb2, dt)
        tag = "rand_" + dt.__name__
        out.update({tag + "/E": e, tag + "/F": f, tag + "/V": v,
                    tag + "/D": oracle.ref_nep_descriptors(m2, nb2, dt)})
    np.savez_compressed(os.path.join(HERE, "nep.npz"), **out)
    print("nep.npz")


def mtp_cases():
    out = {}
    lat, pos = synth.random_packed(48, [8.5, 9.0, 9.5], 2.0, 21)
    for level, nt in ((8, 2), (10, 1), (16, 3)):
        ty = synth.rng_randint(22, 48, nt)
        t = mtp_param.mtp_param(level)
        ref_t = oracle.ref_mtp_param(level)
        for k in ("alpha_index_basic", "alpha_index_times", "alpha_moment_mapping"):
            assert np.array_equal(t[k], ref_t[k])
        m = synth.mtp_model(t, nt, 8, 5.0, 0.5 if level == 10 else 1.8, 3000 + level)
        o = oracle.ref_nblist(lat, ty, pos, 5.0, 100)
        nb = synth.pack_batch([o, o])
        nb["brcs"][1] *= 1.01
        e, f, v = oracle.ref_mtp_efv(m, nb)
        B, P = nb["bilist"].shape
        labels = dict(energy=synth.rng_normal(1, B, -4 * 48, 3),
                      force=synth.rng_normal(2, B * P * 3).reshape(B, P, 3),
                      virial=synth.rng_normal(3, B * 9, 0, 0.5).reshape(B, 9))
        r = oracle.ref_mtp_loss_step(m, nb, (1.0, 0.7, 0.3), labels)
        tag = "L%02d" % level
        out.update({tag + "/E": e, tag + "/F": f, tag + "/V": v})
        for k, val in r.items():
            out[tag + "/loss_" + k] = val
        es, desc = oracle.ref_mtp_esites(m, nb)
        dc, dl, db = oracle.ref_mtp_esites_bwd(m, nb, synth.rng_normal(4, B * P).reshape(B, P))
        out.update({tag + "/esites": es, tag + "/desc": desc, tag + "/es_dcoeffs": dc,
                    tag + "/es_dlinear": dl, tag + "/es_dbias": db})
        # legacy basis operator: its output equals the descriptors; the backward for weights w[B, P, S]
        S = t["alpha_moment_mapping"].size
        bval, bdrcs, bdc = oracle.ref_mtp_basis(m, nb, synth.rng_normal(5, B * P * S).reshape(B, P, S), level)
        assert np.allclose(bval, desc, rtol=1e-12, atol=1e-14)
        out.update({tag + "/basis_drcs": bdrcs[:, :, :int(nb["bnumneigh"].max())], tag + "/basis_dcoeffs": bdc})
        m2 = dict(m)
        m2["q_scaler"] = np.linspace(0.7, 1.4, m["q_scaler"].size)
        A, bv = oracle.ref_mtp_lin_system(m2, nb, (1.0, 0.7, 0.3), labels)
        out.update({tag + "/lin_matrix": A, tag + "/lin_vector": bv,
                    tag + "/orth_coeffs": oracle.ref_mtp_schmidt_orth(m["coeffs"], nt, t["nmus"], 8)})
        out[tag + "/table_sizes"] = np.array([t["alpha_moments_count"], t["alpha_index_basic"].shape[0],
                                              t["alpha_index_times"].shape[0],
                                              t["alpha_moment_mapping"].size, t["nmus"]])
    np.savez_compressed(os.path.join(HERE, "mtp.npz"), **out)
    print("mtp.npz")


def nnmtp_cases():
    """Neural-network MTP: E/F/V and site energies of the reference's NNMtp (fp64)."""
    out = {}
    lat, pos = synth.random_packed(48, [8.5, 9.0, 9.5], 2.0, 21)
    for level, nt, H in ((8, 2, 7), (16, 3, 20), (10, 1, 6)):
        ty = synth.rng_randint(22, 48, nt)
        m = synth.nnmtp_model(mtp_param.mtp_param(level), nt, 8, H, 5.0, 1.8, 3200 + level)
        o = oracle.ref_nblist(lat, ty, pos, 5.0, 100)
        nb = synth.pack_batch([o, o])
        nb["brcs"][1] *= 1.01
        e, f, v, es = oracle.ref_nnmtp_efv(m, nb)
        tag = "L%02d" % level
        out.update({tag + "/E": e, tag + "/F": f, tag + "/V": v, tag + "/esites": es})
        B, P = nb["bilist"].shape
        labels = dict(energy=synth.rng_normal(1, B, -4 * 48, 3),
                      force=synth.rng_normal(2, B * P * 3).reshape(B, P, 3),
                      virial=synth.rng_normal(3, B * 9, 0, 0.5).reshape(B, 9))
        r = oracle.ref_nnmtp_loss_step(m, nb, (1.0, 0.7, 0.3), labels)
        for k, val in r.items():
            out[tag + "/loss_" + k] = val
        if nt == 1:     # the reference's site-energy backward assigns w0 / w1 rows correctly only for one species
            g = oracle.ref_nnmtp_esites_bwd(m, nb, synth.rng_normal(4, B * P).reshape(B, P))
            for k, val in zip(("dcoeffs", "dw0", "dw1", "dbias"), g):
                out[tag + "/es_" + k] = val
    np.savez_compressed(os.path.join(HERE, "nnmtp.npz"), **out)
    print("nnmtp.npz")


def nep_loss_cases():
    """Two small structures, two species: the reference's loss forward + backward (fp64)."""
    out = {}
    lists = []
    for i, n in enumerate((40, 27)):
        lat, pos = synth.random_packed(n, [9.0 + 0.2 * i, 9.5, 10.0], 2.0, 5 + 3 * i)
        lists.append(oracle.ref_nblist(lat, synth.rng_randint(6 + 3 * i, n, 2), pos, 5.0, 80))
    nb = synth.pack_batch(lists)
    w = max(int(nb["bnumneigh"].max()), 1)
    nb["bfirstneigh"] = np.ascontiguousarray(nb["bfirstneigh"][:, :, :w])
    nb["brcs"] = np.ascontiguousarray(nb["brcs"][:, :, :w])
    B, P = nb["bilist"].shape
    m = synth.nep_model(ntypes=2, seed=905, rmax_radial=5.0, rmax_angular=3.5, num_neurons=7)
    m["q_scaler"] = np.linspace(0.7, 1.4, m["q_scaler"].size)
    labels = dict(energy=synth.rng_normal(55, B, -3.0, 1.0), force=synth.rng_normal(56, B * P * 3).reshape(B, P, 3),
                  virial=synth.rng_normal(57, B * 9, 0.0, 0.5).reshape(B, 9))
    for k in ("binum", "bilist", "bnumneigh", "bfirstneigh", "brcs", "btypes"):
        out["in_" + k] = nb[k]
    for k in ("coeffs", "w0", "b0", "w1", "type_bias", "q_scaler", "type_map"):
        out["model_" + k] = np.asarray(m[k])
    out["model_sizes"] = np.array([m["chebyshev_size"], m["n_radial_basis"], m["n_angular_basis"], m["l_max"]])
    out["model_cutoffs"] = np.array([m["rmax_radial"], m["rmax_angular"]])
    for k, v in labels.items():
        out["label_" + k] = v
    for tag, wts in (("efv", (1.0, 0.7, 0.3)), ("ef", (1.0, 0.7, 0.0))):
        r = oracle.ref_nep_loss_step(m, nb, wts, labels)
        out[tag + "/weights"] = np.array(wts)
        for k, v in r.items():
            out[tag + "/" + k] = v
    np.savez_compressed(os.path.join(HERE, "nep_loss.npz"), **out)
    print("nep_loss.npz")


def fvt_cases():
    rng = np.random.default_rng(0)
    inum, U, ng = 10, 6, 3
    nn = rng.integers(0, U + 1, inum).astype(np.int32)
    fn = rng.integers(0, inum + ng, (inum, U)).astype(np.int32)
    il = rng.permutation(inum).astype(np.int32)
    dei = rng.normal(size=(inum, U, 3))
    rcs = rng.normal(size=(inum, U, 3))
    gin = rng.normal(size=(inum + ng, 3))
    f, g = oracle.ref_fvt_force(il, nn, fn, ng, dei, gin)
    v, d1, d2 = oracle.ref_fvt_virial(nn, rcs, dei, True)
    np.savez_compressed(os.path.join(HERE, "fvt.npz"), ilist=il, numneigh=nn, firstneigh=fn, nghost=ng,
                        dei_drij=dei, rcs=rcs, grad_in=gin, force=f, grad_out=g, virial=v, der1=d1, der2=d2)
    print("fvt.npz")


if __name__ == "__main__":
    # usage: make_golden.py [nblist nep mtp nnmtp nep_loss fvt]; default all.  The reference sums
    # energies and forces with OpenMP atomics, so a regenerated floating-point fixture can differ
    # from the committed one in the last bits: regenerate only what changed.
    assert oracle.ref_available("nblist"), "build oracle/_ref first: make -C oracle ref"
    cases = dict(nblist=nblist_cases, nep=nep_cases, mtp=mtp_cases, nnmtp=nnmtp_cases, nep_loss=nep_loss_cases,
                 fvt=fvt_cases)
    for name in (sys.argv[1:] or list(cases)):
        cases[name]()
