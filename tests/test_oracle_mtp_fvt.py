"""Pins the CPU oracle's linear-MTP evaluation, training-loss step and fvt reductions: the
reference's known answer and committed outputs, then finite differences of the energy and of
the loss, radial-function end values and linearity."""
import os

import numpy as np
import pytest

from ai2pot_amd import mtp_param, synth

HERE = os.path.dirname(__file__)


def small_batch(oracle, level, nt):
    lat, pos = synth.random_packed(48, [8.5, 9.0, 9.5], 2.0, 21)
    ty = synth.rng_randint(22, 48, nt)
    t = mtp_param.mtp_param(level)
    m = synth.mtp_model(t, nt, 8, 5.0, 0.5 if level == 10 else 1.8, 3000 + level)
    o = oracle.nblist(lat, ty, pos, 5.0, 100)
    nb = synth.pack_batch([o, o])
    nb["brcs"][1] *= 1.01
    return m, nb, (lat, pos, ty)


def labels_for(nb):
    B, P = nb["bilist"].shape
    return dict(energy=synth.rng_normal(1, B, -4 * 48, 3), force=synth.rng_normal(2, B * P * 3).reshape(B, P, 3),
                virial=synth.rng_normal(3, B * 9, 0, 0.5).reshape(B, 9))


def test_known_answer_of_reference_unit_test(oracle):
    """source/descriptor/mtpr/tests/test_linearMtp.cc (efv_force_accuracy set-up, level 16)."""
    lat, types, frac = synth.mos2_fixture()
    nb = synth.pack_batch([oracle.nblist(lat, types, frac, 5.0, 20, is_cart=False, sort=True)])
    m = synth.mtp_model_closed_form(mtp_param.mtp_param(16))
    e, f, v = oracle.mtp_efv(m, nb)
    assert abs(e[0] - (-0.938157350795572)) < 1e-13
    assert abs(f[0, 1, 2] - (-0.520135157048249)) < 1e-13


@pytest.mark.parametrize("level,nt", [(8, 2), (10, 1), (16, 3)])
def test_against_golden(oracle, level, nt):
    with np.load(os.path.join(HERE, "golden", "mtp.npz")) as z:
        g = {k.split("/")[1]: z[k] for k in z.files if k.startswith("L%02d/" % level)}
    m, nb, _ = small_batch(oracle, level, nt)
    t = mtp_param.mtp_param(level)
    assert list(g["table_sizes"]) == [t["alpha_moments_count"], t["alpha_index_basic"].shape[0],
                                      t["alpha_index_times"].shape[0], t["alpha_moment_mapping"].size,
                                      t["nmus"]]
    e, f, v = oracle.mtp_efv(m, nb)
    for got, key in ((e, "E"), (f, "F"), (v, "V")):
        assert np.abs(got - g[key]).max() <= 1e-12 * np.abs(g[key]).max()
    if level == 16:
        # the forward-mode gradient of level 16 takes a minute; levels 8 and 10 cover it
        return
    r = oracle.mtp_loss_step(m, nb, (1.0, 0.7, 0.3), labels_for(nb))
    for k, val in r.items():
        ref = g["loss_" + k]
        assert np.abs(val - ref).max() <= 1e-11 * max(np.abs(ref).max(), 1e-300), k


@pytest.mark.parametrize("level,nt", [(8, 2), (10, 1), (16, 3)])
def test_site_energies_and_descriptors(oracle, level, nt):
    """Site energies, scalar moments and the site-energy gradient: the reference's committed
    outputs, then what fixes them without it (sum rule, the linear read-out, dE_i/dbias = 1)."""
    with np.load(os.path.join(HERE, "golden", "mtp.npz")) as z:
        g = {k.split("/")[1]: z[k] for k in z.files if k.startswith("L%02d/" % level)}
    m, nb, _ = small_batch(oracle, level, nt)
    B, P = nb["bilist"].shape
    es, desc = oracle.mtp_esites(m, nb)
    assert np.abs(es - g["esites"]).max() <= 1e-12 * np.abs(g["esites"]).max()
    assert np.abs(desc - g["desc"]).max() <= 1e-12 * np.abs(g["desc"]).max()
    e, _, _ = oracle.mtp_efv(m, nb)
    assert np.abs(es.sum(1) - e).max() < 1e-12 * np.abs(e).max()
    # e_i = bias[t_i] + sum_s lin_s * desc_is / q_scaler_s   (linearMtp.h:594-599)
    ti = np.take_along_axis(nb["btypes"], nb["bilist"], 1)
    want = m["type_bias"][ti] + (desc * (m["linear_coeffs"] / m["q_scaler"])).sum(-1)
    assert np.abs(es - want).max() < 1e-12 * np.abs(es).max()
    if level == 16:
        return
    gout = synth.rng_normal(4, B * P).reshape(B, P)
    dc, dl, db = oracle.mtp_esites_bwd(m, nb, gout)
    for got, key in ((dc, "es_dcoeffs"), (dl, "es_dlinear"), (db, "es_dbias")):
        assert np.abs(got - g[key]).max() <= 1e-11 * max(np.abs(g[key]).max(), 1e-300), key
    assert np.abs(dl - np.einsum("bi,bis->bs", gout, desc) / m["q_scaler"]).max() < 1e-11 * np.abs(dl).max()
    for t in range(nt):
        assert np.abs(db[:, t] - (gout * (ti == t)).sum(1)).max() < 1e-12
    h = 1e-6
    for i in (0, 9, m["coeffs"].size - 1):
        mp, mm = dict(m), dict(m)
        mp["coeffs"] = m["coeffs"].copy(); mp["coeffs"][i] += h
        mm["coeffs"] = m["coeffs"].copy(); mm["coeffs"][i] -= h
        fd = ((oracle.mtp_esites(mp, nb)[0] - oracle.mtp_esites(mm, nb)[0]) * gout).sum(1) / (2 * h)
        assert np.abs(fd - dc[:, i]).max() < 1e-6 * max(1.0, np.abs(fd).max())


@pytest.mark.parametrize("level,nt", [(8, 2), (10, 1), (16, 3)])
def test_legacy_basis_operator_backward(oracle, level, nt):
    """Backward of mtpBasisOp for weights w of the scalar moments: the committed outputs of the reference's
    MtpBasis::find_val_der + find_der_backward; then, without it, central differences of the oracle's own
    scalar moments along pair vectors and coefficients, zeros beyond each row and beyond the cutoff, and
    linearity in w."""
    with np.load(os.path.join(HERE, "golden", "mtp.npz")) as z:
        g = {k.split("/")[1]: z[k] for k in z.files if k.startswith("L%02d/" % level)}
    m, nb, _ = small_batch(oracle, level, nt)
    B, P = nb["bilist"].shape
    U = nb["brcs"].shape[2]
    S = m["alpha_moment_mapping"].size
    w = synth.rng_normal(5, B * P * S).reshape(B, P, S)
    drcs, dc = oracle.mtp_basis_bwd(m, nb, w, want_dcoeffs=level != 16)
    width = g["basis_drcs"].shape[2]
    assert np.abs(drcs[:, :, :width] - g["basis_drcs"]).max() <= 1e-11 * np.abs(g["basis_drcs"]).max()
    assert np.all(drcs[:, :, width:] == 0)
    if dc is not None:
        assert np.abs(dc - g["basis_dcoeffs"]).max() <= 1e-11 * np.abs(g["basis_dcoeffs"]).max()
    # entries beyond a row's neighbour count, and neighbours beyond rmax, get nothing
    nn = nb["bnumneigh"]
    beyond = np.arange(U)[None, None, :] >= nn[:, :, None]
    assert np.all(drcs[beyond] == 0)
    r = np.linalg.norm(nb["brcs"], axis=-1)
    assert np.all(drcs[(r > m["rmax"]) & ~beyond] == 0)
    # central differences of sum(w * desc) along three pair vectors and three coefficients
    phi = lambda mm, bb: (oracle.mtp_esites(mm, bb)[1] * w).sum((1, 2))
    h = 1e-6
    for (b, ii, u, a) in ((0, 0, 0, 0), (1, 17, 3, 2), (0, 40, int(nn[0, 40]) - 1, 1)):
        if r[b, ii, u] > m["rmax"] - 1e-3:
            continue
        p_, m_ = dict(nb), dict(nb)
        p_["brcs"] = nb["brcs"].copy(); p_["brcs"][b, ii, u, a] += h
        m_["brcs"] = nb["brcs"].copy(); m_["brcs"][b, ii, u, a] -= h
        fd = (phi(m, p_)[b] - phi(m, m_)[b]) / (2 * h)
        assert abs(fd - drcs[b, ii, u, a]) < 1e-6 * max(1.0, abs(fd)), (b, ii, u, a)
    if dc is not None:
        for i in (0, 7, m["coeffs"].size - 1):
            mp, mm = dict(m), dict(m)
            mp["coeffs"] = m["coeffs"].copy(); mp["coeffs"][i] += h
            mm["coeffs"] = m["coeffs"].copy(); mm["coeffs"][i] -= h
            fd = (phi(mp, nb) - phi(mm, nb)) / (2 * h)
            assert np.abs(fd - dc[:, i]).max() < 1e-6 * max(1.0, np.abs(fd).max())
    d2, _ = oracle.mtp_basis_bwd(m, nb, -2.5 * w, want_dcoeffs=False)
    assert np.abs(d2 + 2.5 * drcs).max() <= 1e-13 * np.abs(drcs).max()


@pytest.mark.parametrize("level,nt", [(8, 2), (10, 1), (16, 3)])
def test_linear_system_and_schmidt(oracle, level, nt):
    """Normal equations of the linear parameters and the Gram-Schmidt of the radial functions: the
    reference's committed outputs; then what fixes them without it: column s of the components is
    the E/F/V of the model with linear_coeffs = e_s (so the system is rebuilt from E/F/V calls),
    the solution of the system reproduces labels generated by a linear model, and the
    orthogonalised functions are orthonormal."""
    with np.load(os.path.join(HERE, "golden", "mtp.npz")) as z:
        g = {k.split("/")[1]: z[k] for k in z.files if k.startswith("L%02d/" % level)}
    m, nb, _ = small_batch(oracle, level, nt)
    m["q_scaler"] = np.linspace(0.7, 1.4, m["q_scaler"].size)
    lab = labels_for(nb)
    w = (1.0, 0.7, 0.3)
    A, b = oracle.mtp_lin_system(m, nb, w, lab)
    assert np.abs(A - g["lin_matrix"]).max() <= 1e-12 * np.abs(g["lin_matrix"]).max()
    assert np.abs(b - g["lin_vector"]).max() <= 1e-12 * np.abs(g["lin_vector"]).max()
    assert np.array_equal(A, A.T)
    K, nmus = m["chebyshev_size"], m["nmus"]
    oc = oracle.mtp_schmidt_orth(m["coeffs"], nt, nmus, K)
    assert np.array_equal(oc, g["orth_coeffs"])
    vecs = oc.reshape(nt * nt, nmus, K).transpose(1, 0, 2).reshape(nmus, -1)
    gram = vecs @ vecs.T
    assert np.abs(gram - np.diag(np.diag(gram))).max() < 1e-12
    assert np.abs(np.diag(gram) - 1).max() < 1e-6           # the reference adds 1e-10 to every squared norm
    if level == 16:
        return
    S = m["q_scaler"].size
    n = S + nt
    B, P = nb["bilist"].shape
    Ec, Fc, Vc = np.zeros((B, n)), np.zeros((B, P, 3, n)), np.zeros((B, 9, n))
    for s_ in range(S):
        one = dict(m, linear_coeffs=np.eye(S)[s_], type_bias=np.zeros(nt))
        Ec[:, s_], Fc[..., s_], Vc[..., s_] = oracle.mtp_efv(one, nb)
    ti = np.take_along_axis(nb["btypes"], nb["bilist"], 1)
    for t_ in range(nt):
        Ec[:, S + t_] = (ti == t_).sum(1)
    F2, V2 = Fc.reshape(-1, n), Vc.reshape(-1, n)
    A2 = w[0] * Ec.T @ Ec + w[1] * F2.T @ F2 + w[2] * V2.T @ V2
    assert np.abs(A2 - A).max() < 1e-12 * np.abs(A).max()
    # labels of a linear model are reproduced by the solution of its own normal equations
    e, f, v = oracle.mtp_efv(m, nb)
    A3, b3 = oracle.mtp_lin_system(m, nb, w, dict(energy=e, force=f, virial=v))
    x_true = np.concatenate([m["linear_coeffs"], m["type_bias"]])
    assert np.abs(A3 @ x_true - b3).max() < 1e-10 * np.abs(b3).max()


def test_energy_force_finite_difference_and_linearity(oracle):
    lat, pos = synth.random_packed(30, [8.0, 8.5, 9.0], 2.0, 31)
    ty = synth.rng_randint(32, 30, 2)
    m = synth.mtp_model(mtp_param.mtp_param(12), 2, 8, 4.0, 1.5, 77)

    def efv(p, model=m):
        return oracle.mtp_efv(model, synth.pack_batch([oracle.nblist(lat, ty, p, 4.0, 120)]))

    e0, f0, v0 = efv(pos)
    h = 1e-5
    for i, a in ((0, 0), (11, 1), (29, 2)):
        p = pos.copy(); p[i, a] += h
        ep = efv(p)[0][0]
        p[i, a] -= 2 * h
        em = efv(p)[0][0]
        assert abs(-(ep - em) / (2 * h) - f0[0, i, a]) < 1e-6 * max(1.0, abs(f0[0, i, a]))
    assert np.abs(f0.sum(1)).max() < 1e-10 * np.abs(f0).max()
    # E - bias is linear in linear_coeffs
    m2 = dict(m)
    m2["linear_coeffs"] = 2.5 * m["linear_coeffs"]
    nbias = np.bincount(ty, minlength=2) @ m["type_bias"]
    e2 = efv(pos, m2)[0][0]
    assert abs((e2 - nbias) - 2.5 * (e0[0] - nbias)) < 1e-11 * abs(e0[0])


def test_radial_function_end_values(oracle):
    """The switch is 1 at rmin and 0 at rmax with zero slope (mtpr/tests/test_basis.cc:106-111):
    a single neighbour at rmin gives M_0 = sum_k c_k T_k(-1) = sum_k (-1)^k c_k; beyond rmax
    and below rmin it contributes nothing (basis.h:157-165)."""
    t = mtp_param.mtp_param(6)
    m = synth.mtp_model(t, 1, 8, 5.0, 2.0, 5)
    m["linear_coeffs"] = np.zeros_like(m["linear_coeffs"]); m["linear_coeffs"][0] = 1.0
    m["type_bias"] = np.zeros(1)
    assert t["alpha_moment_mapping"][0] == 0 and list(t["alpha_index_basic"][0]) == [0, 0, 0, 0]

    def energy(r):
        nb = dict(binum=np.array([1], np.int32), bilist=np.zeros((1, 1), np.int32),
                  bnumneigh=np.array([[1]], np.int32), bfirstneigh=np.zeros((1, 1, 1), np.int32),
                  brcs=np.array([[[[0.0, 0.0, r]]]]), btypes=np.zeros((1, 1), np.int32), nghost=0)
        return oracle.mtp_efv(m, nb)
    c = m["coeffs"][:8]
    assert abs(energy(2.0)[0][0] - np.sum(c * (-1.0) ** np.arange(8))) < 1e-14
    assert energy(5.0)[0][0] == 0.0 and energy(1.999)[0][0] == 0.0
    assert abs(energy(4.999999)[0][0]) < 1e-15
    assert np.abs(energy(5.0 - 1e-9)[1]).max() < 1e-12        # zero slope at the cutoff


def test_loss_gradient_by_finite_differences(oracle):
    """d bloss / d theta from the oracle against central differences of its own forward loss."""
    m, nb, _ = small_batch(oracle, 8, 2)
    lab = labels_for(nb)
    w = (1.0, 0.7, 0.3)
    r0 = oracle.mtp_loss_step(m, nb, w, lab)
    h = 1e-6
    for key, gkey, idxs in (("coeffs", "dcoeffs", (0, 17, 40)), ("linear_coeffs", "dlinear", (0, 5)),
                            ("type_bias", "dbias", (1,))):
        for i in idxs:
            mp, mm = dict(m), dict(m)
            mp[key] = m[key].copy(); mp[key][i] += h
            mm[key] = m[key].copy(); mm[key][i] -= h
            lp = oracle.mtp_loss_step(mp, nb, w, lab)["bloss"]
            lm = oracle.mtp_loss_step(mm, nb, w, lab)["bloss"]
            fd = (lp - lm) / (2 * h)
            assert np.abs(fd - r0[gkey][:, i]).max() < 1e-5 * max(1.0, np.abs(fd).max())


def test_fvt_against_golden_and_closed_form(oracle):
    with np.load(os.path.join(HERE, "golden", "fvt.npz")) as z:
        g = {k: z[k] for k in z.files}
    f, go = oracle.fvt_force(g["ilist"], g["numneigh"], g["firstneigh"], int(g["nghost"]), g["dei_drij"],
                             g["grad_in"])
    v, d1, d2 = oracle.fvt_virial(g["numneigh"], g["rcs"], g["dei_drij"], True)
    assert np.array_equal(f, g["force"]) and np.array_equal(go, g["grad_out"])
    assert np.array_equal(v, g["virial"]) and np.array_equal(d1, g["der1"]) and np.array_equal(d2, g["der2"])
    # closed form: V = - sum_{valid pairs} g (x) r
    mask = np.arange(g["rcs"].shape[1])[None, :] < g["numneigh"][:, None]
    want = -np.einsum("isa,isb->ab", g["dei_drij"] * mask[..., None], g["rcs"])
    assert np.abs(v.reshape(3, 3) - want).max() < 1e-13
