"""CPU checkers for the energy / force / virial hot path.  TEST INFRASTRUCTURE ONLY.

Only the tests, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py``
may import this package; the product (``ai2pot_amd``) never does.

Two families of functions with identical NumPy signatures:

* ``nblist``, ``nep_efv``, ``nep_loss``, ``mtp_efv``, ``mtp_loss_step``, ``mtp_esites``, ``mtp_esites_bwd``, ``mtp_basis_bwd``,
  ``nnmtp_efv``, ``fvt_force``, ``fvt_virial`` --
  this repository's own C++ restatement of the reference algorithm (``oracle/src``,
  ``liboracle.so``), each function citing the reference file:line it follows;
* ``ref_*`` -- the reference's own headers compiled where they lie (``oracle/_ref/*.so``,
  built by ``oracle/Makefile`` when the reference tree is present).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_C = ctypes
_libs = {}


def build(ref=True):
    """Compile liboracle.so and, when the reference tree is present, oracle/_ref."""
    subprocess.check_call(["make", "-s", "-C", _HERE, "oracle"])
    if ref:
        subprocess.check_call(["make", "-s", "-C", _HERE, "ref"])


def _load(name):
    if name in _libs:
        return _libs[name]
    path = os.path.join(_HERE, name)
    lib = _C.CDLL(path) if os.path.exists(path) else None
    _libs[name] = lib
    return lib


def oracle_lib():
    lib = _load("liboracle.so")
    if lib is None:
        build(ref=False)
        _libs.pop("liboracle.so")
        lib = _load("liboracle.so")
    return lib


def ref_available(which="nep"):
    return _load("_ref/libref_%s.so" % which) is not None


def _p(a):
    return None if a is None else a.ctypes.data_as(_C.c_void_p)


def _c(a, dt):
    return np.ascontiguousarray(a, dtype=dt)


_I = _C.c_int
_D = _C.c_double


# ----------------------------------------------------------------------------------------
# neighbor list
# ----------------------------------------------------------------------------------------
def _nblist(lib, prefix, lattice, types, coords, rcut, umax, is_cart, pbc, sort):
    coords = np.ascontiguousarray(coords)
    dt = coords.dtype
    assert dt in (np.float32, np.float64)
    suffix = "f32" if dt == np.float32 else "f64"
    lattice = _c(lattice, dt).reshape(9)
    types = _c(types, np.int32)
    n = coords.shape[0]
    pbc_i = _c([int(bool(x)) for x in pbc], np.int32)
    ilist = np.zeros(n, np.int32)
    numneigh = np.zeros(n, np.int32)
    firstneigh = np.zeros((n, umax), np.int32)
    rcs = np.zeros((n, umax, 3), dt)
    types_out = np.zeros(n, np.int32)
    max_nn = _I(0)
    fn = getattr(lib, "%s_%s" % (prefix, suffix))
    fn.restype = _I
    rc = fn(_p(lattice), _p(types), _p(coords), _I(n), _D(float(rcut)), _I(umax), _I(int(is_cart)),
            _p(pbc_i), _I(int(sort)), _p(ilist), _p(numneigh), _p(firstneigh), _p(rcs),
            _p(types_out), _C.byref(max_nn))
    if rc != 0:
        raise RuntimeError("neighbor count %d exceeds umax_num_neigh_atoms %d" % (max_nn.value, umax))
    return n, ilist, numneigh, firstneigh, rcs, types_out, 0


def ref_nblist(lattice, types, coords, rcut, umax, is_cart=True, pbc=(True, True, True), sort=False):
    return _nblist(_load("_ref/libref_nblist.so"), "ref_nblist", lattice, types, coords, rcut, umax,
                   is_cart, pbc, sort)


def nblist(lattice, types, coords, rcut, umax, is_cart=True, pbc=(True, True, True), sort=False):
    return _nblist(oracle_lib(), "orc_nblist", lattice, types, coords, rcut, umax, is_cart, pbc, sort)


# ----------------------------------------------------------------------------------------
# shared unpacking of the 7-tensor neighbor batch
# ----------------------------------------------------------------------------------------
def _batch(nb, dt):
    binum = _c(nb["binum"], np.int32)
    bilist = _c(nb["bilist"], np.int32)
    bnumneigh = _c(nb["bnumneigh"], np.int32)
    bfirst = _c(nb["bfirstneigh"], np.int32)
    brcs = _c(nb["brcs"], dt)
    btypes = _c(nb["btypes"], np.int32)
    nghost = int(nb.get("nghost", 0))
    B, P = bilist.shape
    U = bfirst.shape[2]
    assert brcs.shape == (B, P, U, 3) and btypes.shape == (B, P + nghost)
    return binum, bilist, bnumneigh, bfirst, brcs, btypes, nghost, B, P, U


# ----------------------------------------------------------------------------------------
# NEP
# ----------------------------------------------------------------------------------------
def _nep_efv(lib, prefix, model, nb, dtype):
    dt = np.dtype(dtype)
    suffix = "f32" if dt == np.float32 else "f64"
    binum, bilist, bnumneigh, bfirst, brcs, btypes, nghost, B, P, U = _batch(nb, dt)
    coeffs = _c(model["coeffs"], dt)
    w0 = _c(model["w0"], dt)
    b0 = _c(model["b0"], dt)
    w1 = _c(model["w1"], dt)
    bias = _c(model["type_bias"], dt)
    q_scaler = _c(model["q_scaler"], dt)
    type_map = _c(model["type_map"], np.int32)
    ntypes = type_map.size
    H = w1.size // ntypes
    e = np.zeros(B, dt)
    f = np.zeros((B, P + nghost, 3), dt)
    v = np.zeros((B, 9), dt)
    mb = _many_body(model)
    fn = getattr(lib, "%s_efv_%s%s" % (prefix, "mb_" if mb else "", suffix))
    fn.restype = None
    fn(_p(e), _p(f), _p(v), _I(model["chebyshev_size"]), _I(model["n_radial_basis"]),
       _I(model["n_angular_basis"]), _I(model["l_max"]), _I(H), _p(coeffs), _p(w0), _p(b0), _p(w1),
       _p(bias), _I(B), _I(P), _p(binum), _p(bilist), _p(bnumneigh), _p(bfirst), _p(brcs),
       _p(btypes), _I(ntypes), _p(type_map), _I(U), _I(nghost), _D(model["rmax_radial"]),
       _D(model["rmax_angular"]), _p(q_scaler), *mb)
    return e, f, v


def _many_body(model):
    """() for the reference's model; (_I(mb4), _I(mb5)) for the extension with a four-body (l_4body = 2) and / or a
    five-body (l_5body = 1) invariant per angular channel (restatement only: the reference has no such terms)."""
    l4, l5 = int(model.get("l_4body", 0)), int(model.get("l_5body", 0))
    if not (l4 or l5):
        return ()
    assert l4 in (0, 2) and l5 in (0, 1) and model["l_max"] >= max(l4, l5)
    return (_I(1 if l4 else 0), _I(1 if l5 else 0))


def _nep_desc(lib, prefix, model, nb, dtype):
    dt = np.dtype(dtype)
    suffix = "f32" if dt == np.float32 else "f64"
    binum, bilist, bnumneigh, bfirst, brcs, btypes, nghost, B, P, U = _batch(nb, dt)
    assert nghost == 0
    coeffs = _c(model["coeffs"], dt)
    type_map = _c(model["type_map"], np.int32)
    n_r, n_a, l_max = model["n_radial_basis"], model["n_angular_basis"], model["l_max"]
    mb = _many_body(model)
    D = n_r + n_a * (l_max + sum(x.value for x in mb))
    d = np.zeros((B, P, D), dt)
    fn = getattr(lib, "%s_desc_%s%s" % (prefix, "mb_" if mb else "", suffix))
    fn.restype = None
    fn(_p(d), _I(model["chebyshev_size"]), _I(n_r), _I(n_a), _I(l_max), _p(coeffs), _I(B), _I(P),
       _p(binum), _p(bilist), _p(bnumneigh), _p(bfirst), _p(brcs), _p(btypes), _I(type_map.size),
       _p(type_map), _I(U), _I(nghost), _D(model["rmax_radial"]), _D(model["rmax_angular"]), *mb)
    return d


def ref_nep_efv(model, nb, dtype=np.float64):
    return _nep_efv(_load("_ref/libref_nep.so"), "ref_nep", model, nb, dtype)


def nep_efv(model, nb, dtype=np.float64):
    return _nep_efv(oracle_lib(), "orc_nep", model, nb, dtype)


def ref_nep_descriptors(model, nb, dtype=np.float64):
    return _nep_desc(_load("_ref/libref_nep.so"), "ref_nep", model, nb, dtype)


def nep_descriptors(model, nb, dtype=np.float64):
    return _nep_desc(oracle_lib(), "orc_nep", model, nb, dtype)


def nep_loss(model, nb, weights, labels):
    """Training loss of the NEP operators, restated from the definitions (nepLoss.h:170-209 per
    structure; nepLoss_cpu_launcher.h:357-406 RMSEs) on top of this package's own E/F/V.
    Returns (bloss[B], rmse[3], etot, force, virial)."""
    e_w, f_w, v_w = weights
    e, f, v = nep_efv(model, nb, np.float64)
    binum = np.asarray(nb["binum"]).reshape(-1)
    bilist = np.asarray(nb["bilist"])
    B = binum.size
    bloss = np.zeros(B)
    e_mse = f_mse = v_mse = 0.0
    nf = 0
    for b in range(B):
        n = int(binum[b])
        idx = bilist[b, :n]
        df = f[b, idx] - np.asarray(labels["force"], np.float64)[b, idx]
        dv = v[b] - np.asarray(labels["virial"], np.float64)[b]
        de = e[b] - float(np.asarray(labels["energy"], np.float64)[b])
        bloss[b] = f_w / (3 * n) * (df ** 2).sum() + v_w / (9 * n) * (dv ** 2).sum() + e_w / n * de ** 2
        e_mse += (de / n) ** 2
        f_mse += (df ** 2).sum()
        nf += 3 * n
        v_mse += (dv ** 2).sum()
    rmse = np.array([np.sqrt(e_mse / B), np.sqrt(f_mse / nf), np.sqrt(v_mse / (9 * B))])
    return bloss, rmse, e, f, v


def nep_loss_dirderiv(model, nb, weights, labels, direction, h=1e-6):
    """d/d eps of bloss[b](theta + eps * direction) at eps = 0 by a central difference in fp64:
    an independent check of the analytic parameter gradients (sum over parameters of
    gradient * direction).  `direction` maps parameter names to arrays of the parameters' shapes."""
    def shifted(sign):
        m = dict(model)
        for k, d in direction.items():
            m[k] = np.asarray(model[k], np.float64) + sign * h * np.asarray(d, np.float64).reshape(np.shape(model[k]))
        return nep_loss(m, nb, weights, labels)[0]
    return (shifted(+1.0) - shifted(-1.0)) / (2.0 * h)


def ref_nep_loss_step(model, nb, weights, labels):
    """The reference's own loss forward + backward (oracle/_ref).  Returns a dict with bloss, rmse,
    etot, force, virial and the per-structure gradients dcoeffs, dw0, db0, dw1, dbias."""
    lib = _load("_ref/libref_nep.so")
    dt = np.dtype(np.float64)
    binum, bilist, bnumneigh, bfirst, brcs, btypes, nghost, B, P, U = _batch(nb, dt)
    assert nghost == 0
    coeffs, w0, b0, w1 = (_c(model[k], dt) for k in ("coeffs", "w0", "b0", "w1"))
    bias = _c(model["type_bias"], dt)
    q_scaler = _c(model["q_scaler"], dt)
    type_map = _c(model["type_map"], np.int32)
    nt = type_map.size
    H = w1.size // nt
    K, n_r, n_a, l_max = (int(model[k]) for k in ("chebyshev_size", "n_radial_basis", "n_angular_basis", "l_max"))
    D = n_r if l_max == 0 else n_r + n_a * l_max
    out = dict(bloss=np.zeros(B), rmse=np.zeros(3), etot=np.zeros(B), force=np.zeros((B, P, 3)),
               virial=np.zeros((B, 9)), dcoeffs=np.zeros((B, nt * nt * (n_r + n_a) * K)),
               dw0=np.zeros((B, nt * H * D)), db0=np.zeros((B, nt * H)), dw1=np.zeros((B, nt * H)),
               dbias=np.zeros((B, nt)))
    e0 = _c(labels["energy"], dt)
    f0 = _c(labels["force"], dt)
    v0 = _c(labels["virial"], dt)
    fn = lib.ref_nep_loss_step_f64
    fn.restype = None
    fn(_p(out["bloss"]), _p(out["rmse"]), _p(out["etot"]), _p(out["force"]), _p(out["virial"]),
       _p(out["dcoeffs"]), _p(out["dw0"]), _p(out["db0"]), _p(out["dw1"]), _p(out["dbias"]),
       _D(weights[0]), _D(weights[1]), _D(weights[2]), _p(e0), _p(f0), _p(v0), _I(K), _I(n_r), _I(n_a),
       _I(l_max), _I(H), _p(coeffs), _p(w0), _p(b0), _p(w1), _p(bias), _I(B), _I(P), _p(binum), _p(bilist),
       _p(bnumneigh), _p(bfirst), _p(brcs), _p(btypes), _I(nt), _p(type_map), _I(U), _I(0),
       _D(model["rmax_radial"]), _D(model["rmax_angular"]), _p(q_scaler))
    return out


# ----------------------------------------------------------------------------------------
# linear MTP
# ----------------------------------------------------------------------------------------
def ref_mtp_param(level, ai2pot_path="/root/reference"):
    """Contraction tables of one level, parsed by the reference's own MtpParam."""
    lib = _load("_ref/libref_mtpr.so")
    saved = os.environ.get("AI2POT_PATH")
    os.environ["AI2POT_PATH"] = ai2pot_path     # the reference reads it with getenv
    try:
        counts = np.zeros(5, np.int32)
        lib.ref_mtp_param.restype = _I
        if lib.ref_mtp_param(_I(level), _p(counts), None, None, None) != 0:
            raise RuntimeError("reference MtpParam failed for level %d" % level)
        basic = np.zeros((counts[1], 4), np.int32)
        times = np.zeros((counts[2], 4), np.int32)
        mapping = np.zeros(counts[3], np.int32)
        lib.ref_mtp_param(_I(level), _p(counts), _p(basic), _p(times), _p(mapping))
    finally:
        if saved is None:
            del os.environ["AI2POT_PATH"]
        else:
            os.environ["AI2POT_PATH"] = saved
    return dict(alpha_moments_count=int(counts[0]), alpha_index_basic=basic,
                alpha_index_times=times, alpha_moment_mapping=mapping, nmus=int(counts[4]))


def _mtp_model_args(model):
    coeffs = _c(model["coeffs"], np.float64)
    lin = _c(model["linear_coeffs"], np.float64)
    bias = _c(model["type_bias"], np.float64)
    basic = _c(model["alpha_index_basic"], np.int32)
    times = _c(model["alpha_index_times"], np.int32)
    mapping = _c(model["alpha_moment_mapping"], np.int32)
    keep = (coeffs, lin, bias, basic, times, mapping)
    args = [_I(model["chebyshev_size"]), _D(model.get("scaling", 1.0)), _p(coeffs), _p(lin), _p(bias),
            _I(model["alpha_moments_count"]), _I(basic.shape[0]), _p(basic), _I(times.shape[0]),
            _p(times), _I(mapping.size), _p(mapping), _I(model["nmus"])]
    return args, keep


def _mtp_list_args(model, nb):
    binum, bilist, bnumneigh, bfirst, brcs, btypes, nghost, B, P, U = _batch(nb, np.float64)
    type_map = _c(model["type_map"], np.int32)
    q_scaler = _c(model["q_scaler"], np.float64)
    keep = (binum, bilist, bnumneigh, bfirst, brcs, btypes, type_map, q_scaler)
    args = [_I(B), _I(P), _p(binum), _p(bilist), _p(bnumneigh), _p(bfirst), _p(brcs), _p(btypes),
            _I(type_map.size), _p(type_map), _I(U), _I(nghost), _D(model["rmax"]), _D(model["rmin"]),
            _p(q_scaler)]
    return args, keep, (B, P, U, nghost, type_map.size)


def _mtp_efv(lib, prefix, model, nb):
    margs, k1 = _mtp_model_args(model)
    largs, k2, (B, P, U, nghost, ntypes) = _mtp_list_args(model, nb)
    e = np.zeros(B)
    f = np.zeros((B, P + nghost, 3))
    v = np.zeros((B, 9))
    fn = getattr(lib, prefix + "_efv_f64")
    fn.restype = None
    fn(_p(e), _p(f), _p(v), *margs, *largs)
    return e, f, v


def _mtp_loss_step(lib, prefix, model, nb, weights, labels):
    margs, k1 = _mtp_model_args(model)
    largs, k2, (B, P, U, nghost, ntypes) = _mtp_list_args(model, nb)
    assert nghost == 0
    K, nmus = model["chebyshev_size"], model["nmus"]
    S = np.asarray(model["alpha_moment_mapping"]).size
    ncoef = ntypes * ntypes * nmus * K
    e_dft = _c(labels["energy"], np.float64)
    f_dft = _c(labels["force"], np.float64)
    v_dft = _c(labels["virial"], np.float64)
    assert e_dft.shape == (B,) and f_dft.shape == (B, P, 3) and v_dft.shape == (B, 9)
    out = dict(bloss=np.zeros(B), rmse=np.zeros(3), energy=np.zeros(B), force=np.zeros((B, P, 3)),
               virial=np.zeros((B, 9)), dcoeffs=np.zeros((B, ncoef)), dlinear=np.zeros((B, S)),
               dbias=np.zeros((B, ntypes)))
    fn = getattr(lib, prefix + "_loss_step_f64")
    fn.restype = None
    fn(_p(out["bloss"]), _p(out["rmse"]), _p(out["energy"]), _p(out["force"]), _p(out["virial"]),
       _p(out["dcoeffs"]), _p(out["dlinear"]), _p(out["dbias"]), _D(weights[0]), _D(weights[1]),
       _D(weights[2]), _p(e_dft), _p(f_dft), _p(v_dft), *margs, *largs)
    return out


def ref_mtp_efv(model, nb):
    return _mtp_efv(_load("_ref/libref_mtpr.so"), "ref_mtp", model, nb)


def mtp_efv(model, nb):
    return _mtp_efv(oracle_lib(), "orc_mtp", model, nb)


def ref_mtp_loss_step(model, nb, weights, labels):
    return _mtp_loss_step(_load("_ref/libref_mtpr.so"), "ref_mtp", model, nb, weights, labels)


def mtp_loss_step(model, nb, weights, labels):
    return _mtp_loss_step(oracle_lib(), "orc_mtp", model, nb, weights, labels)


def _mtp_esites(lib, prefix, model, nb):
    margs, k1 = _mtp_model_args(model)
    largs, k2, (B, P, U, nghost, ntypes) = _mtp_list_args(model, nb)
    S = np.asarray(model["alpha_moment_mapping"]).size
    e_sites = np.zeros((B, P))
    desc = np.zeros((B, P, S))
    fn = getattr(lib, prefix + "_esites_f64")
    fn.restype = None
    fn(_p(e_sites), _p(desc), *margs, *largs)
    return e_sites, desc


def _mtp_esites_bwd(lib, prefix, model, nb, gout):
    margs, k1 = _mtp_model_args(model)
    largs, k2, (B, P, U, nghost, ntypes) = _mtp_list_args(model, nb)
    S = np.asarray(model["alpha_moment_mapping"]).size
    ncoef = ntypes * ntypes * model["nmus"] * model["chebyshev_size"]
    gout = _c(gout, np.float64)
    assert gout.shape == (B, P)
    dc, dl, db = np.zeros((B, ncoef)), np.zeros((B, S)), np.zeros((B, ntypes))
    fn = getattr(lib, prefix + "_esites_bwd_f64")
    fn.restype = None
    fn(_p(dc), _p(dl), _p(db), _p(gout), *margs, *largs)
    return dc, dl, db


def ref_mtp_esites(model, nb):
    """(e_sites[B, P], descriptors[B, P, S]) by the reference (row order, zero beyond inum)."""
    return _mtp_esites(_load("_ref/libref_mtpr.so"), "ref_mtp", model, nb)


def mtp_esites(model, nb):
    return _mtp_esites(oracle_lib(), "orc_mtp", model, nb)


def ref_mtp_esites_bwd(model, nb, gout):
    """Per-structure gradients of sum(gout * e_sites) w.r.t. coeffs, linear_coeffs, type_bias."""
    return _mtp_esites_bwd(_load("_ref/libref_mtpr.so"), "ref_mtp", model, nb, gout)


def mtp_esites_bwd(model, nb, gout):
    return _mtp_esites_bwd(oracle_lib(), "orc_mtp", model, nb, gout)


def ref_mtp_basis(model, nb, w, level, ai2pot_path="/root/reference"):
    """The legacy basis operator by the reference (MtpBasis::find_val_der + find_der_backward):
    (val[B, P, S], drcs[B, P, U, 3], dcoeffs[B, ncoef]) for the weights w[B, P, S]; the tables are those of
    the reference's own MtpParam(level)."""
    lib = _load("_ref/libref_mtpr.so")
    binum, bilist, bnumneigh, bfirst, brcs, btypes, nghost, B, P, U = _batch(nb, np.float64)
    S = np.asarray(model["alpha_moment_mapping"]).size
    ntypes = np.asarray(model["type_map"]).size
    ncoef = ntypes * ntypes * model["nmus"] * model["chebyshev_size"]
    coeffs = _c(model["coeffs"], np.float64)
    w = _c(w, np.float64)
    assert w.shape == (B, P, S)
    val, drcs, dc = np.zeros((B, P, S)), np.zeros((B, P, U, 3)), np.zeros((B, ncoef))
    saved = os.environ.get("AI2POT_PATH")
    os.environ["AI2POT_PATH"] = ai2pot_path     # the reference reads it with getenv
    try:
        lib.ref_mtp_basis_f64.restype = _I
        rc = lib.ref_mtp_basis_f64(_p(val), _p(drcs), _p(dc), _p(w), _I(level), _I(model["chebyshev_size"]),
                                   _D(model.get("scaling", 1.0)), _p(coeffs), _I(B), _I(P), _p(binum), _p(bilist),
                                   _p(bnumneigh), _p(bfirst), _p(brcs), _p(btypes), _I(ntypes), _I(U), _I(nghost),
                                   _D(model["rmax"]), _D(model["rmin"]))
    finally:
        if saved is None:
            del os.environ["AI2POT_PATH"]
        else:
            os.environ["AI2POT_PATH"] = saved
    if rc != 0:
        raise RuntimeError("reference MtpParam failed for level %d" % level)
    return val, drcs, dc


def mtp_basis_bwd(model, nb, w, want_drcs=True, want_dcoeffs=True):
    """(drcs[B, P, U, 3], dcoeffs[B, ncoef]) of sum(w * scalar moments), w[B, P, S]: the backward of the legacy
    basis operator."""
    margs, k1 = _mtp_model_args(model)
    largs, k2, (B, P, U, nghost, ntypes) = _mtp_list_args(model, nb)
    S = np.asarray(model["alpha_moment_mapping"]).size
    ncoef = ntypes * ntypes * model["nmus"] * model["chebyshev_size"]
    w = _c(w, np.float64)
    assert w.shape == (B, P, S)
    drcs = np.zeros((B, P, U, 3)) if want_drcs else None
    dc = np.zeros((B, ncoef)) if want_dcoeffs else None
    fn = oracle_lib().orc_mtp_basis_bwd_f64
    fn.restype = None
    fn(_p(drcs) if want_drcs else None, _p(dc) if want_dcoeffs else None, _p(w), *margs, *largs)
    return drcs, dc


def _mtp_lin_system(lib, prefix, model, nb, weights, labels):
    margs, k1 = _mtp_model_args(model)
    largs, k2, (B, P, U, nghost, ntypes) = _mtp_list_args(model, nb)
    assert nghost == 0
    n = np.asarray(model["alpha_moment_mapping"]).size + ntypes
    e_res = _c(labels["energy"], np.float64)
    f_res = _c(labels["force"], np.float64)
    v_res = _c(labels["virial"], np.float64)
    assert e_res.shape == (B,) and f_res.shape == (B, P, 3) and v_res.shape == (B, 9)
    A, b = np.zeros((n, n)), np.zeros(n)
    fn = getattr(lib, prefix + "_lin_system_f64")
    fn.restype = None
    fn(_p(A), _p(b), _D(weights[0]), _D(weights[1]), _D(weights[2]), _p(e_res), _p(f_res), _p(v_res), *margs, *largs)
    return A, b


def ref_mtp_lin_system(model, nb, weights, labels):
    """(lin_matrix[n, n], lin_vector[n]) of the reference's LinMatrixLinVector CPU launcher."""
    return _mtp_lin_system(_load("_ref/libref_mtpr.so"), "ref_mtp", model, nb, weights, labels)


def mtp_lin_system(model, nb, weights, labels):
    return _mtp_lin_system(oracle_lib(), "orc_mtp", model, nb, weights, labels)


def _schmidt(lib, prefix, coeffs, ntypes, nmus, K):
    c = _c(coeffs, np.float64)
    assert c.size == ntypes * ntypes * nmus * K
    out = np.zeros_like(c)
    fn = getattr(lib, prefix + "_schmidt_orth_f64")
    fn.restype = None
    fn(_p(out), _I(ntypes), _I(nmus), _I(K), _p(c))
    return out


def ref_mtp_schmidt_orth(coeffs, ntypes, nmus, K):
    return _schmidt(_load("_ref/libref_mtpr.so"), "ref_mtp", coeffs, ntypes, nmus, K)


def mtp_schmidt_orth(coeffs, ntypes, nmus, K):
    return _schmidt(oracle_lib(), "orc_mtp", coeffs, ntypes, nmus, K)


# ----------------------------------------------------------------------------------------
# neural-network MTP (fp64)
# ----------------------------------------------------------------------------------------
def _nnmtp_efv(lib, prefix, model, nb, want_esites=True):
    coeffs = _c(model["coeffs"], np.float64)
    w0, w1 = _c(model["w0"], np.float64), _c(model["w1"], np.float64)
    bias = _c(model["type_bias"], np.float64)
    basic = _c(model["alpha_index_basic"], np.int32)
    times = _c(model["alpha_index_times"], np.int32)
    mapping = _c(model["alpha_moment_mapping"], np.int32)
    shift, scale = _c(model["q_shifter"], np.float64), _c(model["q_scaler"], np.float64)
    type_map = _c(model["type_map"], np.int32)
    binum, bilist, bnumneigh, bfirst, brcs, btypes, nghost, B, P, U = _batch(nb, np.float64)
    e, f, v = np.zeros(B), np.zeros((B, P + nghost, 3)), np.zeros((B, 9))
    es = np.zeros((B, P)) if want_esites else None
    fn = getattr(lib, prefix + "_efv_f64")
    fn.restype = None
    fn(_p(e), _p(f), _p(v), _p(es), _I(model["chebyshev_size"]), _I(model["num_neurons"]), _p(coeffs), _p(w0),
       _p(w1), _p(bias), _I(model["alpha_moments_count"]), _I(basic.shape[0]), _p(basic), _I(times.shape[0]),
       _p(times), _I(mapping.size), _p(mapping), _I(model["nmus"]), _I(B), _I(P), _p(binum), _p(bilist),
       _p(bnumneigh), _p(bfirst), _p(brcs), _p(btypes), _I(type_map.size), _p(type_map), _I(U), _I(nghost),
       _D(model["rmax"]), _D(model["rmin"]), _p(shift), _p(scale))
    return e, f, v, es


def ref_nnmtp_efv(model, nb):
    """(E[B], F[B, P+nghost, 3], V[B, 9], e_sites[B, P]) by the reference's NNMtp."""
    return _nnmtp_efv(_load("_ref/libref_nnmtp.so"), "ref_nnmtp", model, nb)


def nnmtp_efv(model, nb):
    return _nnmtp_efv(oracle_lib(), "orc_nnmtp", model, nb)


def _nnmtp_loss_step(lib, prefix, model, nb, weights, labels):
    coeffs = _c(model["coeffs"], np.float64)
    w0, w1 = _c(model["w0"], np.float64), _c(model["w1"], np.float64)
    bias = _c(model["type_bias"], np.float64)
    basic = _c(model["alpha_index_basic"], np.int32)
    times = _c(model["alpha_index_times"], np.int32)
    mapping = _c(model["alpha_moment_mapping"], np.int32)
    shift, scale = _c(model["q_shifter"], np.float64), _c(model["q_scaler"], np.float64)
    type_map = _c(model["type_map"], np.int32)
    binum, bilist, bnumneigh, bfirst, brcs, btypes, nghost, B, P, U = _batch(nb, np.float64)
    assert nghost == 0
    e_dft = _c(labels["energy"], np.float64)
    f_dft = _c(labels["force"], np.float64)
    v_dft = _c(labels["virial"], np.float64)
    assert e_dft.shape == (B,) and f_dft.shape == (B, P, 3) and v_dft.shape == (B, 9)
    out = dict(bloss=np.zeros(B), energy=np.zeros(B), force=np.zeros((B, P, 3)), virial=np.zeros((B, 9)),
               dcoeffs=np.zeros((B, coeffs.size)), dw0=np.zeros((B, w0.size)), dw1=np.zeros((B, w1.size)),
               dbias=np.zeros((B, bias.size)))
    fn = getattr(lib, prefix + "_loss_step_f64")
    fn.restype = None
    fn(_p(out["bloss"]), _p(out["energy"]), _p(out["force"]), _p(out["virial"]), _p(out["dcoeffs"]), _p(out["dw0"]),
       _p(out["dw1"]), _p(out["dbias"]), _D(weights[0]), _D(weights[1]), _D(weights[2]), _p(e_dft), _p(f_dft),
       _p(v_dft), _I(model["chebyshev_size"]), _I(model["num_neurons"]), _p(coeffs), _p(w0), _p(w1), _p(bias),
       _I(model["alpha_moments_count"]), _I(basic.shape[0]), _p(basic), _I(times.shape[0]), _p(times),
       _I(mapping.size), _p(mapping), _I(model["nmus"]), _I(B), _I(P), _p(binum), _p(bilist), _p(bnumneigh),
       _p(bfirst), _p(brcs), _p(btypes), _I(type_map.size), _p(type_map), _I(U), _I(nghost), _D(model["rmax"]),
       _D(model["rmin"]), _p(shift), _p(scale))
    return out


def ref_nnmtp_loss_step(model, nb, weights, labels):
    """Loss forward + the reference's find_loss_backward: per-structure gradients [B, n]."""
    return _nnmtp_loss_step(_load("_ref/libref_nnmtp.so"), "ref_nnmtp", model, nb, weights, labels)


def nnmtp_loss_step(model, nb, weights, labels):
    return _nnmtp_loss_step(oracle_lib(), "orc_nnmtp", model, nb, weights, labels)


def _nnmtp_esites_bwd(lib, prefix, model, nb, gout):
    coeffs = _c(model["coeffs"], np.float64)
    w0, w1 = _c(model["w0"], np.float64), _c(model["w1"], np.float64)
    bias = _c(model["type_bias"], np.float64)
    basic = _c(model["alpha_index_basic"], np.int32)
    times = _c(model["alpha_index_times"], np.int32)
    mapping = _c(model["alpha_moment_mapping"], np.int32)
    shift, scale = _c(model["q_shifter"], np.float64), _c(model["q_scaler"], np.float64)
    type_map = _c(model["type_map"], np.int32)
    binum, bilist, bnumneigh, bfirst, brcs, btypes, nghost, B, P, U = _batch(nb, np.float64)
    gout = _c(gout, np.float64)
    assert gout.shape == (B, P)
    out = (np.zeros((B, coeffs.size)), np.zeros((B, w0.size)), np.zeros((B, w1.size)), np.zeros((B, bias.size)))
    fn = getattr(lib, prefix + "_esites_bwd_f64")
    fn.restype = None
    fn(_p(out[0]), _p(out[1]), _p(out[2]), _p(out[3]), _p(gout), _I(model["chebyshev_size"]),
       _I(model["num_neurons"]), _p(coeffs), _p(w0), _p(w1), _p(bias), _I(model["alpha_moments_count"]),
       _I(basic.shape[0]), _p(basic), _I(times.shape[0]), _p(times), _I(mapping.size), _p(mapping),
       _I(model["nmus"]), _I(B), _I(P), _p(binum), _p(bilist), _p(bnumneigh), _p(bfirst), _p(brcs), _p(btypes),
       _I(type_map.size), _p(type_map), _I(U), _I(nghost), _D(model["rmax"]), _D(model["rmin"]), _p(shift), _p(scale))
    return out


def ref_nnmtp_esites_bwd(model, nb, gout):
    """Per-structure gradients of sum(gout * e_sites) w.r.t. coeffs, w0, w1, type_bias (reference)."""
    return _nnmtp_esites_bwd(_load("_ref/libref_nnmtp.so"), "ref_nnmtp", model, nb, gout)


def nnmtp_esites_bwd(model, nb, gout):
    return _nnmtp_esites_bwd(oracle_lib(), "orc_nnmtp", model, nb, gout)


# ----------------------------------------------------------------------------------------
# ZBL correction (fp64): adds onto copies of the given E/F/V
# ----------------------------------------------------------------------------------------
def _zbl(lib, name, zbl, nb, type_map, efv=None):
    binum, bilist, bnumneigh, bfirst, brcs, btypes, nghost, B, P, U = _batch(nb, np.float64)
    type_map = _c(type_map, np.int32)
    cks, dks = _c(zbl["cks"], np.float64), _c(zbl["dks"], np.float64)
    nt = type_map.size
    assert cks.size == nt * nt * 4 and dks.size == nt * nt * 4
    if efv is None:
        e, f, v = np.zeros(B), np.zeros((B, P + nghost, 3)), np.zeros((B, 9))
    else:
        e, f, v = (np.array(x, np.float64, copy=True) for x in efv)
    fn = getattr(lib, name)
    fn.restype = None
    fn(_p(e), _p(f), _p(v), _D(zbl["rmax"]), _D(zbl["rmin"]), _p(cks), _p(dks), _I(nt), _p(type_map), _I(B), _I(P),
       _I(U), _I(nghost), _p(binum), _p(bilist), _p(bnumneigh), _p(bfirst), _p(brcs), _p(btypes))
    return e, f, v


def ref_zbl_correct(zbl, nb, type_map, efv=None):
    """E/F/V plus the ZBL terms, pair by pair through the reference's PairZBL member functions."""
    return _zbl(_load("_ref/libref_zbl.so"), "ref_zbl_correct_f64", zbl, nb, type_map, efv)


def zbl_correct(zbl, nb, type_map, efv=None):
    return _zbl(oracle_lib(), "orc_zbl_correct_f64", zbl, nb, type_map, efv)


def _zbl_esites(lib, name, zbl, nb, type_map):
    binum, bilist, bnumneigh, bfirst, brcs, btypes, nghost, B, P, U = _batch(nb, np.float64)
    type_map = _c(type_map, np.int32)
    cks, dks = _c(zbl["cks"], np.float64), _c(zbl["dks"], np.float64)
    nt = type_map.size
    es = np.zeros((B, P))
    fn = getattr(lib, name)
    fn.restype = None
    fn(_p(es), _D(zbl["rmax"]), _D(zbl["rmin"]), _p(cks), _p(dks), _I(nt), _p(type_map), _I(B), _I(P), _I(U),
       _I(nghost), _p(binum), _p(bilist), _p(bnumneigh), _p(bfirst), _p(brcs), _p(btypes))
    return es


def ref_zbl_esites(zbl, nb, type_map):
    """Per-row ZBL energies [B, P] by the reference's GroupZBL::correct_e_sites."""
    return _zbl_esites(_load("_ref/libref_zbl.so"), "ref_zbl_esites_f64", zbl, nb, type_map)


def zbl_esites(zbl, nb, type_map):
    return _zbl_esites(oracle_lib(), "orc_zbl_esites_f64", zbl, nb, type_map)


# ----------------------------------------------------------------------------------------
# fvt (single structure, fp64)
# ----------------------------------------------------------------------------------------
def _fvt_force(lib, prefix, ilist, numneigh, firstneigh, nghost, dei_drij, grad_in=None):
    ilist = _c(ilist, np.int32)
    numneigh = _c(numneigh, np.int32)
    firstneigh = _c(firstneigh, np.int32)
    dei = _c(dei_drij, np.float64)
    inum, umax = firstneigh.shape
    force = np.zeros((inum + nghost, 3))
    gout = None
    gin = None
    if grad_in is not None:
        gin = _c(grad_in, np.float64)
        gout = np.zeros((inum, umax, 3))
    fn = getattr(lib, prefix + "_force_f64")
    fn.restype = None
    fn(_p(force), _p(gout), _p(gin), _I(inum), _p(ilist), _p(numneigh), _p(firstneigh), _I(nghost),
       _I(umax), _p(dei))
    return force, gout


def _fvt_virial(lib, prefix, numneigh, rcs, dei_drij, ders=False):
    numneigh = _c(numneigh, np.int32)
    rcs = _c(rcs, np.float64)
    dei = _c(dei_drij, np.float64)
    inum, umax = rcs.shape[:2]
    v = np.zeros(9)
    d1 = np.zeros((9, inum, umax)) if ders else None
    d2 = np.zeros((9, inum, umax)) if ders else None
    fn = getattr(lib, prefix + "_virial_f64")
    fn.restype = None
    fn(_p(v), _p(d1), _p(d2), _I(inum), _p(numneigh), _p(rcs), _I(umax), _p(dei))
    return v, d1, d2


def ref_fvt_force(*a, **k):
    return _fvt_force(_load("_ref/libref_fvt.so"), "ref_fvt", *a, **k)


def fvt_force(*a, **k):
    return _fvt_force(oracle_lib(), "orc_fvt", *a, **k)


def ref_fvt_virial(*a, **k):
    return _fvt_virial(_load("_ref/libref_fvt.so"), "ref_fvt", *a, **k)


def fvt_virial(*a, **k):
    return _fvt_virial(oracle_lib(), "orc_fvt", *a, **k)
