"""The caller contract of the LAMMPS pair style (interface/lammps/AI2POT/pair_ai2pot.cpp:175-249):
one structure, rows for the nlocal owned atoms in the order of LAMMPS' ilist, neighbour indices
into [0, nlocal + nghost), a list built with cutoff + skin (so it holds pairs beyond the model's
cutoff), rcs = x[j] - x[i] in float, types for owned and ghost atoms, and buffers from
torch::empty whose padded entries are never written.  Forces come back for owned and ghost atoms;
LAMMPS folds the ghost forces onto their owners (reverse communication).

Checks: the operators agree with the oracle on such an input (padded entries filled with garbage),
and folding the ghost forces back reproduces the periodic evaluation of the same cell."""
import itertools

import numpy as np
import pytest

from ai2pot_amd import mtp_param, synth


def ghosted_domain(box, pos, types, rc_list, umax, seed, np_dtype=np.float64):
    """One periodic cell as a single LAMMPS domain: every atom is owned, periodic images within
    rc_list of the box are ghosts.  Returns (nb, owner) with owner[a] = owned atom behind a."""
    box = np.asarray(box, float)
    n = pos.shape[0]
    xs, owner = [pos], [np.arange(n)]
    for shift in itertools.product((-1, 0, 1), repeat=3):
        if shift == (0, 0, 0):
            continue
        p = pos + np.asarray(shift) * box
        keep = np.all((p > -rc_list) & (p < box + rc_list), axis=1)
        xs.append(p[keep]); owner.append(np.nonzero(keep)[0])
    x = np.concatenate(xs); owner = np.concatenate(owner)
    nall = x.shape[0]
    rng = np.random.default_rng(seed)
    ilist = rng.permutation(n).astype(np.int32)                  # row ii describes atom ilist[ii]
    numneigh = np.zeros(n, np.int32)
    # what torch::empty leaves behind: arbitrary indices and non-finite displacements
    first = rng.integers(-2**31, 2**31 - 1, size=(n, umax), dtype=np.int64).astype(np.int32)
    rcs = np.full((n, umax, 3), np.nan)
    rcs[::2] = 1e30
    for ii, i in enumerate(ilist):
        d = x - pos[i]
        r2 = (d * d).sum(1)
        nbr = np.nonzero((r2 < rc_list * rc_list) & (np.arange(nall) != i))[0]
        nbr = nbr[rng.permutation(nbr.size)]                     # LAMMPS lists are not sorted by distance
        assert nbr.size <= umax
        numneigh[ii] = nbr.size
        first[ii, :nbr.size] = nbr
        rcs[ii, :nbr.size] = d[nbr]
    nb = dict(binum=np.array([n], np.int32), bilist=ilist[None], bnumneigh=numneigh[None], bfirstneigh=first[None],
              brcs=rcs[None].astype(np_dtype), btypes=types[owner][None].astype(np.int32), nghost=nall - n)
    return nb, owner


def fold(force, owner, n):
    out = np.zeros((n, 3))
    np.add.at(out, owner, force[0].astype(np.float64))
    return out


def cell(n=96, box=(13.0, 14.0, 12.5), nt=3, seed=71):
    lat, pos = synth.random_packed(n, list(box), 2.1, seed)
    return lat, pos, synth.rng_randint(seed + 1, n, nt), box


def close(a, b, tol=1e-10):
    return np.abs(np.asarray(a) - np.asarray(b)).max() <= tol * max(np.abs(b).max(), 1e-300)


def test_oracle_nep_fold_back_equals_periodic(oracle):
    lat, pos, ty, box = cell()
    m = synth.nep_model(rmax_radial=6.0, rmax_angular=4.0)
    nb, owner = ghosted_domain(box, pos, ty, 6.5, 200, 5)
    e, f, v = oracle.nep_efv(m, nb)
    per = synth.pack_batch([oracle.nblist(lat, ty, pos, 6.0, 200)])
    ep, fp, vp = oracle.nep_efv(m, per)
    assert f.shape == (1, owner.size, 3)
    assert close(e, ep) and close(v, vp) and close(fold(f, owner, pos.shape[0]), fp[0])


def test_oracle_mtp_fold_back_equals_periodic(oracle):
    lat, pos, ty, box = cell(nt=2)
    m = synth.mtp_model(mtp_param.mtp_param(12), 2, 8, 5.0, 1.5, 3012)
    nb, owner = ghosted_domain(box, pos, ty, 5.6, 200, 6)
    e, f, v = oracle.mtp_efv(m, nb)
    per = synth.pack_batch([oracle.nblist(lat, ty, pos, 5.0, 200)])
    ep, fp, vp = oracle.mtp_efv(m, per)
    assert close(e, ep) and close(v, vp) and close(fold(f, owner, pos.shape[0]), fp[0])


@pytest.mark.gpu
@pytest.mark.parametrize("np_dtype", [np.float32, np.float64])
def test_nep_operator_under_the_lammps_contract(oracle, np_dtype):
    """float32 is what the pair style sends (pair_ai2pot.cpp:192-196)."""
    from test_gpu_nep import check, run_gpu
    lat, pos, ty, box = cell()
    m = synth.nep_model(rmax_radial=6.0, rmax_angular=4.0)
    nb, owner = ghosted_domain(box, pos, ty, 6.5, 200, 5, np_dtype)
    out = run_gpu(m, nb, np_dtype)
    assert out[1].shape == (1, owner.size, 3) and np.isfinite(out[1]).all()
    check(out, oracle.nep_efv(m, nb, np_dtype), np_dtype)
    e2, f2 = run_gpu(m, nb, np_dtype, virial=False)
    assert np.array_equal(e2, out[0]) and np.array_equal(f2, out[1])
    per = synth.pack_batch([oracle.nblist(lat.astype(np_dtype), ty, pos.astype(np_dtype), 6.0, 200)])
    ep, fp, vp = run_gpu(m, per, np_dtype)
    tol = 1e-10 if np_dtype == np.float64 else 2e-5
    assert close(out[0], ep, tol) and close(out[2], vp, tol)
    assert np.abs(fold(out[1], owner, pos.shape[0]) - fp[0]).max() <= (1e-10 if np_dtype == np.float64 else 1e-4)


@pytest.mark.gpu
@pytest.mark.parametrize("level,nt", [(12, 2), (20, 4)])
def test_mtp_operators_under_the_lammps_contract(oracle, level, nt):
    import torch
    from ai2pot_amd import ops
    from conftest import to_device
    from test_gpu_mtp import esites_args, gpu_efv, model_to_device
    lat, pos, ty, box = cell(nt=nt)
    m = synth.mtp_model(mtp_param.mtp_param(level), nt, 8, 5.0, 1.5, 3000 + level, lo=-0.05, hi=0.05)
    nb, owner = ghosted_domain(box, pos, ty, 5.6, 200, 6)
    e, f, v = gpu_efv(m, nb)
    er, fr, vr = oracle.mtp_efv(m, nb)
    assert f.shape == (1, owner.size, 3) and np.isfinite(f).all()
    assert close(e, er) and close(f, fr) and close(v, vr)
    per = synth.pack_batch([oracle.nblist(lat, ty, pos, 5.0, 200)])
    ep, fp, vp = gpu_efv(m, per)
    assert close(e, ep) and close(v, vp) and close(fold(f, owner, pos.shape[0]), fp[0])
    # site energies of the owned atoms, in row order
    md = model_to_device(m, torch.float64)
    es = ops.linearMtpToEsitesOp(*esites_args(m, md, to_device(nb, torch.float64)), 0.0, 0.0, None, None)[0]
    assert close(es.cpu().numpy(), oracle.mtp_esites(m, nb)[0])
    assert close(es.sum(1).cpu().numpy(), e)
