"""GPU short-range force / virial operators against the CPU oracle and the committed outputs
of the reference's own kernels, plus first and second derivatives by torch's gradcheck (the
property the reference's tests use, test/fromcc/test_forceSrOp.py:57-81: Jacobian entries +-1)."""
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

GOLD = os.path.join(os.path.dirname(__file__), "golden", "fvt.npz")


def dev(a, dtype=None):
    import torch
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.to("cuda:0")


def random_case(B=3, P=17, U=9, nghost=4, seed=0):
    rng = np.random.default_rng(seed)
    binum = rng.integers(P // 2, P + 1, B).astype(np.int32)
    bilist = np.stack([rng.permutation(P) for _ in range(B)]).astype(np.int32)
    nn = rng.integers(0, U + 1, (B, P)).astype(np.int32)
    fn = rng.integers(0, P + nghost, (B, P, U)).astype(np.int32)
    dei = rng.normal(size=(B, P, U, 3))
    rcs = rng.normal(size=(B, P, U, 3))
    return binum, bilist, nn, fn, dei, rcs


def test_against_golden_and_oracle(oracle):
    import torch
    from ai2pot_amd import ops
    with np.load(GOLD) as z:
        g = {k: z[k] for k in z.files}
    ng = int(g["nghost"])
    inum, U = g["firstneigh"].shape
    dei = dev(g["dei_drij"][None]).requires_grad_(True)
    f = ops.ForceSrOp(dev(np.array([inum], np.int32)), dev(g["ilist"][None]), dev(g["numneigh"][None]),
                      dev(g["firstneigh"][None]), ng, U, dei)[0]
    assert np.abs(f[0].detach().cpu().numpy() - g["force"]).max() < 1e-13
    (gd,) = torch.autograd.grad(f, dei, dev(g["grad_in"][None]))
    assert np.abs(gd[0].cpu().numpy() - g["grad_out"]).max() < 1e-13
    v = ops.VirialSrOp(dev(g["numneigh"][None]), dev(g["rcs"][None]), U, dev(g["dei_drij"][None]))[0]
    assert v.shape == (1, 3, 3)
    assert np.abs(v[0].cpu().numpy().reshape(9) - g["virial"]).max() < 1e-13


@pytest.mark.parametrize("np_dtype", [np.float64, np.float32])
def test_batched_random(oracle, np_dtype):
    import torch
    from ai2pot_amd import ops
    tdt = torch.float64 if np_dtype == np.float64 else torch.float32
    binum, bilist, nn, fn, dei, rcs = random_case()
    B, P, U = fn.shape
    f = ops.ForceSrOp(dev(binum), dev(bilist), dev(nn), dev(fn), 4, U, dev(dei, tdt))[0].cpu().numpy()
    v = ops.VirialSrOp(dev(nn), dev(rcs, tdt), U, dev(dei, tdt))[0].cpu().numpy()
    tol = 1e-12 if np_dtype == np.float64 else 2e-5
    for b in range(B):
        n = binum[b]
        fr, _ = oracle.fvt_force(bilist[b, :n], nn[b, :n], fn[b, :n], 4 + P - n, dei[b, :n].astype(np_dtype))
        assert np.abs(f[b] - fr).max() < tol * max(1.0, np.abs(fr).max())
        vr, _, _ = oracle.fvt_virial(nn[b], rcs[b].astype(np_dtype), dei[b].astype(np_dtype))
        assert np.abs(v[b].reshape(9) - vr).max() < tol * max(1.0, np.abs(vr).max())


def test_gradcheck_first_and_second_order():
    import torch
    from ai2pot_amd import ops
    binum, bilist, nn, fn, dei, rcs = random_case(B=2, P=5, U=4, nghost=2, seed=3)
    U = fn.shape[2]
    lists = (dev(binum), dev(bilist), dev(nn), dev(fn))
    d = dev(dei).requires_grad_(True)
    r = dev(rcs).requires_grad_(True)
    force = lambda x: ops.ForceSrOp(lists[0], lists[1], lists[2], lists[3], 2, U, x)[0]
    virial = lambda rr, x: ops.VirialSrOp(lists[2], rr, U, x)[0]
    assert torch.autograd.gradcheck(force, (d,), eps=1e-6, atol=1e-7)
    assert torch.autograd.gradgradcheck(force, (d,), eps=1e-6, atol=1e-7)
    assert torch.autograd.gradcheck(virial, (r, d), eps=1e-6, atol=1e-7)
    assert torch.autograd.gradgradcheck(virial, (r, d), eps=1e-6, atol=1e-7)


def test_large_and_reproducible():
    """4096 rows x 200 slots: the size configuration 2 would hand to these operators."""
    import torch
    from ai2pot_amd import ops
    rng = np.random.default_rng(5)
    P, U = 4096, 200
    nn = rng.integers(30, 70, (1, P)).astype(np.int32)
    fn = rng.integers(0, P, (1, P, U)).astype(np.int32)
    dei = dev(rng.normal(size=(1, P, U, 3)).astype(np.float32))
    args = (dev(np.array([P], np.int32)), dev(np.arange(P, dtype=np.int32)[None]), dev(nn), dev(fn), 0, U, dei)
    f1 = ops.ForceSrOp(*args)[0]
    f2 = ops.ForceSrOp(*args)[0]
    assert torch.equal(f1, f2)                       # bit-reproducible: no floating atomics
    g = dei.cpu().numpy().astype(np.float64)[0]
    valid = np.arange(U)[None, :] < nn[0][:, None]
    want = (g * valid[..., None]).sum(1)
    np.subtract.at(want, fn[0][valid], g[valid])
    assert np.abs(f1.cpu().numpy()[0] - want).max() < 2e-4


def test_errors():
    from ai2pot_amd import ops
    binum, bilist, nn, fn, dei, rcs = random_case()
    U = fn.shape[2]
    with pytest.raises(RuntimeError):
        ops.ForceSrOp(dev(binum), dev(bilist), dev(nn + 100), dev(fn), 4, U, dev(dei))
    with pytest.raises(RuntimeError):
        ops.ForceSrOp(dev(binum), dev(bilist), dev(nn), dev(fn), 4, U + 1, dev(dei))
    with pytest.raises(RuntimeError):
        ops.VirialSrOp(dev(nn), dev(rcs).float(), U, dev(dei))
