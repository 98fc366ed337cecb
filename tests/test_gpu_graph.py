"""HIP-graph replay of the energy / force / virial operators: every replay is checked against the
eager result on the same inputs, with eager work and synchronisations between the replays and the
inputs rewritten in place, for the NEP kernels (8 lanes per atom and a thread per atom) and the MTP."""
import numpy as np
import pytest

from ai2pot_amd import mtp_param, synth
from conftest import to_device

pytestmark = pytest.mark.gpu


def replay_matches_eager(op, args, brcs, n_out):
    import torch
    from ai2pot_amd.graph import GraphedCall
    g = GraphedCall(op, *args)
    base = brcs.clone()
    for it, scale in enumerate((1.0, 1.01, 0.995, 1.0)):
        brcs.copy_(base * scale)                            # new geometry, written into the static input
        want = [t.clone() for t in op(*args, validate=False)]            # eager call between the replays
        torch.cuda.synchronize()
        got = g.replay()
        torch.cuda.synchronize()
        assert len(got) == n_out
        for a, b in zip(got, want):
            assert torch.equal(a, b), "replay %d differs from the eager call" % it
    # outputs respond to the inputs (the graph is not replaying stale data)
    assert not torch.equal(got[0], torch.zeros_like(got[0]))


@pytest.mark.parametrize("reps", [4, 21])
def test_nep_graph(oracle, reps):
    import torch
    from ai2pot_amd import ops
    from test_gpu_nep import _model_to_device
    lat, pos = synth.fcc_cell(reps, 4.6, 0.15, 61)
    ty = synth.rng_randint(62, pos.shape[0], 3)
    nb = synth.pack_batch([oracle.nblist(lat.astype(np.float32), ty, pos.astype(np.float32), 6.0, 100)])
    m = synth.nep_model(rmax_radial=6.0, rmax_angular=4.0)
    md = _model_to_device(m, torch.float32)
    d = to_device(nb, torch.float32)
    args = (m["chebyshev_size"], m["n_radial_basis"], m["n_angular_basis"], m["l_max"], md["coeffs"], md["w0"],
            md["b0"], md["w1"], md["type_bias"], d["binum"], d["bilist"], d["bnumneigh"], d["bfirstneigh"], d["brcs"],
            d["btypes"], md["type_map"], 0, m["rmax_radial"], m["rmax_angular"], md["q_scaler"])
    replay_matches_eager(ops.nepToEFVOp, args, d["brcs"], 3)


@pytest.mark.parametrize("level", [10, 20])
def test_mtp_graph(oracle, level):
    import torch
    from ai2pot_amd import ops
    from test_gpu_mtp import esites_args, model_to_device
    lat, pos = synth.diamond_cell()
    nb = synth.pack_batch([oracle.nblist(lat, np.zeros(216, np.int32), pos, 5.0, 200)])
    m = synth.mtp_model(mtp_param.mtp_param(level), 1, 8, 5.0, 0.5, 3001, lo=-0.05, hi=0.05, type_map=[14])
    md = model_to_device(m, torch.float64)
    d = to_device(nb, torch.float64)
    args = esites_args(m, md, d)
    replay_matches_eager(ops.linearMtpToEFVOp, args, d["brcs"], 3)
    replay_matches_eager(ops.linearMtpToEsitesOp, args, d["brcs"], 1)


def test_graph_survives_a_workspace_change(oracle):
    """A captured graph names the library's workspace by address.  Releasing the workspace (or a later
    call that needs a larger one) is noticed by the next replay, which records the call again instead of
    replaying onto freed memory; the result still equals the eager call."""
    import torch
    from ai2pot_amd import _lib, ops
    from ai2pot_amd.graph import GraphedCall
    from test_gpu_nep import _model_to_device
    lat, pos = synth.fcc_cell(4, 4.6, 0.15, 63)
    ty = synth.rng_randint(64, pos.shape[0], 3)
    nb = synth.pack_batch([oracle.nblist(lat.astype(np.float32), ty, pos.astype(np.float32), 6.0, 100)])
    m = synth.nep_model(rmax_radial=6.0, rmax_angular=4.0)
    md = _model_to_device(m, torch.float32)
    d = to_device(nb, torch.float32)
    args = (m["chebyshev_size"], m["n_radial_basis"], m["n_angular_basis"], m["l_max"], md["coeffs"], md["w0"],
            md["b0"], md["w1"], md["type_bias"], d["binum"], d["bilist"], d["bnumneigh"], d["bfirstneigh"], d["brcs"],
            d["btypes"], md["type_map"], 0, m["rmax_radial"], m["rmax_angular"], md["q_scaler"])
    g = GraphedCall(ops.nepToEFVOp, *args)
    want = [t.clone() for t in ops.nepToEFVOp(*args, validate=False)]
    first = [t.clone() for t in g.replay()]
    torch.cuda.synchronize()
    assert g.valid() and g.recaptures == 0
    _lib.check(_lib.lib().a2p_workspace_release())
    assert not g.valid()
    again = g.replay()
    torch.cuda.synchronize()
    assert g.valid() and g.recaptures == 1
    for a, b, c in zip(first, again, want):
        assert torch.equal(a, c) and torch.equal(b, c)
