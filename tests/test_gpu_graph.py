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


def _md_inputs(n_reps, seed):
    lat, pos = synth.fcc_cell(n_reps, 4.6, 0.12, seed)
    ty = synth.rng_randint(seed + 1, pos.shape[0], 3)
    disp = synth.rng_normal(seed + 2, pos.size, 0.0, 0.02).reshape(-1, 3)
    return lat, pos, ty, disp


@pytest.mark.parametrize("path", ["segments", "gather"])
def test_step_with_rebuild_without_host_synchronisation(oracle, path):
    """Neighbour rebuild + NEP E/F/V with a2p_nblist_sync_free: the bin grid is derived on the device from the
    bound of the first (synchronised) build.  Lists and results are bitwise those of the synchronised build, and
    the whole step replays as a HIP graph on new coordinates."""
    import torch
    from ai2pot_amd.calculator import NepCalculator
    lat, pos, ty, disp = _md_inputs(6, 71)                       # 864 atoms
    n = pos.shape[0]
    m = synth.nep_model(rmax_radial=6.0, rmax_angular=4.0)
    dev = "cuda:0"
    kw = dict(umax=96, dtype=torch.float32, device=dev, path=path)
    free = NepCalculator(m, n, lat, ty, sync_free=True, **kw)
    sync = NepCalculator(m, n, lat, ty, **kw)
    base = torch.from_numpy(pos.astype(np.float32)).to(dev)
    d = torch.from_numpy(disp.astype(np.float32)).to(dev)
    coords = base.clone()                                         # the static input of the graph
    for it, alpha in enumerate((0.0, 1.0, -0.7)):
        coords.copy_(base + alpha * d)
        got = [t.clone() for t in free.step(coords)]
        free.check()
        want = [t.clone() for t in sync.step(coords)]
        sync.check()
        for a, b in zip(got, want):
            assert torch.equal(a, b), "step %d" % it
        for a, b in ((free.numneigh, sync.numneigh), (free.firstneigh, sync.firstneigh), (free.rcs, sync.rcs)):
            nn = sync.numneigh.cpu().numpy()
            fa, fb = a.cpu().numpy(), b.cpu().numpy()
            if fa.ndim == 1:
                assert np.array_equal(fa, fb)
            else:
                for i in range(0, n, 37):
                    assert np.array_equal(fa[i, :nn[i]].view(np.uint8), fb[i, :nn[i]].view(np.uint8))
    # the step as a graph: rebuild and evaluation in one capture, replayed on rewritten coordinates
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        free.step(coords)                                          # warm-up on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    with torch.cuda.graph(graph):
        free.step(coords)
    for it, alpha in enumerate((0.4, -1.1, 0.9, 0.0)):
        coords.copy_(base + alpha * d)
        want = [t.clone() for t in sync.step(coords)]              # eager work between the replays
        sync.check()
        graph.replay()
        torch.cuda.synchronize()
        for a, b in zip((free.etot, free.force, free.virial), want):
            assert torch.equal(a, b), "replay %d" % it
    free.check()


def test_sync_free_build_flags_a_box_that_outgrew_its_bound(oracle):
    """Atoms that spread far beyond the bin box of the last synchronised build: the sync-free build leaves the
    lists empty and flags it (no kernel indexes beyond the bound), check() says so, and the next rebuild
    synchronises again and is right."""
    import torch
    from ai2pot_amd import _lib
    from ai2pot_amd.calculator import NepCalculator
    lat, pos, ty, _ = _md_inputs(5, 81)
    n = pos.shape[0]
    m = synth.nep_model(rmax_radial=6.0, rmax_angular=4.0)
    dev = "cuda:0"
    calc = NepCalculator(m, n, lat, ty, umax=96, dtype=torch.float32, device=dev, path="segments", sync_free=True)
    ref = NepCalculator(m, n, lat, ty, umax=96, dtype=torch.float32, device=dev, path="segments")
    base = torch.from_numpy(pos.astype(np.float32)).to(dev)
    calc.step(base)
    calc.check()
    far = base.clone()
    far[::2] += torch.tensor([4.0 * float(lat[0][0]), 0.0, 0.0], device=dev)   # half of the atoms four cells away
    calc.step(far)
    with pytest.raises(_lib.A2PError) as err:
        calc.check()
    assert err.value.code == _lib.A2P_ERR_GRID
    got = [t.clone() for t in calc.step(far)]                     # synchronised again, bound renewed
    calc.check()
    want = [t.clone() for t in ref.step(far)]
    ref.check()
    for a, b in zip(got, want):
        assert torch.equal(a, b)
    got = [t.clone() for t in calc.step(far)]                     # and sync-free from here on
    calc.check()
    for a, b in zip(got, want):
        assert torch.equal(a, b)


def test_calls_on_two_streams_do_not_overlap(oracle):
    """The library's workspace is shared by all calls on a device: when the stream changes between calls the library
    synchronises the device first, so two streams used in turn give the results of the same calls made one after the
    other on one stream."""
    import torch
    from ai2pot_amd import ops
    from test_gpu_nep import _model_to_device
    m = synth.nep_model(rmax_radial=6.0, rmax_angular=4.0)
    md = _model_to_device(m, torch.float32)
    cases = []
    for reps, seed in ((6, 91), (5, 93)):
        lat, pos = synth.fcc_cell(reps, 4.6, 0.15, seed)
        ty = synth.rng_randint(seed + 1, pos.shape[0], 3)
        nb = synth.pack_batch([oracle.nblist(lat.astype(np.float32), ty, pos.astype(np.float32), 6.0, 100)])
        d = to_device(nb, torch.float32)
        cases.append((m["chebyshev_size"], m["n_radial_basis"], m["n_angular_basis"], m["l_max"], md["coeffs"], md["w0"],
                      md["b0"], md["w1"], md["type_bias"], d["binum"], d["bilist"], d["bnumneigh"], d["bfirstneigh"],
                      d["brcs"], d["btypes"], md["type_map"], 0, m["rmax_radial"], m["rmax_angular"], md["q_scaler"]))
    want = [[t.clone() for t in ops.nepToEFVOp(*a, validate=False)] for a in cases]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    for it in range(4):
        got = []
        for a, s in zip(cases, streams):
            with torch.cuda.stream(s):
                got.append(ops.nepToEFVOp(*a, validate=False))      # no synchronisation by the caller in between
        torch.cuda.synchronize()
        for g, w in zip(got, want):
            for x, y in zip(g, w):
                assert torch.equal(x, y), "round %d" % it
