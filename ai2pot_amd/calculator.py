"""Device-resident molecular-dynamics step: neighbour-list rebuild followed by NEP energy /
force / virial, with every buffer allocated once.

This is the GPU counterpart of the reference's inference call stack
(ai2pot/models/potential_utils.py:217-268 -> ai2pot/utils/usepot.py:76-97 ->
nblist.find_info4mlff -> ai2pot/models/nep/nep.py:298-357 -> torch.ops.nep.nepToEFVOp), minus
the host round trip: positions stay in HBM, the padded 7-tensor neighbour contract is
produced and consumed on the device.
"""
import ctypes

import numpy as np
import torch

from . import _lib

_c = ctypes


def _vp(t):
    return _c.c_void_p(0 if t is None else t.data_ptr())


class NepCalculator:
    """Holds one NEP model and the neighbour buffers of one structure size."""

    def __init__(self, model, natoms, lattice, types, umax=200, rcut=None, pbc=(True, True, True),
                 sort=False, dtype=torch.float32, device="cuda:0", places_from_list=None, path="auto",
                 padded=True, reorder_every=64, sync_free=False):
        """path: "gather" evaluates energy, forces and virial on compact lists cut by the list build (pairs
        inside the angular cutoff handed to the neighbour through claimed slots, radial pairs by gather; common
        model shapes, unsorted rows, umax % 8 == 0); "segments" scatters pair derivatives into reduction
        segments from the padded arrays (any model shape); "auto" takes the gather when it applies.
        padded=False (gather only) skips the padded firstneigh / rcs arrays: the step then produces
        energy, forces and virial alone.  reorder_every: the gather path processes the atoms along a
        space-filling curve; the order is a locality hint only (results do not depend on it beyond
        rounding), so it is recomputed every reorder_every rebuilds and kept in between; reorder_every=0 processes the
        atoms in the caller's order (for inputs that are already ordered in space: a crystal written cell by cell, atoms
        kept sorted by the MD code), which makes the per-atom arrays and the padded rows sequential.
        sync_free: after the first rebuild (which synchronises), later rebuilds size their bin grid from that build's
        bound and never wait for the stream (a2p_nblist_sync_free); the step can then be captured into a HIP graph.
        If the atoms spread beyond the bound, check() raises and the next rebuild synchronises again."""
        self.device = torch.device(device)
        self.dtype = dtype
        self.n = int(natoms)
        self.umax = int(umax)
        self.sort = bool(sort)
        self.m = model
        self.rcut = float(rcut if rcut is not None else model["rmax_radial"])   # nep.py:66
        npdt = np.float32 if dtype == torch.float32 else np.float64
        self.lattice = np.ascontiguousarray(lattice, npdt).reshape(9)
        self.pbc = np.ascontiguousarray([1 if p else 0 for p in pbc], np.int32)
        dev = self.device
        f = lambda a: torch.from_numpy(np.ascontiguousarray(a, np.float64)).to(dtype).to(dev)
        self.coeffs, self.w0, self.b0, self.w1 = f(model["coeffs"]), f(model["w0"]), f(model["b0"]), f(model["w1"])
        self.bias, self.q_scaler = f(model["type_bias"]), f(model["q_scaler"])
        self.ntypes = int(np.asarray(model["type_map"]).size)
        self.H = self.w1.numel() // self.ntypes
        self.types = torch.from_numpy(np.ascontiguousarray(types, np.int32)).to(dev)
        n, U = self.n, self.umax
        i32 = dict(dtype=torch.int32, device=dev)
        self.binum = torch.full((1,), n, **i32)
        self.ilist = torch.empty(n, **i32)
        self.numneigh = torch.empty(n, **i32)
        self.firstneigh = torch.empty((n, U), **i32)
        self.rcs = torch.empty((n, U, 3), dtype=dtype, device=dev)
        self.types_out = torch.empty(n, **i32)
        self.etot = torch.empty(1, dtype=dtype, device=dev)
        self.force = torch.empty((n, 3), dtype=dtype, device=dev)
        self.virial = torch.empty(9, dtype=dtype, device=dev)
        L = _lib.lib()
        f32 = dtype == torch.float32
        self._nbl_build = L.a2p_nblist_build_f32 if f32 else L.a2p_nblist_build_f64
        self._nbl_update = L.a2p_nblist_update_f32 if f32 else L.a2p_nblist_update_f64
        self._have_list = False
        self._nbl_ranked = L.a2p_nblist_build_ranked_f32 if f32 else L.a2p_nblist_build_ranked_f64
        self._efv = L.a2p_nep_efv_ranked_f32 if f32 else L.a2p_nep_efv_ranked_f64
        # Places of the pairs in their targets' reduction segments: an evaluation that is given them
        # needs no atomics.  With places_from_list the list build claims them (unsorted rows only).
        # Otherwise a list that is evaluated a second time is probably kept for a while (a skin):
        # that evaluation records the places (which costs about a sixth more than a plain call), the
        # following ones use them (a seventh less).
        # (the claims cost the list build what they save the first evaluation: worth it only for a
        # list that is evaluated several times, hence off by default)
        self.places_from_list = bool(places_from_list)
        if self.places_from_list and self.sort:
            raise ValueError("places_from_list needs sort=False")
        L.a2p_nblist_compact_bytes.restype = _c.c_size_t
        elem = _c.c_int(4 if f32 else 8)
        can_gather = (not self.sort and not self.places_from_list and
                      self.umax * (16 if f32 else 28) * 4 <= 32 * 1024 and      # a row per wavefront in LDS
                      L.a2p_nblist_compact_bytes(_c.c_int(n), _c.c_int(U), elem) > 0 and
                      L.a2p_nep_efv_compact_supported(_c.c_int(model["chebyshev_size"]), _c.c_int(model["n_radial_basis"]),
                                                      _c.c_int(model["n_angular_basis"]), _c.c_int(model["l_max"]),
                                                      _c.c_int(self.H), _c.c_int(self.ntypes), elem) == 1)
        if path not in ("auto", "gather", "segments"):
            raise ValueError("path must be auto, gather or segments")
        if path == "gather" and not can_gather:
            raise ValueError("the gather path does not cover this model shape / list options")
        # "auto": the gather kernels give every atom a thread and want tens of thousands of them; small
        # systems stay with the lane-group kernel of the segment path
        self.path = "gather" if (can_gather and (path == "gather" or (path == "auto" and self.n >= 32768))) else "segments"
        self.padded = bool(padded) or self.path != "gather"
        self.input_order = int(reorder_every) == 0
        self.reorder_every = max(1, int(reorder_every))
        self.sync_free = bool(sync_free)
        self._resync = False
        self._builds = 0
        if self.path == "gather":
            nbytes = L.a2p_nblist_compact_bytes(_c.c_int(n), _c.c_int(U), elem)
            self.compact = torch.empty(nbytes, dtype=torch.uint8, device=dev)
            if self.input_order:
                # the processing order is the first array of the buffer (csrc/compact_list.h): the caller's own
                # order goes in once and every build is told to keep it
                self.compact[:4 * n].view(torch.int32).copy_(torch.arange(n, dtype=torch.int32, device=dev))
            self._nbl_compact = L.a2p_nblist_build_compact_f32 if f32 else L.a2p_nblist_build_compact_f64
            self._efv_compact = L.a2p_nep_efv_compact_f32 if f32 else L.a2p_nep_efv_compact_f64
            if not self.padded:
                self.ilist = self.numneigh = self.firstneigh = self.rcs = self.types_out = None
        self.rank = None
        self.incoming = None
        self._evals = 0          # evaluations of the current list
        self._places = False     # rank / incoming describe the current list
        if self.places_from_list:
            self._alloc_places()

    def _alloc_places(self):
        if self.rank is None:
            i32 = dict(dtype=torch.int32, device=self.device)
            self.rank = torch.empty((self.n, self.umax), **i32)
            self.incoming = torch.empty(self.n, **i32)

    def rebuild(self, coords, stream):
        before = _lib.lib().a2p_nblist_sync_free(_c.c_int(1 if (self.sync_free and not self._resync) else 0))
        self._resync = False
        try:
            self._rebuild(coords, stream)
        finally:
            _lib.lib().a2p_nblist_sync_free(_c.c_int(before))

    def _rebuild(self, coords, stream):
        # after the first build the list buffers hold a valid list: later builds write each row
        # only as far as its old or new length reaches
        if self.path == "gather":
            m = self.m
            # the processing order is never recomputed inside a graph capture (a library sort would be recorded)
            capturing = torch.cuda.is_current_stream_capturing()
            rc = self._nbl_compact(self.lattice.ctypes.data_as(_c.c_void_p), _vp(self.types), _vp(coords),
                                   _c.c_int(self.n), _c.c_double(self.rcut), _c.c_int(self.umax), _c.c_int(1),
                                   self.pbc.ctypes.data_as(_c.c_void_p),
                                   _c.c_int((1 if (self._have_list and self.padded) else 0) |
                                            (2 if (self.input_order or
                                                   (self._have_list and (self._builds % self.reorder_every or capturing)))
                                             else 0)),
                                   _c.c_double(m["rmax_radial"]), _c.c_double(m["rmax_angular"]),
                                   _vp(self.ilist), _vp(self.numneigh), _vp(self.firstneigh), _vp(self.rcs),
                                   _vp(self.types_out), _vp(self.compact), stream)
        elif self.places_from_list:
            rc = self._nbl_ranked(self.lattice.ctypes.data_as(_c.c_void_p), _vp(self.types), _vp(coords),
                                  _c.c_int(self.n), _c.c_double(self.rcut), _c.c_int(self.umax), _c.c_int(1),
                                  self.pbc.ctypes.data_as(_c.c_void_p), _c.c_int(1 if self._have_list else 0),
                                  _vp(self.ilist), _vp(self.numneigh), _vp(self.firstneigh), _vp(self.rcs),
                                  _vp(self.types_out), _vp(self.rank), _vp(self.incoming), None, stream)
        else:
            fn = self._nbl_update if self._have_list else self._nbl_build
            rc = fn(self.lattice.ctypes.data_as(_c.c_void_p), _vp(self.types), _vp(coords),
                    _c.c_int(self.n), _c.c_double(self.rcut), _c.c_int(self.umax), _c.c_int(1),
                    self.pbc.ctypes.data_as(_c.c_void_p), _c.c_int(1 if self.sort else 0),
                    _vp(self.ilist), _vp(self.numneigh), _vp(self.firstneigh), _vp(self.rcs),
                    _vp(self.types_out), None, stream)
        self._have_list = rc == 0
        self._builds += 1
        self._places = False
        _lib.check(rc)
        self._places = self.places_from_list
        self._evals = 0

    def evaluate(self, stream):
        m = self.m
        if self.path == "gather":
            rc = self._efv_compact(_c.c_int(m["chebyshev_size"]), _c.c_int(m["n_radial_basis"]),
                                   _c.c_int(m["n_angular_basis"]), _c.c_int(m["l_max"]), _c.c_int(self.H),
                                   _c.c_int(self.ntypes), _vp(self.coeffs), _vp(self.w0), _vp(self.b0), _vp(self.w1),
                                   _vp(self.bias), _vp(self.q_scaler), _c.c_double(m["rmax_radial"]),
                                   _c.c_double(m["rmax_angular"]), _c.c_int(self.n), _c.c_int(self.umax),
                                   _vp(self.types), _vp(self.compact), _vp(self.etot), _vp(self.force),
                                   _vp(self.virial), stream)
            _lib.check(rc)
            self._evals += 1
            return
        ranked = self._places or self._evals >= 1
        if ranked:
            self._alloc_places()
        rc = self._efv(_c.c_int(m["chebyshev_size"]), _c.c_int(m["n_radial_basis"]),
                       _c.c_int(m["n_angular_basis"]), _c.c_int(m["l_max"]), _c.c_int(self.H),
                       _c.c_int(self.ntypes), _vp(self.coeffs), _vp(self.w0), _vp(self.b0), _vp(self.w1),
                       _vp(self.bias), _vp(self.q_scaler), _c.c_double(m["rmax_radial"]),
                       _c.c_double(m["rmax_angular"]), _c.c_int(1), _c.c_int(self.n), _c.c_int(self.umax),
                       _c.c_int(0), _vp(self.binum), _vp(self.ilist), _vp(self.numneigh),
                       _vp(self.firstneigh), _vp(self.rcs), _vp(self.types_out), _vp(self.rank) if ranked else None,
                       _vp(self.incoming) if ranked else None, _c.c_int(1 if self._places else 0),
                       _vp(self.etot), _vp(self.force), _vp(self.virial), None, stream)
        _lib.check(rc)
        self._places = ranked
        self._evals += 1

    def step(self, coords):
        """coords: [N, 3] Cartesian tensor on the device.  Returns (E[1], F[N,3], V[9]) views of
        the calculator's own output buffers (overwritten by the next step)."""
        stream = _c.c_void_p(torch.cuda.current_stream(self.device).cuda_stream)
        self.rebuild(coords, stream)
        self.evaluate(stream)
        return self.etot, self.force, self.virial

    def check(self):
        """Raise if any kernel since the last check flagged a contract violation (synchronises)."""
        try:
            _lib.check_status(torch.cuda.current_stream(self.device).cuda_stream)
        except _lib.A2PError as ex:
            if ex.code == _lib.A2P_ERR_GRID:
                self._resync = True          # the next rebuild reads the extents back and renews the bound
                self._have_list = False
            raise
