"""Host-side mirror of the reference's operator interface for the energy / force / virial
path: same operator names, positional arguments, output lists and error conditions as
``torch.ops.nep.*``, ``torch.ops.mtpr.*`` and ``torch.ops.fvt.*`` of the reference
(source/descriptor/nep/bind/nep_bind.cc, source/descriptor/mtpr/bind/mtpr_bind.cc,
source/fvt/bind/fvt_sr_op_bind.cc).  Tensors are torch tensors on a HIP device; torch only
provides memory and the current stream, the compute is the C ABI of libai2pot_hip.so.
"""
import ctypes

import torch

from . import _lib

_c = ctypes


def _ptr(t):
    return _c.c_void_p(0 if t is None else t.data_ptr())


def _stream(device):
    return _c.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def _req(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def _check_float(name, t, dtype, device):
    _req(isinstance(t, torch.Tensor), "%s must be a tensor" % name)
    _req(t.dtype == dtype, "%s must have dtype %s (the dtype of brcs), got %s" % (name, dtype, t.dtype))
    _req(t.device == device, "%s must be on %s (the device of brcs), got %s" % (name, device, t.device))
    _req(t.is_contiguous(), "%s must be contiguous" % name)


def _check_int(name, t, device):
    _req(isinstance(t, torch.Tensor), "%s must be a tensor" % name)
    _req(t.dtype == torch.int32, "%s must have dtype int32, got %s" % (name, t.dtype))
    _req(t.device == device, "%s must be on %s (the device of brcs), got %s" % (name, device, t.device))
    _req(t.is_contiguous(), "%s must be contiguous" % name)


def _batch_shapes(binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, nghost):
    _req(brcs.dim() == 4 and brcs.shape[3] == 3, "brcs must have shape [B, P, U, 3]")
    B, P, U, _ = brcs.shape
    _req(tuple(bfirstneigh.shape) == (B, P, U), "bfirstneigh must have shape [B, P, U]")
    _req(tuple(bilist.shape) == (B, P), "bilist must have shape [B, P]")
    _req(tuple(bnumneigh.shape) == (B, P), "bnumneigh must have shape [B, P]")
    _req(tuple(binum.shape) == (B,), "binum must have shape [B]")
    _req(tuple(btypes.shape) == (B, P + nghost), "btypes must have shape [B, P + nghost]")
    return B, P, U


def _validate_batch(binum, bnumneigh, U, P):
    """Checks the reference leaves to asserts or to luck.  One device->host sync."""
    if binum.numel() == 0 or bnumneigh.numel() == 0:
        return
    max_inum, max_nn = torch.stack([binum.max(), bnumneigh.max()]).tolist()
    _req(max_inum <= P, "binum (%d) exceeds natoms_pad (%d)" % (max_inum, P))
    _req(max_nn <= U, "a neighbour count (%d) exceeds umax_num_neigh_atoms (%d)" % (max_nn, U))


# --------------------------------------------------------------------------------------------
# NEP  (source/descriptor/nep/bind/nep_bind.cc:26-135, 278-311)
# --------------------------------------------------------------------------------------------
def _nep_call(want_virial, want_desc, chebyshev_size, n_radial_basis, n_angular_basis, l_max, coeffs,
              w0, b0, w1, type_bias, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, type_map,
              nghost, rmax_radial, rmax_angular, q_scaler, validate=True):
    _req(isinstance(brcs, torch.Tensor) and brcs.is_cuda,
         "brcs must be a tensor on a HIP device: this build has no CPU path")
    dtype, device = brcs.dtype, brcs.device
    _req(dtype in (torch.float32, torch.float64), "brcs must be float32 or float64")
    _req(brcs.is_contiguous(), "brcs must be contiguous")
    for name, t in (("coeffs", coeffs), ("w0", w0), ("b0", b0), ("w1", w1), ("type_bias", type_bias)):
        _check_float(name, t, dtype, device)
    for name, t in (("binum", binum), ("bilist", bilist), ("bnumneigh", bnumneigh),
                    ("bfirstneigh", bfirstneigh), ("btypes", btypes)):
        _check_int(name, t, device)
    nghost = int(nghost)
    B, P, U = _batch_shapes(binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, nghost)
    ntypes = int(type_map.numel())                       # nepOp.cc:978-981
    _req(ntypes > 0, "type_map is empty")
    _req(0 <= l_max <= 4, "l_max must be in [0, 4]")     # nep.py:50 / nep_utilities.h:46
    H = w1.numel() // ntypes
    D = n_radial_basis + n_angular_basis * l_max if l_max > 0 else n_radial_basis
    _req(w0.numel() == ntypes * H * D, "w0 has %d elements, expected ntypes*H*D = %d"
         % (w0.numel(), ntypes * H * D))
    _req(b0.numel() == ntypes * H and type_bias.numel() == ntypes, "b0 / type_bias size mismatch")
    _req(coeffs.numel() == ntypes * ntypes * (n_radial_basis + n_angular_basis) * chebyshev_size,
         "coeffs size mismatch")
    if want_desc:
        q_scaler_t = torch.ones(D, dtype=dtype, device=device)
    else:
        _check_float("q_scaler", q_scaler, dtype, device)
        _req(q_scaler.numel() == D, "q_scaler must have %d elements" % D)
        q_scaler_t = q_scaler
    if validate:
        _validate_batch(binum, bnumneigh, U, P)

    etot = force = virial = desc = None
    if want_desc:
        desc = torch.zeros((B, P, D), dtype=dtype, device=device)
    else:
        etot = torch.zeros((B,), dtype=dtype, device=device)
        force = torch.zeros((B, P + nghost, 3), dtype=dtype, device=device)
        if want_virial:
            virial = torch.zeros((B, 9), dtype=dtype, device=device)
    L = _lib.lib()
    fn = L.a2p_nep_efv_f32 if dtype == torch.float32 else L.a2p_nep_efv_f64
    with torch.cuda.device(device):
        rc = fn(_c.c_int(chebyshev_size), _c.c_int(n_radial_basis), _c.c_int(n_angular_basis),
                _c.c_int(l_max), _c.c_int(H), _c.c_int(ntypes), _ptr(coeffs), _ptr(w0), _ptr(b0),
                _ptr(w1), _ptr(type_bias), _ptr(q_scaler_t), _c.c_double(rmax_radial),
                _c.c_double(rmax_angular), _c.c_int(B), _c.c_int(P), _c.c_int(U), _c.c_int(nghost),
                _ptr(binum), _ptr(bilist), _ptr(bnumneigh), _ptr(bfirstneigh), _ptr(brcs),
                _ptr(btypes), _ptr(etot), _ptr(force), _ptr(virial), _ptr(desc), _stream(device))
        _lib.check(rc)
        if validate:
            _lib.check_status(torch.cuda.current_stream(device).cuda_stream)
    return etot, force, virial, desc


def _no_zbl(zbl_rmax):
    _req(float(zbl_rmax) == 0.0, "the ZBL correction (zbl_rmax > 0) is not implemented in this build")


def nepToEFVOp(chebyshev_size, n_radial_basis, n_angular_basis, l_max, coeffs, w0, b0, w1, type_bias,
               binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, type_map, nghost, rmax_radial,
               rmax_angular, q_scaler, zbl_rmax=0.0, zbl_rmin=0.0, zbl_cks=None, zbl_dks=None,
               validate=True):
    """[E[B], F[B, P+nghost, 3], V[B, 9]]; nep_bind.cc:81-135, nepOp.cc:947-1284."""
    _no_zbl(zbl_rmax)
    e, f, v, _ = _nep_call(True, False, chebyshev_size, n_radial_basis, n_angular_basis, l_max, coeffs,
                           w0, b0, w1, type_bias, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes,
                           type_map, nghost, rmax_radial, rmax_angular, q_scaler, validate)
    return [e, f, v]


def nepToEFOp(chebyshev_size, n_radial_basis, n_angular_basis, l_max, coeffs, w0, b0, w1, type_bias,
              binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, type_map, nghost, rmax_radial,
              rmax_angular, q_scaler, zbl_rmax=0.0, zbl_rmin=0.0, zbl_cks=None, zbl_dks=None,
              validate=True):
    """[E[B], F[B, P+nghost, 3]]; nep_bind.cc:26-79."""
    _no_zbl(zbl_rmax)
    e, f, _, _ = _nep_call(False, False, chebyshev_size, n_radial_basis, n_angular_basis, l_max, coeffs,
                           w0, b0, w1, type_bias, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes,
                           type_map, nghost, rmax_radial, rmax_angular, q_scaler, validate)
    return [e, f]


def nepToDescriptorsOp(chebyshev_size, n_radial_basis, n_angular_basis, l_max, coeffs, binum, bilist,
                       bnumneigh, bfirstneigh, brcs, btypes, type_map, nghost, rmax_radial,
                       rmax_angular, validate=True):
    """[descriptors[B, P, D]]; nep_bind.cc:278-311."""
    dtype, device = brcs.dtype, brcs.device
    ntypes = int(type_map.numel())
    D = n_radial_basis + n_angular_basis * l_max if l_max > 0 else n_radial_basis
    # the descriptor-only call does not use the network: one zero neuron per species
    z = lambda *s: torch.zeros(s, dtype=dtype, device=device)
    _, _, _, d = _nep_call(False, True, chebyshev_size, n_radial_basis, n_angular_basis, l_max, coeffs,
                           z(ntypes * D), z(ntypes), z(ntypes), z(ntypes), binum, bilist, bnumneigh,
                           bfirstneigh, brcs, btypes, type_map, nghost, rmax_radial, rmax_angular, None,
                           validate)
    return [d]
