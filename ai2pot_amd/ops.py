"""Host-side mirror of the reference's operator interface for the energy / force / virial
path: same operator names, positional arguments, output lists and error conditions as
``torch.ops.nep.*``, ``torch.ops.mtpr.*`` and ``torch.ops.fvt.*`` of the reference
(source/descriptor/nep/bind/nep_bind.cc, source/descriptor/mtpr/bind/mtpr_bind.cc,
source/fvt/bind/fvt_sr_op_bind.cc).  Tensors are torch tensors on a HIP device; torch only
provides memory and the current stream, the compute is the C ABI of libai2pot_hip.so.
"""
import ctypes
import os

import torch

from . import _lib

_c = ctypes


def _ptr(t):
    return _c.c_void_p(0 if t is None else t.data_ptr())


def _stream(device):
    return _c.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def _new_output(shape, dtype, device, written):
    """An output tensor of an operator whose library call writes every element (written = the batch is not empty):
    uninitialised memory, no fill kernel per output per call.  AI2POT_POISON_OUTPUTS=1 fills it with NaN instead, so
    that an element the library leaves out shows."""
    if not written:
        return torch.zeros(shape, dtype=dtype, device=device)
    if os.environ.get("AI2POT_POISON_OUTPUTS") == "1":
        return torch.full(shape, float("nan"), dtype=dtype, device=device)
    return torch.empty(shape, dtype=dtype, device=device)


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


def _status_or_retry(call, B, P, U, nghost, binum, bnumneigh, bfirstneigh, device):
    """Reads the device status of a call.  The fast kernels give every atom a reduction segment of
    umax entries, which a list built with one cutoff never exceeds; a list that names an atom more
    often (half lists, ghosts that collect the pairs of several rows) overflows it.  The status then
    says so, and the call is repeated once with segments sized for the list at hand."""
    L = _lib.lib()
    stream = torch.cuda.current_stream(device).cuda_stream
    try:
        _lib.check_status(stream)
        return
    except _lib.A2PError as ex:
        if ex.code != _lib.A2P_ERR_SEGMENT:
            raise
    most = _c.c_int(0)
    _lib.check(L.a2p_pair_incoming_max(_c.c_int(B), _c.c_int(P), _c.c_int(U), _c.c_int(int(nghost)), _ptr(binum),
                                       _ptr(bnumneigh), _ptr(bfirstneigh), _c.byref(most), _stream(device)))
    old = L.a2p_pair_segment_capacity(_c.c_int(most.value))
    try:
        _lib.check(call())
        _lib.check_status(stream)
    finally:
        L.a2p_pair_segment_capacity(_c.c_int(old))


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
              nghost, rmax_radial, rmax_angular, q_scaler, validate=True, l_4body=0, l_5body=0):
    _req(isinstance(brcs, torch.Tensor) and brcs.is_cuda,
         "brcs must be a tensor on a HIP device: this build has no CPU path")
    dtype, device = brcs.dtype, brcs.device
    _req(dtype in (torch.float32, torch.float64), "brcs must be float32 or float64")
    _req(brcs.is_contiguous(), "brcs must be contiguous")
    many_body = bool(l_4body or l_5body)
    _req(l_4body in (0, 2) and l_5body in (0, 1), "l_4body must be 0 or 2, l_5body 0 or 1")
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
    num_l = l_max + (1 if l_4body else 0) + (1 if l_5body else 0)
    _req(not many_body or l_max >= max(l_4body, l_5body), "the four-body term needs l_max >= 2, the five-body term l_max >= 1")
    D = n_radial_basis + n_angular_basis * num_l if l_max > 0 else n_radial_basis
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
        # the library writes every element of the three outputs (forces are zeroed on entry)
        new = torch.empty if B * P > 0 else torch.zeros
        etot = new((B,), dtype=dtype, device=device)
        force = new((B, P + nghost, 3), dtype=dtype, device=device)
        if want_virial:
            virial = new((B, 9), dtype=dtype, device=device)
    L = _lib.lib()
    if many_body:
        fn = L.a2p_nep_efv_manybody_f32 if dtype == torch.float32 else L.a2p_nep_efv_manybody_f64
        lead = (_c.c_int(l_max), _c.c_int(l_4body), _c.c_int(l_5body))
    else:
        fn = L.a2p_nep_efv_f32 if dtype == torch.float32 else L.a2p_nep_efv_f64
        lead = (_c.c_int(l_max),)
    with torch.cuda.device(device):
        call = lambda: fn(_c.c_int(chebyshev_size), _c.c_int(n_radial_basis), _c.c_int(n_angular_basis),
                *lead, _c.c_int(H), _c.c_int(ntypes), _ptr(coeffs), _ptr(w0), _ptr(b0),
                _ptr(w1), _ptr(type_bias), _ptr(q_scaler_t), _c.c_double(rmax_radial),
                _c.c_double(rmax_angular), _c.c_int(B), _c.c_int(P), _c.c_int(U), _c.c_int(nghost),
                _ptr(binum), _ptr(bilist), _ptr(bnumneigh), _ptr(bfirstneigh), _ptr(brcs),
                _ptr(btypes), _ptr(etot), _ptr(force), _ptr(virial), _ptr(desc), _stream(device))
        _lib.check(call())
        if validate:
            _status_or_retry(call, B, P, U, nghost, binum, bnumneigh, bfirstneigh, device)
    return etot, force, virial, desc


def _zbl_esites(zbl_rmax, zbl_rmin, zbl_cks, zbl_dks, type_map, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes,
                nghost, validate):
    """Per-row ZBL energies [B, P] (half of every pair energy of the row's centre atom;
    GroupZBL::correct_e_sites, correction/include/zbl.h:625-685), or None when zbl_rmax == 0.  The site-energy
    operators add them to the model's rows, so that the rows sum to the energy of the E/F/V operators.  Parity
    unpinned by a run of the reference's operator: its CPU code adds the term first and then assigns the rows
    (linearMtp.h:598), which loses it; the term itself is pinned to correct_e_sites through the oracle."""
    if float(zbl_rmax) == 0.0:
        return None
    dtype, device = brcs.dtype, brcs.device
    ntypes = int(type_map.numel())
    for name, t in (("zbl_cks", zbl_cks), ("zbl_dks", zbl_dks)):
        _check_float(name, t, dtype, device)
        _req(t.numel() == ntypes * ntypes * 4, "%s must have ntypes*ntypes*4 = %d elements" % (name, ntypes * ntypes * 4))
    tm = type_map.to(device=device, dtype=torch.int32).contiguous()
    B, P, U = _batch_shapes(binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, int(nghost))
    out = torch.zeros((B, P), dtype=dtype, device=device)
    L = _lib.lib()
    fn = L.a2p_zbl_esites_f32 if dtype == torch.float32 else L.a2p_zbl_esites_f64
    with torch.cuda.device(device):
        rc = fn(_c.c_double(zbl_rmax), _c.c_double(zbl_rmin), _ptr(zbl_cks), _ptr(zbl_dks), _c.c_int(ntypes), _ptr(tm),
                _c.c_int(B), _c.c_int(P), _c.c_int(U), _c.c_int(int(nghost)), _ptr(binum), _ptr(bilist),
                _ptr(bnumneigh), _ptr(bfirstneigh), _ptr(brcs), _ptr(btypes), _ptr(out), _stream(device))
        _lib.check(rc)
        if validate:
            _lib.check_status(torch.cuda.current_stream(device).cuda_stream)
    return out


def _zbl_add(zbl_rmax, zbl_rmin, zbl_cks, zbl_dks, type_map, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes,
             nghost, etot, force, virial, validate):
    """Adds the ZBL pair repulsion onto a model's E/F/V when zbl_rmax > 0, as the reference's
    operators do on the device (correction/gpu/include/zbl.cuh:422-620; e.g. nepOp.cc:1086-1110).
    The pair formulas are pinned to the reference's PairZBL member functions; the composition per centre
    atom (halves of the pair energy, force on the centre only) is PARITY UNPINNED by a run of the reference:
    its CPU GroupZBL::correct_efv has the force and virial calls commented out, so only the device source
    can be followed."""
    if float(zbl_rmax) == 0.0:
        return
    dtype, device = brcs.dtype, brcs.device
    ntypes = int(type_map.numel())
    for name, t in (("zbl_cks", zbl_cks), ("zbl_dks", zbl_dks)):
        _check_float(name, t, dtype, device)
        _req(t.numel() == ntypes * ntypes * 4, "%s must have ntypes*ntypes*4 = %d elements" % (name, ntypes * ntypes * 4))
    tm = type_map.to(device=device, dtype=torch.int32).contiguous()
    B, P, U = _batch_shapes(binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, int(nghost))
    L = _lib.lib()
    fn = L.a2p_zbl_correct_f32 if dtype == torch.float32 else L.a2p_zbl_correct_f64
    with torch.cuda.device(device):
        rc = fn(_c.c_double(zbl_rmax), _c.c_double(zbl_rmin), _ptr(zbl_cks), _ptr(zbl_dks), _c.c_int(ntypes), _ptr(tm),
                _c.c_int(B), _c.c_int(P), _c.c_int(U), _c.c_int(int(nghost)), _ptr(binum), _ptr(bilist),
                _ptr(bnumneigh), _ptr(bfirstneigh), _ptr(brcs), _ptr(btypes), _ptr(etot), _ptr(force), _ptr(virial),
                _stream(device))
        _lib.check(rc)
        if validate:
            _lib.check_status(torch.cuda.current_stream(device).cuda_stream)


def _zbl_shift_labels(zbl_rmax, zbl_rmin, zbl_cks, zbl_dks, type_map, binum, bilist, bnumneigh, bfirstneigh, brcs,
                      btypes, nghost, betot_dft, bforce_dft, bvirial_dft, validate):
    """Labels of a loss operator with the ZBL pair repulsion taken out.  The correction does not
    depend on the model parameters, so model + ZBL - label = model - (label - ZBL): the loss, its
    RMSEs and its gradients are those of the operator without ZBL on the shifted labels.  The
    reference adds the correction to E/F/V before the loss and before its gradient (e.g.
    nepOp.cc:2552-2575, 3127-3150).  bvirial_dft may be None (operators without virial labels)."""
    if float(zbl_rmax) == 0.0:
        return betot_dft, bforce_dft, bvirial_dft
    _req(int(nghost) == 0, "the loss operator requires nghost == 0, as the reference does")
    dtype, device = brcs.dtype, brcs.device
    for name, t in (("betot_dft", betot_dft), ("bforce_dft", bforce_dft), ("bvirial_dft", bvirial_dft)):
        if t is not None:
            _check_float(name, t, dtype, device)
    B, P = int(brcs.shape[0]), int(brcs.shape[1])
    e0 = torch.zeros((B,), dtype=dtype, device=device)
    f0 = torch.zeros((B, P, 3), dtype=dtype, device=device)
    v0 = torch.zeros((B, 9), dtype=dtype, device=device) if bvirial_dft is not None else None
    _zbl_add(zbl_rmax, zbl_rmin, zbl_cks, zbl_dks, type_map, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes,
             0, e0, f0, v0, validate)
    _req(betot_dft.numel() == B and bforce_dft.numel() == B * P * 3, "label shapes do not match the batch")
    return (betot_dft.detach().reshape(B) - e0, bforce_dft.detach().reshape(B, P, 3) - f0,
            None if bvirial_dft is None else bvirial_dft.detach().reshape(B, 9) - v0)


def nepToEFVOp(chebyshev_size, n_radial_basis, n_angular_basis, l_max, coeffs, w0, b0, w1, type_bias,
               binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, type_map, nghost, rmax_radial,
               rmax_angular, q_scaler, zbl_rmax=0.0, zbl_rmin=0.0, zbl_cks=None, zbl_dks=None,
               validate=True):
    """[E[B], F[B, P+nghost, 3], V[B, 9]]; nep_bind.cc:81-135, nepOp.cc:947-1284."""
    e, f, v, _ = _nep_call(True, False, chebyshev_size, n_radial_basis, n_angular_basis, l_max, coeffs,
                           w0, b0, w1, type_bias, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes,
                           type_map, nghost, rmax_radial, rmax_angular, q_scaler, validate)
    _zbl_add(zbl_rmax, zbl_rmin, zbl_cks, zbl_dks, type_map, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes,
             nghost, e, f, v, validate)
    return [e, f, v]


def nepToEFVManyBodyOp(chebyshev_size, n_radial_basis, n_angular_basis, l_max, l_4body, l_5body, coeffs, w0, b0, w1,
                       type_bias, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, type_map, nghost, rmax_radial,
                       rmax_angular, q_scaler, want_descriptors=False, validate=True):
    """EXTENSION, no counterpart in the reference (PARITY UNPINNED): nepToEFVOp with one four-body invariant (from
    the l = 2 moments, l_4body = 2) and / or one five-body invariant (l = 1, l_5body = 1) per angular channel, the
    descriptors of a channel ordered l = 1 .. l_max, four-body, five-body, so D = n_radial + n_angular * (l_max +
    [l_4body > 0] + [l_5body > 0]) sets the shapes of w0 and q_scaler.  The reference's operators have radial and
    three-body terms only (nep_bind.cc:81-105); its unfinished draft holds the weights
    (source/descriptor/ace/include/nep_descriptor.h:43-54) and no code that uses them.  Checked by rotation
    invariance, finite differences and the reduction to nepToEFVOp.  Returns [E, F, V], or [descriptors] with
    want_descriptors."""
    if want_descriptors:
        ntypes = int(type_map.numel())
        D = n_radial_basis + n_angular_basis * (l_max + (1 if l_4body else 0) + (1 if l_5body else 0))
        z = lambda *sh: torch.zeros(sh, dtype=brcs.dtype, device=brcs.device)
        _, _, _, d = _nep_call(False, True, chebyshev_size, n_radial_basis, n_angular_basis, l_max, coeffs,
                               z(ntypes * D), z(ntypes), z(ntypes), z(ntypes), binum, bilist, bnumneigh, bfirstneigh,
                               brcs, btypes, type_map, nghost, rmax_radial, rmax_angular, None, validate,
                               l_4body=l_4body, l_5body=l_5body)
        return [d]
    e, f, v, _ = _nep_call(True, False, chebyshev_size, n_radial_basis, n_angular_basis, l_max, coeffs, w0, b0, w1,
                           type_bias, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, type_map, nghost,
                           rmax_radial, rmax_angular, q_scaler, validate, l_4body=l_4body, l_5body=l_5body)
    return [e, f, v]


def nepToEFOp(chebyshev_size, n_radial_basis, n_angular_basis, l_max, coeffs, w0, b0, w1, type_bias,
              binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, type_map, nghost, rmax_radial,
              rmax_angular, q_scaler, zbl_rmax=0.0, zbl_rmin=0.0, zbl_cks=None, zbl_dks=None,
              validate=True):
    """[E[B], F[B, P+nghost, 3]]; nep_bind.cc:26-79."""
    e, f, _, _ = _nep_call(False, False, chebyshev_size, n_radial_basis, n_angular_basis, l_max, coeffs,
                           w0, b0, w1, type_bias, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes,
                           type_map, nghost, rmax_radial, rmax_angular, q_scaler, validate)
    _zbl_add(zbl_rmax, zbl_rmin, zbl_cks, zbl_dks, type_map, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes,
             nghost, e, f, None, validate)
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


def nep_loss_step(e_weight, f_weight, v_weight, betot_dft, bforce_dft, bvirial_dft, chebyshev_size,
                  n_radial_basis, n_angular_basis, l_max, coeffs, w0, b0, w1, type_bias, binum, bilist,
                  bnumneigh, bfirstneigh, brcs, btypes, type_map, nghost, rmax_radial, rmax_angular, q_scaler,
                  want_grad=True, validate=True):
    """Forward and (optionally) the per-structure parameter gradients of the NEP training loss in one
    call.  Returns a dict with bloss[B], rmse[3], energy, force, virial and, with want_grad,
    dcoeffs[B, .], dw0[B, .], db0[B, .], dw1[B, .], dbias[B, ntypes] (flattened parameter layouts)."""
    _req(int(nghost) == 0, "the loss operator requires nghost == 0, as the reference does")
    _req(isinstance(brcs, torch.Tensor) and brcs.is_cuda,
         "brcs must be a tensor on a HIP device: this build has no CPU path")
    dtype, device = brcs.dtype, brcs.device
    _req(dtype in (torch.float32, torch.float64), "brcs must be float32 or float64")
    _req(brcs.is_contiguous(), "brcs must be contiguous")
    for name, t in (("coeffs", coeffs), ("w0", w0), ("b0", b0), ("w1", w1), ("type_bias", type_bias),
                    ("q_scaler", q_scaler)):
        _check_float(name, t, dtype, device)
    for name, t in (("binum", binum), ("bilist", bilist), ("bnumneigh", bnumneigh),
                    ("bfirstneigh", bfirstneigh), ("btypes", btypes)):
        _check_int(name, t, device)
    B, P, U = _batch_shapes(binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, 0)
    ntypes = int(type_map.numel())
    _req(ntypes > 0, "type_map is empty")
    _req(0 <= l_max <= 4, "l_max must be in [0, 4]")
    H = w1.numel() // ntypes
    D = n_radial_basis + n_angular_basis * l_max if l_max > 0 else n_radial_basis
    _req(w0.numel() == ntypes * H * D and b0.numel() == ntypes * H and type_bias.numel() == ntypes and
         q_scaler.numel() == D, "w0 / b0 / type_bias / q_scaler size mismatch")
    _req(coeffs.numel() == ntypes * ntypes * (n_radial_basis + n_angular_basis) * chebyshev_size,
         "coeffs size mismatch")
    for name, t, n_expected in (("betot_dft", betot_dft, B), ("bforce_dft", bforce_dft, B * P * 3),
                                ("bvirial_dft", bvirial_dft, B * 9)):
        _check_float(name, t, dtype, device)
        _req(t.numel() == n_expected, "%s has %d elements, expected %d" % (name, t.numel(), n_expected))
    if validate:
        _validate_batch(binum, bnumneigh, U, P)
    z = lambda *s_: _new_output(s_, dtype, device, B * P > 0)
    out = dict(bloss=z(B), rmse=z(3), energy=z(B), force=z(B, P, 3), virial=z(B, 9))
    if want_grad:
        out.update(dcoeffs=z(B, coeffs.numel()), dw0=z(B, w0.numel()), db0=z(B, b0.numel()),
                   dw1=z(B, w1.numel()), dbias=z(B, ntypes))
    L = _lib.lib()
    fn = L.a2p_nep_loss_f32 if dtype == torch.float32 else L.a2p_nep_loss_f64
    with torch.cuda.device(device):
        call = lambda: fn(_c.c_double(e_weight), _c.c_double(f_weight), _c.c_double(v_weight), _ptr(betot_dft),
                _ptr(bforce_dft), _ptr(bvirial_dft), _c.c_int(chebyshev_size), _c.c_int(n_radial_basis),
                _c.c_int(n_angular_basis), _c.c_int(l_max), _c.c_int(H), _c.c_int(ntypes), _ptr(coeffs), _ptr(w0),
                _ptr(b0), _ptr(w1), _ptr(type_bias), _ptr(q_scaler), _c.c_double(rmax_radial),
                _c.c_double(rmax_angular), _c.c_int(B), _c.c_int(P), _c.c_int(U), _ptr(binum), _ptr(bilist),
                _ptr(bnumneigh), _ptr(bfirstneigh), _ptr(brcs), _ptr(btypes), _ptr(out["bloss"]), _ptr(out["rmse"]),
                _ptr(out["energy"]), _ptr(out["force"]), _ptr(out["virial"]), _ptr(out.get("dcoeffs")),
                _ptr(out.get("dw0")), _ptr(out.get("db0")), _ptr(out.get("dw1")), _ptr(out.get("dbias")),
                _stream(device))
        _lib.check(call())
        if validate:
            _status_or_retry(call, B, P, U, 0, binum, bnumneigh, bfirstneigh, device)
    return out


class _NepToLoss(torch.autograd.Function):
    """Autograd wrapper with the reference's contract (nepOp.cc:2359-2960): gradients flow to coeffs,
    w0, b0, w1 and type_bias only, as grad_output[B] @ dloss/dtheta."""

    @staticmethod
    def forward(ctx, coeffs, w0, b0, w1, type_bias, args):
        (e_w, f_w, v_w, e_dft, f_dft, v_dft, K, n_r, n_a, l_max, binum, bilist, bnumneigh, bfirstneigh, brcs,
         btypes, type_map, nghost, rr, ra, q_scaler, validate) = args
        params = (coeffs, w0, b0, w1, type_bias)
        need = any(p.requires_grad for p in params)
        r = nep_loss_step(e_w, f_w, v_w, e_dft, f_dft, v_dft, K, n_r, n_a, l_max, coeffs.detach(), w0.detach(),
                          b0.detach(), w1.detach(), type_bias.detach(), binum, bilist, bnumneigh, bfirstneigh,
                          brcs, btypes, type_map, nghost, rr, ra, q_scaler, want_grad=need, validate=validate)
        if need:
            # unlike the reference, which recomputes E/F/V in backward, the gradients are produced by
            # the same call and kept
            ctx.save_for_backward(r["dcoeffs"], r["dw0"], r["db0"], r["dw1"], r["dbias"])
        ctx.shapes = tuple(p.shape for p in params)
        ctx.have = need
        rm = r["rmse"]
        return r["bloss"], rm[0:1].clone(), rm[1:2].clone(), rm[2:3].clone()

    @staticmethod
    def backward(ctx, gl, ge, gf, gv):
        if not ctx.have:
            return None, None, None, None, None, None
        return tuple(torch.matmul(gl, g).reshape(sh) for g, sh in zip(ctx.saved_tensors, ctx.shapes)) + (None,)


def nepToLossOp(e_weight, f_weight, v_weight, betot_dft, bforce_dft, bvirial_dft, chebyshev_size,
                n_radial_basis, n_angular_basis, l_max, coeffs, w0, b0, w1, type_bias, binum, bilist, bnumneigh,
                bfirstneigh, brcs, btypes, type_map, nghost, rmax_radial, rmax_angular, q_scaler, zbl_rmax=0.0,
                zbl_rmin=0.0, zbl_cks=None, zbl_dks=None, validate=True):
    """[bloss[B], e_rmse[1], f_rmse[1], v_rmse[1]], differentiable w.r.t. coeffs, w0, b0, w1 and
    type_bias; nep_bind.cc:205-276, nepOp.cc:2359-2960."""
    betot_dft, bforce_dft, bvirial_dft = _zbl_shift_labels(
        zbl_rmax, zbl_rmin, zbl_cks, zbl_dks, type_map, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, nghost,
        betot_dft, bforce_dft, bvirial_dft, validate)
    args = (e_weight, f_weight, v_weight, betot_dft, bforce_dft, bvirial_dft, chebyshev_size, n_radial_basis,
            n_angular_basis, l_max, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, type_map, nghost,
            rmax_radial, rmax_angular, q_scaler, validate)
    return list(_NepToLoss.apply(coeffs, w0, b0, w1, type_bias, args))


def nepToEFLossOp(e_weight, f_weight, betot_dft, bforce_dft, chebyshev_size, n_radial_basis, n_angular_basis,
                  l_max, coeffs, w0, b0, w1, type_bias, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes,
                  type_map, nghost, rmax_radial, rmax_angular, q_scaler, zbl_rmax=0.0, zbl_rmin=0.0, zbl_cks=None,
                  zbl_dks=None, validate=True):
    """[bloss[B], e_rmse[1], f_rmse[1]]: the loss without the virial term; nep_bind.cc:136-203,
    nepOp.cc:2962-3484 (nepLoss.h:139-166 is nepLoss.h:170-209 with v_weight = 0)."""
    betot_dft, bforce_dft, _ = _zbl_shift_labels(
        zbl_rmax, zbl_rmin, zbl_cks, zbl_dks, type_map, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, nghost,
        betot_dft, bforce_dft, None, validate)
    B = int(binum.numel())
    v0 = torch.zeros((B, 9), dtype=brcs.dtype, device=brcs.device)
    args = (e_weight, f_weight, 0.0, betot_dft, bforce_dft, v0, chebyshev_size, n_radial_basis, n_angular_basis,
            l_max, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, type_map, nghost, rmax_radial,
            rmax_angular, q_scaler, validate)
    return list(_NepToLoss.apply(coeffs, w0, b0, w1, type_bias, args))[:3]


# --------------------------------------------------------------------------------------------
# linear MTP  (source/descriptor/mtpr/bind/mtpr_bind.cc:30-457)
# --------------------------------------------------------------------------------------------
_plans = {}
_plans_by_content = {}


def set_ai2pot_path(path):
    """torch.ops.mtpr.set_ai2pot_path (mtpr_bind.cc:31-36): where the MTP templates live."""
    from . import mtp_param
    mtp_param.set_ai2pot_path(path)


def mtpParamOp(mtp_level, device="cpu"):
    """The seven int32 tensors of the reference's mtpParamOp (src/mtpParamOp.cc:25-63):
    [alpha_moments_count, alpha_index_basic, alpha_index_times, alpha_moment_mapping,
    num_mus4moms, mus4moms, nmus]."""
    from . import mtp_param
    t = mtp_param.mtp_param(int(mtp_level))
    f = lambda a: torch.from_numpy(a.astype("int32")).to(device)
    return [torch.tensor(t["alpha_moments_count"], dtype=torch.int32, device=device),
            f(t["alpha_index_basic"]), f(t["alpha_index_times"]), f(t["alpha_moment_mapping"]),
            f(t["num_mus4moms"]), f(t["mus4moms"]), torch.tensor(t["nmus"], dtype=torch.int32, device=device)]


def _mtp_plan(alpha_moments_count, basic_t, times_t, mapping_t, device):
    """Plan handle for a set of table tensors.  The tables are model constants (registered
    buffers in the reference, ai2pot/models/mtp/linear_mtp.py:63-69): they are read back to
    the host once.  Two caches: by storage address, shape and version of the three tensors (the entry
    keeps the tensors alive, so an address cannot come back with other contents while it is cached;
    the oldest entries are dropped first), and by the tables' contents, which owns the plan handles
    (never destroyed: a captured graph may still name one, and distinct tables are few)."""
    key = (device.index, int(alpha_moments_count),
           basic_t.data_ptr(), tuple(basic_t.shape), basic_t._version,
           times_t.data_ptr(), tuple(times_t.shape), times_t._version,
           mapping_t.data_ptr(), tuple(mapping_t.shape), mapping_t._version)
    if key in _plans:
        return _plans[key][:2]
    for name, t in (("alpha_index_basic", basic_t), ("alpha_index_times", times_t),
                    ("alpha_moment_mapping", mapping_t)):
        _req(isinstance(t, torch.Tensor) and t.dtype == torch.int32, "%s must be an int32 tensor" % name)
    _req(basic_t.dim() == 2 and basic_t.shape[1] == 4, "alpha_index_basic must have shape [n, 4]")
    _req(times_t.numel() == 0 or (times_t.dim() == 2 and times_t.shape[1] == 4),
         "alpha_index_times must have shape [n, 4]")
    basic = basic_t.detach().cpu().contiguous().numpy()
    times = times_t.detach().cpu().contiguous().numpy().reshape(-1, 4)
    mapping = mapping_t.detach().cpu().contiguous().numpy()
    content = (device.index, int(alpha_moments_count), basic.shape, basic.tobytes(), times.tobytes(), mapping.tobytes())
    if content not in _plans_by_content:
        handle = _c.c_void_p()
        with torch.cuda.device(device):
            rc = _lib.lib().a2p_mtp_plan_create(
                _c.c_int(int(alpha_moments_count)), _c.c_int(basic.shape[0]), basic.ctypes.data_as(_c.c_void_p),
                _c.c_int(times.shape[0]), times.ctypes.data_as(_c.c_void_p), _c.c_int(mapping.size),
                mapping.ctypes.data_as(_c.c_void_p), _c.byref(handle))
        _lib.check(rc)
        _plans_by_content[content] = (handle, mapping.size)
    while len(_plans) >= 64:
        del _plans[next(iter(_plans))]                     # the oldest address entry; its plan stays with its contents
    _plans[key] = _plans_by_content[content] + ((basic_t, times_t, mapping_t),)
    return _plans[key][:2]


def _mtp_common(coeffs, linear_coeffs, type_bias, alpha_moments_count, alpha_index_basic,
                alpha_index_times, alpha_moment_mapping, nmus, binum, bilist, bnumneigh, bfirstneigh, brcs,
                btypes, type_map, nghost, q_scaler, chebyshev_size, validate):
    _req(isinstance(brcs, torch.Tensor) and brcs.is_cuda,
         "brcs must be a tensor on a HIP device: this build has no CPU path")
    dtype, device = brcs.dtype, brcs.device
    _req(dtype in (torch.float32, torch.float64), "brcs must be float32 or float64")
    _req(brcs.is_contiguous(), "brcs must be contiguous")
    for name, t in (("coeffs", coeffs), ("linear_coeffs", linear_coeffs), ("type_bias", type_bias),
                    ("q_scaler", q_scaler)):
        _check_float(name, t, dtype, device)
    for name, t in (("binum", binum), ("bilist", bilist), ("bnumneigh", bnumneigh),
                    ("bfirstneigh", bfirstneigh), ("btypes", btypes)):
        _check_int(name, t, device)
    nghost = int(nghost)
    B, P, U = _batch_shapes(binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, nghost)
    ntypes = int(type_map.numel())
    _req(ntypes > 0, "type_map is empty")
    plan, n_scalar = _mtp_plan(alpha_moments_count, alpha_index_basic, alpha_index_times,
                               alpha_moment_mapping, device)
    _req(coeffs.numel() == ntypes * ntypes * int(nmus) * int(chebyshev_size), "coeffs size mismatch")
    _req(linear_coeffs.numel() == n_scalar and q_scaler.numel() == n_scalar,
         "linear_coeffs and q_scaler must have alpha_scalar_moments = %d elements" % n_scalar)
    _req(type_bias.numel() == ntypes, "type_bias size mismatch")
    if validate:
        _validate_batch(binum, bnumneigh, U, P)
    return dtype, device, B, P, U, nghost, ntypes, plan, n_scalar


def _mtp_efv(want_virial, chebyshev_size, scaling, coeffs, linear_coeffs, type_bias, alpha_moments_count,
             alpha_index_basic, alpha_index_times, alpha_moment_mapping, nmus, binum, bilist, bnumneigh,
             bfirstneigh, brcs, btypes, type_map, nghost, rmax, rmin, q_scaler, zbl, validate):
    dtype, device, B, P, U, nghost, ntypes, plan, _ = _mtp_common(
        coeffs, linear_coeffs, type_bias, alpha_moments_count, alpha_index_basic, alpha_index_times,
        alpha_moment_mapping, nmus, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, type_map, nghost,
        q_scaler, chebyshev_size, validate)
    new = torch.empty if B * P > 0 else torch.zeros      # the library writes every element of the outputs
    etot = new((B,), dtype=dtype, device=device)
    force = new((B, P + nghost, 3), dtype=dtype, device=device)
    virial = new((B, 9), dtype=dtype, device=device) if want_virial else None
    L = _lib.lib()
    fn = L.a2p_mtp_efv_f32 if dtype == torch.float32 else L.a2p_mtp_efv_f64
    with torch.cuda.device(device):
        call = lambda: fn(plan, _c.c_int(chebyshev_size), _c.c_double(scaling), _ptr(coeffs), _ptr(linear_coeffs),
                _ptr(type_bias), _c.c_int(int(nmus)), _c.c_int(ntypes), _ptr(q_scaler), _c.c_double(rmax),
                _c.c_double(rmin), _c.c_int(B), _c.c_int(P), _c.c_int(U), _c.c_int(nghost), _ptr(binum),
                _ptr(bilist), _ptr(bnumneigh), _ptr(bfirstneigh), _ptr(brcs), _ptr(btypes), _ptr(etot),
                _ptr(force), _ptr(virial), _stream(device))
        _lib.check(call())
        if validate:
            _status_or_retry(call, B, P, U, nghost, binum, bnumneigh, bfirstneigh, device)
    _zbl_add(zbl[0], zbl[1], zbl[2], zbl[3], type_map, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, nghost,
             etot, force, virial, validate)
    return etot, force, virial


def linearMtpToEFVOp(chebyshev_size, scaling, coeffs, linear_coeffs, type_bias, alpha_moments_count,
                     alpha_index_basic, alpha_index_times, alpha_moment_mapping, nmus, binum, bilist,
                     bnumneigh, bfirstneigh, brcs, btypes, type_map, nghost, rmax, rmin, q_scaler,
                     zbl_rmax=0.0, zbl_rmin=0.0, zbl_cks=None, zbl_dks=None, validate=True):
    """[E[B], F[B, P+nghost, 3], V[B, 9]]; mtpr_bind.cc:333-394, linearMtpOp.cc:2834-3180."""
    e, f, v = _mtp_efv(True, chebyshev_size, scaling, coeffs, linear_coeffs, type_bias, alpha_moments_count,
                       alpha_index_basic, alpha_index_times, alpha_moment_mapping, nmus, binum, bilist,
                       bnumneigh, bfirstneigh, brcs, btypes, type_map, nghost, rmax, rmin, q_scaler,
                       (zbl_rmax, zbl_rmin, zbl_cks, zbl_dks), validate)
    return [e, f, v]


def linearMtpToEFOp(chebyshev_size, scaling, coeffs, linear_coeffs, type_bias, alpha_moments_count,
                    alpha_index_basic, alpha_index_times, alpha_moment_mapping, nmus, binum, bilist,
                    bnumneigh, bfirstneigh, brcs, btypes, type_map, nghost, rmax, rmin, q_scaler,
                    zbl_rmax=0.0, zbl_rmin=0.0, zbl_cks=None, zbl_dks=None, validate=True):
    """[E[B], F[B, P+nghost, 3]]; mtpr_bind.cc:396-457."""
    e, f, _ = _mtp_efv(False, chebyshev_size, scaling, coeffs, linear_coeffs, type_bias, alpha_moments_count,
                       alpha_index_basic, alpha_index_times, alpha_moment_mapping, nmus, binum, bilist,
                       bnumneigh, bfirstneigh, brcs, btypes, type_map, nghost, rmax, rmin, q_scaler,
                       (zbl_rmax, zbl_rmin, zbl_cks, zbl_dks), validate)
    return [e, f]


def mtp_loss_step(e_weight, f_weight, v_weight, betot_dft, bforce_dft, bvirial_dft, chebyshev_size, scaling,
                  coeffs, linear_coeffs, type_bias, alpha_moments_count, alpha_index_basic, alpha_index_times,
                  alpha_moment_mapping, nmus, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, type_map,
                  nghost, rmax, rmin, q_scaler, want_grad=True, validate=True):
    """Forward and (optionally) the per-structure parameter gradients of the training loss in
    one call.  Returns a dict with bloss[B], rmse[3], energy, force, virial and, with
    want_grad, dcoeffs[B, ncoef], dlinear[B, S], dbias[B, ntypes]."""
    _req(int(nghost) == 0, "the loss operator requires nghost == 0, as the reference does")
    dtype, device, B, P, U, nghost, ntypes, plan, n_scalar = _mtp_common(
        coeffs, linear_coeffs, type_bias, alpha_moments_count, alpha_index_basic, alpha_index_times,
        alpha_moment_mapping, nmus, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, type_map, nghost,
        q_scaler, chebyshev_size, validate)
    for name, t, shape in (("betot_dft", betot_dft, (B,)), ("bforce_dft", bforce_dft, (B, P, 3)),
                           ("bvirial_dft", bvirial_dft, (B, 9))):
        _check_float(name, t, dtype, device)
        n_expected = 1
        for s_ in shape:
            n_expected *= s_
        _req(t.numel() == n_expected, "%s must have shape %s" % (name, shape))
    ncoef = coeffs.numel()
    z = lambda *s: _new_output(s, dtype, device, B * P > 0)
    out = dict(bloss=z(B), rmse=z(3), energy=z(B), force=z(B, P, 3), virial=z(B, 9))
    if want_grad:
        out.update(dcoeffs=z(B, ncoef), dlinear=z(B, n_scalar), dbias=z(B, ntypes))
    L = _lib.lib()
    fn = L.a2p_mtp_loss_f32 if dtype == torch.float32 else L.a2p_mtp_loss_f64
    with torch.cuda.device(device):
        call = lambda: fn(plan, _c.c_double(e_weight), _c.c_double(f_weight), _c.c_double(v_weight), _ptr(betot_dft),
                _ptr(bforce_dft), _ptr(bvirial_dft), _c.c_int(chebyshev_size), _c.c_double(scaling),
                _ptr(coeffs), _ptr(linear_coeffs), _ptr(type_bias), _c.c_int(int(nmus)), _c.c_int(ntypes),
                _ptr(q_scaler), _c.c_double(rmax), _c.c_double(rmin), _c.c_int(B), _c.c_int(P), _c.c_int(U),
                _ptr(binum), _ptr(bilist), _ptr(bnumneigh), _ptr(bfirstneigh), _ptr(brcs), _ptr(btypes),
                _ptr(out["bloss"]), _ptr(out["rmse"]), _ptr(out["energy"]), _ptr(out["force"]),
                _ptr(out["virial"]), _ptr(out.get("dcoeffs")), _ptr(out.get("dlinear")),
                _ptr(out.get("dbias")), _stream(device))
        _lib.check(call())
        if validate:
            _status_or_retry(call, B, P, U, 0, binum, bnumneigh, bfirstneigh, device)
    return out


class _LinearMtpToLoss(torch.autograd.Function):
    """Autograd wrapper with the reference's contract (linearMtpOp.cc:621-1181, 1184-1765):
    gradients flow to coeffs, linear_coeffs and type_bias only, as grad_output[B] @ dloss/dtheta."""

    @staticmethod
    def forward(ctx, coeffs, linear_coeffs, type_bias, args):
        (e_w, f_w, v_w, e_dft, f_dft, v_dft, K, scaling, n_moms, basic, times, mapping, nmus, binum, bilist,
         bnumneigh, bfirstneigh, brcs, btypes, type_map, nghost, rmax, rmin, q_scaler, validate) = args
        need = coeffs.requires_grad or linear_coeffs.requires_grad or type_bias.requires_grad
        r = mtp_loss_step(e_w, f_w, v_w, e_dft, f_dft, v_dft, K, scaling, coeffs.detach(),
                          linear_coeffs.detach(), type_bias.detach(), n_moms, basic, times, mapping, nmus,
                          binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, type_map, nghost, rmax, rmin,
                          q_scaler, want_grad=need, validate=validate)
        if need:
            # unlike the reference, which recomputes E/F/V in backward, the gradients are produced by
            # the same call and kept
            ctx.save_for_backward(r["dcoeffs"], r["dlinear"], r["dbias"])
        ctx.shapes = (coeffs.shape, linear_coeffs.shape, type_bias.shape)
        ctx.have = need
        rm = r["rmse"]
        return r["bloss"], rm[0:1].clone(), rm[1:2].clone(), rm[2:3].clone()

    @staticmethod
    def backward(ctx, gl, ge, gf, gv):
        if not ctx.have:
            return None, None, None, None
        dc, dl, db = ctx.saved_tensors
        sc, sl, sb = ctx.shapes
        return (torch.matmul(gl, dc).reshape(sc), torch.matmul(gl, dl).reshape(sl),
                torch.matmul(gl, db).reshape(sb), None)


def linearMtpToLossOp(e_weight, f_weight, v_weight, betot_dft, bforce_dft, bvirial_dft, chebyshev_size,
                      scaling, coeffs, linear_coeffs, type_bias, alpha_moments_count, alpha_index_basic,
                      alpha_index_times, alpha_moment_mapping, nmus, binum, bilist, bnumneigh, bfirstneigh,
                      brcs, btypes, type_map, nghost, rmax, rmin, q_scaler, zbl_rmax=0.0, zbl_rmin=0.0,
                      zbl_cks=None, zbl_dks=None, validate=True):
    """[bloss[B], e_rmse[1], f_rmse[1], v_rmse[1]], differentiable w.r.t. coeffs, linear_coeffs and
    type_bias; mtpr_bind.cc:189-261."""
    betot_dft, bforce_dft, bvirial_dft = _zbl_shift_labels(
        zbl_rmax, zbl_rmin, zbl_cks, zbl_dks, type_map, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, nghost,
        betot_dft, bforce_dft, bvirial_dft, validate)
    args = (e_weight, f_weight, v_weight, betot_dft, bforce_dft, bvirial_dft, chebyshev_size, scaling,
            alpha_moments_count, alpha_index_basic, alpha_index_times, alpha_moment_mapping, nmus, binum,
            bilist, bnumneigh, bfirstneigh, brcs, btypes, type_map, nghost, rmax, rmin, q_scaler, validate)
    return list(_LinearMtpToLoss.apply(coeffs, linear_coeffs, type_bias, args))


def linearMtpToEFLossOp(e_weight, f_weight, betot_dft, bforce_dft, chebyshev_size, scaling, coeffs,
                        linear_coeffs, type_bias, alpha_moments_count, alpha_index_basic, alpha_index_times,
                        alpha_moment_mapping, nmus, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes,
                        type_map, nghost, rmax, rmin, q_scaler, zbl_rmax=0.0, zbl_rmin=0.0, zbl_cks=None,
                        zbl_dks=None, validate=True):
    """[bloss[B], e_rmse[1], f_rmse[1]]: the loss without virial labels (zero weight, zero labels);
    mtpr_bind.cc:263-331, linearMtpOp.cc:1768-2831."""
    betot_dft, bforce_dft, _ = _zbl_shift_labels(
        zbl_rmax, zbl_rmin, zbl_cks, zbl_dks, type_map, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, nghost,
        betot_dft, bforce_dft, None, validate)
    v_dft = torch.zeros((betot_dft.numel(), 9), dtype=betot_dft.dtype, device=betot_dft.device)
    args = (e_weight, f_weight, 0.0, betot_dft, bforce_dft, v_dft, chebyshev_size, scaling,
            alpha_moments_count, alpha_index_basic, alpha_index_times, alpha_moment_mapping, nmus, binum,
            bilist, bnumneigh, bfirstneigh, brcs, btypes, type_map, nghost, rmax, rmin, q_scaler, validate)
    return list(_LinearMtpToLoss.apply(coeffs, linear_coeffs, type_bias, args))[:3]


def _mtp_esites_raw(chebyshev_size, scaling, coeffs, linear_coeffs, type_bias, alpha_moments_count,
                    alpha_index_basic, alpha_index_times, alpha_moment_mapping, nmus, binum, bilist, bnumneigh,
                    bfirstneigh, brcs, btypes, type_map, nghost, rmax, rmin, q_scaler, want_esites, want_desc,
                    validate):
    dtype, device, B, P, U, nghost, ntypes, plan, n_scalar = _mtp_common(
        coeffs, linear_coeffs, type_bias, alpha_moments_count, alpha_index_basic, alpha_index_times,
        alpha_moment_mapping, nmus, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, type_map, nghost,
        q_scaler, chebyshev_size, validate)
    e_sites = torch.zeros((B, P), dtype=dtype, device=device) if want_esites else None
    desc = torch.zeros((B, P, n_scalar), dtype=dtype, device=device) if want_desc else None
    L = _lib.lib()
    fn = L.a2p_mtp_esites_f32 if dtype == torch.float32 else L.a2p_mtp_esites_f64
    with torch.cuda.device(device):
        call = lambda: fn(plan, _c.c_int(chebyshev_size), _c.c_double(scaling), _ptr(coeffs), _ptr(linear_coeffs),
                _ptr(type_bias), _c.c_int(int(nmus)), _c.c_int(ntypes), _ptr(q_scaler), _c.c_double(rmax),
                _c.c_double(rmin), _c.c_int(B), _c.c_int(P), _c.c_int(U), _c.c_int(nghost), _ptr(binum),
                _ptr(bilist), _ptr(bnumneigh), _ptr(bfirstneigh), _ptr(brcs), _ptr(btypes), _ptr(e_sites),
                _ptr(desc), _stream(device))
        _lib.check(call())
        if validate:
            _status_or_retry(call, B, P, U, nghost, binum, bnumneigh, bfirstneigh, device)
    return e_sites, desc


def mtp_esites_backward(grad_esites, chebyshev_size, scaling, coeffs, linear_coeffs, type_bias,
                        alpha_moments_count, alpha_index_basic, alpha_index_times, alpha_moment_mapping, nmus,
                        binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, type_map, nghost, rmax, rmin,
                        q_scaler, validate=False):
    """Per-structure gradients of sum_i grad_esites[b, i] * e_sites[b, i]:
    (dcoeffs[B, ncoef], dlinear[B, S], dbias[B, ntypes])."""
    dtype, device, B, P, U, nghost, ntypes, plan, n_scalar = _mtp_common(
        coeffs, linear_coeffs, type_bias, alpha_moments_count, alpha_index_basic, alpha_index_times,
        alpha_moment_mapping, nmus, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, type_map, nghost,
        q_scaler, chebyshev_size, validate)
    _check_float("grad_esites", grad_esites, dtype, device)
    _req(tuple(grad_esites.shape) == (B, P), "grad_esites must have shape [B, P]")
    z = lambda *s: torch.zeros(s, dtype=dtype, device=device)
    dc, dl, db = z(B, coeffs.numel()), z(B, n_scalar), z(B, ntypes)
    L = _lib.lib()
    fn = L.a2p_mtp_esites_bwd_f32 if dtype == torch.float32 else L.a2p_mtp_esites_bwd_f64
    with torch.cuda.device(device):
        rc = fn(plan, _c.c_int(chebyshev_size), _c.c_double(scaling), _ptr(coeffs),
                _ptr(linear_coeffs), _ptr(type_bias), _c.c_int(int(nmus)), _c.c_int(ntypes), _ptr(q_scaler),
                _c.c_double(rmax), _c.c_double(rmin), _c.c_int(B), _c.c_int(P), _c.c_int(U), _c.c_int(nghost),
                _ptr(binum), _ptr(bilist), _ptr(bnumneigh), _ptr(bfirstneigh), _ptr(brcs), _ptr(btypes),
                _ptr(grad_esites), _ptr(dc), _ptr(dl), _ptr(db), _stream(device))
        _lib.check(rc)
    return dc, dl, db


class _LinearMtpToEsites(torch.autograd.Function):
    """Site energies with the reference's autograd contract (linearMtpOp.cc:3589-3825, 3829-4027):
    gradients flow to coeffs, linear_coeffs and type_bias only, summed over structures and atoms."""

    @staticmethod
    def forward(ctx, coeffs, linear_coeffs, type_bias, args):
        (K, scaling, n_moms, basic, times, mapping, nmus, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes,
         type_map, nghost, rmax, rmin, q_scaler, validate) = args
        es, _ = _mtp_esites_raw(K, scaling, coeffs.detach(), linear_coeffs.detach(), type_bias.detach(), n_moms,
                                basic, times, mapping, nmus, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes,
                                type_map, nghost, rmax, rmin, q_scaler, True, False, validate)
        ctx.save_for_backward(coeffs, linear_coeffs, type_bias)
        ctx.args = args
        return es

    @staticmethod
    def backward(ctx, ges):
        coeffs, linear_coeffs, type_bias = ctx.saved_tensors
        (K, scaling, n_moms, basic, times, mapping, nmus, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes,
         type_map, nghost, rmax, rmin, q_scaler, _) = ctx.args
        dc, dl, db = mtp_esites_backward(ges.contiguous(), K, scaling, coeffs.detach(), linear_coeffs.detach(),
                                         type_bias.detach(), n_moms, basic, times, mapping, nmus, binum, bilist,
                                         bnumneigh, bfirstneigh, brcs, btypes, type_map, nghost, rmax, rmin,
                                         q_scaler)
        return (dc.sum(0).reshape(coeffs.shape), dl.sum(0).reshape(linear_coeffs.shape),
                db.sum(0).reshape(type_bias.shape), None)


def linearMtpToEsitesOp(chebyshev_size, scaling, coeffs, linear_coeffs, type_bias, alpha_moments_count,
                        alpha_index_basic, alpha_index_times, alpha_moment_mapping, nmus, binum, bilist,
                        bnumneigh, bfirstneigh, brcs, btypes, type_map, nghost, rmax, rmin, q_scaler,
                        zbl_rmax=0.0, zbl_rmin=0.0, zbl_cks=None, zbl_dks=None, validate=True):
    """[e_sites[B, P]] in row order (zero beyond binum), differentiable w.r.t. coeffs, linear_coeffs
    and type_bias; mtpr_bind.cc:458-518.  zbl_rmax > 0 adds each row's half pair energies (_zbl_esites)."""
    args = (chebyshev_size, scaling, alpha_moments_count, alpha_index_basic, alpha_index_times,
            alpha_moment_mapping, nmus, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, type_map, nghost,
            rmax, rmin, q_scaler, validate)
    es = _LinearMtpToEsites.apply(coeffs, linear_coeffs, type_bias, args)
    zb = _zbl_esites(zbl_rmax, zbl_rmin, zbl_cks, zbl_dks, type_map, binum, bilist, bnumneigh, bfirstneigh, brcs,
                     btypes, nghost, validate)
    return [es if zb is None else es + zb]


def linearMtpToDescriptorsOp(chebyshev_size, scaling, coeffs, alpha_moments_count, alpha_index_basic,
                             alpha_index_times, alpha_moment_mapping, nmus, binum, bilist, bnumneigh,
                             bfirstneigh, brcs, btypes, type_map, nghost, rmax, rmin, validate=True):
    """[descriptors[B, P, alpha_scalar_moments]]: the unscaled scalar moments of every row; no
    gradient, as in the reference (mtpr_bind.cc:521-570, linearMtpOp.cc:4030-4240)."""
    n_scalar = int(alpha_moment_mapping.numel())
    ntypes = int(type_map.numel())
    one = torch.ones((n_scalar,), dtype=brcs.dtype, device=brcs.device)
    zero_b = torch.zeros((ntypes,), dtype=brcs.dtype, device=brcs.device)
    _, desc = _mtp_esites_raw(chebyshev_size, scaling, coeffs.detach(), one, zero_b, alpha_moments_count,
                              alpha_index_basic, alpha_index_times, alpha_moment_mapping, nmus, binum, bilist,
                              bnumneigh, bfirstneigh, brcs, btypes, type_map, nghost, rmax, rmin, one, False, True,
                              validate)
    return [desc]


def mtp_basis_backward(grad_desc, chebyshev_size, scaling, coeffs, alpha_moments_count, alpha_index_basic,
                       alpha_index_times, alpha_moment_mapping, nmus, ntypes, binum, bilist, bnumneigh, bfirstneigh,
                       brcs, btypes, rmax, rmin, want_drcs=True, want_dcoeffs=True, nghost=0):
    """Backward of the legacy basis operator for the weights grad_desc[B, P, S] of the scalar moments:
    (drcs[B, P, U, 3], dcoeffs[B, ncoef]) (None where not wanted); mtpBasisOp.cc:220-326, mtpBasis.h:359-394."""
    _req(isinstance(brcs, torch.Tensor) and brcs.is_cuda,
         "brcs must be a tensor on a HIP device: this build has no CPU path")
    dtype, device = brcs.dtype, brcs.device
    _req(dtype in (torch.float32, torch.float64), "brcs must be float32 or float64")
    _req(brcs.is_contiguous(), "brcs must be contiguous")
    _check_float("coeffs", coeffs, dtype, device)
    _check_float("grad_desc", grad_desc, dtype, device)
    for name, t in (("binum", binum), ("bilist", bilist), ("bnumneigh", bnumneigh),
                    ("bfirstneigh", bfirstneigh), ("btypes", btypes)):
        _check_int(name, t, device)
    nghost, ntypes = int(nghost), int(ntypes)
    B, P, U = _batch_shapes(binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, nghost)
    plan, n_scalar = _mtp_plan(alpha_moments_count, alpha_index_basic, alpha_index_times, alpha_moment_mapping,
                               device)
    _req(coeffs.numel() == ntypes * ntypes * int(nmus) * int(chebyshev_size), "coeffs size mismatch")
    _req(tuple(grad_desc.shape) == (B, P, n_scalar), "grad_desc must have shape [B, P, alpha_scalar_moments]")
    drcs = torch.zeros((B, P, U, 3), dtype=dtype, device=device) if want_drcs else None
    dc = torch.zeros((B, coeffs.numel()), dtype=dtype, device=device) if want_dcoeffs else None
    if not (want_drcs or want_dcoeffs):
        return None, None
    L = _lib.lib()
    fn = L.a2p_mtp_basis_bwd_f32 if dtype == torch.float32 else L.a2p_mtp_basis_bwd_f64
    with torch.cuda.device(device):
        rc = fn(plan, _c.c_int(chebyshev_size), _c.c_double(scaling), _ptr(coeffs), _c.c_int(int(nmus)),
                _c.c_int(ntypes), _c.c_double(rmax), _c.c_double(rmin), _c.c_int(B), _c.c_int(P), _c.c_int(U),
                _c.c_int(nghost), _ptr(binum), _ptr(bilist), _ptr(bnumneigh), _ptr(bfirstneigh), _ptr(brcs),
                _ptr(btypes), _ptr(grad_desc), _ptr(drcs), _ptr(dc), _stream(device))
        _lib.check(rc)
    return drcs, dc


class _MtpBasis(torch.autograd.Function):
    """The legacy basis operator with the reference's autograd contract (mtpBasisOp.cc:28-326): the output
    is the scalar moments of every row; gradients flow to coeffs (summed over structures and atoms) and to
    brcs.  The reference keeps dM/d rcs [B, P, S, U, 3] and dM/d coeffs [B, P, S, ncoef] from the forward
    pass; here the backward recomputes the moments and runs one adjoint sweep per row."""

    @staticmethod
    def forward(ctx, coeffs, brcs, args):
        (n_moms, basic, times, mapping, nmus, ntypes, K, scaling, binum, bilist, bnumneigh, bfirstneigh, btypes,
         rmax, rmin, validate) = args
        dtype, device = brcs.dtype, brcs.device
        one = torch.ones((int(mapping.numel()),), dtype=dtype, device=device)
        zero_b = torch.zeros((int(ntypes),), dtype=dtype, device=device)
        type_map = torch.zeros((int(ntypes),), dtype=torch.int32, device=device)     # only its length is used
        _, desc = _mtp_esites_raw(K, scaling, coeffs.detach(), one, zero_b, n_moms, basic, times, mapping, nmus,
                                  binum, bilist, bnumneigh, bfirstneigh, brcs.detach(), btypes, type_map, 0, rmax, rmin,
                                  one, False, True, validate)
        ctx.save_for_backward(coeffs, brcs)
        ctx.args = args
        return desc

    @staticmethod
    def backward(ctx, gdesc):
        coeffs, brcs = ctx.saved_tensors
        (n_moms, basic, times, mapping, nmus, ntypes, K, scaling, binum, bilist, bnumneigh, bfirstneigh, btypes,
         rmax, rmin, _) = ctx.args
        drcs, dc = mtp_basis_backward(gdesc.contiguous(), K, scaling, coeffs.detach(), n_moms, basic, times, mapping,
                                      nmus, ntypes, binum, bilist, bnumneigh, bfirstneigh, brcs.detach(), btypes, rmax,
                                      rmin, want_drcs=ctx.needs_input_grad[1], want_dcoeffs=ctx.needs_input_grad[0])
        return (dc.sum(0).reshape(coeffs.shape) if dc is not None else None, drcs, None)


def mtpBasisOp(alpha_index_basic, alpha_index_times, alpha_moment_mapping, num_mus4moms, mus4moms, nmus, ntypes,
               chebyshev_size, scaling, coeffs, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, umax_num_neighs,
               rmax, rmin, validate=True):
    """[mtp_basis_val[B, P, alpha_scalar_moments]]: the scalar moments of every row, differentiable w.r.t.
    coeffs and brcs; mtpr_bind.cc:140-187 (same argument order).  num_mus4moms / mus4moms (the radial functions
    behind each moment, which the reference's coefficient derivative walks) are not needed: only the first
    dimension of mus4moms, the number of moments, is read.  nmus may be a tensor, as in the reference."""
    nmus = int(nmus.item()) if isinstance(nmus, torch.Tensor) else int(nmus)
    _req(int(umax_num_neighs) == int(brcs.shape[2]), "umax_num_neighs does not match brcs")
    args = (int(mus4moms.shape[0]), alpha_index_basic, alpha_index_times, alpha_moment_mapping, nmus, int(ntypes),
            int(chebyshev_size), float(scaling), binum, bilist, bnumneigh, bfirstneigh, btypes, float(rmax),
            float(rmin), validate)
    return [_MtpBasis.apply(coeffs, brcs, args)]


def mtp_lin_components(chebyshev_size, scaling, coeffs, alpha_moments_count, alpha_index_basic, alpha_index_times,
                       alpha_moment_mapping, nmus, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, type_map,
                       rmax, rmin, q_scaler, validate=True):
    """Energy [B, n], force [B, P, 3, n] and virial [B, 9, n] of every linear parameter taken alone,
    n = alpha_scalar_moments + ntypes (linear_mtp_gram_and_cross.h:125-374)."""
    ntypes = int(type_map.numel())
    S = int(alpha_moment_mapping.numel())
    dtype, device = brcs.dtype, brcs.device
    dummy_lin = torch.zeros((S,), dtype=dtype, device=device)
    dummy_bias = torch.zeros((ntypes,), dtype=dtype, device=device)
    dtype, device, B, P, U, nghost, ntypes, plan, n_scalar = _mtp_common(
        coeffs, dummy_lin, dummy_bias, alpha_moments_count, alpha_index_basic, alpha_index_times,
        alpha_moment_mapping, nmus, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, type_map, 0, q_scaler,
        chebyshev_size, validate)
    n = n_scalar + ntypes
    z = lambda *sh: torch.empty(sh, dtype=dtype, device=device)       # the library writes every element
    ecomp, fcomp, vcomp = z(B, n), z(B, P, 3, n), z(B, 9, n)
    L = _lib.lib()
    fn = L.a2p_mtp_lin_components_f32 if dtype == torch.float32 else L.a2p_mtp_lin_components_f64
    with torch.cuda.device(device):
        call = lambda: fn(plan, _c.c_int(chebyshev_size), _c.c_double(scaling), _ptr(coeffs), _c.c_int(int(nmus)),
                _c.c_int(ntypes), _ptr(q_scaler), _c.c_double(rmax), _c.c_double(rmin), _c.c_int(B), _c.c_int(P),
                _c.c_int(U), _ptr(binum), _ptr(bilist), _ptr(bnumneigh), _ptr(bfirstneigh), _ptr(brcs), _ptr(btypes),
                _ptr(ecomp), _ptr(fcomp), _ptr(vcomp), _stream(device))
        _lib.check(call())
        if validate:
            _status_or_retry(call, B, P, U, 0, binum, bnumneigh, bfirstneigh, device)
    return ecomp, fcomp, vcomp


def _gram(X, y):
    """X^T X [n, n] and X^T y [n] of a tall matrix X [N, n].  The rows are cut into up to 64 blocks whose products run as
    one batched GEMM and are added afterwards: a single GEMM with n of about a hundred and N in the tens of thousands
    occupies one tile of the chip (0.66 ms against 0.03 ms for 24576 x 95 in fp64)."""
    N, n = X.shape
    R = torch.cat([X, y.reshape(N, 1)], dim=1)
    chunks = max(1, min(64, N // 256))
    k = N // chunks
    head = k * chunks
    G = torch.bmm(X[:head].reshape(chunks, k, n).transpose(1, 2), R[:head].reshape(chunks, k, n + 1)).sum(0)
    if head < N:
        G = G + X[head:].t() @ R[head:]
    return G[:, :n], G[:, n]


def LinMatrixLinVectorOp(e_weight, f_weight, v_weight, betot_dft, bforce_dft, bvirial_dft, chebyshev_size, scaling,
                         coeffs, linear_coeffs, type_bias, alpha_moments_count, alpha_index_basic,
                         alpha_index_times, alpha_moment_mapping, nmus, binum, bilist, bnumneigh, bfirstneigh, brcs,
                         btypes, type_map, nghost, rmax, rmin, q_scaler, zbl_rmax=0.0, zbl_rmin=0.0, zbl_cks=None,
                         zbl_dks=None, validate=True):
    """[lin_matrix[n, n], lin_vector[n]]: the normal equations of the linear parameters
    (linear_coeffs / q_scaler, then type_bias) for fixed radial coefficients; mtpr_bind.cc:57-131,
    linear_mtp_gram_and_cross.h:446-575.  linear_coeffs and type_bias do not enter, as in the
    reference; no gradient.  zbl_rmax > 0: the labels enter with the ZBL energy, forces and virial taken out
    (src/linear_mtp_gram_and_cross_op.cc:309-338)."""
    _req(int(nghost) == 0, "LinMatrixLinVectorOp requires nghost == 0: the reference's force components "
                           "have natoms_pad rows")
    betot_dft, bforce_dft, bvirial_dft = _zbl_shift_labels(
        zbl_rmax, zbl_rmin, zbl_cks, zbl_dks, type_map, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, nghost,
        betot_dft, bforce_dft, bvirial_dft, validate)
    ecomp, fcomp, vcomp = mtp_lin_components(chebyshev_size, scaling, coeffs.detach(), alpha_moments_count,
                                             alpha_index_basic, alpha_index_times, alpha_moment_mapping, nmus,
                                             binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, type_map, rmax,
                                             rmin, q_scaler, validate)
    B, P = bilist.shape
    n = ecomp.shape[1]
    for name, t, numel in (("betot_dft", betot_dft, B), ("bforce_dft", bforce_dft, B * P * 3),
                           ("bvirial_dft", bvirial_dft, B * 9)):
        _check_float(name, t, brcs.dtype, brcs.device)
        _req(t.numel() == numel, "%s has %d elements, expected %d" % (name, t.numel(), numel))
    F = fcomp.reshape(B * P * 3, n)          # rows of padded atoms are zero
    V = vcomp.reshape(B * 9, n)
    (ae, be), (af, bf), (av, bv) = (_gram(ecomp, betot_dft.reshape(B)), _gram(F, bforce_dft.reshape(-1)),
                                    _gram(V, bvirial_dft.reshape(-1)))
    lin_matrix = e_weight * ae + f_weight * af + v_weight * av
    lin_vector = e_weight * be + f_weight * bf + v_weight * bv
    return [lin_matrix.contiguous(), lin_vector.contiguous()]


def CoeffsSchmidtOrthOp(ntypes, nmus, chebyshev_size, coeffs):
    """[orth_coeffs]: Gram-Schmidt over the nmus radial functions (mtpr_bind.cc:38-55,
    schmidt_orth.h:38-116); same shape as coeffs, no gradient."""
    _req(isinstance(coeffs, torch.Tensor) and coeffs.is_cuda, "coeffs must be a tensor on a HIP device")
    _req(coeffs.dtype in (torch.float32, torch.float64) and coeffs.is_contiguous(),
         "coeffs must be a contiguous float32 or float64 tensor")
    _req(coeffs.numel() == int(ntypes) * int(ntypes) * int(nmus) * int(chebyshev_size), "coeffs size mismatch")
    src = coeffs.detach()
    out = torch.empty_like(src)
    L = _lib.lib()
    fn = L.a2p_mtp_schmidt_orth_f32 if src.dtype == torch.float32 else L.a2p_mtp_schmidt_orth_f64
    with torch.cuda.device(src.device):
        _lib.check(fn(_c.c_int(int(ntypes)), _c.c_int(int(nmus)), _c.c_int(int(chebyshev_size)), _ptr(src),
                      _ptr(out), _stream(src.device)))
    return [out]


# --------------------------------------------------------------------------------------------
# neural-network MTP  (source/descriptor/nnmtp/bind/nnmtp_bind.cc:193-430)
# --------------------------------------------------------------------------------------------
def _nnmtp_call(want, chebyshev_size, coeffs, w0, w1, type_bias, alpha_moments_count, alpha_index_basic,
                alpha_index_times, alpha_moment_mapping, nmus, binum, bilist, bnumneigh, bfirstneigh, brcs,
                btypes, type_map, nghost, rmax, rmin, q_shifter, q_scaler, validate):
    """want: subset of {"e", "f", "v", "es"}.  Returns (etot, force, virial, e_sites), None where not asked."""
    _req(isinstance(brcs, torch.Tensor) and brcs.is_cuda,
         "brcs must be a tensor on a HIP device: this build has no CPU path")
    dtype, device = brcs.dtype, brcs.device
    _req(dtype in (torch.float32, torch.float64), "brcs must be float32 or float64")
    _req(brcs.is_contiguous(), "brcs must be contiguous")
    for name, t in (("coeffs", coeffs), ("w0", w0), ("w1", w1), ("type_bias", type_bias),
                    ("q_shifter", q_shifter), ("q_scaler", q_scaler)):
        _check_float(name, t, dtype, device)
    for name, t in (("binum", binum), ("bilist", bilist), ("bnumneigh", bnumneigh),
                    ("bfirstneigh", bfirstneigh), ("btypes", btypes)):
        _check_int(name, t, device)
    nghost = int(nghost)
    B, P, U = _batch_shapes(binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, nghost)
    ntypes = int(type_map.numel())
    _req(ntypes > 0, "type_map is empty")
    plan, n_scalar = _mtp_plan(alpha_moments_count, alpha_index_basic, alpha_index_times,
                               alpha_moment_mapping, device)
    _req(coeffs.numel() == ntypes * ntypes * int(nmus) * int(chebyshev_size), "coeffs size mismatch")
    _req(w1.numel() % ntypes == 0 and w1.numel() > 0, "w1 must have ntypes * num_neurons elements")
    H = w1.numel() // ntypes                                    # nnMtpOp.cc: num_neurons = w1.size(1)
    _req(w0.numel() == ntypes * H * n_scalar, "w0 has %d elements, expected ntypes*H*alpha_scalar_moments = %d"
         % (w0.numel(), ntypes * H * n_scalar))
    _req(q_shifter.numel() == n_scalar and q_scaler.numel() == n_scalar,
         "q_shifter and q_scaler must have alpha_scalar_moments = %d elements" % n_scalar)
    _req(type_bias.numel() == ntypes, "type_bias size mismatch")
    if validate:
        _validate_batch(binum, bnumneigh, U, P)
    z = lambda *sh: torch.zeros(sh, dtype=dtype, device=device)
    new = (lambda *sh: torch.empty(sh, dtype=dtype, device=device)) if B * P > 0 else z   # written in full by the library
    etot = new(B) if "e" in want else None
    force = new(B, P + nghost, 3) if "f" in want else None
    virial = new(B, 9) if "v" in want else None
    e_sites = z(B, P) if "es" in want else None
    L = _lib.lib()
    fn = L.a2p_nnmtp_efv_f32 if dtype == torch.float32 else L.a2p_nnmtp_efv_f64
    with torch.cuda.device(device):
        call = lambda: fn(plan, _c.c_int(chebyshev_size), _c.c_int(H), _ptr(coeffs), _ptr(w0), _ptr(w1), _ptr(type_bias),
                _c.c_int(int(nmus)), _c.c_int(ntypes), _ptr(q_shifter), _ptr(q_scaler), _c.c_double(rmax),
                _c.c_double(rmin), _c.c_int(B), _c.c_int(P), _c.c_int(U), _c.c_int(nghost), _ptr(binum),
                _ptr(bilist), _ptr(bnumneigh), _ptr(bfirstneigh), _ptr(brcs), _ptr(btypes), _ptr(etot),
                _ptr(force), _ptr(virial), _ptr(e_sites), _stream(device))
        _lib.check(call())
        if validate:
            _status_or_retry(call, B, P, U, nghost, binum, bnumneigh, bfirstneigh, device)
    return etot, force, virial, e_sites


def nnMtpToEFVOp(chebyshev_size, coeffs, w0, w1, type_bias, alpha_moments_count, alpha_index_basic,
                 alpha_index_times, alpha_moment_mapping, nmus, binum, bilist, bnumneigh, bfirstneigh, brcs,
                 btypes, type_map, nghost, rmax, rmin, q_shifter, q_scaler, zbl_rmax=0.0, zbl_rmin=0.0,
                 zbl_cks=None, zbl_dks=None, validate=True):
    """[E[B], F[B, P+nghost, 3], V[B, 9]]; nnmtp_bind.cc:258-322, nnMtpOp.cc:2785-3010."""
    e, f, v, _ = _nnmtp_call("efv", chebyshev_size, coeffs, w0, w1, type_bias, alpha_moments_count,
                             alpha_index_basic, alpha_index_times, alpha_moment_mapping, nmus, binum, bilist,
                             bnumneigh, bfirstneigh, brcs, btypes, type_map, nghost, rmax, rmin, q_shifter,
                             q_scaler, validate)
    _zbl_add(zbl_rmax, zbl_rmin, zbl_cks, zbl_dks, type_map, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes,
             nghost, e, f, v, validate)
    return [e, f, v]


def nnMtpToEFOp(chebyshev_size, coeffs, w0, w1, type_bias, alpha_moments_count, alpha_index_basic,
                alpha_index_times, alpha_moment_mapping, nmus, binum, bilist, bnumneigh, bfirstneigh, brcs,
                btypes, type_map, nghost, rmax, rmin, q_shifter, q_scaler, zbl_rmax=0.0, zbl_rmin=0.0,
                zbl_cks=None, zbl_dks=None, validate=True):
    """[E[B], F[B, P+nghost, 3]]; nnmtp_bind.cc:193-256."""
    e, f, _, _ = _nnmtp_call("ef", chebyshev_size, coeffs, w0, w1, type_bias, alpha_moments_count,
                             alpha_index_basic, alpha_index_times, alpha_moment_mapping, nmus, binum, bilist,
                             bnumneigh, bfirstneigh, brcs, btypes, type_map, nghost, rmax, rmin, q_shifter,
                             q_scaler, validate)
    _zbl_add(zbl_rmax, zbl_rmin, zbl_cks, zbl_dks, type_map, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes,
             nghost, e, f, None, validate)
    return [e, f]


def nnmtp_esites_backward(grad_esites, chebyshev_size, coeffs, w0, w1, type_bias, alpha_moments_count,
                          alpha_index_basic, alpha_index_times, alpha_moment_mapping, nmus, binum, bilist,
                          bnumneigh, bfirstneigh, brcs, btypes, type_map, nghost, rmax, rmin, q_shifter, q_scaler):
    """Per-structure gradients of sum_i grad_esites[b, i] * e_sites[b, i]:
    (dcoeffs[B, ncoef], dw0[B, ntypes*H*S], dw1[B, ntypes*H], dbias[B, ntypes])."""
    dtype, device = brcs.dtype, brcs.device
    nghost = int(nghost)
    B, P, U = _batch_shapes(binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, nghost)
    ntypes = int(type_map.numel())
    plan, n_scalar = _mtp_plan(alpha_moments_count, alpha_index_basic, alpha_index_times,
                               alpha_moment_mapping, device)
    H = w1.numel() // ntypes
    _check_float("grad_esites", grad_esites, dtype, device)
    _req(tuple(grad_esites.shape) == (B, P), "grad_esites must have shape [B, P]")
    z = lambda *sh: torch.zeros(sh, dtype=dtype, device=device)
    out = (z(B, coeffs.numel()), z(B, w0.numel()), z(B, w1.numel()), z(B, ntypes))
    L = _lib.lib()
    fn = L.a2p_nnmtp_esites_bwd_f32 if dtype == torch.float32 else L.a2p_nnmtp_esites_bwd_f64
    with torch.cuda.device(device):
        rc = fn(plan, _c.c_int(chebyshev_size), _c.c_int(H), _ptr(coeffs), _ptr(w0), _ptr(w1), _ptr(type_bias),
                _c.c_int(int(nmus)), _c.c_int(ntypes), _ptr(q_shifter), _ptr(q_scaler), _c.c_double(rmax),
                _c.c_double(rmin), _c.c_int(B), _c.c_int(P), _c.c_int(U), _c.c_int(nghost), _ptr(binum),
                _ptr(bilist), _ptr(bnumneigh), _ptr(bfirstneigh), _ptr(brcs), _ptr(btypes), _ptr(grad_esites),
                _ptr(out[0]), _ptr(out[1]), _ptr(out[2]), _ptr(out[3]), _stream(device))
        _lib.check(rc)
    return out


class _NNMtpToEsites(torch.autograd.Function):
    """Site energies of the neural-network MTP; gradients flow to coeffs, w0, w1, type_bias, summed
    over structures and rows (nnMtpOp.cc:4170-4330).  The reference fills its per-row derivative
    tensors for w0 and w1 without the species offset (nnMtp.h:965-971 index rows of num_neurons
    entries inside tensors allocated with ntypes * num_neurons, nnMtpOp.cc:4236-4239), so for more
    than one species its result is mis-assigned; this build returns the derivative itself, which
    coincides with the reference for a single species."""

    @staticmethod
    def forward(ctx, coeffs, w0, w1, type_bias, args):
        (K, n_moms, basic, times, mapping, nmus, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, type_map,
         nghost, rmax, rmin, q_shifter, q_scaler, validate) = args
        _, _, _, es = _nnmtp_call(("es",), K, coeffs.detach(), w0.detach(), w1.detach(), type_bias.detach(), n_moms,
                                  basic, times, mapping, nmus, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes,
                                  type_map, nghost, rmax, rmin, q_shifter, q_scaler, validate)
        ctx.save_for_backward(coeffs, w0, w1, type_bias)
        ctx.args = args
        return es

    @staticmethod
    def backward(ctx, ges):
        coeffs, w0, w1, type_bias = ctx.saved_tensors
        (K, n_moms, basic, times, mapping, nmus, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, type_map,
         nghost, rmax, rmin, q_shifter, q_scaler, _) = ctx.args
        g = nnmtp_esites_backward(ges.contiguous(), K, coeffs.detach(), w0.detach(), w1.detach(),
                                  type_bias.detach(), n_moms, basic, times, mapping, nmus, binum, bilist, bnumneigh,
                                  bfirstneigh, brcs, btypes, type_map, nghost, rmax, rmin, q_shifter, q_scaler)
        return tuple(x.sum(0).reshape(p.shape) for x, p in zip(g, (coeffs, w0, w1, type_bias))) + (None,)


def nnMtpToEsitesOp(chebyshev_size, coeffs, w0, w1, type_bias, alpha_moments_count, alpha_index_basic,
                    alpha_index_times, alpha_moment_mapping, nmus, binum, bilist, bnumneigh, bfirstneigh, brcs,
                    btypes, type_map, nghost, rmax, rmin, q_shifter, q_scaler, zbl_rmax=0.0, zbl_rmin=0.0,
                    zbl_cks=None, zbl_dks=None, validate=True):
    """[e_sites[B, P]] in row order, differentiable w.r.t. coeffs, w0, w1, type_bias;
    nnmtp_bind.cc:370-430.  zbl_rmax > 0 adds each row's half pair energies (_zbl_esites)."""
    args = (chebyshev_size, alpha_moments_count, alpha_index_basic, alpha_index_times, alpha_moment_mapping, nmus,
            binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, type_map, nghost, rmax, rmin, q_shifter, q_scaler,
            validate)
    es = _NNMtpToEsites.apply(coeffs, w0, w1, type_bias, args)
    zb = _zbl_esites(zbl_rmax, zbl_rmin, zbl_cks, zbl_dks, type_map, binum, bilist, bnumneigh, bfirstneigh, brcs,
                     btypes, nghost, validate)
    return [es if zb is None else es + zb]


def nnMtpToDescriptorsOp(chebyshev_size, coeffs, alpha_moments_count, alpha_index_basic, alpha_index_times,
                         alpha_moment_mapping, nmus, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes,
                         type_map, nghost, rmax, rmin, validate=True):
    """[descriptors[B, P, alpha_scalar_moments]]: the scalar moments, i.e. the linear-MTP descriptors
    at scaling 1 (nnmtp_bind.cc:323-368, nnMtp.h:570-645)."""
    return linearMtpToDescriptorsOp(chebyshev_size, 1.0, coeffs, alpha_moments_count, alpha_index_basic,
                                    alpha_index_times, alpha_moment_mapping, nmus, binum, bilist, bnumneigh,
                                    bfirstneigh, brcs, btypes, type_map, nghost, rmax, rmin, validate)


def nnmtp_loss_step(e_weight, f_weight, v_weight, betot_dft, bforce_dft, bvirial_dft, chebyshev_size, coeffs, w0,
                    w1, type_bias, alpha_moments_count, alpha_index_basic, alpha_index_times,
                    alpha_moment_mapping, nmus, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, type_map,
                    nghost, rmax, rmin, q_shifter, q_scaler, want_grad=True, exact_gradient=False, validate=True):
    """Forward and (optionally) the per-structure parameter gradients of the NN-MTP training loss.
    Returns a dict with bloss[B], energy, force, virial and, with want_grad, dcoeffs[B, ncoef],
    dw0[B, ntypes*H*S], dw1[B, ntypes*H], dbias[B, ntypes].  exact_gradient=False evaluates the
    reference's backward formulas (nnMtpLoss.h:216-610), which are not the full derivative of the
    loss for the force and virial terms; exact_gradient=True returns the full derivative."""
    _req(int(nghost) == 0, "the loss operator requires nghost == 0, as the reference does")
    _req(isinstance(brcs, torch.Tensor) and brcs.is_cuda,
         "brcs must be a tensor on a HIP device: this build has no CPU path")
    dtype, device = brcs.dtype, brcs.device
    _req(dtype in (torch.float32, torch.float64), "brcs must be float32 or float64")
    _req(brcs.is_contiguous(), "brcs must be contiguous")
    for name, t in (("coeffs", coeffs), ("w0", w0), ("w1", w1), ("type_bias", type_bias),
                    ("q_shifter", q_shifter), ("q_scaler", q_scaler)):
        _check_float(name, t, dtype, device)
    for name, t in (("binum", binum), ("bilist", bilist), ("bnumneigh", bnumneigh),
                    ("bfirstneigh", bfirstneigh), ("btypes", btypes)):
        _check_int(name, t, device)
    B, P, U = _batch_shapes(binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, 0)
    ntypes = int(type_map.numel())
    _req(ntypes > 0, "type_map is empty")
    plan, n_scalar = _mtp_plan(alpha_moments_count, alpha_index_basic, alpha_index_times,
                               alpha_moment_mapping, device)
    _req(coeffs.numel() == ntypes * ntypes * int(nmus) * int(chebyshev_size), "coeffs size mismatch")
    _req(w1.numel() % ntypes == 0 and w1.numel() > 0, "w1 must have ntypes * num_neurons elements")
    H = w1.numel() // ntypes
    _req(w0.numel() == ntypes * H * n_scalar, "w0 must have ntypes*H*alpha_scalar_moments elements")
    _req(q_shifter.numel() == n_scalar and q_scaler.numel() == n_scalar,
         "q_shifter and q_scaler must have alpha_scalar_moments = %d elements" % n_scalar)
    _req(type_bias.numel() == ntypes, "type_bias size mismatch")
    for name, t, n_expected in (("betot_dft", betot_dft, B), ("bforce_dft", bforce_dft, B * P * 3),
                                ("bvirial_dft", bvirial_dft, B * 9)):
        _check_float(name, t, dtype, device)
        _req(t.numel() == n_expected, "%s has %d elements, expected %d" % (name, t.numel(), n_expected))
    if validate:
        _validate_batch(binum, bnumneigh, U, P)
    z = lambda *sh: torch.zeros(sh, dtype=dtype, device=device)
    out = dict(bloss=z(B), energy=z(B), force=z(B, P, 3), virial=z(B, 9))
    if want_grad:
        out.update(dcoeffs=z(B, coeffs.numel()), dw0=z(B, w0.numel()), dw1=z(B, w1.numel()), dbias=z(B, ntypes))
    L = _lib.lib()
    fn = L.a2p_nnmtp_loss_f32 if dtype == torch.float32 else L.a2p_nnmtp_loss_f64
    with torch.cuda.device(device):
        call = lambda: fn(plan, _c.c_double(e_weight), _c.c_double(f_weight), _c.c_double(v_weight), _ptr(betot_dft),
                _ptr(bforce_dft), _ptr(bvirial_dft), _c.c_int(chebyshev_size), _c.c_int(H), _ptr(coeffs), _ptr(w0),
                _ptr(w1), _ptr(type_bias), _c.c_int(int(nmus)), _c.c_int(ntypes), _ptr(q_shifter), _ptr(q_scaler),
                _c.c_double(rmax), _c.c_double(rmin), _c.c_int(B), _c.c_int(P), _c.c_int(U), _ptr(binum),
                _ptr(bilist), _ptr(bnumneigh), _ptr(bfirstneigh), _ptr(brcs), _ptr(btypes), _ptr(out["bloss"]),
                _ptr(out["energy"]), _ptr(out["force"]), _ptr(out["virial"]), _ptr(out.get("dcoeffs")),
                _ptr(out.get("dw0")), _ptr(out.get("dw1")), _ptr(out.get("dbias")),
                _c.c_int(1 if exact_gradient else 0), _stream(device))
        _lib.check(call())
        if validate:
            _status_or_retry(call, B, P, U, 0, binum, bnumneigh, bfirstneigh, device)
    return out


class _NNMtpToLoss(torch.autograd.Function):
    """Autograd wrapper with the reference's contract (nnMtpOp.cc:1641-2780): one output, bloss[B];
    gradients flow to coeffs, w0, w1 and type_bias as grad_output[B] @ dloss/dtheta."""

    @staticmethod
    def forward(ctx, coeffs, w0, w1, type_bias, args):
        (e_w, f_w, v_w, e_dft, f_dft, v_dft, K, n_moms, basic, times, mapping, nmus, binum, bilist, bnumneigh,
         bfirstneigh, brcs, btypes, type_map, nghost, rmax, rmin, q_shifter, q_scaler, exact, validate) = args
        need = any(t.requires_grad for t in (coeffs, w0, w1, type_bias))
        r = nnmtp_loss_step(e_w, f_w, v_w, e_dft, f_dft, v_dft, K, coeffs.detach(), w0.detach(), w1.detach(),
                            type_bias.detach(), n_moms, basic, times, mapping, nmus, binum, bilist, bnumneigh,
                            bfirstneigh, brcs, btypes, type_map, nghost, rmax, rmin, q_shifter, q_scaler,
                            want_grad=need, exact_gradient=exact, validate=validate)
        if need:
            ctx.save_for_backward(r["dcoeffs"], r["dw0"], r["dw1"], r["dbias"])
        ctx.shapes = (coeffs.shape, w0.shape, w1.shape, type_bias.shape)
        ctx.have = need
        return r["bloss"]

    @staticmethod
    def backward(ctx, gl):
        if not ctx.have:
            return None, None, None, None, None
        return tuple(torch.matmul(gl, g).reshape(sh) for g, sh in zip(ctx.saved_tensors, ctx.shapes)) + (None,)


def nnMtpToLossOp(e_weight, f_weight, v_weight, betot_dft, bforce_dft, bvirial_dft, chebyshev_size, coeffs, w0, w1,
                  type_bias, alpha_moments_count, alpha_index_basic, alpha_index_times, alpha_moment_mapping, nmus,
                  binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, type_map, nghost, rmax, rmin, q_shifter,
                  q_scaler, zbl_rmax=0.0, zbl_rmin=0.0, zbl_cks=None, zbl_dks=None, exact_gradient=False,
                  validate=True):
    """[bloss[B]], differentiable w.r.t. coeffs, w0, w1, type_bias; nnmtp_bind.cc:116-191."""
    betot_dft, bforce_dft, bvirial_dft = _zbl_shift_labels(
        zbl_rmax, zbl_rmin, zbl_cks, zbl_dks, type_map, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, nghost,
        betot_dft, bforce_dft, bvirial_dft, validate)
    args = (e_weight, f_weight, v_weight, betot_dft, bforce_dft, bvirial_dft, chebyshev_size, alpha_moments_count,
            alpha_index_basic, alpha_index_times, alpha_moment_mapping, nmus, binum, bilist, bnumneigh, bfirstneigh,
            brcs, btypes, type_map, nghost, rmax, rmin, q_shifter, q_scaler, exact_gradient, validate)
    return [_NNMtpToLoss.apply(coeffs, w0, w1, type_bias, args)]


def nnMtpToEFLossOp(e_weight, f_weight, betot_dft, bforce_dft, chebyshev_size, coeffs, w0, w1, type_bias,
                    alpha_moments_count, alpha_index_basic, alpha_index_times, alpha_moment_mapping, nmus, binum,
                    bilist, bnumneigh, bfirstneigh, brcs, btypes, type_map, nghost, rmax, rmin, q_shifter, q_scaler,
                    zbl_rmax=0.0, zbl_rmin=0.0, zbl_cks=None, zbl_dks=None, exact_gradient=False, validate=True):
    """[bloss[B]] without virial labels (zero weight, zero labels); nnmtp_bind.cc:43-114."""
    betot_dft, bforce_dft, _ = _zbl_shift_labels(
        zbl_rmax, zbl_rmin, zbl_cks, zbl_dks, type_map, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, nghost,
        betot_dft, bforce_dft, None, validate)
    v_dft = torch.zeros((betot_dft.numel(), 9), dtype=betot_dft.dtype, device=betot_dft.device)
    args = (e_weight, f_weight, 0.0, betot_dft, bforce_dft, v_dft, chebyshev_size, alpha_moments_count,
            alpha_index_basic, alpha_index_times, alpha_moment_mapping, nmus, binum, bilist, bnumneigh, bfirstneigh,
            brcs, btypes, type_map, nghost, rmax, rmin, q_shifter, q_scaler, exact_gradient, validate)
    return [_NNMtpToLoss.apply(coeffs, w0, w1, type_bias, args)]


# --------------------------------------------------------------------------------------------
# fvt  (source/fvt/bind/fvt_sr_op_bind.cc:9-46)
# --------------------------------------------------------------------------------------------
def _fvt_fn(name, dtype):
    return getattr(_lib.lib(), "a2p_fvt_%s_%s" % (name, "f32" if dtype == torch.float32 else "f64"))


def _fvt_force_raw(binum, bilist, bnumneigh, bfirstneigh, nghost, dei):
    B, P, U, _ = dei.shape
    force = torch.empty((B, P + nghost, 3), dtype=dei.dtype, device=dei.device)
    with torch.cuda.device(dei.device):
        _lib.check(_fvt_fn("force_fwd", dei.dtype)(
            _c.c_int(B), _c.c_int(P), _c.c_int(U), _c.c_int(nghost), _ptr(binum), _ptr(bilist),
            _ptr(bnumneigh), _ptr(bfirstneigh), _ptr(dei), _ptr(force), _stream(dei.device)))
    return force


def _fvt_force_bwd_raw(binum, bilist, bnumneigh, bfirstneigh, nghost, U, gF):
    B, P = bilist.shape
    out = torch.empty((B, P, U, 3), dtype=gF.dtype, device=gF.device)
    with torch.cuda.device(gF.device):
        _lib.check(_fvt_fn("force_bwd", gF.dtype)(
            _c.c_int(B), _c.c_int(P), _c.c_int(U), _c.c_int(nghost), _ptr(binum), _ptr(bilist),
            _ptr(bnumneigh), _ptr(bfirstneigh), _ptr(gF), _ptr(out), _stream(gF.device)))
    return out


class _ForceSr(torch.autograd.Function):
    """dei -> force.  The map is linear, so its backward is the adjoint gather and the
    backward of that is this map again: any order of differentiation stays on the kernels."""

    @staticmethod
    def forward(ctx, dei, lists):
        ctx.lists = lists
        binum, bilist, bnumneigh, bfirstneigh, nghost = lists
        return _fvt_force_raw(binum, bilist, bnumneigh, bfirstneigh, nghost, dei.contiguous())

    @staticmethod
    def backward(ctx, gF):
        return _ForceSrAdjoint.apply(gF, ctx.lists), None


class _ForceSrAdjoint(torch.autograd.Function):
    @staticmethod
    def forward(ctx, gF, lists):
        ctx.lists = lists
        binum, bilist, bnumneigh, bfirstneigh, nghost = lists
        return _fvt_force_bwd_raw(binum, bilist, bnumneigh, bfirstneigh, nghost, bfirstneigh.shape[2],
                                  gF.contiguous())

    @staticmethod
    def backward(ctx, gg):
        return _ForceSr.apply(gg, ctx.lists), None


def ForceSrOp(binum, bilist, bnumneigh, bfirstneigh, nghost, umax_num_neighs, bdei_drij):
    """[force[B, nlocal+nghost, 3]], differentiable w.r.t. bdei_drij to any order;
    fvt_sr_op_bind.cc:9-29, src/force_sr_op.cc:11-179."""
    _req(isinstance(bdei_drij, torch.Tensor) and bdei_drij.is_cuda,
         "bdei_drij must be a tensor on a HIP device: this build has no CPU path")
    dtype, device = bdei_drij.dtype, bdei_drij.device
    _req(dtype in (torch.float32, torch.float64), "bdei_drij must be float32 or float64")
    for name, t in (("binum", binum), ("bilist", bilist), ("bnumneigh", bnumneigh),
                    ("bfirstneigh", bfirstneigh)):
        _check_int(name, t, device)
    _req(bdei_drij.dim() == 4 and bdei_drij.shape[3] == 3, "bdei_drij must have shape [B, nlocal, umax, 3]")
    B, P, U, _ = bdei_drij.shape
    _req(int(umax_num_neighs) == U, "umax_num_neighs does not match bdei_drij")
    _req(tuple(bfirstneigh.shape) == (B, P, U) and tuple(bilist.shape) == (B, P) and
         tuple(bnumneigh.shape) == (B, P) and tuple(binum.shape) == (B,), "neighbour tensors do not match")
    _validate_batch(binum, bnumneigh, U, P)
    out = _ForceSr.apply(bdei_drij, (binum, bilist, bnumneigh, bfirstneigh, int(nghost)))
    _lib.check_status(torch.cuda.current_stream(device).cuda_stream)
    return [out]


def _fvt_virial_raw(bnumneigh, rcs, dei):
    B, P, U, _ = dei.shape
    v = torch.empty((B, 9), dtype=dei.dtype, device=dei.device)
    with torch.cuda.device(dei.device):
        _lib.check(_fvt_fn("virial_fwd", dei.dtype)(
            _c.c_int(B), _c.c_int(P), _c.c_int(U), _ptr(bnumneigh), _ptr(rcs), _ptr(dei), _ptr(v),
            _stream(dei.device)))
    return v.view(B, 3, 3)


def _fvt_virial_bwd_raw(bnumneigh, rcs, dei, gV, want_dei, want_rcs):
    B, P, U, _ = dei.shape
    gd = torch.empty_like(dei) if want_dei else None
    gr = torch.empty_like(rcs) if want_rcs else None
    with torch.cuda.device(dei.device):
        _lib.check(_fvt_fn("virial_bwd", dei.dtype)(
            _c.c_int(B), _c.c_int(P), _c.c_int(U), _ptr(bnumneigh), _ptr(rcs), _ptr(dei),
            _ptr(gV.contiguous()), _ptr(gd), _ptr(gr), _stream(dei.device)))
    return gd, gr


class _VirialSr(torch.autograd.Function):
    """(rcs, dei) -> virial, bilinear.  Backward is itself a Function of (gV, rcs, dei), so
    create_graph=True callers (ai2pot/models/deepmd/se_r.py:316-330) differentiate again."""

    @staticmethod
    def forward(ctx, rcs, dei, bnumneigh):
        ctx.save_for_backward(rcs, dei)
        ctx.bnumneigh = bnumneigh
        return _fvt_virial_raw(bnumneigh, rcs.contiguous(), dei.contiguous())

    @staticmethod
    def backward(ctx, gV):
        rcs, dei = ctx.saved_tensors
        grcs, gdei = _VirialSrBackward.apply(gV, rcs, dei, ctx.bnumneigh)
        return grcs, gdei, None


class _VirialSrBackward(torch.autograd.Function):
    @staticmethod
    def forward(ctx, gV, rcs, dei, bnumneigh):
        ctx.save_for_backward(gV, rcs, dei)
        ctx.bnumneigh = bnumneigh
        gd, gr = _fvt_virial_bwd_raw(bnumneigh, rcs.contiguous(), dei.contiguous(), gV, True, True)
        return gr, gd

    @staticmethod
    def backward(ctx, ggr, ggd):
        gV, rcs, dei = ctx.saved_tensors
        nn = ctx.bnumneigh
        # d/dgV: - sum ggd (x) rcs - sum dei (x) ggr, i.e. two forward virials
        d_gV = _VirialSr.apply(rcs, ggd, nn) + _VirialSr.apply(ggr, dei, nn)
        # d/drcs[.,b] = - sum_a gV[a,b] ggd[.,a];  d/ddei[.,a] = - sum_b gV[a,b] ggr[.,b]
        d_rcs, _ = _VirialSrBackward.apply(gV, rcs, ggd, nn)
        _, d_dei = _VirialSrBackward.apply(gV, ggr, dei, nn)
        return d_gV, d_rcs, d_dei, None


def VirialSrOp(bnumneigh, brcs, umax_num_neighs, bdei_drij):
    """[virial[B, 3, 3]], differentiable w.r.t. brcs and bdei_drij;
    fvt_sr_op_bind.cc:31-46, src/virial_sr_op.cc:10-164."""
    _req(isinstance(bdei_drij, torch.Tensor) and bdei_drij.is_cuda,
         "bdei_drij must be a tensor on a HIP device: this build has no CPU path")
    dtype, device = bdei_drij.dtype, bdei_drij.device
    _req(dtype in (torch.float32, torch.float64), "bdei_drij must be float32 or float64")
    _check_int("bnumneigh", bnumneigh, device)
    _req(isinstance(brcs, torch.Tensor) and brcs.dtype == dtype and brcs.device == device,
         "brcs must match bdei_drij in dtype and device")
    _req(bdei_drij.dim() == 4 and bdei_drij.shape[3] == 3 and brcs.shape == bdei_drij.shape,
         "brcs and bdei_drij must have shape [B, nlocal, umax, 3]")
    B, P, U, _ = bdei_drij.shape
    _req(int(umax_num_neighs) == U and tuple(bnumneigh.shape) == (B, P), "shapes do not match")
    if bnumneigh.numel():
        _req(int(bnumneigh.max().item()) <= U, "a neighbour count exceeds umax_num_neighs")
    return [_VirialSr.apply(brcs, bdei_drij, bnumneigh)]
