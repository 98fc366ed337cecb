"""Neighbour list with the reference's ``nblist`` module interface.

``find_info4mlff(lattice, types, coords, rcut, umax, is_cart, pbc_xyz, sort)`` takes and
returns NumPy arrays exactly like the reference's CPython extension
(source/nblist/bind/nblist_bind.cc:35-189): positional arguments, the same type checks
(``TypeError`` otherwise), dtype of lattice/coords selecting float32 or float64, int32 or
int64 types, and the 7-tuple ``(inum, ilist, numneigh, firstneigh, rcs, types, nghost)``.
The list is built on the GPU (libai2pot_hip.so); unlike the reference, a neighbour count
above ``umax`` raises instead of overrunning the arrays.

``find_info4mlff_device`` is the same operation on tensors already resident on the device,
for molecular dynamics loops that rebuild the list every step without leaving the GPU.
"""
import ctypes

import numpy as np
import torch

from . import _lib

_c = ctypes


def _build(lattice_np, types_t, coords_t, rcut, umax, is_cart, pbc, sort, check=True):
    device = coords_t.device
    dtype = coords_t.dtype
    n = coords_t.shape[0]
    npdt = np.float32 if dtype == torch.float32 else np.float64
    lat = np.ascontiguousarray(lattice_np, npdt).reshape(9)
    pbc_i = np.ascontiguousarray([1 if bool(x) else 0 for x in pbc], np.int32)
    ilist = torch.empty(n, dtype=torch.int32, device=device)
    numneigh = torch.empty(n, dtype=torch.int32, device=device)
    firstneigh = torch.empty((n, umax), dtype=torch.int32, device=device)
    rcs = torch.empty((n, umax, 3), dtype=dtype, device=device)
    types_out = torch.empty(n, dtype=torch.int32, device=device)
    max_nn = _c.c_int(0)
    L = _lib.lib()
    fn = L.a2p_nblist_build_f32 if dtype == torch.float32 else L.a2p_nblist_build_f64
    with torch.cuda.device(device):
        rc = fn(lat.ctypes.data_as(_c.c_void_p), _c.c_void_p(types_t.data_ptr()),
                _c.c_void_p(coords_t.data_ptr()), _c.c_int(n), _c.c_double(float(rcut)),
                _c.c_int(int(umax)), _c.c_int(1 if is_cart else 0), pbc_i.ctypes.data_as(_c.c_void_p),
                _c.c_int(1 if sort else 0), _c.c_void_p(ilist.data_ptr()),
                _c.c_void_p(numneigh.data_ptr()), _c.c_void_p(firstneigh.data_ptr()),
                _c.c_void_p(rcs.data_ptr()), _c.c_void_p(types_out.data_ptr()),
                _c.byref(max_nn) if check else None,
                _c.c_void_p(torch.cuda.current_stream(device).cuda_stream))
    _lib.check(rc)
    return ilist, numneigh, firstneigh, rcs, types_out, max_nn.value


def find_info4mlff_device(lattice, types, coords, rcut, umax, is_cart=True, pbc_xyz=(True, True, True),
                          sort=False, check=True):
    """Device-resident variant: ``types`` int32[N] and ``coords`` float[N, 3] are tensors on a
    HIP device, ``lattice`` a 3x3 host array.  Returns (inum, ilist, numneigh, firstneigh, rcs,
    types, nghost) with tensors on the same device.  With check=False the overflow check is
    deferred (no final synchronisation); call ai2pot_amd._lib.check_status later."""
    if not (isinstance(coords, torch.Tensor) and coords.is_cuda):
        raise RuntimeError("coords must be a tensor on a HIP device")
    if coords.dtype not in (torch.float32, torch.float64) or coords.dim() != 2 or coords.shape[1] != 3:
        raise RuntimeError("coords must be float32 or float64 of shape [N, 3]")
    if types.dtype != torch.int32 or types.device != coords.device or types.shape != (coords.shape[0],):
        raise RuntimeError("types must be int32[N] on the device of coords")
    if not (coords.is_contiguous() and types.is_contiguous()):
        raise RuntimeError("coords and types must be contiguous")
    if coords.shape[0] == 0:
        raise RuntimeError("the structure has no atoms")
    lat = lattice.detach().cpu().numpy() if isinstance(lattice, torch.Tensor) else np.asarray(lattice)
    ilist, numneigh, firstneigh, rcs, types_out, _ = _build(lat, types, coords, rcut, umax, is_cart,
                                                            pbc_xyz, sort, check)
    return coords.shape[0], ilist, numneigh, firstneigh, rcs, types_out, 0


def find_info4mlff(lattice, types, coords, rcut, umax, is_cart, pbc_xyz, sort):
    if not (isinstance(lattice, np.ndarray) and isinstance(types, np.ndarray) and
            isinstance(coords, np.ndarray) and isinstance(rcut, float) and
            isinstance(umax, int) and not isinstance(umax, bool) and isinstance(is_cart, bool) and
            isinstance(pbc_xyz, list) and isinstance(sort, bool)):
        raise TypeError("Please check the parameter in interface of py_find_info4mlff().")
    if coords.dtype not in (np.float32, np.float64) or lattice.dtype != coords.dtype:
        raise TypeError("lattice and coords must share dtype float32 or float64")
    if types.dtype not in (np.int32, np.int64):
        raise TypeError("types must be int32 or int64")
    if len(pbc_xyz) != 3:
        raise TypeError("pbc_xyz must have three entries")
    n = coords.shape[0]
    if n == 0:
        raise RuntimeError("the structure has no atoms")
    dev = torch.device("cuda", torch.cuda.current_device())
    coords_t = torch.from_numpy(np.ascontiguousarray(coords).reshape(n, 3)).to(dev)
    types_t = torch.from_numpy(np.ascontiguousarray(types.astype(np.int32))).to(dev)
    ilist, numneigh, firstneigh, rcs, types_out, _ = _build(lattice, types_t, coords_t, rcut, umax, is_cart,
                                                            pbc_xyz, sort, True)
    return (n, ilist.cpu().numpy(), numneigh.cpu().numpy(), firstneigh.cpu().numpy(), rcs.cpu().numpy(),
            types_out.cpu().numpy(), 0)
