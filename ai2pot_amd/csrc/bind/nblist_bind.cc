// libnblist_bind.so -- the neighbour list as registered operators on device tensors.
//
// The reference's only neighbour-list entry point is the CPython function
// nblist.find_info4mlff(lattice, types, coords, rcut, umax, is_cart, pbc_xyz, sort) on NumPy arrays
// (source/nblist/bind/nblist_bind.cc:35-189; loaded by ai2pot/fromcc/__init__.py:53-134), which this
// repository also ships (nblist_module.cc).  A molecular-dynamics loop that keeps its positions on
// the GPU would pay two PCIe copies of the padded arrays per step through it, so the same operation
// is registered here with the same arguments and the same seven results, as tensors:
//   torch.ops.nblist.find_info4mlff(lattice, types, coords, rcut, umax, is_cart, pbc_xyz, sort)
//       -> [inum[1], ilist[N], numneigh[N], firstneigh[N, umax], rcs[N, umax, 3], types[N], nghost[1]]
//   torch.ops.nblist.find_info4mlff_(... same ..., ilist, numneigh, firstneigh, rcs, types_out, update)
//       writes into the caller's tensors (update = true: they hold an earlier result, rows are rewritten
//       only as far as their old or new length reaches)
//   torch.ops.nblist.set_sync_free(bool)   builds without a host synchronisation (a2p_nblist_sync_free)
//   torch.ops.nblist.compact_bytes / find_info4mlff_compact_   the build that also cuts the compact
//       lists torch.ops.nep.nepToEFVCompactOp consumes (include/ai2pot_hip.h: a2p_nblist_build_compact_*)
// lattice is a 3x3 tensor of the dtype of coords, on the host (preferred) or on the device (copied to the
// host, which synchronises); types int32[N] and coords [N, 3] are device tensors.  Results are
// bit-identical to the reference's in both sort modes.  A neighbour count above umax raises (with
// validation on; the reference overruns its arrays, neighborList.h:550).
#include "bind_common.h"

using namespace a2p_bind;

namespace {

struct ListArgs {
    at::Tensor lattice_host;
    int pbc[3];
    int N;
    bool f32;
};

ListArgs check_list_args(const at::Tensor& lattice, const at::Tensor& types, const at::Tensor& coords, int64_t umax,
                         const c10::List<bool>& pbc_xyz)
{
    TORCH_CHECK(coords.is_cuda(), "coords must be on a HIP device: this build has no CPU path");
    TORCH_CHECK(coords.scalar_type() == at::kFloat || coords.scalar_type() == at::kDouble,
                "coords must be float32 or float64");
    TORCH_CHECK(coords.dim() == 2 && coords.size(1) == 3 && coords.is_contiguous(), "coords must be contiguous [N, 3]");
    TORCH_CHECK(coords.size(0) > 0, "the structure has no atoms");
    TORCH_CHECK(lattice.numel() == 9 && lattice.scalar_type() == coords.scalar_type(),
                "lattice must have 9 elements of the dtype of coords");
    check_device_int(coords, types, "types");
    TORCH_CHECK(types.numel() == coords.size(0), "types must have one entry per atom");
    TORCH_CHECK(pbc_xyz.size() == 3, "pbc_xyz must have three entries");
    TORCH_CHECK(umax > 0, "umax must be positive");
    ListArgs a;
    a.lattice_host = lattice.to(at::kCPU).contiguous();
    for (int i = 0; i < 3; i++) a.pbc[i] = pbc_xyz[i] ? 1 : 0;
    a.N = (int)coords.size(0);
    a.f32 = coords.scalar_type() == at::kFloat;
    return a;
}

void check_outputs(const at::Tensor& coords, int64_t umax, const at::Tensor& ilist, const at::Tensor& numneigh,
                   const at::Tensor& firstneigh, const at::Tensor& rcs, const at::Tensor& types_out)
{
    const int64_t N = coords.size(0);
    check_device_int(coords, ilist, "ilist");
    check_device_int(coords, numneigh, "numneigh");
    check_device_int(coords, firstneigh, "firstneigh");
    check_device_int(coords, types_out, "types_out");
    check_device_float(coords, rcs, "rcs");
    TORCH_CHECK(ilist.numel() == N && numneigh.numel() == N && types_out.numel() == N, "ilist, numneigh and types_out must have N elements");
    TORCH_CHECK(firstneigh.numel() == N * umax && rcs.numel() == N * umax * 3, "firstneigh must be [N, umax] and rcs [N, umax, 3]");
}

void build_into(const ListArgs& a, const at::Tensor& types, const at::Tensor& coords, double rcut, int64_t umax,
                bool is_cart, bool sort, bool update, at::Tensor ilist, at::Tensor numneigh, at::Tensor firstneigh,
                at::Tensor rcs, at::Tensor types_out)
{
    DeviceGuard guard(coords);
    void* st = current_stream(coords);
    int rc;
    if (a.f32) {
        auto fn = update ? a2p_nblist_update_f32 : a2p_nblist_build_f32;
        rc = fn(a.lattice_host.data_ptr<float>(), types.data_ptr<int>(), coords.data_ptr<float>(), a.N, rcut, (int)umax,
                is_cart ? 1 : 0, a.pbc, sort ? 1 : 0, ilist.data_ptr<int>(), numneigh.data_ptr<int>(),
                firstneigh.data_ptr<int>(), rcs.data_ptr<float>(), types_out.data_ptr<int>(), nullptr, st);
    } else {
        auto fn = update ? a2p_nblist_update_f64 : a2p_nblist_build_f64;
        rc = fn(a.lattice_host.data_ptr<double>(), types.data_ptr<int>(), coords.data_ptr<double>(), a.N, rcut, (int)umax,
                is_cart ? 1 : 0, a.pbc, sort ? 1 : 0, ilist.data_ptr<int>(), numneigh.data_ptr<int>(),
                firstneigh.data_ptr<int>(), rcs.data_ptr<double>(), types_out.data_ptr<int>(), nullptr, st);
    }
    check_rc(rc);
    check_device_status(coords);
}

void list_out(const at::Tensor& lattice, const at::Tensor& types, const at::Tensor& coords, double rcut, int64_t umax,
              bool is_cart, c10::List<bool> pbc_xyz, bool sort, at::Tensor ilist, at::Tensor numneigh,
              at::Tensor firstneigh, at::Tensor rcs, at::Tensor types_out, bool update)
{
    const ListArgs a = check_list_args(lattice, types, coords, umax, pbc_xyz);
    check_outputs(coords, umax, ilist, numneigh, firstneigh, rcs, types_out);
    build_into(a, types, coords, rcut, umax, is_cart, sort, update, ilist, numneigh, firstneigh, rcs, types_out);
}

void compact_out(const at::Tensor& lattice, const at::Tensor& types, const at::Tensor& coords, double rcut, int64_t umax,
             bool is_cart, c10::List<bool> pbc_xyz, double rcut_outer, double rcut_inner, int64_t update,
             const c10::optional<at::Tensor>& ilist, const c10::optional<at::Tensor>& numneigh,
             const c10::optional<at::Tensor>& firstneigh, const c10::optional<at::Tensor>& rcs,
             const c10::optional<at::Tensor>& types_out, at::Tensor compact)
{
    const ListArgs a = check_list_args(lattice, types, coords, umax, pbc_xyz);
    const bool rows = ilist.has_value();
    TORCH_CHECK(rows == numneigh.has_value() && rows == firstneigh.has_value() && rows == rcs.has_value() &&
                    rows == types_out.has_value(), "the padded outputs come all or none");
    if (rows) check_outputs(coords, umax, *ilist, *numneigh, *firstneigh, *rcs, *types_out);
    const size_t need = a2p_nblist_compact_bytes(a.N, (int)umax, a.f32 ? 4 : 8);
    TORCH_CHECK(need > 0, "compact lists need umax % 8 == 0 and fewer than 2^28 atoms");
    TORCH_CHECK(compact.is_cuda() && compact.device() == coords.device() && compact.is_contiguous() &&
                    (size_t)compact.nbytes() >= need,
                "compact must be a contiguous device tensor of at least compact_bytes(natoms, umax, itemsize) bytes");
    DeviceGuard guard(coords);
    void* st = current_stream(coords);
    int rc;
    if (a.f32)
        rc = a2p_nblist_build_compact_f32(a.lattice_host.data_ptr<float>(), types.data_ptr<int>(),
                                          coords.data_ptr<float>(), a.N, rcut, (int)umax, is_cart ? 1 : 0, a.pbc,
                                          (int)update, rcut_outer, rcut_inner,
                                          rows ? ilist->data_ptr<int>() : nullptr,
                                          rows ? numneigh->data_ptr<int>() : nullptr,
                                          rows ? firstneigh->data_ptr<int>() : nullptr,
                                          rows ? rcs->data_ptr<float>() : nullptr,
                                          rows ? types_out->data_ptr<int>() : nullptr, compact.data_ptr(), st);
    else
        rc = a2p_nblist_build_compact_f64(a.lattice_host.data_ptr<double>(), types.data_ptr<int>(),
                                          coords.data_ptr<double>(), a.N, rcut, (int)umax, is_cart ? 1 : 0, a.pbc,
                                          (int)update, rcut_outer, rcut_inner,
                                          rows ? ilist->data_ptr<int>() : nullptr,
                                          rows ? numneigh->data_ptr<int>() : nullptr,
                                          rows ? firstneigh->data_ptr<int>() : nullptr,
                                          rows ? rcs->data_ptr<double>() : nullptr,
                                          rows ? types_out->data_ptr<int>() : nullptr, compact.data_ptr(), st);
    check_rc(rc);
    check_device_status(coords);
}

}  // namespace

TORCH_LIBRARY(nblist, m)
{
    m.def("set_validate", [](bool on) { validate_flag() = on; });
    m.def("check_status", [](const at::Tensor& any_device_tensor) {
        DeviceGuard guard(any_device_tensor);
        check_rc(a2p_check_status(current_stream(any_device_tensor)));
    });
    // builds of a structure seen before size their bin grid from that build's bound and never wait for the stream
    // (include/ai2pot_hip.h: a2p_nblist_sync_free; per host thread); returns the previous setting
    m.def("set_sync_free", [](bool on) -> bool { return a2p_nblist_sync_free(on ? 1 : 0) != 0; });
    m.def("find_info4mlff",
          [](const at::Tensor& lattice, const at::Tensor& types, const at::Tensor& coords, double rcut, int64_t umax,
             bool is_cart, c10::List<bool> pbc_xyz, bool sort) -> std::vector<at::Tensor> {
              const ListArgs a = check_list_args(lattice, types, coords, umax, pbc_xyz);
              auto iopt = coords.options().dtype(at::kInt);
              at::Tensor ilist = at::empty({a.N}, iopt), numneigh = at::empty({a.N}, iopt),
                         firstneigh = at::empty({a.N, umax}, iopt), rcs = at::empty({a.N, umax, 3}, coords.options()),
                         types_out = at::empty({a.N}, iopt);
              build_into(a, types, coords, rcut, umax, is_cart, sort, false, ilist, numneigh, firstneigh, rcs, types_out);
              return {at::full({1}, a.N, iopt), ilist, numneigh, firstneigh, rcs, types_out, at::zeros({1}, iopt)};
          });
    m.def("find_info4mlff_(Tensor lattice, Tensor types, Tensor coords, float rcut, int umax, bool is_cart, bool[] pbc_xyz, "
          "bool sort, Tensor(a!) ilist, Tensor(b!) numneigh, Tensor(c!) firstneigh, Tensor(d!) rcs, Tensor(e!) types_out, "
          "bool update) -> ()", &list_out);
    m.def("compact_bytes", [](int64_t natoms, int64_t umax, int64_t elem_size) -> int64_t {
        return (int64_t)a2p_nblist_compact_bytes((int)natoms, (int)umax, (int)elem_size);
    });
    // update: bit 0 = the padded tensors hold an earlier result, bit 1 = keep the processing order in `compact`.
    // The five padded tensors are optional (all or none).
    m.def("find_info4mlff_compact_(Tensor lattice, Tensor types, Tensor coords, float rcut, int umax, bool is_cart, "
          "bool[] pbc_xyz, float rcut_outer, float rcut_inner, int update, Tensor(a!)? ilist, Tensor(b!)? numneigh, "
          "Tensor(c!)? firstneigh, Tensor(d!)? rcs, Tensor(e!)? types_out, Tensor(f!) compact) -> ()", &compact_out);
}
