// Shared helpers of the operator bind libraries (libnep_bind.so, libmtpr_bind.so,
// libfvt_sr_op_bind.so): argument checks with TORCH_CHECK, raw pointers, the current HIP
// stream, and translation of libai2pot_hip status codes into c10::Error.
#pragma once
#include <torch/extension.h>
#include <torch/library.h>
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime_api.h>

#include <cstdlib>

#include "../../../include/ai2pot_hip.h"

namespace a2p_bind {

// Makes the tensor's device current for the duration of a call: libai2pot_hip keeps its
// workspace per current device.
struct DeviceGuard {
    int prev = -1;
    explicit DeviceGuard(const at::Tensor& t)
    {
        TORCH_CHECK(hipGetDevice(&prev) == hipSuccess, "hipGetDevice failed");
        const int want = t.device().index();
        if (want >= 0 && want != prev) {
            TORCH_CHECK(hipSetDevice(want) == hipSuccess, "hipSetDevice failed");
        } else {
            prev = -1;
        }
    }
    ~DeviceGuard() { if (prev >= 0) (void)hipSetDevice(prev); }
};

inline void* current_stream(const at::Tensor& t)
{
    return (void*)c10::hip::getCurrentHIPStream(t.device().index()).stream();
}

inline void check_rc(int rc)
{
    TORCH_CHECK(rc == A2P_OK, "libai2pot_hip error ", rc, ": ", a2p_last_error());
}

inline void check_device_float(const at::Tensor& ref, const at::Tensor& t, const char* name)
{
    TORCH_CHECK(t.defined(), name, " is undefined");
    TORCH_CHECK(t.scalar_type() == ref.scalar_type(), name, " must have the dtype of brcs (", ref.scalar_type(),
                "), got ", t.scalar_type());
    TORCH_CHECK(t.device() == ref.device(), name, " must be on the device of brcs");
    TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
}

inline void check_device_int(const at::Tensor& ref, const at::Tensor& t, const char* name)
{
    TORCH_CHECK(t.defined(), name, " is undefined");
    TORCH_CHECK(t.scalar_type() == at::kInt, name, " must be int32");
    TORCH_CHECK(t.device() == ref.device(), name, " must be on the device of brcs");
    TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
}

struct Batch {
    int B, P, U, nghost;
};

// The 7-tensor neighbour contract (source/descriptor/mtpr/README.md:4-9).
inline Batch check_batch(const at::Tensor& binum, const at::Tensor& bilist, const at::Tensor& bnumneigh,
                         const at::Tensor& bfirstneigh, const at::Tensor& brcs, const at::Tensor& btypes,
                         int64_t nghost)
{
    TORCH_CHECK(brcs.is_cuda(), "brcs must be on a HIP device: this build has no CPU path");
    TORCH_CHECK(brcs.scalar_type() == at::kFloat || brcs.scalar_type() == at::kDouble,
                "brcs must be float32 or float64");
    TORCH_CHECK(brcs.is_contiguous() && brcs.dim() == 4 && brcs.size(3) == 3, "brcs must be contiguous [B, P, U, 3]");
    check_device_int(brcs, binum, "binum");
    check_device_int(brcs, bilist, "bilist");
    check_device_int(brcs, bnumneigh, "bnumneigh");
    check_device_int(brcs, bfirstneigh, "bfirstneigh");
    check_device_int(brcs, btypes, "btypes");
    Batch s{(int)brcs.size(0), (int)brcs.size(1), (int)brcs.size(2), (int)nghost};
    TORCH_CHECK(nghost >= 0, "nghost must be non-negative");
    TORCH_CHECK(bfirstneigh.dim() == 3 && bfirstneigh.size(0) == s.B && bfirstneigh.size(1) == s.P &&
                    bfirstneigh.size(2) == s.U, "bfirstneigh must have shape [B, P, U]");
    TORCH_CHECK(bilist.numel() == (int64_t)s.B * s.P && bnumneigh.numel() == (int64_t)s.B * s.P,
                "bilist and bnumneigh must have shape [B, P]");
    TORCH_CHECK(binum.numel() == s.B, "binum must have shape [B]");
    TORCH_CHECK(btypes.numel() == (int64_t)s.B * (s.P + s.nghost), "btypes must have shape [B, P + nghost]");
    return s;
}

// Validation switch of an operator library: on (the default), every call ends by reading the device
// status word, which synchronises the stream; off (set_validate(false), or AI2POT_HIP_VALIDATE=0 in
// the environment), calls only enqueue work and a caller checks when it chooses to
// (torch.ops.<lib>.check_status()).  A loop of calls can then run ahead of the device.
inline bool& validate_flag()
{
    static bool on = [] {
        const char* env = std::getenv("AI2POT_HIP_VALIDATE");
        return !(env && env[0] == '0');
    }();
    return on;
}

// Errors the reference leaves to a commented-out assert (source/nblist/include/neighborList.h:550)
// or to out-of-bounds reads; one device status read per call.
inline void check_device_status(const at::Tensor& t)
{
    if (validate_flag()) check_rc(a2p_check_status(current_stream(t)));
}

// Runs an energy / force / virial (or loss) call and, with validation on, reads the device status.
// A list that names an atom more often than a row is long (half lists, ghosts collecting the pairs of
// several rows) overflows the fixed reduction segments of the fast kernels: the status says so and
// the call is repeated once with segments sized for the list at hand.
template <class Call>
inline void run_checked(const at::Tensor& brcs, const at::Tensor& binum, const at::Tensor& bnumneigh,
                        const at::Tensor& bfirstneigh, int nghost, Call&& call)
{
    check_rc(call());
    if (!validate_flag()) return;
    void* st = current_stream(brcs);
    int rc = a2p_check_status(st);
    if (rc == A2P_ERR_SEGMENT) {
        int most = 0;
        check_rc(a2p_pair_incoming_max((int)brcs.size(0), (int)brcs.size(1), (int)brcs.size(2), nghost,
                                       binum.data_ptr<int>(), bnumneigh.data_ptr<int>(), bfirstneigh.data_ptr<int>(),
                                       &most, st));
        const int old = a2p_pair_segment_capacity(most);
        rc = call();
        if (rc == A2P_OK) rc = a2p_check_status(st);
        a2p_pair_segment_capacity(old);
    }
    check_rc(rc);
}

// Adds the ZBL pair repulsion onto a model's E/F/V when zbl_rmax > 0, as the reference's operators
// do on the device (correction/gpu/include/zbl.cuh:422-620); v may be undefined.
inline void apply_zbl(double zbl_rmax, double zbl_rmin, const at::Tensor& cks, const at::Tensor& dks,
                      const at::Tensor& type_map, const at::Tensor& binum, const at::Tensor& bilist,
                      const at::Tensor& bnumneigh, const at::Tensor& bfirstneigh, const at::Tensor& brcs,
                      const at::Tensor& btypes, int64_t nghost, at::Tensor e, at::Tensor f, at::Tensor v)
{
    if (zbl_rmax == 0.0) return;
    const int ntypes = (int)type_map.numel();
    check_device_float(brcs, cks, "zbl_cks");
    check_device_float(brcs, dks, "zbl_dks");
    TORCH_CHECK(cks.numel() == (int64_t)ntypes * ntypes * 4 && dks.numel() == (int64_t)ntypes * ntypes * 4,
                "zbl_cks and zbl_dks must have ntypes * ntypes * 4 elements");
    at::Tensor tm = type_map.to(brcs.device(), at::kInt).contiguous();
    DeviceGuard guard(brcs);
    const int B = (int)brcs.size(0), P = (int)brcs.size(1), U = (int)brcs.size(2);
    void* st = current_stream(brcs);
    int rc;
    if (brcs.scalar_type() == at::kDouble) {
        auto p = [](const at::Tensor& t) { return t.defined() ? t.data_ptr<double>() : nullptr; };
        rc = a2p_zbl_correct_f64(zbl_rmax, zbl_rmin, p(cks), p(dks), ntypes, tm.data_ptr<int>(), B, P, U, (int)nghost,
                                 binum.data_ptr<int>(), bilist.data_ptr<int>(), bnumneigh.data_ptr<int>(),
                                 bfirstneigh.data_ptr<int>(), p(brcs), btypes.data_ptr<int>(), p(e), p(f), p(v), st);
    } else {
        auto p = [](const at::Tensor& t) { return t.defined() ? t.data_ptr<float>() : nullptr; };
        rc = a2p_zbl_correct_f32(zbl_rmax, zbl_rmin, p(cks), p(dks), ntypes, tm.data_ptr<int>(), B, P, U, (int)nghost,
                                 binum.data_ptr<int>(), bilist.data_ptr<int>(), bnumneigh.data_ptr<int>(),
                                 bfirstneigh.data_ptr<int>(), p(brcs), btypes.data_ptr<int>(), p(e), p(f), p(v), st);
    }
    check_rc(rc);
    check_device_status(brcs);
}

// Per-row ZBL energies [B, P] of the site-energy operators (GroupZBL::correct_e_sites, zbl.h:625-685): half of
// every pair energy of the row's centre atom; undefined when zbl_rmax == 0.  The reference's CPU operators add the
// term and then assign the rows (linearMtp.h:598), which loses it; here the rows keep it.
inline at::Tensor zbl_esites(double zbl_rmax, double zbl_rmin, const at::Tensor& cks, const at::Tensor& dks,
                             const at::Tensor& type_map, const at::Tensor& binum, const at::Tensor& bilist,
                             const at::Tensor& bnumneigh, const at::Tensor& bfirstneigh, const at::Tensor& brcs,
                             const at::Tensor& btypes, int64_t nghost)
{
    if (zbl_rmax == 0.0) return at::Tensor();
    const int ntypes = (int)type_map.numel();
    check_device_float(brcs, cks, "zbl_cks");
    check_device_float(brcs, dks, "zbl_dks");
    TORCH_CHECK(cks.numel() == (int64_t)ntypes * ntypes * 4 && dks.numel() == (int64_t)ntypes * ntypes * 4,
                "zbl_cks and zbl_dks must have ntypes * ntypes * 4 elements");
    TORCH_CHECK(brcs.dim() == 4, "brcs must have shape [B, P, U, 3]");
    at::Tensor tm = type_map.to(brcs.device(), at::kInt).contiguous();
    DeviceGuard guard(brcs);
    const int B = (int)brcs.size(0), P = (int)brcs.size(1), U = (int)brcs.size(2);
    at::Tensor out = at::zeros({B, P}, brcs.options());
    void* st = current_stream(brcs);
    int rc;
    if (brcs.scalar_type() == at::kDouble)
        rc = a2p_zbl_esites_f64(zbl_rmax, zbl_rmin, cks.data_ptr<double>(), dks.data_ptr<double>(), ntypes,
                                tm.data_ptr<int>(), B, P, U, (int)nghost, binum.data_ptr<int>(), bilist.data_ptr<int>(),
                                bnumneigh.data_ptr<int>(), bfirstneigh.data_ptr<int>(), brcs.data_ptr<double>(),
                                btypes.data_ptr<int>(), out.data_ptr<double>(), st);
    else
        rc = a2p_zbl_esites_f32(zbl_rmax, zbl_rmin, cks.data_ptr<float>(), dks.data_ptr<float>(), ntypes,
                                tm.data_ptr<int>(), B, P, U, (int)nghost, binum.data_ptr<int>(), bilist.data_ptr<int>(),
                                bnumneigh.data_ptr<int>(), bfirstneigh.data_ptr<int>(), brcs.data_ptr<float>(),
                                btypes.data_ptr<int>(), out.data_ptr<float>(), st);
    check_rc(rc);
    check_device_status(brcs);
    return out;
}

// Labels of a loss operator with the ZBL pair repulsion taken out.  The correction does not depend
// on the model parameters, so model + ZBL - label = model - (label - ZBL): the loss, its RMSEs and
// its gradients are those of the operator without ZBL on the shifted labels.  The reference adds
// the correction to E/F/V before the loss and before its gradient (e.g. nepOp.cc:2552-2575,
// 3127-3150).  v_dft may be undefined (operators without virial labels).
struct ShiftedLabels {
    at::Tensor e, f, v;
};
inline ShiftedLabels zbl_shift_labels(double zbl_rmax, double zbl_rmin, const at::Tensor& cks, const at::Tensor& dks,
                                      const at::Tensor& type_map, const at::Tensor& binum, const at::Tensor& bilist,
                                      const at::Tensor& bnumneigh, const at::Tensor& bfirstneigh,
                                      const at::Tensor& brcs, const at::Tensor& btypes, int64_t nghost,
                                      const at::Tensor& e_dft, const at::Tensor& f_dft, const at::Tensor& v_dft)
{
    ShiftedLabels out{e_dft, f_dft, v_dft};
    if (zbl_rmax == 0.0) return out;
    TORCH_CHECK(nghost == 0, "the loss operator requires nghost == 0, as the reference does");
    TORCH_CHECK(brcs.dim() == 4, "brcs must have shape [B, P, U, 3]");
    check_device_float(brcs, e_dft, "betot_dft");
    check_device_float(brcs, f_dft, "bforce_dft");
    if (v_dft.defined()) check_device_float(brcs, v_dft, "bvirial_dft");
    const int64_t B = brcs.size(0), P = brcs.size(1);
    TORCH_CHECK(e_dft.numel() == B && f_dft.numel() == B * P * 3 && (!v_dft.defined() || v_dft.numel() == B * 9),
                "label shapes do not match the batch");
    auto opt = brcs.options();
    at::Tensor e0 = at::zeros({B}, opt), f0 = at::zeros({B, P, 3}, opt), v0;
    if (v_dft.defined()) v0 = at::zeros({B, 9}, opt);
    apply_zbl(zbl_rmax, zbl_rmin, cks, dks, type_map, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, 0, e0, f0, v0);
    out.e = e_dft.detach().reshape({B}) - e0;
    out.f = f_dft.detach().reshape({B, P, 3}) - f0;
    if (v_dft.defined()) out.v = v_dft.detach().reshape({B, 9}) - v0;
    return out;
}

}  // namespace a2p_bind
