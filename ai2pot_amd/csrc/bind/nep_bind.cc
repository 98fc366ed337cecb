// libnep_bind.so -- registers torch.ops.nep.* with the reference's schemas
// (source/descriptor/nep/bind/nep_bind.cc:23-312) on top of libai2pot_hip.so.
// nepToEFOp / nepToEFVOp / nepToDescriptorsOp run on the GPU; like the reference's, they are
// inference operators: no gradient flows to any input (src/nepOp.cc:1287-1312).
// The NEP training-loss operators are registered with their reference signatures and raise.
#include "bind_common.h"

using namespace a2p_bind;
using torch::autograd::variable_list;

namespace {

struct NepModel {
    int K, n_r, n_a, l_max, H, ntypes, D;
};

NepModel check_model(int64_t K, int64_t n_r, int64_t n_a, int64_t l_max, const at::Tensor& coeffs,
                     const at::Tensor& w0, const at::Tensor& b0, const at::Tensor& w1, const at::Tensor& bias,
                     const at::Tensor& type_map, const at::Tensor& brcs)
{
    NepModel m;
    m.K = (int)K; m.n_r = (int)n_r; m.n_a = (int)n_a; m.l_max = (int)l_max;
    m.ntypes = (int)type_map.numel();                                  // nepOp.cc:978-981
    TORCH_CHECK(m.ntypes > 0, "type_map is empty");
    TORCH_CHECK(l_max >= 0 && l_max <= 4, "l_max must be in [0, 4]");  // nep_utilities.h:46
    check_device_float(brcs, coeffs, "coeffs");
    check_device_float(brcs, w0, "w0");
    check_device_float(brcs, b0, "b0");
    check_device_float(brcs, w1, "w1");
    check_device_float(brcs, bias, "type_bias");
    m.H = (int)(w1.numel() / m.ntypes);
    m.D = l_max == 0 ? m.n_r : m.n_r + m.n_a * m.l_max;
    TORCH_CHECK(m.H > 0 && w0.numel() == (int64_t)m.ntypes * m.H * m.D, "w0 must have ntypes*H*D elements");
    TORCH_CHECK(b0.numel() == (int64_t)m.ntypes * m.H && bias.numel() == m.ntypes, "b0 / type_bias size mismatch");
    TORCH_CHECK(coeffs.numel() == (int64_t)m.ntypes * m.ntypes * (m.n_r + m.n_a) * m.K, "coeffs size mismatch");
    return m;
}

variable_list nep_run(bool want_virial, bool want_desc, int64_t K, int64_t n_r, int64_t n_a, int64_t l_max,
                      const at::Tensor& coeffs, const at::Tensor& w0, const at::Tensor& b0, const at::Tensor& w1,
                      const at::Tensor& bias, const at::Tensor& binum, const at::Tensor& bilist,
                      const at::Tensor& bnumneigh, const at::Tensor& bfirstneigh, const at::Tensor& brcs,
                      const at::Tensor& btypes, const at::Tensor& type_map, int64_t nghost, double rr, double ra,
                      const at::Tensor& q_scaler)
{
    Batch s = check_batch(binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, nghost);
    NepModel m = check_model(K, n_r, n_a, l_max, coeffs, w0, b0, w1, bias, type_map, brcs);
    check_device_float(brcs, q_scaler, "q_scaler");
    TORCH_CHECK(q_scaler.numel() == m.D, "q_scaler must have ", m.D, " elements");
    a2p_bind::DeviceGuard guard(brcs);
    auto opt = brcs.options();
    at::Tensor e, f, v, d;
    if (want_desc) d = at::zeros({s.B, s.P, m.D}, opt);
    else {
        e = at::zeros({s.B}, opt);
        f = at::zeros({s.B, s.P + s.nghost, 3}, opt);
        if (want_virial) v = at::zeros({s.B, 9}, opt);
    }
    void* st = current_stream(brcs);
    int rc;
    if (brcs.scalar_type() == at::kFloat) {
        rc = a2p_nep_efv_f32(m.K, m.n_r, m.n_a, m.l_max, m.H, m.ntypes, coeffs.data_ptr<float>(),
                             w0.data_ptr<float>(), b0.data_ptr<float>(), w1.data_ptr<float>(),
                             bias.data_ptr<float>(), q_scaler.data_ptr<float>(), rr, ra, s.B, s.P, s.U, s.nghost,
                             binum.data_ptr<int>(), bilist.data_ptr<int>(), bnumneigh.data_ptr<int>(),
                             bfirstneigh.data_ptr<int>(), brcs.data_ptr<float>(), btypes.data_ptr<int>(),
                             e.defined() ? e.data_ptr<float>() : nullptr, f.defined() ? f.data_ptr<float>() : nullptr,
                             v.defined() ? v.data_ptr<float>() : nullptr, d.defined() ? d.data_ptr<float>() : nullptr,
                             st);
    } else {
        rc = a2p_nep_efv_f64(m.K, m.n_r, m.n_a, m.l_max, m.H, m.ntypes, coeffs.data_ptr<double>(),
                             w0.data_ptr<double>(), b0.data_ptr<double>(), w1.data_ptr<double>(),
                             bias.data_ptr<double>(), q_scaler.data_ptr<double>(), rr, ra, s.B, s.P, s.U, s.nghost,
                             binum.data_ptr<int>(), bilist.data_ptr<int>(), bnumneigh.data_ptr<int>(),
                             bfirstneigh.data_ptr<int>(), brcs.data_ptr<double>(), btypes.data_ptr<int>(),
                             e.defined() ? e.data_ptr<double>() : nullptr,
                             f.defined() ? f.data_ptr<double>() : nullptr,
                             v.defined() ? v.data_ptr<double>() : nullptr,
                             d.defined() ? d.data_ptr<double>() : nullptr, st);
    }
    check_rc(rc);
    check_device_status(brcs);
    if (want_desc) return {d};
    if (want_virial) return {e, f, v};
    return {e, f};
}

}  // namespace

TORCH_LIBRARY(nep, m)
{
    m.def("nepToEFOp",
          [](int64_t K, int64_t n_r, int64_t n_a, int64_t l_max, const at::Tensor& coeffs, const at::Tensor& w0,
             const at::Tensor& b0, const at::Tensor& w1, const at::Tensor& bias, const at::Tensor& binum,
             const at::Tensor& bilist, const at::Tensor& bnumneigh, const at::Tensor& bfirstneigh,
             const at::Tensor& brcs, const at::Tensor& btypes, const at::Tensor& type_map, int64_t nghost,
             double rr, double ra, const at::Tensor& q_scaler, double zbl_rmax, double zbl_rmin,
             const at::Tensor& zbl_cks, const at::Tensor& zbl_dks) -> variable_list {
              require_no_zbl(zbl_rmax);
              return nep_run(false, false, K, n_r, n_a, l_max, coeffs, w0, b0, w1, bias, binum, bilist, bnumneigh,
                             bfirstneigh, brcs, btypes, type_map, nghost, rr, ra, q_scaler);
          });
    m.def("nepToEFVOp",
          [](int64_t K, int64_t n_r, int64_t n_a, int64_t l_max, const at::Tensor& coeffs, const at::Tensor& w0,
             const at::Tensor& b0, const at::Tensor& w1, const at::Tensor& bias, const at::Tensor& binum,
             const at::Tensor& bilist, const at::Tensor& bnumneigh, const at::Tensor& bfirstneigh,
             const at::Tensor& brcs, const at::Tensor& btypes, const at::Tensor& type_map, int64_t nghost,
             double rr, double ra, const at::Tensor& q_scaler, double zbl_rmax, double zbl_rmin,
             const at::Tensor& zbl_cks, const at::Tensor& zbl_dks) -> variable_list {
              require_no_zbl(zbl_rmax);
              return nep_run(true, false, K, n_r, n_a, l_max, coeffs, w0, b0, w1, bias, binum, bilist, bnumneigh,
                             bfirstneigh, brcs, btypes, type_map, nghost, rr, ra, q_scaler);
          });
    m.def("nepToLossOp",
          [](double e_w, double f_w, double v_w, const at::Tensor& e_dft, const at::Tensor& f_dft,
             const at::Tensor& v_dft, int64_t K, int64_t n_r, int64_t n_a, int64_t l_max, const at::Tensor& coeffs,
             const at::Tensor& w0, const at::Tensor& b0, const at::Tensor& w1, const at::Tensor& bias,
             const at::Tensor& binum, const at::Tensor& bilist, const at::Tensor& bnumneigh,
             const at::Tensor& bfirstneigh, const at::Tensor& brcs, const at::Tensor& btypes,
             const at::Tensor& type_map, int64_t nghost, double rr, double ra, const at::Tensor& q_scaler,
             double zbl_rmax, double zbl_rmin, const at::Tensor& zbl_cks,
             const at::Tensor& zbl_dks) -> variable_list {
              TORCH_CHECK(false, "nepToLossOp (NEP training loss) is not implemented in this build");
              return {};
          });
    m.def("nepToEFLossOp",
          [](double e_w, double f_w, const at::Tensor& e_dft, const at::Tensor& f_dft, int64_t K, int64_t n_r,
             int64_t n_a, int64_t l_max, const at::Tensor& coeffs, const at::Tensor& w0, const at::Tensor& b0,
             const at::Tensor& w1, const at::Tensor& bias, const at::Tensor& binum, const at::Tensor& bilist,
             const at::Tensor& bnumneigh, const at::Tensor& bfirstneigh, const at::Tensor& brcs,
             const at::Tensor& btypes, const at::Tensor& type_map, int64_t nghost, double rr, double ra,
             const at::Tensor& q_scaler, double zbl_rmax, double zbl_rmin, const at::Tensor& zbl_cks,
             const at::Tensor& zbl_dks) -> variable_list {
              TORCH_CHECK(false, "nepToEFLossOp (NEP training loss) is not implemented in this build");
              return {};
          });
    m.def("nepToDescriptorsOp",
          [](int64_t K, int64_t n_r, int64_t n_a, int64_t l_max, const at::Tensor& coeffs, const at::Tensor& binum,
             const at::Tensor& bilist, const at::Tensor& bnumneigh, const at::Tensor& bfirstneigh,
             const at::Tensor& brcs, const at::Tensor& btypes, const at::Tensor& type_map, int64_t nghost,
             double rr, double ra) -> variable_list {
              // descriptors do not involve the network: one zero neuron per species
              const int64_t nt = type_map.numel();
              const int64_t D = l_max == 0 ? n_r : n_r + n_a * l_max;
              auto opt = brcs.options();
              return nep_run(false, true, K, n_r, n_a, l_max, coeffs, at::zeros({nt * D}, opt), at::zeros({nt}, opt),
                             at::zeros({nt}, opt), at::zeros({nt}, opt), binum, bilist, bnumneigh, bfirstneigh, brcs,
                             btypes, type_map, nghost, rr, ra, at::ones({D}, opt));
          });
}
