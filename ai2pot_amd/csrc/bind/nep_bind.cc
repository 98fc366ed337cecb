// libnep_bind.so -- registers torch.ops.nep.* with the reference's schemas
// (source/descriptor/nep/bind/nep_bind.cc:23-312) on top of libai2pot_hip.so.
// nepToEFOp / nepToEFVOp / nepToDescriptorsOp are inference operators like the reference's: no
// gradient flows to any input (src/nepOp.cc:1287-1312).  nepToLossOp / nepToEFLossOp return the
// per-structure loss and the RMSEs and back-propagate grad_output @ dloss/dtheta to coeffs, w0,
// b0, w1 and type_bias (src/nepOp.cc:2359-3484); the gradients are produced by the forward call
// and kept, where the reference recomputes E/F/V in backward.
#include "bind_common.h"

using namespace a2p_bind;
using torch::autograd::variable_list;

namespace {

struct NepModel {
    int K, n_r, n_a, l_max, H, ntypes, D;
};

NepModel check_model(int64_t K, int64_t n_r, int64_t n_a, int64_t l_max, const at::Tensor& coeffs,
                     const at::Tensor& w0, const at::Tensor& b0, const at::Tensor& w1, const at::Tensor& bias,
                     const at::Tensor& type_map, const at::Tensor& brcs, int64_t l4 = 0, int64_t l5 = 0)
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
    TORCH_CHECK((l4 == 0 || l4 == 2) && (l5 == 0 || l5 == 1) && l_max >= l4 && l_max >= l5,
                "l_4body must be 0 or 2, l_5body 0 or 1, and l_max at least as large");
    m.D = l_max == 0 ? m.n_r : m.n_r + m.n_a * (m.l_max + (l4 ? 1 : 0) + (l5 ? 1 : 0));
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
                      const at::Tensor& q_scaler, int64_t l4 = 0, int64_t l5 = 0)
{
    Batch s = check_batch(binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, nghost);
    NepModel m = check_model(K, n_r, n_a, l_max, coeffs, w0, b0, w1, bias, type_map, brcs, l4, l5);
    check_device_float(brcs, q_scaler, "q_scaler");
    TORCH_CHECK(q_scaler.numel() == m.D, "q_scaler must have ", m.D, " elements");
    a2p_bind::DeviceGuard guard(brcs);
    auto opt = brcs.options();
    at::Tensor e, f, v, d;
    if (want_desc) d = at::zeros({s.B, s.P, m.D}, opt);
    else {
        // the library writes every element of the three outputs (forces are zeroed on entry)
        const bool fresh = s.B > 0 && s.P > 0;
        e = fresh ? at::empty({s.B}, opt) : at::zeros({s.B}, opt);
        f = fresh ? at::empty({s.B, s.P + s.nghost, 3}, opt) : at::zeros({s.B, s.P + s.nghost, 3}, opt);
        if (want_virial) v = fresh ? at::empty({s.B, 9}, opt) : at::zeros({s.B, 9}, opt);
    }
    void* st = current_stream(brcs);
    auto call = [&]() -> int {
        int rc;
        if (l4 || l5) {        // the extension with four- / five-body invariants: its own entry points
            if (brcs.scalar_type() == at::kFloat)
                rc = a2p_nep_efv_manybody_f32(m.K, m.n_r, m.n_a, m.l_max, (int)l4, (int)l5, m.H, m.ntypes,
                                              coeffs.data_ptr<float>(), w0.data_ptr<float>(), b0.data_ptr<float>(),
                                              w1.data_ptr<float>(), bias.data_ptr<float>(), q_scaler.data_ptr<float>(), rr,
                                              ra, s.B, s.P, s.U, s.nghost, binum.data_ptr<int>(), bilist.data_ptr<int>(),
                                              bnumneigh.data_ptr<int>(), bfirstneigh.data_ptr<int>(),
                                              brcs.data_ptr<float>(), btypes.data_ptr<int>(), e.data_ptr<float>(),
                                              f.data_ptr<float>(), v.data_ptr<float>(), nullptr, st);
            else
                rc = a2p_nep_efv_manybody_f64(m.K, m.n_r, m.n_a, m.l_max, (int)l4, (int)l5, m.H, m.ntypes,
                                              coeffs.data_ptr<double>(), w0.data_ptr<double>(), b0.data_ptr<double>(),
                                              w1.data_ptr<double>(), bias.data_ptr<double>(), q_scaler.data_ptr<double>(),
                                              rr, ra, s.B, s.P, s.U, s.nghost, binum.data_ptr<int>(),
                                              bilist.data_ptr<int>(), bnumneigh.data_ptr<int>(),
                                              bfirstneigh.data_ptr<int>(), brcs.data_ptr<double>(), btypes.data_ptr<int>(),
                                              e.data_ptr<double>(), f.data_ptr<double>(), v.data_ptr<double>(), nullptr, st);
        } else if (brcs.scalar_type() == at::kFloat) {
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
        return rc;
    };
    run_checked(brcs, binum, bnumneigh, bfirstneigh, s.nghost, call);
    if (want_desc) return {d};
    if (want_virial) return {e, f, v};
    return {e, f};
}

// Energy, forces and virial of ONE periodic structure from the compact lists cut by
// torch.ops.nblist.find_info4mlff_compact_ (no counterpart in the reference: its operators take the
// padded 7-tensor contract only).  The forces are a gather over each atom's own list, without
// atomics; see include/ai2pot_hip.h, a2p_nep_efv_compact_*.
variable_list nep_run_compact(int64_t K, int64_t n_r, int64_t n_a, int64_t l_max, const at::Tensor& coeffs,
                              const at::Tensor& w0, const at::Tensor& b0, const at::Tensor& w1, const at::Tensor& bias,
                              const at::Tensor& types, const at::Tensor& compact, int64_t umax,
                              const at::Tensor& type_map, double rr, double ra, const at::Tensor& q_scaler)
{
    TORCH_CHECK(coeffs.is_cuda() && (coeffs.scalar_type() == at::kFloat || coeffs.scalar_type() == at::kDouble),
                "coeffs must be a float32 or float64 tensor on a HIP device");
    NepModel m = check_model(K, n_r, n_a, l_max, coeffs, w0, b0, w1, bias, type_map, coeffs);
    check_device_float(coeffs, q_scaler, "q_scaler");
    TORCH_CHECK(q_scaler.numel() == m.D, "q_scaler must have ", m.D, " elements");
    check_device_int(coeffs, types, "types");
    const int N = (int)types.numel();
    const bool f32 = coeffs.scalar_type() == at::kFloat;
    TORCH_CHECK(a2p_nep_efv_compact_supported(m.K, m.n_r, m.n_a, m.l_max, m.H, m.ntypes, f32 ? 4 : 8) == 1,
                "nepToEFVCompactOp covers chebyshev_size 8, n_radial 4 or 6, n_angular 4, l_max 4, at most 4 species; "
                "use nepToEFVOp for this model");
    const size_t need = a2p_nblist_compact_bytes(N, (int)umax, f32 ? 4 : 8);
    TORCH_CHECK(need > 0 && compact.is_cuda() && compact.device() == coeffs.device() && compact.is_contiguous() &&
                    (size_t)compact.nbytes() >= need,
                "compact must be the device buffer filled by find_info4mlff_compact_ for these natoms and umax");
    a2p_bind::DeviceGuard guard(coeffs);
    auto opt = coeffs.options();
    at::Tensor e = at::empty({1}, opt), f = at::empty({1, N, 3}, opt), v = at::empty({1, 9}, opt);
    void* st = current_stream(coeffs);
    int rc;
    if (f32)
        rc = a2p_nep_efv_compact_f32(m.K, m.n_r, m.n_a, m.l_max, m.H, m.ntypes, coeffs.data_ptr<float>(),
                                     w0.data_ptr<float>(), b0.data_ptr<float>(), w1.data_ptr<float>(),
                                     bias.data_ptr<float>(), q_scaler.data_ptr<float>(), rr, ra, N, (int)umax,
                                     types.data_ptr<int>(), compact.data_ptr(), e.data_ptr<float>(),
                                     f.data_ptr<float>(), v.data_ptr<float>(), st);
    else
        rc = a2p_nep_efv_compact_f64(m.K, m.n_r, m.n_a, m.l_max, m.H, m.ntypes, coeffs.data_ptr<double>(),
                                     w0.data_ptr<double>(), b0.data_ptr<double>(), w1.data_ptr<double>(),
                                     bias.data_ptr<double>(), q_scaler.data_ptr<double>(), rr, ra, N, (int)umax,
                                     types.data_ptr<int>(), compact.data_ptr(), e.data_ptr<double>(),
                                     f.data_ptr<double>(), v.data_ptr<double>(), st);
    check_rc(rc);
    check_device_status(coeffs);
    return {e, f, v};
}

struct NepLossFunction : public torch::autograd::Function<NepLossFunction> {
    static variable_list forward(torch::autograd::AutogradContext* ctx, bool with_virial, double e_w, double f_w,
                                 double v_w, const at::Tensor& e_dft, const at::Tensor& f_dft,
                                 const at::Tensor& v_dft_in, int64_t K, int64_t n_r, int64_t n_a, int64_t l_max,
                                 const at::Tensor& coeffs, const at::Tensor& w0, const at::Tensor& b0,
                                 const at::Tensor& w1, const at::Tensor& bias, const at::Tensor& binum,
                                 const at::Tensor& bilist, const at::Tensor& bnumneigh, const at::Tensor& bfirstneigh,
                                 const at::Tensor& brcs, const at::Tensor& btypes, const at::Tensor& type_map,
                                 int64_t nghost, double rr, double ra, const at::Tensor& q_scaler)
    {
        TORCH_CHECK(nghost == 0, "the loss operator requires nghost == 0, as the reference does");
        Batch s = check_batch(binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, nghost);
        NepModel m = check_model(K, n_r, n_a, l_max, coeffs, w0, b0, w1, bias, type_map, brcs);
        check_device_float(brcs, q_scaler, "q_scaler");
        TORCH_CHECK(q_scaler.numel() == m.D, "q_scaler must have ", m.D, " elements");
        a2p_bind::DeviceGuard guard(brcs);
        auto opt = brcs.options();
        const int B = s.B, P = s.P;
        at::Tensor v_dft = with_virial ? v_dft_in : at::zeros({B, 9}, opt);
        check_device_float(brcs, e_dft, "betot_dft");
        check_device_float(brcs, f_dft, "bforce_dft");
        check_device_float(brcs, v_dft, "bvirial_dft");
        TORCH_CHECK(e_dft.numel() == B && f_dft.numel() == (int64_t)B * P * 3 && v_dft.numel() == (int64_t)B * 9,
                    "label tensors must have shapes [B], [B, P, 3], [B, 9]");
        const bool need = coeffs.requires_grad() || w0.requires_grad() || b0.requires_grad() ||
                          w1.requires_grad() || bias.requires_grad();
        // the library writes every element of these outputs when the batch is not empty
        auto out = [&](at::IntArrayRef shape) { return B > 0 && P > 0 ? at::empty(shape, opt) : at::zeros(shape, opt); };
        at::Tensor bloss = out({B}), rmse = out({3}), e = out({B}), f = out({B, P, 3}), v = out({B, 9}), dc, dw0, db0, dw1, db;
        if (need) {
            dc = out({B, coeffs.numel()});
            dw0 = out({B, w0.numel()});
            db0 = out({B, b0.numel()});
            dw1 = out({B, w1.numel()});
            db = out({B, bias.numel()});
        }
        void* st = current_stream(brcs);
        auto call = [&]() -> int {
            int rc;
            if (brcs.scalar_type() == at::kDouble) {
                auto p = [](const at::Tensor& t) { return t.defined() ? t.data_ptr<double>() : nullptr; };
                rc = a2p_nep_loss_f64(e_w, f_w, with_virial ? v_w : 0.0, p(e_dft), p(f_dft), p(v_dft), m.K, m.n_r, m.n_a,
                                      m.l_max, m.H, m.ntypes, p(coeffs), p(w0), p(b0), p(w1), p(bias), p(q_scaler), rr, ra,
                                      B, P, s.U, binum.data_ptr<int>(), bilist.data_ptr<int>(), bnumneigh.data_ptr<int>(),
                                      bfirstneigh.data_ptr<int>(), p(brcs), btypes.data_ptr<int>(), p(bloss), p(rmse),
                                      p(e), p(f), p(v), p(dc), p(dw0), p(db0), p(dw1), p(db), st);
            } else {
                auto p = [](const at::Tensor& t) { return t.defined() ? t.data_ptr<float>() : nullptr; };
                rc = a2p_nep_loss_f32(e_w, f_w, with_virial ? v_w : 0.0, p(e_dft), p(f_dft), p(v_dft), m.K, m.n_r, m.n_a,
                                      m.l_max, m.H, m.ntypes, p(coeffs), p(w0), p(b0), p(w1), p(bias), p(q_scaler), rr, ra,
                                      B, P, s.U, binum.data_ptr<int>(), bilist.data_ptr<int>(), bnumneigh.data_ptr<int>(),
                                      bfirstneigh.data_ptr<int>(), p(brcs), btypes.data_ptr<int>(), p(bloss), p(rmse),
                                      p(e), p(f), p(v), p(dc), p(dw0), p(db0), p(dw1), p(db), st);
            }
            return rc;
        };
        run_checked(brcs, binum, bnumneigh, bfirstneigh, 0, call);
        ctx->saved_data["need"] = need;
        if (need) ctx->save_for_backward({dc, dw0, db0, dw1, db});
        ctx->saved_data["shape_c"] = coeffs.sizes().vec();
        ctx->saved_data["shape_w0"] = w0.sizes().vec();
        ctx->saved_data["shape_b0"] = b0.sizes().vec();
        ctx->saved_data["shape_w1"] = w1.sizes().vec();
        ctx->saved_data["shape_b"] = bias.sizes().vec();
        if (with_virial)
            return {bloss, rmse.slice(0, 0, 1).clone(), rmse.slice(0, 1, 2).clone(), rmse.slice(0, 2, 3).clone()};
        return {bloss, rmse.slice(0, 0, 1).clone(), rmse.slice(0, 1, 2).clone()};
    }

    static variable_list backward(torch::autograd::AutogradContext* ctx, variable_list grads)
    {
        variable_list out(27);                   // one slot per forward argument after ctx
        if (!ctx->saved_data["need"].toBool()) return out;
        auto saved = ctx->get_saved_variables();
        at::Tensor gl = grads[0].contiguous();
        const char* keys[5] = {"shape_c", "shape_w0", "shape_b0", "shape_w1", "shape_b"};
        for (int i = 0; i < 5; i++)              // coeffs, w0, b0, w1, type_bias are arguments 11..15
            out[11 + i] = torch::matmul(gl, saved[i]).reshape(ctx->saved_data[keys[i]].toIntVector());
        return out;
    }
};

}  // namespace

TORCH_LIBRARY(nep, m)
{
    m.def("nepToEFVCompactOp", &nep_run_compact);
    // no counterpart in the reference: the per-call device status check (one stream synchronisation per
    // call) can be switched off for loops that should run ahead of the device, and asked for explicitly
    m.def("set_validate", [](bool on) { validate_flag() = on; });
    m.def("check_status", [](const at::Tensor& any_device_tensor) {
        DeviceGuard guard(any_device_tensor);
        check_rc(a2p_check_status(current_stream(any_device_tensor)));
    });
    m.def("nepToEFOp",
          [](int64_t K, int64_t n_r, int64_t n_a, int64_t l_max, const at::Tensor& coeffs, const at::Tensor& w0,
             const at::Tensor& b0, const at::Tensor& w1, const at::Tensor& bias, const at::Tensor& binum,
             const at::Tensor& bilist, const at::Tensor& bnumneigh, const at::Tensor& bfirstneigh,
             const at::Tensor& brcs, const at::Tensor& btypes, const at::Tensor& type_map, int64_t nghost,
             double rr, double ra, const at::Tensor& q_scaler, double zbl_rmax, double zbl_rmin,
             const at::Tensor& zbl_cks, const at::Tensor& zbl_dks) -> variable_list {
              variable_list out = nep_run(false, false, K, n_r, n_a, l_max, coeffs, w0, b0, w1, bias, binum, bilist,
                                          bnumneigh, bfirstneigh, brcs, btypes, type_map, nghost, rr, ra, q_scaler);
              apply_zbl(zbl_rmax, zbl_rmin, zbl_cks, zbl_dks, type_map, binum, bilist, bnumneigh, bfirstneigh, brcs,
                        btypes, nghost, out[0], out[1], at::Tensor());
              return out;
          });
    m.def("nepToEFVOp",
          [](int64_t K, int64_t n_r, int64_t n_a, int64_t l_max, const at::Tensor& coeffs, const at::Tensor& w0,
             const at::Tensor& b0, const at::Tensor& w1, const at::Tensor& bias, const at::Tensor& binum,
             const at::Tensor& bilist, const at::Tensor& bnumneigh, const at::Tensor& bfirstneigh,
             const at::Tensor& brcs, const at::Tensor& btypes, const at::Tensor& type_map, int64_t nghost,
             double rr, double ra, const at::Tensor& q_scaler, double zbl_rmax, double zbl_rmin,
             const at::Tensor& zbl_cks, const at::Tensor& zbl_dks) -> variable_list {
              variable_list out = nep_run(true, false, K, n_r, n_a, l_max, coeffs, w0, b0, w1, bias, binum, bilist,
                                          bnumneigh, bfirstneigh, brcs, btypes, type_map, nghost, rr, ra, q_scaler);
              apply_zbl(zbl_rmax, zbl_rmin, zbl_cks, zbl_dks, type_map, binum, bilist, bnumneigh, bfirstneigh, brcs,
                        btypes, nghost, out[0], out[1], out[2]);
              return out;
          });
    // EXTENSION, no counterpart in the reference (parity unpinned): nepToEFVOp with one four-body (l_4body = 2) and /
    // or one five-body (l_5body = 1) invariant per angular channel; see include/ai2pot_hip.h, a2p_nep_efv_manybody_*
    m.def("nepToEFVManyBodyOp",
          [](int64_t K, int64_t n_r, int64_t n_a, int64_t l_max, int64_t l_4body, int64_t l_5body,
             const at::Tensor& coeffs, const at::Tensor& w0, const at::Tensor& b0, const at::Tensor& w1,
             const at::Tensor& bias, const at::Tensor& binum, const at::Tensor& bilist, const at::Tensor& bnumneigh,
             const at::Tensor& bfirstneigh, const at::Tensor& brcs, const at::Tensor& btypes,
             const at::Tensor& type_map, int64_t nghost, double rr, double ra,
             const at::Tensor& q_scaler) -> variable_list {
              return nep_run(true, false, K, n_r, n_a, l_max, coeffs, w0, b0, w1, bias, binum, bilist, bnumneigh,
                             bfirstneigh, brcs, btypes, type_map, nghost, rr, ra, q_scaler, l_4body, l_5body);
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
              auto lab = zbl_shift_labels(zbl_rmax, zbl_rmin, zbl_cks, zbl_dks, type_map, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, nghost, e_dft, f_dft, v_dft);
              return NepLossFunction::apply(true, e_w, f_w, v_w, lab.e, lab.f, lab.v, K, n_r, n_a, l_max, coeffs, w0,
                                            b0, w1, bias, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes,
                                            type_map, nghost, rr, ra, q_scaler);
          });
    m.def("nepToEFLossOp",
          [](double e_w, double f_w, const at::Tensor& e_dft, const at::Tensor& f_dft, int64_t K, int64_t n_r,
             int64_t n_a, int64_t l_max, const at::Tensor& coeffs, const at::Tensor& w0, const at::Tensor& b0,
             const at::Tensor& w1, const at::Tensor& bias, const at::Tensor& binum, const at::Tensor& bilist,
             const at::Tensor& bnumneigh, const at::Tensor& bfirstneigh, const at::Tensor& brcs,
             const at::Tensor& btypes, const at::Tensor& type_map, int64_t nghost, double rr, double ra,
             const at::Tensor& q_scaler, double zbl_rmax, double zbl_rmin, const at::Tensor& zbl_cks,
             const at::Tensor& zbl_dks) -> variable_list {
              auto lab = zbl_shift_labels(zbl_rmax, zbl_rmin, zbl_cks, zbl_dks, type_map, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, nghost, e_dft, f_dft, at::Tensor());
              return NepLossFunction::apply(false, e_w, f_w, 0.0, lab.e, lab.f, at::zeros({(int64_t)binum.numel(), 9}, brcs.options()),
                                            K, n_r, n_a, l_max, coeffs, w0, b0, w1, bias, binum, bilist, bnumneigh,
                                            bfirstneigh, brcs, btypes, type_map, nghost, rr, ra, q_scaler);
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
