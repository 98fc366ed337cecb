// libnnmtp_bind.so -- registers torch.ops.nnmtp.* with the reference's schemas
// (source/descriptor/nnmtp/bind/nnmtp_bind.cc:27-430) on top of libai2pot_hip.so:
// set_ai2pot_path, mtpParamOp, nnMtpToEFVOp, nnMtpToEFOp, nnMtpToEsitesOp, nnMtpToDescriptorsOp,
// nnMtpToLossOp and nnMtpToEFLossOp (autograd to coeffs, w0, w1, type_bias as
// src/nnMtpOp.cc:2748-2780, 4170-4330).
// The loss operators evaluate the reference's backward formulas, which are not the complete
// derivative of the loss (see include/ai2pot_hip.h, a2p_nnmtp_loss_*); with the environment variable
// A2P_NNMTP_EXACT_GRADIENT=1 they return the complete derivative instead.
#include "mtp_bind_common.h"

#include <cstdlib>

namespace {

#define NNMTP_ARGS int64_t K, const at::Tensor& coeffs, const at::Tensor& w0, const at::Tensor& w1, \
    const at::Tensor& bias, int64_t n_moms, const at::Tensor& basic, const at::Tensor& times, \
    const at::Tensor& mapping, int64_t nmus, const at::Tensor& binum, const at::Tensor& bilist, \
    const at::Tensor& bnumneigh, const at::Tensor& bfirstneigh, const at::Tensor& brcs, \
    const at::Tensor& btypes, const at::Tensor& type_map, int64_t nghost, double rmax, double rmin, \
    const at::Tensor& q_shifter, const at::Tensor& q_scaler, double zbl_rmax, double zbl_rmin, \
    const at::Tensor& zbl_cks, const at::Tensor& zbl_dks
#define NNMTP_PASS K, coeffs, w0, w1, bias, n_moms, basic, times, mapping, nmus, binum, bilist, bnumneigh, \
    bfirstneigh, brcs, btypes, type_map, nghost, rmax, rmin, q_shifter, q_scaler

// want_e: E and F (and V with want_v); want_es: the site energies
variable_list nnmtp_run(bool want_e, bool want_v, bool want_es, int64_t K, const at::Tensor& coeffs,
                        const at::Tensor& w0, const at::Tensor& w1, const at::Tensor& bias, int64_t n_moms,
                        const at::Tensor& basic, const at::Tensor& times, const at::Tensor& mapping, int64_t nmus,
                        const at::Tensor& binum, const at::Tensor& bilist, const at::Tensor& bnumneigh,
                        const at::Tensor& bfirstneigh, const at::Tensor& brcs, const at::Tensor& btypes,
                        const at::Tensor& type_map, int64_t nghost, double rmax, double rmin,
                        const at::Tensor& q_shifter, const at::Tensor& q_scaler)
{
    Batch s = check_batch(binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, nghost);
    const int ntypes = (int)type_map.numel();
    TORCH_CHECK(ntypes > 0, "type_map is empty");
    for (auto& pr : {std::make_pair(&coeffs, "coeffs"), std::make_pair(&w0, "w0"), std::make_pair(&w1, "w1"),
                     std::make_pair(&bias, "type_bias"), std::make_pair(&q_shifter, "q_shifter"),
                     std::make_pair(&q_scaler, "q_scaler")})
        check_device_float(brcs, *pr.first, pr.second);
    a2p_bind::DeviceGuard guard(brcs);
    PlanEntry plan = get_plan(brcs.device().index(), n_moms, basic, times, mapping);
    TORCH_CHECK(coeffs.numel() == (int64_t)ntypes * ntypes * nmus * K, "coeffs size mismatch");
    TORCH_CHECK(w1.numel() > 0 && w1.numel() % ntypes == 0, "w1 must have ntypes * num_neurons elements");
    const int H = (int)(w1.numel() / ntypes);
    TORCH_CHECK(w0.numel() == (int64_t)ntypes * H * plan.n_scalar,
                "w0 must have ntypes * num_neurons * alpha_scalar_moments elements");
    TORCH_CHECK(q_shifter.numel() == plan.n_scalar && q_scaler.numel() == plan.n_scalar,
                "q_shifter and q_scaler must have alpha_scalar_moments elements");
    TORCH_CHECK(bias.numel() == ntypes, "type_bias size mismatch");
    auto opt = brcs.options();
    at::Tensor e, f, v, es;
    if (want_e) {
        // the library writes every element of the three outputs (forces are zeroed on entry)
        const bool fresh = s.B > 0 && s.P > 0;
        e = fresh ? at::empty({s.B}, opt) : at::zeros({s.B}, opt);
        f = fresh ? at::empty({s.B, s.P + s.nghost, 3}, opt) : at::zeros({s.B, s.P + s.nghost, 3}, opt);
        if (want_v) v = fresh ? at::empty({s.B, 9}, opt) : at::zeros({s.B, 9}, opt);
    }
    if (want_es) es = at::zeros({s.B, s.P}, opt);
    void* st = current_stream(brcs);
    auto call = [&]() -> int {
        int rc;
        if (brcs.scalar_type() == at::kDouble) {
            auto p = [](const at::Tensor& t) { return t.defined() ? t.data_ptr<double>() : nullptr; };
            rc = a2p_nnmtp_efv_f64(plan.handle, (int)K, H, p(coeffs), p(w0), p(w1), p(bias), (int)nmus, ntypes,
                                   p(q_shifter), p(q_scaler), rmax, rmin, s.B, s.P, s.U, s.nghost,
                                   binum.data_ptr<int>(), bilist.data_ptr<int>(), bnumneigh.data_ptr<int>(),
                                   bfirstneigh.data_ptr<int>(), p(brcs), btypes.data_ptr<int>(), p(e), p(f), p(v), p(es),
                                   st);
        } else {
            auto p = [](const at::Tensor& t) { return t.defined() ? t.data_ptr<float>() : nullptr; };
            rc = a2p_nnmtp_efv_f32(plan.handle, (int)K, H, p(coeffs), p(w0), p(w1), p(bias), (int)nmus, ntypes,
                                   p(q_shifter), p(q_scaler), rmax, rmin, s.B, s.P, s.U, s.nghost,
                                   binum.data_ptr<int>(), bilist.data_ptr<int>(), bnumneigh.data_ptr<int>(),
                                   bfirstneigh.data_ptr<int>(), p(brcs), btypes.data_ptr<int>(), p(e), p(f), p(v), p(es),
                                   st);
        }
        return rc;
    };
    run_checked(brcs, binum, bnumneigh, bfirstneigh, s.nghost, call);
    if (want_es) return {es};
    if (want_v) return {e, f, v};
    return {e, f};
}

variable_list nnmtp_descriptors(int64_t K, const at::Tensor& coeffs, int64_t n_moms, const at::Tensor& basic,
                                const at::Tensor& times, const at::Tensor& mapping, int64_t nmus,
                                const at::Tensor& binum, const at::Tensor& bilist, const at::Tensor& bnumneigh,
                                const at::Tensor& bfirstneigh, const at::Tensor& brcs, const at::Tensor& btypes,
                                const at::Tensor& type_map, int64_t nghost, double rmax, double rmin)
{
    // the scalar moments themselves (nnMtp.h:570-645): the linear-MTP kernel at scaling 1
    Batch s = check_batch(binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, nghost);
    const int ntypes = (int)type_map.numel();
    TORCH_CHECK(ntypes > 0, "type_map is empty");
    check_device_float(brcs, coeffs, "coeffs");
    a2p_bind::DeviceGuard guard(brcs);
    PlanEntry plan = get_plan(brcs.device().index(), n_moms, basic, times, mapping);
    TORCH_CHECK(coeffs.numel() == (int64_t)ntypes * ntypes * nmus * K, "coeffs size mismatch");
    auto opt = brcs.options();
    at::Tensor one = at::ones({plan.n_scalar}, opt), zero = at::zeros({ntypes}, opt);
    at::Tensor desc = at::zeros({s.B, s.P, plan.n_scalar}, opt);
    void* st = current_stream(brcs);
    auto call = [&]() -> int {
        int rc;
        if (brcs.scalar_type() == at::kDouble) {
            auto p = [](const at::Tensor& t) { return t.data_ptr<double>(); };
            rc = a2p_mtp_esites_f64(plan.handle, (int)K, 1.0, p(coeffs), p(one), p(zero), (int)nmus, ntypes, p(one), rmax,
                                    rmin, s.B, s.P, s.U, s.nghost, binum.data_ptr<int>(), bilist.data_ptr<int>(),
                                    bnumneigh.data_ptr<int>(), bfirstneigh.data_ptr<int>(), p(brcs),
                                    btypes.data_ptr<int>(), nullptr, p(desc), st);
        } else {
            auto p = [](const at::Tensor& t) { return t.data_ptr<float>(); };
            rc = a2p_mtp_esites_f32(plan.handle, (int)K, 1.0, p(coeffs), p(one), p(zero), (int)nmus, ntypes, p(one), rmax,
                                    rmin, s.B, s.P, s.U, s.nghost, binum.data_ptr<int>(), bilist.data_ptr<int>(),
                                    bnumneigh.data_ptr<int>(), bfirstneigh.data_ptr<int>(), p(brcs),
                                    btypes.data_ptr<int>(), nullptr, p(desc), st);
        }
        return rc;
    };
    run_checked(brcs, binum, bnumneigh, bfirstneigh, s.nghost, call);
    return {desc};
}

// forward: [e_sites[B, P]]; backward: sum over structures and rows of grad * d e_sites / d theta.
// The reference writes its per-row w0 / w1 derivatives without the species offset
// (nnMtp.h:965-971 against the allocation at nnMtpOp.cc:4236-4239), which mis-assigns them for more
// than one species; this returns the derivative itself (identical for a single species).
struct NNEsitesFunction : public torch::autograd::Function<NNEsitesFunction> {
    static variable_list forward(AutogradContext* ctx, int64_t K, const at::Tensor& coeffs, const at::Tensor& w0,
                                 const at::Tensor& w1, const at::Tensor& bias, int64_t n_moms,
                                 const at::Tensor& basic, const at::Tensor& times, const at::Tensor& mapping,
                                 int64_t nmus, const at::Tensor& binum, const at::Tensor& bilist,
                                 const at::Tensor& bnumneigh, const at::Tensor& bfirstneigh, const at::Tensor& brcs,
                                 const at::Tensor& btypes, const at::Tensor& type_map, int64_t nghost, double rmax,
                                 double rmin, const at::Tensor& q_shifter, const at::Tensor& q_scaler)
    {
        variable_list out = nnmtp_run(false, false, true, NNMTP_PASS);
        ctx->save_for_backward({coeffs, w0, w1, bias, basic, times, mapping, binum, bilist, bnumneigh, bfirstneigh,
                                brcs, btypes, type_map, q_shifter, q_scaler});
        ctx->saved_data["K"] = K;
        ctx->saved_data["n_moms"] = n_moms;
        ctx->saved_data["nmus"] = nmus;
        ctx->saved_data["nghost"] = nghost;
        ctx->saved_data["rmax"] = rmax;
        ctx->saved_data["rmin"] = rmin;
        return out;
    }

    static variable_list backward(AutogradContext* ctx, variable_list grads)
    {
        variable_list out(22);                   // one slot per forward argument after ctx
        auto sv = ctx->get_saved_variables();
        const at::Tensor &coeffs = sv[0], &w0 = sv[1], &w1 = sv[2], &bias = sv[3], &brcs = sv[11];
        const int64_t K = ctx->saved_data["K"].toInt(), nmus = ctx->saved_data["nmus"].toInt(),
                      nghost = ctx->saved_data["nghost"].toInt();
        Batch s = check_batch(sv[7], sv[8], sv[9], sv[10], brcs, sv[12], nghost);
        const int ntypes = (int)sv[13].numel();
        a2p_bind::DeviceGuard guard(brcs);
        PlanEntry plan = get_plan(brcs.device().index(), ctx->saved_data["n_moms"].toInt(), sv[4], sv[5], sv[6]);
        const int H = (int)(w1.numel() / ntypes);
        auto opt = brcs.options();
        at::Tensor g = grads[0].contiguous();
        TORCH_CHECK(g.dim() == 2 && g.size(0) == s.B && g.size(1) == s.P, "grad of e_sites must be [B, P]");
        at::Tensor dc = at::zeros({s.B, coeffs.numel()}, opt), d0 = at::zeros({s.B, w0.numel()}, opt),
                   d1 = at::zeros({s.B, w1.numel()}, opt), db = at::zeros({s.B, bias.numel()}, opt);
        const double rmax = ctx->saved_data["rmax"].toDouble(), rmin = ctx->saved_data["rmin"].toDouble();
        void* st = current_stream(brcs);
        int rc;
        if (brcs.scalar_type() == at::kDouble) {
            auto p = [](const at::Tensor& t) { return t.data_ptr<double>(); };
            rc = a2p_nnmtp_esites_bwd_f64(plan.handle, (int)K, H, p(coeffs), p(w0), p(w1), p(bias), (int)nmus, ntypes,
                                          p(sv[14]), p(sv[15]), rmax, rmin, s.B, s.P, s.U, s.nghost,
                                          sv[7].data_ptr<int>(), sv[8].data_ptr<int>(), sv[9].data_ptr<int>(),
                                          sv[10].data_ptr<int>(), p(brcs), sv[12].data_ptr<int>(), p(g), p(dc), p(d0),
                                          p(d1), p(db), st);
        } else {
            auto p = [](const at::Tensor& t) { return t.data_ptr<float>(); };
            rc = a2p_nnmtp_esites_bwd_f32(plan.handle, (int)K, H, p(coeffs), p(w0), p(w1), p(bias), (int)nmus, ntypes,
                                          p(sv[14]), p(sv[15]), rmax, rmin, s.B, s.P, s.U, s.nghost,
                                          sv[7].data_ptr<int>(), sv[8].data_ptr<int>(), sv[9].data_ptr<int>(),
                                          sv[10].data_ptr<int>(), p(brcs), sv[12].data_ptr<int>(), p(g), p(dc), p(d0),
                                          p(d1), p(db), st);
        }
        check_rc(rc);
        out[1] = dc.sum(0).reshape(coeffs.sizes());
        out[2] = d0.sum(0).reshape(w0.sizes());
        out[3] = d1.sum(0).reshape(w1.sizes());
        out[4] = db.sum(0).reshape(bias.sizes());
        return out;
    }
};

// forward: [bloss]; backward: grad_output @ per-structure gradients
struct NNLossFunction : public torch::autograd::Function<NNLossFunction> {
    static variable_list forward(AutogradContext* ctx, bool with_virial, double e_w, double f_w, double v_w,
                                 const at::Tensor& e_dft, const at::Tensor& f_dft, const at::Tensor& v_dft_in,
                                 int64_t K, const at::Tensor& coeffs, const at::Tensor& w0, const at::Tensor& w1,
                                 const at::Tensor& bias, int64_t n_moms, const at::Tensor& basic,
                                 const at::Tensor& times, const at::Tensor& mapping, int64_t nmus,
                                 const at::Tensor& binum, const at::Tensor& bilist, const at::Tensor& bnumneigh,
                                 const at::Tensor& bfirstneigh, const at::Tensor& brcs, const at::Tensor& btypes,
                                 const at::Tensor& type_map, int64_t nghost, double rmax, double rmin,
                                 const at::Tensor& q_shifter, const at::Tensor& q_scaler)
    {
        TORCH_CHECK(nghost == 0, "the loss operator requires nghost == 0, as the reference does");
        Batch s = check_batch(binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, nghost);
        const int ntypes = (int)type_map.numel();
        TORCH_CHECK(ntypes > 0, "type_map is empty");
        for (auto& pr : {std::make_pair(&coeffs, "coeffs"), std::make_pair(&w0, "w0"), std::make_pair(&w1, "w1"),
                         std::make_pair(&bias, "type_bias"), std::make_pair(&q_shifter, "q_shifter"),
                         std::make_pair(&q_scaler, "q_scaler"), std::make_pair(&e_dft, "betot_dft"),
                         std::make_pair(&f_dft, "bforce_dft")})
            check_device_float(brcs, *pr.first, pr.second);
        a2p_bind::DeviceGuard guard(brcs);
        PlanEntry plan = get_plan(brcs.device().index(), n_moms, basic, times, mapping);
        TORCH_CHECK(coeffs.numel() == (int64_t)ntypes * ntypes * nmus * K, "coeffs size mismatch");
        TORCH_CHECK(w1.numel() > 0 && w1.numel() % ntypes == 0, "w1 must have ntypes * num_neurons elements");
        const int H = (int)(w1.numel() / ntypes);
        TORCH_CHECK(w0.numel() == (int64_t)ntypes * H * plan.n_scalar,
                    "w0 must have ntypes * num_neurons * alpha_scalar_moments elements");
        TORCH_CHECK(q_shifter.numel() == plan.n_scalar && q_scaler.numel() == plan.n_scalar,
                    "q_shifter and q_scaler must have alpha_scalar_moments elements");
        TORCH_CHECK(bias.numel() == ntypes, "type_bias size mismatch");
        auto opt = brcs.options();
        const int B = s.B, P = s.P;
        at::Tensor v_dft = with_virial ? v_dft_in : at::zeros({B, 9}, opt);
        check_device_float(brcs, v_dft, "bvirial_dft");
        TORCH_CHECK(e_dft.numel() == B && f_dft.numel() == (int64_t)B * P * 3 && v_dft.numel() == (int64_t)B * 9,
                    "label tensors must have shapes [B], [B, P, 3], [B, 9]");
        const bool need = coeffs.requires_grad() || w0.requires_grad() || w1.requires_grad() || bias.requires_grad();
        at::Tensor bloss = at::zeros({B}, opt), e = at::zeros({B}, opt), f = at::zeros({B, P, 3}, opt),
                   v = at::zeros({B, 9}, opt), dc, d0, d1, db;
        if (need) {
            dc = at::zeros({B, coeffs.numel()}, opt);
            d0 = at::zeros({B, w0.numel()}, opt);
            d1 = at::zeros({B, w1.numel()}, opt);
            db = at::zeros({B, bias.numel()}, opt);
        }
        const char* env = std::getenv("A2P_NNMTP_EXACT_GRADIENT");
        const int exact = env && env[0] == '1';
        void* st = current_stream(brcs);
        auto call = [&]() -> int {
            int rc;
            if (brcs.scalar_type() == at::kDouble) {
                auto p = [](const at::Tensor& t) { return t.defined() ? t.data_ptr<double>() : nullptr; };
                rc = a2p_nnmtp_loss_f64(plan.handle, e_w, f_w, with_virial ? v_w : 0.0, p(e_dft), p(f_dft), p(v_dft), (int)K,
                                        H, p(coeffs), p(w0), p(w1), p(bias), (int)nmus, ntypes, p(q_shifter), p(q_scaler),
                                        rmax, rmin, B, P, s.U, binum.data_ptr<int>(), bilist.data_ptr<int>(),
                                        bnumneigh.data_ptr<int>(), bfirstneigh.data_ptr<int>(), p(brcs),
                                        btypes.data_ptr<int>(), p(bloss), p(e), p(f), p(v), p(dc), p(d0), p(d1), p(db),
                                        exact, st);
            } else {
                auto p = [](const at::Tensor& t) { return t.defined() ? t.data_ptr<float>() : nullptr; };
                rc = a2p_nnmtp_loss_f32(plan.handle, e_w, f_w, with_virial ? v_w : 0.0, p(e_dft), p(f_dft), p(v_dft), (int)K,
                                        H, p(coeffs), p(w0), p(w1), p(bias), (int)nmus, ntypes, p(q_shifter), p(q_scaler),
                                        rmax, rmin, B, P, s.U, binum.data_ptr<int>(), bilist.data_ptr<int>(),
                                        bnumneigh.data_ptr<int>(), bfirstneigh.data_ptr<int>(), p(brcs),
                                        btypes.data_ptr<int>(), p(bloss), p(e), p(f), p(v), p(dc), p(d0), p(d1), p(db),
                                        exact, st);
            }
            return rc;
        };
        run_checked(brcs, binum, bnumneigh, bfirstneigh, 0, call);
        ctx->saved_data["need"] = need;
        if (need) ctx->save_for_backward({dc, d0, d1, db});
        ctx->saved_data["shape_c"] = coeffs.sizes().vec();
        ctx->saved_data["shape_0"] = w0.sizes().vec();
        ctx->saved_data["shape_1"] = w1.sizes().vec();
        ctx->saved_data["shape_b"] = bias.sizes().vec();
        return {bloss};
    }

    static variable_list backward(AutogradContext* ctx, variable_list grads)
    {
        variable_list out(29);                   // one slot per forward argument after ctx
        if (!ctx->saved_data["need"].toBool()) return out;
        auto saved = ctx->get_saved_variables();
        at::Tensor gl = grads[0].contiguous();
        out[8] = torch::matmul(gl, saved[0]).reshape(ctx->saved_data["shape_c"].toIntVector());
        out[9] = torch::matmul(gl, saved[1]).reshape(ctx->saved_data["shape_0"].toIntVector());
        out[10] = torch::matmul(gl, saved[2]).reshape(ctx->saved_data["shape_1"].toIntVector());
        out[11] = torch::matmul(gl, saved[3]).reshape(ctx->saved_data["shape_b"].toIntVector());
        return out;
    }
};

}  // namespace

TORCH_LIBRARY(nnmtp, m)
{
    // no counterpart in the reference: the per-call device status check (one stream synchronisation per
    // call) can be switched off for loops that should run ahead of the device, and asked for explicitly
    m.def("set_validate", [](bool on) { validate_flag() = on; });
    m.def("check_status", [](const at::Tensor& any_device_tensor) {
        DeviceGuard guard(any_device_tensor);
        check_rc(a2p_check_status(current_stream(any_device_tensor)));
    });
    m.def("set_ai2pot_path", [](const std::string& path) { g_ai2pot_path = path; });
    m.def("mtpParamOp", [](int64_t level) -> variable_list { return mtp_param_op(level); });
    m.def("nnMtpToEFVOp", [](NNMTP_ARGS) -> variable_list {
        variable_list out = nnmtp_run(true, true, false, NNMTP_PASS);
        apply_zbl(zbl_rmax, zbl_rmin, zbl_cks, zbl_dks, type_map, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes,
                  nghost, out[0], out[1], out[2]);
        return out;
    });
    m.def("nnMtpToEFOp", [](NNMTP_ARGS) -> variable_list {
        variable_list out = nnmtp_run(true, false, false, NNMTP_PASS);
        apply_zbl(zbl_rmax, zbl_rmin, zbl_cks, zbl_dks, type_map, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes,
                  nghost, out[0], out[1], at::Tensor());
        return out;
    });
    m.def("nnMtpToEsitesOp", [](NNMTP_ARGS) -> variable_list {
        variable_list out = NNEsitesFunction::apply(NNMTP_PASS);
        at::Tensor zb = zbl_esites(zbl_rmax, zbl_rmin, zbl_cks, zbl_dks, type_map, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, nghost);
        if (zb.defined()) out[0] = out[0] + zb;
        return out;
    });
    m.def("nnMtpToDescriptorsOp",
          [](int64_t K, const at::Tensor& coeffs, int64_t n_moms, const at::Tensor& basic, const at::Tensor& times,
             const at::Tensor& mapping, int64_t nmus, const at::Tensor& binum, const at::Tensor& bilist,
             const at::Tensor& bnumneigh, const at::Tensor& bfirstneigh, const at::Tensor& brcs,
             const at::Tensor& btypes, const at::Tensor& type_map, int64_t nghost, double rmax,
             double rmin) -> variable_list {
              return nnmtp_descriptors(K, coeffs, n_moms, basic, times, mapping, nmus, binum, bilist, bnumneigh,
                                       bfirstneigh, brcs, btypes, type_map, nghost, rmax, rmin);
          });
    m.def("nnMtpToLossOp",
          [](double e_w, double f_w, double v_w, const at::Tensor& e_dft, const at::Tensor& f_dft,
             const at::Tensor& v_dft, NNMTP_ARGS) -> variable_list {
              auto lab = zbl_shift_labels(zbl_rmax, zbl_rmin, zbl_cks, zbl_dks, type_map, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, nghost, e_dft, f_dft, v_dft);
              return NNLossFunction::apply(true, e_w, f_w, v_w, lab.e, lab.f, lab.v, NNMTP_PASS);
          });
    m.def("nnMtpToEFLossOp",
          [](double e_w, double f_w, const at::Tensor& e_dft, const at::Tensor& f_dft, NNMTP_ARGS) -> variable_list {
              auto lab = zbl_shift_labels(zbl_rmax, zbl_rmin, zbl_cks, zbl_dks, type_map, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, nghost, e_dft, f_dft, at::Tensor());
              return NNLossFunction::apply(false, e_w, f_w, 0.0, lab.e, lab.f,
                                           at::zeros({e_dft.numel(), 9}, e_dft.options()), NNMTP_PASS);
          });
}
