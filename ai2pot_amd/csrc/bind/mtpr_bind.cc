// libmtpr_bind.so -- registers torch.ops.mtpr.* with the reference's schemas
// (source/descriptor/mtpr/bind/mtpr_bind.cc:30-569) on top of libai2pot_hip.so:
// set_ai2pot_path, mtpParamOp, linearMtpToEFVOp, linearMtpToEFOp, linearMtpToLossOp,
// linearMtpToEFLossOp, linearMtpToEsitesOp (autograd to coeffs, linear_coeffs, type_bias only, as
// src/linearMtpOp.cc:1732-1765, 4002-4027), linearMtpToDescriptorsOp, and the linear-solver
// operators LinMatrixLinVectorOp and CoeffsSchmidtOrthOp, and the legacy mtpBasisOp (autograd to coeffs
// and brcs, src/mtpBasisOp.cc:28-326).
#include "mtp_bind_common.h"

namespace {

struct MtpCtx {
    Batch s;
    int ntypes;
    PlanEntry plan;
};

MtpCtx check_mtp(int64_t K, const at::Tensor& coeffs, const at::Tensor& lin, const at::Tensor& bias,
                 int64_t n_moms, const at::Tensor& basic, const at::Tensor& times, const at::Tensor& mapping,
                 int64_t nmus, const at::Tensor& binum, const at::Tensor& bilist, const at::Tensor& bnumneigh,
                 const at::Tensor& bfirstneigh, const at::Tensor& brcs, const at::Tensor& btypes,
                 const at::Tensor& type_map, int64_t nghost, const at::Tensor& q_scaler)
{
    MtpCtx c;
    c.s = check_batch(binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, nghost);
    c.ntypes = (int)type_map.numel();
    TORCH_CHECK(c.ntypes > 0, "type_map is empty");
    check_device_float(brcs, coeffs, "coeffs");
    check_device_float(brcs, lin, "linear_coeffs");
    check_device_float(brcs, bias, "type_bias");
    check_device_float(brcs, q_scaler, "q_scaler");
    a2p_bind::DeviceGuard guard(brcs);
    c.plan = get_plan(brcs.device().index(), n_moms, basic, times, mapping);
    TORCH_CHECK(coeffs.numel() == (int64_t)c.ntypes * c.ntypes * nmus * K, "coeffs size mismatch");
    TORCH_CHECK(lin.numel() == c.plan.n_scalar && q_scaler.numel() == c.plan.n_scalar,
                "linear_coeffs and q_scaler must have alpha_scalar_moments elements");
    TORCH_CHECK(bias.numel() == c.ntypes, "type_bias size mismatch");
    return c;
}

variable_list mtp_efv(bool want_virial, int64_t K, double scaling, const at::Tensor& coeffs,
                      const at::Tensor& lin, const at::Tensor& bias, int64_t n_moms, const at::Tensor& basic,
                      const at::Tensor& times, const at::Tensor& mapping, int64_t nmus, const at::Tensor& binum,
                      const at::Tensor& bilist, const at::Tensor& bnumneigh, const at::Tensor& bfirstneigh,
                      const at::Tensor& brcs, const at::Tensor& btypes, const at::Tensor& type_map, int64_t nghost,
                      double rmax, double rmin, const at::Tensor& q_scaler, double zbl_rmax, double zbl_rmin,
                      const at::Tensor& zbl_cks, const at::Tensor& zbl_dks)
{
    MtpCtx c = check_mtp(K, coeffs, lin, bias, n_moms, basic, times, mapping, nmus, binum, bilist, bnumneigh,
                         bfirstneigh, brcs, btypes, type_map, nghost, q_scaler);
    a2p_bind::DeviceGuard guard(brcs);
    auto opt = brcs.options();
    // the library writes every element of the three outputs (forces are zeroed on entry)
    const bool fresh = c.s.B > 0 && c.s.P > 0;
    at::Tensor e = fresh ? at::empty({c.s.B}, opt) : at::zeros({c.s.B}, opt);
    at::Tensor f = fresh ? at::empty({c.s.B, c.s.P + c.s.nghost, 3}, opt) : at::zeros({c.s.B, c.s.P + c.s.nghost, 3}, opt);
    at::Tensor v;
    if (want_virial) v = fresh ? at::empty({c.s.B, 9}, opt) : at::zeros({c.s.B, 9}, opt);
    void* st = current_stream(brcs);
    auto call = [&]() -> int {
        int rc;
        if (brcs.scalar_type() == at::kDouble)
            rc = a2p_mtp_efv_f64(c.plan.handle, (int)K, scaling, coeffs.data_ptr<double>(), lin.data_ptr<double>(),
                                 bias.data_ptr<double>(), (int)nmus, c.ntypes, q_scaler.data_ptr<double>(), rmax, rmin,
                                 c.s.B, c.s.P, c.s.U, c.s.nghost, binum.data_ptr<int>(), bilist.data_ptr<int>(),
                                 bnumneigh.data_ptr<int>(), bfirstneigh.data_ptr<int>(), brcs.data_ptr<double>(),
                                 btypes.data_ptr<int>(), e.data_ptr<double>(), f.data_ptr<double>(),
                                 v.defined() ? v.data_ptr<double>() : nullptr, st);
        else
            rc = a2p_mtp_efv_f32(c.plan.handle, (int)K, scaling, coeffs.data_ptr<float>(), lin.data_ptr<float>(),
                                 bias.data_ptr<float>(), (int)nmus, c.ntypes, q_scaler.data_ptr<float>(), rmax, rmin,
                                 c.s.B, c.s.P, c.s.U, c.s.nghost, binum.data_ptr<int>(), bilist.data_ptr<int>(),
                                 bnumneigh.data_ptr<int>(), bfirstneigh.data_ptr<int>(), brcs.data_ptr<float>(),
                                 btypes.data_ptr<int>(), e.data_ptr<float>(), f.data_ptr<float>(),
                                 v.defined() ? v.data_ptr<float>() : nullptr, st);
        return rc;
    };
    run_checked(brcs, binum, bnumneigh, bfirstneigh, c.s.nghost, call);
    apply_zbl(zbl_rmax, zbl_rmin, zbl_cks, zbl_dks, type_map, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, nghost,
              e, f, v);
    if (want_virial) return {e, f, v};
    return {e, f};
}

// forward: [bloss, e_rmse, f_rmse(, v_rmse)]; backward: grad_output @ per-structure gradients
struct LossFunction : public torch::autograd::Function<LossFunction> {
    static variable_list forward(AutogradContext* ctx, bool with_virial, double e_w, double f_w, double v_w,
                                 const at::Tensor& e_dft, const at::Tensor& f_dft, const at::Tensor& v_dft_in,
                                 int64_t K, double scaling, const at::Tensor& coeffs, const at::Tensor& lin,
                                 const at::Tensor& bias, int64_t n_moms, const at::Tensor& basic,
                                 const at::Tensor& times, const at::Tensor& mapping, int64_t nmus,
                                 const at::Tensor& binum, const at::Tensor& bilist, const at::Tensor& bnumneigh,
                                 const at::Tensor& bfirstneigh, const at::Tensor& brcs, const at::Tensor& btypes,
                                 const at::Tensor& type_map, int64_t nghost, double rmax, double rmin,
                                 const at::Tensor& q_scaler)
    {
        TORCH_CHECK(nghost == 0, "the loss operator requires nghost == 0, as the reference does");
        MtpCtx c = check_mtp(K, coeffs, lin, bias, n_moms, basic, times, mapping, nmus, binum, bilist, bnumneigh,
                             bfirstneigh, brcs, btypes, type_map, nghost, q_scaler);
        a2p_bind::DeviceGuard guard(brcs);
        auto opt = brcs.options();
        const int B = c.s.B, P = c.s.P;
        at::Tensor v_dft = with_virial ? v_dft_in : at::zeros({B, 9}, opt);
        check_device_float(brcs, e_dft, "betot_dft");
        check_device_float(brcs, f_dft, "bforce_dft");
        check_device_float(brcs, v_dft, "bvirial_dft");
        TORCH_CHECK(e_dft.numel() == B && f_dft.numel() == (int64_t)B * P * 3 && v_dft.numel() == (int64_t)B * 9,
                    "label tensors must have shapes [B], [B, P, 3], [B, 9]");
        const bool need = coeffs.requires_grad() || lin.requires_grad() || bias.requires_grad();
        // the library writes every element of these outputs when the batch is not empty
        auto out = [&](at::IntArrayRef shape) { return B > 0 && P > 0 ? at::empty(shape, opt) : at::zeros(shape, opt); };
        at::Tensor bloss = out({B}), rmse = out({3}), e = out({B}), f = out({B, P, 3}), v = out({B, 9}), dc, dl, db;
        if (need) {
            dc = out({B, coeffs.numel()});
            dl = out({B, lin.numel()});
            db = out({B, bias.numel()});
        }
        void* st = current_stream(brcs);
        auto call = [&]() -> int {
            int rc;
            if (brcs.scalar_type() == at::kDouble) {
                auto p = [](const at::Tensor& t) { return t.defined() ? t.data_ptr<double>() : nullptr; };
                rc = a2p_mtp_loss_f64(c.plan.handle, e_w, f_w, with_virial ? v_w : 0.0, p(e_dft), p(f_dft), p(v_dft),
                                      (int)K, scaling, p(coeffs), p(lin), p(bias), (int)nmus, c.ntypes, p(q_scaler),
                                      rmax, rmin, B, P, c.s.U, binum.data_ptr<int>(), bilist.data_ptr<int>(),
                                      bnumneigh.data_ptr<int>(), bfirstneigh.data_ptr<int>(), p(brcs),
                                      btypes.data_ptr<int>(), p(bloss), p(rmse), p(e), p(f), p(v), p(dc), p(dl), p(db),
                                      st);
            } else {
                auto p = [](const at::Tensor& t) { return t.defined() ? t.data_ptr<float>() : nullptr; };
                rc = a2p_mtp_loss_f32(c.plan.handle, e_w, f_w, with_virial ? v_w : 0.0, p(e_dft), p(f_dft), p(v_dft),
                                      (int)K, scaling, p(coeffs), p(lin), p(bias), (int)nmus, c.ntypes, p(q_scaler),
                                      rmax, rmin, B, P, c.s.U, binum.data_ptr<int>(), bilist.data_ptr<int>(),
                                      bnumneigh.data_ptr<int>(), bfirstneigh.data_ptr<int>(), p(brcs),
                                      btypes.data_ptr<int>(), p(bloss), p(rmse), p(e), p(f), p(v), p(dc), p(dl), p(db),
                                      st);
            }
            return rc;
        };
        run_checked(brcs, binum, bnumneigh, bfirstneigh, 0, call);
        ctx->saved_data["need"] = need;
        if (need) ctx->save_for_backward({dc, dl, db});
        ctx->saved_data["shape_c"] = coeffs.sizes().vec();
        ctx->saved_data["shape_l"] = lin.sizes().vec();
        ctx->saved_data["shape_b"] = bias.sizes().vec();
        if (with_virial) return {bloss, rmse.slice(0, 0, 1).clone(), rmse.slice(0, 1, 2).clone(), rmse.slice(0, 2, 3).clone()};
        return {bloss, rmse.slice(0, 0, 1).clone(), rmse.slice(0, 1, 2).clone()};
    }

    static variable_list backward(AutogradContext* ctx, variable_list grads)
    {
        variable_list out(28);                   // one slot per forward argument after ctx
        if (!ctx->saved_data["need"].toBool()) return out;
        auto saved = ctx->get_saved_variables();
        at::Tensor gl = grads[0].contiguous();
        out[9] = torch::matmul(gl, saved[0]).reshape(ctx->saved_data["shape_c"].toIntVector());
        out[10] = torch::matmul(gl, saved[1]).reshape(ctx->saved_data["shape_l"].toIntVector());
        out[11] = torch::matmul(gl, saved[2]).reshape(ctx->saved_data["shape_b"].toIntVector());
        return out;
    }
};

// e_sites[B, P] and / or descriptors[B, P, S] of one batch
void run_esites(const MtpCtx& c, int64_t K, double scaling, const at::Tensor& coeffs, const at::Tensor& lin,
                const at::Tensor& bias, int64_t nmus, const at::Tensor& binum, const at::Tensor& bilist,
                const at::Tensor& bnumneigh, const at::Tensor& bfirstneigh, const at::Tensor& brcs,
                const at::Tensor& btypes, double rmax, double rmin, const at::Tensor& q_scaler, at::Tensor es,
                at::Tensor desc)
{
    a2p_bind::DeviceGuard guard(brcs);
    void* st = current_stream(brcs);
    auto call = [&]() -> int {
        int rc;
        if (brcs.scalar_type() == at::kDouble) {
            auto p = [](const at::Tensor& t) { return t.defined() ? t.data_ptr<double>() : nullptr; };
            rc = a2p_mtp_esites_f64(c.plan.handle, (int)K, scaling, p(coeffs), p(lin), p(bias), (int)nmus, c.ntypes,
                                    p(q_scaler), rmax, rmin, c.s.B, c.s.P, c.s.U, c.s.nghost, binum.data_ptr<int>(),
                                    bilist.data_ptr<int>(), bnumneigh.data_ptr<int>(), bfirstneigh.data_ptr<int>(),
                                    p(brcs), btypes.data_ptr<int>(), p(es), p(desc), st);
        } else {
            auto p = [](const at::Tensor& t) { return t.defined() ? t.data_ptr<float>() : nullptr; };
            rc = a2p_mtp_esites_f32(c.plan.handle, (int)K, scaling, p(coeffs), p(lin), p(bias), (int)nmus, c.ntypes,
                                    p(q_scaler), rmax, rmin, c.s.B, c.s.P, c.s.U, c.s.nghost, binum.data_ptr<int>(),
                                    bilist.data_ptr<int>(), bnumneigh.data_ptr<int>(), bfirstneigh.data_ptr<int>(),
                                    p(brcs), btypes.data_ptr<int>(), p(es), p(desc), st);
        }
        return rc;
    };
    run_checked(brcs, binum, bnumneigh, bfirstneigh, c.s.nghost, call);
}

// forward: [e_sites[B, P]]; backward: sum over structures and rows of grad * d e_sites / d theta
struct EsitesFunction : public torch::autograd::Function<EsitesFunction> {
    static variable_list forward(AutogradContext* ctx, int64_t K, double scaling, const at::Tensor& coeffs,
                                 const at::Tensor& lin, const at::Tensor& bias, int64_t n_moms,
                                 const at::Tensor& basic, const at::Tensor& times, const at::Tensor& mapping,
                                 int64_t nmus, const at::Tensor& binum, const at::Tensor& bilist,
                                 const at::Tensor& bnumneigh, const at::Tensor& bfirstneigh, const at::Tensor& brcs,
                                 const at::Tensor& btypes, const at::Tensor& type_map, int64_t nghost, double rmax,
                                 double rmin, const at::Tensor& q_scaler)
    {
        MtpCtx c = check_mtp(K, coeffs, lin, bias, n_moms, basic, times, mapping, nmus, binum, bilist, bnumneigh,
                             bfirstneigh, brcs, btypes, type_map, nghost, q_scaler);
        a2p_bind::DeviceGuard guard(brcs);
        at::Tensor es = at::zeros({c.s.B, c.s.P}, brcs.options());
        run_esites(c, K, scaling, coeffs, lin, bias, nmus, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, rmax,
                   rmin, q_scaler, es, at::Tensor());
        ctx->save_for_backward({coeffs, lin, bias, basic, times, mapping, binum, bilist, bnumneigh, bfirstneigh, brcs,
                                btypes, type_map, q_scaler});
        ctx->saved_data["K"] = K;
        ctx->saved_data["scaling"] = scaling;
        ctx->saved_data["n_moms"] = n_moms;
        ctx->saved_data["nmus"] = nmus;
        ctx->saved_data["nghost"] = nghost;
        ctx->saved_data["rmax"] = rmax;
        ctx->saved_data["rmin"] = rmin;
        return {es};
    }

    static variable_list backward(AutogradContext* ctx, variable_list grads)
    {
        variable_list out(21);                   // one slot per forward argument after ctx
        auto sv = ctx->get_saved_variables();
        const at::Tensor &coeffs = sv[0], &lin = sv[1], &bias = sv[2], &brcs = sv[10], &q_scaler = sv[13];
        const int64_t K = ctx->saved_data["K"].toInt(), nmus = ctx->saved_data["nmus"].toInt();
        MtpCtx c = check_mtp(K, coeffs, lin, bias, ctx->saved_data["n_moms"].toInt(), sv[3], sv[4], sv[5], nmus,
                             sv[6], sv[7], sv[8], sv[9], brcs, sv[11], sv[12], ctx->saved_data["nghost"].toInt(),
                             q_scaler);
        a2p_bind::DeviceGuard guard(brcs);
        auto opt = brcs.options();
        at::Tensor g = grads[0].contiguous();
        TORCH_CHECK(g.dim() == 2 && g.size(0) == c.s.B && g.size(1) == c.s.P, "grad of e_sites must be [B, P]");
        at::Tensor dc = at::zeros({c.s.B, coeffs.numel()}, opt), dl = at::zeros({c.s.B, lin.numel()}, opt),
                   db = at::zeros({c.s.B, bias.numel()}, opt);
        const double scaling = ctx->saved_data["scaling"].toDouble(), rmax = ctx->saved_data["rmax"].toDouble(),
                     rmin = ctx->saved_data["rmin"].toDouble();
        void* st = current_stream(brcs);
        int rc;
        if (brcs.scalar_type() == at::kDouble) {
            auto p = [](const at::Tensor& t) { return t.data_ptr<double>(); };
            rc = a2p_mtp_esites_bwd_f64(c.plan.handle, (int)K, scaling, p(coeffs), p(lin), p(bias), (int)nmus,
                                        c.ntypes, p(q_scaler), rmax, rmin, c.s.B, c.s.P, c.s.U, c.s.nghost,
                                        sv[6].data_ptr<int>(), sv[7].data_ptr<int>(), sv[8].data_ptr<int>(),
                                        sv[9].data_ptr<int>(), p(brcs), sv[11].data_ptr<int>(), p(g), p(dc), p(dl),
                                        p(db), st);
        } else {
            auto p = [](const at::Tensor& t) { return t.data_ptr<float>(); };
            rc = a2p_mtp_esites_bwd_f32(c.plan.handle, (int)K, scaling, p(coeffs), p(lin), p(bias), (int)nmus,
                                        c.ntypes, p(q_scaler), rmax, rmin, c.s.B, c.s.P, c.s.U, c.s.nghost,
                                        sv[6].data_ptr<int>(), sv[7].data_ptr<int>(), sv[8].data_ptr<int>(),
                                        sv[9].data_ptr<int>(), p(brcs), sv[11].data_ptr<int>(), p(g), p(dc), p(dl),
                                        p(db), st);
        }
        check_rc(rc);
        out[2] = dc.sum(0).reshape(coeffs.sizes());
        out[3] = dl.sum(0).reshape(lin.sizes());
        out[4] = db.sum(0).reshape(bias.sizes());
        return out;
    }
};

variable_list mtp_descriptors(int64_t K, double scaling, const at::Tensor& coeffs, int64_t n_moms,
                              const at::Tensor& basic, const at::Tensor& times, const at::Tensor& mapping,
                              int64_t nmus, const at::Tensor& binum, const at::Tensor& bilist,
                              const at::Tensor& bnumneigh, const at::Tensor& bfirstneigh, const at::Tensor& brcs,
                              const at::Tensor& btypes, const at::Tensor& type_map, int64_t nghost, double rmax,
                              double rmin)
{
    // the descriptors do not depend on the read-out: unit weights and scalers, zero bias
    at::Tensor one = at::ones({mapping.numel()}, brcs.options()), zero = at::zeros({type_map.numel()}, brcs.options());
    MtpCtx c = check_mtp(K, coeffs, one, zero, n_moms, basic, times, mapping, nmus, binum, bilist, bnumneigh,
                         bfirstneigh, brcs, btypes, type_map, nghost, one);
    a2p_bind::DeviceGuard guard(brcs);
    at::Tensor desc = at::zeros({c.s.B, c.s.P, c.plan.n_scalar}, brcs.options());
    run_esites(c, K, scaling, coeffs.detach(), one, zero, nmus, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes,
               rmax, rmin, one, at::Tensor(), desc);
    return {desc};
}

// The legacy basis operator (src/mtpBasisOp.cc:28-326): forward = the scalar moments of every row; backward =
// one adjoint sweep per row from the incoming weights (a2p_mtp_basis_bwd_*), where the reference contracts
// dense derivative arrays kept from its forward pass (mtpBasis.h:359-394).
struct BasisFunction : public torch::autograd::Function<BasisFunction> {
    static variable_list forward(AutogradContext* ctx, const at::Tensor& basic, const at::Tensor& times,
                                 const at::Tensor& mapping, int64_t n_moms, int64_t nmus, int64_t ntypes, int64_t K,
                                 double scaling, const at::Tensor& coeffs, const at::Tensor& binum,
                                 const at::Tensor& bilist, const at::Tensor& bnumneigh, const at::Tensor& bfirstneigh,
                                 const at::Tensor& brcs, const at::Tensor& btypes, double rmax, double rmin)
    {
        at::Tensor type_map = at::zeros({ntypes}, binum.options());     // only its length is used
        at::Tensor desc = mtp_descriptors(K, scaling, coeffs, n_moms, basic, times, mapping, nmus, binum, bilist,
                                          bnumneigh, bfirstneigh, brcs.detach(), btypes, type_map, 0, rmax, rmin)[0];
        ctx->save_for_backward({coeffs, basic, times, mapping, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes});
        ctx->saved_data["K"] = K;
        ctx->saved_data["scaling"] = scaling;
        ctx->saved_data["n_moms"] = n_moms;
        ctx->saved_data["nmus"] = nmus;
        ctx->saved_data["ntypes"] = ntypes;
        ctx->saved_data["rmax"] = rmax;
        ctx->saved_data["rmin"] = rmin;
        return {desc};
    }

    static variable_list backward(AutogradContext* ctx, variable_list grads)
    {
        variable_list out(17);                   // one slot per forward argument after ctx
        auto sv = ctx->get_saved_variables();
        const at::Tensor &coeffs = sv[0], &brcs = sv[8];
        // needs_input_grad counts the tensor arguments only: coeffs is the fourth, brcs the ninth
        const bool want_c = ctx->needs_input_grad(3), want_r = ctx->needs_input_grad(8);
        if (!want_c && !want_r) return out;
        const int64_t K = ctx->saved_data["K"].toInt(), nmus = ctx->saved_data["nmus"].toInt(),
                      ntypes = ctx->saved_data["ntypes"].toInt();
        Batch s = check_batch(sv[4], sv[5], sv[6], sv[7], brcs, sv[9], 0);
        a2p_bind::DeviceGuard guard(brcs);
        PlanEntry plan = get_plan(brcs.device().index(), ctx->saved_data["n_moms"].toInt(), sv[1], sv[2], sv[3]);
        auto opt = brcs.options();
        at::Tensor g = grads[0].contiguous();
        TORCH_CHECK(g.dim() == 3 && g.size(0) == s.B && g.size(1) == s.P && g.size(2) == plan.n_scalar,
                    "grad of the basis values must be [B, P, alpha_scalar_moments]");
        at::Tensor dr, dc;
        if (want_r) dr = at::zeros({s.B, s.P, s.U, 3}, opt);
        if (want_c) dc = at::zeros({s.B, coeffs.numel()}, opt);
        const double scaling = ctx->saved_data["scaling"].toDouble(), rmax = ctx->saved_data["rmax"].toDouble(),
                     rmin = ctx->saved_data["rmin"].toDouble();
        void* st = current_stream(brcs);
        int rc;
        if (brcs.scalar_type() == at::kDouble) {
            auto p = [](const at::Tensor& t) { return t.defined() ? t.data_ptr<double>() : nullptr; };
            rc = a2p_mtp_basis_bwd_f64(plan.handle, (int)K, scaling, p(coeffs), (int)nmus, (int)ntypes, rmax, rmin, s.B,
                                       s.P, s.U, 0, sv[4].data_ptr<int>(), sv[5].data_ptr<int>(), sv[6].data_ptr<int>(),
                                       sv[7].data_ptr<int>(), p(brcs), sv[9].data_ptr<int>(), p(g), p(dr), p(dc), st);
        } else {
            auto p = [](const at::Tensor& t) { return t.defined() ? t.data_ptr<float>() : nullptr; };
            rc = a2p_mtp_basis_bwd_f32(plan.handle, (int)K, scaling, p(coeffs), (int)nmus, (int)ntypes, rmax, rmin, s.B,
                                       s.P, s.U, 0, sv[4].data_ptr<int>(), sv[5].data_ptr<int>(), sv[6].data_ptr<int>(),
                                       sv[7].data_ptr<int>(), p(brcs), sv[9].data_ptr<int>(), p(g), p(dr), p(dc), st);
        }
        check_rc(rc);
        if (want_c) out[8] = dc.sum(0).reshape(coeffs.sizes());
        if (want_r) out[13] = dr;
        return out;
    }
};

// X^T X [n, n] and X^T y [n] of a tall matrix X [N, n]: the rows are cut into up to 64 blocks whose products run
// as one batched GEMM and are added afterwards (a single GEMM with n of about a hundred and N in the tens of
// thousands occupies one tile of the chip: 0.66 ms against 0.03 ms for 24576 x 95 in fp64)
std::pair<at::Tensor, at::Tensor> gram(const at::Tensor& X, const at::Tensor& y)
{
    const int64_t N = X.size(0), n = X.size(1);
    at::Tensor R = at::cat({X, y.reshape({N, 1})}, 1);
    const int64_t chunks = std::max<int64_t>(1, std::min<int64_t>(64, N / 256));
    const int64_t k = N / chunks, head = k * chunks;
    at::Tensor G = at::bmm(X.narrow(0, 0, head).reshape({chunks, k, n}).transpose(1, 2),
                           R.narrow(0, 0, head).reshape({chunks, k, n + 1})).sum(0);
    if (head < N) G = G + at::matmul(X.narrow(0, head, N - head).t(), R.narrow(0, head, N - head));
    return {G.narrow(1, 0, n), G.select(1, n)};
}

// normal equations of the linear parameters (linear_mtp_gram_and_cross.h:446-575): components by the
// library, Gram products by torch's BLAS
variable_list lin_matrix_lin_vector(double e_w, double f_w, double v_w, const at::Tensor& e_dft,
                                    const at::Tensor& f_dft, const at::Tensor& v_dft, int64_t K, double scaling,
                                    const at::Tensor& coeffs, int64_t n_moms, const at::Tensor& basic,
                                    const at::Tensor& times, const at::Tensor& mapping, int64_t nmus,
                                    const at::Tensor& binum, const at::Tensor& bilist, const at::Tensor& bnumneigh,
                                    const at::Tensor& bfirstneigh, const at::Tensor& brcs, const at::Tensor& btypes,
                                    const at::Tensor& type_map, int64_t nghost, double rmax, double rmin,
                                    const at::Tensor& q_scaler)
{
    TORCH_CHECK(nghost == 0, "LinMatrixLinVectorOp requires nghost == 0: the reference's force components have "
                             "natoms_pad rows");
    auto opt = brcs.options();
    at::Tensor lin0 = at::zeros({mapping.numel()}, opt), bias0 = at::zeros({type_map.numel()}, opt);
    MtpCtx c = check_mtp(K, coeffs, lin0, bias0, n_moms, basic, times, mapping, nmus, binum, bilist, bnumneigh,
                         bfirstneigh, brcs, btypes, type_map, nghost, q_scaler);
    check_device_float(brcs, e_dft, "betot_dft");
    check_device_float(brcs, f_dft, "bforce_dft");
    check_device_float(brcs, v_dft, "bvirial_dft");
    const int B = c.s.B, P = c.s.P;
    const int64_t n = c.plan.n_scalar + c.ntypes;
    TORCH_CHECK(e_dft.numel() == B && f_dft.numel() == (int64_t)B * P * 3 && v_dft.numel() == (int64_t)B * 9,
                "label tensors must have shapes [B], [B, P, 3], [B, 9]");
    a2p_bind::DeviceGuard guard(brcs);
    // (the library writes every element)
    at::Tensor ec = at::empty({B, n}, opt), fc = at::empty({(int64_t)B * P * 3, n}, opt), vc = at::empty({B * 9, n}, opt);
    void* st = current_stream(brcs);
    auto call = [&]() -> int {
        int rc;
        if (brcs.scalar_type() == at::kDouble) {
            auto p = [](const at::Tensor& t) { return t.data_ptr<double>(); };
            rc = a2p_mtp_lin_components_f64(c.plan.handle, (int)K, scaling, p(coeffs), (int)nmus, c.ntypes, p(q_scaler), rmax,
                                            rmin, B, P, c.s.U, binum.data_ptr<int>(), bilist.data_ptr<int>(),
                                            bnumneigh.data_ptr<int>(), bfirstneigh.data_ptr<int>(), p(brcs),
                                            btypes.data_ptr<int>(), p(ec), p(fc), p(vc), st);
        } else {
            auto p = [](const at::Tensor& t) { return t.data_ptr<float>(); };
            rc = a2p_mtp_lin_components_f32(c.plan.handle, (int)K, scaling, p(coeffs), (int)nmus, c.ntypes, p(q_scaler), rmax,
                                            rmin, B, P, c.s.U, binum.data_ptr<int>(), bilist.data_ptr<int>(),
                                            bnumneigh.data_ptr<int>(), bfirstneigh.data_ptr<int>(), p(brcs),
                                            btypes.data_ptr<int>(), p(ec), p(fc), p(vc), st);
        }
        return rc;
    };
    run_checked(brcs, binum, bnumneigh, bfirstneigh, 0, call);
    auto ge = gram(ec, e_dft.reshape({B})), gf = gram(fc, f_dft.reshape({-1})), gv = gram(vc, v_dft.reshape({-1}));
    at::Tensor A = e_w * ge.first + f_w * gf.first + v_w * gv.first;
    at::Tensor b = e_w * ge.second + f_w * gf.second + v_w * gv.second;
    return {A.contiguous(), b.contiguous()};
}

variable_list schmidt_orth(int64_t ntypes, int64_t nmus, int64_t K, const at::Tensor& coeffs)
{
    TORCH_CHECK(coeffs.is_cuda(), "coeffs must be on a HIP device: this build has no CPU path");
    TORCH_CHECK((coeffs.scalar_type() == at::kFloat || coeffs.scalar_type() == at::kDouble) && coeffs.is_contiguous(),
                "coeffs must be a contiguous float32 or float64 tensor");
    TORCH_CHECK(coeffs.numel() == ntypes * ntypes * nmus * K, "coeffs size mismatch");
    a2p_bind::DeviceGuard guard(coeffs);
    at::Tensor src = coeffs.detach(), out = at::empty_like(src);
    void* st = current_stream(coeffs);
    const int rc = coeffs.scalar_type() == at::kDouble
                       ? a2p_mtp_schmidt_orth_f64((int)ntypes, (int)nmus, (int)K, src.data_ptr<double>(),
                                                  out.data_ptr<double>(), st)
                       : a2p_mtp_schmidt_orth_f32((int)ntypes, (int)nmus, (int)K, src.data_ptr<float>(),
                                                  out.data_ptr<float>(), st);
    check_rc(rc);
    return {out};
}

}  // namespace

#define MTP_EFV_ARGS int64_t K, double scaling, const at::Tensor& coeffs, const at::Tensor& lin, \
    const at::Tensor& bias, int64_t n_moms, const at::Tensor& basic, const at::Tensor& times, \
    const at::Tensor& mapping, int64_t nmus, const at::Tensor& binum, const at::Tensor& bilist, \
    const at::Tensor& bnumneigh, const at::Tensor& bfirstneigh, const at::Tensor& brcs, \
    const at::Tensor& btypes, const at::Tensor& type_map, int64_t nghost, double rmax, double rmin, \
    const at::Tensor& q_scaler, double zbl_rmax, double zbl_rmin, const at::Tensor& zbl_cks, \
    const at::Tensor& zbl_dks
#define MTP_EFV_PASS K, scaling, coeffs, lin, bias, n_moms, basic, times, mapping, nmus, binum, bilist, \
    bnumneigh, bfirstneigh, brcs, btypes, type_map, nghost, rmax, rmin, q_scaler

TORCH_LIBRARY(mtpr, m)
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
    m.def("linearMtpToEFVOp", [](MTP_EFV_ARGS) -> variable_list { return mtp_efv(true, MTP_EFV_PASS, zbl_rmax, zbl_rmin, zbl_cks, zbl_dks); });
    m.def("linearMtpToEFOp", [](MTP_EFV_ARGS) -> variable_list { return mtp_efv(false, MTP_EFV_PASS, zbl_rmax, zbl_rmin, zbl_cks, zbl_dks); });
    m.def("linearMtpToLossOp",
          [](double e_w, double f_w, double v_w, const at::Tensor& e_dft, const at::Tensor& f_dft,
             const at::Tensor& v_dft, MTP_EFV_ARGS) -> variable_list {
              // the reference's forward passes the model's cutoffs to the ZBL launcher
              // (linearMtpOp.cc:819-820) where its backward passes the ZBL ones (:1400-1401); here both
              // use the ZBL cutoffs
              auto lab = zbl_shift_labels(zbl_rmax, zbl_rmin, zbl_cks, zbl_dks, type_map, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, nghost, e_dft, f_dft, v_dft);
              return LossFunction::apply(true, e_w, f_w, v_w, lab.e, lab.f, lab.v, MTP_EFV_PASS);
          });
    m.def("linearMtpToEFLossOp",
          [](double e_w, double f_w, const at::Tensor& e_dft, const at::Tensor& f_dft,
             MTP_EFV_ARGS) -> variable_list {
              auto lab = zbl_shift_labels(zbl_rmax, zbl_rmin, zbl_cks, zbl_dks, type_map, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, nghost, e_dft, f_dft, at::Tensor());
              // no virial labels in this variant: zero weight, zero labels
              return LossFunction::apply(false, e_w, f_w, 0.0, lab.e, lab.f,
                                         at::zeros({e_dft.numel(), 9}, e_dft.options()), MTP_EFV_PASS);
          });
    m.def("LinMatrixLinVectorOp",
          [](double e_w, double f_w, double v_w, const at::Tensor& e_dft, const at::Tensor& f_dft,
             const at::Tensor& v_dft, MTP_EFV_ARGS) -> variable_list {
              // labels minus the ZBL energy, forces and virial (src/linear_mtp_gram_and_cross_op.cc:309-338)
              auto lab = zbl_shift_labels(zbl_rmax, zbl_rmin, zbl_cks, zbl_dks, type_map, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, nghost, e_dft, f_dft, v_dft);
              return lin_matrix_lin_vector(e_w, f_w, v_w, lab.e, lab.f, lab.v, K, scaling, coeffs, n_moms, basic, times,
                                           mapping, nmus, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, type_map,
                                           nghost, rmax, rmin, q_scaler);
          });
    m.def("CoeffsSchmidtOrthOp", [](int64_t ntypes, int64_t nmus, int64_t K, const at::Tensor& coeffs) -> variable_list {
        return schmidt_orth(ntypes, nmus, K, coeffs);
    });
    m.def("linearMtpToEsitesOp", [](MTP_EFV_ARGS) -> variable_list {
        variable_list out = EsitesFunction::apply(MTP_EFV_PASS);
        at::Tensor zb = zbl_esites(zbl_rmax, zbl_rmin, zbl_cks, zbl_dks, type_map, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, nghost);
        if (zb.defined()) out[0] = out[0] + zb;
        return out;
    });
    // mtpr_bind.cc:140-187: num_mus4moms / mus4moms (the radial functions behind each moment, which the reference's
    // coefficient derivative walks) are not needed here; the first dimension of mus4moms is the number of moments
    m.def("mtpBasisOp",
          [](const at::Tensor& basic, const at::Tensor& times, const at::Tensor& mapping, const at::Tensor& num_mus4moms,
             const at::Tensor& mus4moms, const at::Tensor& nmus, int64_t ntypes, int64_t K, double scaling,
             const at::Tensor& coeffs, const at::Tensor& binum, const at::Tensor& bilist, const at::Tensor& bnumneigh,
             const at::Tensor& bfirstneigh, const at::Tensor& brcs, const at::Tensor& btypes, int64_t umax,
             double rmax, double rmin) -> variable_list {
              TORCH_CHECK(brcs.dim() == 4 && umax == brcs.size(2), "umax_num_neighs does not match brcs");
              return BasisFunction::apply(basic, times, mapping, mus4moms.size(0), (int64_t)nmus.item<int>(), ntypes, K,
                                          scaling, coeffs, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, rmax,
                                          rmin);
          });
    m.def("linearMtpToDescriptorsOp",
          [](int64_t K, double scaling, const at::Tensor& coeffs, int64_t n_moms, const at::Tensor& basic,
             const at::Tensor& times, const at::Tensor& mapping, int64_t nmus, const at::Tensor& binum,
             const at::Tensor& bilist, const at::Tensor& bnumneigh, const at::Tensor& bfirstneigh,
             const at::Tensor& brcs, const at::Tensor& btypes, const at::Tensor& type_map, int64_t nghost,
             double rmax, double rmin) -> variable_list {
              return mtp_descriptors(K, scaling, coeffs, n_moms, basic, times, mapping, nmus, binum, bilist,
                                     bnumneigh, bfirstneigh, brcs, btypes, type_map, nghost, rmax, rmin);
          });
}
