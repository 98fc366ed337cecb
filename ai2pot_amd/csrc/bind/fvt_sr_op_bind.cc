// libfvt_sr_op_bind.so -- registers torch.ops.fvt.ForceSrOp / VirialSrOp with the reference's
// schemas (source/fvt/bind/fvt_sr_op_bind.cc:9-46) on top of libai2pot_hip.so.  Both maps are
// (bi)linear, so each backward is itself an autograd Function built from the same kernels and
// callers that differentiate twice (ai2pot/models/deepmd/se_r.py:316-330) stay on the GPU.
// The reference's operators are host-only and build dense Jacobians (src/force_sr_op.cc:44).
#include "bind_common.h"

using namespace a2p_bind;
using torch::autograd::AutogradContext;
using torch::autograd::variable_list;

namespace {

struct Lists {
    at::Tensor binum, bilist, bnumneigh, bfirstneigh;
    int nghost;
};

at::Tensor force_raw(const Lists& l, const at::Tensor& dei_in)
{
    at::Tensor dei = dei_in.contiguous();
    a2p_bind::DeviceGuard guard(dei);
    const int B = (int)dei.size(0), P = (int)dei.size(1), U = (int)dei.size(2);
    at::Tensor f = at::empty({B, P + l.nghost, 3}, dei.options());
    void* st = current_stream(dei);
    int rc = dei.scalar_type() == at::kFloat
        ? a2p_fvt_force_fwd_f32(B, P, U, l.nghost, l.binum.data_ptr<int>(), l.bilist.data_ptr<int>(),
                                l.bnumneigh.data_ptr<int>(), l.bfirstneigh.data_ptr<int>(), dei.data_ptr<float>(),
                                f.data_ptr<float>(), st)
        : a2p_fvt_force_fwd_f64(B, P, U, l.nghost, l.binum.data_ptr<int>(), l.bilist.data_ptr<int>(),
                                l.bnumneigh.data_ptr<int>(), l.bfirstneigh.data_ptr<int>(), dei.data_ptr<double>(),
                                f.data_ptr<double>(), st);
    check_rc(rc);
    return f;
}

at::Tensor force_adjoint_raw(const Lists& l, const at::Tensor& gF_in)
{
    at::Tensor gF = gF_in.contiguous();
    a2p_bind::DeviceGuard guard(gF);
    const int B = (int)l.bfirstneigh.size(0), P = (int)l.bfirstneigh.size(1), U = (int)l.bfirstneigh.size(2);
    at::Tensor out = at::empty({B, P, U, 3}, gF.options());
    void* st = current_stream(gF);
    int rc = gF.scalar_type() == at::kFloat
        ? a2p_fvt_force_bwd_f32(B, P, U, l.nghost, l.binum.data_ptr<int>(), l.bilist.data_ptr<int>(),
                                l.bnumneigh.data_ptr<int>(), l.bfirstneigh.data_ptr<int>(), gF.data_ptr<float>(),
                                out.data_ptr<float>(), st)
        : a2p_fvt_force_bwd_f64(B, P, U, l.nghost, l.binum.data_ptr<int>(), l.bilist.data_ptr<int>(),
                                l.bnumneigh.data_ptr<int>(), l.bfirstneigh.data_ptr<int>(), gF.data_ptr<double>(),
                                out.data_ptr<double>(), st);
    check_rc(rc);
    return out;
}

struct ForceAdjoint;

struct ForceSr : public torch::autograd::Function<ForceSr> {
    static at::Tensor forward(AutogradContext* ctx, const at::Tensor& dei, const at::Tensor& binum,
                              const at::Tensor& bilist, const at::Tensor& bnumneigh, const at::Tensor& bfirstneigh,
                              int64_t nghost)
    {
        ctx->save_for_backward({binum, bilist, bnumneigh, bfirstneigh});
        ctx->saved_data["nghost"] = nghost;
        return force_raw(Lists{binum, bilist, bnumneigh, bfirstneigh, (int)nghost}, dei);
    }
    static variable_list backward(AutogradContext* ctx, variable_list g);
};

struct ForceAdjoint : public torch::autograd::Function<ForceAdjoint> {
    static at::Tensor forward(AutogradContext* ctx, const at::Tensor& gF, const at::Tensor& binum,
                              const at::Tensor& bilist, const at::Tensor& bnumneigh, const at::Tensor& bfirstneigh,
                              int64_t nghost)
    {
        ctx->save_for_backward({binum, bilist, bnumneigh, bfirstneigh});
        ctx->saved_data["nghost"] = nghost;
        return force_adjoint_raw(Lists{binum, bilist, bnumneigh, bfirstneigh, (int)nghost}, gF);
    }
    static variable_list backward(AutogradContext* ctx, variable_list g)
    {
        auto s = ctx->get_saved_variables();
        return {ForceSr::apply(g[0], s[0], s[1], s[2], s[3], ctx->saved_data["nghost"].toInt()), at::Tensor(),
                at::Tensor(), at::Tensor(), at::Tensor(), at::Tensor()};
    }
};

variable_list ForceSr::backward(AutogradContext* ctx, variable_list g)
{
    auto s = ctx->get_saved_variables();
    return {ForceAdjoint::apply(g[0], s[0], s[1], s[2], s[3], ctx->saved_data["nghost"].toInt()), at::Tensor(),
            at::Tensor(), at::Tensor(), at::Tensor(), at::Tensor()};
}

at::Tensor virial_raw(const at::Tensor& nn, const at::Tensor& rcs_in, const at::Tensor& dei_in)
{
    at::Tensor rcs = rcs_in.contiguous(), dei = dei_in.contiguous();
    a2p_bind::DeviceGuard guard(dei);
    const int B = (int)dei.size(0), P = (int)dei.size(1), U = (int)dei.size(2);
    at::Tensor v = at::empty({B, 9}, dei.options());
    void* st = current_stream(dei);
    int rc = dei.scalar_type() == at::kFloat
        ? a2p_fvt_virial_fwd_f32(B, P, U, nn.data_ptr<int>(), rcs.data_ptr<float>(), dei.data_ptr<float>(),
                                 v.data_ptr<float>(), st)
        : a2p_fvt_virial_fwd_f64(B, P, U, nn.data_ptr<int>(), rcs.data_ptr<double>(), dei.data_ptr<double>(),
                                 v.data_ptr<double>(), st);
    check_rc(rc);
    return v.view({B, 3, 3});
}

// returns {grad_rcs, grad_dei}
variable_list virial_bwd_raw(const at::Tensor& nn, const at::Tensor& gV_in, const at::Tensor& rcs_in,
                             const at::Tensor& dei_in)
{
    at::Tensor rcs = rcs_in.contiguous(), dei = dei_in.contiguous(), gV = gV_in.contiguous();
    a2p_bind::DeviceGuard guard(dei);
    const int B = (int)dei.size(0), P = (int)dei.size(1), U = (int)dei.size(2);
    at::Tensor gd = at::empty_like(dei), gr = at::empty_like(rcs);
    void* st = current_stream(dei);
    int rc = dei.scalar_type() == at::kFloat
        ? a2p_fvt_virial_bwd_f32(B, P, U, nn.data_ptr<int>(), rcs.data_ptr<float>(), dei.data_ptr<float>(),
                                 gV.data_ptr<float>(), gd.data_ptr<float>(), gr.data_ptr<float>(), st)
        : a2p_fvt_virial_bwd_f64(B, P, U, nn.data_ptr<int>(), rcs.data_ptr<double>(), dei.data_ptr<double>(),
                                 gV.data_ptr<double>(), gd.data_ptr<double>(), gr.data_ptr<double>(), st);
    check_rc(rc);
    return {gr, gd};
}

struct VirialBackward;

struct VirialSr : public torch::autograd::Function<VirialSr> {
    static at::Tensor forward(AutogradContext* ctx, const at::Tensor& rcs, const at::Tensor& dei,
                              const at::Tensor& nn)
    {
        ctx->save_for_backward({rcs, dei, nn});
        return virial_raw(nn, rcs, dei);
    }
    static variable_list backward(AutogradContext* ctx, variable_list g);
};

struct VirialBackward : public torch::autograd::Function<VirialBackward> {
    static variable_list forward(AutogradContext* ctx, const at::Tensor& gV, const at::Tensor& rcs,
                                 const at::Tensor& dei, const at::Tensor& nn)
    {
        ctx->save_for_backward({gV, rcs, dei, nn});
        return virial_bwd_raw(nn, gV, rcs, dei);
    }
    static variable_list backward(AutogradContext* ctx, variable_list gg)
    {
        auto s = ctx->get_saved_variables();
        const at::Tensor &gV = s[0], &rcs = s[1], &dei = s[2], &nn = s[3];
        at::Tensor ggr = gg[0].defined() ? gg[0] : at::zeros_like(rcs);
        at::Tensor ggd = gg[1].defined() ? gg[1] : at::zeros_like(dei);
        at::Tensor d_gV = VirialSr::apply(rcs, ggd, nn) + VirialSr::apply(ggr, dei, nn);
        at::Tensor d_rcs = VirialBackward::apply(gV, rcs, ggd, nn)[0];
        at::Tensor d_dei = VirialBackward::apply(gV, ggr, dei, nn)[1];
        return {d_gV, d_rcs, d_dei, at::Tensor()};
    }
};

variable_list VirialSr::backward(AutogradContext* ctx, variable_list g)
{
    auto s = ctx->get_saved_variables();
    auto r = VirialBackward::apply(g[0], s[0], s[1], s[2]);
    return {r[0], r[1], at::Tensor()};
}

}  // namespace

TORCH_LIBRARY(fvt, m)
{
    // no counterpart in the reference: the per-call device status check (one stream synchronisation per
    // call) can be switched off for loops that should run ahead of the device, and asked for explicitly
    m.def("set_validate", [](bool on) { validate_flag() = on; });
    m.def("check_status", [](const at::Tensor& any_device_tensor) {
        DeviceGuard guard(any_device_tensor);
        check_rc(a2p_check_status(current_stream(any_device_tensor)));
    });
    m.def("ForceSrOp",
          [](const at::Tensor& binum, const at::Tensor& bilist, const at::Tensor& bnumneigh,
             const at::Tensor& bfirstneigh, int64_t nghost, int64_t umax, const at::Tensor& dei) -> variable_list {
              TORCH_CHECK(dei.is_cuda(), "bdei_drij must be on a HIP device: this build has no CPU path");
              TORCH_CHECK(dei.scalar_type() == at::kFloat || dei.scalar_type() == at::kDouble,
                          "bdei_drij must be float32 or float64");
              TORCH_CHECK(dei.dim() == 4 && dei.size(3) == 3 && dei.size(2) == umax,
                          "bdei_drij must have shape [B, nlocal, umax, 3]");
              check_device_int(dei, binum, "binum");
              check_device_int(dei, bilist, "bilist");
              check_device_int(dei, bnumneigh, "bnumneigh");
              check_device_int(dei, bfirstneigh, "bfirstneigh");
              TORCH_CHECK(bfirstneigh.dim() == 3 && bfirstneigh.size(0) == dei.size(0) &&
                              bfirstneigh.size(1) == dei.size(1) && bfirstneigh.size(2) == umax &&
                              bilist.numel() == dei.size(0) * dei.size(1) &&
                              bnumneigh.numel() == dei.size(0) * dei.size(1) && binum.numel() == dei.size(0),
                          "neighbour tensors do not match bdei_drij");
              at::Tensor f = ForceSr::apply(dei, binum, bilist, bnumneigh, bfirstneigh, nghost);
              check_device_status(dei);
              return {f};
          });
    m.def("VirialSrOp",
          [](const at::Tensor& bnumneigh, const at::Tensor& brcs, int64_t umax,
             const at::Tensor& dei) -> variable_list {
              TORCH_CHECK(dei.is_cuda(), "bdei_drij must be on a HIP device: this build has no CPU path");
              TORCH_CHECK(dei.scalar_type() == at::kFloat || dei.scalar_type() == at::kDouble,
                          "bdei_drij must be float32 or float64");
              TORCH_CHECK(dei.dim() == 4 && dei.size(3) == 3 && dei.size(2) == umax && brcs.sizes() == dei.sizes(),
                          "brcs and bdei_drij must have shape [B, nlocal, umax, 3]");
              TORCH_CHECK(brcs.scalar_type() == dei.scalar_type() && brcs.device() == dei.device(),
                          "brcs must match bdei_drij in dtype and device");
              check_device_int(dei, bnumneigh, "bnumneigh");
              TORCH_CHECK(bnumneigh.numel() == dei.size(0) * dei.size(1), "bnumneigh must have shape [B, nlocal]");
              if (bnumneigh.numel())
                  TORCH_CHECK(bnumneigh.max().item<int>() <= umax, "a neighbour count exceeds umax_num_neighs");
              return {VirialSr::apply(brcs, dei, bnumneigh)};
          });
}
