// TEST INFRASTRUCTURE ONLY. extern "C" driver around the reference's neural-network MTP
// (REF_ROOT/source/descriptor/nnmtp/include/nnMtp.h:378-567 find_efv, :648-753 find_e_sites,
// :570-645 find_descriptors), called per structure as the operator's CPU branch does
// (src/nnMtpOp.cc:2857-2927), built into oracle/_ref/libref_nnmtp.so.  The loss step follows
// NNMtpToLossFunction::{forward,backward} on the CPU branch (src/nnMtpOp.cc:1641-2780): E/F/V,
// NNMtpLoss::find_loss (include/nnMtpLoss.h:141-181), then find_loss_backward (:216-610) per
// structure, i.e. the per-structure gradients before the grad_output matmul.
#include <cstring>
#include <vector>
#include "descriptor/nnmtp/include/nnMtp.h"

using namespace ai2pot::nnmtp;

extern "C" {

void ref_nnmtp_efv_f64(double* betot, double* bforce, double* bvirial, double* e_sites, int K, int H,
                       const double* coeffs, const double* w0, const double* w1, const double* bias, int n_moms,
                       int n_basic, const int* basic, int n_times, const int* times, int n_scalar,
                       const int* mapping, int nmus, int B, int P, const int* binum, const int* bilist,
                       const int* bnumneigh, const int* bfirstneigh, const double* brcs, const int* btypes,
                       int ntypes, const int* type_map, int U, int nghost, double rmax, double rmin,
                       const double* q_shifter, const double* q_scaler)
{
    // the operator allocates its outputs with at::zeros (nnMtpOp.cc:2845-2847); find_efv only
    // accumulates into the virial
    std::memset(betot, 0, sizeof(double) * B);
    std::memset(bforce, 0, sizeof(double) * B * (P + nghost) * 3);
    std::memset(bvirial, 0, sizeof(double) * B * 9);
    for (int b = 0; b < B; b++) {
        int* il = const_cast<int*>(&bilist[(size_t)b * P]);
        int* nn = const_cast<int*>(&bnumneigh[(size_t)b * P]);
        int* fn = const_cast<int*>(&bfirstneigh[(size_t)b * P * U]);
        double(*rc)[3] = (double(*)[3])const_cast<double*>(&brcs[(size_t)b * P * U * 3]);
        int* ty = const_cast<int*>(&btypes[(size_t)b * (P + nghost)]);
        NNMtp<double>::find_efv(betot[b], (double(*)[3])&bforce[(size_t)b * (P + nghost) * 3], &bvirial[b * 9], K, H,
                                const_cast<double*>(coeffs), const_cast<double*>(w0), const_cast<double*>(w1),
                                const_cast<double*>(bias), n_moms, n_basic, (const int(*)[4])basic, n_times,
                                (const int(*)[4])times, n_scalar, mapping, nmus, binum[b], il, nn, fn, rc, ty, ntypes,
                                const_cast<int*>(type_map), U, nghost, rmax, rmin, const_cast<double*>(q_shifter),
                                const_cast<double*>(q_scaler));
        if (e_sites)
            NNMtp<double>::find_e_sites(&e_sites[(size_t)b * P], K, H, const_cast<double*>(coeffs),
                                        const_cast<double*>(w0), const_cast<double*>(w1), const_cast<double*>(bias),
                                        n_moms, n_basic, (const int(*)[4])basic, n_times, (const int(*)[4])times,
                                        n_scalar, mapping, nmus, binum[b], il, nn, fn, rc, ty, ntypes,
                                        const_cast<int*>(type_map), U, nghost, rmax, rmin,
                                        const_cast<double*>(q_shifter), const_cast<double*>(q_scaler));
    }
}

void ref_nnmtp_loss_step_f64(double* bloss, double* betot, double* bforce, double* bvirial, double* dcoeffs,
                             double* dw0, double* dw1, double* dbias, double e_w, double f_w, double v_w,
                             const double* e_dft, const double* f_dft, const double* v_dft, int K, int H,
                             const double* coeffs, const double* w0, const double* w1, const double* bias,
                             int n_moms, int n_basic, const int* basic, int n_times, const int* times,
                             int n_scalar, const int* mapping, int nmus, int B, int P, const int* binum,
                             const int* bilist, const int* bnumneigh, const int* bfirstneigh, const double* brcs,
                             const int* btypes, int ntypes, const int* type_map, int U, int nghost, double rmax,
                             double rmin, const double* q_shifter, const double* q_scaler)
{
    ref_nnmtp_efv_f64(betot, bforce, bvirial, nullptr, K, H, coeffs, w0, w1, bias, n_moms, n_basic, basic, n_times,
                      times, n_scalar, mapping, nmus, B, P, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, ntypes,
                      type_map, U, nghost, rmax, rmin, q_shifter, q_scaler);
    const int ncoef = ntypes * ntypes * nmus * K, nw0 = ntypes * H * n_scalar, nw1 = ntypes * H;
    std::memset(dcoeffs, 0, sizeof(double) * B * ncoef);
    std::memset(dw0, 0, sizeof(double) * B * nw0);
    std::memset(dw1, 0, sizeof(double) * B * nw1);
    std::memset(dbias, 0, sizeof(double) * B * ntypes);
    for (int b = 0; b < B; b++) {
        int* il = const_cast<int*>(&bilist[(size_t)b * P]);
        double(*fm)[3] = (double(*)[3])&bforce[(size_t)b * (P + nghost) * 3];
        double(*fd)[3] = (double(*)[3])const_cast<double*>(&f_dft[(size_t)b * P * 3]);
        NNMtpLoss<double>::find_loss(bloss[b], binum[b], il, e_w, f_w, v_w, betot[b], e_dft[b], fm, fd,
                                     &bvirial[b * 9], const_cast<double*>(&v_dft[b * 9]));
        NNMtpLoss<double>::find_loss_backward(
            &dcoeffs[(size_t)b * ncoef], &dw0[(size_t)b * nw0], &dw1[(size_t)b * nw1], &dbias[(size_t)b * ntypes], e_w,
            f_w, v_w, betot[b], e_dft[b], fm, fd, &bvirial[b * 9], const_cast<double*>(&v_dft[b * 9]), K, H,
            const_cast<double*>(coeffs), const_cast<double*>(w0), const_cast<double*>(w1), const_cast<double*>(bias),
            n_moms, n_basic, (const int(*)[4])basic, n_times, (const int(*)[4])times, n_scalar, mapping, nmus, binum[b],
            il, const_cast<int*>(&bnumneigh[(size_t)b * P]), const_cast<int*>(&bfirstneigh[(size_t)b * P * U]),
            (double(*)[3])const_cast<double*>(&brcs[(size_t)b * P * U * 3]),
            const_cast<int*>(&btypes[(size_t)b * (P + nghost)]), ntypes, const_cast<int*>(type_map), U, nghost, rmax,
            rmin, const_cast<double*>(q_shifter), const_cast<double*>(q_scaler));
    }
}

// per-row derivatives of the site energies (nnMtp.h:756-990), contracted with gout[B, P] per structure
// as the operator's backward does before its sum over the batch
void ref_nnmtp_esites_bwd_f64(double* dcoeffs, double* dw0, double* dw1, double* dbias, const double* gout, int K,
                              int H, const double* coeffs, const double* w0, const double* w1, const double* bias,
                              int n_moms, int n_basic, const int* basic, int n_times, const int* times,
                              int n_scalar, const int* mapping, int nmus, int B, int P, const int* binum,
                              const int* bilist, const int* bnumneigh, const int* bfirstneigh, const double* brcs,
                              const int* btypes, int ntypes, const int* type_map, int U, int nghost, double rmax,
                              double rmin, const double* q_shifter, const double* q_scaler)
{
    const int ncoef = ntypes * ntypes * nmus * K, nw0 = ntypes * H * n_scalar, nw1 = ntypes * H;
    std::vector<double> pc((size_t)P * ncoef), p0((size_t)P * nw0), p1((size_t)P * nw1), pb((size_t)P * ntypes);
    for (int b = 0; b < B; b++) {
        std::fill(pc.begin(), pc.end(), 0.0);
        std::fill(p0.begin(), p0.end(), 0.0);
        std::fill(p1.begin(), p1.end(), 0.0);
        std::fill(pb.begin(), pb.end(), 0.0);
        NNMtp<double>::find_e_sites_backward(
            pc.data(), p0.data(), p1.data(), pb.data(), K, H, const_cast<double*>(coeffs), const_cast<double*>(w0),
            const_cast<double*>(w1), const_cast<double*>(bias), n_moms, n_basic, (const int(*)[4])basic, n_times,
            (const int(*)[4])times, n_scalar, mapping, nmus, binum[b], const_cast<int*>(&bilist[(size_t)b * P]),
            const_cast<int*>(&bnumneigh[(size_t)b * P]), const_cast<int*>(&bfirstneigh[(size_t)b * P * U]),
            (double(*)[3])const_cast<double*>(&brcs[(size_t)b * P * U * 3]),
            const_cast<int*>(&btypes[(size_t)b * (P + nghost)]), ntypes, const_cast<int*>(type_map), U, nghost, rmax,
            rmin, const_cast<double*>(q_shifter), const_cast<double*>(q_scaler));
        auto contract = [&](const std::vector<double>& per, int n, double* out) {
            for (int q = 0; q < n; q++) {
                double a = 0;
                for (int ii = 0; ii < binum[b]; ii++) a += gout[(size_t)b * P + ii] * per[(size_t)ii * n + q];
                out[(size_t)b * n + q] = a;
            }
        };
        contract(pc, ncoef, dcoeffs);
        contract(p0, nw0, dw0);
        contract(p1, nw1, dw1);
        contract(pb, ntypes, dbias);
    }
}
}
