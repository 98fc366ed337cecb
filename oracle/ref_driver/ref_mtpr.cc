// TEST INFRASTRUCTURE ONLY. extern "C" driver around the reference's linear-MTP CPU
// launchers (REF_ROOT/source/descriptor/mtpr/include/linearMtp_cpu_launcher.h:128-203,
// linearMtpLoss_cpu_launcher.h:151-194, 233-337, 477-527) and its template parser
// (src/mtpParam.cc, compiled alongside), built into oracle/_ref/libref_mtpr.so.
// The loss-step entry follows LinearMtpToLossFunction::{forward,backward}
// (src/linearMtpOp.cc:621-1181, 1184-1765): E/F/V, per-structure loss, RMSEs, then the
// per-structure parameter gradients [B, n] before the grad_output matmul.
#include <cstring>
#include <vector>
#include <algorithm>
#include <string>
#include "descriptor/mtpr/include/mtpParam.h"
#include "descriptor/mtpr/include/mtpBasis.h"
#include "descriptor/mtpr/include/linearMtp_cpu_launcher.h"
#include "descriptor/mtpr/include/linearMtpLoss_cpu_launcher.h"
#include "descriptor/mtpr/include/linear_mtp_gram_and_cross.h"
#include "descriptor/mtpr/include/schmidt_orth.h"

using namespace ai2pot::mtpr;

extern "C" {

// Two-call protocol: with out pointers null only the counts are returned.
// counts = {alpha_moments_count, basic_count, times_count, scalar_moments, nmus}
int ref_mtp_param(int level, int* counts, int* basic, int* times, int* mapping)
{
    try {
        MtpParam p(level);
        counts[0] = p.alpha_moments_count();
        counts[1] = p.alpha_index_basic_count();
        counts[2] = p.alpha_index_times_count();
        counts[3] = p.alpha_scalar_moments();
        counts[4] = p.nmus();
        if (basic) std::memcpy(basic, p.alpha_index_basic(), sizeof(int) * 4 * counts[1]);
        if (times) std::memcpy(times, p.alpha_index_times(), sizeof(int) * 4 * counts[2]);
        if (mapping) std::memcpy(mapping, p.alpha_moment_mapping(), sizeof(int) * counts[3]);
        return 0;
    } catch (MtpException& e) {
        return 1;
    }
}

#define MTP_MODEL_ARGS int K, double scaling, const double* coeffs, const double* lin, \
    const double* bias, int n_moms, int n_basic, const int* basic, int n_times, const int* times, \
    int n_scalar, const int* mapping, int nmus
#define MTP_LIST_ARGS int B, int P, const int* binum, const int* bilist, const int* bnumneigh, \
    const int* bfirstneigh, const double* brcs, const int* btypes, int ntypes, \
    const int* type_map, int U, int nghost, double rmax, double rmin, const double* q_scaler

#define MTP_MODEL_PASS K, scaling, const_cast<double*>(coeffs), const_cast<double*>(lin), \
    const_cast<double*>(bias), n_moms, n_basic, (const int(*)[4])basic, n_times, \
    (const int(*)[4])times, n_scalar, mapping, nmus
#define MTP_LIST_PASS B, P, const_cast<int*>(binum), const_cast<int*>(bilist), \
    const_cast<int*>(bnumneigh), const_cast<int*>(bfirstneigh), \
    (double(*)[3])const_cast<double*>(brcs), const_cast<int*>(btypes), ntypes, \
    const_cast<int*>(type_map), U, nghost, rmax, rmin, const_cast<double*>(q_scaler)

void ref_mtp_efv_f64(double* betot, double* bforce, double* bvirial, MTP_MODEL_ARGS, MTP_LIST_ARGS)
{
    find_efv_cpu_launcher<double>(betot, (double(*)[3])bforce, bvirial, MTP_MODEL_PASS, MTP_LIST_PASS);
}

// forward + backward of the training-loss op. Outputs: bloss[B], rmse[3] (e,f,v),
// E/F/V of the model, and per-structure gradients dcoeffs[B,ncoef], dlin[B,S], dbias[B,ntypes].
void ref_mtp_loss_step_f64(double* bloss, double* rmse, double* betot, double* bforce, double* bvirial,
                           double* dcoeffs, double* dlin, double* dbias, double e_w, double f_w,
                           double v_w, const double* e_dft, const double* f_dft, const double* v_dft,
                           MTP_MODEL_ARGS, MTP_LIST_ARGS)
{
    find_efv_cpu_launcher<double>(betot, (double(*)[3])bforce, bvirial, MTP_MODEL_PASS, MTP_LIST_PASS);
    find_loss_cpu_launcher<double>(bloss, B, P, const_cast<int*>(binum), const_cast<int*>(bilist),
                                   e_w, f_w, v_w, betot, const_cast<double*>(e_dft),
                                   (double(*)[3])bforce, (double(*)[3])const_cast<double*>(f_dft),
                                   bvirial, const_cast<double*>(v_dft));
    find_efv_rmse_cpu_launcher<double>(rmse[0], rmse[1], rmse[2], B, P, const_cast<int*>(binum),
                                       const_cast<int*>(bilist), betot, const_cast<double*>(e_dft),
                                       (double(*)[3])bforce, (double(*)[3])const_cast<double*>(f_dft),
                                       bvirial, const_cast<double*>(v_dft));
    int ncoef = ntypes * ntypes * nmus * K;
    std::memset(dcoeffs, 0, sizeof(double) * B * ncoef);
    std::memset(dlin, 0, sizeof(double) * B * n_scalar);
    std::memset(dbias, 0, sizeof(double) * B * ntypes);
    find_loss_backward_cpu_launcher<double>(dcoeffs, dlin, dbias, e_w, f_w, v_w, betot,
                                            const_cast<double*>(e_dft), (double(*)[3])bforce,
                                            (double(*)[3])const_cast<double*>(f_dft), bvirial,
                                            const_cast<double*>(v_dft), MTP_MODEL_PASS, MTP_LIST_PASS);
}


// site energies and scalar moments by the reference (linearMtp.h:514-611, 821-890), per structure as
// the operator's CPU branch calls them (linearMtpOp.cc:3680-3760, 4110-4190)
void ref_mtp_esites_f64(double* e_sites, double* desc, MTP_MODEL_ARGS, MTP_LIST_ARGS)
{
    for (int b = 0; b < B; b++) {
        int* il = const_cast<int*>(&bilist[(size_t)b * P]);
        int* nn = const_cast<int*>(&bnumneigh[(size_t)b * P]);
        int* fn = const_cast<int*>(&bfirstneigh[(size_t)b * P * U]);
        double(*rc)[3] = (double(*)[3])const_cast<double*>(&brcs[(size_t)b * P * U * 3]);
        int* ty = const_cast<int*>(&btypes[(size_t)b * (P + nghost)]);
        if (e_sites)
            LinearMtp<double>::find_e_sites(&e_sites[(size_t)b * P], K, scaling, const_cast<double*>(coeffs),
                                            const_cast<double*>(lin), const_cast<double*>(bias), n_moms, n_basic,
                                            (const int(*)[4])basic, n_times, (const int(*)[4])times, n_scalar, mapping,
                                            nmus, binum[b], il, nn, fn, rc, ty, ntypes, const_cast<int*>(type_map), U,
                                            nghost, rmax, rmin, const_cast<double*>(q_scaler));
        if (desc)
            LinearMtp<double>::find_descriptors(&desc[(size_t)b * P * n_scalar], K, scaling,
                                                const_cast<double*>(coeffs), n_moms, n_basic, (const int(*)[4])basic,
                                                n_times, (const int(*)[4])times, n_scalar, mapping, nmus, binum[b], il,
                                                nn, fn, rc, ty, ntypes, const_cast<int*>(type_map), U, nghost, rmax,
                                                rmin);
    }
}

// per-row derivatives of the site energies (linearMtp.h:616-818), contracted with gout[B, P] per
// structure as the operator's backward does (linearMtpOp.cc:4002-4005, before its sum over the batch)
void ref_mtp_esites_bwd_f64(double* dcoeffs, double* dlin, double* dbias, const double* gout, MTP_MODEL_ARGS,
                            MTP_LIST_ARGS)
{
    const int ncoef = ntypes * ntypes * nmus * K;
    std::vector<double> dc((size_t)P * ncoef), dl((size_t)P * n_scalar), db((size_t)P * ntypes);
    for (int b = 0; b < B; b++) {
        std::fill(dc.begin(), dc.end(), 0.0);
        std::fill(dl.begin(), dl.end(), 0.0);
        std::fill(db.begin(), db.end(), 0.0);
        LinearMtp<double>::find_e_sites_backward(
            dc.data(), dl.data(), db.data(), K, scaling, const_cast<double*>(coeffs), const_cast<double*>(lin),
            const_cast<double*>(bias), n_moms, n_basic, (const int(*)[4])basic, n_times, (const int(*)[4])times,
            n_scalar, mapping, nmus, binum[b], const_cast<int*>(&bilist[(size_t)b * P]),
            const_cast<int*>(&bnumneigh[(size_t)b * P]), const_cast<int*>(&bfirstneigh[(size_t)b * P * U]),
            (double(*)[3])const_cast<double*>(&brcs[(size_t)b * P * U * 3]),
            const_cast<int*>(&btypes[(size_t)b * (P + nghost)]), ntypes, const_cast<int*>(type_map), U, nghost, rmax,
            rmin, const_cast<double*>(q_scaler));
        for (int q = 0; q < ncoef; q++) {
            double a = 0;
            for (int ii = 0; ii < binum[b]; ii++) a += gout[(size_t)b * P + ii] * dc[(size_t)ii * ncoef + q];
            dcoeffs[(size_t)b * ncoef + q] = a;
        }
        for (int q = 0; q < n_scalar; q++) {
            double a = 0;
            for (int ii = 0; ii < binum[b]; ii++) a += gout[(size_t)b * P + ii] * dl[(size_t)ii * n_scalar + q];
            dlin[(size_t)b * n_scalar + q] = a;
        }
        for (int q = 0; q < ntypes; q++) {
            double a = 0;
            for (int ii = 0; ii < binum[b]; ii++) a += gout[(size_t)b * P + ii] * db[(size_t)ii * ntypes + q];
            dbias[(size_t)b * ntypes + q] = a;
        }
    }
}

// normal equations of the linear parameters by the reference's CPU launcher
// (linear_mtp_gram_and_cross.h:446-575), residuals = labels (the operator subtracts only a ZBL part)
void ref_mtp_lin_system_f64(double* lin_matrix, double* lin_vector, double e_w, double f_w, double v_w,
                            const double* e_res, const double* f_res, const double* v_res, MTP_MODEL_ARGS,
                            MTP_LIST_ARGS)
{
    LinearMtpGramAndCross<double>::find_lin_matrix_lin_vector_launcher(
        lin_matrix, lin_vector, e_w, f_w, v_w, const_cast<double*>(e_res), (double(*)[3])const_cast<double*>(f_res),
        const_cast<double*>(v_res), K, scaling, const_cast<double*>(coeffs), const_cast<double*>(lin),
        const_cast<double*>(bias), n_moms, n_basic, (const int(*)[4])basic, n_times, (const int(*)[4])times, n_scalar,
        mapping, nmus, B, P, const_cast<int*>(binum), const_cast<int*>(bilist), const_cast<int*>(bnumneigh),
        const_cast<int*>(bfirstneigh), (double(*)[3])const_cast<double*>(brcs), const_cast<int*>(btypes), ntypes,
        const_cast<int*>(type_map), U, nghost, rmax, rmin, const_cast<double*>(q_scaler));
}

// The legacy basis operator by the reference: MtpBasis::find_val_der (mtpBasis.h:107-356) with both dense
// derivative arrays, then find_der_backward (:359-394) with the weights w[B, P, n_scalar], per structure as
// the operator calls them (src/mtpBasisOp.cc:107-140, 277-300).  The tables, including the lists of radial
// functions behind each moment, are the reference's own (MtpParam of the level).  dcoeffs is kept per
// structure [B, ncoef] (the operator adds all structures into one vector).  Returns 1 if MtpParam fails.
int ref_mtp_basis_f64(double* val, double* drcs, double* dcoeffs, const double* w, int level, int K, double scaling,
                      const double* coeffs, int B, int P, const int* binum, const int* bilist, const int* bnumneigh,
                      const int* bfirstneigh, const double* brcs, const int* btypes, int ntypes, int U, int nghost,
                      double rmax, double rmin)
{
    try {
        MtpParam p(level);
        const int S = p.alpha_scalar_moments();
        const int ncoef = ntypes * ntypes * p.nmus() * K;
        std::vector<double> der((size_t)P * S * U * 3), der2c((size_t)P * S * ncoef);
        std::memset(val, 0, sizeof(double) * (size_t)B * P * S);
        std::memset(drcs, 0, sizeof(double) * (size_t)B * P * U * 3);
        std::memset(dcoeffs, 0, sizeof(double) * (size_t)B * ncoef);
        for (int b = 0; b < B; b++) {
            std::fill(der.begin(), der.end(), 0.0);
            std::fill(der2c.begin(), der2c.end(), 0.0);
            MtpBasis<double>::find_val_der(
                &val[(size_t)b * P * S], (double(*)[3])der.data(), der2c.data(), true, true, K, scaling,
                const_cast<double*>(coeffs), p.alpha_moments_count(), p.alpha_index_basic_count(), p.alpha_index_basic(),
                p.alpha_index_times_count(), p.alpha_index_times(), S, p.alpha_moment_mapping(), p.max_num_mus4mom(),
                p.num_mus4moms(), p.mus4moms_ptr(), p.nmus(), binum[b], const_cast<int*>(&bilist[(size_t)b * P]),
                const_cast<int*>(&bnumneigh[(size_t)b * P]), const_cast<int*>(&bfirstneigh[(size_t)b * P * U]),
                (double(*)[3])const_cast<double*>(&brcs[(size_t)b * P * U * 3]),
                const_cast<int*>(&btypes[(size_t)b * (P + nghost)]), ntypes, U, rmax, rmin);
            MtpBasis<double>::find_der_backward(&drcs[(size_t)b * P * U * 3], &dcoeffs[(size_t)b * ncoef], true, true,
                                                const_cast<double*>(&w[(size_t)b * P * S]), der.data(), der2c.data(), S,
                                                binum[b], U, ncoef);
        }
        return 0;
    } catch (MtpException& e) {
        return 1;
    }
}

void ref_mtp_schmidt_orth_f64(double* out, int ntypes, int nmus, int K, const double* in)
{
    CoeffsSchmidtOrth<double>::find_orthogonal_basis_set(out, ntypes, nmus, K, const_cast<double*>(in));
}
}
