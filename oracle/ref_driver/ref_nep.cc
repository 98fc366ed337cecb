// TEST INFRASTRUCTURE ONLY. extern "C" driver around the reference's NEP CPU launchers
// (REF_ROOT/source/descriptor/nep/include/nep_cpu_launcher.h:186-255, 259-317), compiled
// from the reference headers where they lie into oracle/_ref/libref_nep.so.
// Output buffers are zeroed here because the reference op allocates them with at::zeros
// (source/descriptor/nep/src/nepOp.cc:998-1000) and Nep::find_efv only accumulates.
#include <cstring>
#include "descriptor/nep/include/nep_cpu_launcher.h"
#include "descriptor/nep/include/nepLoss_cpu_launcher.h"

namespace {
template <typename T>
void efv(T* betot, T* bforce, T* bvirial, int K, int n_r, int n_a, int l_max, int H,
         const T* coeffs, const T* w0, const T* b0, const T* w1, const T* bias,
         int B, int P, const int* binum, const int* bilist, const int* bnumneigh,
         const int* bfirstneigh, const T* brcs, const int* btypes, int ntypes, const int* type_map,
         int U, int nghost, double rr, double ra, const T* q_scaler)
{
    std::memset(betot, 0, sizeof(T) * B);
    std::memset(bforce, 0, sizeof(T) * B * (P + nghost) * 3);
    std::memset(bvirial, 0, sizeof(T) * B * 9);
    ai2pot::nep::find_efv_cpu_launcher<T>(
        betot, (T(*)[3])bforce, bvirial, K, n_r, n_a, l_max, H,
        const_cast<T*>(coeffs), const_cast<T*>(w0), const_cast<T*>(b0), const_cast<T*>(w1),
        const_cast<T*>(bias), B, P, const_cast<int*>(binum), const_cast<int*>(bilist),
        const_cast<int*>(bnumneigh), const_cast<int*>(bfirstneigh), (T(*)[3])const_cast<T*>(brcs),
        const_cast<int*>(btypes), ntypes, const_cast<int*>(type_map), U, nghost, (T)rr, (T)ra,
        const_cast<T*>(q_scaler));
}

template <typename T>
void desc(T* bdesc, int K, int n_r, int n_a, int l_max, const T* coeffs, int B, int P,
          const int* binum, const int* bilist, const int* bnumneigh, const int* bfirstneigh,
          const T* brcs, const int* btypes, int ntypes, const int* type_map, int U, int nghost,
          double rr, double ra)
{
    int D = ai2pot::nep::NepIndex::get_num_descriptors(n_r, n_a, l_max);
    std::memset(bdesc, 0, sizeof(T) * B * P * D);
    ai2pot::nep::find_descriptors_cpu_launcher<T>(
        bdesc, K, n_r, n_a, l_max, const_cast<T*>(coeffs), B, P, const_cast<int*>(binum),
        const_cast<int*>(bilist), const_cast<int*>(bnumneigh), const_cast<int*>(bfirstneigh),
        (T(*)[3])const_cast<T*>(brcs), const_cast<int*>(btypes), ntypes,
        const_cast<int*>(type_map), U, nghost, (T)rr, (T)ra);
}
}  // namespace

#define ARGS_EFV(T) T* betot, T* bforce, T* bvirial, int K, int n_r, int n_a, int l_max, int H, \
    const T* coeffs, const T* w0, const T* b0, const T* w1, const T* bias, int B, int P, \
    const int* binum, const int* bilist, const int* bnumneigh, const int* bfirstneigh, \
    const T* brcs, const int* btypes, int ntypes, const int* type_map, int U, int nghost, \
    double rr, double ra, const T* q_scaler
#define PASS_EFV betot, bforce, bvirial, K, n_r, n_a, l_max, H, coeffs, w0, b0, w1, bias, B, P, \
    binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, ntypes, type_map, U, nghost, rr, ra, q_scaler
#define ARGS_DESC(T) T* bdesc, int K, int n_r, int n_a, int l_max, const T* coeffs, int B, int P, \
    const int* binum, const int* bilist, const int* bnumneigh, const int* bfirstneigh, \
    const T* brcs, const int* btypes, int ntypes, const int* type_map, int U, int nghost, \
    double rr, double ra
#define PASS_DESC bdesc, K, n_r, n_a, l_max, coeffs, B, P, binum, bilist, bnumneigh, bfirstneigh, \
    brcs, btypes, ntypes, type_map, U, nghost, rr, ra

extern "C" {
// forward + backward of the training-loss op (nepOp.cc:2359-2960 on the CPU branch): E/F/V of the
// model, bloss[B], rmse[3] (e, f, v) and the per-structure gradients
// dcoeffs[B,ncoef], dw0[B,ntypes*H*D], db0[B,ntypes*H], dw1[B,ntypes*H], dbias[B,ntypes].
void ref_nep_loss_step_f64(double* bloss, double* rmse, double* betot, double* bforce, double* bvirial,
                           double* dcoeffs, double* dw0, double* db0, double* dw1, double* dbias, double e_w,
                           double f_w, double v_w, const double* e_dft, const double* f_dft, const double* v_dft,
                           int K, int n_r, int n_a, int l_max, int H, const double* coeffs, const double* w0,
                           const double* b0, const double* w1, const double* bias, int B, int P, const int* binum,
                           const int* bilist, const int* bnumneigh, const int* bfirstneigh, const double* brcs,
                           const int* btypes, int ntypes, const int* type_map, int U, int nghost, double rr,
                           double ra, const double* q_scaler)
{
    using namespace ai2pot::nep;
    efv<double>(betot, bforce, bvirial, K, n_r, n_a, l_max, H, coeffs, w0, b0, w1, bias, B, P, binum, bilist,
                bnumneigh, bfirstneigh, brcs, btypes, ntypes, type_map, U, nghost, rr, ra, q_scaler);
    double* e0 = const_cast<double*>(e_dft);
    double(*f0)[3] = (double(*)[3])const_cast<double*>(f_dft);
    double* v0 = const_cast<double*>(v_dft);
    find_loss_cpu_launcher<double>(bloss, B, P, const_cast<int*>(binum), const_cast<int*>(bilist), e_w, f_w, v_w,
                                   betot, e0, (double(*)[3])bforce, f0, bvirial, v0);
    find_efv_rmse_cpu_launcher<double>(rmse[0], rmse[1], rmse[2], B, P, const_cast<int*>(binum),
                                       const_cast<int*>(bilist), betot, e0, (double(*)[3])bforce, f0, bvirial, v0);
    const int D = NepIndex::get_num_descriptors(n_r, n_a, l_max);
    std::memset(dcoeffs, 0, sizeof(double) * B * ntypes * ntypes * (n_r + n_a) * K);
    std::memset(dw0, 0, sizeof(double) * B * ntypes * H * D);
    std::memset(db0, 0, sizeof(double) * B * ntypes * H);
    std::memset(dw1, 0, sizeof(double) * B * ntypes * H);
    std::memset(dbias, 0, sizeof(double) * B * ntypes);
    find_loss_backward_cpu_launcher<double>(
        dcoeffs, dw0, db0, dw1, dbias, e_w, f_w, v_w, betot, e0, (double(*)[3])bforce, f0, bvirial, v0, K, n_r, n_a,
        l_max, H, const_cast<double*>(coeffs), const_cast<double*>(w0), const_cast<double*>(b0),
        const_cast<double*>(w1), const_cast<double*>(bias), B, P, const_cast<int*>(binum), const_cast<int*>(bilist),
        const_cast<int*>(bnumneigh), const_cast<int*>(bfirstneigh), (double(*)[3])const_cast<double*>(brcs),
        const_cast<int*>(btypes), ntypes, const_cast<int*>(type_map), U, nghost, rr, ra,
        const_cast<double*>(q_scaler));
}

void ref_nep_efv_f32(ARGS_EFV(float)) { efv<float>(PASS_EFV); }
void ref_nep_efv_f64(ARGS_EFV(double)) { efv<double>(PASS_EFV); }
void ref_nep_desc_f32(ARGS_DESC(float)) { desc<float>(PASS_DESC); }
void ref_nep_desc_f64(ARGS_DESC(double)) { desc<double>(PASS_DESC); }
}
