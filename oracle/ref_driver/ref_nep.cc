// TEST INFRASTRUCTURE ONLY. extern "C" driver around the reference's NEP CPU launchers
// (REF_ROOT/source/descriptor/nep/include/nep_cpu_launcher.h:186-255, 259-317), compiled
// from the reference headers where they lie into oracle/_ref/libref_nep.so.
// Output buffers are zeroed here because the reference op allocates them with at::zeros
// (source/descriptor/nep/src/nepOp.cc:998-1000) and Nep::find_efv only accumulates.
#include <cstring>
#include "descriptor/nep/include/nep_cpu_launcher.h"

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
void ref_nep_efv_f32(ARGS_EFV(float)) { efv<float>(PASS_EFV); }
void ref_nep_efv_f64(ARGS_EFV(double)) { efv<double>(PASS_EFV); }
void ref_nep_desc_f32(ARGS_DESC(float)) { desc<float>(PASS_DESC); }
void ref_nep_desc_f64(ARGS_DESC(double)) { desc<double>(PASS_DESC); }
}
