// TEST INFRASTRUCTURE ONLY. extern "C" driver around the reference's neural-network MTP
// (REF_ROOT/source/descriptor/nnmtp/include/nnMtp.h:378-567 find_efv, :648-753 find_e_sites,
// :570-645 find_descriptors), called per structure as the operator's CPU branch does
// (src/nnMtpOp.cc:2857-2927), built into oracle/_ref/libref_nnmtp.so.
#include <cstring>
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
}
