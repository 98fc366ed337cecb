// Training-loss forward pieces shared by the MTP and NEP loss operators: per-structure loss,
// the scaled residuals the gradient kernels need, and the batch RMSEs.
#pragma once
#include "a2p_common.h"

namespace a2p {
namespace losskern {

// One block per structure: loss (linearMtpLoss.h:138-176 = nepLoss.h:170-209), the scaled
// residuals the gradient kernel needs, and the per-structure squared errors for the RMSEs.
template <typename T>
__global__ void __launch_bounds__(256)
loss_forward_kernel(int P, const int* __restrict__ binum, const int* __restrict__ bilist, T e_w, T f_w,
                        T v_w, const T* __restrict__ etot, const T* __restrict__ e_dft,
                        const T* __restrict__ force, const T* __restrict__ f_dft,
                        const T* __restrict__ virial, const T* __restrict__ v_dft, T* __restrict__ bloss,
                        T* __restrict__ cE, T* __restrict__ dFs, T* __restrict__ dVs,
                        double* __restrict__ sq,   // [B, 3]: (dE/N)^2, sum dF^2, sum (dV/N)^2 or sum dV^2
                        int virial_per_atom)       // 1: linearMtpLoss_cpu_launcher.h:477-527; 0: nepLoss_cpu_launcher.h:376-405
{
    __shared__ double sh[4];
    const int b = blockIdx.x;
    const int inum = binum[b];
    const T fscale = (T)2 * f_w / (T)(3 * inum);
    for (int q = threadIdx.x; q < P * 3; q += 256) dFs[(size_t)b * P * 3 + q] = (T)0;
    __syncthreads();
    double fl = 0.0;
    for (int ii = threadIdx.x; ii < inum; ii += 256) {
        const int c = bilist[(size_t)b * P + ii];
        for (int q = 0; q < 3; q++) {
            const T dlt = force[((size_t)b * P + c) * 3 + q] - f_dft[((size_t)b * P + c) * 3 + q];
            fl += (double)dlt * (double)dlt;
            dFs[((size_t)b * P + c) * 3 + q] = fscale * dlt;
        }
    }
    fl = wave_sum(fl);
    if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = fl;
    __syncthreads();
    if (threadIdx.x == 0) {
        const double fsum = sh[0] + sh[1] + sh[2] + sh[3];
        double vsum = 0.0;
        for (int q = 0; q < 9; q++) {
            const T dlt = virial[b * 9 + q] - v_dft[b * 9 + q];
            vsum += (double)dlt * (double)dlt;
            dVs[b * 9 + q] = (T)2 * v_w / (T)(9 * inum) * dlt;
        }
        const T de = etot[b] - e_dft[b];
        cE[b] = (T)2 * e_w / (T)inum * de;
        bloss[b] = (T)((double)f_w / (3.0 * inum) * fsum + (double)v_w / (9.0 * inum) * vsum +
                       (double)e_w / inum * (double)de * (double)de);
        sq[b * 3 + 0] = ((double)de / inum) * ((double)de / inum);
        sq[b * 3 + 1] = fsum;
        sq[b * 3 + 2] = virial_per_atom ? vsum / ((double)inum * inum) : vsum;
    }
}

template <typename T>
__global__ void loss_rmse_kernel(int B, const int* __restrict__ binum, const double* __restrict__ sq,
                                T* __restrict__ rmse)
{
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    double e = 0, f = 0, v = 0;
    long nf = 0;
    for (int b = 0; b < B; b++) { e += sq[b * 3]; f += sq[b * 3 + 1]; v += sq[b * 3 + 2]; nf += 3L * binum[b]; }
    rmse[0] = (T)sqrt(e / B);
    rmse[1] = (T)sqrt(f / (double)nf);
    rmse[2] = (T)sqrt(v / (9.0 * B));
}

}  // namespace losskern
}  // namespace a2p
