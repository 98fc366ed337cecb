// ZBL short-range correction added onto energies, forces and virials: the screened nuclear
// repulsion of the reference (source/descriptor/correction/include/zbl.h:262-395: switching
// function, screening function, pair energy, force and virial of one ordered pair), composed per
// centre atom as its device code does (correction/gpu/include/zbl.cuh:422-500, 502-620):
//   every ordered pair (i, j) of the list with r <= rmax gives  0.5 E_pair  to the energy,
//   dE_pair/dr * r_vec / r  to the force of the CENTRE atom i only (the pair (j, i) of a full list
//   supplies the other half; ghosts receive nothing), and  -0.5 r_a dE_pair/dr r_b / r  to the virial.
// The site-energy operators take the per-row sums of the 0.5 E_pair terms instead (GroupZBL::correct_e_sites,
// zbl.h:625-685).
// One thread per row; the force is written by its row's thread alone, energy and virial leave
// each workgroup as fp64 partial sums that a second kernel adds onto the outputs in block order.
#include "a2p_common.h"

namespace a2p {
namespace {

constexpr int ZB = 256;

template <typename T> __device__ __forceinline__ T exp_t(T x);
template <> __device__ __forceinline__ float exp_t<float>(float x) { return expf(x); }
template <> __device__ __forceinline__ double exp_t<double>(double x) { return exp(x); }
template <typename T> __device__ __forceinline__ T pow_t(T x, T y);
template <> __device__ __forceinline__ float pow_t<float>(float x, float y) { return powf(x, y); }
template <> __device__ __forceinline__ double pow_t<double>(double x, double y) { return pow(x, y); }
template <typename T> __device__ __forceinline__ T sqrt_t(T x);
template <> __device__ __forceinline__ float sqrt_t<float>(float x) { return sqrtf(x); }
template <> __device__ __forceinline__ double sqrt_t<double>(double x) { return sqrt(x); }

template <typename T>
__global__ void __launch_bounds__(ZB)
zbl_kernel(int B, int P, int U, int nghost, const int* __restrict__ binum, const int* __restrict__ bilist,
           const int* __restrict__ bnumneigh, const int* __restrict__ bfirstneigh, const T* __restrict__ brcs,
           const int* __restrict__ btypes, int ntypes, const int* __restrict__ type_map, T rmax, T rmin,
           const T* __restrict__ cks, const T* __restrict__ dks, T* __restrict__ force,
           double* __restrict__ partial, int nblocks, int* __restrict__ status, T* __restrict__ e_sites)
{
    __shared__ double red[ZB / 64][10];
    const int b = blockIdx.y, ii = blockIdx.x * ZB + threadIdx.x;
    const int NF = P + nghost;
    const T kc = (T)14.399645;                          // zbl.h:34, 1 / (4 pi eps0) in eV Angstrom
    double acc[10];
#pragma unroll
    for (int q = 0; q < 10; q++) acc[q] = 0.0;
    if (ii < P && ii < binum[b]) {
        const size_t row = (size_t)b * P + ii;
        const int* types = btypes + (size_t)b * NF;
        int center = bilist[row];
        int nn = min(bnumneigh[row], U);
        if ((unsigned)center >= (unsigned)NF) { atomicOr(status, ST_BAD_NEIGHBOR); center = 0; nn = 0; }
        int ti = types[center];
        if ((unsigned)ti >= (unsigned)ntypes) { atomicOr(status, ST_BAD_TYPE); ti = 0; nn = 0; }
        const T Zi = (T)type_map[ti];
        const T zi23 = pow_t(Zi, (T)0.23);
        T e = (T)0, f[3] = {(T)0, (T)0, (T)0}, v[9];
#pragma unroll
        for (int q = 0; q < 9; q++) v[q] = (T)0;
        for (int jj = 0; jj < nn; jj++) {
            const T* p = brcs + (row * U + jj) * 3;
            const T x = p[0], y = p[1], z = p[2];
            const T r = sqrt_t(x * x + y * y + z * z);
            if (r > rmax) continue;                                            // zbl.cuh:455-456
            int nj = bfirstneigh[row * U + jj];
            if ((unsigned)nj >= (unsigned)NF) { atomicOr(status, ST_BAD_NEIGHBOR); continue; }
            int tj = types[nj];
            if ((unsigned)tj >= (unsigned)ntypes) { atomicOr(status, ST_BAD_TYPE); continue; }
            const T Zj = (T)type_map[tj];
            const T* ck = cks + (size_t)(ti * ntypes + tj) * 4;
            const T* dk = dks + (size_t)(ti * ntypes + tj) * 4;
            const T a = (T)0.46848 / (zi23 + pow_t(Zj, (T)0.23));               // zbl.h:291-318
            T phi = (T)0, dphi = (T)0;
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const T ex = exp_t(-dk[k] * r / a);
                phi += ck[k] * ex;
                dphi -= ck[k] * dk[k] / a * ex;
            }
            T sw = (T)1, dsw = (T)0;                                           // zbl.h:262-288
            if (r >= rmin) {
                const T u = (r - rmin) / (rmax - rmin);
                sw = u * u * u * ((T)-6 * u * u + (T)15 * u - (T)10) + (T)1;
                dsw = (T)1 / (rmax - rmin) * ((T)-30 * u * u * u * u + (T)60 * u * u * u - (T)30 * u * u);
            }
            const T A = kc * Zi * Zj / r, dA = -kc * Zi * Zj / (r * r);
            e += (T)0.5 * A * phi * sw;                                        // zbl.h:331-339
            const T dEdr = dA * phi * sw + A * dphi * sw + A * phi * dsw;      // zbl.h:343-365
            const T rv[3] = {x, y, z};
#pragma unroll
            for (int c = 0; c < 3; c++) {
                f[c] += dEdr * rv[c] / r;
#pragma unroll
                for (int d = 0; d < 3; d++) v[c * 3 + d] += (T)-0.5 * rv[c] * (dEdr * rv[d] / r);   // zbl.h:369-393
            }
        }
        if (force) {
            T* fo = force + ((size_t)b * NF + center) * 3;
            fo[0] += f[0]; fo[1] += f[1]; fo[2] += f[2];
        }
        if (e_sites) e_sites[row] += e;                     // GroupZBL::correct_e_sites, zbl.h:625-685
        acc[0] = (double)e;
#pragma unroll
        for (int q = 0; q < 9; q++) acc[1 + q] = (double)v[q];
    }
#pragma unroll
    for (int q = 0; q < 10; q++) {
        const double s = wave_sum(acc[q]);
        if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6][q] = s;
    }
    __syncthreads();
    if (threadIdx.x < 10) {
        double s = 0.0;
        for (int w = 0; w < ZB / 64; w++) s += red[w][threadIdx.x];
        partial[((size_t)b * nblocks + blockIdx.x) * 10 + threadIdx.x] = s;
    }
}

// etot[b] += sum of the blocks' energies, virial[b, q] += sum of their virials, in block order
template <typename T>
__global__ void zbl_add_kernel(const double* __restrict__ partial, int nblocks, T* __restrict__ etot,
                               T* __restrict__ virial)
{
    const int b = blockIdx.x, q = threadIdx.x;
    if (q >= 10) return;
    double s = 0.0;
    for (int k = 0; k < nblocks; k++) s += partial[((size_t)b * nblocks + k) * 10 + q];
    if (q == 0) { if (etot) etot[b] = (T)((double)etot[b] + s); }
    else if (virial) virial[(size_t)b * 9 + q - 1] = (T)((double)virial[(size_t)b * 9 + q - 1] + s);
}

template <typename T>
int zbl_correct(double rmax, double rmin, const T* cks, const T* dks, int ntypes, const int* type_map, int B, int P,
                int U, int nghost, const int* binum, const int* bilist, const int* bnumneigh, const int* bfirstneigh,
                const T* brcs, const int* btypes, T* etot, T* force, T* virial, hipStream_t stream,
                T* e_sites = nullptr)
{
    A2P_REQUIRE(rmax > rmin && rmin >= 0, A2P_ERR_INVALID, "zbl: need 0 <= zbl_rmin < zbl_rmax");
    A2P_REQUIRE(cks && dks && type_map && binum && bilist && bnumneigh && bfirstneigh && brcs && btypes,
                A2P_ERR_INVALID, "zbl: null input pointer");
    A2P_REQUIRE(ntypes >= 1 && B >= 0 && P >= 0 && U >= 1 && nghost >= 0, A2P_ERR_INVALID, "zbl: bad shape");
    if (B == 0 || P == 0 || (!etot && !force && !virial && !e_sites)) return A2P_OK;
    const int nblocks = ceil_div(P, ZB);
    void* ws = nullptr;
    int rc = ws_get(WS_FLAGS, 64, &ws);
    if (rc) return rc;
    int* status = (int*)ws;
    rc = ws_get(WS_PARTIAL, (size_t)B * nblocks * 10 * sizeof(double), &ws);
    if (rc) return rc;
    double* partial = (double*)ws;
    prof_begin("zbl_kernel", stream);
    hipLaunchKernelGGL(zbl_kernel<T>, dim3(nblocks, B), dim3(ZB), 0, stream, B, P, U, nghost, binum, bilist,
                       bnumneigh, bfirstneigh, brcs, btypes, ntypes, type_map, (T)rmax, (T)rmin, cks, dks, force,
                       partial, nblocks, status, e_sites);
    if (etot || virial)
        hipLaunchKernelGGL(zbl_add_kernel<T>, dim3(B), dim3(64), 0, stream, partial, nblocks, etot, virial);
    prof_end(stream);
    A2P_HIP_CHECK(hipGetLastError());
    return A2P_OK;
}

}  // namespace
}  // namespace a2p

extern "C" {
int a2p_zbl_correct_f64(double zbl_rmax, double zbl_rmin, const double* zbl_cks, const double* zbl_dks, int ntypes,
                        const int* type_map, int B, int P, int U, int nghost, const int* binum, const int* bilist,
                        const int* bnumneigh, const int* bfirstneigh, const double* brcs, const int* btypes,
                        double* etot, double* force, double* virial, void* stream)
{
    return a2p::zbl_correct<double>(zbl_rmax, zbl_rmin, zbl_cks, zbl_dks, ntypes, type_map, B, P, U, nghost, binum,
                                    bilist, bnumneigh, bfirstneigh, brcs, btypes, etot, force, virial,
                                    (hipStream_t)stream);
}
int a2p_zbl_correct_f32(double zbl_rmax, double zbl_rmin, const float* zbl_cks, const float* zbl_dks, int ntypes,
                        const int* type_map, int B, int P, int U, int nghost, const int* binum, const int* bilist,
                        const int* bnumneigh, const int* bfirstneigh, const float* brcs, const int* btypes,
                        float* etot, float* force, float* virial, void* stream)
{
    return a2p::zbl_correct<float>(zbl_rmax, zbl_rmin, zbl_cks, zbl_dks, ntypes, type_map, B, P, U, nghost, binum,
                                   bilist, bnumneigh, bfirstneigh, brcs, btypes, etot, force, virial,
                                   (hipStream_t)stream);
}
int a2p_zbl_esites_f64(double zbl_rmax, double zbl_rmin, const double* zbl_cks, const double* zbl_dks, int ntypes,
                       const int* type_map, int B, int P, int U, int nghost, const int* binum, const int* bilist,
                       const int* bnumneigh, const int* bfirstneigh, const double* brcs, const int* btypes,
                       double* be_sites, void* stream)
{
    A2P_REQUIRE(be_sites, A2P_ERR_INVALID, "zbl: null be_sites");
    return a2p::zbl_correct<double>(zbl_rmax, zbl_rmin, zbl_cks, zbl_dks, ntypes, type_map, B, P, U, nghost, binum,
                                    bilist, bnumneigh, bfirstneigh, brcs, btypes, nullptr, nullptr, nullptr,
                                    (hipStream_t)stream, be_sites);
}
int a2p_zbl_esites_f32(double zbl_rmax, double zbl_rmin, const float* zbl_cks, const float* zbl_dks, int ntypes,
                       const int* type_map, int B, int P, int U, int nghost, const int* binum, const int* bilist,
                       const int* bnumneigh, const int* bfirstneigh, const float* brcs, const int* btypes,
                       float* be_sites, void* stream)
{
    A2P_REQUIRE(be_sites, A2P_ERR_INVALID, "zbl: null be_sites");
    return a2p::zbl_correct<float>(zbl_rmax, zbl_rmin, zbl_cks, zbl_dks, ntypes, type_map, B, P, U, nghost, binum,
                                   bilist, bnumneigh, bfirstneigh, brcs, btypes, nullptr, nullptr, nullptr,
                                   (hipStream_t)stream, be_sites);
}
}
