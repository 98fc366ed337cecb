// Short-range force and virial from per-pair derivatives dE_i/dr_ij, and their
// vector-Jacobian products, for gfx950.
//
//   force : F[c] = sum_s g[ii,s] - sum over pairs whose neighbour is c of g   (c = ilist[ii])
//           reference: source/fvt/include/force_sr.h:50-84.  The own-row sum is one wavefront
//           per row; the neighbour part is a2p::pair_reduce (no floating-point atomics).
//   virial: V[a,b] = - sum_{ii,s} g[ii,s,a] r[ii,s,b]          source/fvt/include/virial_sr.h:24-51
// The reference materialises dense Jacobians [(nlocal+nghost)*3, nlocal*umax] and
// [9, nlocal*umax] (src/force_sr_op.cc:44, src/virial_sr_op.cc:31-32) and multiplies by them
// in backward; the Jacobian entries are +-1, -r and -g, so the products are written directly:
//   dL/dg[ii,s,k]  = gF[c,k] - gF[j,k]                         (force_sr.h:99-124)
//   dL/dg[ii,s,a]  = - sum_b gV[a,b] r[ii,s,b],   dL/dr[ii,s,b] = - sum_a gV[a,b] g[ii,s,a]
#include "a2p_common.h"

#include <mutex>

namespace a2p {
namespace {

template <typename T>
__global__ void __launch_bounds__(256)
force_own_kernel(T* __restrict__ force, const T* __restrict__ g, int B, int P, int U, int NF,
                 const int* __restrict__ binum, const int* __restrict__ bilist,
                 const int* __restrict__ bnumneigh, int* __restrict__ status)
{
    const int row = (blockIdx.x * 256 + threadIdx.x) >> 6, lane = threadIdx.x & 63;
    if (row >= B * P) return;
    const int b = row / P, ii = row - b * P;
    if (ii >= binum[b]) return;
    int nn = bnumneigh[row];
    if (nn > U) { if (lane == 0) atomicOr(status, ST_NEIGH_OVERFLOW); nn = U; }
    const int c = bilist[row];
    if ((unsigned)c >= (unsigned)NF) { if (lane == 0) atomicOr(status, ST_BAD_NEIGHBOR); return; }
    const T* gr = g + (size_t)row * U * 3;
    T sx = 0, sy = 0, sz = 0;
    for (int s = lane; s < nn; s += 64) { sx += gr[s * 3]; sy += gr[s * 3 + 1]; sz += gr[s * 3 + 2]; }
    sx = wave_sum(sx); sy = wave_sum(sy); sz = wave_sum(sz);
    if (lane == 0) {
        T* f = force + ((size_t)b * NF + c) * 3;
        f[0] = sx; f[1] = sy; f[2] = sz;
    }
}

template <typename T>
__global__ void __launch_bounds__(256)
force_bwd_kernel(T* __restrict__ gout, const T* __restrict__ gF, int B, int P, int U, int NF,
                 const int* __restrict__ binum, const int* __restrict__ bilist,
                 const int* __restrict__ bnumneigh, const int* __restrict__ bfirstneigh)
{
    const int row = (blockIdx.x * 256 + threadIdx.x) >> 6, lane = threadIdx.x & 63;
    if (row >= B * P) return;
    const int b = row / P, ii = row - b * P;
    int nn = 0, c = 0;
    if (ii < binum[b]) {
        nn = min(bnumneigh[row], U);
        c = bilist[row];
        if ((unsigned)c >= (unsigned)NF) nn = 0;
    }
    T* out = gout + (size_t)row * U * 3;
    const T* fc = gF + ((size_t)b * NF + c) * 3;
    const int* first = bfirstneigh + (size_t)row * U;
    for (int s = lane; s < U; s += 64) {
        T v0 = 0, v1 = 0, v2 = 0;
        if (s < nn) {
            const int j = first[s];
            if ((unsigned)j < (unsigned)NF) {
                const T* fj = gF + ((size_t)b * NF + j) * 3;
                v0 = fc[0] - fj[0]; v1 = fc[1] - fj[1]; v2 = fc[2] - fj[2];
            }
        }
        out[s * 3] = v0; out[s * 3 + 1] = v1; out[s * 3 + 2] = v2;
    }
}

// one wavefront per row -> 9 partial sums per row (fp64), reduced by finish_partials
template <typename T>
__global__ void __launch_bounds__(256)
virial_rows_kernel(double* __restrict__ partial, const T* __restrict__ g, const T* __restrict__ r, int B,
                   int P, int U, const int* __restrict__ bnumneigh)
{
    const int row = (blockIdx.x * 256 + threadIdx.x) >> 6, lane = threadIdx.x & 63;
    if (row >= B * P) return;
    const int nn = min(bnumneigh[row], U);
    const T* gr = g + (size_t)row * U * 3;
    const T* rr = r + (size_t)row * U * 3;
    double v[9];
#pragma unroll
    for (int q = 0; q < 9; q++) v[q] = 0.0;
    for (int s = lane; s < nn; s += 64) {
#pragma unroll
        for (int a = 0; a < 3; a++)
#pragma unroll
            for (int c = 0; c < 3; c++) v[a * 3 + c] -= (double)gr[s * 3 + a] * (double)rr[s * 3 + c];
    }
#pragma unroll
    for (int q = 0; q < 9; q++) {
        const double t = wave_sum(v[q]);
        if (lane == 0) partial[(size_t)row * 9 + q] = t;
    }
}

template <typename T>
__global__ void __launch_bounds__(256)
virial_bwd_kernel(T* __restrict__ gg, T* __restrict__ gr, const T* __restrict__ gV, const T* __restrict__ g,
                  const T* __restrict__ r, int B, int P, int U, const int* __restrict__ bnumneigh)
{
    const int row = (blockIdx.x * 256 + threadIdx.x) >> 6, lane = threadIdx.x & 63;
    if (row >= B * P) return;
    const int b = row / P;
    const int nn = min(bnumneigh[row], U);
    T m[9];
#pragma unroll
    for (int q = 0; q < 9; q++) m[q] = gV[b * 9 + q];
    const size_t base = (size_t)row * U * 3;
    for (int s = lane; s < U; s += 64) {
        T og[3] = {0, 0, 0}, orr[3] = {0, 0, 0};
        if (s < nn) {
            const T g0 = g[base + s * 3], g1 = g[base + s * 3 + 1], g2 = g[base + s * 3 + 2];
            const T r0 = r[base + s * 3], r1 = r[base + s * 3 + 1], r2 = r[base + s * 3 + 2];
#pragma unroll
            for (int a = 0; a < 3; a++) og[a] = -(m[a * 3] * r0 + m[a * 3 + 1] * r1 + m[a * 3 + 2] * r2);
#pragma unroll
            for (int c = 0; c < 3; c++) orr[c] = -(m[c] * g0 + m[3 + c] * g1 + m[6 + c] * g2);
        }
        if (gg) { gg[base + s * 3] = og[0]; gg[base + s * 3 + 1] = og[1]; gg[base + s * 3 + 2] = og[2]; }
        if (gr) { gr[base + s * 3] = orr[0]; gr[base + s * 3 + 1] = orr[1]; gr[base + s * 3 + 2] = orr[2]; }
    }
}

int check_shape(int B, int P, int U, int nghost)
{
    A2P_REQUIRE(B >= 0 && P >= 0 && U >= 1 && nghost >= 0, A2P_ERR_INVALID, "fvt: bad shape");
    A2P_REQUIRE((long long)B * P * U < (1ll << 31), A2P_ERR_INVALID, "fvt: batch too large");
    return A2P_OK;
}

template <typename T>
int force_fwd(int B, int P, int U, int nghost, const int* binum, const int* bilist, const int* bnumneigh,
              const int* bfirstneigh, const T* dei, T* force, hipStream_t stream)
{
    int rc = check_shape(B, P, U, nghost);
    if (rc) return rc;
    A2P_REQUIRE(binum && bilist && bnumneigh && bfirstneigh && dei && force, A2P_ERR_INVALID,
                "fvt force: null pointer");
    if (B == 0 || P == 0) return A2P_OK;
    void* flags = nullptr;
    rc = ws_get(WS_FLAGS, 64, &flags);
    if (rc) return rc;
    rc = fill_zero(force, (size_t)B * (P + nghost) * 3 * sizeof(T), stream);
    if (rc) return rc;
    prof_begin("fvt_force_own", stream);
    hipLaunchKernelGGL(force_own_kernel<T>, dim3(ceil_div((long long)B * P * 64, 256)), dim3(256), 0, stream,
                       force, dei, B, P, U, P + nghost, binum, bilist, bnumneigh, (int*)flags);
    prof_end(stream);
    A2P_HIP_CHECK(hipGetLastError());
    return pair_reduce<T>(force, dei, B, P, U, nghost, binum, bnumneigh, bfirstneigh, stream);
}

template <typename T>
int force_bwd(int B, int P, int U, int nghost, const int* binum, const int* bilist, const int* bnumneigh,
              const int* bfirstneigh, const T* grad_force, T* grad_dei, hipStream_t stream)
{
    int rc = check_shape(B, P, U, nghost);
    if (rc) return rc;
    A2P_REQUIRE(binum && bilist && bnumneigh && bfirstneigh && grad_force && grad_dei, A2P_ERR_INVALID,
                "fvt force backward: null pointer");
    if (B == 0 || P == 0) return A2P_OK;
    prof_begin("fvt_force_bwd", stream);
    hipLaunchKernelGGL(force_bwd_kernel<T>, dim3(ceil_div((long long)B * P * 64, 256)), dim3(256), 0, stream,
                       grad_dei, grad_force, B, P, U, P + nghost, binum, bilist, bnumneigh, bfirstneigh);
    prof_end(stream);
    A2P_HIP_CHECK(hipGetLastError());
    return A2P_OK;
}

template <typename T>
int virial_fwd(int B, int P, int U, const int* bnumneigh, const T* rcs, const T* dei, T* virial,
               hipStream_t stream)
{
    int rc = check_shape(B, P, U, 0);
    if (rc) return rc;
    A2P_REQUIRE(bnumneigh && rcs && dei && virial, A2P_ERR_INVALID, "fvt virial: null pointer");
    if (B == 0) return A2P_OK;
    if (P == 0) return fill_zero(virial, (size_t)B * 9 * sizeof(T), stream);
    void* ws = nullptr;
    rc = ws_get(WS_PARTIAL, (size_t)B * P * 9 * sizeof(double), &ws);
    if (rc) return rc;
    prof_begin("fvt_virial_rows", stream);
    hipLaunchKernelGGL(virial_rows_kernel<T>, dim3(ceil_div((long long)B * P * 64, 256)), dim3(256), 0, stream,
                       (double*)ws, dei, rcs, B, P, U, bnumneigh);
    prof_end(stream);
    A2P_HIP_CHECK(hipGetLastError());
    return finish_partials<T>(virial, (const double*)ws, B, P, 9, 9, 9, stream);
}

template <typename T>
int virial_bwd(int B, int P, int U, const int* bnumneigh, const T* rcs, const T* dei, const T* grad_virial,
               T* grad_dei, T* grad_rcs, hipStream_t stream)
{
    int rc = check_shape(B, P, U, 0);
    if (rc) return rc;
    A2P_REQUIRE(bnumneigh && rcs && dei && grad_virial && (grad_dei || grad_rcs), A2P_ERR_INVALID,
                "fvt virial backward: null pointer");
    if (B == 0 || P == 0) return A2P_OK;
    prof_begin("fvt_virial_bwd", stream);
    hipLaunchKernelGGL(virial_bwd_kernel<T>, dim3(ceil_div((long long)B * P * 64, 256)), dim3(256), 0, stream,
                       grad_dei, grad_rcs, grad_virial, dei, rcs, B, P, U, bnumneigh);
    prof_end(stream);
    A2P_HIP_CHECK(hipGetLastError());
    return A2P_OK;
}

// ---- virial without any allocation ------------------------------------------------------------
// The row partial sums of virial_fwd live in a per-device workspace that is allocated on demand.
// Callers that must not allocate (HIP graph capture, serving loops, harnesses that forbid it) get
// the same two kernels on a buffer that is part of the library's image: each GPU the library runs
// on holds its own copy of `scratch` from the first use until the process ends.
constexpr int kNoAllocMaxRows = 65536;                           // batch * nlocal, 4.5 MiB of partial sums
static __device__ __align__(256) double scratch[(size_t)kNoAllocMaxRows * 9];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
double* g_scratch_ptr[kMaxDevices];                              // device address of `scratch`, per device

// Device address of `scratch` on the current device (its name is only a host-side stand-in).
int scratch_address(double** out)
{
    int dev = -1;
    A2P_HIP_CHECK(hipGetDevice(&dev));
    A2P_REQUIRE(dev >= 0 && dev < kMaxDevices, A2P_ERR_INVALID, "fvt virial (no allocation): device %d not supported", dev);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        A2P_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        A2P_REQUIRE(p != nullptr, A2P_ERR_HIP, "fvt virial (no allocation): scratch has no device address");
        g_scratch_ptr[dev] = (double*)p;
    }
    *out = g_scratch_ptr[dev];
    return A2P_OK;
}

int virial_fwd_noalloc(int B, int P, int U, const int* bnumneigh, const float* rcs, const float* dei, float* virial,
                       hipStream_t stream)
{
    int rc = check_shape(B, P, U, 0);
    if (rc) return rc;
    A2P_REQUIRE(bnumneigh && rcs && dei && virial, A2P_ERR_INVALID, "fvt virial: null pointer");
    A2P_REQUIRE((long long)B * P <= kNoAllocMaxRows, A2P_ERR_INVALID,
                "fvt virial (no allocation): batch * nlocal = %lld exceeds the %d rows of the built-in scratch; "
                "use a2p_fvt_virial_fwd_f32", (long long)B * P, kNoAllocMaxRows);
    if (B == 0) return A2P_OK;
    double* partial = nullptr;
    rc = scratch_address(&partial);
    if (rc) return rc;
    rc = enter_stream(stream);          // the scratch is shared by every stream of the device
    if (rc) return rc;
    // every row below batch * nlocal is written by the first kernel before the second reads it, so
    // what an earlier call left in the buffer never shows; nlocal == 0 leaves nothing to sum (zeros)
    if (P > 0) {
        hipLaunchKernelGGL(virial_rows_kernel<float>, dim3(ceil_div((long long)B * P * 64, 256)), dim3(256), 0, stream,
                           partial, dei, rcs, B, P, U, bnumneigh);
        A2P_HIP_CHECK(hipGetLastError());
    }
    return finish_partials<float>(virial, (const double*)partial, B, P, 9, 9, 9, stream, false);
}

}  // namespace
}  // namespace a2p

#define FVT_LIST const int* binum, const int* bilist, const int* bnumneigh, const int* bfirstneigh

extern "C" {
int a2p_fvt_force_fwd_f32(int B, int P, int U, int nghost, FVT_LIST, const float* dei, float* force, void* s)
{ return a2p::force_fwd<float>(B, P, U, nghost, binum, bilist, bnumneigh, bfirstneigh, dei, force, (hipStream_t)s); }
int a2p_fvt_force_fwd_f64(int B, int P, int U, int nghost, FVT_LIST, const double* dei, double* force, void* s)
{ return a2p::force_fwd<double>(B, P, U, nghost, binum, bilist, bnumneigh, bfirstneigh, dei, force, (hipStream_t)s); }
int a2p_fvt_force_bwd_f32(int B, int P, int U, int nghost, FVT_LIST, const float* gF, float* gdei, void* s)
{ return a2p::force_bwd<float>(B, P, U, nghost, binum, bilist, bnumneigh, bfirstneigh, gF, gdei, (hipStream_t)s); }
int a2p_fvt_force_bwd_f64(int B, int P, int U, int nghost, FVT_LIST, const double* gF, double* gdei, void* s)
{ return a2p::force_bwd<double>(B, P, U, nghost, binum, bilist, bnumneigh, bfirstneigh, gF, gdei, (hipStream_t)s); }
int a2p_fvt_virial_fwd_f32(int B, int P, int U, const int* bnumneigh, const float* rcs, const float* dei,
                           float* virial, void* s)
{ return a2p::virial_fwd<float>(B, P, U, bnumneigh, rcs, dei, virial, (hipStream_t)s); }
int a2p_fvt_virial_fwd_f64(int B, int P, int U, const int* bnumneigh, const double* rcs, const double* dei,
                           double* virial, void* s)
{ return a2p::virial_fwd<double>(B, P, U, bnumneigh, rcs, dei, virial, (hipStream_t)s); }
int a2p_fvt_virial_fwd_noalloc_f32(int B, int P, int U, const int* bnumneigh, const float* rcs, const float* dei,
                                   float* virial, void* s)
{ return a2p::virial_fwd_noalloc(B, P, U, bnumneigh, rcs, dei, virial, (hipStream_t)s); }
int a2p_fvt_virial_bwd_f32(int B, int P, int U, const int* bnumneigh, const float* rcs, const float* dei,
                           const float* gV, float* gdei, float* grcs, void* s)
{ return a2p::virial_bwd<float>(B, P, U, bnumneigh, rcs, dei, gV, gdei, grcs, (hipStream_t)s); }
int a2p_fvt_virial_bwd_f64(int B, int P, int U, const int* bnumneigh, const double* rcs, const double* dei,
                           const double* gV, double* gdei, double* grcs, void* s)
{ return a2p::virial_bwd<double>(B, P, U, bnumneigh, rcs, dei, gV, gdei, grcs, (hipStream_t)s); }
}
