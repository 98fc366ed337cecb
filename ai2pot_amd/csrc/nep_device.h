// Device-side pieces shared by the NEP kernels: argument block, three-body weights, Chebyshev
// radial functions with cosine cutoff, and the 24 real solid harmonics b_lm with their gradients.
// Formulas follow the reference's source/descriptor/nep/include/{basis.h:137-158,300-332,
// 519-530; nep_utilities.h:25-31,100-379}.
#pragma once
#include "a2p_common.h"

namespace a2p {
namespace nepdev {

// three-body weights, nep_utilities.h:25-31 (a double table whose odd entries carry an `f`
// suffix in the reference; kept so that fp64 results agree to the last digits)
__device__ constexpr double kC3B[24] = {
    0.238732414637843, 0.119366207318922f, 0.119366207318922f, 0.099471839432435f,
    0.596831036594608, 0.596831036594608f, 0.149207759148652f, 0.149207759148652f,
    0.139260575205408, 0.104445431404056f, 0.104445431404056f, 1.044454314040563f,
    1.044454314040563, 0.174075719006761f, 0.174075719006761f, 0.011190581936149f,
    0.223811638722978, 0.223811638722978f, 0.111905819361489f, 0.111905819361489f,
    1.566681471060845, 1.566681471060845f, 0.195835183882606f, 0.195835183882606f};

// weights of the four- and five-body invariants of the extension (source/descriptor/ace/include/nep_descriptor.h:43-54;
// the reference never evaluates them)
__device__ constexpr double kC4B[5] = {-0.007499480826664, -0.134990654879954, 0.067495327439977, 0.404971964639861,
                                       -0.809943929279723};
__device__ constexpr double kC5B[3] = {0.026596810706114, 0.053193621412227, 0.026596810706114};

template <typename T>
struct NepArgs {
    int K, n_r, n_a, l_max, H, ntypes, D;
    const T *coeffs, *w0, *b0, *w1, *bias, *q_scaler;
    T rr, ra;
    int B, P, U, nghost, nblocks;
    const int *binum, *bilist, *bnumneigh, *bfirstneigh;
    const T* brcs;
    const int* btypes;
    T* force;        // [B, P+nghost, 3] or null
    T* pair_g;       // [B*P, U, 3] or null (needed when force != null)
    T* desc;         // [B, P, D] or null
    double* partial; // [B, nblocks, 10]
    int* status;
    int want_virial;
    int w_in_lds;    // network weights staged in LDS (else read from global memory)
    // optional: places of the pairs in their targets' reduction segments, kept by the caller from
    // call to call while the list stays the same: brank[B, P, U], and bincoming[B, P+nghost] pairs
    // naming each atom.  ranks_valid = 0: this call claims the places and records them there;
    // 1: it uses what an earlier call recorded.
    int* brank;
    int* bincoming;
    int ranks_valid;
    int mb4 = 0, mb5 = 0;   // extension (generic kernel only): four- / five-body invariant per angular channel
};

__device__ __forceinline__ void sincospi_t(float x, float* s, float* c) { sincospif(x, s, c); }
__device__ __forceinline__ void sincospi_t(double x, double* s, double* c) { sincospi(x, s, c); }
__device__ __forceinline__ float tanh_t(float x) { return tanhf(x); }
__device__ __forceinline__ double tanh_t(double x) { return tanh(x); }
__device__ __forceinline__ float sqrt_t(float x) { return sqrtf(x); }
__device__ __forceinline__ double sqrt_t(double x) { return sqrt(x); }

// f_k(r) = 1/2 (T_k(x)+1) fc(r), x = 2 (r/rc - 1)^2 - 1, fc = 1/2 (1 + cos(pi r/rc));
// basis.h:137-158, 300-332, 519-530.  Caller guarantees r <= rc.
template <typename T, int KC, bool DER>
__device__ __forceinline__ void radial_basis(T r, T rc_inv, int K, T (&f)[KC], T (&df)[KC])
{
    const T t = r * rc_inv;
    const T xr = t - (T)1;
    const T x = (T)2 * xr * xr - (T)1;
    const T dxdr = (T)4 * rc_inv * xr;
    T sn, cs;
    sincospi_t(t, &sn, &cs);
    const T fc = (T)0.5 * ((T)1 + cs);
    const T dfc = (T)(-0.5 * 3.14159265358979323846) * sn * rc_inv;
    T t0 = (T)1, t1 = x, d0 = (T)0, d1 = (T)1;
#pragma unroll
    for (int k = 0; k < KC; k++) {
        T tv, dv;
        if (k == 0) { tv = t0; dv = d0; }
        else if (k == 1) { tv = t1; dv = d1; }
        else {
            tv = (T)2 * x * t1 - t0;
            dv = (T)2 * t1 + (T)2 * x * d1 - d0;
            t0 = t1; t1 = tv; d0 = d1; d1 = dv;
        }
        const T v = (T)0.5 * (tv + (T)1);
        f[k] = (k < K) ? fc * v : (T)0;
        if (DER) df[k] = (k < K) ? dfc * v + fc * (T)0.5 * dv * dxdr : (T)0;
    }
}

// b_lm(u) for unit vector u, flat index l*l-1+mp (nep_utilities.h:110-203 with r = 1)
template <typename T, int LC>
__device__ __forceinline__ void blm_values(T x, T y, T z, T (&b)[LC * LC + 2 * LC])
{
    const T x2 = x * x, y2 = y * y, z2 = z * z;
    if (LC >= 1) { b[0] = z; b[1] = x; b[2] = y; }
    if (LC >= 2) {
        b[3] = (T)3 * z2 - (T)1; b[4] = x * z; b[5] = y * z; b[6] = x2 - y2; b[7] = (T)2 * x * y;
    }
    if (LC >= 3) {
        b[8] = ((T)5 * z2 - (T)3) * z;
        b[9] = ((T)5 * z2 - (T)1) * x;
        b[10] = ((T)5 * z2 - (T)1) * y;
        b[11] = (x2 - y2) * z;
        b[12] = (T)2 * x * y * z;
        b[13] = (x2 - (T)3 * y2) * x;
        b[14] = ((T)3 * x2 - y2) * y;
    }
    if (LC >= 4) {
        b[15] = ((T)35 * z2 - (T)30) * z2 + (T)3;
        b[16] = ((T)7 * z2 - (T)3) * x * z;
        b[17] = ((T)7 * z2 - (T)3) * y * z;
        b[18] = ((T)7 * z2 - (T)1) * (x2 - y2);
        b[19] = ((T)7 * z2 - (T)1) * (T)2 * x * y;
        b[20] = (x2 - (T)3 * y2) * x * z;
        b[21] = ((T)3 * x2 - y2) * y * z;
        b[22] = (x2 - y2) * (x2 - y2) - (T)4 * x2 * y2;
        b[23] = (T)4 * (x2 - y2) * x * y;
    }
}

// w += sum_lm a[lm] * grad b_lm(u): Cartesian gradients of the homogeneous polynomials
// b_lm, evaluated on the unit sphere (nep_utilities.h:206-379 with r = 1)
template <typename T, int LC>
__device__ __forceinline__ void blm_grad_dot(T x, T y, T z, const T (&a)[LC * LC + 2 * LC], T& wx,
                                             T& wy, T& wz)
{
    const T x2 = x * x, y2 = y * y, z2 = z * z;
    const T xy = x * y, xz = x * z, yz = y * z;
    if (LC >= 1) { wz += a[0]; wx += a[1]; wy += a[2]; }
    if (LC >= 2) {
        wx += a[3] * ((T)-2 * x) + a[4] * z + a[6] * ((T)2 * x) + a[7] * ((T)2 * y);
        wy += a[3] * ((T)-2 * y) + a[5] * z - a[6] * ((T)2 * y) + a[7] * ((T)2 * x);
        wz += a[3] * ((T)4 * z) + a[4] * x + a[5] * y;
    }
    if (LC >= 3) {
        const T c = (T)5 * z2 - (T)1;
        wx += a[8] * ((T)-6 * xz) + a[9] * (c - (T)2 * x2) + a[10] * ((T)-2 * xy) +
              a[11] * ((T)2 * xz) + a[12] * ((T)2 * yz) + a[13] * ((T)3 * (x2 - y2)) +
              a[14] * ((T)6 * xy);
        wy += a[8] * ((T)-6 * yz) + a[9] * ((T)-2 * xy) + a[10] * (c - (T)2 * y2) +
              a[11] * ((T)-2 * yz) + a[12] * ((T)2 * xz) + a[13] * ((T)-6 * xy) +
              a[14] * ((T)3 * (x2 - y2));
        wz += a[8] * ((T)9 * z2 - (T)3) + a[9] * ((T)8 * xz) + a[10] * ((T)8 * yz) +
              a[11] * (x2 - y2) + a[12] * ((T)2 * xy);
    }
    if (LC >= 4) {
        const T z3 = z2 * z, x3 = x2 * x, y3 = y2 * y;
        const T c73 = (T)7 * z3 - (T)3 * z;
        wx += a[15] * ((T)-60 * x * z2 + (T)12 * x) + a[16] * ((T)-6 * x2 * z + c73) +
              a[17] * ((T)-6 * xy * z) +
              a[18] * ((T)-2 * x3 + (T)2 * x * y2 + (T)14 * x * z2 - (T)2 * x) +
              a[19] * ((T)-4 * x2 * y + (T)14 * y * z2 - (T)2 * y) + a[20] * ((T)3 * (x2 - y2) * z) +
              a[21] * ((T)6 * xy * z) + a[22] * ((T)4 * x3 - (T)12 * x * y2) +
              a[23] * ((T)12 * x2 * y - (T)4 * y3);
        wy += a[15] * ((T)-60 * y * z2 + (T)12 * y) + a[16] * ((T)-6 * xy * z) +
              a[17] * ((T)-6 * y2 * z + c73) +
              a[18] * ((T)-2 * x2 * y + (T)2 * y3 - (T)14 * y * z2 + (T)2 * y) +
              a[19] * ((T)-4 * x * y2 + (T)14 * x * z2 - (T)2 * x) + a[20] * ((T)-6 * xy * z) +
              a[21] * ((T)3 * (x2 - y2) * z) + a[22] * ((T)4 * y3 - (T)12 * x2 * y) +
              a[23] * ((T)4 * x3 - (T)12 * x * y2);
        wz += a[15] * ((T)80 * z3 - (T)48 * z) + a[16] * ((T)15 * x * z2 - (T)3 * x) +
              a[17] * ((T)15 * y * z2 - (T)3 * y) + a[18] * ((T)12 * z * (x2 - y2)) +
              a[19] * ((T)24 * xy * z) + a[20] * ((x2 - (T)3 * y2) * x) +
              a[21] * (((T)3 * x2 - y2) * y);
    }
}

// d[lm] = w . grad b_lm(u): the directional derivative of every homogeneous polynomial b_lm along
// w, evaluated on the unit sphere (the same gradients as blm_grad_dot, taken apart per lm)
template <typename T, int LC>
__device__ __forceinline__ void blm_dir_derivs(T x, T y, T z, T wx, T wy, T wz, T (&d)[LC * LC + 2 * LC])
{
    const T x2 = x * x, y2 = y * y, z2 = z * z;
    const T xy = x * y, xz = x * z, yz = y * z;
    if (LC >= 1) { d[0] = wz; d[1] = wx; d[2] = wy; }
    if (LC >= 2) {
        d[3] = (T)-2 * x * wx + (T)-2 * y * wy + (T)4 * z * wz;
        d[4] = z * wx + x * wz;
        d[5] = z * wy + y * wz;
        d[6] = (T)2 * x * wx - (T)2 * y * wy;
        d[7] = (T)2 * y * wx + (T)2 * x * wy;
    }
    if (LC >= 3) {
        const T c = (T)5 * z2 - (T)1;
        d[8] = (T)-6 * xz * wx + (T)-6 * yz * wy + ((T)9 * z2 - (T)3) * wz;
        d[9] = (c - (T)2 * x2) * wx + (T)-2 * xy * wy + (T)8 * xz * wz;
        d[10] = (T)-2 * xy * wx + (c - (T)2 * y2) * wy + (T)8 * yz * wz;
        d[11] = (T)2 * xz * wx + (T)-2 * yz * wy + (x2 - y2) * wz;
        d[12] = (T)2 * yz * wx + (T)2 * xz * wy + (T)2 * xy * wz;
        d[13] = (T)3 * (x2 - y2) * wx + (T)-6 * xy * wy;
        d[14] = (T)6 * xy * wx + (T)3 * (x2 - y2) * wy;
    }
    if (LC >= 4) {
        const T z3 = z2 * z, x3 = x2 * x, y3 = y2 * y;
        const T c73 = (T)7 * z3 - (T)3 * z;
        d[15] = ((T)-60 * x * z2 + (T)12 * x) * wx + ((T)-60 * y * z2 + (T)12 * y) * wy +
                ((T)80 * z3 - (T)48 * z) * wz;
        d[16] = ((T)-6 * x2 * z + c73) * wx + ((T)-6 * xy * z) * wy + ((T)15 * x * z2 - (T)3 * x) * wz;
        d[17] = ((T)-6 * xy * z) * wx + ((T)-6 * y2 * z + c73) * wy + ((T)15 * y * z2 - (T)3 * y) * wz;
        d[18] = ((T)-2 * x3 + (T)2 * x * y2 + (T)14 * x * z2 - (T)2 * x) * wx +
                ((T)-2 * x2 * y + (T)2 * y3 - (T)14 * y * z2 + (T)2 * y) * wy + ((T)12 * z * (x2 - y2)) * wz;
        d[19] = ((T)-4 * x2 * y + (T)14 * y * z2 - (T)2 * y) * wx +
                ((T)-4 * x * y2 + (T)14 * x * z2 - (T)2 * x) * wy + ((T)24 * xy * z) * wz;
        d[20] = ((T)3 * (x2 - y2) * z) * wx + ((T)-6 * xy * z) * wy + ((x2 - (T)3 * y2) * x) * wz;
        d[21] = ((T)6 * xy * z) * wx + ((T)3 * (x2 - y2) * z) * wy + (((T)3 * x2 - y2) * y) * wz;
        d[22] = ((T)4 * x3 - (T)12 * x * y2) * wx + ((T)4 * y3 - (T)12 * x2 * y) * wy;
        d[23] = ((T)12 * x2 * y - (T)4 * y3) * wx + ((T)4 * x3 - (T)12 * x * y2) * wy;
    }
}

}  // namespace nepdev

// The staged kernel for the common model shape (nep_staged.hip).  staged_supported() tells
// whether it applies; nep_staged_run() performs forces' zero-fill, pair counting, the kernel and
// the pair reduction, whose launch also sums the workgroup partial sums of a.partial (a.nblocks
// is set by staged_nblocks()) into etot and virial.
// The same model shape with 8 lanes per atom (nep_group.hip): an atom's latency is an eighth of
// the staged kernel's and a workgroup holds 32 atoms, which is what a small system needs to
// occupy the device; per atom it executes more instructions, so large systems stay with the
// staged kernel.
template <typename T>
bool nep_group_supported(const nepdev::NepArgs<T>& a, size_t* lds_bytes);
int nep_group_nblocks(int P);
template <typename T>
int nep_group_run(const nepdev::NepArgs<T>& a, size_t lds_bytes, T* etot, T* virial, hipStream_t stream);

template <typename T>
bool nep_staged_supported(const nepdev::NepArgs<T>& a, size_t* lds_bytes);
int nep_staged_nblocks(int P);
template <typename T>
int nep_staged_run(const nepdev::NepArgs<T>& a, size_t lds_bytes, T* etot, T* virial, hipStream_t stream);

}  // namespace a2p
