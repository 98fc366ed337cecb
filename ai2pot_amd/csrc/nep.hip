// NEP energy / force / virial for gfx950: radial + three-body angular descriptors with
// Chebyshev radial functions, one tanh hidden layer per species, fused chain rule.
//
// One thread per centre atom, BLOCK atoms per workgroup.  Model tables (coefficients and
// network weights) are staged in LDS once per workgroup.  Per atom four sweeps over its
// neighbour row:
//   1. radial sweep   : q_n += g_n(r); neighbours inside the angular cutoff are marked in a
//                       per-thread bit mask kept in LDS, so that sweep 2 and 4 visit only
//                       those (an unsorted list would otherwise diverge on every neighbour)
//   2. angular sweep  : S_{n,lm} += g_n(r) b_lm(u)          (u = r_ij / r)
//      then q_{n,l} = sum_m w_m C_lm S^2, the hidden layer, dE/dq and dE/dS in registers
//   3. radial force   : g_ij = sum_n dE/dq_n g'_n(r) u      -> pair buffer
//   4. angular force  : g_ij += u sum_lm (A'_lm - l/r A_lm) b_lm + 1/r sum_lm A_lm grad b_lm
// with A_lm = sum_n dE/dS_{n,lm} g_n, A'_lm likewise with g'_n.  The radial functions are
// contracted with the coefficients once per neighbour (the reference re-multiplies them
// inside its innermost loop, include/nepBasis.h:153-167).  The per-pair derivatives go to a
// pair buffer that a2p::pair_reduce folds onto the neighbours without floating atomics;
// energy and virial leave each workgroup as fp64 partial sums.
//
// Formulas follow the reference's source/descriptor/nep/include/{basis.h:137-158,300-332,
// 519-530; nep_utilities.h:25-31,100-379; nepBasis.h:57-196; nep.h:320-529}.
#include "a2p_common.h"

namespace a2p {
namespace {

constexpr int NEP_BLOCK = 128;

// three-body weights, nep_utilities.h:25-31 (a double table whose odd entries carry an `f`
// suffix in the reference; kept so that fp64 results agree to the last digits)
__device__ constexpr double kC3B[24] = {
    0.238732414637843, 0.119366207318922f, 0.119366207318922f, 0.099471839432435f,
    0.596831036594608, 0.596831036594608f, 0.149207759148652f, 0.149207759148652f,
    0.139260575205408, 0.104445431404056f, 0.104445431404056f, 1.044454314040563f,
    1.044454314040563, 0.174075719006761f, 0.174075719006761f, 0.011190581936149f,
    0.223811638722978, 0.223811638722978f, 0.111905819361489f, 0.111905819361489f,
    1.566681471060845, 1.566681471060845f, 0.195835183882606f, 0.195835183882606f};

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

// KC, NRC, NAC, LC: compile-time capacities; the runtime sizes in `a` must not exceed them.
// EXACT: the runtime sizes equal the capacities and the network weights are in LDS (fast
// path: every loop bound and descriptor slot is a compile-time constant).
template <typename T, int KC, int NRC, int NAC, int LC, bool EXACT>
__global__ void __launch_bounds__(NEP_BLOCK)
nep_efv_kernel(const NepArgs<T> a)
{
    constexpr int NLM = LC * LC + 2 * LC;
    constexpr int DC = NRC + NAC * LC;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    const int tid = threadIdx.x;
    const int b = blockIdx.y;
    const int ii = blockIdx.x * NEP_BLOCK + tid;
    const int K = EXACT ? KC : a.K, n_r = EXACT ? NRC : a.n_r, n_a = EXACT ? NAC : a.n_a;
    const int l_max = EXACT ? LC : a.l_max, H = a.H, D = EXACT ? DC : a.D;
    const bool w_in_lds = EXACT ? true : (a.w_in_lds != 0);
    const int nbas = n_r + n_a;
    const int NF = a.P + a.nghost;
    const int nwords = (a.U + 31) >> 5;

    // ---- LDS layout: coeffs | [w0 b0 w1] | bias q_scaler | masks[nwords][BLOCK] ------------
    T* s_coef = (T*)smem_raw;
    const int ncoef = a.ntypes * a.ntypes * nbas * K;
    T* s_w0 = s_coef + ncoef;
    const int nw0 = w_in_lds ? a.ntypes * H * D : 0;
    T* s_b0 = s_w0 + nw0;
    const int nb0 = w_in_lds ? a.ntypes * H : 0;
    T* s_w1 = s_b0 + nb0;
    T* s_qs = s_w1 + nb0;
    unsigned* s_mask = (unsigned*)(s_qs + ((D + 3) & ~3));
    for (int i = tid; i < ncoef; i += NEP_BLOCK) s_coef[i] = a.coeffs[i];
    for (int i = tid; i < nw0; i += NEP_BLOCK) s_w0[i] = a.w0[i];
    for (int i = tid; i < nb0; i += NEP_BLOCK) { s_b0[i] = a.b0[i]; s_w1[i] = a.w1[i]; }
    for (int i = tid; i < D; i += NEP_BLOCK) s_qs[i] = a.q_scaler[i];
    __syncthreads();

    const int inum = a.binum[b];
    const bool active = ii < inum;
    const size_t row = (size_t)b * a.P + ii;
    int center = 0, ti = 0, nn = 0;
    if (active) {
        center = a.bilist[row];
        nn = a.bnumneigh[row];
        if (nn > a.U) { atomicOr(a.status, ST_NEIGH_OVERFLOW); nn = a.U; }
        if ((unsigned)center >= (unsigned)NF) { atomicOr(a.status, ST_BAD_NEIGHBOR); center = 0; nn = 0; }
        ti = a.btypes[(size_t)b * NF + center];
        if ((unsigned)ti >= (unsigned)a.ntypes) { atomicOr(a.status, ST_BAD_TYPE); ti = 0; nn = 0; }
    }
    const int* first = a.bfirstneigh + row * a.U;
    const T* rcs = a.brcs + row * a.U * 3;
    const int* types = a.btypes + (size_t)b * NF;
    const T rr = a.rr, ra = a.ra;
    const T rr_inv = (T)1 / rr, ra_inv = (T)1 / ra;

    T q[DC];
    T S[NAC][NLM];
#pragma unroll
    for (int k = 0; k < DC; k++) q[k] = (T)0;
#pragma unroll
    for (int n = 0; n < NAC; n++)
#pragma unroll
        for (int m = 0; m < NLM; m++) S[n][m] = (T)0;

    // ---- sweep 1: radial descriptors, mark angular neighbours ------------------------------
    int n_ang = 0;
    {
        unsigned cur = 0;
        for (int jj = 0; jj < nn; jj++) {
            const T x = rcs[jj * 3 + 0], y = rcs[jj * 3 + 1], z = rcs[jj * 3 + 2];
            const T r = sqrt_t(x * x + y * y + z * z);
            if (r <= rr) {
                int nj = first[jj];
                if ((unsigned)nj >= (unsigned)NF) { atomicOr(a.status, ST_BAD_NEIGHBOR); nj = center; }
                int tj = types[nj];
                if ((unsigned)tj >= (unsigned)a.ntypes) { atomicOr(a.status, ST_BAD_TYPE); tj = 0; }
                const T* c = s_coef + (ti * a.ntypes + tj) * nbas * K;
                T f[KC], df[KC];
                radial_basis<T, KC, false>(r, rr_inv, K, f, df);
#pragma unroll
                for (int n = 0; n < NRC; n++) {
                    if (n < n_r) {
                        T g = (T)0;
#pragma unroll
                        for (int k = 0; k < KC; k++)
                            if (k < K) g += c[n * K + k] * f[k];
                        q[n] += g;
                    }
                }
                if (l_max > 0 && r <= ra) { cur |= 1u << (jj & 31); n_ang++; }
            }
            if ((jj & 31) == 31 || jj == nn - 1) {
                s_mask[(jj >> 5) * NEP_BLOCK + tid] = cur;
                cur = 0;
            }
        }
    }

    // ---- sweep 2: angular moments -----------------------------------------------------------
    if (n_ang > 0) {
        const int nw_used = (nn + 31) >> 5;
        for (int w = 0; w < nw_used; w++) {
            unsigned bits = s_mask[w * NEP_BLOCK + tid];
            while (bits) {
                const int jj = (w << 5) + __ffs(bits) - 1;
                bits &= bits - 1;
                const T x = rcs[jj * 3 + 0], y = rcs[jj * 3 + 1], z = rcs[jj * 3 + 2];
                const T r = sqrt_t(x * x + y * y + z * z);
                const T rinv = (T)1 / r;
                int nj = first[jj];
                if ((unsigned)nj >= (unsigned)NF) nj = center;
                int tj = types[nj];
                if ((unsigned)tj >= (unsigned)a.ntypes) tj = 0;
                const T* c = s_coef + ((ti * a.ntypes + tj) * nbas + n_r) * K;
                T f[KC], df[KC];
                radial_basis<T, KC, false>(r, ra_inv, K, f, df);
                T bl[NLM];
                blm_values<T, LC>(x * rinv, y * rinv, z * rinv, bl);
#pragma unroll
                for (int n = 0; n < NAC; n++) {
                    if (n < n_a) {
                        T g = (T)0;
#pragma unroll
                        for (int k = 0; k < KC; k++)
                            if (k < K) g += c[n * K + k] * f[k];
#pragma unroll
                        for (int m = 0; m < NLM; m++) S[n][m] += g * bl[m];
                    }
                }
            }
        }
    }
    // q_{n,l} = sum_m w_m C_lm S^2  (nepBasis.h:174-190)
#pragma unroll
    for (int n = 0; n < NAC; n++)
#pragma unroll
        for (int l = 1; l <= LC; l++) {
            if (n < n_a && l <= l_max) {
                T acc = (T)0;
#pragma unroll
                for (int mp = 0; mp < 2 * l + 1; mp++) {
                    const int m = l * l - 1 + mp;
                    acc += (T)(mp == 0 ? 1.0 : 2.0) * (T)kC3B[m] * S[n][m] * S[n][m];
                }
                q[NRC + n * LC + (l - 1)] = acc;
            }
        }

    // Static slot j of q[] holds the descriptor whose index in the reference's runtime order
    // (n_r radial, then n*l_max + l-1) is kmap(j); -1 marks a slot the runtime sizes leave unused.
    auto kmap = [&](int j) -> int {
        if (EXACT) return j;
        if (j < NRC) return (j < n_r) ? j : -1;
        const int n = (j - NRC) / LC, l = (j - NRC) % LC;
        return (n < n_a && l < l_max) ? n_r + n * l_max + l : -1;
    };

    if (active && a.desc) {
        T* dst = a.desc + row * D;
#pragma unroll
        for (int j = 0; j < DC; j++) {
            const int k = kmap(j);
            if (k >= 0) dst[k] = q[j];
        }
    }

    // ---- hidden layer (nep.h:415-447) -------------------------------------------------------
    T dEdq[DC];
    T e_site = (T)0;
    {
        const T* W0 = w_in_lds ? s_w0 : a.w0;
        const T* B0 = w_in_lds ? s_b0 : a.b0;
        const T* W1 = w_in_lds ? s_w1 : a.w1;
        T qn[DC];
        T qsinv[DC];
#pragma unroll
        for (int j = 0; j < DC; j++) {
            const int k = kmap(j);
            const T qs = (k >= 0) ? s_qs[k] : (T)1;
            qsinv[j] = (T)1 / qs;
            qn[j] = (k >= 0) ? q[j] / qs : (T)0;
            dEdq[j] = (T)0;
        }
        e_site = active ? a.bias[ti] : (T)0;
        for (int p = 0; p < H; p++) {
            const T* wrow = W0 + ((size_t)ti * H + p) * D;
            T h = B0[ti * H + p];
            T wv[DC];
#pragma unroll
            for (int j = 0; j < DC; j++) {
                const int k = kmap(j);
                wv[j] = (k >= 0) ? wrow[k] : (T)0;
                h += wv[j] * qn[j];
            }
            const T t = tanh_t(h);
            const T w1p = W1[ti * H + p];
            e_site += w1p * t;
            const T sde = w1p * ((T)1 - t * t);
#pragma unroll
            for (int j = 0; j < DC; j++) dEdq[j] += sde * wv[j];
        }
#pragma unroll
        for (int j = 0; j < DC; j++) dEdq[j] *= qsinv[j];
    }
    // dE/dS (nep.h:450-466), overwriting S
#pragma unroll
    for (int n = 0; n < NAC; n++)
#pragma unroll
        for (int l = 1; l <= LC; l++)
#pragma unroll
            for (int mp = 0; mp < 2 * l + 1; mp++) {
                const int m = l * l - 1 + mp;
                S[n][m] *= dEdq[NRC + n * LC + (l - 1)] * (T)(mp == 0 ? 2.0 : 4.0) * (T)kC3B[m];
            }

    // ---- sweeps 3 and 4: pair derivatives ----------------------------------------------------
    T fx = (T)0, fy = (T)0, fz = (T)0;
    T vir[9];
#pragma unroll
    for (int i = 0; i < 9; i++) vir[i] = (T)0;
    if (a.force != nullptr) {
        T* grow = a.pair_g + row * a.U * 3;
        for (int jj = 0; jj < nn; jj++) {
            const T x = rcs[jj * 3 + 0], y = rcs[jj * 3 + 1], z = rcs[jj * 3 + 2];
            const T r = sqrt_t(x * x + y * y + z * z);
            T gx = (T)0, gy = (T)0, gz = (T)0;
            if (r <= rr) {
                int nj = first[jj];
                if ((unsigned)nj >= (unsigned)NF) nj = center;
                int tj = types[nj];
                if ((unsigned)tj >= (unsigned)a.ntypes) tj = 0;
                const T* c = s_coef + (ti * a.ntypes + tj) * nbas * K;
                T f[KC], df[KC];
                radial_basis<T, KC, true>(r, rr_inv, K, f, df);
                T s = (T)0;
#pragma unroll
                for (int n = 0; n < NRC; n++) {
                    if (n < n_r) {
                        T dg = (T)0;
#pragma unroll
                        for (int k = 0; k < KC; k++)
                            if (k < K) dg += c[n * K + k] * df[k];
                        s += dEdq[n] * dg;
                    }
                }
                s /= r;
                gx = s * x; gy = s * y; gz = s * z;
            }
            grow[jj * 3 + 0] = gx; grow[jj * 3 + 1] = gy; grow[jj * 3 + 2] = gz;
            fx += gx; fy += gy; fz += gz;
            vir[0] -= gx * x; vir[1] -= gx * y; vir[2] -= gx * z;
            vir[3] -= gy * x; vir[4] -= gy * y; vir[5] -= gy * z;
            vir[6] -= gz * x; vir[7] -= gz * y; vir[8] -= gz * z;
        }
        if (n_ang > 0) {
            const int nw_used = (nn + 31) >> 5;
            for (int w = 0; w < nw_used; w++) {
                unsigned bits = s_mask[w * NEP_BLOCK + tid];
                while (bits) {
                    const int jj = (w << 5) + __ffs(bits) - 1;
                    bits &= bits - 1;
                    const T x = rcs[jj * 3 + 0], y = rcs[jj * 3 + 1], z = rcs[jj * 3 + 2];
                    const T r = sqrt_t(x * x + y * y + z * z);
                    const T rinv = (T)1 / r;
                    const T ux = x * rinv, uy = y * rinv, uz = z * rinv;
                    int nj = first[jj];
                    if ((unsigned)nj >= (unsigned)NF) nj = center;
                    int tj = types[nj];
                    if ((unsigned)tj >= (unsigned)a.ntypes) tj = 0;
                    const T* c = s_coef + ((ti * a.ntypes + tj) * nbas + n_r) * K;
                    T f[KC], df[KC];
                    radial_basis<T, KC, true>(r, ra_inv, K, f, df);
                    T A[NLM], Ad[NLM];
#pragma unroll
                    for (int m = 0; m < NLM; m++) { A[m] = (T)0; Ad[m] = (T)0; }
#pragma unroll
                    for (int n = 0; n < NAC; n++) {
                        if (n < n_a) {
                            T g = (T)0, dg = (T)0;
#pragma unroll
                            for (int k = 0; k < KC; k++)
                                if (k < K) { g += c[n * K + k] * f[k]; dg += c[n * K + k] * df[k]; }
#pragma unroll
                            for (int m = 0; m < NLM; m++) { A[m] += S[n][m] * g; Ad[m] += S[n][m] * dg; }
                        }
                    }
                    T bl[NLM];
                    blm_values<T, LC>(ux, uy, uz, bl);
                    T srad = (T)0;
#pragma unroll
                    for (int l = 1; l <= LC; l++)
#pragma unroll
                        for (int mp = 0; mp < 2 * l + 1; mp++) {
                            const int m = l * l - 1 + mp;
                            if (l <= l_max) srad += (Ad[m] - (T)l * rinv * A[m]) * bl[m];
                            else A[m] = (T)0;
                        }
                    T wx = (T)0, wy = (T)0, wz = (T)0;
                    blm_grad_dot<T, LC>(ux, uy, uz, A, wx, wy, wz);
                    const T gx = srad * ux + wx * rinv;
                    const T gy = srad * uy + wy * rinv;
                    const T gz = srad * uz + wz * rinv;
                    grow[jj * 3 + 0] += gx; grow[jj * 3 + 1] += gy; grow[jj * 3 + 2] += gz;
                    fx += gx; fy += gy; fz += gz;
                    vir[0] -= gx * x; vir[1] -= gx * y; vir[2] -= gx * z;
                    vir[3] -= gy * x; vir[4] -= gy * y; vir[5] -= gy * z;
                    vir[6] -= gz * x; vir[7] -= gz * y; vir[8] -= gz * z;
                }
            }
        }
        if (active) {
            T* fo = a.force + ((size_t)b * NF + center) * 3;
            fo[0] = fx; fo[1] = fy; fo[2] = fz;
        }
    }

    // ---- workgroup partial sums of energy and virial (fp64) ---------------------------------
    __syncthreads();   // all threads are done with the LDS tables; reuse the front as scratch
    double* s_red = (double*)smem_raw;
    double vals[10];
    vals[0] = active ? (double)e_site : 0.0;
#pragma unroll
    for (int i = 0; i < 9; i++) vals[1 + i] = active ? (double)vir[i] : 0.0;
#pragma unroll
    for (int i = 0; i < 10; i++) {
        double v = wave_sum(vals[i]);
        if ((tid & 63) == 0) s_red[(tid >> 6) * 10 + i] = v;
    }
    __syncthreads();
    if (tid < 10) {
        double v = 0.0;
        for (int w = 0; w < NEP_BLOCK / 64; w++) v += s_red[w * 10 + tid];
        a.partial[((size_t)b * a.nblocks + blockIdx.x) * 10 + tid] = v;
    }
}

// ---- staged kernel for the common model shape (K=8, n_r=6, n_a=4, l_max=4, <= 4 species) ----
// The generic kernel above lets every thread walk its own neighbour row, so each wave-wide
// load touches 64 different cache lines.  Here the workgroup stages FCH slots of its FB rows
// through LDS per round with row-contiguous loads (FCH lanes per row), the neighbour's species
// is gathered by the loading lane and packed next to its index, and every thread then reads its
// own FCH entries from LDS without bank conflicts.  Two passes over the rounds:
//   pass 1: per-species sums of the radial functions (contracted with the coefficients once
//           per atom afterwards) and the angular moments of the neighbours inside the angular
//           cutoff; hidden layer, dE/dq, dE/dS
//   pass 2: pair derivatives (radial and angular part of a pair together), stored straight
//           into the target atom's reduction segment (a2p::PairCsr), own force, virial.
// Inside a round a thread first processes the entries within the angular cutoff, then the
// radial-only ones, each as a compacted bit-mask loop, so lanes of a wave work on the same kind
// of entry.
constexpr int FB = 256;        // atoms (threads) per workgroup
constexpr int FCH = 8;         // neighbour slots staged per round
constexpr int FLS = FB + 8;    // padded row length of the staging arrays
constexpr int FDP = 24;        // padded descriptor count (22)

__device__ __forceinline__ void lds_load4(const float* p, float (&o)[4])
{
    const float4 v = *reinterpret_cast<const float4*>(p);
    o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
}
__device__ __forceinline__ void lds_load4(const double* p, double (&o)[4])
{
    const double2 v0 = *reinterpret_cast<const double2*>(p);
    const double2 v1 = *reinterpret_cast<const double2*>(p + 2);
    o[0] = v0.x; o[1] = v0.y; o[2] = v1.x; o[3] = v1.y;
}

template <typename T>
struct StagedLds {
    T *w0, *coef, *b0, *w1, *qs, *acc, *x, *y, *z;
    int *w, *nn, *red;
};

__host__ __device__ __forceinline__ size_t lds_round16(size_t bytes) { return (bytes + 15) & ~(size_t)15; }

// LDS layout of the staged kernel; 16-byte aligned vector rows first.  Returns the total size.
template <typename T>
__host__ __device__ __forceinline__ size_t staged_lds_layout(int ntypes, int H, int ntc, unsigned char* base,
                                                             StagedLds<T>& L)
{
    size_t off = 0;
    L.w0 = (T*)(base + off);   off += lds_round16((size_t)ntypes * H * FDP * sizeof(T));
    L.coef = (T*)(base + off); off += lds_round16((size_t)ntypes * ntypes * 10 * 8 * sizeof(T));
    L.b0 = (T*)(base + off);   off += lds_round16((size_t)ntypes * H * sizeof(T));
    L.w1 = (T*)(base + off);   off += lds_round16((size_t)ntypes * H * sizeof(T));
    L.qs = (T*)(base + off);   off += lds_round16((size_t)FDP * sizeof(T));
    L.acc = (T*)(base + off);  off += lds_round16((size_t)ntc * 8 * FB * sizeof(T));
    L.x = (T*)(base + off);    off += lds_round16((size_t)FCH * FLS * sizeof(T));
    L.y = (T*)(base + off);    off += lds_round16((size_t)FCH * FLS * sizeof(T));
    L.z = (T*)(base + off);    off += lds_round16((size_t)FCH * FLS * sizeof(T));
    L.w = (int*)(base + off);  off += lds_round16((size_t)FCH * FLS * sizeof(int));
    L.nn = (int*)(base + off); off += lds_round16((size_t)FB * sizeof(int));
    L.red = (int*)(base + off); off += lds_round16((size_t)(FB / 64) * 10 * sizeof(double));
    return off;
}

// Stage slots [c0, c0 + FCH) of the workgroup's rows: thread e handles row e / FCH, slot e % FCH,
// so FCH consecutive lanes read one row's contiguous coordinates and indices.  Entries past a
// row's end (or with an index out of range) are stored far outside every cutoff.
template <typename T>
__device__ __forceinline__ void staged_load(const NepArgs<T>& a, const StagedLds<T>& L, int tid, int c0,
                                            size_t rowbase, const int* __restrict__ types, int NF)
{
#pragma unroll
    for (int it = 0; it < FCH; it++) {
        const int e = it * FB + tid;
        const int la = e / FCH, s = e % FCH;
        const int slot = c0 + s;
        T x = (T)1.0e18, y = (T)0, z = (T)0;
        int w = 0;
        if (slot < L.nn[la]) {
            const size_t pr = (rowbase + la) * a.U + slot;
            const T* p = a.brcs + pr * 3;
            const int nj = a.bfirstneigh[pr];
            if ((unsigned)nj >= (unsigned)NF) {
                atomicOr(a.status, ST_BAD_NEIGHBOR);
            } else {
                x = p[0]; y = p[1]; z = p[2];
                int tj = types[nj];
                if ((unsigned)tj >= (unsigned)a.ntypes) { atomicOr(a.status, ST_BAD_TYPE); tj = 0; }
                w = nj | (tj << 28);
            }
        }
        L.x[s * FLS + la] = x; L.y[s * FLS + la] = y; L.z[s * FLS + la] = z; L.w[s * FLS + la] = w;
    }
}

// Bit masks of a thread's staged entries: bits 0..FCH-1 inside the angular cutoff, bits
// 16..16+FCH-1 radial only.
template <typename T>
__device__ __forceinline__ unsigned staged_classify(const StagedLds<T>& L, int tid, T rr, T ra)
{
    unsigned m = 0;
#pragma unroll
    for (int s = 0; s < FCH; s++) {
        const T x = L.x[s * FLS + tid], y = L.y[s * FLS + tid], z = L.z[s * FLS + tid];
        const T r = sqrt_t(x * x + y * y + z * z);
        if (r <= ra) m |= 1u << s;
        else if (r <= rr) m |= 0x10000u << s;
    }
    return m;
}

template <typename T, int NTC>
__global__ void __launch_bounds__(FB, (sizeof(T) == 4 ? 2 : 1))
nep_staged_kernel(const NepArgs<T> a, const int* __restrict__ seg_offsets, int* __restrict__ seg_cursor,
                  T* __restrict__ seg_g)
{
    constexpr int KC = 8, NRC = 6, NAC = 4, LC = 4, NLM = 24, DC = 22, NB = NRC + NAC;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    const int tid = threadIdx.x;
    const int b = blockIdx.y;
    const int ii = blockIdx.x * FB + tid;
    const int H = a.H, nt = a.ntypes;
    const int NF = a.P + a.nghost;
    StagedLds<T> L;
    staged_lds_layout<T>(nt, H, NTC, smem_raw, L);

    // ---- model tables ------------------------------------------------------------------------
    for (int i = tid; i < nt * H * FDP; i += FB) {
        const int r = i / FDP, j = i - r * FDP;
        L.w0[i] = j < DC ? a.w0[(size_t)r * DC + j] : (T)0;
    }
    for (int i = tid; i < nt * nt * NB * KC; i += FB) L.coef[i] = a.coeffs[i];
    for (int i = tid; i < nt * H; i += FB) { L.b0[i] = a.b0[i]; L.w1[i] = a.w1[i]; }
    if (tid < FDP) L.qs[tid] = tid < DC ? (T)1 / a.q_scaler[tid] : (T)0;
#pragma unroll
    for (int i = 0; i < NTC * KC; i++) L.acc[i * FB + tid] = (T)0;

    const int inum = a.binum[b];
    const bool active = ii < inum;
    const size_t rowbase = (size_t)b * a.P + (size_t)blockIdx.x * FB;
    const size_t row = rowbase + tid;
    int center = 0, ti = 0, nn = 0;
    if (active) {
        center = a.bilist[row];
        nn = a.bnumneigh[row];
        if (nn > a.U) { atomicOr(a.status, ST_NEIGH_OVERFLOW); nn = a.U; }
        if ((unsigned)center >= (unsigned)NF) { atomicOr(a.status, ST_BAD_NEIGHBOR); center = 0; nn = 0; }
        ti = a.btypes[(size_t)b * NF + center];
        if ((unsigned)ti >= (unsigned)nt) { atomicOr(a.status, ST_BAD_TYPE); ti = 0; nn = 0; }
    }
    L.nn[tid] = nn;
    {
        int m = nn;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) m = max(m, __shfl_xor(m, off, 64));
        if ((tid & 63) == 0) L.red[tid >> 6] = m;
    }
    __syncthreads();
    int maxnn = 0;
#pragma unroll
    for (int w = 0; w < FB / 64; w++) maxnn = max(maxnn, L.red[w]);

    const int* types = a.btypes + (size_t)b * NF;
    const T rr = a.rr, ra = a.ra;
    const T rr_inv = (T)1 / rr, ra_inv = (T)1 / ra;

    T S[NAC][NLM];
#pragma unroll
    for (int n = 0; n < NAC; n++)
#pragma unroll
        for (int m = 0; m < NLM; m++) S[n][m] = (T)0;

    // ---- pass 1 -------------------------------------------------------------------------------
    for (int c0 = 0; c0 < maxnn; c0 += FCH) {
        __syncthreads();
        staged_load<T>(a, L, tid, c0, rowbase, types, NF);
        __syncthreads();
        const unsigned cls = staged_classify<T>(L, tid, rr, ra);
        unsigned am = cls & 0xffffu, rm = cls >> 16;
        while (am) {
            const int s = __ffs(am) - 1;
            am &= am - 1;
            const T x = L.x[s * FLS + tid], y = L.y[s * FLS + tid], z = L.z[s * FLS + tid];
            const int tj = L.w[s * FLS + tid] >> 28;
            const T r = sqrt_t(x * x + y * y + z * z);
            const T rinv = (T)1 / r;
            T f[KC], df[KC];
            if (r <= rr) {
                radial_basis<T, KC, false>(r, rr_inv, KC, f, df);
#pragma unroll
                for (int k = 0; k < KC; k++) L.acc[(tj * KC + k) * FB + tid] += f[k];
            }
            radial_basis<T, KC, false>(r, ra_inv, KC, f, df);
            const T* c = L.coef + ((ti * nt + tj) * NB + NRC) * KC;
            T bl[NLM];
            blm_values<T, LC>(x * rinv, y * rinv, z * rinv, bl);
#pragma unroll
            for (int n = 0; n < NAC; n++) {
                T c0v[4], c1v[4];
                lds_load4(c + n * KC, c0v);
                lds_load4(c + n * KC + 4, c1v);
                T g = (T)0;
#pragma unroll
                for (int k = 0; k < 4; k++) g += c0v[k] * f[k];
#pragma unroll
                for (int k = 0; k < 4; k++) g += c1v[k] * f[4 + k];
#pragma unroll
                for (int m = 0; m < NLM; m++) S[n][m] += g * bl[m];
            }
        }
        while (rm) {
            const int s = __ffs(rm) - 1;
            rm &= rm - 1;
            const T x = L.x[s * FLS + tid], y = L.y[s * FLS + tid], z = L.z[s * FLS + tid];
            const int tj = L.w[s * FLS + tid] >> 28;
            const T r = sqrt_t(x * x + y * y + z * z);
            T f[KC], df[KC];
            radial_basis<T, KC, false>(r, rr_inv, KC, f, df);
#pragma unroll
            for (int k = 0; k < KC; k++) L.acc[(tj * KC + k) * FB + tid] += f[k];
        }
    }

    // ---- descriptors --------------------------------------------------------------------------
    T q[DC];
#pragma unroll
    for (int j = 0; j < DC; j++) q[j] = (T)0;
    for (int t = 0; t < nt; t++) {
        const T* c = L.coef + (ti * nt + t) * NB * KC;
        T fs[KC];
#pragma unroll
        for (int k = 0; k < KC; k++) fs[k] = L.acc[(t * KC + k) * FB + tid];
#pragma unroll
        for (int n = 0; n < NRC; n++) {
            T c0v[4], c1v[4];
            lds_load4(c + n * KC, c0v);
            lds_load4(c + n * KC + 4, c1v);
#pragma unroll
            for (int k = 0; k < 4; k++) q[n] += c0v[k] * fs[k];
#pragma unroll
            for (int k = 0; k < 4; k++) q[n] += c1v[k] * fs[4 + k];
        }
    }
    // q_{n,l} = sum_m w_m C_lm S^2  (nepBasis.h:174-190)
#pragma unroll
    for (int n = 0; n < NAC; n++)
#pragma unroll
        for (int l = 1; l <= LC; l++) {
            T acc = (T)0;
#pragma unroll
            for (int mp = 0; mp < 2 * l + 1; mp++) {
                const int m = l * l - 1 + mp;
                acc += (T)(mp == 0 ? 1.0 : 2.0) * (T)kC3B[m] * S[n][m] * S[n][m];
            }
            q[NRC + n * LC + (l - 1)] = acc;
        }
    if (active && a.desc) {
        T* dst = a.desc + row * DC;
#pragma unroll
        for (int j = 0; j < DC; j++) dst[j] = q[j];
    }

    // ---- hidden layer (nep.h:415-447) ----------------------------------------------------------
    T dEdq[DC];
    T e_site = active ? a.bias[ti] : (T)0;
    {
        T qn[DC];
#pragma unroll
        for (int j = 0; j < DC; j++) { qn[j] = q[j] * L.qs[j]; dEdq[j] = (T)0; }
        for (int p = 0; p < H; p++) {
            const T* wrow = L.w0 + (size_t)(ti * H + p) * FDP;
            T wv[FDP];
#pragma unroll
            for (int j = 0; j < FDP; j += 4) {
                T v[4];
                lds_load4(wrow + j, v);
                wv[j] = v[0]; wv[j + 1] = v[1]; wv[j + 2] = v[2]; wv[j + 3] = v[3];
            }
            T h = L.b0[ti * H + p];
#pragma unroll
            for (int j = 0; j < DC; j++) h += wv[j] * qn[j];
            const T t = tanh_t(h);
            const T w1p = L.w1[ti * H + p];
            e_site += w1p * t;
            const T sde = w1p * ((T)1 - t * t);
#pragma unroll
            for (int j = 0; j < DC; j++) dEdq[j] += sde * wv[j];
        }
#pragma unroll
        for (int j = 0; j < DC; j++) dEdq[j] *= L.qs[j];
    }
    // dE/dS (nep.h:450-466), overwriting S
#pragma unroll
    for (int n = 0; n < NAC; n++)
#pragma unroll
        for (int l = 1; l <= LC; l++)
#pragma unroll
            for (int mp = 0; mp < 2 * l + 1; mp++) {
                const int m = l * l - 1 + mp;
                S[n][m] *= dEdq[NRC + n * LC + (l - 1)] * (T)(mp == 0 ? 2.0 : 4.0) * (T)kC3B[m];
            }

    // ---- pass 2: pair derivatives ---------------------------------------------------------------
    T fx = (T)0, fy = (T)0, fz = (T)0;
    T vir[9];
#pragma unroll
    for (int i = 0; i < 9; i++) vir[i] = (T)0;
    if (a.force != nullptr || a.want_virial) {
        // radial coefficients contracted with dE/dq, per neighbour species (thread-private cells)
        for (int t = 0; t < nt; t++) {
            const T* c = L.coef + (ti * nt + t) * NB * KC;
            T cc[KC];
#pragma unroll
            for (int k = 0; k < KC; k++) cc[k] = (T)0;
#pragma unroll
            for (int n = 0; n < NRC; n++) {
                T c0v[4], c1v[4];
                lds_load4(c + n * KC, c0v);
                lds_load4(c + n * KC + 4, c1v);
#pragma unroll
                for (int k = 0; k < 4; k++) { cc[k] += dEdq[n] * c0v[k]; cc[4 + k] += dEdq[n] * c1v[k]; }
            }
#pragma unroll
            for (int k = 0; k < KC; k++) L.acc[(t * KC + k) * FB + tid] = cc[k];
        }
        const size_t tbase = (size_t)b * NF;
        auto emit = [&](int w, T x, T y, T z, T gx, T gy, T gz) __attribute__((always_inline)) {
            if (seg_g) {
                const size_t t = tbase + (size_t)(w & 0x0fffffff);
                const int pos = seg_offsets[t] + atomicAdd(&seg_cursor[t], 1);
                T* dst = seg_g + (size_t)pos * 3;
                dst[0] = gx; dst[1] = gy; dst[2] = gz;
            }
            fx += gx; fy += gy; fz += gz;
            vir[0] -= gx * x; vir[1] -= gx * y; vir[2] -= gx * z;
            vir[3] -= gy * x; vir[4] -= gy * y; vir[5] -= gy * z;
            vir[6] -= gz * x; vir[7] -= gz * y; vir[8] -= gz * z;
        };
        for (int c0 = 0; c0 < maxnn; c0 += FCH) {
            __syncthreads();
            staged_load<T>(a, L, tid, c0, rowbase, types, NF);
            __syncthreads();
            const unsigned cls = staged_classify<T>(L, tid, rr, ra);
            unsigned am = cls & 0xffffu, rm = cls >> 16;
            while (am) {
                const int s = __ffs(am) - 1;
                am &= am - 1;
                const T x = L.x[s * FLS + tid], y = L.y[s * FLS + tid], z = L.z[s * FLS + tid];
                const int w = L.w[s * FLS + tid];
                const int tj = w >> 28;
                const T r = sqrt_t(x * x + y * y + z * z);
                const T rinv = (T)1 / r;
                const T ux = x * rinv, uy = y * rinv, uz = z * rinv;
                T f[KC], df[KC];
                T srad = (T)0;
                if (r <= rr) {
                    radial_basis<T, KC, true>(r, rr_inv, KC, f, df);
#pragma unroll
                    for (int k = 0; k < KC; k++) srad += L.acc[(tj * KC + k) * FB + tid] * df[k];
                }
                radial_basis<T, KC, true>(r, ra_inv, KC, f, df);
                const T* c = L.coef + ((ti * nt + tj) * NB + NRC) * KC;
                T A[NLM], Ad[NLM];
#pragma unroll
                for (int m = 0; m < NLM; m++) { A[m] = (T)0; Ad[m] = (T)0; }
#pragma unroll
                for (int n = 0; n < NAC; n++) {
                    T c0v[4], c1v[4];
                    lds_load4(c + n * KC, c0v);
                    lds_load4(c + n * KC + 4, c1v);
                    T g = (T)0, dg = (T)0;
#pragma unroll
                    for (int k = 0; k < 4; k++) { g += c0v[k] * f[k]; dg += c0v[k] * df[k]; }
#pragma unroll
                    for (int k = 0; k < 4; k++) { g += c1v[k] * f[4 + k]; dg += c1v[k] * df[4 + k]; }
#pragma unroll
                    for (int m = 0; m < NLM; m++) { A[m] += S[n][m] * g; Ad[m] += S[n][m] * dg; }
                }
                T bl[NLM];
                blm_values<T, LC>(ux, uy, uz, bl);
#pragma unroll
                for (int l = 1; l <= LC; l++)
#pragma unroll
                    for (int mp = 0; mp < 2 * l + 1; mp++) {
                        const int m = l * l - 1 + mp;
                        srad += (Ad[m] - (T)l * rinv * A[m]) * bl[m];
                    }
                T wx = (T)0, wy = (T)0, wz = (T)0;
                blm_grad_dot<T, LC>(ux, uy, uz, A, wx, wy, wz);
                emit(w, x, y, z, srad * ux + wx * rinv, srad * uy + wy * rinv, srad * uz + wz * rinv);
            }
            while (rm) {
                const int s = __ffs(rm) - 1;
                rm &= rm - 1;
                const T x = L.x[s * FLS + tid], y = L.y[s * FLS + tid], z = L.z[s * FLS + tid];
                const int w = L.w[s * FLS + tid];
                const int tj = w >> 28;
                const T r = sqrt_t(x * x + y * y + z * z);
                T f[KC], df[KC];
                radial_basis<T, KC, true>(r, rr_inv, KC, f, df);
                T sr = (T)0;
#pragma unroll
                for (int k = 0; k < KC; k++) sr += L.acc[(tj * KC + k) * FB + tid] * df[k];
                sr /= r;
                emit(w, x, y, z, sr * x, sr * y, sr * z);
            }
        }
        if (active && a.force) {
            T* fo = a.force + ((size_t)b * NF + center) * 3;
            fo[0] = fx; fo[1] = fy; fo[2] = fz;
        }
    }

    // ---- workgroup partial sums of energy and virial (fp64) ---------------------------------
    __syncthreads();
    double* s_red = (double*)L.red;
    double vals[10];
    vals[0] = active ? (double)e_site : 0.0;
#pragma unroll
    for (int i = 0; i < 9; i++) vals[1 + i] = active ? (double)vir[i] : 0.0;
#pragma unroll
    for (int i = 0; i < 10; i++) {
        double v = wave_sum(vals[i]);
        if ((tid & 63) == 0) s_red[(tid >> 6) * 10 + i] = v;
    }
    __syncthreads();
    if (tid < 10) {
        double v = 0.0;
        for (int w = 0; w < FB / 64; w++) v += s_red[w * 10 + tid];
        a.partial[((size_t)b * a.nblocks + blockIdx.x) * 10 + tid] = v;
    }
}

template <typename T, int NTC>
int launch_staged(const NepArgs<T>& a, size_t lds, const PairCsr& csr, hipStream_t stream)
{
    auto kern = nep_staged_kernel<T, NTC>;
    if (lds > 48 * 1024)
        A2P_HIP_CHECK(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                                          (int)lds));
    prof_begin("nep_staged_kernel", stream);
    hipLaunchKernelGGL(kern, dim3(a.nblocks, a.B), dim3(FB), lds, stream, a, (const int*)csr.offsets,
                       csr.cursor, (T*)csr.seg_g);
    prof_end(stream);
    A2P_HIP_CHECK(hipGetLastError());
    return A2P_OK;
}

template <typename T>
size_t nep_lds_bytes(const NepArgs<T>& a)
{
    size_t n = (size_t)a.ntypes * a.ntypes * (a.n_r + a.n_a) * a.K;
    if (a.w_in_lds) n += (size_t)a.ntypes * a.H * a.D + 2 * (size_t)a.ntypes * a.H;
    n += (a.D + 3) & ~3;
    size_t bytes = n * sizeof(T) + (size_t)((a.U + 31) >> 5) * NEP_BLOCK * sizeof(unsigned);
    return std::max(bytes, (size_t)(NEP_BLOCK / 64) * 10 * sizeof(double));
}

template <typename T, int KC, int NRC, int NAC, int LC, bool EXACT>
int launch(const NepArgs<T>& a, size_t lds, hipStream_t stream)
{
    auto kern = nep_efv_kernel<T, KC, NRC, NAC, LC, EXACT>;
    if (lds > 48 * 1024)
        A2P_HIP_CHECK(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                                          (int)lds));
    prof_begin("nep_efv_kernel", stream);
    hipLaunchKernelGGL(kern, dim3(a.nblocks, a.B), dim3(NEP_BLOCK), lds, stream, a);
    prof_end(stream);
    A2P_HIP_CHECK(hipGetLastError());
    return A2P_OK;
}

template <typename T>
int nep_efv(int K, int n_r, int n_a, int l_max, int H, int ntypes, const T* coeffs, const T* w0,
            const T* b0, const T* w1, const T* bias, const T* q_scaler, double rr, double ra, int B,
            int P, int U, int nghost, const int* binum, const int* bilist, const int* bnumneigh,
            const int* bfirstneigh, const T* brcs, const int* btypes, T* etot, T* force, T* virial,
            T* desc, hipStream_t stream)
{
    A2P_REQUIRE(K >= 1 && K <= 16, A2P_ERR_INVALID, "nep: chebyshev_size %d outside [1, 16]", K);
    A2P_REQUIRE(n_r >= 1 && n_r <= 12, A2P_ERR_INVALID, "nep: n_radial_basis %d outside [1, 12]", n_r);
    A2P_REQUIRE(l_max >= 0 && l_max <= 4, A2P_ERR_INVALID, "nep: l_max %d outside [0, 4]", l_max);
    A2P_REQUIRE(n_a >= 0 && n_a <= 8, A2P_ERR_INVALID, "nep: n_angular_basis %d outside [0, 8]", n_a);
    A2P_REQUIRE(H >= 1 && ntypes >= 1, A2P_ERR_INVALID, "nep: num_neurons and ntypes must be positive");
    A2P_REQUIRE(B >= 0 && P >= 0 && U >= 1 && nghost >= 0, A2P_ERR_INVALID, "nep: bad batch shape");
    A2P_REQUIRE(rr > 0 && ra > 0, A2P_ERR_INVALID, "nep: cutoffs must be positive");
    A2P_REQUIRE(coeffs && w0 && b0 && w1 && bias && q_scaler && binum && bilist && bnumneigh &&
                    bfirstneigh && brcs && btypes,
                A2P_ERR_INVALID, "nep: null input pointer");
    A2P_REQUIRE((long long)B * P * U < (1ll << 31), A2P_ERR_INVALID,
                "nep: batch*natoms_pad*umax exceeds 32-bit pair indexing");
    if (B == 0 || P == 0) return A2P_OK;

    NepArgs<T> a;
    a.K = K; a.n_r = n_r; a.n_a = n_a; a.l_max = l_max; a.H = H; a.ntypes = ntypes;
    a.D = (l_max == 0) ? n_r : n_r + n_a * l_max;     // nep_utilities.h:39-49
    a.coeffs = coeffs; a.w0 = w0; a.b0 = b0; a.w1 = w1; a.bias = bias; a.q_scaler = q_scaler;
    a.rr = (T)rr; a.ra = (T)ra;
    a.B = B; a.P = P; a.U = U; a.nghost = nghost; a.nblocks = ceil_div(P, NEP_BLOCK);
    a.binum = binum; a.bilist = bilist; a.bnumneigh = bnumneigh; a.bfirstneigh = bfirstneigh;
    a.brcs = brcs; a.btypes = btypes; a.desc = desc; a.want_virial = virial != nullptr;
    a.w_in_lds = 1;
    size_t lds = nep_lds_bytes(a);
    if (lds > 64 * 1024) {          // keep only the coefficient table in LDS
        a.w_in_lds = 0;
        lds = nep_lds_bytes(a);
    }
    A2P_REQUIRE(lds <= 150 * 1024, A2P_ERR_INVALID,
                "nep: coefficient table (%zu bytes with neighbour masks) does not fit in LDS", lds);

    // staged kernel: the common model shape with up to four species
    const long long NF = (long long)P + nghost;
    const int ntc = ntypes <= 1 ? 1 : ntypes == 2 ? 2 : ntypes == 3 ? 3 : 4;
    StagedLds<T> lds_unused;
    const size_t lds_staged = staged_lds_layout<T>(ntypes, H, ntc, nullptr, lds_unused);
    const bool staged = K == 8 && n_r == 6 && n_a == 4 && l_max == 4 && ntypes <= 4 &&
                        NF < (1ll << 28) && lds_staged <= 150 * 1024;
    if (staged) a.nblocks = ceil_div(P, FB);

    void* ws = nullptr;
    int rc = ws_get(WS_FLAGS, 64, &ws);
    if (rc) return rc;
    a.status = (int*)ws;
    rc = ws_get(WS_PARTIAL, (size_t)B * a.nblocks * 10 * sizeof(double), &ws);
    if (rc) return rc;
    a.partial = (double*)ws;
    a.pair_g = nullptr;
    a.force = force;
    const size_t force_bytes = (size_t)B * (P + nghost) * 3 * sizeof(T);

    if (staged) {
        PairCsr csr{};
        if (force) {
            rc = fill_zero(force, force_bytes, stream);
            if (rc) return rc;
            rc = pair_csr_begin<T>(&csr, B, P, U, nghost, binum, bnumneigh, bfirstneigh, stream);
            if (rc) return rc;
        }
        switch (ntc) {
        case 1: rc = launch_staged<T, 1>(a, lds_staged, csr, stream); break;
        case 2: rc = launch_staged<T, 2>(a, lds_staged, csr, stream); break;
        case 3: rc = launch_staged<T, 3>(a, lds_staged, csr, stream); break;
        default: rc = launch_staged<T, 4>(a, lds_staged, csr, stream); break;
        }
        if (rc) return rc;
        if (force) {
            rc = pair_csr_finish<T>(force, csr, stream);
            if (rc) return rc;
        }
    } else {
        if (!force && virial) {     // the virial needs the pair derivatives: use a scratch force
            rc = ws_get(WS_MISC, force_bytes, &ws);
            if (rc) return rc;
            a.force = (T*)ws;
        }
        if (a.force) {
            rc = ws_get(WS_PAIR_G, (size_t)B * P * U * 3 * sizeof(T), &ws);
            if (rc) return rc;
            a.pair_g = (T*)ws;
            rc = fill_zero(a.force, force_bytes, stream);
            if (rc) return rc;
        }
        if (K <= 8 && n_r <= 6 && n_a <= 4 && l_max <= 3)
            rc = launch<T, 8, 6, 4, 3, false>(a, lds, stream);
        else if (K <= 8 && n_r <= 6 && n_a <= 4)
            rc = launch<T, 8, 6, 4, 4, false>(a, lds, stream);
        else if (K <= 12 && n_r <= 8 && n_a <= 6)
            rc = launch<T, 12, 8, 6, 4, false>(a, lds, stream);
        else
            rc = launch<T, 16, 12, 8, 4, false>(a, lds, stream);
        if (rc) return rc;
        if (force) {
            rc = pair_reduce<T>(force, a.pair_g, B, P, U, nghost, binum, bnumneigh, bfirstneigh, stream);
            if (rc) return rc;
        }
    }
    if (etot) {
        rc = finish_partials<T>(etot, a.partial, B, a.nblocks, 1, 10, 1, stream);
        if (rc) return rc;
    }
    if (virial) {
        rc = finish_partials<T>(virial, a.partial + 1, B, a.nblocks, 9, 10, 9, stream);
        if (rc) return rc;
    }
    return A2P_OK;
}

}  // namespace
}  // namespace a2p

extern "C" {

int a2p_nep_efv_f32(int K, int n_r, int n_a, int l_max, int H, int ntypes, const float* coeffs,
                    const float* w0, const float* b0, const float* w1, const float* bias,
                    const float* q_scaler, double rr, double ra, int B, int P, int U, int nghost,
                    const int* binum, const int* bilist, const int* bnumneigh, const int* bfirstneigh,
                    const float* brcs, const int* btypes, float* etot, float* force, float* virial,
                    float* desc, void* stream)
{
    return a2p::nep_efv<float>(K, n_r, n_a, l_max, H, ntypes, coeffs, w0, b0, w1, bias, q_scaler, rr, ra,
                               B, P, U, nghost, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, etot,
                               force, virial, desc, (hipStream_t)stream);
}

int a2p_nep_efv_f64(int K, int n_r, int n_a, int l_max, int H, int ntypes, const double* coeffs,
                    const double* w0, const double* b0, const double* w1, const double* bias,
                    const double* q_scaler, double rr, double ra, int B, int P, int U, int nghost,
                    const int* binum, const int* bilist, const int* bnumneigh, const int* bfirstneigh,
                    const double* brcs, const int* btypes, double* etot, double* force, double* virial,
                    double* desc, void* stream)
{
    return a2p::nep_efv<double>(K, n_r, n_a, l_max, H, ntypes, coeffs, w0, b0, w1, bias, q_scaler, rr, ra,
                                B, P, U, nghost, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, etot,
                                force, virial, desc, (hipStream_t)stream);
}
}
