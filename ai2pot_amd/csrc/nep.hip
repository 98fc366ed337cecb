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
#include "nep_device.h"

namespace a2p {
using namespace nepdev;
namespace {

constexpr int NEP_BLOCK = 128;

// KC, NRC, NAC, LC: compile-time capacities; the runtime sizes in `a` must not exceed them.
// EXACT: the runtime sizes equal the capacities and the network weights are in LDS (fast
// path: every loop bound and descriptor slot is a compile-time constant).
// MB: the extension with one four-body (from the l = 2 moments) and / or one five-body (l = 1) invariant per angular
// channel (a.mb4, a.mb5; weights of source/descriptor/ace/include/nep_descriptor.h:43-54, whose routines for them
// are declared and never defined: there is no reference result for these descriptors).  Descriptor order per
// channel: l = 1 .. l_max, then the four-body, then the five-body entry.
template <typename T, int KC, int NRC, int NAC, int LC, bool EXACT, bool MB = false>
__global__ void __launch_bounds__(NEP_BLOCK)
nep_efv_kernel(const NepArgs<T> a)
{
    static_assert(!(MB && EXACT), "the many-body extension runs with runtime sizes");
    constexpr int NLM = LC * LC + 2 * LC;
    constexpr int LCX = LC + (MB ? 2 : 0);       // descriptor slots per angular channel
    constexpr int DC = NRC + NAC * LCX;
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
                q[NRC + n * LCX + (l - 1)] = acc;
            }
        }
    if (MB) {
        // q_4b from s[3..7] (l = 2), q_5b from s[0..2] (l = 1)
#pragma unroll
        for (int n = 0; n < NAC; n++) {
            if (n < n_a) {
                const T* s = S[n];
                if (LC >= 2 && a.mb4)
                    q[NRC + n * LCX + LC] = (T)kC4B[0] * s[3] * s[3] * s[3] + (T)kC4B[1] * s[3] * (s[4] * s[4] + s[5] * s[5]) +
                                            (T)kC4B[2] * s[3] * (s[6] * s[6] + s[7] * s[7]) +
                                            (T)kC4B[3] * s[6] * (s[5] * s[5] - s[4] * s[4]) + (T)kC4B[4] * s[4] * s[5] * s[7];
                if (a.mb5) {
                    const T p0 = s[0] * s[0], p1 = s[1] * s[1] + s[2] * s[2];
                    q[NRC + n * LCX + LC + 1] = (T)kC5B[0] * p0 * p0 + (T)kC5B[1] * p0 * p1 + (T)kC5B[2] * p1 * p1;
                }
            }
        }
    }

    // Static slot j of q[] holds the descriptor whose index in the reference's runtime order
    // (n_r radial, then n*l_max + l-1) is kmap(j); -1 marks a slot the runtime sizes leave unused.
    auto kmap = [&](int j) -> int {
        if (EXACT) return j;
        if (j < NRC) return (j < n_r) ? j : -1;
        const int n = (j - NRC) / LCX, l = (j - NRC) % LCX;
        if (!MB) return (n < n_a && l < l_max) ? n_r + n * l_max + l : -1;
        const int num_l = l_max + a.mb4 + a.mb5;
        if (n >= n_a) return -1;
        if (l < LC) return l < l_max ? n_r + n * num_l + l : -1;
        if (l == LC) return a.mb4 ? n_r + n * num_l + l_max : -1;
        return a.mb5 ? n_r + n * num_l + l_max + a.mb4 : -1;
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
    for (int n = 0; n < NAC; n++) {
        T extra[8];
#pragma unroll
        for (int k = 0; k < 8; k++) extra[k] = (T)0;
        if (MB && n < n_a) {
            const T* s = S[n];
            if (LC >= 2 && a.mb4) {
                const T w = dEdq[NRC + n * LCX + LC];
                extra[3] = w * ((T)3 * (T)kC4B[0] * s[3] * s[3] + (T)kC4B[1] * (s[4] * s[4] + s[5] * s[5]) +
                                (T)kC4B[2] * (s[6] * s[6] + s[7] * s[7]));
                extra[4] = w * ((T)2 * (T)kC4B[1] * s[3] * s[4] - (T)2 * (T)kC4B[3] * s[6] * s[4] + (T)kC4B[4] * s[5] * s[7]);
                extra[5] = w * ((T)2 * (T)kC4B[1] * s[3] * s[5] + (T)2 * (T)kC4B[3] * s[6] * s[5] + (T)kC4B[4] * s[4] * s[7]);
                extra[6] = w * ((T)2 * (T)kC4B[2] * s[3] * s[6] + (T)kC4B[3] * (s[5] * s[5] - s[4] * s[4]));
                extra[7] = w * ((T)2 * (T)kC4B[2] * s[3] * s[7] + (T)kC4B[4] * s[4] * s[5]);
            }
            if (a.mb5) {
                const T w = dEdq[NRC + n * LCX + LC + 1];
                const T p0 = s[0] * s[0], p1 = s[1] * s[1] + s[2] * s[2];
                extra[0] = w * ((T)4 * (T)kC5B[0] * p0 * s[0] + (T)2 * (T)kC5B[1] * s[0] * p1);
                extra[1] = w * ((T)2 * (T)kC5B[1] * p0 * s[1] + (T)4 * (T)kC5B[2] * p1 * s[1]);
                extra[2] = w * ((T)2 * (T)kC5B[1] * p0 * s[2] + (T)4 * (T)kC5B[2] * p1 * s[2]);
            }
        }
#pragma unroll
        for (int l = 1; l <= LC; l++)
#pragma unroll
            for (int mp = 0; mp < 2 * l + 1; mp++) {
                const int m = l * l - 1 + mp;
                S[n][m] *= dEdq[NRC + n * LCX + (l - 1)] * (T)(mp == 0 ? 2.0 : 4.0) * (T)kC3B[m];
                if (MB && m < 8) S[n][m] += extra[m];
            }
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

template <typename T>
size_t nep_lds_bytes(const NepArgs<T>& a)
{
    size_t n = (size_t)a.ntypes * a.ntypes * (a.n_r + a.n_a) * a.K;
    if (a.w_in_lds) n += (size_t)a.ntypes * a.H * a.D + 2 * (size_t)a.ntypes * a.H;
    n += (a.D + 3) & ~3;
    size_t bytes = n * sizeof(T) + (size_t)((a.U + 31) >> 5) * NEP_BLOCK * sizeof(unsigned);
    return std::max(bytes, (size_t)(NEP_BLOCK / 64) * 10 * sizeof(double));
}

template <typename T, int KC, int NRC, int NAC, int LC, bool EXACT, bool MB = false>
int launch(const NepArgs<T>& a, size_t lds, hipStream_t stream)
{
    auto kern = nep_efv_kernel<T, KC, NRC, NAC, LC, EXACT, MB>;
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
            T* desc, hipStream_t stream, int* brank = nullptr, int* bincoming = nullptr, int ranks_valid = 0,
            int mb4 = 0, int mb5 = 0)
{
    A2P_REQUIRE((mb4 == 0 || l_max >= 2) && (mb5 == 0 || l_max >= 1) && (mb4 | mb5 | 1) == 1, A2P_ERR_INVALID,
                "nep: the four-body term needs l_max >= 2, the five-body term l_max >= 1");
    A2P_REQUIRE((brank == nullptr) == (bincoming == nullptr), A2P_ERR_INVALID,
                "nep: pair ranks and incoming counts come together");
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
    a.mb4 = mb4; a.mb5 = mb5;
    a.D = (l_max == 0) ? n_r : n_r + n_a * (l_max + mb4 + mb5);     // nep_utilities.h:39-49
    a.coeffs = coeffs; a.w0 = w0; a.b0 = b0; a.w1 = w1; a.bias = bias; a.q_scaler = q_scaler;
    a.rr = (T)rr; a.ra = (T)ra;
    a.B = B; a.P = P; a.U = U; a.nghost = nghost; a.nblocks = ceil_div(P, NEP_BLOCK);
    a.binum = binum; a.bilist = bilist; a.bnumneigh = bnumneigh; a.bfirstneigh = bfirstneigh;
    a.brcs = brcs; a.btypes = btypes; a.desc = desc; a.want_virial = virial != nullptr;
    a.brank = brank; a.bincoming = bincoming; a.ranks_valid = ranks_valid;
    a.w_in_lds = 1;
    size_t lds = nep_lds_bytes(a);
    if (lds > 64 * 1024) {          // keep only the coefficient table in LDS
        a.w_in_lds = 0;
        lds = nep_lds_bytes(a);
    }
    A2P_REQUIRE(lds <= 150 * 1024, A2P_ERR_INVALID,
                "nep: coefficient table (%zu bytes with neighbour masks) does not fit in LDS", lds);

    // staged kernel: the common model shape with up to four species
    a.force = force;
    a.pair_g = nullptr;
    size_t lds_staged = 0;
    const bool staged = !(mb4 || mb5) && nep_staged_supported<T>(a, &lds_staged);
    if (staged) a.nblocks = nep_staged_nblocks(P);
    size_t lds_group = 0;
    // fewer staged workgroups than half the compute units: the system is small, spread it wider
    const bool group = staged && (long long)B * nep_staged_nblocks(P) < 128 && nep_group_supported<T>(a, &lds_group);
    if (group) a.nblocks = nep_group_nblocks(P);

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

    if (group) {
        return nep_group_run<T>(a, lds_group, etot, virial, stream);     // includes the energy / virial sums
    } else if (staged) {
        return nep_staged_run<T>(a, lds_staged, etot, virial, stream);
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
        if (mb4 || mb5)
            rc = (K <= 8 && n_r <= 6 && n_a <= 4) ? launch<T, 8, 6, 4, 4, false, true>(a, lds, stream)
                                                  : launch<T, 16, 12, 8, 4, false, true>(a, lds, stream);
        else if (K <= 8 && n_r <= 6 && n_a <= 4 && l_max <= 3)
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
    return finish_energy_virial<T>(etot, virial, a.partial, B, a.nblocks, stream);
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

int a2p_nep_efv_ranked_f32(int K, int n_r, int n_a, int l_max, int H, int ntypes, const float* coeffs,
                           const float* w0, const float* b0, const float* w1, const float* bias,
                           const float* q_scaler, double rr, double ra, int B, int P, int U, int nghost,
                           const int* binum, const int* bilist, const int* bnumneigh, const int* bfirstneigh,
                           const float* brcs, const int* btypes, int* brank, int* bincoming,
                           int ranks_valid, float* etot, float* force, float* virial, float* desc, void* stream)
{
    return a2p::nep_efv<float>(K, n_r, n_a, l_max, H, ntypes, coeffs, w0, b0, w1, bias, q_scaler, rr, ra,
                               B, P, U, nghost, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, etot,
                               force, virial, desc, (hipStream_t)stream, brank, bincoming, ranks_valid);
}

int a2p_nep_efv_ranked_f64(int K, int n_r, int n_a, int l_max, int H, int ntypes, const double* coeffs,
                           const double* w0, const double* b0, const double* w1, const double* bias,
                           const double* q_scaler, double rr, double ra, int B, int P, int U, int nghost,
                           const int* binum, const int* bilist, const int* bnumneigh, const int* bfirstneigh,
                           const double* brcs, const int* btypes, int* brank, int* bincoming,
                           int ranks_valid, double* etot, double* force, double* virial, double* desc, void* stream)
{
    return a2p::nep_efv<double>(K, n_r, n_a, l_max, H, ntypes, coeffs, w0, b0, w1, bias, q_scaler, rr, ra,
                                B, P, U, nghost, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, etot,
                                force, virial, desc, (hipStream_t)stream, brank, bincoming, ranks_valid);
}

/* extension: four- / five-body invariants (l_4body 0 or 2, l_5body 0 or 1); no counterpart in the reference */
int a2p_nep_efv_manybody_f32(int K, int n_r, int n_a, int l_max, int l_4body, int l_5body, int H, int ntypes,
                             const float* coeffs, const float* w0, const float* b0, const float* w1, const float* bias,
                             const float* q_scaler, double rr, double ra, int B, int P, int U, int nghost,
                             const int* binum, const int* bilist, const int* bnumneigh, const int* bfirstneigh,
                             const float* brcs, const int* btypes, float* etot, float* force, float* virial,
                             float* desc, void* stream)
{
    A2P_REQUIRE((l_4body == 0 || l_4body == 2) && (l_5body == 0 || l_5body == 1), A2P_ERR_INVALID,
                "nep: l_4body must be 0 or 2, l_5body 0 or 1");
    return a2p::nep_efv<float>(K, n_r, n_a, l_max, H, ntypes, coeffs, w0, b0, w1, bias, q_scaler, rr, ra, B, P, U,
                               nghost, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, etot, force, virial, desc,
                               (hipStream_t)stream, nullptr, nullptr, 0, l_4body ? 1 : 0, l_5body ? 1 : 0);
}

int a2p_nep_efv_manybody_f64(int K, int n_r, int n_a, int l_max, int l_4body, int l_5body, int H, int ntypes,
                             const double* coeffs, const double* w0, const double* b0, const double* w1,
                             const double* bias, const double* q_scaler, double rr, double ra, int B, int P, int U,
                             int nghost, const int* binum, const int* bilist, const int* bnumneigh,
                             const int* bfirstneigh, const double* brcs, const int* btypes, double* etot, double* force,
                             double* virial, double* desc, void* stream)
{
    A2P_REQUIRE((l_4body == 0 || l_4body == 2) && (l_5body == 0 || l_5body == 1), A2P_ERR_INVALID,
                "nep: l_4body must be 0 or 2, l_5body 0 or 1");
    return a2p::nep_efv<double>(K, n_r, n_a, l_max, H, ntypes, coeffs, w0, b0, w1, bias, q_scaler, rr, ra, B, P, U,
                                nghost, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, etot, force, virial, desc,
                                (hipStream_t)stream, nullptr, nullptr, 0, l_4body ? 1 : 0, l_5body ? 1 : 0);
}
}
