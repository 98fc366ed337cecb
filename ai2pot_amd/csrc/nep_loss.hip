// NEP training loss: forward value and analytic gradient w.r.t. coeffs, w0, b0, w1, type_bias
// (the reference: source/descriptor/nep/include/nepLoss.h:170-209 loss, :752-1298 backward;
// nepLoss_cpu_launcher.h:167-330, 360-406; src/nepOp.cc:2359-3484 operator).
//
// Per structure  L = e_w/N (E - E0)^2 + f_w/(3N) sum |F - F0|^2 + v_w/(9N) sum (V - V0)^2.  With the
// scaled residuals  cE = 2 e_w/N (E - E0),  dF = 2 f_w/(3N) (F - F0),  dV = 2 v_w/(9N) (V - V0)
// and forces / virial linear in the pair derivatives g_ij = dE_i/dr_ij
// (F_i += g_ij, F_j -= g_ij, V_ab -= g_ij,a r_ij,b), the gradient is a sum over centre atoms of
//     d/dtheta [ cE E_i + sum_j w_ij . g_ij ],      w_ij = dF_i - dF_j - dV r_ij,
// and  sum_j w_ij . g_ij  is the directional derivative of E_i along the displacement field w:
// a tangent ("dotted") copy of every quantity on the way from the neighbours to the energy.
// For one atom (q descriptors, S angular moments, h hidden pre-activations, t = tanh h):
//     Phi = cE (bias + sum_p w1_p t_p) + sum_p w1_p (1 - t_p^2) hdot_p
//     alpha_p = dPhi/dh_p = w1_p (1 - t_p^2) (cE - 2 t_p hdot_p),   beta_p = dPhi/dhdot_p = w1_p (1 - t_p^2)
//     dPhi/db0_p = alpha_p,  dPhi/dw1_p = cE t_p + (1 - t_p^2) hdot_p,  dPhi/dbias = cE
//     dPhi/dW0_pd = alpha_p q_d/s_d + beta_p qdot_d/s_d
//     a_d = dPhi/dq_d = sum_p alpha_p W0_pd / s_d,   b_d = dPhi/dqdot_d = sum_p beta_p W0_pd / s_d
//     radial:  dPhi/dc[ti,t,n,k] = a_n F[t][k] + b_n Fdot[t][k],
//              F[t][k] = sum_{j of species t} f_k(r_j),  Fdot[t][k] = sum f'_k(r_j) (u_j . w_j)
//     angular: sigma_nlm = dPhi/dS_nlm = 2 w_m C_lm (a_nl S_nlm + b_nl Sdot_nlm),  tau_nlm = dPhi/dSdot_nlm
//              = 2 w_m C_lm b_nl S_nlm;  per neighbour  P_n(j) = sum_lm sigma Y_lm(j) + tau Ydot_lm(j),
//              Q_n(j) = (u.w) sum_lm tau Y_lm(j);  dPhi/dc[ti,tj,n_r+n,k] = sum_j fa_k(r_j) P_n(j) + fa'_k(r_j) Q_n(j)
// with Ydot_lm = (1/r) (w . grad b_lm(u) - l b_lm(u) (u.w)).
//
// One workgroup of 128 threads per centre atom, neighbours in chunks of 32 with a per-neighbour
// table in LDS; every sum runs in a fixed order (no atomics).  Per-atom gradient rows (the
// blocks of the centre's species only) are summed per structure in atom order by a second kernel.
#include "a2p_common.h"
#include "loss_kernels.h"
#include "nep_device.h"

namespace a2p {
using namespace nepdev;
namespace {

constexpr int LNT = 128;     // threads per atom
constexpr int LNC = 32;      // neighbours per chunk
constexpr int LKMAX = 16;
constexpr int LNLM = 24;

template <typename T>
struct NepLossArgs {
    int K, n_r, n_a, l_max, H, ntypes, D;
    const T *coeffs, *w0, *b0, *w1, *q_scaler;
    T rr, ra;
    int B, P, U;
    const int *binum, *bilist, *bnumneigh, *bfirstneigh;
    const T* brcs;
    const int* btypes;
    const T *cE, *dFs, *dVs;
    T* gpart;          // [B, P, nrow]
    int nrow;          // ntypes*(n_r+n_a)*K + H*D + 2H + 1
    int E;             // table entries per neighbour
    int* status;
};

template <typename T>
struct LossLds {
    T *tab, *G, *dG, *F, *Fd, *S, *Sd, *q, *qd, *av, *bv, *alpha, *beta, *sigma, *tau, *gca;
    int* tjs;
};

template <typename T>
__host__ __device__ inline size_t loss_lds_layout(const NepLossArgs<T>& a, unsigned char* base, LossLds<T>& L)
{
    size_t off = 0;
    auto take = [&](size_t n) { T* p = (T*)(base + off); off += ((n * sizeof(T) + 15) / 16) * 16; return p; };
    L.tab = take((size_t)LNC * a.E);
    L.G = take((size_t)LNC * a.n_a + 1);
    L.dG = take((size_t)LNC * a.n_a + 1);
    L.F = take((size_t)a.ntypes * a.K);
    L.Fd = take((size_t)a.ntypes * a.K);
    L.S = take((size_t)a.n_a * LNLM + 1);
    L.Sd = take((size_t)a.n_a * LNLM + 1);
    L.q = take(a.D);
    L.qd = take(a.D);
    L.av = take(a.D);
    L.bv = take(a.D);
    L.alpha = take(a.H);
    L.beta = take(a.H);
    L.sigma = take((size_t)a.n_a * LNLM + 1);
    L.tau = take((size_t)a.n_a * LNLM + 1);
    L.gca = take((size_t)a.ntypes * a.n_a * a.K + 1);
    L.tjs = (int*)(base + off);
    off += LNC * sizeof(int);
    return off;
}

__device__ __forceinline__ int l_of_lm(int m) { return m < 3 ? 1 : m < 8 ? 2 : m < 15 ? 3 : 4; }

// Table of neighbours [c0, c0+nc): per neighbour  f[K] f'[K] (radial cutoff; zero outside) |
// fa[K] fa'[K] (angular cutoff; zero outside) | Y[24] | Ydot[24] | u.w
template <typename T>
__device__ __forceinline__ void build_table(const NepLossArgs<T>& a, const LossLds<T>& L, int tid, int nc, int c0,
                                            size_t row, int b, int center, int ti)
{
    const int K = a.K;
    if (tid < nc) {
        const int jj = c0 + tid;
        const size_t pr = row * a.U + jj;
        const T x = a.brcs[pr * 3 + 0], y = a.brcs[pr * 3 + 1], z = a.brcs[pr * 3 + 2];
        int nj = a.bfirstneigh[pr];
        if ((unsigned)nj >= (unsigned)a.P) { atomicOr(a.status, ST_BAD_NEIGHBOR); nj = center; }
        int tj = a.btypes[(size_t)b * a.P + nj];
        if ((unsigned)tj >= (unsigned)a.ntypes) { atomicOr(a.status, ST_BAD_TYPE); tj = 0; }
        L.tjs[tid] = tj;
        const T r = sqrt_t(x * x + y * y + z * z);
        const T rinv = (T)1 / r;
        const T ux = x * rinv, uy = y * rinv, uz = z * rinv;
        const T* fc = a.dFs + ((size_t)b * a.P + center) * 3;
        const T* fn = a.dFs + ((size_t)b * a.P + nj) * 3;
        const T* dv = a.dVs + (size_t)b * 9;
        T w[3];
#pragma unroll
        for (int q = 0; q < 3; q++) w[q] = fc[q] - fn[q] - (dv[q * 3 + 0] * x + dv[q * 3 + 1] * y + dv[q * 3 + 2] * z);
        const T uw = w[0] * ux + w[1] * uy + w[2] * uz;
        T* t = L.tab + (size_t)tid * a.E;
        T f[LKMAX], df[LKMAX];
        if (r <= a.rr) radial_basis<T, LKMAX, true>(r, (T)1 / a.rr, K, f, df);
        else
#pragma unroll
            for (int k = 0; k < LKMAX; k++) { f[k] = (T)0; df[k] = (T)0; }
        for (int k = 0; k < K; k++) { t[k] = f[k]; t[K + k] = df[k]; }
        const bool ang = a.l_max > 0 && r <= a.ra && r <= a.rr;     // nepBasis.h:106, 135
        if (ang) radial_basis<T, LKMAX, true>(r, (T)1 / a.ra, K, f, df);
        else
#pragma unroll
            for (int k = 0; k < LKMAX; k++) { f[k] = (T)0; df[k] = (T)0; }
        for (int k = 0; k < K; k++) { t[2 * K + k] = f[k]; t[3 * K + k] = df[k]; }
        T Y[LNLM], Gd[LNLM];
        blm_values<T, 4>(ux, uy, uz, Y);
        blm_dir_derivs<T, 4>(ux, uy, uz, w[0], w[1], w[2], Gd);
        T* ty = t + 4 * K;
#pragma unroll
        for (int m = 0; m < LNLM; m++) {
            ty[m] = Y[m];
            ty[LNLM + m] = rinv * (Gd[m] - (T)l_of_lm(m) * Y[m] * uw);
        }
        ty[2 * LNLM] = uw;
    }
}

template <typename T>
__global__ void __launch_bounds__(LNT) nep_loss_grad_kernel(const NepLossArgs<T> a)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    LossLds<T> L;
    loss_lds_layout<T>(a, smem_raw, L);
    const int tid = threadIdx.x;
    const int ii = blockIdx.x, b = blockIdx.y;
    const size_t row = (size_t)b * a.P + ii;
    const int K = a.K, n_r = a.n_r, l_max = a.l_max, H = a.H, nt = a.ntypes, D = a.D;
    const int nb = n_r + a.n_a;                     // layout of the coefficient tensor
    const int n_a = l_max > 0 ? a.n_a : 0;          // angular functions in use
    const int ncl = nt * nb * K;                    // coefficient block of one centre species
    T* grow = a.gpart + row * a.nrow;
    if (ii >= a.binum[b]) {
        for (int q = tid; q < a.nrow; q += LNT) grow[q] = (T)0;
        return;
    }
    int center = a.bilist[row];
    int nn = a.bnumneigh[row];
    if (nn > a.U) { if (tid == 0) atomicOr(a.status, ST_NEIGH_OVERFLOW); nn = a.U; }
    if ((unsigned)center >= (unsigned)a.P) { if (tid == 0) atomicOr(a.status, ST_BAD_NEIGHBOR); center = 0; nn = 0; }
    int ti = a.btypes[(size_t)b * a.P + center];
    if ((unsigned)ti >= (unsigned)nt) { if (tid == 0) atomicOr(a.status, ST_BAD_TYPE); ti = 0; nn = 0; }
    const T cE = a.cE[b];
    const T* cti = a.coeffs + (size_t)ti * nt * nb * K;     // c[ti][tj][n][k]
    const int E = a.E;
    const int OY = 4 * K, OYD = 4 * K + LNLM, OUW = 4 * K + 2 * LNLM;

    for (int q = tid; q < a.nrow; q += LNT) grow[q] = (T)0;
    for (int o = tid; o < nt * K; o += LNT) { L.F[o] = (T)0; L.Fd[o] = (T)0; }
    for (int o = tid; o < n_a * LNLM; o += LNT) { L.S[o] = (T)0; L.Sd[o] = (T)0; }
    for (int o = tid; o < nt * n_a * K; o += LNT) L.gca[o] = (T)0;
    __syncthreads();

    // ---- pass A: per-species radial sums, angular moments, and their tangents -----------------
    for (int c0 = 0; c0 < nn; c0 += LNC) {
        const int nc = min(LNC, nn - c0);
        build_table<T>(a, L, tid, nc, c0, row, b, center, ti);
        __syncthreads();
        for (int it = tid; it < nc * n_a; it += LNT) {
            const int j = it / n_a, n = it - j * n_a;
            const T* t = L.tab + (size_t)j * E;
            const T* c = cti + ((size_t)L.tjs[j] * nb + n_r + n) * K;
            T g = (T)0, dg = (T)0;
            for (int k = 0; k < K; k++) { g += c[k] * t[2 * K + k]; dg += c[k] * t[3 * K + k]; }
            L.G[it] = g; L.dG[it] = dg;
        }
        for (int o = tid; o < nt * K; o += LNT) {
            const int ts = o / K, k = o - ts * K;
            T f = L.F[o], fd = L.Fd[o];
            for (int j = 0; j < nc; j++) {
                if (L.tjs[j] != ts) continue;
                const T* t = L.tab + (size_t)j * E;
                f += t[k];
                fd += t[K + k] * t[OUW];
            }
            L.F[o] = f; L.Fd[o] = fd;
        }
        __syncthreads();
        for (int o = tid; o < n_a * LNLM; o += LNT) {
            const int n = o / LNLM, m = o - n * LNLM;
            T s = L.S[o], sd = L.Sd[o];
            for (int j = 0; j < nc; j++) {
                const T* t = L.tab + (size_t)j * E;
                const T g = L.G[j * n_a + n], dg = L.dG[j * n_a + n];
                s += g * t[OY + m];
                sd += dg * t[OUW] * t[OY + m] + g * t[OYD + m];
            }
            L.S[o] = s; L.Sd[o] = sd;
        }
        __syncthreads();
    }

    // ---- descriptors and their tangents (nepBasis.h:153-190) ----------------------------------
    for (int d = tid; d < D; d += LNT) {
        T q = (T)0, qd = (T)0;
        if (d < n_r) {
            for (int ts = 0; ts < nt; ts++) {
                const T* c = cti + ((size_t)ts * nb + d) * K;
                for (int k = 0; k < K; k++) { q += c[k] * L.F[ts * K + k]; qd += c[k] * L.Fd[ts * K + k]; }
            }
        } else {
            const int n = (d - n_r) / l_max, l = (d - n_r) % l_max + 1;
            for (int mp = 0; mp < 2 * l + 1; mp++) {
                const int m = l * l - 1 + mp;
                const T wc = (T)(mp == 0 ? 1.0 : 2.0) * (T)kC3B[m];
                const T s = L.S[n * LNLM + m], sd = L.Sd[n * LNLM + m];
                q += wc * s * s;
                qd += (T)2 * wc * s * sd;
            }
        }
        const T qs = a.q_scaler[d];
        L.q[d] = q / qs;           // scaled descriptor and tangent
        L.qd[d] = qd / qs;
    }
    __syncthreads();

    // ---- hidden layer, alpha / beta, gradients of b0, w1 ---------------------------------------
    T* g_w0 = grow + ncl;
    T* g_b0 = g_w0 + (size_t)H * D;
    T* g_w1 = g_b0 + H;
    for (int p = tid; p < H; p += LNT) {
        const T* wrow = a.w0 + ((size_t)ti * H + p) * D;
        T h = a.b0[ti * H + p], hd = (T)0;
        for (int d = 0; d < D; d++) { h += wrow[d] * L.q[d]; hd += wrow[d] * L.qd[d]; }
        const T t = tanh_t(h);
        const T s = (T)1 - t * t;
        const T w1p = a.w1[ti * H + p];
        const T al = w1p * s * (cE - (T)2 * t * hd);
        const T be = w1p * s;
        L.alpha[p] = al; L.beta[p] = be;
        g_b0[p] = al;
        g_w1[p] = cE * t + s * hd;
    }
    if (tid == 0) grow[a.nrow - 1] = cE;       // type_bias
    __syncthreads();
    for (int o = tid; o < H * D; o += LNT) {
        const int p = o / D, d = o - p * D;
        g_w0[o] = L.alpha[p] * L.q[d] + L.beta[p] * L.qd[d];
    }
    for (int d = tid; d < D; d += LNT) {
        T av = (T)0, bv = (T)0;
        for (int p = 0; p < H; p++) {
            const T w = a.w0[((size_t)ti * H + p) * D + d];
            av += L.alpha[p] * w; bv += L.beta[p] * w;
        }
        const T qs = a.q_scaler[d];
        L.av[d] = av / qs; L.bv[d] = bv / qs;
    }
    __syncthreads();

    // ---- radial coefficient gradient; sigma, tau ------------------------------------------------
    for (int o = tid; o < nt * n_r * K; o += LNT) {
        const int ts = o / (n_r * K), rem = o - ts * n_r * K, n = rem / K, k = rem - n * K;
        grow[((size_t)ts * nb + n) * K + k] = L.av[n] * L.F[ts * K + k] + L.bv[n] * L.Fd[ts * K + k];
    }
    for (int o = tid; o < n_a * LNLM; o += LNT) {
        const int n = o / LNLM, m = o - n * LNLM;
        const int l = l_of_lm(m);
        T sg = (T)0, ta = (T)0;
        if (l <= l_max) {
            const int mp = m - (l * l - 1);
            const T wc2 = (T)2 * (T)(mp == 0 ? 1.0 : 2.0) * (T)kC3B[m];
            const int d = n_r + n * l_max + (l - 1);
            sg = wc2 * (L.av[d] * L.S[o] + L.bv[d] * L.Sd[o]);
            ta = wc2 * L.bv[d] * L.S[o];
        }
        L.sigma[o] = sg; L.tau[o] = ta;
    }
    __syncthreads();

    // ---- pass B: angular coefficient gradient -----------------------------------------------------
    if (n_a > 0 && l_max > 0) {
        for (int c0 = 0; c0 < nn; c0 += LNC) {
            const int nc = min(LNC, nn - c0);
            build_table<T>(a, L, tid, nc, c0, row, b, center, ti);
            __syncthreads();
            for (int it = tid; it < nc * n_a; it += LNT) {
                const int j = it / n_a, n = it - j * n_a;
                const T* t = L.tab + (size_t)j * E;
                T pv = (T)0, qv = (T)0;
                for (int m = 0; m < LNLM; m++) {
                    pv += L.sigma[n * LNLM + m] * t[OY + m] + L.tau[n * LNLM + m] * t[OYD + m];
                    qv += L.tau[n * LNLM + m] * t[OY + m];
                }
                L.G[it] = pv; L.dG[it] = qv * t[OUW];
            }
            __syncthreads();
            for (int o = tid; o < nt * n_a * K; o += LNT) {
                const int ts = o / (n_a * K), rem = o - ts * n_a * K, n = rem / K, k = rem - n * K;
                T acc = L.gca[o];
                for (int j = 0; j < nc; j++) {
                    if (L.tjs[j] != ts) continue;
                    const T* t = L.tab + (size_t)j * E;
                    acc += t[2 * K + k] * L.G[j * n_a + n] + t[3 * K + k] * L.dG[j * n_a + n];
                }
                L.gca[o] = acc;
            }
            __syncthreads();
        }
    }
    for (int o = tid; o < nt * n_a * K; o += LNT) {
        const int ts = o / (n_a * K), rem = o - ts * n_a * K, n = rem / K, k = rem - n * K;
        grow[((size_t)ts * nb + n_r + n) * K + k] = L.gca[o];
    }
}

// Full-layout gradients of one structure: element e of the layout belongs to centre species t(e)
// and position q(e) of the per-atom row; sum the rows of the atoms of that species (four runs of rows in atom order,
// then the runs).
template <typename T>
__global__ void __launch_bounds__(256)
nep_grad_reduce_kernel(NepLossArgs<T> a, T* __restrict__ dcoeffs, T* __restrict__ dw0, T* __restrict__ db0,
                       T* __restrict__ dw1, T* __restrict__ dbias)
{
    const int b = blockIdx.y;
    const int nt = a.ntypes, H = a.H, D = a.D, nb = a.n_r + a.n_a, K = a.K;
    const int ncl = nt * nb * K;
    const int n_c = nt * ncl, n_w0 = nt * H * D, n_h = nt * H;
    const int total = n_c + n_w0 + 2 * n_h + nt;
    // 64 elements per workgroup, the rows of the structure in four runs (one per wavefront) whose sums are added in
    // run order: the chain of dependent loads per row (centre, species, entry) is a quarter as long
    __shared__ T red[4][64];
    const int e = blockIdx.x * 64 + (threadIdx.x & 63), part = threadIdx.x >> 6;
    int t = 0, q = 0;
    T* out = nullptr;
    if (e < total) {
        if (e < n_c) { t = e / ncl; q = e - t * ncl; out = dcoeffs ? dcoeffs + (size_t)b * n_c + e : nullptr; }
        else if (e < n_c + n_w0) { const int r = e - n_c; t = r / (H * D); q = ncl + r - t * H * D; out = dw0 ? dw0 + (size_t)b * n_w0 + r : nullptr; }
        else if (e < n_c + n_w0 + n_h) { const int r = e - n_c - n_w0; t = r / H; q = ncl + H * D + r - t * H; out = db0 ? db0 + (size_t)b * n_h + r : nullptr; }
        else if (e < n_c + n_w0 + 2 * n_h) { const int r = e - n_c - n_w0 - n_h; t = r / H; q = ncl + H * D + H + r - t * H; out = dw1 ? dw1 + (size_t)b * n_h + r : nullptr; }
        else { t = e - n_c - n_w0 - 2 * n_h; q = a.nrow - 1; out = dbias ? dbias + (size_t)b * nt + t : nullptr; }
    }
    const int inum = a.binum[b];
    const int run = ((inum + 3) / 4 + 7) / 8 * 8;
    const int i_end = min(inum, (part + 1) * run);
    T acc = (T)0;
    if (out) {
        // eight rows in flight; the rows of other species are skipped, the order of the sum is the atom order
        for (int i0 = part * run; i0 < i_end; i0 += 8) {
            int c[8], ty[8];
            T v[8];
#pragma unroll
            for (int u = 0; u < 8; u++) c[u] = a.bilist[(size_t)b * a.P + min(i0 + u, i_end - 1)];
#pragma unroll
            for (int u = 0; u < 8; u++) {
                const bool ok = i0 + u < i_end && (unsigned)c[u] < (unsigned)a.P;
                ty[u] = a.btypes[(size_t)b * a.P + (ok ? c[u] : 0)];
                if (!ok) ty[u] = -1;
            }
#pragma unroll
            for (int u = 0; u < 8; u++) {        // (a row of another species is not read: its lanes are masked off)
                v[u] = (T)0;
                if (ty[u] == t) v[u] = a.gpart[((size_t)b * a.P + min(i0 + u, i_end - 1)) * a.nrow + q];
            }
#pragma unroll
            for (int u = 0; u < 8; u++) acc += v[u];
        }
    }
    red[part][threadIdx.x & 63] = acc;
    __syncthreads();
    if (part == 0 && out) *out = ((red[0][threadIdx.x] + red[1][threadIdx.x]) + red[2][threadIdx.x]) + red[3][threadIdx.x];
}

inline int efv_call(int K, int n_r, int n_a, int l_max, int H, int ntypes, const float* c, const float* w0,
                    const float* b0, const float* w1, const float* bias, const float* qs, double rr, double ra, int B,
                    int P, int U, const int* binum, const int* bilist, const int* bnn, const int* bfn, const float* brcs,
                    const int* btypes, float* e, float* f, float* v, void* stream)
{
    return a2p_nep_efv_f32(K, n_r, n_a, l_max, H, ntypes, c, w0, b0, w1, bias, qs, rr, ra, B, P, U, 0, binum, bilist,
                           bnn, bfn, brcs, btypes, e, f, v, nullptr, stream);
}
inline int efv_call(int K, int n_r, int n_a, int l_max, int H, int ntypes, const double* c, const double* w0,
                    const double* b0, const double* w1, const double* bias, const double* qs, double rr, double ra,
                    int B, int P, int U, const int* binum, const int* bilist, const int* bnn, const int* bfn,
                    const double* brcs, const int* btypes, double* e, double* f, double* v, void* stream)
{
    return a2p_nep_efv_f64(K, n_r, n_a, l_max, H, ntypes, c, w0, b0, w1, bias, qs, rr, ra, B, P, U, 0, binum, bilist,
                           bnn, bfn, brcs, btypes, e, f, v, nullptr, stream);
}

template <typename T>
int nep_loss(double e_w, double f_w, double v_w, const T* e_dft, const T* f_dft, const T* v_dft, int K, int n_r,
             int n_a, int l_max, int H, int ntypes, const T* coeffs, const T* w0, const T* b0, const T* w1,
             const T* bias, const T* q_scaler, double rr, double ra, int B, int P, int U, const int* binum,
             const int* bilist, const int* bnumneigh, const int* bfirstneigh, const T* brcs, const int* btypes,
             T* bloss, T* rmse, T* etot, T* force, T* virial, T* dcoeffs, T* dw0, T* db0, T* dw1, T* dbias,
             hipStream_t stream)
{
    A2P_REQUIRE(e_dft && f_dft && v_dft && bloss && etot && force && virial, A2P_ERR_INVALID,
                "nep loss: null label or output pointer");
    A2P_REQUIRE(K <= LKMAX, A2P_ERR_INVALID, "nep loss: chebyshev_size %d above %d", K, LKMAX);
    int rc = efv_call(K, n_r, n_a, l_max, H, ntypes, coeffs, w0, b0, w1, bias, q_scaler, rr, ra, B, P, U, binum,
                      bilist, bnumneigh, bfirstneigh, brcs, btypes, etot, force, virial, (void*)stream);
    if (rc) return rc;
    if (B == 0 || P == 0) return A2P_OK;
    NepLossArgs<T> a;
    a.K = K; a.n_r = n_r; a.n_a = n_a; a.l_max = l_max; a.H = H; a.ntypes = ntypes;
    a.D = (l_max == 0) ? n_r : n_r + n_a * l_max;
    a.coeffs = coeffs; a.w0 = w0; a.b0 = b0; a.w1 = w1; a.q_scaler = q_scaler;
    a.rr = (T)rr; a.ra = (T)ra;
    a.B = B; a.P = P; a.U = U;
    a.binum = binum; a.bilist = bilist; a.bnumneigh = bnumneigh; a.bfirstneigh = bfirstneigh;
    a.brcs = brcs; a.btypes = btypes;
    a.nrow = ntypes * (n_r + n_a) * K + H * a.D + 2 * H + 1;
    a.E = 4 * K + 2 * LNLM + 1;
    if ((a.E & 1) == 0) a.E++;
    const bool want_grad = dcoeffs || dw0 || db0 || dw1 || dbias;
    // workspace: cE[B] | dVs[B*9] | dFs[B*P*3] | gpart[B*P*nrow] | sq[B*3] (double)
    size_t nT = (size_t)B + (size_t)B * 9 + (size_t)B * P * 3 + (want_grad ? (size_t)B * P * a.nrow : 0);
    size_t bytesT = (nT * sizeof(T) + 15) / 16 * 16;
    void* ws = nullptr;
    rc = ws_get(WS_MTP, bytesT + (size_t)B * 3 * sizeof(double), &ws);
    if (rc) return rc;
    T* cE = (T*)ws;
    T* dVs = cE + B;
    T* dFs = dVs + (size_t)B * 9;
    a.gpart = dFs + (size_t)B * P * 3;
    double* sq = (double*)((char*)ws + bytesT);
    rc = ws_get(WS_FLAGS, 64, &ws);
    if (rc) return rc;
    a.status = (int*)ws;
    prof_begin("nep_loss_forward", stream);
    hipLaunchKernelGGL(losskern::loss_forward_kernel<T>, dim3(B), dim3(256), 0, stream, P, binum, bilist, (T)e_w,
                       (T)f_w, (T)v_w, etot, e_dft, force, f_dft, virial, v_dft, bloss, cE, dFs, dVs, sq, 0);
    if (rmse) hipLaunchKernelGGL(losskern::loss_rmse_kernel<T>, dim3(1), dim3(64), 0, stream, B, binum, sq, rmse);
    prof_end(stream);
    A2P_HIP_CHECK(hipGetLastError());
    if (!want_grad) return A2P_OK;
    a.cE = cE; a.dFs = dFs; a.dVs = dVs;
    LossLds<T> unused;
    const size_t lds = loss_lds_layout<T>(a, nullptr, unused);
    A2P_REQUIRE(lds <= 150 * 1024, A2P_ERR_INVALID, "nep loss: model too large for LDS (%zu bytes)", lds);
    auto kern = nep_loss_grad_kernel<T>;
    if (lds > 48 * 1024)
        A2P_HIP_CHECK(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    prof_begin("nep_loss_bwd_kernel", stream);
    hipLaunchKernelGGL(kern, dim3(P, B), dim3(LNT), lds, stream, a);
    prof_end(stream);
    const int total = ntypes * ntypes * (n_r + n_a) * K + ntypes * H * a.D + 2 * ntypes * H + ntypes;
    prof_begin("nep_grad_reduce", stream);
    hipLaunchKernelGGL(nep_grad_reduce_kernel<T>, dim3(ceil_div(total, 64), B), dim3(256), 0, stream, a, dcoeffs, dw0,
                       db0, dw1, dbias);
    prof_end(stream);
    A2P_HIP_CHECK(hipGetLastError());
    return A2P_OK;
}

}  // namespace
}  // namespace a2p

extern "C" {

int a2p_nep_loss_f64(double e_weight, double f_weight, double v_weight, const double* e_dft, const double* f_dft,
                     const double* v_dft, int K, int n_r, int n_a, int l_max, int H, int ntypes, const double* coeffs,
                     const double* w0, const double* b0, const double* w1, const double* bias, const double* q_scaler,
                     double rr, double ra, int B, int P, int U, const int* binum, const int* bilist,
                     const int* bnumneigh, const int* bfirstneigh, const double* brcs, const int* btypes,
                     double* bloss, double* rmse, double* etot, double* force, double* virial, double* dcoeffs,
                     double* dw0, double* db0, double* dw1, double* dbias, void* stream)
{
    return a2p::nep_loss<double>(e_weight, f_weight, v_weight, e_dft, f_dft, v_dft, K, n_r, n_a, l_max, H, ntypes,
                                 coeffs, w0, b0, w1, bias, q_scaler, rr, ra, B, P, U, binum, bilist, bnumneigh,
                                 bfirstneigh, brcs, btypes, bloss, rmse, etot, force, virial, dcoeffs, dw0, db0, dw1,
                                 dbias, (hipStream_t)stream);
}

int a2p_nep_loss_f32(double e_weight, double f_weight, double v_weight, const float* e_dft, const float* f_dft,
                     const float* v_dft, int K, int n_r, int n_a, int l_max, int H, int ntypes, const float* coeffs,
                     const float* w0, const float* b0, const float* w1, const float* bias, const float* q_scaler,
                     double rr, double ra, int B, int P, int U, const int* binum, const int* bilist,
                     const int* bnumneigh, const int* bfirstneigh, const float* brcs, const int* btypes, float* bloss,
                     float* rmse, float* etot, float* force, float* virial, float* dcoeffs, float* dw0, float* db0,
                     float* dw1, float* dbias, void* stream)
{
    return a2p::nep_loss<float>(e_weight, f_weight, v_weight, e_dft, f_dft, v_dft, K, n_r, n_a, l_max, H, ntypes,
                                coeffs, w0, b0, w1, bias, q_scaler, rr, ra, B, P, U, binum, bilist, bnumneigh,
                                bfirstneigh, brcs, btypes, bloss, rmse, etot, force, virial, dcoeffs, dw0, db0, dw1,
                                dbias, (hipStream_t)stream);
}
}
