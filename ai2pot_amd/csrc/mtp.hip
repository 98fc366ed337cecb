// Linear Moment Tensor Potential for gfx950: energy / force / virial, and the analytic
// gradient of the training loss w.r.t. coeffs, linear_coeffs and type_bias.
//
// One workgroup (64 threads, or 256 for the larger levels) per centre atom; the moment vector M,
// its adjoint and (for the loss gradient) the tangent and mixed vectors live in LDS.  Neighbours
// are processed in equal chunks of at most 32 to 48: a per-neighbour table (powers of the unit vector, contracted
// radial functions g_mu(r) = sum_k c[ti,tj,mu,k] f_k(r) and their r-derivatives) is staged
// in LDS, then
//   basic moments : lane <- basic moment i,  M_i += sum_j g_mu(r_j) ux^a uy^b uz^c
//                   (x^a y^b z^c / r^(a+b+c) of the reference, include/mtpBasis.h:472-519,
//                    written with the unit vector u = r_ij / r)
//   products      : level-ordered gather over the host-built plan (mtp_plan.h)
//   energy        : E_i = bias[t] + sum_s lin[s] M[map[s]] / q_scaler[s]  (linearMtp.h:281-285)
//   adjoint       : seed + reverse gather                                  (linearMtp.h:292-306)
//   pair forces   : lane <- (neighbour, a share of the monomial rows x^a y^b z^*):
//                   dE_i/dr_ij = u sum_i adj_i m_i (g' - k g / r) + (1/r) sum_i adj_i g grad_u m_i
//                   with the adjoints gathered by monomial and z^c by recurrence (pair_walk; three uniform
//                   LDS reads per monomial instead of ten scattered ones per basic moment)
//                   -> reduction segments of the neighbours (a2p::PairCsr), summed without float atomics
// The loss gradient adds the tangent sweep (include/linearMtpLoss.h:371-398), the mixed
// adjoint (:417-434) and the coefficient-gradient pass (:438-536) in the same structure;
// per-structure gradients are accumulated per workgroup and summed by a second kernel.
#include "a2p_common.h"
#include "mtp_plan.h"
#include "loss_kernels.h"

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <set>
#include <string>

namespace a2p {
namespace {

constexpr int MTP_NC = 32;        // neighbours per chunk (rows of the LDS table); the energy / force / virial
constexpr int MTP_NC_MAX = 48;    // the launch picks between MTP_NC_MIN and MTP_NC_MAX rows (launch_atoms)
constexpr int MTP_NC_MIN = 16;

// The group sums of the last pass over the neighbours (four per thread for the pair derivatives, two
// for the loss gradient) live in the moment vector (loss mode: moments and tangents) when it is long
// enough, else behind the neighbour table.
__host__ __device__ inline bool mtp_gred_in_moments(bool loss, int n_moms)
{
    return loss ? 2 * n_moms >= 512 : n_moms >= 1024;
}
// entries of the region that holds the neighbour table (+ group sums) and doubles as the sweeps' partial sums.
// In the energy / force / virial kernel the group sums (4 per thread) are written over the table once every
// thread has finished reading it.
// The adjoints live in this region too, behind the partial sums (mtp_adjoint_offset): they are needed from the end of
// the forward sweep to the last pass over the neighbours, which is when the neighbour table is not.  That pass needs
// the adjoints of the basic moments only: the energy / force / virial kernel gathers them into its dense array, the
// loss kernel copies them behind the region first.
__host__ __device__ inline int mtp_adjoint_offset(int max_level_slots)
{
    return ((max_level_slots > 8 ? max_level_slots : 8) + 1) & ~1;     // at least the scratch of a block sum
}
// keep (energy / force / virial kernel, when the LDS allows it without costing a workgroup per CU): the adjoints lie
// behind the table instead of inside it, so that a row of one chunk finds its table still in place in the last pass.
__host__ __device__ inline int mtp_table_entries(int nc, int E, bool loss, int n_moms, int nt)
{
    int a = loss ? nc * E + (mtp_gred_in_moments(loss, n_moms) ? 0 : (256 / 32) * 32 * 4) : nc * E;
    if (!loss && a < nt * 4) a = nt * 4;          // four group sums per thread
    return (a + 1) & ~1;
}
__host__ __device__ inline int mtp_table_region(int nc, int E, bool loss, int n_moms, int max_level_slots, int nt,
                                                bool keep = false)
{
    const int a = mtp_table_entries(nc, E, loss, n_moms, nt);
    // loss mode: two partial-sum arrays, then the adjoints and the mixed adjoints
    const int b = loss ? mtp_adjoint_offset(2 * max_level_slots) + 2 * n_moms : mtp_adjoint_offset(max_level_slots) + n_moms;
    if (keep) return a + n_moms;
    return a > b ? a : b;
}
// the dense adjoint array of the pair-derivative pass takes the place of the moments when it fits
__host__ __device__ inline bool mtp_dense_in_moments(int nq, int nmp, int n_moms) { return nq * nmp <= n_moms; }
constexpr int MTP_NGMAX = 16;     // most thread groups that share the basic moments of a chunk
constexpr int MTP_KMAX = 16;      // radial basis size limit
constexpr int MTP_NMUS_MAX = 8;   // radial function count limit
constexpr int MTP_NODE_CAP = 4094; // most (scalar moment, ancestor) nodes of one launch of the components kernel

template <typename T>
struct MtpArgs {
    MtpPlanDevice p;
    int K, ntypes;
    T scaling, rmax, rmin;
    const T *coeffs, *lin, *bias, *q_scaler;
    int B, P, U, nghost;
    const int *binum, *bilist, *bnumneigh, *bfirstneigh;
    const T* brcs;
    const int* btypes;
    T* force;          // [B, P+nghost, 3]
    int* seg_cursor;   // reduction segments of fixed capacity U (a2p::PairCsr): entries claimed per target,
    T* seg_g;          // the entries, and the entry that takes what overflows a segment;
    int seg_spare;     // seg_cursor is null when no forces are wanted
    int seg_cap;       // capacity of a segment
    double* partial;   // [B, P, 10]  energy + virial per atom
    int* status;
    int E;             // table entries per neighbour
    // loss gradient mode
    const T* cE;       // [B]        2 e_w / N (E - E_dft)
    const T* dFs;      // [B, P, 3]  2 f_w / (3N) (F - F_dft)
    const T* dVs;      // [B, 9]     2 v_w / (9N) (V - V_dft)
    T* gpart;          // [B, P, ngrad] per-atom gradient rows (ngrad = ncoef + n_scalar + ntypes)
    int ngrad;
    int lds_basic_off;  // byte offset of the packed basic-moment table in LDS
    int nc_cap;         // rows of the LDS neighbour table: a row is processed in chunks of at most nc_cap
    int keep_table;     // energy / force / virial kernel: the adjoints lie behind the table (mtp_table_region)
    // site-energy / descriptor mode (linearMtp.h:514-611, 821-890)
    T* e_sites;        // [B, P] per-row energies, or null
    T* desc;           // [B, P, n_scalar] scalar moments, or null
    int energy_only;   // stop after the energy: no adjoint, no pair derivatives
    int cE_per_atom;   // loss-gradient mode: cE is indexed per row (weights of the site energies)
    int no_tangent;    // loss-gradient mode: the force and virial residuals are zero (site-energy and basis backward),
                       // so the tangents and mixed adjoints vanish: their sweeps and terms are left out
    // neural-network read-out (source/descriptor/nnmtp/include/nnMtp.h:470-507) when H > 0:
    // e_i = bias + sum_p w1[t,p] tanh(sum_k w0[t,p,k] (M_k - q_shift[k]) / q_scaler[k]); `lin` is unused
    int H;
    const T *w0, *w1, *q_shift;
    int nn_exact;      // loss mode: 1 = complete derivative, 0 = the reference's formulas (see nnmtp_loss)
    // backward of the legacy basis operator (mtpBasis.h:359-394): the adjoint sweep starts from the caller's
    // weights of each row's scalar moments instead of a read-out (`lin`, `bias`, `q_scaler` are unused)
    const T* row_seed; // [B, P, n_scalar], or null
    T* pair_out;       // [B, P, U, 3] derivative of the row's weighted moments along each pair vector, or null
};

__device__ __forceinline__ float tanh_t(float x) { return tanhf(x); }
__device__ __forceinline__ double tanh_t(double x) { return tanh(x); }

__device__ __forceinline__ float sqrt_t(float x) { return sqrtf(x); }
__device__ __forceinline__ double sqrt_t(double x) { return sqrt(x); }

// Per-neighbour table for neighbours [c0, c0+nc) of the row.
// Layout per neighbour (E entries of T): ux^0..kmax | uy^.. | uz^.. | g[nmus] | dg[nmus] |
// ux uy uz 1/r | (loss mode) wx wy wz w.u | f[K] | df[K]
// The work is spread over nc * (nmus + 3) tasks: task (role, j) computes for neighbour j either
// one radial function g_role(r) with its derivative (role < nmus; coefficients from the LDS copy
// `cf` of the centre species' block) or the powers of one unit-vector component (role - nmus),
// so the table costs one Chebyshev recurrence of latency instead of nmus of them on nc lanes.
// Lanes j < nc also return the neighbour's index, validity and displacement.
template <typename T, bool LOSS, int NT>
__device__ __forceinline__ void build_table(const MtpArgs<T>& a, T* tab, const T* cf, int lane, int nc, int c0,
                                            const T* rcs, const int* first, const int* types, int center,
                                            int b, int NF, int* nj_out, bool* valid_out, T* d_out, bool fill = true)
{
    const int kmax = a.p.kmax, nmus = a.p.nmus, K = a.K;
    const int OG = 3 * (kmax + 1), ODG = OG + nmus, OU = ODG + nmus, OW = OU + 4, OF = OW + 4, ODF = OF + K;
    *valid_out = false;
    *nj_out = center;
    if (lane < nc) {
        const int jj = c0 + lane;
        const T x = rcs[jj * 3 + 0], y = rcs[jj * 3 + 1], z = rcs[jj * 3 + 2];
        d_out[0] = x; d_out[1] = y; d_out[2] = z;
        int nj = first[jj];
        if ((unsigned)nj >= (unsigned)NF) { atomicOr(a.status, ST_BAD_NEIGHBOR); nj = center; }
        if ((unsigned)types[nj] >= (unsigned)a.ntypes) atomicOr(a.status, ST_BAD_TYPE);
        *nj_out = nj;
        *valid_out = !(sqrt_t(x * x + y * y + z * z) > a.rmax);      // mtpBasis.h:457, linearMtp.h:316
    }
    const int ntask = fill ? nc * (nmus + 3) : 0;          // fill = false: the table is in place, only the lanes' own
    for (int task = lane; task < ntask; task += NT) {      // neighbours are returned
        const int role = task / nc, j = task - role * nc;
        const int jj = c0 + j;
        const T x = rcs[jj * 3 + 0], y = rcs[jj * 3 + 1], z = rcs[jj * 3 + 2];
        const T r = sqrt_t(x * x + y * y + z * z);
        T* t = tab + j * a.E;
        // radial functions, basis.h:154-196, 351-381, 620-637
        const T span = a.rmax - a.rmin;
        const T xx = ((T)2 * r - (a.rmax + a.rmin)) / span;
        const T dxx = (T)2 / span;
        const T u = (r - a.rmin) / span;
        T s = (T)0, ds = (T)0;
        if (!(r > a.rmax) && r >= a.rmin && r < a.rmax) {
            s = u * u * u * ((T)-6 * u * u + (T)15 * u - (T)10) + (T)1;
            ds = (T)1 / span * ((T)-30 * u * u * u * u + (T)60 * u * u * u - (T)30 * u * u);
        }
        int nj = first[jj];
        if ((unsigned)nj >= (unsigned)NF) nj = center;
        if (role < nmus || (LOSS && role == nmus + 1)) {
            int tj = types[nj];
            if ((unsigned)tj >= (unsigned)a.ntypes) tj = 0;
            const T* c = cf + (tj * nmus + (role < nmus ? role : 0)) * K;
            T g = (T)0, dg = (T)0;
            T t0 = (T)1, t1 = xx, d0 = (T)0, d1 = (T)1;
            for (int k = 0; k < K; k++) {
                T tv, dv;
                if (k == 0) { tv = t0; dv = d0; }
                else if (k == 1) { tv = t1; dv = d1; }
                else {
                    tv = (T)2 * xx * t1 - t0;
                    dv = (T)2 * t1 + (T)2 * xx * d1 - d0;
                    t0 = t1; t1 = tv; d0 = d1; d1 = dv;
                }
                const T f = a.scaling * s * tv;
                const T df = a.scaling * (ds * tv + s * dv * dxx);
                if (role < nmus) { g += c[k] * f; dg += c[k] * df; }
                else { t[OF + k] = f; t[ODF + k] = df; }
            }
            if (role < nmus) { t[OG + role] = g; t[ODG + role] = dg; }
        }
        if (role >= nmus) {
            const int ax = role - nmus;
            const T rinv = (T)1 / r;
            const T ux = x * rinv, uy = y * rinv, uz = z * rinv;
            const T uc = ax == 0 ? ux : (ax == 1 ? uy : uz);
            T pw = (T)1;
            T* tp = t + ax * (kmax + 1);
            for (int k = 0; k <= kmax; k++) { tp[k] = pw; pw *= uc; }
            if (ax == 0) { t[OU + 0] = ux; t[OU + 1] = uy; t[OU + 2] = uz; t[OU + 3] = rinv; }
            if (LOSS && ax == 2) {
                // w_a = dFs[centre]_a - dFs[neighbour]_a - sum_b dVs[a,b] r_b   (linearMtpLoss.h:371-386)
                const T* fc = a.dFs + ((size_t)b * a.P + center) * 3;
                const T* fn = a.dFs + ((size_t)b * a.P + nj) * 3;
                const T* dv = a.dVs + (size_t)b * 9;
                T w[3];
#pragma unroll
                for (int q = 0; q < 3; q++)
                    w[q] = fc[q] - fn[q] - (dv[q * 3 + 0] * x + dv[q * 3 + 1] * y + dv[q * 3 + 2] * z);
                t[OW + 0] = w[0]; t[OW + 1] = w[1]; t[OW + 2] = w[2];
                t[OW + 3] = w[0] * ux + w[1] * uy + w[2] * uz;
            }
        }
    }
}

// Sum over the pieces of a list (mtp_plan.h): the pieces sit in neighbouring lanes of one wavefront, `rem` is the
// number of pieces behind the lane's own in its list; after `steps` doubling steps the lane of a list's first piece
// holds the list's sum (pieces in a fixed tree order).  All 64 lanes take part.
template <typename T>
__device__ __forceinline__ T piece_sum(T v, int rem, int steps)
{
    for (int k = 0; k < steps; k++) {
        const int d = 1 << k;
        const T o = __shfl_down(v, d, 64);
        v += rem >= d ? o : (T)0;
    }
    return v;
}

// A plan term names its two moments by byte offsets into an array of doubles (index * 8): no shift between the
// word and the LDS address in fp64.
template <typename T>
__device__ __forceinline__ T plan_entry(const T* base, unsigned off)
{
    return *(const T*)((const char*)base + (sizeof(T) == 8 ? off : off >> 1));
}

// forward products: M[dst] = sum mult M[m0] M[m1]; with TANGENT also the product rule on Tg.
template <typename T, bool TANGENT, int NT>
__device__ __forceinline__ void sweep_forward(const MtpPlanDevice& p, T* M, T* Tg, int tid)
{
    for (int l = 0; l < p.n_levels; l++) {
        const int s0 = p.f_level[l], s1 = p.f_level[l + 1];     // whole groups of 64 slots: every lane of a wave walks one
        for (int s = s0 + tid; s < s1; s += NT) {
            const int grp = __builtin_amdgcn_readfirstlane(s >> 6);     // the wavefront's group: scalar loads below
            const int steps = p.f_multi[grp];                // of the group: only groups with cut lists pay for the sums
            const int depth = p.f_gdepth[grp];               // shared by the 64 lanes of the group, a multiple of MTP_DEPTH_STEP
            const int2* tp = p.f_terms + p.f_gbase[grp] + (s & 63);
            const int dst = p.f_dst[s];                      // requested with the two words above
            const int rem = steps ? p.f_rem[s] : 0;
            T acc = (T)0, tacc = (T)0;
            // all the slot's words (at most MTP_SLOT_CAP, the depth is shared by the wavefront) are requested
            // before the first is used: one trip to memory per slot
            int2 w[MTP_SLOT_CAP];
#pragma unroll
            for (int k = 0; k < MTP_SLOT_CAP; k += MTP_DEPTH_STEP)
                if (k < depth) {
#pragma unroll
                    for (int u = 0; u < MTP_DEPTH_STEP; u++) w[k + u] = tp[(k + u) * 64];
                }
#pragma unroll
            for (int k = 0; k < MTP_SLOT_CAP; k += MTP_DEPTH_STEP)
                if (k < depth) {
#pragma unroll
                    for (int u = k; u < k + MTP_DEPTH_STEP; u++) {
                        const unsigned m0 = (unsigned)w[u].x & 0xffffu, m1 = (unsigned)w[u].x >> 16;
                        const T mult = (T)w[u].y;
                        const T v0 = plan_entry(M, m0), v1 = plan_entry(M, m1);
                        acc += mult * v0 * v1;
                        if (TANGENT) tacc += plan_entry(Tg, m0) * mult * v1 + plan_entry(Tg, m1) * mult * v0;
                    }
                }
            if (steps) {
                acc = piece_sum(acc, rem, steps);
                if (TANGENT) tacc = piece_sum(tacc, rem, steps);
            }
            if (dst >= 0) {                                  // the first piece of a list
                M[dst] = acc;
                if (TANGENT) Tg[dst] = tacc;
            }
        }
        __syncthreads();
    }
}

// reverse gather: X[m] += sum mult (X[dst] M[other] (+ A[dst] Tg[other] when MIXED))
template <typename T, bool MIXED, int NT>
__device__ __forceinline__ void sweep_reverse(const MtpPlanDevice& p, const T* M, T* X, const T* A,
                                              const T* Tg, int tid)
{
    for (int l = p.n_levels - 1; l >= 0; l--) {
        const int s0 = p.r_level[l], s1 = p.r_level[l + 1];
        for (int s = s0 + tid; s < s1; s += NT) {
            const int grp = __builtin_amdgcn_readfirstlane(s >> 6);
            const int steps = p.r_multi[grp];
            const int depth = p.r_gdepth[grp];
            const int2* tp = p.r_terms + p.r_gbase[grp] + (s & 63);
            const int src = p.r_src[s];
            const int rem = steps ? p.r_rem[s] : 0;
            T acc = (T)0;
            int2 w[MTP_SLOT_CAP];
#pragma unroll
            for (int k = 0; k < MTP_SLOT_CAP; k += MTP_DEPTH_STEP)
                if (k < depth) {
#pragma unroll
                    for (int u = 0; u < MTP_DEPTH_STEP; u++) w[k + u] = tp[(k + u) * 64];
                }
#pragma unroll
            for (int k = 0; k < MTP_SLOT_CAP; k += MTP_DEPTH_STEP)
                if (k < depth) {
#pragma unroll
                    for (int u = k; u < k + MTP_DEPTH_STEP; u++) {
                        const unsigned dst = (unsigned)w[u].x & 0xffffu, other = (unsigned)w[u].x >> 16;
                        const T mult = (T)w[u].y;
                        acc += plan_entry(X, dst) * mult * plan_entry(M, other);
                        if (MIXED) acc += mult * plan_entry(A, dst) * plan_entry(Tg, other);
                    }
                }
            if (steps) acc = piece_sum(acc, rem, steps);
            if (src >= 0) X[src] += acc;
        }
        __syncthreads();
    }
}

// sum over the NT threads of a workgroup in a fixed order (wave sums, then wave 0 .. last)
template <typename T, int NT>
__device__ __forceinline__ T block_sum(T v, T* scratch, int tid)
{
    v = wave_sum(v);
    if (NT == 64) return v;
    __syncthreads();
    if ((tid & 63) == 0) scratch[tid >> 6] = v;
    __syncthreads();
    T t = (T)0;
#pragma unroll
    for (int w = 0; w < NT / 64; w++) t += scratch[w];
    return t;
}

// Pair derivatives of one neighbour by a walk over the monomial rows (mtp_plan.h): the lane owns the
// neighbour whose table row is `t`, takes rows h, h + ng, ... and returns its share of
//   gs = sum_i adj_i m_i (g' - k g / r),   w = sum_i adj_i g grad_u m_i,
// with  c_q = sum_mu AD[q][mu] g_mu  and  d_q = sum_mu AD[q][mu] g'_mu  formed once per monomial:
//   gs += m_q (d_q - k_q c_q / r),  w_x += c_q a x^(a-1) y^b z^c,  w_y += c_q b x^a y^(b-1) z^c,
//   w_z += c_q c x^a y^b z^(c-1).
template <typename T, int NMP>
__device__ __forceinline__ void pair_walk(const T* __restrict__ t, const T* __restrict__ AD, const int* __restrict__ rows,
                                          int nrows, int h, int ng, int kmax, int nmus, int OX, int OY, int OZ, int OG,
                                          int ODG, T rinv, T& gs, T& wx, T& wy, T& wz)
{
    T g[NMP], dg[NMP];
#pragma unroll
    for (int mu = 0; mu < NMP; mu++) {
        g[mu] = mu < nmus ? t[OG + mu] : (T)0;
        dg[mu] = mu < nmus ? t[ODG + mu] : (T)0;
    }
    const T z = t[OZ + 1];
    for (int r = h; r < nrows; r += ng) {
        const int rw = rows[r];
        const int ea = rw & 255, eb = (rw >> 8) & 255;
        const int len = kmax - ea - eb + 1;
        const T xa = t[OX + ea], yb = t[OY + eb];
        const T xy = xa * yb;
        const T Wx = (T)ea * t[OX + max(ea - 1, 0)] * yb;
        const T Wy = (T)eb * xa * t[OY + max(eb - 1, 0)];
        const T* ad = AD + (size_t)(rw >> 16) * NMP;
        T zc = (T)1, zcm = (T)0, kf = (T)(ea + eb), cf = (T)0;
        for (int c = 0; c < len; c++) {
            T cq = (T)0, dq = (T)0;
#pragma unroll
            for (int mu = 0; mu < NMP; mu++) {
                const T v = ad[mu];
                cq += v * g[mu];
                dq += v * dg[mu];
            }
            gs += xy * zc * (dq - kf * cq * rinv);
            const T cz = cq * zc;
            wx += cz * Wx;
            wy += cz * Wy;
            wz += cq * cf * zcm * xy;
            zcm = zc; zc *= z; kf += (T)1; cf += (T)1;
            ad += NMP;
        }
    }
}

// NT threads per centre atom: 64 for small tables, 256 when there is enough work per atom
// (four workgroups of 256 threads fit the LDS of a CU at the larger levels: keep the registers to match)
// SEED: the instance of the energy / force / virial kernel that can start its adjoint sweep from per-row weights
// (row_seed, pair_out); the loss-gradient kernel tests the pointer at run time.
template <typename T, bool LOSS, int NT, bool SEED = false>
__global__ void __launch_bounds__(NT, (!LOSS ? 4 : 1)) mtp_atom_kernel(const MtpArgs<T> a)
{
    const bool seeded = (SEED || LOSS) && a.row_seed != nullptr;
    const bool no_tan = LOSS && a.no_tangent != 0;      // uniform over the launch
    extern __shared__ __align__(16) unsigned char smem_raw[];
    const MtpPlanDevice& p = a.p;
    const int lane = threadIdx.x;     // thread in the workgroup
    const int ii = blockIdx.x, b = blockIdx.y;
    const int NF = a.P + a.nghost;
    const size_t row = (size_t)b * a.P + ii;
    const int n_moms = p.n_moms, n_basic = p.n_basic, nmus = p.nmus, kmax = p.kmax, K = a.K, E = a.E;
    const int OX = 0, OY = kmax + 1, OZ = 2 * (kmax + 1), OG = 3 * (kmax + 1), ODG = OG + nmus,
              OU = ODG + nmus, OW = OU + 4, OF = OW + 4, ODF = OF + K;
    const int ncoef = a.ntypes * a.ntypes * nmus * K;

    const int MTP_NC = a.nc_cap;
    // moments | (loss mode: their tangents) | coefficients | region of the neighbour table
    T* M = (T*)smem_raw;
    T* Tg = M + n_moms;
    T* cf = Tg + (LOSS ? n_moms : 0);        // coefficients of the centre species: [ntypes][nmus][K]
    T* tab = cf + a.ntypes * nmus * K;
    // the adjoints (loss mode: and the mixed adjoints) share the table's region, behind the sweeps' partial sums
    const bool keep = !LOSS && a.keep_table != 0;       // uniform over the launch
    T* A = tab + (keep ? mtp_table_entries(MTP_NC, E, LOSS, n_moms, NT) : mtp_adjoint_offset((LOSS ? 2 : 1) * p.max_level_slots));
    T* Bm = A + n_moms;
    // [256/32][32][4] partial sums of the thread groups.  They are needed only in the last pass over the
    // neighbours, when the moments (and, in loss mode, their tangents) are dead: a long enough moment
    // vector lends them its place
    const bool share = mtp_gred_in_moments(LOSS, n_moms);
    // energy / force / virial kernel: the group sums are written over the table once it has been read
    T* gred = LOSS ? (share ? M : tab + MTP_NC * E) : tab;
    // loss mode, behind the region: adjoints and mixed adjoints of the basic moments (copies for the last pass) |
    // P[nc][nmus] | Q[nc][nmus] | ...
    T* Ab = tab + mtp_table_region(MTP_NC, E, LOSS, n_moms, p.max_level_slots, NT, keep);
    T* Bb = Ab + n_basic;
    T* pq = LOSS ? Bb + n_basic : Ab;

    if (ii >= a.binum[b]) {                  // padded row: contributes nothing
        if (!LOSS && a.partial && lane < 10) a.partial[row * 10 + lane] = 0.0;
        if (!LOSS && a.e_sites && lane == 0) a.e_sites[row] = (T)0;
        if (!LOSS && a.desc)
            for (int s = lane; s < p.n_scalar; s += NT) a.desc[row * p.n_scalar + s] = (T)0;
        if (LOSS)
            for (int q = lane; q < a.ngrad; q += NT) a.gpart[row * a.ngrad + q] = (T)0;
        return;
    }
    int center = a.bilist[row];
    int nn = a.bnumneigh[row];
    if (nn > a.U) { if (lane == 0) atomicOr(a.status, ST_NEIGH_OVERFLOW); nn = a.U; }
    if ((unsigned)center >= (unsigned)NF) { if (lane == 0) atomicOr(a.status, ST_BAD_NEIGHBOR); center = 0; nn = 0; }
    const int* types = a.btypes + (size_t)b * NF;
    int ti = types[center];
    if ((unsigned)ti >= (unsigned)a.ntypes) { if (lane == 0) atomicOr(a.status, ST_BAD_TYPE); ti = 0; nn = 0; }
    const int* first = a.bfirstneigh + row * a.U;
    const T* rcs = a.brcs + row * a.U * 3;

    // (mu, a, b, c) of every basic moment, one byte each, behind everything else in LDS
    unsigned* bas = (unsigned*)(smem_raw + a.lds_basic_off);
    for (int i = lane; i < n_basic; i += NT)
        bas[i] = (unsigned)p.basic[i * 4] | ((unsigned)p.basic[i * 4 + 1] << 8) |
                 ((unsigned)p.basic[i * 4 + 2] << 16) | ((unsigned)p.basic[i * 4 + 3] << 24);
    int* rws = (int*)(bas + n_basic);        // monomial rows of the pair-derivative walk
    if (!LOSS) {
        for (int i = lane; i < p.nrows; i += NT) rws[i] = p.rows[i];
    }
    for (int q = lane; q < a.ntypes * nmus * K; q += NT) cf[q] = a.coeffs[(size_t)ti * a.ntypes * nmus * K + q];
    for (int i = lane; i < n_moms; i += NT) {
        M[i] = (T)0;
        if (LOSS) Tg[i] = (T)0;
    }
    __syncthreads();

    // ---- basic moments (and their tangents) --------------------------------------------------
    const int chunk = nn > 0 ? (nn + (nn + MTP_NC - 1) / MTP_NC - 1) / ((nn + MTP_NC - 1) / MTP_NC) : 1;
    for (int c0 = 0; c0 < nn; c0 += chunk) {
        const int nc = min(chunk, nn - c0);
        int nj; bool valid; T d[3];
        build_table<T, LOSS, NT>(a, tab, cf, lane, nc, c0, rcs, first, types, center, b, NF, &nj, &valid, d);
        __syncthreads();
        for (int i = lane; i < n_basic; i += NT) {
            const unsigned bw = bas[i];
            const int mu = bw & 255, ea = (bw >> 8) & 255, eb = (bw >> 16) & 255, ec = bw >> 24;
            const T kk = (T)(ea + eb + ec);
            T acc = (T)0, tacc = (T)0;
            for (int j = 0; j < nc; j++) {
                const T* t = tab + j * E;
                const T g = t[OG + mu];
                const T xa = t[OX + ea], yb = t[OY + eb], zc = t[OZ + ec];
                const T m = xa * yb * zc;
                acc += g * m;
                if (LOSS && !no_tan) {
                    const T dg = t[ODG + mu], rinv = t[OU + 3], wu = t[OW + 3];
                    const T gm = (T)ea * t[OX + max(ea - 1, 0)] * yb * zc * t[OW + 0] +
                                 (T)eb * xa * t[OY + max(eb - 1, 0)] * zc * t[OW + 1] +
                                 (T)ec * xa * yb * t[OZ + max(ec - 1, 0)] * t[OW + 2];
                    tacc += wu * m * (dg - kk * g * rinv) + g * rinv * gm;
                }
            }
            M[i] += acc;
            if (LOSS) Tg[i] += tacc;
        }
        __syncthreads();
    }

    // ---- products, energy, adjoint ------------------------------------------------------------
    if (LOSS && !no_tan) sweep_forward<T, LOSS, NT>(p, M, Tg, lane);
    else sweep_forward<T, false, NT>(p, M, Tg, lane);
    for (int i = lane; i < n_moms; i += NT) {    // the table is dead: its place now holds the adjoints
        A[i] = (T)0;
        if (LOSS) Bm[i] = (T)0;
    }
    __syncthreads();
    T e_part = (T)0;
    // network buffers (H > 0): inputs q[S]; per neuron w1 tanh', and in loss mode tanh, tanh', tanh'', tau
    T* nnb = LOSS ? pq + 2 * MTP_NC * nmus + MTP_NC + a.ntypes * nmus * K : pq;
    if (a.H > 0) {
        // one tanh layer of the centre's species on the shifted, scaled scalar moments; the
        // adjoint is seeded with dE_i/dM_k = sum_p w1_p tanh'(h_p) w0_pk / q_scaler_k
        // (nnMtp.h:470-507).  Loss mode also needs the derivative of that seed along the tangent:
        // tau_p = sum_k w0_pk Tg_k / q_scaler_k is the tangent of h_p, and the adjoint of
        // D_w E = sum_p w1_p tanh'(h_p) tau_p  w.r.t. M_k is  sum_p w1_p tanh''(h_p) tau_p w0_pk / q_scaler_k,
        // the seed of the mixed sweep (nnMtpLoss.h:216-610 computes the same quantities atom by atom).
        const int S = p.n_scalar, H = a.H;
        T* qv = nnb;                          // [S] network inputs
        T* hv = nnb + S;                      // [H] pre-activations, then w1 * tanh'
        T* n_th = hv + H;                     // loss mode: tanh, tanh', tanh'', tau   [H] each
        T* n_d1 = n_th + H;
        T* n_d2 = n_d1 + H;
        T* n_tau = n_d2 + H;
        const T* w0 = a.w0 + (size_t)ti * H * S;
        const T* w1 = a.w1 + (size_t)ti * H;
        for (int s = lane; s < S; s += NT) qv[s] = (M[p.mapping[s]] - a.q_shift[s]) / a.q_scaler[s];
        __syncthreads();
        for (int n = lane >> 6; n < H; n += NT / 64) {          // one wave per neuron
            T acc = (T)0, tac = (T)0;
            for (int k = lane & 63; k < S; k += 64) {
                acc += w0[(size_t)n * S + k] * qv[k];
                if (LOSS) tac += w0[(size_t)n * S + k] * Tg[p.mapping[k]] / a.q_scaler[k];
            }
            acc = wave_sum(acc);
            if (LOSS) tac = wave_sum(tac);
            if ((lane & 63) == 0) {
                hv[n] = acc;
                if (LOSS) n_tau[n] = tac;
            }
        }
        __syncthreads();
        for (int n = lane; n < H; n += NT) {
            const T th = tanh_t(hv[n]);
            const T d1 = (T)1 - th * th;
            e_part += w1[n] * th;
            hv[n] = w1[n] * d1;
            if (LOSS) { n_th[n] = th; n_d1[n] = d1; n_d2[n] = (T)-2 * th * d1; }
        }
        __syncthreads();
        for (int k = lane; k < S; k += NT) {
            T acc = (T)0, bac = (T)0;
            for (int n = 0; n < H; n++) {
                const T w = w0[(size_t)n * S + k];
                acc += hv[n] * w;
                if (LOSS) bac += w1[n] * n_d2[n] * n_tau[n] * w;
            }
            A[p.mapping[k]] = acc / a.q_scaler[k];
            if (LOSS && a.nn_exact) Bm[p.mapping[k]] = bac / a.q_scaler[k];
        }
    } else if (seeded) {
        for (int s = lane; s < p.n_scalar; s += NT) A[p.mapping[s]] = a.row_seed[row * p.n_scalar + s];
    } else {
        for (int s = lane; s < p.n_scalar; s += NT) {
            e_part += a.lin[s] * M[p.mapping[s]] / a.q_scaler[s];
            A[p.mapping[s]] = a.lin[s] / a.q_scaler[s];
        }
    }
    if (!LOSS && (a.e_sites || a.desc)) {
        if (a.desc)                                          // linearMtp.h:884-885: unscaled scalar moments
            for (int s = lane; s < p.n_scalar; s += NT) a.desc[row * p.n_scalar + s] = M[p.mapping[s]];
        const T e_row = block_sum<T, NT>(e_part, tab, lane) + a.bias[ti];      // the table is idle between the sweeps
        if (a.e_sites && lane == 0) a.e_sites[row] = e_row;  // linearMtp.h:594-599
        if (a.energy_only) return;
    }
    __syncthreads();
    sweep_reverse<T, false, NT>(p, M, A, nullptr, nullptr, lane);

    if (!LOSS) {
        // ---- pair derivatives ------------------------------------------------------------------
        // The adjoints of the basic moments, gathered by monomial (mtp_plan.h); the moments are dead
        T* AD = mtp_dense_in_moments(p.nq, p.nmp, n_moms) ? M : nnb + (a.H > 0 ? p.n_scalar + a.H : 0);
        __syncthreads();
        if (p.dense_unique) {
            for (int e = lane; e < p.nq * p.nmp; e += NT) AD[e] = (T)0;
            __syncthreads();
            for (int i = lane; i < n_basic; i += NT) AD[p.dense_pos[i]] = A[i];
        } else {
            for (int e = lane; e < p.nq * p.nmp; e += NT) {
                const int src = p.dense_src[e];
                T v = (T)0;
                if (src >= 0) v = A[src];
                else if (src == -2)
                    for (int q = p.dense_off[e]; q < p.dense_off[e + 1]; q++) v += A[p.dense_items[q]];
                AD[e] = v;
            }
        }
        // The row is cut into equal chunks of at most MTP_NC neighbours; within a chunk of nc
        // neighbours thread = group h * nc + neighbour j, and the groups (as many as fit, at most one
        // per monomial row) share the rows, so a short chunk still keeps the workgroup busy.
        T fx = (T)0, fy = (T)0, fz = (T)0;
        T vir[9];
#pragma unroll
        for (int q = 0; q < 9; q++) vir[q] = (T)0;
        const int nchunks = (nn + MTP_NC - 1) / MTP_NC;
        const int csize = nchunks > 0 ? (nn + nchunks - 1) / nchunks : 1;
        for (int c0 = 0; c0 < nn; c0 += csize) {
            const int nc = min(csize, nn - c0);
            const int ng = min(NT / nc, p.nrows);
            const int h = lane / nc, j = lane - h * nc;
            int nj; bool valid; T d[3] = {(T)0, (T)0, (T)0};
            __syncthreads();
            // (a row of one chunk finds the table of the first pass still in place when the adjoints lie behind it)
            build_table<T, false, NT>(a, tab, cf, lane, nc, c0, rcs, first, types, center, b, NF, &nj, &valid, d,
                                      !(keep && nchunks == 1));
            __syncthreads();
            T gs = (T)0, wx = (T)0, wy = (T)0, wz = (T)0;
            T ux = (T)0, uy = (T)0, uz = (T)0, rinv = (T)0;
            if (h < ng) {
                const T* t = tab + j * E;
                ux = t[OU + 0]; uy = t[OU + 1]; uz = t[OU + 2]; rinv = t[OU + 3];
                switch (p.nmp) {
                case 2: pair_walk<T, 2>(t, AD, rws, p.nrows, h, ng, kmax, nmus, OX, OY, OZ, OG, ODG, rinv, gs, wx, wy, wz); break;
                case 4: pair_walk<T, 4>(t, AD, rws, p.nrows, h, ng, kmax, nmus, OX, OY, OZ, OG, ODG, rinv, gs, wx, wy, wz); break;
                case 6: pair_walk<T, 6>(t, AD, rws, p.nrows, h, ng, kmax, nmus, OX, OY, OZ, OG, ODG, rinv, gs, wx, wy, wz); break;
                default: pair_walk<T, 8>(t, AD, rws, p.nrows, h, ng, kmax, nmus, OX, OY, OZ, OG, ODG, rinv, gs, wx, wy, wz); break;
                }
            }
            __syncthreads();            // every thread has read its table row: the group sums take its place
            // group sums in the order h = 0 .. ng-1
            {
                T* gr = gred + lane * 4;
                gr[0] = gs; gr[1] = wx; gr[2] = wy; gr[3] = wz;
            }
            __syncthreads();
            if (h == 0) {
                for (int hh = 1; hh < ng; hh++) {
                    const T* gr = gred + (hh * nc + j) * 4;
                    gs += gr[0]; wx += gr[1]; wy += gr[2]; wz += gr[3];
                }
            }
            if (h == 0) {
                T gx = gs * ux + wx * rinv;
                T gy = gs * uy + wy * rinv;
                T gz = gs * uz + wz * rinv;
                if (!valid) { gx = (T)0; gy = (T)0; gz = (T)0; }
                if (a.seg_cursor && j < nc) {
                    // the pair claims an entry of its target's segment (zeros too: the count of a segment
                    // is the number of pairs naming the target)
                    const int tg = b * NF + nj;
                    const int rk = atomicAdd(&a.seg_cursor[tg], 1);
                    T* dst = a.seg_g + (size_t)(rk < a.seg_cap ? tg * a.seg_cap + rk : a.seg_spare) * 3;
                    if (rk >= a.seg_cap) atomicOr(a.status, ST_SEG_OVERFLOW);
                    dst[0] = gx; dst[1] = gy; dst[2] = gz;
                }
                if (SEED && a.pair_out) {         // padded layout of brcs; entries beyond the row stay zero
                    T* dst = a.pair_out + (row * a.U + c0 + j) * 3;
                    dst[0] = gx; dst[1] = gy; dst[2] = gz;
                }
                fx += gx; fy += gy; fz += gz;
                vir[0] -= gx * d[0]; vir[1] -= gx * d[1]; vir[2] -= gx * d[2];
                vir[3] -= gy * d[0]; vir[4] -= gy * d[1]; vir[5] -= gy * d[2];
                vir[6] -= gz * d[0]; vir[7] -= gz * d[1]; vir[8] -= gz * d[2];
            }
        }
        // only the threads of group 0 (inside wave 0) hold force and virial terms: the other wavefronts are done
        const double e_atom = (double)block_sum<T, NT>(e_part, gred, lane);
        if (lane >= 64) return;
        fx = wave_sum(fx); fy = wave_sum(fy); fz = wave_sum(fz);
        double out[10];
        out[0] = e_atom + (seeded ? 0.0 : (double)a.bias[ti]);
#pragma unroll
        for (int q = 0; q < 9; q++) out[1 + q] = (double)wave_sum(vir[q]);
        if (lane == 0) {
            if (!SEED || a.force) {
                T* fo = a.force + ((size_t)b * NF + center) * 3;
                fo[0] = fx; fo[1] = fy; fo[2] = fz;
            }
            if (!SEED || a.partial) {
#pragma unroll
                for (int q = 0; q < 10; q++) a.partial[row * 10 + q] = out[q];
            }
        }
        return;
    }

    // ---- loss gradient ------------------------------------------------------------------------
    if (LOSS) {
        const T cE = seeded ? (T)1 : (a.cE_per_atom ? a.cE[row] : a.cE[b]);
        // linearMtpLoss.h:417-434; the reference's network backward has no such term (Bm stays zero)
        if (!no_tan && (a.H == 0 || a.nn_exact)) sweep_reverse<T, true, NT>(p, M, Bm, A, Tg, lane);
        // the last pass needs the adjoints of the basic moments while the table is back in its region
        for (int i = lane; i < n_basic; i += NT) { Ab[i] = A[i]; Bb[i] = Bm[i]; }
        T* grow = a.gpart + row * a.ngrad;
        for (int q = lane; q < a.ngrad; q += NT) grow[q] = (T)0;
        __syncthreads();         // other threads overwrite some of these entries below
        // everything but the coefficient block is written now: the pass over the neighbours below does
        // not read the moments or their tangents, and the group sums may take their place
        if (a.H > 0) {
            // compact row of the centre species: coefficient block | w0[H, S] | w1[H] | bias
            const int S = p.n_scalar, H = a.H, nblk = a.ntypes * nmus * K;
            const T* qv = nnb;
            const T* n_th = nnb + S + H;
            const T* n_d1 = n_th + H;
            const T* n_d2 = n_d1 + H;
            const T* n_tau = n_d2 + H;
            const T* w1 = a.w1 + (size_t)ti * H;
            const T* w0 = a.w0 + (size_t)ti * H * S;
            for (int q = lane; q < H * S; q += NT) {
                const int n = q / S, k = q - n * S;
                const T tk = Tg[p.mapping[k]] / a.q_scaler[k];
                if (a.nn_exact)
                    grow[nblk + q] = w1[n] * ((cE * n_d1[n] + n_d2[n] * n_tau[n]) * qv[k] + n_d1[n] * tk);
                else        // nnMtpLoss.h:560-585: only the k' = k term of tau
                    grow[nblk + q] = w1[n] * (cE * n_d1[n] * qv[k] + tk * (n_d1[n] + n_d2[n] * w0[q] * qv[k]));
            }
            for (int n = lane; n < H; n += NT) grow[nblk + H * S + n] = cE * n_th[n] + n_d1[n] * n_tau[n];
            if (lane == 0) grow[nblk + H * S + H] = cE;
        } else if (!seeded) {
            // linear coefficients and bias: linearMtpLoss.h:539-554
            for (int s = lane; s < p.n_scalar; s += NT)
                grow[ncoef + s] = (cE * M[p.mapping[s]] + Tg[p.mapping[s]]) / a.q_scaler[s];
            if (lane == 0) grow[ncoef + p.n_scalar + ti] = cE;
        }
        T* Pm = pq;
        T* Qm = pq + MTP_NC * nmus;
        int* tjs = (int*)(pq + 2 * MTP_NC * nmus);
        T* gacc = pq + 2 * MTP_NC * nmus + MTP_NC;          // [ntypes][nmus][K] for this centre type
        for (int q = lane; q < a.ntypes * nmus * K; q += NT) gacc[q] = (T)0;
        const int nchunks = (nn + MTP_NC - 1) / MTP_NC;
        const int csize = nchunks > 0 ? (nn + nchunks - 1) / nchunks : 1;
        for (int c0 = 0; c0 < nn; c0 += csize) {
            // equal chunks and as many thread groups per chunk as fit, as in the pair-derivative pass
            const int nc = min(csize, nn - c0);
            const int ng = min(NT / nc, MTP_NGMAX);
            const int h = lane / nc, j = lane - h * nc;
            int nj; bool valid; T d[3];
            __syncthreads();
            build_table<T, true, NT>(a, tab, cf, lane, nc, c0, rcs, first, types, center, b, NF, &nj, &valid, d);
            __syncthreads();
            // P_mu(j), Q_mu(j): linearMtpLoss.h:438-536 with the k-sum factored out
            for (int mu = 0; mu < nmus; mu++) {
                T Pv = (T)0, Qv = (T)0;
                if (h < ng) {
                    const T* t = tab + j * E;
                    const T rinv = t[OU + 3], wu = t[OW + 3];
                    for (int i = p.mu_begin[mu] + h; i < p.mu_begin[mu + 1]; i += ng) {
                        const unsigned bw = bas[i];
                        const int ea = (bw >> 8) & 255, eb = (bw >> 16) & 255, ec = bw >> 24;
                        const T xa = t[OX + ea], yb = t[OY + eb], zc = t[OZ + ec];
                        const T m = xa * yb * zc;
                        const T adj = Ab[i];
                        if (no_tan) {                 // w = 0: only the energy term is left
                            Pv += cE * adj * m;
                            continue;
                        }
                        const T gm = (T)ea * t[OX + max(ea - 1, 0)] * yb * zc * t[OW + 0] +
                                     (T)eb * xa * t[OY + max(eb - 1, 0)] * zc * t[OW + 1] +
                                     (T)ec * xa * yb * t[OZ + max(ec - 1, 0)] * t[OW + 2];
                        Pv += (cE * adj + Bb[i]) * m + adj * rinv * (gm - (T)(ea + eb + ec) * m * wu);
                        Qv += adj * m * wu;
                    }
                }
                {
                    T* gr = gred + lane * 2;
                    gr[0] = Pv; gr[1] = Qv;
                }
                __syncthreads();
                if (h == 0) {
                    for (int hh = 1; hh < ng; hh++) {
                        const T* gr = gred + (hh * nc + j) * 2;
                        Pv += gr[0]; Qv += gr[1];
                    }
                    Pm[j * nmus + mu] = Pv; Qm[j * nmus + mu] = Qv;
                }
                __syncthreads();
            }
            // tj of each neighbour of the chunk, for the accumulation below
            if (h == 0) tjs[j] = valid ? types[nj] : -1;
            __syncthreads();
            // lanes <- (mu, k): sequential over neighbours keeps the sum order fixed
            for (int q = lane; q < nmus * K; q += NT) {
                const int mu = q / K, k = q - mu * K;
                for (int jn = 0; jn < nc; jn++) {
                    const int tj = tjs[jn];
                    if (tj < 0) continue;
                    const T* t = tab + jn * E;
                    gacc[tj * nmus * K + q] += t[OF + k] * Pm[jn * nmus + mu] + t[ODF + k] * Qm[jn * nmus + mu];
                }
            }
        }
        __syncthreads();
        if (a.H > 0) {
            for (int q = lane; q < a.ntypes * nmus * K; q += NT) grow[q] = gacc[q];
            return;
        }
        for (int q = lane; q < a.ntypes * nmus * K; q += NT)
            grow[(size_t)ti * a.ntypes * nmus * K + q] = gacc[q];
    }
}

// out[b, q] = sum over atoms ii < binum[b] of gpart[b, ii, q], in atom order
template <typename T>
__global__ void __launch_bounds__(256)
mtp_grad_reduce_kernel(int P, int ncoef, int nlin, int nbias, const int* __restrict__ binum,
                       const T* __restrict__ gpart, T* __restrict__ dcoeffs, T* __restrict__ dlin,
                       T* __restrict__ dbias)
{
    const int b = blockIdx.y;
    const int ngrad = ncoef + nlin + nbias;
    const int q = blockIdx.x * 256 + threadIdx.x;
    if (q >= ngrad) return;
    const int inum = binum[b];
    T acc = (T)0;
    const T* src = gpart + (size_t)b * P * ngrad + q;
    int ii = 0;
    for (; ii + 8 <= inum; ii += 8) {            // eight rows in flight, added in atom order
        T v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) v[u] = src[(size_t)(ii + u) * ngrad];
#pragma unroll
        for (int u = 0; u < 8; u++) acc += v[u];
    }
    for (; ii < inum; ii++) acc += src[(size_t)ii * ngrad];
    if (q < ncoef) { if (dcoeffs) dcoeffs[(size_t)b * ncoef + q] = acc; }
    else if (q < ncoef + nlin) { if (dlin) dlin[(size_t)b * nlin + q - ncoef] = acc; }
    else if (dbias) dbias[(size_t)b * nbias + q - ncoef - nlin] = acc;
}

// The same for the compact rows of the neural-network MTP: row = [coefficient block of the centre
// species | w0[H, S] | w1[H] | bias]; out[b] is laid out coeffs[ntypes^2 nmus K] | w0[ntypes H S] |
// w1[ntypes H] | bias[ntypes].  Thread q of block (x, t, b) sums entry q of the rows of species t.
template <typename T>
__global__ void __launch_bounds__(256)
nnmtp_grad_reduce_kernel(int P, int NF, int nblk, int HS, int H, int ntypes, const int* __restrict__ binum,
                         const int* __restrict__ bilist, const int* __restrict__ btypes,
                         const T* __restrict__ gpart, T* __restrict__ dcoeffs, T* __restrict__ dw0,
                         T* __restrict__ dw1, T* __restrict__ dbias)
{
    const int b = blockIdx.z, t = blockIdx.y;
    const int nrow = nblk + HS + H + 1;
    const int q = blockIdx.x * 256 + threadIdx.x;
    if (q >= nrow) return;
    const int inum = binum[b];
    T acc = (T)0;
    // eight rows in flight; the rows of other species are skipped, the order of the sum is the atom order
    for (int i0 = 0; i0 < inum; i0 += 8) {
        int c[8], ty[8];
        T v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) c[u] = bilist[(size_t)b * P + min(i0 + u, inum - 1)];
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const bool ok = i0 + u < inum && (unsigned)c[u] < (unsigned)NF;
            ty[u] = btypes[(size_t)b * NF + (ok ? c[u] : 0)];
            if (!ok) ty[u] = -1;
        }
#pragma unroll
        for (int u = 0; u < 8; u++) {            // (a row of another species is not read)
            v[u] = (T)0;
            if (ty[u] == t) v[u] = gpart[((size_t)b * P + min(i0 + u, inum - 1)) * nrow + q];
        }
#pragma unroll
        for (int u = 0; u < 8; u++) acc += v[u];
    }
    if (q < nblk) { if (dcoeffs) dcoeffs[((size_t)b * ntypes + t) * nblk + q] = acc; }
    else if (q < nblk + HS) { if (dw0) dw0[((size_t)b * ntypes + t) * HS + q - nblk] = acc; }
    else if (q < nblk + HS + H) { if (dw1) dw1[((size_t)b * ntypes + t) * H + q - nblk - HS] = acc; }
    else if (dbias) dbias[(size_t)b * ntypes + t] = acc;
}

// dst[(i * ncols) + col] = src[i] for i < n: one column of a row-major matrix
template <typename T>
__global__ void __launch_bounds__(256)
column_store_kernel(T* __restrict__ dst, const T* __restrict__ src, long long n, int ncols, int col)
{
    const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    if (i < n) dst[i * ncols + col] = src[i];
}

// ---- linear-solver components, all scalar moments in one pass ------------------------------------------------
// Column s of the components is the E/F/V of the read-out e_s / q_scaler[s].  Its adjoint is non-zero on the
// ancestors of scalar moment s only (15 of 350 moments on average at level 16, 25 of 1352 at level 20), so the adjoints
// of all columns together are one reverse gather over the nodes (scalar moment, ancestor) of the plan, about as
// long as one ordinary reverse sweep, and a pair derivative sums over the basic ancestors of its column only.
// The kernel computes the moments once per atom, runs that gather, and writes the pair derivatives of every column
// to pb[pair][3][slots]; the kernels below add them up per atom (own pairs minus the pairs that name the atom, the
// latter in the fixed order of a sorted list) and per structure.
template <typename T>
struct CompArgs {
    T* pb;                  // [pairs, 3, n_scalar]
    const int* pair_off;    // [rows + 1] first pair of each row
    const int* nnc;         // [rows] checked neighbour count of each row (0 for rows that are not evaluated)
    T* desc;                // [rows, n_scalar] scalar moments
    T* rowpart;             // [rows, 12, n_scalar] per row and column: sum of the pair derivatives (3), virial (9)
    int nc_cap, lds_basic_off;
};

template <typename T, int NT>
__global__ void __launch_bounds__(NT) mtp_components_kernel(const MtpArgs<T> a, const CompArgs<T> c)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    const MtpPlanDevice& p = a.p;
    const int lane = threadIdx.x;
    const int ii = blockIdx.x, b = blockIdx.y;
    const int NF = a.P;
    const size_t row = (size_t)b * a.P + ii;
    const int n_moms = p.n_moms, n_basic = p.n_basic, nmus = p.nmus, kmax = p.kmax, K = a.K, E = a.E;
    const int OX = 0, OY = kmax + 1, OZ = 2 * (kmax + 1), OG = 3 * (kmax + 1), ODG = OG + nmus, OU = ODG + nmus;
    const int S = p.n_scalar;
    // moments | node adjoints (+ the zero entry) | coefficients | neighbour table
    T* M = (T*)smem_raw;
    T* X = M + n_moms;
    T* cf = X + ((p.x_nodes + 2) & ~1);
    T* tab = cf + a.ntypes * nmus * K;
    unsigned* bas = (unsigned*)(smem_raw + c.lds_basic_off);
    const int nn = c.nnc[row];
    if (ii >= a.binum[b] || nn == 0) {                       // padded or refused row (k_rows flags the reasons)
        for (int s = lane; s < S; s += NT) c.desc[row * S + s] = (T)0;
        for (int q = lane; q < 12 * S; q += NT) c.rowpart[row * 12 * S + q] = (T)0;
        return;
    }
    int center = a.bilist[row];
    if ((unsigned)center >= (unsigned)NF) center = 0;
    const int* types = a.btypes + (size_t)b * NF;
    int ti = types[center];
    if ((unsigned)ti >= (unsigned)a.ntypes) ti = 0;
    const int* first = a.bfirstneigh + row * a.U;
    const T* rcs = a.brcs + row * a.U * 3;
    for (int i = lane; i < n_basic; i += NT)
        bas[i] = (unsigned)p.basic[i * 4] | ((unsigned)p.basic[i * 4 + 1] << 8) |
                 ((unsigned)p.basic[i * 4 + 2] << 16) | ((unsigned)p.basic[i * 4 + 3] << 24);
    for (int q = lane; q < a.ntypes * nmus * K; q += NT) cf[q] = a.coeffs[(size_t)ti * a.ntypes * nmus * K + q];
    for (int i = lane; i < n_moms; i += NT) M[i] = (T)0;
    for (int i = lane; i <= p.x_nodes; i += NT) X[i] = (T)0;
    __syncthreads();

    // basic moments (as in mtp_atom_kernel)
    const int MTP_NC = c.nc_cap;
    const int nchunks = (nn + MTP_NC - 1) / MTP_NC;
    const int chunk = nchunks > 0 ? (nn + nchunks - 1) / nchunks : 1;
    for (int c0 = 0; c0 < nn; c0 += chunk) {
        const int nc = min(chunk, nn - c0);
        int nj; bool valid; T d[3];
        build_table<T, false, NT>(a, tab, cf, lane, nc, c0, rcs, first, types, center, b, NF, &nj, &valid, d);
        __syncthreads();
        for (int i = lane; i < n_basic; i += NT) {
            const unsigned bw = bas[i];
            const int mu = bw & 255, ea = (bw >> 8) & 255, eb = (bw >> 16) & 255, ec = bw >> 24;
            T acc = (T)0;
            for (int j = 0; j < nc; j++) {
                const T* t = tab + j * E;
                acc += t[OG + mu] * (t[OX + ea] * t[OY + eb] * t[OZ + ec]);
            }
            M[i] += acc;
        }
        __syncthreads();
    }
    sweep_forward<T, false, NT>(p, M, (T*)nullptr, lane);
    for (int s = lane; s < S; s += NT) {
        c.desc[row * S + s] = M[p.mapping[s]];
        if (p.x_root[s] >= 0) X[p.x_root[s]] = (T)1 / a.q_scaler[s];       // (the columns of this launch)
    }
    __syncthreads();
    {
        MtpPlanDevice px = p;              // the reverse gather over the nodes
        px.r_level = p.x_level; px.r_multi = p.x_multi; px.r_src = p.x_src; px.r_rem = p.x_rem;
        px.r_gbase = p.x_gbase; px.r_gdepth = p.x_gdepth; px.r_terms = p.x_terms;
        sweep_reverse<T, false, NT>(px, M, X, (const T*)nullptr, (const T*)nullptr, lane);
    }

    // Pair derivatives.  A wavefront takes a neighbour j: its lanes first form, for every basic moment, the vector
    //   D_b = d(g_mu x^a y^b z^c)/dr_j = m (g' - k g / r) u + g / r grad_u m
    // from the neighbour's table row into the wavefront's own LDS buffer; then a lane owns a column and sums
    // adj * D_b over the column's basic ancestors (three reads and three FMAs per ancestor).  The own-row sums of the
    // columns (force of the centre, virial) are kept per lane and added over the wavefronts at the end.
    const int ngroups = p.x_slots >> 6;
    const int l64 = lane & 63, wv = lane >> 6;
    T* D = tab + (size_t)c.nc_cap * E + (size_t)wv * n_basic * 3;
    for (int c0 = 0; c0 < nn; c0 += chunk) {
        const int nc = min(chunk, nn - c0);
        if (nchunks > 1) {                                  // (a single chunk's table is still in place)
            int nj; bool valid; T d[3];
            __syncthreads();
            build_table<T, false, NT>(a, tab, cf, lane, nc, c0, rcs, first, types, center, b, NF, &nj, &valid, d);
            __syncthreads();
        }
        for (int j = wv; j < nc; j += NT / 64) {
            const T* t = tab + j * E;
            const T ux = t[OU + 0], uy = t[OU + 1], uz = t[OU + 2], rinv = t[OU + 3];
            __builtin_amdgcn_wave_barrier();               // the last neighbour's sums have read D
            for (int i = l64; i < n_basic; i += 64) {
                const unsigned bw = bas[i];
                const int mu = bw & 255, ea = (bw >> 8) & 255, eb = (bw >> 16) & 255, ec = bw >> 24;
                const T gm = t[OG + mu], dg = t[ODG + mu];
                const T xa = t[OX + ea], yb = t[OY + eb], zc = t[OZ + ec];
                const T gs = xa * yb * zc * (dg - (T)(ea + eb + ec) * gm * rinv);
                const T gr = gm * rinv;
                D[i * 3 + 0] = gs * ux + gr * ((T)ea * t[OX + max(ea - 1, 0)] * yb * zc);
                D[i * 3 + 1] = gs * uy + gr * ((T)eb * xa * t[OY + max(eb - 1, 0)] * zc);
                D[i * 3 + 2] = gs * uz + gr * ((T)ec * xa * yb * t[OZ + max(ec - 1, 0)]);
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            for (int g = 0; g < ngroups; g++) {
                const int depth = p.x_bdepth[g], steps = p.x_bsteps[g];
                const int* wp = p.x_bwords + p.x_bbase[g] + l64;
                const int col = p.x_seed[g * 64 + l64];
                T gx = (T)0, gy = (T)0, gz = (T)0;
                // all words of the slot (at most MTP_SLOT_CAP; the depth is a multiple of four and shared by the
                // wavefront) are requested before the first is used
                int w[MTP_SLOT_CAP];
#pragma unroll
                for (int k = 0; k < MTP_SLOT_CAP; k += 4)
                    if (k < depth) {
#pragma unroll
                        for (int u = 0; u < 4; u++) w[k + u] = wp[(k + u) * 64];
                    }
#pragma unroll
                for (int k = 0; k < MTP_SLOT_CAP; k += 4)
                    if (k < depth) {
#pragma unroll
                        for (int u = k; u < k + 4; u++) {
                            const T adj = X[(unsigned)w[u] & 0xffffu];
                            const T* dv = D + ((unsigned)w[u] >> 16) * 3;
                            gx += adj * dv[0]; gy += adj * dv[1]; gz += adj * dv[2];
                        }
                    }
                if (steps) {                                // a long list's pieces sit in neighbouring lanes
                    const int rem = p.x_brem[g * 64 + l64];
                    gx = piece_sum(gx, rem, steps); gy = piece_sum(gy, rem, steps); gz = piece_sum(gz, rem, steps);
                }
                if (col >= 0) {
                    T* dst = c.pb + ((size_t)(c.pair_off[row] + c0 + j) * 3) * S + col;
                    dst[0] = gx;
                    dst[S] = gy;
                    dst[2 * S] = gz;
                }
            }
        }
    }
    // own-row sums of every column (force of the centre, virial), in neighbour order, from the pair derivatives this
    // workgroup has just written: rowpart[row][12][S]
    __syncthreads();
    for (int q = lane; q < S; q += NT) {
        if (p.x_root[q] < 0) continue;                      // a column of another launch
        T f[3] = {(T)0, (T)0, (T)0}, v[9];
#pragma unroll
        for (int i = 0; i < 9; i++) v[i] = (T)0;
        const T* g = c.pb + (size_t)c.pair_off[row] * 3 * S + q;
        for (int j = 0; j < nn; j++) {
            const T gx = g[0], gy = g[S], gz = g[2 * S];
            const T dx = rcs[j * 3], dy = rcs[j * 3 + 1], dz = rcs[j * 3 + 2];
            f[0] += gx; f[1] += gy; f[2] += gz;
            v[0] -= gx * dx; v[1] -= gx * dy; v[2] -= gx * dz;
            v[3] -= gy * dx; v[4] -= gy * dy; v[5] -= gy * dz;
            v[6] -= gz * dx; v[7] -= gz * dy; v[8] -= gz * dz;
            g += 3 * (size_t)S;
        }
        T* o = c.rowpart + row * 12 * S + q;
#pragma unroll
        for (int i = 0; i < 3; i++) o[(size_t)i * S] = f[i];
#pragma unroll
        for (int i = 0; i < 9; i++) o[(size_t)(3 + i) * S] = v[i];
    }
}

// rows that the components kernel evaluates, with the checks of mtp_atom_kernel; row_of1[b, atom] = 1 + the row whose
// centre the atom is
__global__ void __launch_bounds__(256)
comp_rows_kernel(int B, int P, int U, int ntypes, const int* __restrict__ binum, const int* __restrict__ bilist,
                 const int* __restrict__ bnumneigh, const int* __restrict__ btypes, int* __restrict__ nnc,
                 int* __restrict__ row_of1, int* __restrict__ status)
{
    const int row = blockIdx.x * 256 + threadIdx.x;
    if (row > B * P) return;
    if (row == B * P) { nnc[row] = 0; return; }
    const int b = row / P, ii = row - b * P;
    int nn = 0;
    if (ii < binum[b]) {
        nn = bnumneigh[row];
        if (nn > U) { atomicOr(status, ST_NEIGH_OVERFLOW); nn = U; }
        if (nn < 0) nn = 0;
        const int center = bilist[row];
        if ((unsigned)center >= (unsigned)P) { atomicOr(status, ST_BAD_NEIGHBOR); nn = 0; }
        else {
            if ((unsigned)btypes[(size_t)b * P + center] >= (unsigned)ntypes) { atomicOr(status, ST_BAD_TYPE); nn = 0; }
            row_of1[(size_t)b * P + center] = row + 1;
        }
    }
    nnc[row] = nn;
}

// the pairs that name each atom: counted, then listed (comp_incoming_fill), then put in order (comp_incoming_sort)
__global__ void __launch_bounds__(256)
comp_incoming_kernel(int B, int P, int U, const int* __restrict__ nnc, const int* __restrict__ pair_off,
                     const int* __restrict__ bfirstneigh, int* __restrict__ cnt, const int* __restrict__ ioff,
                     int* __restrict__ inc)
{
    const long long q = (long long)blockIdx.x * 256 + threadIdx.x;
    if (q >= (long long)B * P * U) return;
    const int row = (int)(q / U), j = (int)(q - (long long)row * U);
    if (j >= nnc[row]) return;
    const int nj = bfirstneigh[q];
    if ((unsigned)nj >= (unsigned)P) return;             // flagged by the components kernel's table
    const int tg = (row / P) * P + nj;
    const int place = atomicAdd(cnt + tg, 1);
    if (inc) inc[ioff[tg] + place] = pair_off[row] + j;
}

__global__ void __launch_bounds__(256)
comp_incoming_sort_kernel(int n, const int* __restrict__ ioff, int* __restrict__ inc)
{
    const int t = blockIdx.x * 256 + threadIdx.x;
    if (t >= n) return;
    int* v = inc + ioff[t];
    const int m = ioff[t + 1] - ioff[t];
    for (int i = 1; i < m; i++) {
        const int x = v[i];
        int k = i - 1;
        while (k >= 0 && v[k] > x) { v[k + 1] = v[k]; k--; }
        v[k + 1] = x;
    }
}

// force column of every atom: its own row's sum minus the pairs that name it, in the order of the sorted list
template <typename T>
__global__ void __launch_bounds__(64)
comp_force_kernel(int S, int n, const int* __restrict__ row_of1, const int* __restrict__ ioff,
                  const int* __restrict__ inc, const T* __restrict__ pb, const T* __restrict__ rowpart,
                  T* __restrict__ fcomp)
{
    const int t = blockIdx.x, s = blockIdx.y * 64 + threadIdx.x;
    if (s >= S) return;
    T f[3] = {(T)0, (T)0, (T)0};
    const int r1 = row_of1[t];
    if (r1 > 0) {
        const T* o = rowpart + (size_t)(r1 - 1) * 12 * S + s;
#pragma unroll
        for (int i = 0; i < 3; i++) f[i] = o[(size_t)i * S];
    }
    for (int k = ioff[t]; k < ioff[t + 1]; k++) {
        const T* g = pb + (size_t)inc[k] * 3 * S + s;
        f[0] -= g[0]; f[1] -= g[S]; f[2] -= g[2 * S];
    }
#pragma unroll
    for (int i = 0; i < 3; i++) fcomp[((size_t)t * 3 + i) * n + s] = f[i];
}

// energy and virial columns per structure: sums over the rows in row order, in two steps (blocks of COMP_ROWS rows,
// then the blocks); part[B][nblocks][10][S]
constexpr int COMP_ROWS = 32;

template <typename T>
__global__ void __launch_bounds__(64)
comp_structure_blocks_kernel(int S, int P, int nblocks, const int* __restrict__ binum, const T* __restrict__ desc,
                             const T* __restrict__ rowpart, T* __restrict__ part)
{
    const int b = blockIdx.x, s = blockIdx.y * 64 + threadIdx.x, blk = blockIdx.z;
    if (s >= S) return;
    T e = (T)0, v[9];
#pragma unroll
    for (int i = 0; i < 9; i++) v[i] = (T)0;
    const int i1 = min(binum[b], (blk + 1) * COMP_ROWS);
    for (int ii = blk * COMP_ROWS; ii < i1; ii++) {
        const size_t row = (size_t)b * P + ii;
        e += desc[row * S + s];
        const T* o = rowpart + row * 12 * S + s;
#pragma unroll
        for (int i = 0; i < 9; i++) v[i] += o[(size_t)(3 + i) * S];
    }
    T* o = part + ((size_t)b * nblocks + blk) * 10 * S + s;
    o[0] = e;
#pragma unroll
    for (int i = 0; i < 9; i++) o[(size_t)(1 + i) * S] = v[i];
}

template <typename T>
__global__ void __launch_bounds__(64)
comp_structure_kernel(int n, int S, int nblocks, const T* __restrict__ q_scaler, const T* __restrict__ part,
                      T* __restrict__ ecomp, T* __restrict__ vcomp)
{
    const int b = blockIdx.x, s = blockIdx.y * 64 + threadIdx.x;
    if (s >= S) return;
    T acc[10];
#pragma unroll
    for (int i = 0; i < 10; i++) acc[i] = (T)0;
    for (int blk = 0; blk < nblocks; blk++) {
        const T* o = part + ((size_t)b * nblocks + blk) * 10 * S + s;
#pragma unroll
        for (int i = 0; i < 10; i++) acc[i] += o[(size_t)i * S];
    }
    ecomp[(size_t)b * n + s] = acc[0] / q_scaler[s];
#pragma unroll
    for (int i = 0; i < 9; i++) vcomp[((size_t)b * 9 + i) * n + s] = acc[1 + i];
}

// counts[b, t] += 1 for every evaluated row whose centre has species t (integer atomics: exact in any order)
__global__ void __launch_bounds__(256)
species_count_kernel(int B, int P, int ntypes, const int* __restrict__ binum, const int* __restrict__ bilist,
                     const int* __restrict__ btypes, int* __restrict__ counts)
{
    const int row = blockIdx.x * 256 + threadIdx.x;
    if (row >= B * P) return;
    const int b = row / P, ii = row - b * P;
    if (ii >= binum[b]) return;
    const int c = bilist[row];
    if ((unsigned)c >= (unsigned)P) return;
    const int t = btypes[(size_t)b * P + c];
    if ((unsigned)t < (unsigned)ntypes) atomicAdd(counts + b * ntypes + t, 1);
}

// eye[s * S + s] = 1 (the matrix is zero-filled before, may be null); ecomp[b, S + t] = counts[b, t]
template <typename T>
__global__ void __launch_bounds__(256)
lin_components_init_kernel(T* __restrict__ eye, int S, T* __restrict__ ecomp, int B, int ntypes,
                           const int* __restrict__ counts)
{
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (eye && i < S) eye[(size_t)i * S + i] = (T)1;
    if (i < B * ntypes) {
        const int b = i / ntypes, t = i - b * ntypes;
        ecomp[(size_t)b * (S + ntypes) + S + t] = (T)counts[i];
    }
}

// Gram-Schmidt over the nmus radial functions, each the vector of its ntypes^2 * K coefficients
// (schmidt_orth.h:38-116), in the reference's summation order by one thread (the problem is tiny).
template <typename T>
__global__ void schmidt_orth_kernel(T* __restrict__ out, const T* __restrict__ in, int npairs, int nmus, int K)
{
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    const int n = npairs * nmus * K;
    for (int i = 0; i < n; i++) out[i] = in[i];
    for (int k1 = 0; k1 < nmus; k1++) {
        for (int k2 = 0; k2 < k1; k2++) {
            T norm2 = (T)0, scal = (T)0;
            for (int pr = 0; pr < npairs; pr++)
                for (int xi = 0; xi < K; xi++) {
                    const T v1 = out[(pr * nmus + k1) * K + xi], v2 = out[(pr * nmus + k2) * K + xi];
                    norm2 += v2 * v2;
                    scal += v1 * v2;
                }
            for (int pr = 0; pr < npairs; pr++)
                for (int xi = 0; xi < K; xi++)
                    out[(pr * nmus + k1) * K + xi] -= out[(pr * nmus + k2) * K + xi] * scal / norm2;
        }
        T norm2 = (T)1e-10;
        for (int pr = 0; pr < npairs; pr++)
            for (int xi = 0; xi < K; xi++) {
                const T v = out[(pr * nmus + k1) * K + xi];
                norm2 += v * v;
            }
        const T norm = sqrt_t(norm2);
        for (int pr = 0; pr < npairs; pr++)
            for (int xi = 0; xi < K; xi++) out[(pr * nmus + k1) * K + xi] /= norm;
    }
}

// ---- plan construction ---------------------------------------------------------------------------
std::mutex g_plan_mutex;
std::set<MtpPlan*> g_plans;

int plan_create(int n_moms, int n_basic, const int* basic, int n_times, const int* times, int n_scalar,
                const int* mapping, MtpPlan** out)
{
    A2P_REQUIRE(n_moms > 0 && n_basic > 0 && n_basic <= n_moms && n_times >= 0 && n_scalar > 0,
                A2P_ERR_INVALID, "mtp plan: bad table sizes");
    A2P_REQUIRE(basic && mapping && (times || n_times == 0), A2P_ERR_INVALID, "mtp plan: null table");
    int nmus = 0, kmax = 0;
    for (int i = 0; i < n_basic; i++) {
        const int* q = basic + i * 4;
        A2P_REQUIRE(q[0] >= 0 && q[1] >= 0 && q[2] >= 0 && q[3] >= 0, A2P_ERR_INVALID,
                    "mtp plan: negative entry in alpha_index_basic");
        A2P_REQUIRE(i == 0 || q[0] >= basic[(i - 1) * 4], A2P_ERR_INVALID,
                    "mtp plan: alpha_index_basic is not grouped by radial function index");
        nmus = std::max(nmus, q[0] + 1);
        kmax = std::max(kmax, q[1] + q[2] + q[3]);
    }
    A2P_REQUIRE(nmus <= MTP_NMUS_MAX, A2P_ERR_INVALID, "mtp plan: more than %d radial functions", MTP_NMUS_MAX);
    A2P_REQUIRE(kmax <= 24, A2P_ERR_INVALID, "mtp plan: monomial degree %d too large", kmax);
    std::vector<int> level(n_moms, 0), last_write(n_moms, -1);
    for (int e = 0; e < n_times; e++) {
        const int* q = times + e * 4;
        A2P_REQUIRE(q[0] >= 0 && q[0] < n_moms && q[1] >= 0 && q[1] < n_moms && q[3] >= n_basic &&
                        q[3] < n_moms,
                    A2P_ERR_INVALID, "mtp plan: alpha_index_times entry %d out of range", e);
        last_write[q[3]] = e;
    }
    int n_levels = 0;
    for (int e = 0; e < n_times; e++) {
        const int* q = times + e * 4;
        for (int s = 0; s < 2; s++)
            A2P_REQUIRE(last_write[q[s]] < e, A2P_ERR_INVALID,
                        "mtp plan: moment %d is read by product %d before its last contribution (%d); "
                        "the table cannot be executed level by level", q[s], e, last_write[q[s]]);
        level[q[3]] = std::max(level[q[3]], 1 + std::max(level[q[0]], level[q[1]]));
        n_levels = std::max(n_levels, level[q[3]]);
    }
    std::vector<char> seen(n_moms, 0);
    for (int s = 0; s < n_scalar; s++) {
        A2P_REQUIRE(mapping[s] >= 0 && mapping[s] < n_moms, A2P_ERR_INVALID, "mtp plan: mapping out of range");
        A2P_REQUIRE(!seen[mapping[s]], A2P_ERR_INVALID, "mtp plan: alpha_moment_mapping repeats a moment");
        seen[mapping[s]] = 1;
    }
    A2P_REQUIRE(n_moms < 8192, A2P_ERR_INVALID, "mtp plan: more than 8191 moments");    // 16-bit byte offsets
    // Interleaved gather lists (see mtp_plan.h).  `lists[m]` holds the packed terms of moment m.
    struct Ell {
        std::vector<int> level, lend, multi, slot, lead, gbase, gdepth;   // multi: doubling steps; lead: pieces behind
        std::vector<int2> terms;
        int max_slots = 0;
        bool too_long = false;
    };
    auto build_ell = [&](const std::vector<std::vector<int2>>& lists, const std::vector<std::vector<int>>& by_level) {
        Ell e;
        for (const auto& members : by_level) {
            const int first_slot = (int)e.slot.size();
            e.level.push_back(first_slot);
            std::vector<int> ms = members;
            std::stable_sort(ms.begin(), ms.end(),
                             [&](int x, int y) { return lists[x].size() > lists[y].size(); });
            // slots of the level: (list, first term, term count, pieces behind this one); the pieces of a list are
            // adjacent and stay inside one group of 64 slots (one wavefront adds them up with shuffles)
            struct Piece { int m, t0, n, rem; };
            std::vector<Piece> pieces;
            int most = 1;
            for (int m : ms) {
                const int n = (int)lists[m].size();
                const int np = (n + MTP_SLOT_CAP - 1) / MTP_SLOT_CAP;
                if (np > 64) { e.too_long = true; continue; }
                most = std::max(most, np);
                if ((int)(pieces.size() % 64) + np > 64)
                    while (pieces.size() % 64) pieces.push_back({-1, 0, 0, 0});
                for (int q = 0; q < np; q++)
                    pieces.push_back({m, q * MTP_SLOT_CAP, std::min(MTP_SLOT_CAP, n - q * MTP_SLOT_CAP), np - 1 - q});
            }
            (void)most;
            for (size_t g0 = 0; g0 < pieces.size(); g0 += 64) {
                const size_t g1 = std::min(pieces.size(), g0 + 64);
                int depth = 0, longest = 1;
                for (size_t q = g0; q < g1; q++) {
                    depth = std::max(depth, pieces[q].n);
                    longest = std::max(longest, pieces[q].rem + 1);
                }
                int steps = 0;                      // doubling steps that add up the pieces of this group's lists
                while ((1 << steps) < longest) steps++;
                e.multi.push_back(steps);
                depth = (depth + MTP_DEPTH_STEP - 1) / MTP_DEPTH_STEP * MTP_DEPTH_STEP;    // the sweeps fetch that many terms at a time
                e.gbase.push_back((int)e.terms.size());
                e.gdepth.push_back(depth);
                e.terms.resize(e.terms.size() + (size_t)depth * 64, make_int2(0, 0));
                for (size_t q = g0; q < g1; q++) {
                    const Piece& pc = pieces[q];
                    for (int k = 0; k < pc.n; k++)
                        e.terms[e.gbase.back() + (size_t)k * 64 + (q - g0)] = lists[pc.m][pc.t0 + k];
                    e.slot.push_back(pc.t0 == 0 ? pc.m : -1);      // the first piece of a list names the moment
                    e.lead.push_back(pc.rem);
                }
            }
            e.lend.push_back((int)e.slot.size());
            e.max_slots = std::max(e.max_slots, (int)e.slot.size() - first_slot);
            while (e.slot.size() % 64) { e.slot.push_back(-1); e.lead.push_back(0); }
        }
        e.level.push_back((int)e.slot.size());
        e.lend.push_back((int)e.slot.size());
        if (e.terms.empty()) e.terms.push_back(make_int2(0, 0));
        if (e.gbase.empty()) { e.gbase.push_back(0); e.gdepth.push_back(0); e.multi.push_back(0); }
        if (e.slot.empty()) { e.slot.push_back(-1); e.lead.push_back(0); }
        return e;
    };
    // forward: terms per destination in file order; level l >= 1 at index l - 1
    std::vector<std::vector<int2>> fl(n_moms), rl(n_moms);
    for (int e = 0; e < n_times; e++) {
        const int* q = times + e * 4;
        fl[q[3]].push_back(make_int2((q[0] * 8) | ((q[1] * 8) << 16), q[2]));
    }
    std::vector<std::vector<int>> f_by(n_levels), r_by(n_levels);
    for (int m = n_basic; m < n_moms; m++)
        if (level[m] >= 1 && !fl[m].empty()) f_by[level[m] - 1].push_back(m);
    // reverse: terms per source in reverse file order
    for (int e = n_times - 1; e >= 0; e--) {
        const int* q = times + e * 4;
        rl[q[1]].push_back(make_int2((q[3] * 8) | ((q[0] * 8) << 16), q[2]));     // adj[m1] += adj[dst] mult M[m0]
        rl[q[0]].push_back(make_int2((q[3] * 8) | ((q[1] * 8) << 16), q[2]));     // adj[m0] += adj[dst] mult M[m1]
    }
    for (int m = 0; m < n_moms; m++)
        if (level[m] < n_levels && !rl[m].empty()) r_by[level[m]].push_back(m);
    const Ell F = build_ell(fl, f_by), R = build_ell(rl, r_by);
    A2P_REQUIRE(!F.too_long && !R.too_long, A2P_ERR_INVALID,
                "mtp plan: a moment takes part in more than %d products; this level is too large", 64 * MTP_SLOT_CAP);
    std::vector<int> mu_begin(nmus + 1, n_basic);
    for (int i = n_basic - 1; i >= 0; i--) mu_begin[basic[i * 4]] = i;
    for (int m = nmus - 1; m >= 0; m--) mu_begin[m] = std::min(mu_begin[m], mu_begin[m + 1]);
    mu_begin[0] = 0;

    // monomial rows and the dense adjoint map of the pair-derivative pass (mtp_plan.h)
    const int nmp = (nmus + 1) / 2 * 2;
    std::vector<int> row_base((kmax + 1) * (kmax + 1), -1), rows;
    int nq = 0;
    for (int a = 0; a <= kmax; a++)
        for (int b = 0; a + b <= kmax; b++) {
            row_base[a * (kmax + 1) + b] = nq;
            rows.push_back(a | (b << 8) | (nq << 16));
            nq += kmax - a - b + 1;
        }
    A2P_REQUIRE(nq < 32768, A2P_ERR_INVALID, "mtp plan: too many monomials");
    std::stable_sort(rows.begin(), rows.end(), [&](int x, int y) {
        return (x & 255) + ((x >> 8) & 255) < (y & 255) + ((y >> 8) & 255);     // longest rows first
    });
    std::vector<std::vector<int>> dense_lists((size_t)nq * nmp);
    for (int i = 0; i < n_basic; i++) {
        const int* q = basic + i * 4;
        dense_lists[(size_t)(row_base[q[1] * (kmax + 1) + q[2]] + q[3]) * nmp + q[0]].push_back(i);
    }
    std::vector<int> dense_src((size_t)nq * nmp), dense_off((size_t)nq * nmp + 1, 0), dense_items, dense_pos(n_basic);
    int dense_unique = 1;
    for (size_t e = 0; e < dense_lists.size(); e++) {
        dense_src[e] = dense_lists[e].empty() ? -1 : (dense_lists[e].size() == 1 ? dense_lists[e][0] : -2);
        dense_off[e] = (int)dense_items.size();
        if (dense_lists[e].size() > 1) dense_unique = 0;
        for (int i : dense_lists[e]) dense_pos[i] = (int)e;
        dense_items.insert(dense_items.end(), dense_lists[e].begin(), dense_lists[e].end());
    }
    dense_off[dense_lists.size()] = (int)dense_items.size();

    // nodes (scalar moment, ancestor) and their reverse gather (mtp_plan.h), for batches of scalar moments whose node
    // adjoints fit MTP_NODE_CAP entries of LDS
    struct XHost {
        std::vector<int> root, seed, brem, bsteps, bbase, bdepth, bwords;
        Ell ell;
        int nodes = 0;
    };
    std::vector<XHost> xhosts;
    if (n_basic < 64 * MTP_SLOT_CAP) {
        std::vector<std::vector<int>> terms_of(n_moms);
        for (int e = 0; e < n_times; e++) terms_of[times[e * 4 + 3]].push_back(e);
        std::vector<int> node_of(n_moms, -1), anc, stack;
        auto ancestors = [&](int s, int first_node) {          // fills anc and node_of; returns the number of nodes
            anc.clear();
            stack.assign(1, mapping[s]);
            int nd = first_node;
            while (!stack.empty()) {
                const int m = stack.back();
                stack.pop_back();
                if (node_of[m] >= 0) continue;
                node_of[m] = nd++;
                anc.push_back(m);
                for (int e : terms_of[m]) { stack.push_back(times[e * 4]); stack.push_back(times[e * 4 + 1]); }
            }
            return nd - first_node;
        };
        // batches: scalar moments in table order, as many as fit
        std::vector<std::vector<int>> batches(1);
        int in_batch = 0;
        bool fits = true;
        for (int s = 0; s < n_scalar; s++) {
            const int cnt = ancestors(s, 0);
            for (int m : anc) node_of[m] = -1;
            if (cnt > MTP_NODE_CAP) fits = false;
            if (in_batch + cnt > MTP_NODE_CAP) { batches.emplace_back(); in_batch = 0; }
            batches.back().push_back(s);
            in_batch += cnt;
        }
        if (!fits) batches.clear();
        for (const auto& seeds : batches) {
            xhosts.emplace_back();
            XHost& h = xhosts.back();
            h.root.assign(n_scalar, -1);
            std::vector<std::vector<int2>> xl;
            std::vector<std::vector<int>> x_by(n_levels);
            std::vector<std::vector<int>> seed_basic(n_scalar);
            for (int s : seeds) {
                const int cnt = ancestors(s, h.nodes);
                h.nodes += cnt;
                xl.resize(h.nodes);
                h.root[s] = node_of[mapping[s]];
                for (int e = n_times - 1; e >= 0; e--) {          // reverse file order, as in the reverse gather above
                    const int* q = times + e * 4;
                    if (node_of[q[3]] < 0) continue;
                    const int nd = node_of[q[3]];
                    xl[node_of[q[1]]].push_back(make_int2((nd * 8) | ((q[0] * 8) << 16), q[2]));
                    xl[node_of[q[0]]].push_back(make_int2((nd * 8) | ((q[1] * 8) << 16), q[2]));
                }
                for (int m : anc) {
                    if (level[m] < n_levels && !xl[node_of[m]].empty()) x_by[level[m]].push_back(node_of[m]);
                    if (m < n_basic) seed_basic[s].push_back(node_of[m] | (m << 16));
                }
                for (int m : anc) node_of[m] = -1;
            }
            if (xl.empty()) xl.emplace_back();
            h.ell = build_ell(xl, x_by);
            A2P_REQUIRE(!h.ell.too_long, A2P_ERR_INVALID, "mtp plan: a moment takes part in more than %d products",
                        64 * MTP_SLOT_CAP);
            std::vector<int> by_len = seeds;
            std::stable_sort(by_len.begin(), by_len.end(),
                             [&](int x, int y) { return seed_basic[x].size() > seed_basic[y].size(); });
            struct Piece { int s, t0, n, rem; };
            std::vector<Piece> pieces;
            for (int s : by_len) {
                const int len = (int)seed_basic[s].size();
                const int np = std::max(1, (len + MTP_SLOT_CAP - 1) / MTP_SLOT_CAP);      // <= 64: n_basic < 64 * cap
                if ((int)(pieces.size() % 64) + np > 64)
                    while (pieces.size() % 64) pieces.push_back({-1, 0, 0, 0});
                for (int q = 0; q < np; q++)
                    pieces.push_back({s, q * MTP_SLOT_CAP, std::min(MTP_SLOT_CAP, len - q * MTP_SLOT_CAP), np - 1 - q});
            }
            while (pieces.empty() || pieces.size() % 64) pieces.push_back({-1, 0, 0, 0});
            for (size_t g0 = 0; g0 < pieces.size(); g0 += 64) {
                int depth = 0, most = 1;
                for (size_t q = g0; q < g0 + 64; q++) {
                    depth = std::max(depth, pieces[q].n);
                    most = std::max(most, pieces[q].rem + 1);
                }
                int steps = 0;
                while ((1 << steps) < most) steps++;
                depth = (depth + 3) / 4 * 4;            // the kernel fetches four words at a time
                h.bbase.push_back((int)h.bwords.size());
                h.bdepth.push_back(depth);
                h.bsteps.push_back(steps);
                h.bwords.resize(h.bwords.size() + (size_t)depth * 64, h.nodes);       // node `nodes` (a zero), basic moment 0
                for (size_t q = g0; q < g0 + 64; q++) {
                    const Piece& pc = pieces[q];
                    for (int k = 0; k < pc.n; k++)
                        h.bwords[h.bbase.back() + (size_t)k * 64 + (q - g0)] = seed_basic[pc.s][pc.t0 + k];
                    h.seed.push_back(pc.s >= 0 && pc.t0 == 0 ? pc.s : -1);
                    h.brem.push_back(pc.rem);
                }
            }
            if (h.bwords.empty()) h.bwords.push_back(0);
        }
    }

    // one device block
    struct Seg { const void* src; size_t bytes; size_t off; };
    std::vector<Seg> segs;
    size_t total = 0;
    auto add = [&](const void* src, size_t bytes) {
        size_t off = total;
        segs.push_back({src, bytes, off});
        total += (bytes + 15) / 16 * 16;
        return off;
    };
    const size_t o_basic = add(basic, sizeof(int) * 4 * n_basic);
    const size_t o_mu = add(mu_begin.data(), sizeof(int) * mu_begin.size());
    const size_t o_map = add(mapping, sizeof(int) * n_scalar);
    const size_t o_fl = add(F.level.data(), sizeof(int) * F.level.size());
    const size_t o_fe = add(F.lend.data(), sizeof(int) * F.lend.size());
    const size_t o_fx = add(F.multi.data(), sizeof(int) * F.multi.size());
    const size_t o_fd = add(F.slot.data(), sizeof(int) * F.slot.size());
    const size_t o_fc = add(F.lead.data(), sizeof(int) * F.lead.size());
    const size_t o_fg = add(F.gbase.data(), sizeof(int) * F.gbase.size());
    const size_t o_fh = add(F.gdepth.data(), sizeof(int) * F.gdepth.size());
    const size_t o_ft = add(F.terms.data(), sizeof(int2) * F.terms.size());
    const size_t o_rl = add(R.level.data(), sizeof(int) * R.level.size());
    const size_t o_re = add(R.lend.data(), sizeof(int) * R.lend.size());
    const size_t o_rx = add(R.multi.data(), sizeof(int) * R.multi.size());
    const size_t o_rs = add(R.slot.data(), sizeof(int) * R.slot.size());
    const size_t o_rc = add(R.lead.data(), sizeof(int) * R.lead.size());
    const size_t o_rg = add(R.gbase.data(), sizeof(int) * R.gbase.size());
    const size_t o_rh = add(R.gdepth.data(), sizeof(int) * R.gdepth.size());
    const size_t o_rt = add(R.terms.data(), sizeof(int2) * R.terms.size());
    const size_t o_rows = add(rows.data(), sizeof(int) * rows.size());
    const size_t o_dsrc = add(dense_src.data(), sizeof(int) * dense_src.size());
    const size_t o_doff = add(dense_off.data(), sizeof(int) * dense_off.size());
    const size_t o_dit = add(dense_items.data(), sizeof(int) * dense_items.size());
    const size_t o_dpos = add(dense_pos.data(), sizeof(int) * dense_pos.size());
    struct XOff { size_t root, seed, level, multi, src, rem, gbase, gdepth, terms, bbase, bdepth, bsteps, brem, bwords; };
    std::vector<XOff> xoffs;
    for (const XHost& h : xhosts) {
        XOff o;
        o.root = add(h.root.data(), sizeof(int) * h.root.size());
        o.seed = add(h.seed.data(), sizeof(int) * h.seed.size());
        o.level = add(h.ell.level.data(), sizeof(int) * h.ell.level.size());
        o.multi = add(h.ell.multi.data(), sizeof(int) * h.ell.multi.size());
        o.src = add(h.ell.slot.data(), sizeof(int) * h.ell.slot.size());
        o.rem = add(h.ell.lead.data(), sizeof(int) * h.ell.lead.size());
        o.gbase = add(h.ell.gbase.data(), sizeof(int) * h.ell.gbase.size());
        o.gdepth = add(h.ell.gdepth.data(), sizeof(int) * h.ell.gdepth.size());
        o.terms = add(h.ell.terms.data(), sizeof(int2) * h.ell.terms.size());
        o.bbase = add(h.bbase.data(), sizeof(int) * h.bbase.size());
        o.bdepth = add(h.bdepth.data(), sizeof(int) * h.bdepth.size());
        o.bsteps = add(h.bsteps.data(), sizeof(int) * h.bsteps.size());
        o.brem = add(h.brem.data(), sizeof(int) * h.brem.size());
        o.bwords = add(h.bwords.data(), sizeof(int) * h.bwords.size());
        xoffs.push_back(o);
    }
    std::vector<unsigned char> host(total + 16, 0);
    for (auto& s : segs)
        if (s.bytes) std::memcpy(host.data() + s.off, s.src, s.bytes);
    MtpPlan* plan = new MtpPlan();
    A2P_HIP_CHECK(hipGetDevice(&plan->device));
    A2P_HIP_CHECK(hipMalloc(&plan->device_block, total + 16));
    A2P_HIP_CHECK(hipMemcpy(plan->device_block, host.data(), total + 16, hipMemcpyHostToDevice));
    char* base = (char*)plan->device_block;
    MtpPlanDevice& d = plan->d;
    d.n_moms = n_moms; d.n_basic = n_basic; d.n_times = n_times; d.n_scalar = n_scalar;
    d.nmus = nmus; d.kmax = kmax; d.n_levels = n_levels;
    d.basic = (const int*)(base + o_basic); d.mu_begin = (const int*)(base + o_mu);
    d.mapping = (const int*)(base + o_map);
    d.f_level = (const int*)(base + o_fl); d.f_lend = (const int*)(base + o_fe);
    d.f_multi = (const int*)(base + o_fx);
    d.f_dst = (const int*)(base + o_fd); d.f_rem = (const int*)(base + o_fc);
    d.f_gbase = (const int*)(base + o_fg); d.f_gdepth = (const int*)(base + o_fh);
    d.f_terms = (const int2*)(base + o_ft);
    d.r_level = (const int*)(base + o_rl); d.r_lend = (const int*)(base + o_re);
    d.r_multi = (const int*)(base + o_rx);
    d.r_src = (const int*)(base + o_rs); d.r_rem = (const int*)(base + o_rc);
    d.r_gbase = (const int*)(base + o_rg); d.r_gdepth = (const int*)(base + o_rh);
    d.r_terms = (const int2*)(base + o_rt);
    d.max_level_slots = 0;       // the sweeps keep no partial sums in LDS
    d.nq = nq; d.nmp = nmp; d.nrows = (int)rows.size();
    d.rows = (const int*)(base + o_rows); d.dense_src = (const int*)(base + o_dsrc);
    d.dense_off = (const int*)(base + o_doff); d.dense_items = (const int*)(base + o_dit);
    d.dense_pos = (const int*)(base + o_dpos); d.dense_unique = dense_unique;
    d.x_nodes = 0; d.x_slots = 0;                // set per batch by the components call (MtpPlan::xbatches)
    for (size_t i = 0; i < xhosts.size(); i++) {
        const XOff& o = xoffs[i];
        MtpXBatch xb;
        xb.nodes = xhosts[i].nodes; xb.slots = (int)xhosts[i].seed.size();
        xb.root = (const int*)(base + o.root); xb.seed = (const int*)(base + o.seed);
        xb.level = (const int*)(base + o.level); xb.multi = (const int*)(base + o.multi);
        xb.src = (const int*)(base + o.src); xb.rem = (const int*)(base + o.rem);
        xb.gbase = (const int*)(base + o.gbase); xb.gdepth = (const int*)(base + o.gdepth);
        xb.terms = (const int2*)(base + o.terms);
        xb.bbase = (const int*)(base + o.bbase); xb.bdepth = (const int*)(base + o.bdepth);
        xb.bsteps = (const int*)(base + o.bsteps); xb.brem = (const int*)(base + o.brem);
        xb.bwords = (const int*)(base + o.bwords);
        plan->xbatches.push_back(xb);
    }
    {
        std::lock_guard<std::mutex> lock(g_plan_mutex);
        g_plans.insert(plan);
    }
    *out = plan;
    return A2P_OK;
}

int plan_check(void* handle, MtpPlan** out)
{
    std::lock_guard<std::mutex> lock(g_plan_mutex);
    A2P_REQUIRE(handle && g_plans.count((MtpPlan*)handle), A2P_ERR_INVALID, "mtp: invalid plan handle");
    *out = (MtpPlan*)handle;
    return A2P_OK;
}

template <typename T>
int table_entries(const MtpPlanDevice& p, int K, bool loss)
{
    int E = 3 * (p.kmax + 1) + 2 * p.nmus + 4;
    if (loss) E += 4 + 2 * K;
    if ((E & 1) == 0) E++;            // odd stride: neighbours land in different LDS banks
    return E;
}

template <typename T>
size_t lds_bytes(const MtpPlanDevice& p, int E, bool loss, int ntypes, int K, int H, int MTP_NC, int nt,
                 bool keep = false)
{
    // the neighbour table and the group sums double as the sweeps' partial-sum arrays
    const size_t tabs = (size_t)mtp_table_region(MTP_NC, E, loss, p.n_moms, p.max_level_slots, nt, keep);
    size_t n = (size_t)p.n_moms * (loss ? 2 : 1) + tabs + (loss ? 2 * (size_t)p.n_basic : 0) +
               (size_t)ntypes * p.nmus * K;   // + the coefficient copy
    // loss mode: P, Q, the neighbour types and the per-atom coefficient-gradient block
    if (loss) n += 2 * (size_t)MTP_NC * p.nmus + MTP_NC + (size_t)ntypes * p.nmus * K;
    if (H > 0) n += (size_t)p.n_scalar + (loss ? 5 : 1) * (size_t)H;     // network inputs and per-neuron values
    if (!loss && !mtp_dense_in_moments(p.nq, p.nmp, p.n_moms)) n += (size_t)p.nq * p.nmp;
    return n * sizeof(T) + 64;      // the packed basic-moment table (4 n_basic bytes) follows
}

template <typename T>
int fill_args(MtpArgs<T>& a, MtpPlan* plan, int K, double scaling, const T* coeffs, const T* lin,
              const T* bias, int nmus, int ntypes, const T* q_scaler, double rmax, double rmin, int B, int P,
              int U, int nghost, const int* binum, const int* bilist, const int* bnumneigh,
              const int* bfirstneigh, const T* brcs, const int* btypes, bool readout = true)
{
    A2P_REQUIRE(K >= 1 && K <= MTP_KMAX, A2P_ERR_INVALID, "mtp: chebyshev_size %d outside [1, %d]", K, MTP_KMAX);
    A2P_REQUIRE(nmus == plan->d.nmus, A2P_ERR_INVALID, "mtp: nmus %d does not match the tables (%d)", nmus,
                plan->d.nmus);
    A2P_REQUIRE(ntypes >= 1 && B >= 0 && P >= 0 && U >= 1 && nghost >= 0, A2P_ERR_INVALID, "mtp: bad shape");
    A2P_REQUIRE(rmax > rmin && rmin >= 0, A2P_ERR_INVALID, "mtp: need 0 <= rmin < rmax");
    A2P_REQUIRE(coeffs && (!readout || (bias && q_scaler)) && binum && bilist && bnumneigh && bfirstneigh && brcs &&
                    btypes, A2P_ERR_INVALID, "mtp: null input pointer");
    A2P_REQUIRE((long long)B * P * U < (1ll << 31), A2P_ERR_INVALID, "mtp: batch too large");
    a.p = plan->d;
    a.K = K; a.ntypes = ntypes; a.scaling = (T)scaling; a.rmax = (T)rmax; a.rmin = (T)rmin;
    a.coeffs = coeffs; a.lin = lin; a.bias = bias; a.q_scaler = q_scaler;
    a.B = B; a.P = P; a.U = U; a.nghost = nghost;
    a.binum = binum; a.bilist = bilist; a.bnumneigh = bnumneigh; a.bfirstneigh = bfirstneigh;
    a.brcs = brcs; a.btypes = btypes;
    a.cE = nullptr; a.dFs = nullptr; a.dVs = nullptr; a.gpart = nullptr; a.ngrad = 0;
    a.force = nullptr; a.seg_cursor = nullptr; a.seg_g = nullptr; a.seg_spare = 0; a.seg_cap = 0; a.partial = nullptr;
    a.e_sites = nullptr; a.desc = nullptr; a.energy_only = 0; a.cE_per_atom = 0; a.no_tangent = 0; a.keep_table = 0;
    a.nn_exact = 1;
    a.row_seed = nullptr; a.pair_out = nullptr;
    a.H = 0; a.w0 = nullptr; a.w1 = nullptr; a.q_shift = nullptr;
    void* ws = nullptr;
    int rc = ws_get(WS_FLAGS, 64, &ws);
    if (rc) return rc;
    a.status = (int*)ws;
    return A2P_OK;
}

int g_keep_table = 1;      // (measurement switch: AI2POT_MTP_KEEP_TABLE=0)

template <typename T, bool LOSS, bool SEED = false>
int launch_atoms(const MtpArgs<T>& a, hipStream_t stream)
{
    {
        static const char* e = getenv("AI2POT_MTP_KEEP_TABLE");
        if (e) g_keep_table = e[0] != '0';
    }
    const bool wide = a.p.n_moms >= (LOSS ? 300 : 1000);   // enough work per atom to keep 256 threads busy
    auto lds_for = [&](int nc, size_t* main, bool keep = false) {
        *main = (lds_bytes<T>(a.p, a.E, LOSS, a.ntypes, a.K, a.H, nc, wide ? 256 : 64, keep) + 15) / 16 * 16;
        // the packed basic-moment table; energy / force / virial kernel: + the monomial rows
        return *main + (LOSS ? (size_t)a.p.n_basic : (size_t)a.p.n_basic + a.p.nrows) * sizeof(unsigned);
    };
    size_t lds_main = 0;
    int nc_cap = MTP_NC;
    size_t lds = lds_for(nc_cap, &lds_main);
    // Rows of the neighbour table (energy / force / virial kernel; the loss kernels keep MTP_NC): the kernel waits on
    // dependent LDS reads and barriers, so workgroups per CU count first (level 16: 12 -> 16 workgroups, 0.136 -> 0.122 ms
    // although rows of more than 20 neighbours then take two chunks), and among the tables that allow as many
    // workgroups as the registers do (four waves per SIMD), or as the shortest table does, the longest is taken
    // (level 20: a row of 35 neighbours in one chunk instead of two, 0.45 -> 0.41 ms).
    if (!LOSS) {
        // LDS is handed out in pieces of 1280 bytes on this chip
        auto per_cu = [](size_t l) { return (size_t)(160 * 1024) / ((l + 1279) / 1280 * 1280); };
        size_t m = 0;
        const size_t by_registers = wide ? 4 : 16;
        const size_t want = std::min(by_registers, per_cu(lds_for(MTP_NC_MIN, &m)));
        for (int nc : {MTP_NC_MAX, 40, 32, 24, 20, MTP_NC_MIN}) {
            const size_t l = lds_for(nc, &m);
            if (per_cu(l) >= want || nc == MTP_NC_MIN) { nc_cap = nc; lds = l; lds_main = m; break; }
        }
        // The table kept through the sweeps (adjoints behind it) saves a row of one chunk its second table build: taken
        // when a table of at least 32 rows fits that way at the same number of workgroups per CU (level 20: 0.387 ->
        // 0.368 ms, level 10: 0.026 -> 0.023 ms; at level 16 the sixteen workgroups per CU count for more).  Not in the
        // modes that use the table's place as scratch between the sweeps (site energies, descriptors).
        int keep = 0;
        if (!a.e_sites && !a.desc && !a.energy_only && g_keep_table)
            for (int nc : {MTP_NC_MAX, 40, 32}) {
                const size_t l = lds_for(nc, &m, true);
                if (per_cu(l) >= want) { keep = 1; nc_cap = nc; lds = l; lds_main = m; break; }
            }
        const_cast<MtpArgs<T>&>(a).keep_table = keep;
    }
    const_cast<MtpArgs<T>&>(a).lds_basic_off = (int)lds_main;
    const_cast<MtpArgs<T>&>(a).nc_cap = nc_cap;
    A2P_REQUIRE(lds <= 160 * 1024, A2P_ERR_INVALID,
                "mtp: %d moments need %zu bytes of LDS per atom; this level is too large", a.p.n_moms, lds);
    auto kern = wide ? mtp_atom_kernel<T, LOSS, 256, SEED> : mtp_atom_kernel<T, LOSS, 64, SEED>;
    if (lds > 48 * 1024)
        A2P_HIP_CHECK(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                                          (int)lds));
    prof_begin(LOSS ? "mtp_loss_bwd_kernel" : "mtp_efv_kernel", stream);
    hipLaunchKernelGGL(kern, dim3(a.P, a.B), dim3(wide ? 256 : 64), lds, stream, a);
    prof_end(stream);
    A2P_HIP_CHECK(hipGetLastError());
    return A2P_OK;
}

// network of the neural-network MTP: w0[ntypes, H, n_scalar], w1[ntypes, H], q_shift[n_scalar]
template <typename T>
struct MtpNet {
    int H;
    const T *w0, *w1, *q_shift;
};

template <typename T>
int set_net(MtpArgs<T>& a, const MtpNet<T>* net)
{
    if (!net) {
        A2P_REQUIRE(a.lin, A2P_ERR_INVALID, "mtp: null linear_coeffs");
        return A2P_OK;
    }
    A2P_REQUIRE(net->H >= 1 && net->w0 && net->w1 && net->q_shift, A2P_ERR_INVALID,
                "nnmtp: need num_neurons >= 1 and non-null w0, w1, q_shifter");
    a.H = net->H; a.w0 = net->w0; a.w1 = net->w1; a.q_shift = net->q_shift;
    return A2P_OK;
}

template <typename T>
int mtp_efv(void* handle, int K, double scaling, const T* coeffs, const T* lin, const T* bias, int nmus,
            int ntypes, const T* q_scaler, double rmax, double rmin, int B, int P, int U, int nghost,
            const int* binum, const int* bilist, const int* bnumneigh, const int* bfirstneigh, const T* brcs,
            const int* btypes, T* etot, T* force, T* virial, hipStream_t stream,
            const MtpNet<T>* net = nullptr, T* e_sites = nullptr)
{
    MtpPlan* plan = nullptr;
    int rc = plan_check(handle, &plan);
    if (rc) return rc;
    MtpArgs<T> a;
    rc = fill_args(a, plan, K, scaling, coeffs, lin, bias, nmus, ntypes, q_scaler, rmax, rmin, B, P, U, nghost,
                   binum, bilist, bnumneigh, bfirstneigh, brcs, btypes);
    if (rc) return rc;
    rc = set_net(a, net);
    if (rc) return rc;
    if (B == 0 || P == 0) return A2P_OK;
    a.e_sites = e_sites;
    a.E = table_entries<T>(a.p, K, false);
    void* ws = nullptr;
    rc = ws_get(WS_PARTIAL, (size_t)B * P * 10 * sizeof(double), &ws);
    if (rc) return rc;
    a.partial = (double*)ws;
    const size_t force_bytes = (size_t)B * (P + nghost) * 3 * sizeof(T);
    a.force = force;
    if (!force) {
        rc = ws_get(WS_MISC, force_bytes, &ws);
        if (rc) return rc;
        a.force = (T*)ws;
    }
    PairCsr csr{};
    if (force) {       // the force array is zeroed with the cursors (the reference zeroes on entry, linearMtp.h:228-230)
        rc = pair_fixed_begin<T>(&csr, B, P, U, nghost, stream, a.force, force_bytes);
        if (rc) return rc;
        a.seg_cursor = csr.cursor;
        a.seg_g = (T*)csr.seg_g;
        a.seg_spare = csr.n * csr.seg_cap;
        a.seg_cap = csr.seg_cap;
    } else {
        rc = fill_zero(a.force, force_bytes, stream);
        if (rc) return rc;
    }
    rc = launch_atoms<T, false>(a, stream);
    if (rc) return rc;
    if (force)       // the segment sums and the energy / virial sums share a launch
        return pair_csr_finish<T>(force, csr, stream, etot, virial, a.partial, B, P);
    return finish_energy_virial<T>(etot, virial, a.partial, B, P, stream);
}

template <typename T>
int mtp_loss(void* handle, double e_w, double f_w, double v_w, const T* e_dft, const T* f_dft, const T* v_dft,
             int K, double scaling, const T* coeffs, const T* lin, const T* bias, int nmus, int ntypes,
             const T* q_scaler, double rmax, double rmin, int B, int P, int U, const int* binum,
             const int* bilist, const int* bnumneigh, const int* bfirstneigh, const T* brcs, const int* btypes,
             T* bloss, T* rmse, T* etot, T* force, T* virial, T* dcoeffs, T* dlin, T* dbias,
             hipStream_t stream)
{
    A2P_REQUIRE(e_dft && f_dft && v_dft && bloss && etot && force && virial && lin, A2P_ERR_INVALID,
                "mtp loss: null label, parameter or output pointer");
    int rc = mtp_efv<T>(handle, K, scaling, coeffs, lin, bias, nmus, ntypes, q_scaler, rmax, rmin, B, P, U, 0,
                        binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, etot, force, virial, stream);
    if (rc) return rc;
    if (B == 0 || P == 0) return A2P_OK;
    MtpPlan* plan = nullptr;
    rc = plan_check(handle, &plan);
    if (rc) return rc;
    MtpArgs<T> a;
    rc = fill_args(a, plan, K, scaling, coeffs, lin, bias, nmus, ntypes, q_scaler, rmax, rmin, B, P, U, 0,
                   binum, bilist, bnumneigh, bfirstneigh, brcs, btypes);
    if (rc) return rc;
    const int ncoef = ntypes * ntypes * nmus * K;
    const int ngrad = ncoef + a.p.n_scalar + ntypes;
    const bool want_grad = dcoeffs || dlin || dbias;
    // workspace: cE[B] | dVs[B*9] | dFs[B*P*3] | gpart[B*P*ngrad] | sq[B*3] (double)
    size_t nT = (size_t)B + (size_t)B * 9 + (size_t)B * P * 3 + (want_grad ? (size_t)B * P * ngrad : 0);
    size_t bytesT = (nT * sizeof(T) + 15) / 16 * 16;
    void* ws = nullptr;
    rc = ws_get(WS_MTP, bytesT + (size_t)B * 3 * sizeof(double), &ws);
    if (rc) return rc;
    T* cE = (T*)ws;
    T* dVs = cE + B;
    T* dFs = dVs + (size_t)B * 9;
    T* gpart = dFs + (size_t)B * P * 3;
    double* sq = (double*)((char*)ws + bytesT);
    prof_begin("mtp_loss_forward", stream);
    hipLaunchKernelGGL(losskern::loss_forward_kernel<T>, dim3(B), dim3(256), 0, stream, P, binum, bilist, (T)e_w,
                       (T)f_w, (T)v_w, etot, e_dft, force, f_dft, virial, v_dft, bloss, cE, dFs, dVs, sq, 1);
    if (rmse) hipLaunchKernelGGL(losskern::loss_rmse_kernel<T>, dim3(1), dim3(64), 0, stream, B, binum, sq, rmse);
    prof_end(stream);
    A2P_HIP_CHECK(hipGetLastError());
    if (!want_grad) return A2P_OK;
    a.E = table_entries<T>(a.p, K, true);
    a.cE = cE; a.dFs = dFs; a.dVs = dVs; a.gpart = gpart; a.ngrad = ngrad;
    rc = launch_atoms<T, true>(a, stream);
    if (rc) return rc;
    prof_begin("mtp_grad_reduce", stream);
    hipLaunchKernelGGL(mtp_grad_reduce_kernel<T>, dim3(ceil_div(ngrad, 256), B), dim3(256), 0, stream, P, ncoef,
                       a.p.n_scalar, ntypes, binum, gpart, dcoeffs, dlin, dbias);
    prof_end(stream);
    A2P_HIP_CHECK(hipGetLastError());
    return A2P_OK;
}

// Training loss of the neural-network MTP: E/F/V, per-structure loss and the per-structure gradients
// w.r.t. coeffs, w0, w1, type_bias (nnMtpLoss.h:141-181, 216-610; nnMtpOp.cc:1641-2780).
// exact = 0 evaluates the reference's backward formulas, which leave out two contributions of the
// force and virial terms: in d/dcoeffs the dependence of the adjoint on the moments (the mixed
// sweep of the linear MTP, linearMtpLoss.h:417-434, and the tanh'' term), and in d/dw0[p,k] the
// k' != k part of the tangent of the pre-activation (nnMtpLoss.h:497-529, 560-585).  exact = 1 is the
// complete derivative of the loss (it agrees with finite differences; the reference's does not).
template <typename T>
int nnmtp_loss(void* handle, double e_w, double f_w, double v_w, const T* e_dft, const T* f_dft, const T* v_dft,
               int K, const MtpNet<T>& net, const T* coeffs, const T* bias, int nmus, int ntypes,
               const T* q_scaler, double rmax, double rmin, int B, int P, int U, const int* binum,
               const int* bilist, const int* bnumneigh, const int* bfirstneigh, const T* brcs, const int* btypes,
               T* bloss, T* etot, T* force, T* virial, T* dcoeffs, T* dw0, T* dw1, T* dbias, int exact,
               hipStream_t stream)
{
    A2P_REQUIRE(e_dft && f_dft && v_dft && bloss && etot && force && virial, A2P_ERR_INVALID,
                "nnmtp loss: null label or output pointer");
    int rc = mtp_efv<T>(handle, K, 1.0, coeffs, nullptr, bias, nmus, ntypes, q_scaler, rmax, rmin, B, P, U, 0, binum,
                        bilist, bnumneigh, bfirstneigh, brcs, btypes, etot, force, virial, stream, &net);
    if (rc) return rc;
    if (B == 0 || P == 0) return A2P_OK;
    MtpPlan* plan = nullptr;
    rc = plan_check(handle, &plan);
    if (rc) return rc;
    MtpArgs<T> a;
    rc = fill_args(a, plan, K, 1.0, coeffs, (const T*)nullptr, bias, nmus, ntypes, q_scaler, rmax, rmin, B, P, U, 0,
                   binum, bilist, bnumneigh, bfirstneigh, brcs, btypes);
    if (rc) return rc;
    rc = set_net(a, &net);
    if (rc) return rc;
    const int S = a.p.n_scalar, H = net.H;
    const int nblk = ntypes * nmus * K;
    const int nrow = nblk + H * S + H + 1;
    const bool want_grad = dcoeffs || dw0 || dw1 || dbias;
    // workspace: cE[B] | dVs[B*9] | dFs[B*P*3] | gpart[B*P*nrow] | sq[B*3] (double)
    size_t nT = (size_t)B + (size_t)B * 9 + (size_t)B * P * 3 + (want_grad ? (size_t)B * P * nrow : 0);
    size_t bytesT = (nT * sizeof(T) + 15) / 16 * 16;
    void* ws = nullptr;
    rc = ws_get(WS_MTP, bytesT + (size_t)B * 3 * sizeof(double), &ws);
    if (rc) return rc;
    T* cE = (T*)ws;
    T* dVs = cE + B;
    T* dFs = dVs + (size_t)B * 9;
    T* gpart = dFs + (size_t)B * P * 3;
    double* sq = (double*)((char*)ws + bytesT);
    prof_begin("mtp_loss_forward", stream);
    hipLaunchKernelGGL(losskern::loss_forward_kernel<T>, dim3(B), dim3(256), 0, stream, P, binum, bilist, (T)e_w,
                       (T)f_w, (T)v_w, etot, e_dft, force, f_dft, virial, v_dft, bloss, cE, dFs, dVs, sq, 1);
    prof_end(stream);
    A2P_HIP_CHECK(hipGetLastError());
    if (!want_grad) return A2P_OK;
    a.E = table_entries<T>(a.p, K, true);
    a.cE = cE; a.dFs = dFs; a.dVs = dVs; a.gpart = gpart; a.ngrad = nrow;
    a.nn_exact = exact ? 1 : 0;
    rc = launch_atoms<T, true>(a, stream);
    if (rc) return rc;
    prof_begin("mtp_grad_reduce", stream);
    hipLaunchKernelGGL(nnmtp_grad_reduce_kernel<T>, dim3(ceil_div(nrow, 256), ntypes, B), dim3(256), 0, stream, P, P,
                       nblk, H * S, H, ntypes, binum, bilist, btypes, gpart, dcoeffs, dw0, dw1, dbias);
    prof_end(stream);
    A2P_HIP_CHECK(hipGetLastError());
    return A2P_OK;
}

// Site energies e_sites[B, P] (row order) and / or the scalar moments desc[B, P, n_scalar].
template <typename T>
int mtp_esites(void* handle, int K, double scaling, const T* coeffs, const T* lin, const T* bias, int nmus,
               int ntypes, const T* q_scaler, double rmax, double rmin, int B, int P, int U, int nghost,
               const int* binum, const int* bilist, const int* bnumneigh, const int* bfirstneigh, const T* brcs,
               const int* btypes, T* e_sites, T* desc, hipStream_t stream, const MtpNet<T>* net = nullptr)
{
    MtpPlan* plan = nullptr;
    int rc = plan_check(handle, &plan);
    if (rc) return rc;
    A2P_REQUIRE(e_sites || desc, A2P_ERR_INVALID, "mtp e_sites: no output requested");
    MtpArgs<T> a;
    rc = fill_args(a, plan, K, scaling, coeffs, lin, bias, nmus, ntypes, q_scaler, rmax, rmin, B, P, U, nghost,
                   binum, bilist, bnumneigh, bfirstneigh, brcs, btypes);
    if (rc) return rc;
    rc = set_net(a, net);
    if (rc) return rc;
    if (B == 0 || P == 0) return A2P_OK;
    a.E = table_entries<T>(a.p, K, false);
    a.e_sites = e_sites; a.desc = desc; a.energy_only = 1;
    return launch_atoms<T, false>(a, stream);
}

// sum over rows of gout[b, ii] * d e_sites[b, ii] / d(coeffs, linear_coeffs, type_bias), per structure:
// the loss-gradient kernel with the per-row weight in place of cE and no force / virial residuals.
template <typename T>
int mtp_esites_bwd(void* handle, int K, double scaling, const T* coeffs, const T* lin, const T* bias, int nmus,
                   int ntypes, const T* q_scaler, double rmax, double rmin, int B, int P, int U, int nghost,
                   const int* binum, const int* bilist, const int* bnumneigh, const int* bfirstneigh,
                   const T* brcs, const int* btypes, const T* gout, T* dcoeffs, T* dlin, T* dbias,
                   hipStream_t stream)
{
    MtpPlan* plan = nullptr;
    int rc = plan_check(handle, &plan);
    if (rc) return rc;
    A2P_REQUIRE(gout && lin && (dcoeffs || dlin || dbias), A2P_ERR_INVALID, "mtp e_sites backward: null pointer");
    MtpArgs<T> a;
    rc = fill_args(a, plan, K, scaling, coeffs, lin, bias, nmus, ntypes, q_scaler, rmax, rmin, B, P, U, nghost,
                   binum, bilist, bnumneigh, bfirstneigh, brcs, btypes);
    if (rc) return rc;
    if (B == 0 || P == 0) return A2P_OK;
    const int ncoef = ntypes * ntypes * nmus * K;
    const int ngrad = ncoef + a.p.n_scalar + ntypes;
    // workspace: dVs[B*9] | dFs[(B*P + nghost)*3] (both zero) | gpart[B*P*ngrad]
    const size_t nzero = (size_t)B * 9 + ((size_t)B * P + nghost) * 3;
    void* ws = nullptr;
    rc = ws_get(WS_MTP, (nzero + (size_t)B * P * ngrad) * sizeof(T), &ws);
    if (rc) return rc;
    T* dVs = (T*)ws;
    T* dFs = dVs + (size_t)B * 9;
    T* gpart = (T*)ws + nzero;
    rc = fill_zero(ws, ((nzero * sizeof(T) + 3) / 4) * 4, stream);
    if (rc) return rc;
    a.E = table_entries<T>(a.p, K, true);
    a.cE = gout; a.cE_per_atom = 1; a.no_tangent = 1; a.dFs = dFs; a.dVs = dVs; a.gpart = gpart; a.ngrad = ngrad;
    rc = launch_atoms<T, true>(a, stream);
    if (rc) return rc;
    prof_begin("mtp_grad_reduce", stream);
    hipLaunchKernelGGL(mtp_grad_reduce_kernel<T>, dim3(ceil_div(ngrad, 256), B), dim3(256), 0, stream, P, ncoef,
                       a.p.n_scalar, ntypes, binum, gpart, dcoeffs, dlin, dbias);
    prof_end(stream);
    A2P_HIP_CHECK(hipGetLastError());
    return A2P_OK;
}

// Backward of the legacy basis operator (mtpBasisOp.cc:220-326; mtpBasis.h:359-394 contracts the dense derivative
// arrays that find_val_der, :107-356, filled in the forward pass): with w = grad_desc[b, ii, :] the weights of
// the row's scalar moments,  drcs[b, ii, u, :] = sum_s w_s dM_s / d rcs[b, ii, u, :]  and
// dcoeffs[b, :] = sum_ii sum_s w_s dM_s / d coeffs.  Nothing dense is kept between the passes: the moments are
// recomputed and the adjoint sweep of the E/F/V kernel (pair derivatives) and of the loss-gradient kernel
// (coefficient gradient; with zero force and virial residuals its tangent vectors vanish) starts from w.
template <typename T>
int mtp_basis_bwd(void* handle, int K, double scaling, const T* coeffs, int nmus, int ntypes, double rmax,
                  double rmin, int B, int P, int U, int nghost, const int* binum, const int* bilist,
                  const int* bnumneigh, const int* bfirstneigh, const T* brcs, const int* btypes, const T* grad_desc,
                  T* drcs, T* dcoeffs, hipStream_t stream)
{
    MtpPlan* plan = nullptr;
    int rc = plan_check(handle, &plan);
    if (rc) return rc;
    A2P_REQUIRE(grad_desc && (drcs || dcoeffs), A2P_ERR_INVALID, "mtp basis backward: null pointer");
    MtpArgs<T> a;
    rc = fill_args(a, plan, K, scaling, coeffs, (const T*)nullptr, (const T*)nullptr, nmus, ntypes, (const T*)nullptr,
                   rmax, rmin, B, P, U, nghost, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, false);
    if (rc) return rc;
    if (B == 0 || P == 0) return A2P_OK;
    a.row_seed = grad_desc;
    if (drcs) {
        rc = fill_zero(drcs, (size_t)B * P * U * 3 * sizeof(T), stream);
        if (rc) return rc;
        MtpArgs<T> e = a;
        e.E = table_entries<T>(e.p, K, false);
        e.pair_out = drcs;
        rc = launch_atoms<T, false, true>(e, stream);
        if (rc) return rc;
    }
    if (dcoeffs) {
        const int ncoef = ntypes * ntypes * nmus * K;
        // workspace: dVs[B*9] | dFs[(B*P + nghost)*3] (both zero) | gpart[B*P*ncoef]
        const size_t nzero = (size_t)B * 9 + ((size_t)B * P + nghost) * 3;
        void* ws = nullptr;
        rc = ws_get(WS_MTP, (nzero + (size_t)B * P * ncoef) * sizeof(T), &ws);
        if (rc) return rc;
        T* dVs = (T*)ws;
        T* dFs = dVs + (size_t)B * 9;
        T* gpart = (T*)ws + nzero;
        rc = fill_zero(ws, ((nzero * sizeof(T) + 3) / 4) * 4, stream);
        if (rc) return rc;
        MtpArgs<T> g = a;
        g.E = table_entries<T>(g.p, K, true);
        g.dFs = dFs; g.dVs = dVs; g.gpart = gpart; g.ngrad = ncoef; g.no_tangent = 1;
        rc = launch_atoms<T, true>(g, stream);
        if (rc) return rc;
        prof_begin("mtp_grad_reduce", stream);
        hipLaunchKernelGGL(mtp_grad_reduce_kernel<T>, dim3(ceil_div(ncoef, 256), B), dim3(256), 0, stream, P, ncoef, 0, 0,
                           binum, gpart, dcoeffs, (T*)nullptr, (T*)nullptr);
        prof_end(stream);
        A2P_HIP_CHECK(hipGetLastError());
    }
    return A2P_OK;
}

// Which route a2p_mtp_lin_components_* takes: 1 = all columns in one pass over the atoms (when the plan has the node
// graph and it fits in LDS), 0 = one E/F/V pass per column.  AI2POT_MTP_COMPONENTS=passes|nodes sets the initial value,
// a2p_mtp_components_route changes it at run time.
int g_components_route = -1;
int components_route()
{
    if (g_components_route < 0) {
        const char* e = getenv("AI2POT_MTP_COMPONENTS");
        g_components_route = (e && std::string(e) == "passes") ? 0 : 1;
    }
    return g_components_route;
}

template <typename T>
int mtp_lin_components_nodes(MtpPlan* plan, MtpArgs<T>& a, int S, int n, T* ecomp, T* fcomp, T* vcomp,
                             hipStream_t stream)
{
    const int B = a.B, P = a.P, U = a.U;
    const int rows = B * P;
    // integer scratch: nnc[rows+1] | pair_off[rows+1] | cnt[rows+1] | ioff[rows+1] | row_of1[rows] | scan tmp
    const int ntmp = scan_tmp_ints(rows + 1);
    void* wsI = nullptr;
    int rc = ws_get(WS_CSR, ((size_t)(rows + 1) * 4 + rows + ntmp) * sizeof(int), &wsI);
    if (rc) return rc;
    int* nnc = (int*)wsI;
    int* pair_off = nnc + rows + 1;
    int* cnt = pair_off + rows + 1;
    int* ioff = cnt + rows + 1;
    int* row_of1 = ioff + rows + 1;
    int* tmp = row_of1 + rows;
    rc = fill_zero2(cnt, (size_t)(rows + 1) * sizeof(int), row_of1, (size_t)rows * sizeof(int), stream);
    if (rc) return rc;
    prof_begin("mtp_components_lists", stream);
    hipLaunchKernelGGL(comp_rows_kernel, dim3(ceil_div(rows + 1, 256)), dim3(256), 0, stream, B, P, U, a.ntypes, a.binum,
                       a.bilist, a.bnumneigh, a.btypes, nnc, row_of1, a.status);
    prof_end(stream);
    rc = exclusive_scan_i32(nnc, pair_off, rows + 1, tmp, stream);
    if (rc) return rc;
    int npairs = 0;                         // sizes the pair buffer: one read-back per call
    A2P_HIP_CHECK(hipMemcpyAsync(&npairs, pair_off + rows, sizeof(int), hipMemcpyDeviceToHost, stream));
    A2P_HIP_CHECK(hipStreamSynchronize(stream));
    if (npairs < 0) npairs = 0;
    // pair derivatives | row sums | scalar moments | list of the pairs that name each atom
    const size_t n_pb = (size_t)std::max(npairs, 1) * 3 * S, n_rp = (size_t)rows * 12 * S, n_desc = (size_t)rows * S;
    void* wsT = nullptr;
    rc = ws_get(WS_MTP, (n_pb + n_rp + n_desc) * sizeof(T) + ((size_t)npairs + 1) * sizeof(int), &wsT);
    if (rc) return rc;
    T* pb = (T*)wsT;
    T* rowpart = pb + n_pb;
    T* desc = rowpart + n_rp;
    int* inc = (int*)(desc + n_desc);
    const long long nslots = (long long)rows * U;
    prof_begin("mtp_components_lists", stream);
    hipLaunchKernelGGL(comp_incoming_kernel, dim3(ceil_div(nslots, 256)), dim3(256), 0, stream, B, P, U, (const int*)nnc,
                       (const int*)pair_off, a.bfirstneigh, cnt, (const int*)nullptr, (int*)nullptr);
    prof_end(stream);
    rc = exclusive_scan_i32(cnt, ioff, rows + 1, tmp, stream);
    if (rc) return rc;
    rc = fill_zero(cnt, (size_t)(rows + 1) * sizeof(int), stream);
    if (rc) return rc;
    prof_begin("mtp_components_lists", stream);
    hipLaunchKernelGGL(comp_incoming_kernel, dim3(ceil_div(nslots, 256)), dim3(256), 0, stream, B, P, U, (const int*)nnc,
                       (const int*)pair_off, a.bfirstneigh, cnt, (const int*)ioff, inc);
    hipLaunchKernelGGL(comp_incoming_sort_kernel, dim3(ceil_div(rows, 256)), dim3(256), 0, stream, rows, (const int*)ioff,
                       inc);
    prof_end(stream);

    CompArgs<T> c;
    c.pb = pb; c.pair_off = pair_off; c.nnc = nnc; c.desc = desc; c.rowpart = rowpart;
    auto kern = mtp_components_kernel<T, 256>;
    for (const MtpXBatch& xb : plan->xbatches) {
        MtpPlanDevice& p = a.p;
        p.x_nodes = xb.nodes; p.x_slots = xb.slots; p.x_root = xb.root; p.x_seed = xb.seed;
        p.x_level = xb.level; p.x_multi = xb.multi; p.x_src = xb.src; p.x_rem = xb.rem;
        p.x_gbase = xb.gbase; p.x_gdepth = xb.gdepth; p.x_terms = xb.terms;
        p.x_bbase = xb.bbase; p.x_bdepth = xb.bdepth; p.x_bsteps = xb.bsteps; p.x_brem = xb.brem; p.x_bwords = xb.bwords;
        // LDS: moments | node adjoints | coefficients | table of nc rows | 3 n_basic values per wavefront; then the
        // packed basic moments.  Workgroups per CU count first, then the longest table that still allows them.
        auto lds_for = [&](int nc, size_t* main) {
            const size_t vals = (size_t)p.n_moms + ((p.x_nodes + 2) & ~1) + (size_t)a.ntypes * p.nmus * a.K +
                                (size_t)nc * a.E + (size_t)4 * p.n_basic * 3;
            *main = (vals * sizeof(T) + 15) / 16 * 16;
            return *main + (size_t)p.n_basic * sizeof(unsigned);
        };
        auto per_cu = [](size_t l) { return (size_t)(160 * 1024) / ((l + 1279) / 1280 * 1280); };
        size_t m = 0;
        const size_t want = std::min<size_t>(per_cu(lds_for(MTP_NC_MIN, &m)), 8);
        A2P_REQUIRE(want >= 1, A2P_ERR_INVALID, "mtp components: %d moments need %zu bytes of LDS per atom", p.n_moms,
                    lds_for(MTP_NC_MIN, &m));
        int nc_cap = MTP_NC_MIN;
        for (int nc : {MTP_NC_MAX, 40, 32, 24, 20, MTP_NC_MIN})
            if (per_cu(lds_for(nc, &m)) >= want) { nc_cap = nc; break; }
        const size_t lds = lds_for(nc_cap, &m);
        c.nc_cap = nc_cap; c.lds_basic_off = (int)m;
        if (lds > 48 * 1024)
            A2P_HIP_CHECK(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        prof_begin("mtp_components_kernel", stream);
        hipLaunchKernelGGL(kern, dim3(P, B), dim3(256), lds, stream, a, c);
        prof_end(stream);
    }
    prof_begin("mtp_components_sums", stream);
    hipLaunchKernelGGL(comp_force_kernel<T>, dim3(rows, ceil_div(S, 64)), dim3(64), 0, stream, S, n, (const int*)row_of1,
                       (const int*)ioff, (const int*)inc, (const T*)pb, (const T*)rowpart, fcomp);
    const int nblocks = ceil_div(P, COMP_ROWS);
    void* wsP = nullptr;
    rc = ws_get(WS_MISC, (size_t)B * nblocks * 10 * S * sizeof(T), &wsP);
    if (rc) return rc;
    hipLaunchKernelGGL(comp_structure_blocks_kernel<T>, dim3(B, ceil_div(S, 64), nblocks), dim3(64), 0, stream, S, P,
                       nblocks, a.binum, (const T*)desc, (const T*)rowpart, (T*)wsP);
    hipLaunchKernelGGL(comp_structure_kernel<T>, dim3(B, ceil_div(S, 64)), dim3(64), 0, stream, n, S, nblocks, a.q_scaler,
                       (const T*)wsP, ecomp, vcomp);
    prof_end(stream);
    A2P_HIP_CHECK(hipGetLastError());
    return A2P_OK;
}

// Energy, force and virial of every linear parameter taken alone (linear_mtp_gram_and_cross.h:125-374):
// ecomp[B, n], fcomp[B, P, 3, n], vcomp[B, 9, n] with n = n_scalar + ntypes.  Column s < n_scalar is the
// E/F/V of the model with linear_coeffs = e_s and no bias (the reference obtains the same numbers by
// differentiating each scalar moment along every pair displacement); column n_scalar + t counts the
// atoms of species t in the energy and is zero in force and virial.  All columns come from one pass over the
// atoms (mtp_components_kernel); levels whose node graph is too large take one E/F/V pass per scalar moment.
template <typename T>
int mtp_lin_components(void* handle, int K, double scaling, const T* coeffs, int nmus, int ntypes,
                       const T* q_scaler, double rmax, double rmin, int B, int P, int U, const int* binum,
                       const int* bilist, const int* bnumneigh, const int* bfirstneigh, const T* brcs,
                       const int* btypes, T* ecomp, T* fcomp, T* vcomp, hipStream_t stream)
{
    MtpPlan* plan = nullptr;
    int rc = plan_check(handle, &plan);
    if (rc) return rc;
    A2P_REQUIRE(ecomp && fcomp && vcomp, A2P_ERR_INVALID, "mtp components: null output pointer");
    A2P_REQUIRE(ntypes >= 1 && B >= 0 && P >= 0, A2P_ERR_INVALID, "mtp components: bad shape");
    const int S = plan->d.n_scalar, n = S + ntypes;
    if (B == 0 || P == 0) return A2P_OK;
    rc = fill_zero(ecomp, (size_t)B * n * sizeof(T), stream);
    if (rc) return rc;
    rc = fill_zero(fcomp, (size_t)B * P * 3 * n * sizeof(T), stream);
    if (rc) return rc;
    rc = fill_zero(vcomp, (size_t)B * 9 * n * sizeof(T), stream);
    if (rc) return rc;
    // atoms of each species per structure (the bias columns of the energy)
    void* wsC = nullptr;
    rc = ws_get(WS_PARTIAL, (size_t)B * ntypes * sizeof(int), &wsC);
    if (rc) return rc;
    int* counts = (int*)wsC;
    rc = fill_zero(counts, (size_t)B * ntypes * sizeof(int), stream);
    if (rc) return rc;
    hipLaunchKernelGGL(species_count_kernel, dim3(ceil_div(B * P, 256)), dim3(256), 0, stream, B, P, ntypes, binum, bilist,
                       btypes, counts);
    A2P_HIP_CHECK(hipGetLastError());
    if (components_route() == 1 && !plan->xbatches.empty()) {
        MtpArgs<T> a;
        rc = fill_args(a, plan, K, scaling, coeffs, (const T*)nullptr, (const T*)nullptr, nmus, ntypes, q_scaler, rmax,
                       rmin, B, P, U, 0, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, false);
        if (rc) return rc;
        A2P_REQUIRE(q_scaler, A2P_ERR_INVALID, "mtp components: null q_scaler");
        a.E = table_entries<T>(a.p, K, false);
        hipLaunchKernelGGL(lin_components_init_kernel<T>, dim3(ceil_div(B * ntypes, 256)), dim3(256), 0, stream,
                           (T*)nullptr, S, ecomp, B, ntypes, (const int*)counts);
        A2P_HIP_CHECK(hipGetLastError());
        return mtp_lin_components_nodes<T>(plan, a, S, n, ecomp, fcomp, vcomp, stream);
    }
    // one E/F/V pass per scalar moment with a one-hot read-out
    // workspace: eye[S*S] | zero bias[ntypes] | etot[B] | force[B*P*3] | virial[B*9]
    const size_t nT = (size_t)S * S + ntypes + B + (size_t)B * P * 3 + (size_t)B * 9;
    void* ws = nullptr;
    rc = ws_get(WS_MISC, nT * sizeof(T), &ws);
    if (rc) return rc;
    T* eye = (T*)ws;
    T* zero_bias = eye + (size_t)S * S;
    T* etot = zero_bias + ntypes;
    T* force = etot + B;
    T* virial = force + (size_t)B * P * 3;
    rc = fill_zero(ws, (((size_t)S * S + ntypes) * sizeof(T) + 3) / 4 * 4, stream);
    if (rc) return rc;
    hipLaunchKernelGGL(lin_components_init_kernel<T>, dim3(ceil_div(std::max(S, B * ntypes), 256)), dim3(256), 0,
                       stream, eye, S, ecomp, B, ntypes, (const int*)counts);
    A2P_HIP_CHECK(hipGetLastError());
    for (int s = 0; s < S; s++) {
        // force / virial go to WS_MISC, which mtp_efv does not touch when a force pointer is given
        rc = mtp_efv<T>(handle, K, scaling, coeffs, eye + (size_t)s * S, zero_bias, nmus, ntypes, q_scaler, rmax, rmin,
                        B, P, U, 0, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, etot, force, virial, stream);
        if (rc) return rc;
        hipLaunchKernelGGL(column_store_kernel<T>, dim3(ceil_div(B, 256)), dim3(256), 0, stream, ecomp, etot,
                           (long long)B, n, s);
        hipLaunchKernelGGL(column_store_kernel<T>, dim3(ceil_div((long long)B * P * 3, 256)), dim3(256), 0, stream,
                           fcomp, force, (long long)B * P * 3, n, s);
        hipLaunchKernelGGL(column_store_kernel<T>, dim3(ceil_div(B * 9, 256)), dim3(256), 0, stream, vcomp, virial,
                           (long long)B * 9, n, s);
        A2P_HIP_CHECK(hipGetLastError());
    }
    return A2P_OK;
}

template <typename T>
int mtp_schmidt_orth(int ntypes, int nmus, int K, const T* coeffs, T* out, hipStream_t stream)
{
    A2P_REQUIRE(ntypes >= 1 && nmus >= 1 && K >= 1 && coeffs && out && coeffs != out, A2P_ERR_INVALID,
                "schmidt orth: bad argument");
    hipLaunchKernelGGL(schmidt_orth_kernel<T>, dim3(1), dim3(64), 0, stream, out, coeffs, ntypes * ntypes, nmus, K);
    A2P_HIP_CHECK(hipGetLastError());
    return A2P_OK;
}

// The same for the neural-network MTP: gradients w.r.t. coeffs, w0, w1, type_bias
// (nnMtp.h:756-990, contracted with gout as nnMtpOp.cc does after find_e_sites_backward).
template <typename T>
int nnmtp_esites_bwd(void* handle, int K, const MtpNet<T>& net, const T* coeffs, const T* bias, int nmus,
                     int ntypes, const T* q_scaler, double rmax, double rmin, int B, int P, int U, int nghost,
                     const int* binum, const int* bilist, const int* bnumneigh, const int* bfirstneigh,
                     const T* brcs, const int* btypes, const T* gout, T* dcoeffs, T* dw0, T* dw1, T* dbias,
                     hipStream_t stream)
{
    MtpPlan* plan = nullptr;
    int rc = plan_check(handle, &plan);
    if (rc) return rc;
    A2P_REQUIRE(gout && (dcoeffs || dw0 || dw1 || dbias), A2P_ERR_INVALID, "nnmtp e_sites backward: null pointer");
    MtpArgs<T> a;
    rc = fill_args(a, plan, K, 1.0, coeffs, (const T*)nullptr, bias, nmus, ntypes, q_scaler, rmax, rmin, B, P, U,
                   nghost, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes);
    if (rc) return rc;
    rc = set_net(a, &net);
    if (rc) return rc;
    if (B == 0 || P == 0) return A2P_OK;
    const int S = a.p.n_scalar, H = net.H;
    const int nblk = ntypes * nmus * K;
    const int nrow = nblk + H * S + H + 1;
    // workspace: dVs[B*9] | dFs[(B*P + nghost)*3] (both zero) | gpart[B*P*nrow]
    const size_t nzero = (size_t)B * 9 + ((size_t)B * P + nghost) * 3;
    void* ws = nullptr;
    rc = ws_get(WS_MTP, (nzero + (size_t)B * P * nrow) * sizeof(T), &ws);
    if (rc) return rc;
    T* dVs = (T*)ws;
    T* dFs = dVs + (size_t)B * 9;
    T* gpart = (T*)ws + nzero;
    rc = fill_zero(ws, ((nzero * sizeof(T) + 3) / 4) * 4, stream);
    if (rc) return rc;
    a.E = table_entries<T>(a.p, K, true);
    a.cE = gout; a.cE_per_atom = 1; a.no_tangent = 1; a.dFs = dFs; a.dVs = dVs; a.gpart = gpart; a.ngrad = nrow;
    rc = launch_atoms<T, true>(a, stream);
    if (rc) return rc;
    prof_begin("mtp_grad_reduce", stream);
    hipLaunchKernelGGL(nnmtp_grad_reduce_kernel<T>, dim3(ceil_div(nrow, 256), ntypes, B), dim3(256), 0, stream, P,
                       P + nghost, nblk, H * S, H, ntypes, binum, bilist, btypes, gpart, dcoeffs, dw0, dw1, dbias);
    prof_end(stream);
    A2P_HIP_CHECK(hipGetLastError());
    return A2P_OK;
}

}  // namespace
}  // namespace a2p

extern "C" {

int a2p_mtp_plan_create(int n_moms, int n_basic, const int* basic, int n_times, const int* times,
                        int n_scalar, const int* mapping, void** plan)
{
    A2P_REQUIRE(plan, A2P_ERR_INVALID, "mtp plan: null output");
    a2p::MtpPlan* p = nullptr;
    int rc = a2p::plan_create(n_moms, n_basic, basic, n_times, times, n_scalar, mapping, &p);
    if (rc) return rc;
    *plan = p;
    return A2P_OK;
}

int a2p_mtp_components_route(int route)
{
    const int before = a2p::components_route();
    if (route == 0 || route == 1) a2p::g_components_route = route;
    return before;
}

int a2p_mtp_plan_destroy(void* handle)
{
    a2p::MtpPlan* p = nullptr;
    int rc = a2p::plan_check(handle, &p);
    if (rc) return rc;
    {
        std::lock_guard<std::mutex> lock(a2p::g_plan_mutex);
        a2p::g_plans.erase(p);
    }
    A2P_HIP_CHECK(hipFree(p->device_block));
    delete p;
    return A2P_OK;
}

#define MTP_MODEL(T) int K, double scaling, const T* coeffs, const T* lin, const T* bias, int nmus, \
    int ntypes, const T* q_scaler, double rmax, double rmin
#define MTP_MODEL_PASS K, scaling, coeffs, lin, bias, nmus, ntypes, q_scaler, rmax, rmin
#define MTP_BATCH(T) const int* binum, const int* bilist, const int* bnumneigh, const int* bfirstneigh, \
    const T* brcs, const int* btypes
#define MTP_BATCH_PASS binum, bilist, bnumneigh, bfirstneigh, brcs, btypes

int a2p_mtp_efv_f64(void* plan, MTP_MODEL(double), int B, int P, int U, int nghost, MTP_BATCH(double),
                    double* etot, double* force, double* virial, void* stream)
{
    return a2p::mtp_efv<double>(plan, MTP_MODEL_PASS, B, P, U, nghost, binum, bilist, bnumneigh, bfirstneigh,
                                brcs, btypes, etot, force, virial, (hipStream_t)stream);
}

int a2p_mtp_efv_f32(void* plan, MTP_MODEL(float), int B, int P, int U, int nghost, MTP_BATCH(float),
                    float* etot, float* force, float* virial, void* stream)
{
    return a2p::mtp_efv<float>(plan, MTP_MODEL_PASS, B, P, U, nghost, binum, bilist, bnumneigh, bfirstneigh,
                               brcs, btypes, etot, force, virial, (hipStream_t)stream);
}

int a2p_mtp_loss_f64(void* plan, double e_weight, double f_weight, double v_weight, const double* e_dft,
                     const double* f_dft, const double* v_dft, MTP_MODEL(double), int B, int P, int U,
                     MTP_BATCH(double), double* bloss, double* rmse, double* etot, double* force,
                     double* virial, double* dcoeffs, double* dlinear, double* dbias, void* stream)
{
    return a2p::mtp_loss<double>(plan, e_weight, f_weight, v_weight, e_dft, f_dft, v_dft, MTP_MODEL_PASS, B, P,
                                 U, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, bloss, rmse, etot,
                                 force, virial, dcoeffs, dlinear, dbias, (hipStream_t)stream);
}

int a2p_mtp_loss_f32(void* plan, double e_weight, double f_weight, double v_weight, const float* e_dft,
                     const float* f_dft, const float* v_dft, MTP_MODEL(float), int B, int P, int U,
                     MTP_BATCH(float), float* bloss, float* rmse, float* etot, float* force, float* virial,
                     float* dcoeffs, float* dlinear, float* dbias, void* stream)
{
    return a2p::mtp_loss<float>(plan, e_weight, f_weight, v_weight, e_dft, f_dft, v_dft, MTP_MODEL_PASS, B, P,
                                U, binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, bloss, rmse, etot, force,
                                virial, dcoeffs, dlinear, dbias, (hipStream_t)stream);
}

int a2p_mtp_esites_f64(void* plan, MTP_MODEL(double), int B, int P, int U, int nghost, MTP_BATCH(double),
                       double* e_sites, double* descriptors, void* stream)
{
    return a2p::mtp_esites<double>(plan, MTP_MODEL_PASS, B, P, U, nghost, MTP_BATCH_PASS, e_sites, descriptors,
                                   (hipStream_t)stream);
}
int a2p_mtp_esites_f32(void* plan, MTP_MODEL(float), int B, int P, int U, int nghost, MTP_BATCH(float),
                       float* e_sites, float* descriptors, void* stream)
{
    return a2p::mtp_esites<float>(plan, MTP_MODEL_PASS, B, P, U, nghost, MTP_BATCH_PASS, e_sites, descriptors,
                                  (hipStream_t)stream);
}
#define NNMTP_ENTRY(T, SUFFIX)                                                                                  \
    int a2p_nnmtp_efv_##SUFFIX(void* plan, int K, int H, const T* coeffs, const T* w0, const T* w1, const T* bias, \
                               int nmus, int ntypes, const T* q_shifter, const T* q_scaler, double rmax,          \
                               double rmin, int B, int P, int U, int nghost, MTP_BATCH(T), T* etot, T* force,      \
                               T* virial, T* e_sites, void* stream)                                               \
    {                                                                                                           \
        a2p::MtpNet<T> net{H, w0, w1, q_shifter};                                                                 \
        if (!etot && !force && !virial)                                                                           \
            return a2p::mtp_esites<T>(plan, K, 1.0, coeffs, nullptr, bias, nmus, ntypes, q_scaler, rmax, rmin, B, \
                                      P, U, nghost, MTP_BATCH_PASS, e_sites, nullptr, (hipStream_t)stream, &net); \
        return a2p::mtp_efv<T>(plan, K, 1.0, coeffs, nullptr, bias, nmus, ntypes, q_scaler, rmax, rmin, B, P, U,   \
                               nghost, MTP_BATCH_PASS, etot, force, virial, (hipStream_t)stream, &net, e_sites);  \
    }
NNMTP_ENTRY(double, f64)
NNMTP_ENTRY(float, f32)

#define MTP_SOLVER_ENTRIES(T, SUFFIX)                                                                            \
    int a2p_mtp_lin_components_##SUFFIX(void* plan, int K, double scaling, const T* coeffs, int nmus, int ntypes,   \
                                        const T* q_scaler, double rmax, double rmin, int B, int P, int U,           \
                                        MTP_BATCH(T), T* ecomp, T* fcomp, T* vcomp, void* stream)                   \
    {                                                                                                             \
        return a2p::mtp_lin_components<T>(plan, K, scaling, coeffs, nmus, ntypes, q_scaler, rmax, rmin, B, P, U,    \
                                          MTP_BATCH_PASS, ecomp, fcomp, vcomp, (hipStream_t)stream);                \
    }                                                                                                             \
    int a2p_mtp_schmidt_orth_##SUFFIX(int ntypes, int nmus, int K, const T* coeffs, T* orth_coeffs, void* stream)   \
    {                                                                                                             \
        return a2p::mtp_schmidt_orth<T>(ntypes, nmus, K, coeffs, orth_coeffs, (hipStream_t)stream);                 \
    }
MTP_SOLVER_ENTRIES(double, f64)
MTP_SOLVER_ENTRIES(float, f32)

#define NNMTP_ESITES_BWD_ENTRY(T, SUFFIX)                                                                         \
    int a2p_nnmtp_esites_bwd_##SUFFIX(void* plan, int K, int H, const T* coeffs, const T* w0, const T* w1,          \
                                      const T* bias, int nmus, int ntypes, const T* q_shifter, const T* q_scaler,   \
                                      double rmax, double rmin, int B, int P, int U, int nghost, MTP_BATCH(T),      \
                                      const T* grad_e_sites, T* dcoeffs, T* dw0, T* dw1, T* dbias, void* stream)    \
    {                                                                                                             \
        a2p::MtpNet<T> net{H, w0, w1, q_shifter};                                                                   \
        return a2p::nnmtp_esites_bwd<T>(plan, K, net, coeffs, bias, nmus, ntypes, q_scaler, rmax, rmin, B, P, U,    \
                                        nghost, MTP_BATCH_PASS, grad_e_sites, dcoeffs, dw0, dw1, dbias,            \
                                        (hipStream_t)stream);                                                       \
    }
NNMTP_ESITES_BWD_ENTRY(double, f64)
NNMTP_ESITES_BWD_ENTRY(float, f32)

#define NNMTP_LOSS_ENTRY(T, SUFFIX)                                                                              \
    int a2p_nnmtp_loss_##SUFFIX(void* plan, double e_w, double f_w, double v_w, const T* e_dft, const T* f_dft,    \
                                const T* v_dft, int K, int H, const T* coeffs, const T* w0, const T* w1,           \
                                const T* bias, int nmus, int ntypes, const T* q_shifter, const T* q_scaler,        \
                                double rmax, double rmin, int B, int P, int U, MTP_BATCH(T), T* bloss, T* etot,    \
                                T* force, T* virial, T* dcoeffs, T* dw0, T* dw1, T* dbias, int exact_gradient,     \
                                void* stream)                                                                      \
    {                                                                                                            \
        a2p::MtpNet<T> net{H, w0, w1, q_shifter};                                                                  \
        return a2p::nnmtp_loss<T>(plan, e_w, f_w, v_w, e_dft, f_dft, v_dft, K, net, coeffs, bias, nmus, ntypes,    \
                                  q_scaler, rmax, rmin, B, P, U, MTP_BATCH_PASS, bloss, etot, force, virial,       \
                                  dcoeffs, dw0, dw1, dbias, exact_gradient, (hipStream_t)stream);                  \
    }
NNMTP_LOSS_ENTRY(double, f64)
NNMTP_LOSS_ENTRY(float, f32)

int a2p_mtp_esites_bwd_f64(void* plan, MTP_MODEL(double), int B, int P, int U, int nghost, MTP_BATCH(double),
                           const double* grad_e_sites, double* dcoeffs, double* dlinear, double* dbias, void* stream)
{
    return a2p::mtp_esites_bwd<double>(plan, MTP_MODEL_PASS, B, P, U, nghost, MTP_BATCH_PASS, grad_e_sites, dcoeffs,
                                       dlinear, dbias, (hipStream_t)stream);
}
int a2p_mtp_esites_bwd_f32(void* plan, MTP_MODEL(float), int B, int P, int U, int nghost, MTP_BATCH(float),
                           const float* grad_e_sites, float* dcoeffs, float* dlinear, float* dbias, void* stream)
{
    return a2p::mtp_esites_bwd<float>(plan, MTP_MODEL_PASS, B, P, U, nghost, MTP_BATCH_PASS, grad_e_sites, dcoeffs,
                                      dlinear, dbias, (hipStream_t)stream);
}

int a2p_mtp_basis_bwd_f64(void* plan, int K, double scaling, const double* coeffs, int nmus, int ntypes, double rmax,
                          double rmin, int B, int P, int U, int nghost, MTP_BATCH(double), const double* grad_desc,
                          double* drcs, double* dcoeffs, void* stream)
{
    return a2p::mtp_basis_bwd<double>(plan, K, scaling, coeffs, nmus, ntypes, rmax, rmin, B, P, U, nghost,
                                      MTP_BATCH_PASS, grad_desc, drcs, dcoeffs, (hipStream_t)stream);
}

int a2p_mtp_basis_bwd_f32(void* plan, int K, double scaling, const float* coeffs, int nmus, int ntypes, double rmax,
                          double rmin, int B, int P, int U, int nghost, MTP_BATCH(float), const float* grad_desc,
                          float* drcs, float* dcoeffs, void* stream)
{
    return a2p::mtp_basis_bwd<float>(plan, K, scaling, coeffs, nmus, ntypes, rmax, rmin, B, P, U, nghost,
                                     MTP_BATCH_PASS, grad_desc, drcs, dcoeffs, (hipStream_t)stream);
}
}
