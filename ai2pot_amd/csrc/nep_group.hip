// NEP energy / force / virial, lane-group kernel for the common model shapes
// (chebyshev_size 8, n_radial 4 or 6, n_angular 4, l_max 4, up to 4 species), used for small systems:
// it spreads an atom over 8 lanes and a workgroup over 32 atoms, so a few thousand atoms already
// occupy the device, at the price of more instructions per atom than the staged kernel.
//
// The generic kernel (nep.hip) gives every atom one thread that walks its neighbour row four
// times: each wave-wide load touches 64 different cache lines, rows are re-read from HBM, and
// the pair derivatives pass through a [row, slot, 3] buffer.  This kernel is built around the
// memory system instead:
//   * GL = 8 lanes work on one atom, a wave on 8 atoms, a workgroup of 256 threads on 32;
//   * a wave reads the rows of its atoms one after the other with lane = slot, i.e. whole rows
//     as contiguous, fully used cache lines, exactly once; the same lanes gather the
//     neighbour's species and claim the pair's place in its target's reduction segment with an
//     integer atomic (a2p::PairCsr, fixed-capacity segments), classify the pair against the two cutoffs and compact the row with
//     wave ballots into LDS: pairs inside the angular cutoff from the front of the atom's
//     tile, radial-only pairs from the back;
//   * the tile stays in LDS for both passes (rows longer than the tile are processed in
//     several tiles and only then read twice), so nothing per pair is spilled to global memory;
//   * the 8 lanes of an atom take the compacted entries round-robin; per-atom sums (radial
//     sums per species, angular moments, hidden-layer partial sums, own force) are combined
//     with a fixed three-step DPP butterfly, which leaves the identical total in all 8 lanes;
//   * the hidden layer is split over the 8 lanes by neuron;
//   * pair derivatives are stored straight into the reduction segments.
// Pass 1: radial sums, angular moments; then descriptors, hidden layer, dE/dq, dE/dS.
// Pass 2: pair derivatives (radial and angular part of a pair together), own force, virial.
//
// Formulas: source/descriptor/nep/include/{nepBasis.h:57-196; nep.h:320-529}.
#include "a2p_common.h"
#include "nep_device.h"

#include <type_traits>

namespace a2p {
using namespace nepdev;
namespace {

constexpr int GL = 8;                    // lanes per atom
constexpr int GTHREADS = 256;            // threads per workgroup
constexpr int GATOMS = GTHREADS / GL;    // atoms per workgroup
constexpr int GWAVES = GTHREADS / 64;
constexpr int FDP = 24;                  // padded descriptor count (at most 24: n_radial <= 8)
constexpr int KC = 8, NAC = 4, LC = 4, NLM = 24;     // n_radial: template parameter NR of the kernel (4 and 6)

// Tile capacity (pairs per atom held in LDS) and padded tile length.  With CAPP = 8 (mod 16)
// the 16-byte entry reads of 16 consecutive lanes (2 atoms x 8 lanes) fall into distinct banks.
template <typename T> struct Tile { static constexpr int CAP = sizeof(T) == 4 ? 64 : 32; static constexpr int CAPP = CAP + 8; };

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

// tile entries: [x y z species]
__device__ __forceinline__ void ent_store(float* p, float x, float y, float z, int w)
{
    *reinterpret_cast<float4*>(p) = make_float4(x, y, z, __int_as_float(w));
}
__device__ __forceinline__ void ent_load(const float* p, float& x, float& y, float& z, int& w)
{
    const float4 v = *reinterpret_cast<const float4*>(p);
    x = v.x; y = v.y; z = v.z; w = __float_as_int(v.w);
}
__device__ __forceinline__ void ent_store(double* p, double x, double y, double z, int w)
{
    *reinterpret_cast<double2*>(p) = make_double2(x, y);
    *reinterpret_cast<double2*>(p + 2) = make_double2(z, __longlong_as_double((long long)w));
}
__device__ __forceinline__ void ent_load(const double* p, double& x, double& y, double& z, int& w)
{
    const double2 v0 = *reinterpret_cast<const double2*>(p);
    const double2 v1 = *reinterpret_cast<const double2*>(p + 2);
    x = v0.x; y = v0.y; z = v1.x; w = (int)__double_as_longlong(v1.y);
}

// ---- sum over the 8 lanes of an atom; every lane receives the same bits ---------------------
// lane ^ 1 and lane ^ 2 inside a quad, then the mirror image inside the half row (lane i <-> 7-i),
// which pairs the two quads.
template <int CTRL>
__device__ __forceinline__ int dpp_move(int v)
{
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, true);
}
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) { return __int_as_float(dpp_move<CTRL>(__float_as_int(v))); }
template <int CTRL>
__device__ __forceinline__ double dpp_move(double v)
{
    const long long b = __double_as_longlong(v);
    const int lo = dpp_move<CTRL>((int)(b & 0xffffffffll));
    const int hi = dpp_move<CTRL>((int)(b >> 32));
    return __longlong_as_double(((long long)hi << 32) | (unsigned int)lo);
}
template <typename T>
__device__ __forceinline__ T group_sum(T v)
{
    v += dpp_move<0xB1>(v);    // quad_perm [1,0,3,2]
    v += dpp_move<0x4E>(v);    // quad_perm [2,3,0,1]
    v += dpp_move<0x141>(v);   // row_half_mirror
    return v;
}

template <typename T>
struct GroupLds {
    T *w0, *coef, *b0, *w1, *qs;   // model tables
    T* ent;                        // [GATOMS][CAPP][4] tile entries
    int* pos;                      // [GATOMS][CAPP] place of the pair in its reduction segment
    T* cc;                         // [GATOMS][NTC][KC] radial coefficients contracted with dE/dq
    double* red;
};

__host__ __device__ __forceinline__ size_t lds_round16(size_t bytes) { return (bytes + 15) & ~(size_t)15; }

template <typename T>
__host__ __device__ __forceinline__ size_t group_lds_layout(int ntypes, int H, int ntc, int nb, unsigned char* base,
                                                            GroupLds<T>& L)
{
    constexpr int CAPP = Tile<T>::CAPP;
    size_t off = 0;
    L.w0 = (T*)(base + off);   off += lds_round16((size_t)ntypes * H * FDP * sizeof(T));
    L.coef = (T*)(base + off); off += lds_round16((size_t)ntypes * ntypes * nb * KC * sizeof(T));
    L.b0 = (T*)(base + off);   off += lds_round16((size_t)ntypes * H * sizeof(T));
    L.w1 = (T*)(base + off);   off += lds_round16((size_t)ntypes * H * sizeof(T));
    L.qs = (T*)(base + off);   off += lds_round16((size_t)FDP * sizeof(T));
    L.ent = (T*)(base + off);  off += lds_round16((size_t)GATOMS * CAPP * 4 * sizeof(T));
    L.pos = (int*)(base + off); off += lds_round16((size_t)GATOMS * CAPP * sizeof(int));
    L.cc = (T*)(base + off);   off += lds_round16((size_t)GATOMS * ntc * KC * sizeof(T));
    L.red = (double*)(base + off); off += lds_round16((size_t)GWAVES * 10 * sizeof(double));
    return off;
}

struct SegArgs {
    int* cursor;   // [B * NF] entries claimed so far in each target's reduction segment, or null (no forces)
    int cap;       // capacity of a segment
    int spare;     // entry that takes what overflows a segment
};

// Load slots [t*CAP, (t+1)*CAP) of the rows of the wave's 8 atoms (lane = slot) and compact them
// into the atoms' tiles.  nn and the returned counts are per lane-group (atom); nA / nR are the
// numbers of entries at the front (inside the angular cutoff) / back (radial only) of the
// caller's own tile.
template <typename T>
__device__ __forceinline__ void load_tile(const NepArgs<T>& a, const SegArgs& seg, T* __restrict__ seg_g,
                                          const GroupLds<T>& L, int t, int lane, int wave, size_t wave_row0, int b,
                                          int NF, int nn, T rr, T ra, int& nA, int& nR, bool claim)
{
    constexpr int CAP = Tile<T>::CAP, CAPP = Tile<T>::CAPP;
    const int* types = a.btypes + (size_t)b * NF;
    const unsigned long long lt = (1ull << lane) - 1ull;
    const int grp = lane >> 3;
#pragma unroll 2
    for (int j = 0; j < 8; j++) {
        const int nn_j = __builtin_amdgcn_readlane(nn, j * GL);
        const int slot = t * CAP + lane;
        T x = (T)0, y = (T)0, z = (T)0;
        int tj = 0, pos = 0;
        bool valid = lane < CAP && slot < nn_j;
        if (valid) {
            const size_t pr = (wave_row0 + j) * a.U + slot;
            const int nj = a.bfirstneigh[pr];
            if ((unsigned)nj >= (unsigned)NF) {
                atomicOr(a.status, ST_BAD_NEIGHBOR);
                valid = false;
            } else {
                const T* p = a.brcs + pr * 3;
                x = p[0]; y = p[1]; z = p[2];
                tj = types[nj];
                if (seg.cursor && claim) {
                    // fixed-capacity segments: the pair claims its entry here (a2p::PairCsr), or takes the place
                    // an earlier call on the same list recorded (no atomic then; the call that claims records)
                    const int tg = b * NF + nj;
                    int rk;
                    if (a.brank && a.ranks_valid) {
                        rk = a.brank[pr];
                    } else {
                        rk = atomicAdd(&seg.cursor[tg], 1);
                        if (a.brank) a.brank[pr] = rk;
                    }
                    pos = (unsigned)rk < (unsigned)seg.cap ? tg * seg.cap + rk : seg.spare;
                    if ((unsigned)rk >= (unsigned)seg.cap) atomicOr(a.status, ST_SEG_OVERFLOW);
                }
                if ((unsigned)tj >= (unsigned)a.ntypes) { atomicOr(a.status, ST_BAD_TYPE); tj = 0; }
            }
        }
        const T r = sqrt_t(x * x + y * y + z * z);
        const bool inA = valid && r <= ra && r <= rr;   // nepBasis.h:106, 135: beyond the radial cutoff a neighbour is skipped
        const bool inR = valid && !inA && r <= rr;
        const unsigned long long mA = __ballot(inA), mR = __ballot(inR);
        T* ent = L.ent + (size_t)(wave * 8 + j) * CAPP * 4;
        int* epos = L.pos + (wave * 8 + j) * CAPP;
        if (inA || inR) {
            const int k = inA ? __popcll(mA & lt) : CAP - 1 - __popcll(mR & lt);
            ent_store(ent + k * 4, x, y, z, tj);
            epos[k] = pos;
        } else if (valid && seg_g && claim) {
            // a pair of the list beyond both cutoffs still owns a place in its segment
            T* dst = seg_g + (size_t)pos * 3;
            dst[0] = (T)0; dst[1] = (T)0; dst[2] = (T)0;
        }
        if (grp == j) { nA = __popcll(mA); nR = __popcll(mR); }
    }
    __builtin_amdgcn_wave_barrier();
}

template <typename T, int NTC, int NR>
__global__ void __launch_bounds__(GTHREADS, (sizeof(T) == 4 ? 2 : 1))
nep_group_kernel(const NepArgs<T> a, const SegArgs seg, T* __restrict__ seg_g)
{
    constexpr int CAP = Tile<T>::CAP, CAPP = Tile<T>::CAPP;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int sub = lane & (GL - 1);
    const int al = tid >> 3;                       // atom slot of this lane group in the workgroup
    const int b = blockIdx.y;
    const int ii = blockIdx.x * GATOMS + al;
    const int H = a.H, nt = a.ntypes;
    const int NF = a.P + a.nghost;
    constexpr int NRC = NR, NB = NR + NAC, DC = NR + NAC * LC;
    static_assert(DC <= FDP, "descriptor count exceeds the padded row");
    GroupLds<T> L;
    group_lds_layout<T>(nt, H, NTC, NB, smem_raw, L);

    for (int i = tid; i < nt * H * FDP; i += GTHREADS) {
        const int r = i / FDP, j = i - r * FDP;
        L.w0[i] = j < DC ? a.w0[(size_t)r * DC + j] : (T)0;
    }
    for (int i = tid; i < nt * nt * NB * KC; i += GTHREADS) L.coef[i] = a.coeffs[i];
    for (int i = tid; i < nt * H; i += GTHREADS) { L.b0[i] = a.b0[i]; L.w1[i] = a.w1[i]; }
    if (tid < FDP) L.qs[tid] = tid < DC ? (T)1 / a.q_scaler[tid] : (T)0;

    const int inum = a.binum[b];
    const bool active = ii < inum;
    const size_t row = (size_t)b * a.P + ii;
    const size_t wave_row0 = (size_t)b * a.P + (size_t)blockIdx.x * GATOMS + wave * 8;
    int center = 0, ti = 0, nn = 0;
    if (active) {
        center = a.bilist[row];
        nn = a.bnumneigh[row];
        if (nn > a.U) { atomicOr(a.status, ST_NEIGH_OVERFLOW); nn = a.U; }
        if ((unsigned)center >= (unsigned)NF) { atomicOr(a.status, ST_BAD_NEIGHBOR); center = 0; nn = 0; }
        ti = a.btypes[(size_t)b * NF + center];
        if ((unsigned)ti >= (unsigned)nt) { atomicOr(a.status, ST_BAD_TYPE); ti = 0; nn = 0; }
    }
    __syncthreads();
    const int ntiles = (wave_max(nn) + CAP - 1) / CAP;     // wave-uniform

    const T rr = a.rr, ra = a.ra;
    const T rr_inv = (T)1 / rr, ra_inv = (T)1 / ra;
    const T* ent = L.ent + (size_t)al * CAPP * 4;
    const int* epos = L.pos + al * CAPP;

    T S[NAC][NLM];
#pragma unroll
    for (int n = 0; n < NAC; n++)
#pragma unroll
        for (int m = 0; m < NLM; m++) S[n][m] = (T)0;
    T F[NTC][KC];
#pragma unroll
    for (int t = 0; t < NTC; t++)
#pragma unroll
        for (int k = 0; k < KC; k++) F[t][k] = (T)0;

    // ---- pass 1 -------------------------------------------------------------------------------
    int nA = 0, nR = 0;
    for (int t = 0; t < ntiles; t++) {
        if (t > 0) __builtin_amdgcn_wave_barrier();
        // a tile is loaded once when the rows fit one tile and again in pass 2 otherwise: the pairs
        // claim their segment entries in the last load
        load_tile<T>(a, seg, seg_g, L, t, lane, wave, wave_row0, b, NF, nn, rr, ra, nA, nR, ntiles == 1);
        for (int k = sub; k < nA; k += GL) {
            T x, y, z;
            int tj;
            ent_load(ent + k * 4, x, y, z, tj);
            const T r = sqrt_t(x * x + y * y + z * z);
            const T rinv = (T)1 / r;
            T f[KC], df[KC];
            if (r <= rr) {
                radial_basis<T, KC, false>(r, rr_inv, KC, f, df);
#pragma unroll
                for (int t2 = 0; t2 < NTC; t2++)
#pragma unroll
                    for (int kk = 0; kk < KC; kk++) F[t2][kk] += (tj == t2) ? f[kk] : (T)0;
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
                for (int kk = 0; kk < 4; kk++) g += c0v[kk] * f[kk];
#pragma unroll
                for (int kk = 0; kk < 4; kk++) g += c1v[kk] * f[4 + kk];
#pragma unroll
                for (int m = 0; m < NLM; m++) S[n][m] += g * bl[m];
            }
        }
        for (int k = sub; k < nR; k += GL) {
            T x, y, z;
            int tj;
            ent_load(ent + (CAP - 1 - k) * 4, x, y, z, tj);
            const T r = sqrt_t(x * x + y * y + z * z);
            T f[KC], df[KC];
            radial_basis<T, KC, false>(r, rr_inv, KC, f, df);
#pragma unroll
            for (int t2 = 0; t2 < NTC; t2++)
#pragma unroll
                for (int kk = 0; kk < KC; kk++) F[t2][kk] += (tj == t2) ? f[kk] : (T)0;
        }
    }
    // totals over the atom's lanes
#pragma unroll
    for (int t = 0; t < NTC; t++)
#pragma unroll
        for (int k = 0; k < KC; k++) F[t][k] = group_sum(F[t][k]);
#pragma unroll
    for (int n = 0; n < NAC; n++)
#pragma unroll
        for (int m = 0; m < NLM; m++) S[n][m] = group_sum(S[n][m]);

    // ---- descriptors --------------------------------------------------------------------------
    T q[DC];
#pragma unroll
    for (int j = 0; j < DC; j++) q[j] = (T)0;
#pragma unroll
    for (int t = 0; t < NTC; t++) {
        if (t < nt) {
            const T* c = L.coef + (ti * nt + t) * NB * KC;
#pragma unroll
            for (int n = 0; n < NRC; n++) {
                T c0v[4], c1v[4];
                lds_load4(c + n * KC, c0v);
                lds_load4(c + n * KC + 4, c1v);
#pragma unroll
                for (int k = 0; k < 4; k++) q[n] += c0v[k] * F[t][k];
#pragma unroll
                for (int k = 0; k < 4; k++) q[n] += c1v[k] * F[t][4 + k];
            }
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
    if (active && a.desc && sub == 0) {
        T* dst = a.desc + row * DC;
#pragma unroll
        for (int j = 0; j < DC; j++) dst[j] = q[j];
    }

    // ---- hidden layer (nep.h:415-447), neurons split over the atom's lanes ---------------------
    T dEdq[DC];
    T e_site = (T)0;
    {
        T qn[DC];
#pragma unroll
        for (int j = 0; j < DC; j++) { qn[j] = q[j] * L.qs[j]; dEdq[j] = (T)0; }
        for (int p = sub; p < H; p += GL) {
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
            const T th = tanh_t(h);
            const T w1p = L.w1[ti * H + p];
            e_site += w1p * th;
            const T sde = w1p * ((T)1 - th * th);
#pragma unroll
            for (int j = 0; j < DC; j++) dEdq[j] += sde * wv[j];
        }
        e_site = group_sum(e_site);
        if (active) e_site += a.bias[ti];
#pragma unroll
        for (int j = 0; j < DC; j++) dEdq[j] = group_sum(dEdq[j]) * L.qs[j];
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
        // radial coefficients contracted with dE/dq: lane `sub` makes cc[t][k = sub] for every
        // neighbour species t
        T* ccw = L.cc + (size_t)al * NTC * KC;
#pragma unroll
        for (int t = 0; t < NTC; t++) {
            T v = (T)0;
            if (t < nt) {
                const T* c = L.coef + (ti * nt + t) * NB * KC + sub;
#pragma unroll
                for (int n = 0; n < NRC; n++) v += dEdq[n] * c[n * KC];
            }
            ccw[t * KC + sub] = v;
        }
        __builtin_amdgcn_wave_barrier();
        auto emit = [&](int pos, T x, T y, T z, T gx, T gy, T gz) __attribute__((always_inline)) {
            if (seg_g) {
                T* dst = seg_g + (size_t)pos * 3;
                dst[0] = gx; dst[1] = gy; dst[2] = gz;
            }
            fx += gx; fy += gy; fz += gz;
            vir[0] -= gx * x; vir[1] -= gx * y; vir[2] -= gx * z;
            vir[3] -= gy * x; vir[4] -= gy * y; vir[5] -= gy * z;
            vir[6] -= gz * x; vir[7] -= gz * y; vir[8] -= gz * z;
        };
        for (int t = 0; t < ntiles; t++) {
            if (ntiles > 1) {      // the tiles of pass 1 are gone: read the rows again
                __builtin_amdgcn_wave_barrier();
                load_tile<T>(a, seg, seg_g, L, t, lane, wave, wave_row0, b, NF, nn, rr, ra, nA, nR, true);
            }
            // pairs inside the angular cutoff, radial and angular part together
            for (int k = sub; k < nA; k += GL) {
                T x, y, z;
                int tj;
                ent_load(ent + k * 4, x, y, z, tj);
                const int pos = epos[k];
                const T r = sqrt_t(x * x + y * y + z * z);
                const T rinv = (T)1 / r;
                const T ux = x * rinv, uy = y * rinv, uz = z * rinv;
                T f[KC], df[KC];
                T srad = (T)0;
                if (r <= rr) {
                    radial_basis<T, KC, true>(r, rr_inv, KC, f, df);
                    T c0v[4], c1v[4];
                    lds_load4(ccw + tj * KC, c0v);
                    lds_load4(ccw + tj * KC + 4, c1v);
#pragma unroll
                    for (int kk = 0; kk < 4; kk++) srad += c0v[kk] * df[kk];
#pragma unroll
                    for (int kk = 0; kk < 4; kk++) srad += c1v[kk] * df[4 + kk];
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
                    for (int kk = 0; kk < 4; kk++) { g += c0v[kk] * f[kk]; dg += c0v[kk] * df[kk]; }
#pragma unroll
                    for (int kk = 0; kk < 4; kk++) { g += c1v[kk] * f[4 + kk]; dg += c1v[kk] * df[4 + kk]; }
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
                emit(pos, x, y, z, srad * ux + wx * rinv, srad * uy + wy * rinv, srad * uz + wz * rinv);
            }
            // radial-only pairs
            for (int k = sub; k < nR; k += GL) {
                T x, y, z;
                int tj;
                ent_load(ent + (CAP - 1 - k) * 4, x, y, z, tj);
                const int pos = epos[CAP - 1 - k];
                const T r = sqrt_t(x * x + y * y + z * z);
                T f[KC], df[KC];
                radial_basis<T, KC, true>(r, rr_inv, KC, f, df);
                T c0v[4], c1v[4];
                lds_load4(ccw + tj * KC, c0v);
                lds_load4(ccw + tj * KC + 4, c1v);
                T sr = (T)0;
#pragma unroll
                for (int kk = 0; kk < 4; kk++) sr += c0v[kk] * df[kk];
#pragma unroll
                for (int kk = 0; kk < 4; kk++) sr += c1v[kk] * df[4 + kk];
                sr /= r;
                emit(pos, x, y, z, sr * x, sr * y, sr * z);
            }
        }
        fx = group_sum(fx); fy = group_sum(fy); fz = group_sum(fz);
        if (active && a.force && sub == 0) {
            T* fo = a.force + ((size_t)b * NF + center) * 3;
            fo[0] = fx; fo[1] = fy; fo[2] = fz;
        }
    }

    // ---- workgroup partial sums of energy and virial (fp64) ---------------------------------
    double vals[10];
    vals[0] = (active && sub == 0) ? (double)e_site : 0.0;
#pragma unroll
    for (int i = 0; i < 9; i++) vals[1 + i] = (double)vir[i];
#pragma unroll
    for (int i = 0; i < 10; i++) {
        double v = wave_sum(vals[i]);
        if (lane == 0) L.red[wave * 10 + i] = v;
    }
    __syncthreads();
    if (tid < 10) {
        double v = 0.0;
        for (int w = 0; w < GWAVES; w++) v += L.red[w * 10 + tid];
        a.partial[((size_t)b * a.nblocks + blockIdx.x) * 10 + tid] = v;
    }
}

template <typename T, int NTC, int NR>
int launch_group(const NepArgs<T>& a, size_t lds, const PairCsr& csr, hipStream_t stream)
{
    SegArgs seg{csr.cursor, csr.seg_cap, csr.n * csr.seg_cap};
    auto kern = nep_group_kernel<T, NTC, NR>;
    if (lds > 48 * 1024)
        A2P_HIP_CHECK(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                                          (int)lds));
    prof_begin("nep_group_kernel", stream);
    hipLaunchKernelGGL(kern, dim3(a.nblocks, a.B), dim3(GTHREADS), lds, stream, a, seg, (T*)csr.seg_g);
    prof_end(stream);
    A2P_HIP_CHECK(hipGetLastError());
    return A2P_OK;
}

int ntc_of(int ntypes) { return ntypes <= 1 ? 1 : ntypes == 2 ? 2 : ntypes == 3 ? 3 : 4; }

}  // namespace

int nep_group_nblocks(int P) { return ceil_div(P, GATOMS); }

template <typename T>
bool nep_group_supported(const NepArgs<T>& a, size_t* lds_bytes)
{
    if (!(a.K == KC && (a.n_r == 4 || a.n_r == 6) && a.n_a == NAC && a.l_max == LC && a.ntypes <= 4)) return false;
    GroupLds<T> unused;
    *lds_bytes = group_lds_layout<T>(a.ntypes, a.H, ntc_of(a.ntypes), a.n_r + NAC, nullptr, unused);
    return *lds_bytes <= 150 * 1024;
}

template <typename T>
int nep_group_run(const NepArgs<T>& a, size_t lds_bytes, T* etot, T* virial, hipStream_t stream)
{
    PairCsr csr{};
    int rc;
    if (a.force) {
        rc = pair_fixed_begin<T>(&csr, a.B, a.P, a.U, a.nghost, stream, a.force,
                                 (size_t)a.B * (a.P + a.nghost) * 3 * sizeof(T), a.bincoming,
                                 a.bincoming != nullptr && a.ranks_valid != 0);
        if (rc) return rc;
    }
    auto launch = [&](auto nr) {
        constexpr int NR = decltype(nr)::value;
        switch (ntc_of(a.ntypes)) {
        case 1: return launch_group<T, 1, NR>(a, lds_bytes, csr, stream);
        case 2: return launch_group<T, 2, NR>(a, lds_bytes, csr, stream);
        case 3: return launch_group<T, 3, NR>(a, lds_bytes, csr, stream);
        default: return launch_group<T, 4, NR>(a, lds_bytes, csr, stream);
        }
    };
    rc = a.n_r == 4 ? launch(std::integral_constant<int, 4>{}) : launch(std::integral_constant<int, 6>{});
    if (rc) return rc;
    if (a.force) return pair_csr_finish<T>(a.force, csr, stream, etot, virial, a.partial, a.B, a.nblocks);
    return finish_energy_virial<T>(etot, virial, a.partial, a.B, a.nblocks, stream);
}

template bool nep_group_supported<float>(const NepArgs<float>&, size_t*);
template bool nep_group_supported<double>(const NepArgs<double>&, size_t*);
template int nep_group_run<float>(const NepArgs<float>&, size_t, float*, float*, hipStream_t);
template int nep_group_run<double>(const NepArgs<double>&, size_t, double*, double*, hipStream_t);

}  // namespace a2p
