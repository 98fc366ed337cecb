// NEP energy / force / virial, staged kernels for the common model shapes
// (chebyshev_size 8, n_radial 4 or 6, n_angular 4, l_max 4, up to 4 species).
//
// The generic kernel (nep.hip) lets every thread walk its own neighbour row four times, so each
// wave-wide load touches 64 different cache lines, and it holds the pair derivatives in a
// [row, slot, 3] buffer that a separate pass copies into the reduction segments.  Here
//   * the neighbour rows are read ONCE: the workgroup stages SCH slots of its SB rows through
//     LDS per round with row-contiguous loads (SCH consecutive lanes per row); the loading lane
//     also gathers the neighbour's species and the pair's place in its target's reduction
//     segment with an integer atomic (a2p::PairCsr, fixed-capacity segments);
//   * every thread copies its staged entries into two compact per-thread lists in global
//     scratch, laid out [entry][thread] so that the k-th entries of a wave are contiguous:
//     radial-only neighbours from the front, neighbours inside the angular cutoff from the back.
//     All later loops run over these dense lists with coalesced 16-byte loads, the trip count of
//     the longest list of the wave, no barriers and several entries in flight;
//   * the radial functions are summed per neighbour species and contracted with the
//     coefficients once per atom (pass 1), and the coefficients are contracted with dE/dq once
//     per atom before the radial derivative loop (pass 2);
//   * pair derivatives are stored straight into the reduction segments.
// Two kernels.  nep_stage_kernel does the rounds (radial sums, lists, places in the reduction
// segments): it needs few registers, so many waves per SIMD hide the latency of its gathers and
// atomics.  nep_staged_kernel holds the angular moments in registers (two waves per SIMD) and only
// streams the dense lists: angular moments over the back list; descriptors, hidden layer, dE/dq,
// dE/dS; then the pair derivatives of the radial-only pairs (front list) and of the pairs inside
// the angular cutoff, both parts together (back list); own force, virial.
//
// Formulas: source/descriptor/nep/include/{nepBasis.h:57-196; nep.h:320-529}.
#include "a2p_common.h"
#include "nep_device.h"

#include <type_traits>

namespace a2p {
using namespace nepdev;
namespace {

constexpr int FB = 256;        // atoms (threads) per workgroup of the model kernel; geometry of the lists
constexpr int SB = 256;        // atoms (threads) per workgroup of the staging kernel (divides FB)
constexpr int SCH = 8;         // neighbour slots staged per round
constexpr int SLS = SB + 8;    // padded row length of the staging arrays
constexpr int FDP = 24;        // padded descriptor count (at most 24: n_radial <= 8)
constexpr int KC = 8, NAC = 4, LC = 4, NLM = 24;
// n_radial is a template parameter NR of the model kernel: 4 (the reference's default model,
// ai2pot/models/nep/nep.py:36) and 6 are instantiated

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

// LDS of the staging kernel: staging arrays [SCH][SLS] and the rows' lengths
template <typename T>
struct StageLds {
    T *x, *y, *z;
    int* p;                  // place of the pair in its target's reduction segment
    unsigned char* w;        // species of the neighbour
    int *nn, *red;
};

__host__ __device__ __forceinline__ size_t lds_round16(size_t bytes) { return (bytes + 15) & ~(size_t)15; }

template <typename T>
__host__ __device__ __forceinline__ size_t stage_lds_layout(unsigned char* base, StageLds<T>& L)
{
    size_t off = 0;
    L.x = (T*)(base + off);    off += lds_round16((size_t)SCH * SLS * sizeof(T));
    L.y = (T*)(base + off);    off += lds_round16((size_t)SCH * SLS * sizeof(T));
    L.z = (T*)(base + off);    off += lds_round16((size_t)SCH * SLS * sizeof(T));
    L.p = (int*)(base + off);  off += lds_round16((size_t)SCH * SLS * sizeof(int));
    L.w = base + off;          off += lds_round16((size_t)SCH * SLS);
    L.nn = (int*)(base + off); off += lds_round16((size_t)SB * sizeof(int));
    L.red = (int*)(base + off); off += lds_round16((size_t)(SB / 64) * sizeof(int));
    return off;
}

// LDS of the model kernel: coefficients; network tables (before pass 2) and the contracted radial
// coefficients (pass 2) share one region; partial sums
template <typename T>
struct StagedLds {
    T* coef;
    T *w0, *b0, *w1, *qs;
    T* acc;
    double* red;
};

template <typename T>
__host__ __device__ __forceinline__ size_t staged_lds_layout(int ntypes, int H, int ntc, int nb, unsigned char* base,
                                                             StagedLds<T>& L)
{
    size_t off = 0;
    L.coef = (T*)(base + off); off += lds_round16((size_t)ntypes * ntypes * nb * KC * sizeof(T));
    const size_t u0 = off;
    L.acc = (T*)(base + off);  off += lds_round16((size_t)ntc * KC * FB * sizeof(T));
    const size_t u1 = off;
    off = u0;
    L.w0 = (T*)(base + off);   off += lds_round16((size_t)ntypes * H * FDP * sizeof(T));
    L.b0 = (T*)(base + off);   off += lds_round16((size_t)ntypes * H * sizeof(T));
    L.w1 = (T*)(base + off);   off += lds_round16((size_t)ntypes * H * sizeof(T));
    L.qs = (T*)(base + off);   off += lds_round16((size_t)FDP * sizeof(T));
    off = off > u1 ? off : u1;
    L.red = (double*)(base + off); off += lds_round16((size_t)(FB / 64) * 10 * sizeof(double));
    return off;
}

struct SegArgs {
    int* cursor;   // [B * NF] entries claimed so far in each target's reduction segment, or null (no forces)
    int cap;       // capacity of a segment
    int spare;     // entry that takes what overflows a segment
};

// Row of the padded arrays that local row `la` of the workgroup starting at `rowbase` (= b * P + first
// row) loads from: its own, or the structure's last row for the tail of the last workgroup
__host__ __device__ __forceinline__ size_t staged_row_index(size_t rowbase, int la, int b, int P)
{
    const size_t last = (size_t)b * P + (size_t)(P - 1);
    const size_t r = rowbase + (size_t)la;
    return r < last ? r : last;
}

// Stage slots [c0, c0 + SCH) of the workgroup's rows: thread e handles row e / SCH, slot e % SCH,
// so SCH consecutive lanes read one row's contiguous coordinates and indices.  Entries past a
// row's end (or with an index out of range) are stored far outside every cutoff.
// Three phases, each over all SCH entries of the thread, so that the loads of the entries overlap:
// neighbour indices and vectors; species gathers and segment atomics; LDS stores.  (Letting the
// atomics of the entries overlap as well needs more registers than it gains: their rate, not
// their latency, is what the kernel waits for.)
template <typename T>
__device__ __forceinline__ void staged_load(const NepArgs<T>& a, const SegArgs& seg, const StageLds<T>& L,
                                            int tid, int c0, size_t rowbase, int b, int NF)
{
    const int* types = a.btypes + (size_t)b * NF;
    int nj[SCH], w[SCH], pos[SCH];
    T x[SCH], y[SCH], z[SCH];
    bool have[SCH];
#pragma unroll
    for (int it = 0; it < SCH; it++) {
        const int e = it * SB + tid;
        const int la = e / SCH, slot = c0 + e % SCH;
        have[it] = slot < L.nn[la];
        // a slot past the row's end reads the row's first slot instead, and a row past the
        // structure's last one (the tail of the last workgroup) the structure's last row: the
        // address stays inside the caller's arrays whatever their allocation
        const size_t pr = staged_row_index(rowbase, la, b, a.P) * a.U + (have[it] ? slot : 0);
        const T* p = a.brcs + pr * 3;
        nj[it] = a.bfirstneigh[pr];
        x[it] = p[0]; y[it] = p[1]; z[it] = p[2];
        pos[it] = a.brank && a.ranks_valid ? a.brank[pr] : 0;     // the pair's rank when an earlier call recorded it
    }
    int err = 0;
#pragma unroll
    for (int it = 0; it < SCH; it++) {
        w[it] = 0;
        if (have[it] && (unsigned)nj[it] >= (unsigned)NF) { err |= ST_BAD_NEIGHBOR; have[it] = false; }
        const int njc = have[it] ? nj[it] : 0;
        w[it] = types[njc];
        if (have[it] && seg.cursor) {
            const int t = b * NF + njc;
            int rk;
            if (a.brank && a.ranks_valid) {
                rk = pos[it];
            } else {
                rk = atomicAdd(&seg.cursor[t], 1);
                if (a.brank) {                         // recorded for the later calls on the same list
                    const int e = it * SB + tid;
                    a.brank[(rowbase + e / SCH) * a.U + c0 + e % SCH] = rk;
                }
            }
            pos[it] = rk < seg.cap ? t * seg.cap + rk : seg.spare;
            if ((unsigned)rk >= (unsigned)seg.cap) { err |= ST_SEG_OVERFLOW; pos[it] = seg.spare; }
        } else {
            pos[it] = 0;
        }
    }
#pragma unroll
    for (int it = 0; it < SCH; it++) {
        const int e = it * SB + tid;
        const int la = e / SCH, s = e % SCH;
        if (have[it] && (unsigned)w[it] >= (unsigned)a.ntypes) { err |= ST_BAD_TYPE; w[it] = 0; }
        L.x[s * SLS + la] = have[it] ? x[it] : (T)1.0e18;
        L.y[s * SLS + la] = have[it] ? y[it] : (T)0;
        L.z[s * SLS + la] = have[it] ? z[it] : (T)0;
        L.w[s * SLS + la] = (unsigned char)(have[it] ? w[it] : 0);
        L.p[s * SLS + la] = pos[it];
    }
    if (err) atomicOr(a.status, err);
}

// Bit masks of a thread's staged entries: bit s of mA set when entry s lies inside the angular
// cutoff, of mR inside the radial cutoff, of mV when the entry is a pair of the list at all.
template <typename T>
__device__ __forceinline__ void staged_classify(const StageLds<T>& L, int tid, T rr, T ra, unsigned& mA,
                                                unsigned& mR, unsigned& mV)
{
    mA = 0; mR = 0; mV = 0;
#pragma unroll
    for (int s = 0; s < SCH; s++) {
        const T x = L.x[s * SLS + tid], y = L.y[s * SLS + tid], z = L.z[s * SLS + tid];
        const T r = sqrt_t(x * x + y * y + z * z);
        if (r <= ra && r <= rr) mA |= 1u << s;     // nepBasis.h:106, 135: beyond the radial cutoff a neighbour is skipped
        if (r <= rr) mR |= 1u << s;
        if (x < (T)1.0e17) mV |= 1u << s;
    }
}

// Compact-list entries: [x y z place-in-segment]; the species (two bits) of 16 consecutive entries
// of a thread's list share one word of a separate array
__device__ __forceinline__ void ang_store(float* p, float x, float y, float z, int w)
{
    *reinterpret_cast<float4*>(p) = make_float4(x, y, z, __int_as_float(w));
}
__device__ __forceinline__ void ang_load(const float* p, float& x, float& y, float& z, int& w)
{
    const float4 v = *reinterpret_cast<const float4*>(p);
    x = v.x; y = v.y; z = v.z; w = __float_as_int(v.w);
}
__device__ __forceinline__ void ang_store(double* p, double x, double y, double z, int w)
{
    *reinterpret_cast<double2*>(p) = make_double2(x, y);
    *reinterpret_cast<double2*>(p + 2) = make_double2(z, __longlong_as_double((long long)w));
}
__device__ __forceinline__ void ang_load(const double* p, double& x, double& y, double& z, int& w)
{
    const double2 v0 = *reinterpret_cast<const double2*>(p);
    const double2 v1 = *reinterpret_cast<const double2*>(p + 2);
    x = v0.x; y = v0.y; z = v1.x; w = (int)__double_as_longlong(v1.y);
}

// Rows' header shared by both kernels: centre, its species and the row length, with the checks
template <typename T>
__device__ __forceinline__ void row_header(const NepArgs<T>& a, bool active, size_t row, int b, int NF,
                                           int& center, int& ti, int& nn)
{
    center = 0; ti = 0; nn = 0;
    if (active) {
        center = a.bilist[row];
        nn = a.bnumneigh[row];
        if (nn > a.U) { atomicOr(a.status, ST_NEIGH_OVERFLOW); nn = a.U; }
        if ((unsigned)center >= (unsigned)NF) { atomicOr(a.status, ST_BAD_NEIGHBOR); center = 0; nn = 0; }
        ti = a.btypes[(size_t)b * NF + center];
        if ((unsigned)ti >= (unsigned)a.ntypes) { atomicOr(a.status, ST_BAD_TYPE); ti = 0; nn = 0; }
    }
}

// Staging kernel.  Per row: radial functions summed per neighbour species (radial[k][row], k <
// NTC*KC), list lengths (counts[0][row] radial-only, counts[1][row] inside the angular cutoff),
// the two compact lists, and zeros in the reduction segments for pairs beyond both cutoffs.
template <typename T, int NTC>
__global__ void __launch_bounds__(SB, (sizeof(T) == 4 ? 3 : 2))
nep_stage_kernel(const NepArgs<T> a, const SegArgs seg, T* __restrict__ seg_g, T* __restrict__ ang_xyz,
                 unsigned* __restrict__ typew, T* __restrict__ radial, int* __restrict__ counts)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    const int tid = threadIdx.x;
    const int b = blockIdx.y;
    const int r0 = blockIdx.x * SB;             // first row of the workgroup within the batch
    const int ii = r0 + tid;
    const int NF = a.P + a.nghost;
    StageLds<T> L;
    stage_lds_layout<T>(smem_raw, L);

    const bool active = ii < a.binum[b];
    const size_t rowbase = (size_t)b * a.P + r0;
    int center, ti, nn;
    row_header<T>(a, active, rowbase + tid, b, NF, center, ti, nn);
    L.nn[tid] = nn;
    {
        const int m = wave_max(nn);
        if ((tid & 63) == 0) L.red[tid >> 6] = m;
    }
    __syncthreads();
    int maxnn = 0;
#pragma unroll
    for (int w = 0; w < SB / 64; w++) maxnn = max(maxnn, L.red[w]);

    const T rr = a.rr, ra = a.ra;
    const T rr_inv = (T)1 / rr;
    // compact lists of this row: entry k at [k * FB]; radial-only entries occupy k = 0 ..
    // n_rad-1, entries inside the angular cutoff k = U-1 .. U-n_ang (n_rad + n_ang <= nn <= U)
    const int mblk = ii / FB, mtid = ii - mblk * FB;
    const size_t list0 = (size_t)(b * a.nblocks + mblk) * a.U * FB + mtid;
    T* const lxyz = ang_xyz + list0 * 4;
    const int back = a.U - 1;
    const bool want_pairs = a.force != nullptr || a.want_virial;
    // species words of the two lists: word w of the front list at typew[w * plane + o], of the
    // back list (counted from its own first entry) behind the front list's NW words
    const size_t o = (size_t)(b * a.nblocks + mblk) * FB + mtid;
    const size_t plane = (size_t)a.B * a.nblocks * FB;
    unsigned* const tw_front = typew + o;
    unsigned* const tw_back = typew + (size_t)((a.U + 15) / 16) * plane + o;
    unsigned tw_rad = 0u, tw_ang = 0u;

    T F[NTC][KC];                 // radial functions summed per neighbour species
#pragma unroll
    for (int t = 0; t < NTC; t++)
#pragma unroll
        for (int k = 0; k < KC; k++) F[t][k] = (T)0;
    int n_ang = 0, n_rad = 0;
    for (int c0 = 0; c0 < maxnn; c0 += SCH) {
        __syncthreads();
        staged_load<T>(a, seg, L, tid, c0, rowbase, b, NF);
        __syncthreads();
        unsigned mA, mR, mV;
        staged_classify<T>(L, tid, rr, ra, mA, mR, mV);
        unsigned bits = mR;
        while (bits) {
            const int s = __ffs(bits) - 1;
            bits &= bits - 1;
            const T x = L.x[s * SLS + tid], y = L.y[s * SLS + tid], z = L.z[s * SLS + tid];
            const int tj = L.w[s * SLS + tid];
            const T r = sqrt_t(x * x + y * y + z * z);
            T f[KC], df[KC];
            radial_basis<T, KC, false>(r, rr_inv, KC, f, df);
#pragma unroll
            for (int t = 0; t < NTC; t++)
#pragma unroll
                for (int k = 0; k < KC; k++) F[t][k] += (tj == t) ? f[k] : (T)0;
            if (want_pairs && !((mA >> s) & 1u)) {
                ang_store(lxyz + (size_t)n_rad * FB * 4, x, y, z, L.p[s * SLS + tid]);
                tw_rad |= (unsigned)tj << (2 * (n_rad & 15));
                n_rad++;
                if ((n_rad & 15) == 0) { tw_front[(size_t)((n_rad >> 4) - 1) * plane] = tw_rad; tw_rad = 0u; }
            }
        }
        bits = mA;
        while (bits) {
            const int s = __ffs(bits) - 1;
            bits &= bits - 1;
            const int k = back - n_ang;
            ang_store(lxyz + (size_t)k * FB * 4, L.x[s * SLS + tid], L.y[s * SLS + tid], L.z[s * SLS + tid],
                      L.p[s * SLS + tid]);
            tw_ang |= (unsigned)L.w[s * SLS + tid] << (2 * (n_ang & 15));
            n_ang++;
            if ((n_ang & 15) == 0) { tw_back[(size_t)((n_ang >> 4) - 1) * plane] = tw_ang; tw_ang = 0u; }
        }
        // pairs of the list beyond both cutoffs still own a place in their segment
        bits = mV & ~mR & ~mA;
        while (bits && seg_g) {
            const int s = __ffs(bits) - 1;
            bits &= bits - 1;
            T* dst = seg_g + (size_t)L.p[s * SLS + tid] * 3;
            dst[0] = (T)0; dst[1] = (T)0; dst[2] = (T)0;
        }
    }
    if (n_rad & 15) tw_front[(size_t)(n_rad >> 4) * plane] = tw_rad;
    if (n_ang & 15) tw_back[(size_t)(n_ang >> 4) * plane] = tw_ang;
    if (ii < a.P) {
#pragma unroll
        for (int t = 0; t < NTC; t++)
#pragma unroll
            for (int k = 0; k < KC; k++) radial[(size_t)(t * KC + k) * plane + o] = F[t][k];
        counts[o] = n_rad;
        counts[plane + o] = n_ang;
    }
}

template <typename T, int NTC, int NR>
__global__ void __launch_bounds__(FB, (sizeof(T) == 4 ? 2 : 1))
nep_staged_kernel(const NepArgs<T> a, T* __restrict__ seg_g, int spare, const T* __restrict__ ang_xyz,
                  const unsigned* __restrict__ typew, const T* __restrict__ radial, const int* __restrict__ counts)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    const int tid = threadIdx.x;
    const int b = blockIdx.y;
    const int ii = blockIdx.x * FB + tid;
    const int H = a.H, nt = a.ntypes;
    const int NF = a.P + a.nghost;
    constexpr int NRC = NR, NB = NR + NAC, DC = NR + NAC * LC;
    static_assert(DC <= FDP, "descriptor count exceeds the padded row");
    StagedLds<T> L;
    staged_lds_layout<T>(nt, H, NTC, NB, smem_raw, L);

    for (int i = tid; i < nt * nt * NB * KC; i += FB) L.coef[i] = a.coeffs[i];
    for (int i = tid; i < nt * H * FDP; i += FB) {
        const int r = i / FDP, j = i - r * FDP;
        L.w0[i] = j < DC ? a.w0[(size_t)r * DC + j] : (T)0;
    }
    for (int i = tid; i < nt * H; i += FB) { L.b0[i] = a.b0[i]; L.w1[i] = a.w1[i]; }
    if (tid < FDP) L.qs[tid] = tid < DC ? (T)1 / a.q_scaler[tid] : (T)0;

    const bool active = ii < a.binum[b];
    const size_t row = (size_t)b * a.P + (size_t)blockIdx.x * FB + tid;
    int center, ti, nn;
    row_header<T>(a, active, row, b, NF, center, ti, nn);

    const T rr = a.rr, ra = a.ra;
    const T rr_inv = (T)1 / rr, ra_inv = (T)1 / ra;
    const size_t o = (size_t)(b * a.nblocks + blockIdx.x) * FB + tid;
    const size_t plane = (size_t)a.B * a.nblocks * FB;
    const size_t list0 = (size_t)(b * a.nblocks + blockIdx.x) * a.U * FB + tid;
    const T* const lxyz = ang_xyz + list0 * 4;
    const unsigned* const tw_front = typew + o;
    const unsigned* const tw_back = typew + (size_t)((a.U + 15) / 16) * plane + o;
    const int back = a.U - 1;
    const bool want_pairs = a.force != nullptr || a.want_virial;
    // rows past P were not staged
    const bool staged_row = ii < a.P;
    const int n_rad = staged_row ? counts[o] : 0;
    const int n_ang = staged_row ? counts[plane + o] : 0;
    T F[NTC][KC];
#pragma unroll
    for (int t = 0; t < NTC; t++)
#pragma unroll
        for (int k = 0; k < KC; k++) F[t][k] = staged_row ? radial[(size_t)(t * KC + k) * plane + o] : (T)0;

    T S[NAC][NLM];
#pragma unroll
    for (int n = 0; n < NAC; n++)
#pragma unroll
        for (int m = 0; m < NLM; m++) S[n][m] = (T)0;
    __syncthreads();

    // Walks one of the thread's lists and calls body(valid, x, y, z, place, species) per entry.
    // Every lane makes the same number of trips (the longest list of the wavefront, in steps of
    // PD); a lane past the end of its own list computes on a unit vector with valid = false.  The loop body is straight-line code with one load, and in the derivative passes one
    // store, per entry, none of them conditional: the compiler can then count the memory
    // operations in flight and wait for the entry loaded PD entries ago without waiting for the
    // scattered stores issued since (with conditional loads or stores it falls back to waiting
    // for everything, and every trip would wait for the previous trip's store to be acknowledged).
    const int last_word = (a.U + 15) / 16 - 1;
    auto walk = [&](auto depth, int n, bool front, const unsigned* __restrict__ words, auto&& body) __attribute__((always_inline)) {
        constexpr int PD = decltype(depth)::value;
        const int trips = __builtin_amdgcn_readfirstlane(wave_max(n));
        if (trips == 0) return;
        T qx[PD], qy[PD], qz[PD];
        int qw[PD];
#pragma unroll
        for (int d = 0; d < PD; d++)
            ang_load(lxyz + (size_t)(front ? d : back - d) * FB * 4, qx[d], qy[d], qz[d], qw[d]);
        unsigned tw = words[0], twn = 0u;
        for (int e0 = 0; e0 < trips; e0 += PD) {
            if ((e0 & 15) == 0 && e0 > 0) tw = twn;
            twn = words[(size_t)min((e0 >> 4) + 1, last_word) * plane];
#pragma unroll
            for (int d = 0; d < PD; d++) {
                const int e = e0 + d;
                // past the end of the list: a harmless unit vector instead of whatever the slot holds
                const bool valid = e < n;
                const T x = valid ? qx[d] : (T)1, y = valid ? qy[d] : (T)0, z = valid ? qz[d] : (T)0;
                const int place = qw[d];
                const int nxt = min(e + PD, back);
                ang_load(lxyz + (size_t)(front ? nxt : back - nxt) * FB * 4, qx[d], qy[d], qz[d], qw[d]);
                body(valid, x, y, z, place, min((int)((tw >> (2 * (e & 15))) & 3u), nt - 1));
            }
        }
    };

    // angular moments over the back list
    walk(std::integral_constant<int, (sizeof(T) == 4 ? 2 : 1)>{}, n_ang, false, tw_back, [&](bool valid, T x, T y, T z, int, int tj) __attribute__((always_inline)) {
        const T r = sqrt_t(x * x + y * y + z * z);
        const T rinv = (T)1 / r;
        T f[KC], df[KC];
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
            g = valid ? g : (T)0;
#pragma unroll
            for (int m = 0; m < NLM; m++) S[n][m] += g * bl[m];
        }
    });

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
    __syncthreads();   // every thread is done with the network tables: their memory becomes L.acc
    if (want_pairs) {
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
        // one pair: its derivative goes into the target's segment (STORE) and into the thread's sums;
        // an entry past the end of the list stores into the spare entry and adds zeros
        auto emit = [&](auto store, bool valid, int place, T x, T y, T z, T gx, T gy, T gz) __attribute__((always_inline)) {
            if (decltype(store)::value) {
                T* dst = seg_g + (size_t)(valid ? place : spare) * 3;
                dst[0] = gx; dst[1] = gy; dst[2] = gz;
            }
            gx = valid ? gx : (T)0; gy = valid ? gy : (T)0; gz = valid ? gz : (T)0;
            fx += gx; fy += gy; fz += gz;
            vir[0] -= gx * x; vir[1] -= gx * y; vir[2] -= gx * z;
            vir[3] -= gy * x; vir[4] -= gy * y; vir[5] -= gy * z;
            vir[6] -= gz * x; vir[7] -= gz * y; vir[8] -= gz * z;
        };
        auto pass2 = [&](auto store) __attribute__((always_inline)) {
            // radial-only pairs (front list)
            walk(std::integral_constant<int, (sizeof(T) == 4 ? 4 : 2)>{}, n_rad, true, tw_front, [&](bool valid, T x, T y, T z, int place, int tj) __attribute__((always_inline)) {
                const T r = sqrt_t(x * x + y * y + z * z);
                T f[KC], df[KC];
                radial_basis<T, KC, true>(r, rr_inv, KC, f, df);
                T sr = (T)0;
#pragma unroll
                for (int k = 0; k < KC; k++) sr += L.acc[(tj * KC + k) * FB + tid] * df[k];
                sr /= r;
                emit(store, valid, place, x, y, z, sr * x, sr * y, sr * z);
            });
            // pairs inside the angular cutoff, radial and angular part together (back list)
            walk(std::integral_constant<int, (sizeof(T) == 4 ? 2 : 1)>{}, n_ang, false, tw_back, [&](bool valid, T x, T y, T z, int place, int tj) __attribute__((always_inline)) {
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
                emit(store, valid, place, x, y, z, srad * ux + wx * rinv, srad * uy + wy * rinv, srad * uz + wz * rinv);
            });
        };
        if (seg_g) pass2(std::true_type{});
        else pass2(std::false_type{});
        if (active && a.force) {
            T* fo = a.force + ((size_t)b * NF + center) * 3;
            fo[0] = fx; fo[1] = fy; fo[2] = fz;
        }
    }

    // ---- workgroup partial sums of energy and virial (fp64) ---------------------------------
    __syncthreads();
    double* s_red = L.red;
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

template <typename T, int NTC, int NR>
int launch_staged(const NepArgs<T>& a, size_t lds, const PairCsr& csr, hipStream_t stream)
{
    // workspace: compact lists [workgroup][entry < U][thread] of 4 T; species words of the front and
    // of the back list, [2][ceil(U / 16)][row]; per row the summed radial functions [NTC*KC] and the
    // two list lengths
    const size_t plane = (size_t)a.B * a.nblocks * FB;
    const size_t nent = plane * a.U;
    const size_t nwords = 2 * (size_t)((a.U + 15) / 16) * plane;
    void* ws = nullptr;
    int rc = ws_get(WS_PAIR_G, nent * 4 * sizeof(T) + nwords * sizeof(unsigned) +
                                   plane * (NTC * KC * sizeof(T) + 2 * sizeof(int)), &ws);
    if (rc) return rc;
    T* ang_xyz = (T*)ws;
    unsigned* typew = (unsigned*)((char*)ws + nent * 4 * sizeof(T));
    T* radial = (T*)((char*)ws + nent * 4 * sizeof(T) + nwords * sizeof(unsigned));
    int* counts = (int*)(radial + plane * NTC * KC);
    SegArgs seg{csr.cursor, csr.seg_cap, csr.n * csr.seg_cap};
    StageLds<T> unused;
    const size_t lds_stage = stage_lds_layout<T>(nullptr, unused);
    auto stage = nep_stage_kernel<T, NTC>;
    if (lds_stage > 48 * 1024)
        A2P_HIP_CHECK(hipFuncSetAttribute((const void*)stage, hipFuncAttributeMaxDynamicSharedMemorySize,
                                          (int)lds_stage));
    prof_begin("nep_stage_kernel", stream);
    hipLaunchKernelGGL(stage, dim3(ceil_div(a.P, SB), a.B), dim3(SB), lds_stage, stream, a, seg, (T*)csr.seg_g,
                       ang_xyz, typew, radial, counts);
    prof_end(stream);
    auto kern = nep_staged_kernel<T, NTC, NR>;
    if (lds > 48 * 1024)
        A2P_HIP_CHECK(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                                          (int)lds));
    prof_begin("nep_staged_kernel", stream);
    hipLaunchKernelGGL(kern, dim3(a.nblocks, a.B), dim3(FB), lds, stream, a, (T*)csr.seg_g, seg.spare, (const T*)ang_xyz,
                       (const unsigned*)typew, (const T*)radial, (const int*)counts);
    prof_end(stream);
    A2P_HIP_CHECK(hipGetLastError());
    return A2P_OK;
}

int ntc_of(int ntypes) { return ntypes <= 1 ? 1 : ntypes == 2 ? 2 : ntypes == 3 ? 3 : 4; }

}  // namespace

int nep_staged_nblocks(int P) { return ceil_div(P, FB); }

template <typename T>
bool nep_staged_supported(const NepArgs<T>& a, size_t* lds_bytes)
{
    if (!(a.K == KC && (a.n_r == 4 || a.n_r == 6) && a.n_a == NAC && a.l_max == LC && a.ntypes <= 4)) return false;
    StagedLds<T> unused;
    *lds_bytes = staged_lds_layout<T>(a.ntypes, a.H, ntc_of(a.ntypes), a.n_r + NAC, nullptr, unused);
    static_assert(FB % SB == 0, "a staging workgroup must not straddle two model workgroups");
    return *lds_bytes <= 150 * 1024;
}

template <typename T>
int nep_staged_run(const NepArgs<T>& a, size_t lds_bytes, T* etot, T* virial, hipStream_t stream)
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
        case 1: return launch_staged<T, 1, NR>(a, lds_bytes, csr, stream);
        case 2: return launch_staged<T, 2, NR>(a, lds_bytes, csr, stream);
        case 3: return launch_staged<T, 3, NR>(a, lds_bytes, csr, stream);
        default: return launch_staged<T, 4, NR>(a, lds_bytes, csr, stream);
        }
    };
    rc = a.n_r == 4 ? launch(std::integral_constant<int, 4>{}) : launch(std::integral_constant<int, 6>{});
    if (rc) return rc;
    if (a.force) return pair_csr_finish<T>(a.force, csr, stream, etot, virial, a.partial, a.B, a.nblocks);
    return finish_energy_virial<T>(etot, virial, a.partial, a.B, a.nblocks, stream);
}

template bool nep_staged_supported<float>(const NepArgs<float>&, size_t*);
template bool nep_staged_supported<double>(const NepArgs<double>&, size_t*);
template int nep_staged_run<float>(const NepArgs<float>&, size_t, float*, float*, hipStream_t);
template int nep_staged_run<double>(const NepArgs<double>&, size_t, double*, double*, hipStream_t);

}  // namespace a2p
