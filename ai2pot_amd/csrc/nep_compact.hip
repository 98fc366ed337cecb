// NEP energy / force / virial for neighbour lists this library built itself
// (a2p_nblist_build_compact_*: one periodic structure, no ghosts, every pair listed from both ends).
//
// The reference scatters: atom i computes g_ij = dE_i/dr_ij for each neighbour and does
// F_i += g_ij, F_j -= g_ij (source/descriptor/nep/include/nep.h:468-515).  With a list that holds
// every pair from both ends the same forces are
//     F_i = sum_j (g_ij - g_ji),        V = - sum_i sum_j g_ij r_ij^T.
// Two kernels over the atoms, one thread per atom, 256 per workgroup:
//   nep_adjoint_kernel : radial sums and angular moments over the compact lists, descriptors, hidden layer,
//                        dE/dq, dE/dS (kept in registers); then the pairs inside the angular cutoff once
//                        more: g_ij with both parts, summed into F_i and the virial, and handed to atom j
//                        through a slot array, slots[place][j], the place claimed with an atomic counter
//                        per target (an atom is named by as many pairs as its own list has entries; places
//                        beyond the array's depth are added to a spare row of 64-bit integers in the fixed
//                        point of the slot sums, so the result does not depend on their order either).
//                        It also stores, per atom, the radial coefficients contracted with dE/dq,
//                        cc_i[t][k] = sum_n dE_i/dq_n c[t_i][t][n][k] (species x 8 values).
//   nep_gather_kernel  : the pairs between the cutoffs, which have a radial part only: g_ij - g_ji is a
//                        function of the one distance and of cc_i[t_j] + cc_j[t_i], so the neighbour's 32 bytes
//                        are gathered and nothing is stored per pair; then the slots of the atom are summed
//                        (in fixed point, so that the result does not depend on which pair got which
//                        place) and the force is written.
// Atoms are processed in the Morton order of the list build and workgroups are dealt to the XCDs in contiguous
// runs.  The lists are read in 8 KiB chunks (8 slots of 64 positions), staged through LDS by each wavefront
// for itself: global loads are contiguous, LDS reads are one 16-byte entry per lane.
//
// Formulas: source/descriptor/nep/include/{nepBasis.h:57-196; nep.h:320-529}.
#include "a2p_common.h"
#include "compact_list.h"
#include "nep_device.h"

#include <cstdlib>
#include <string>
#include <type_traits>

namespace a2p {
using namespace nepdev;
namespace {

constexpr int CB = 256;                 // positions (threads) per workgroup
constexpr int KC = 8, NAC = 4, LC = 4, NLM = 24, FDP = 24;
constexpr int NSLOT = 32;               // depth of the slot array: places 0 .. NSLOT-1 of every atom
constexpr int STP = CL_CHUNK + 1;       // staged slots per position, padded: 16-byte reads of 8 lanes hit 8 banks

template <typename T>
struct GatherArgs {
    int H, ntypes;
    const T *coeffs, *w0, *b0, *w1, *bias, *q_scaler;
    T rr, ra;
    CompactView<T> cv;
    const int* types;     // [natoms]
    // the next four are indexed by position in the processing order, like the index field of the list entries
    T* rcc;               // [natoms][NTC * KC] radial coefficients contracted with dE/dq
    T* slots;             // [NSLOT][natoms][4] derivatives handed to the neighbour, by place
    // the next two live in a workspace slot that is zero when a call starts: nep_gather_kernel clears what it read
    unsigned long long* overflow;   // [natoms][OverflowRow<T>::WORDS] the same for places >= NSLOT: fixed-point sums
    int* incoming;        // [natoms] places claimed so far
    double overflow_limit; // largest magnitude a spare row accepts per value (sums of umax values must fit)
    T* force;             // [natoms][3] or null
    double* partial;      // [nblocks][10]: energy and virial, each workgroup's share
    int* status;
    int want_virial;
};

__device__ __forceinline__ void ld4(const float* p, float (&o)[4])
{
    const float4 v = *reinterpret_cast<const float4*>(p);
    o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
}
__device__ __forceinline__ void ld4(const double* p, double (&o)[4])
{
    const double2 v0 = *reinterpret_cast<const double2*>(p);
    const double2 v1 = *reinterpret_cast<const double2*>(p + 2);
    o[0] = v0.x; o[1] = v0.y; o[2] = v1.x; o[3] = v1.y;
}
__device__ __forceinline__ void st4(float* p, const float (&v)[4])
{
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ void st4(double* p, const double (&v)[4])
{
    *reinterpret_cast<double2*>(p) = make_double2(v[0], v[1]);
    *reinterpret_cast<double2*>(p + 2) = make_double2(v[2], v[3]);
}
// the same past the caches (non-temporal): for the list entries and the filled slots, which a kernel streams through
// once or twice; with ordinary loads they push the rows that many lanes gather (contracted coefficients) out of the L2
__device__ __forceinline__ void ld4_stream(const float* p, float (&o)[4])
{
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    const f32x4 v = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p));
    o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
}
__device__ __forceinline__ void ld4_stream(const double* p, double (&o)[4])
{
    typedef double f64x2 __attribute__((ext_vector_type(2)));
    const f64x2 v0 = __builtin_nontemporal_load(reinterpret_cast<const f64x2*>(p));
    const f64x2 v1 = __builtin_nontemporal_load(reinterpret_cast<const f64x2*>(p + 2));
    o[0] = v0.x; o[1] = v0.y; o[2] = v1.x; o[3] = v1.y;
}
__device__ __forceinline__ int entry_bits(float w) { return __float_as_int(w); }
__device__ __forceinline__ int entry_bits(double w) { return (int)__double_as_longlong(w); }

// nep_device.h's radial_basis (f_k = 1/2 (T_k(x)+1) fc(r), basis.h:137-158, 300-332, 519-530) for all KC functions
template <typename T, bool DER>
__device__ __forceinline__ void radial_functions(T r, T rc_inv, T (&f)[KC], T (&df)[KC])
{
    const T t = r * rc_inv;
    const T xr = t - (T)1;
    const T x = (T)2 * xr * xr - (T)1, x2 = x + x;
    T sn, cs;
    sincospi_t(t, &sn, &cs);
    const T fc = (T)0.5 * ((T)1 + cs), hfc = (T)0.5 * fc;
    const T dfc = (T)(-0.5 * 3.14159265358979323846) * sn * rc_inv, hdfc = (T)0.5 * dfc;
    const T w = hfc * ((T)4 * rc_inv * xr);                  // 1/2 fc dx/dr
    T t0 = (T)1, t1 = x, d0 = (T)0, d1 = (T)1;
    f[0] = fc; f[1] = hfc * x + hfc;
    if (DER) { df[0] = dfc; df[1] = hdfc * x + hdfc + w; }
#pragma unroll
    for (int k = 2; k < KC; k++) {
        const T tv = x2 * t1 - t0;
        f[k] = hfc * tv + hfc;
        if (DER) {
            const T dv = (T)2 * t1 + (x2 * d1 - d0);
            df[k] = (hdfc * tv + hdfc) + w * dv;
            d0 = d1; d1 = dv;
        }
        t0 = t1; t1 = tv;
    }
}

// sum_k a_k f_k'(r) without the functions themselves:
//   1/2 fc' (sum a_k T_k + sum a_k) + 1/2 fc x' sum a_k T_k'
template <typename T>
__device__ __forceinline__ T radial_derivative_dot(T r, T rc_inv, const T (&a)[KC])
{
    const T t = r * rc_inv;
    const T xr = t - (T)1;
    const T x = (T)2 * xr * xr - (T)1, x2 = x + x;
    T sn, cs;
    sincospi_t(t, &sn, &cs);
    const T hfc = (T)0.25 * ((T)1 + cs);
    const T hdfc = (T)(-0.25 * 3.14159265358979323846) * sn * rc_inv;
    T t0 = (T)1, t1 = x, d0 = (T)0, d1 = (T)1;
    T s0 = a[0] + a[1], st = a[0] + a[1] * x, sd = a[1];
#pragma unroll
    for (int k = 2; k < KC; k++) {
        const T tv = x2 * t1 - t0;
        const T dv = (T)2 * t1 + (x2 * d1 - d0);
        s0 += a[k]; st += a[k] * tv; sd += a[k] * dv;
        t0 = t1; t1 = tv; d0 = d1; d1 = dv;
    }
    return hdfc * (st + s0) + hfc * ((T)4 * rc_inv * xr) * sd;
}

__host__ __device__ __forceinline__ size_t lds16(size_t bytes) { return (bytes + 15) & ~(size_t)15; }

// Workgroups are handed to the 8 XCDs round robin; giving XCD k the k-th contiguous run of blocks
// keeps neighbours in space on one L2.
__device__ __forceinline__ int xcd_block(int w, int nb)
{
    const int per = nb >> 3, rem = nb & 7, k = w & 7;
    return k * per + min(k, rem) + (w >> 3);
}

// One chunk (8 slots of the tile's 64 positions, contiguous in memory) on its way into the wavefront's
// staging buffer (position-major with STP slots per position): contiguous loads, then 16-byte LDS stores.
template <typename T>
__device__ __forceinline__ void chunk_load(const T* __restrict__ g, int lane, T (&v)[CL_CHUNK][4])
{
#pragma unroll
    for (int it = 0; it < CL_CHUNK; it++) ld4_stream(g + (size_t)(it * 64 + lane) * 4, v[it]);
}
template <typename T>
__device__ __forceinline__ void chunk_store(T* __restrict__ st, int lane, const T (&v)[CL_CHUNK][4])
{
#pragma unroll
    for (int it = 0; it < CL_CHUNK; it++) {
        const int idx = it * 64 + lane;
        st4(st + ((idx >> 3) * STP + (idx & 7)) * 4, v[it]);
    }
}

// Walks one of the two lists of the wavefront's 64 positions: chunk after chunk through the staging
// buffer, every lane making the trips of the longest list; body(valid, x, y, z, bits).  A lane past
// the end of its own list gets a unit vector and valid = false.  With AHEAD the next chunk is requested
// before the trips of the current one and waits in registers (32 of them) meanwhile.
template <typename T, bool AHEAD = false, typename Body>
__device__ __forceinline__ void walk_list(const CompactView<T>& cv, int tile, int lane, T* st, int n, bool inner,
                                          Body&& body)
{
    const int trips = __builtin_amdgcn_readfirstlane(wave_max(n));
    T v[CL_CHUNK][4];
    if (AHEAD && trips > 0)
        chunk_load<T>(cv.entries + compact_chunk_offset<T>(cv.nch, tile, inner ? cv.nch - 1 : 0), lane, v);
    for (int c = 0; c * CL_CHUNK < trips; c++) {
        const int chunk = inner ? cv.nch - 1 - c : c;
        if (!AHEAD) chunk_load<T>(cv.entries + compact_chunk_offset<T>(cv.nch, tile, chunk), lane, v);
        __builtin_amdgcn_wave_barrier();
        chunk_store<T>(st, lane, v);
        __builtin_amdgcn_wave_barrier();
        if (AHEAD && (c + 1) * CL_CHUNK < trips)
            chunk_load<T>(cv.entries + compact_chunk_offset<T>(cv.nch, tile, inner ? chunk - 1 : chunk + 1), lane, v);
        for (int s = 0; s < CL_CHUNK; s++) {
            const int e = c * CL_CHUNK + s;
            if (e >= trips) break;                               // wave-uniform
            T w[4];
            ld4(st + (lane * STP + (inner ? CL_CHUNK - 1 - s : s)) * 4, w);
            const bool valid = e < n;
            body(valid, valid ? w[0] : (T)1, valid ? w[1] : (T)0, valid ? w[2] : (T)0, entry_bits(w[3]));
        }
    }
}

// position -> atom, species, list lengths; with the checks
template <typename T>
__device__ __forceinline__ bool position_header(const GatherArgs<T>& a, int p, int& atom, int& ti, int& n_outer,
                                                int& n_inner)
{
    atom = 0; ti = 0; n_outer = 0; n_inner = 0;
    if (p >= a.cv.natoms) return false;
    atom = a.cv.order[p];
    if ((unsigned)atom >= (unsigned)a.cv.natoms) { atomicOr(a.status, ST_BAD_NEIGHBOR); atom = 0; return false; }
    ti = a.types[atom];
    if ((unsigned)ti >= (unsigned)a.ntypes) { atomicOr(a.status, ST_BAD_TYPE); ti = 0; return false; }
    n_outer = a.cv.n_outer[p];
    n_inner = a.cv.n_inner[p];
    if (n_outer < 0 || n_inner < 0 || n_outer + n_inner > a.cv.umax) {
        atomicOr(a.status, ST_NEIGH_OVERFLOW);
        n_outer = 0; n_inner = 0;
    }
    return true;
}

// Exact, order-independent sum of a few floating-point values: fixed point in 64-bit integers.
// fp32 values are kept to 2^-40 (a thousandth of the last bit of a 1e-3 eV/A component), fp64 values in two
// limbs to 2^-84.  The magnitudes summed into one FixedSum must stay below 2^21 IN TOTAL (kFixedSumLimit): the
// callers track the sum of magnitudes and give NaN beyond it.
template <typename T>
struct FixedSum;
template <>
struct FixedSum<float> {
    long long s = 0;
    __device__ __forceinline__ void add(float x) { s += (long long)((double)x * 0x1p40); }
    __device__ __forceinline__ double value() const { return (double)s * 0x1p-40; }
};
template <>
struct FixedSum<double> {
    long long hi = 0, lo = 0;
    __device__ __forceinline__ void add(double x)
    {
        const double v = x * 0x1p32, h = trunc(v);
        hi += (long long)h;
        lo += (long long)((v - h) * 0x1p52);
    }
    __device__ __forceinline__ double value() const { return (double)hi * 0x1p-32 + (double)lo * 0x1p-84; }
};
constexpr double kFixedSumLimit = 0x1p21;

// The spare row of an atom: the same fixed point, added to with 64-bit integer atomics (order-independent).
// Word BAD counts values that were not finite or too large to convert; the reader then gives NaN.
template <typename T>
struct OverflowRow;
template <>
struct OverflowRow<float> {
    static constexpr int WORDS = 4, BAD = 3;
    static __device__ __forceinline__ void add(unsigned long long* row, int c, float x)
    {
        atomicAdd(row + c, (unsigned long long)(long long)((double)x * 0x1p40));
    }
    static __device__ __forceinline__ void take(unsigned long long* row, int c, FixedSum<float>& s)
    {
        s.s += (long long)row[c];
        row[c] = 0ull;
    }
};
template <>
struct OverflowRow<double> {
    static constexpr int WORDS = 8, BAD = 6;
    static __device__ __forceinline__ void add(unsigned long long* row, int c, double x)
    {
        const double v = x * 0x1p32, h = trunc(v);
        atomicAdd(row + 2 * c, (unsigned long long)(long long)h);
        atomicAdd(row + 2 * c + 1, (unsigned long long)(long long)((v - h) * 0x1p52));
    }
    static __device__ __forceinline__ void take(unsigned long long* row, int c, FixedSum<double>& s)
    {
        s.hi += (long long)row[2 * c];
        s.lo += (long long)row[2 * c + 1];
        row[2 * c] = 0ull;
        row[2 * c + 1] = 0ull;
    }
};

template <typename T>
struct AdjointLds {
    T *coef, *w0, *w0t, *b0, *w1, *qs, *acc, *stage;
    double* red;
};
constexpr int HM_HP = 64;               // neurons of the zero-padded tables of the matrix-core hidden layer
constexpr int HM_HPT = 68;              // row length of the transposed table: 16 lanes reading 16 rows hit 16 bank groups
// The network tables (w0, b0, w1, qs) are dead once the hidden layer is done; the threads' contracted
// radial coefficients (acc, [NTC * KC][CB]) are laid over them for the second walk.
// hm: tables of the matrix-core hidden layer: H padded to HM_HP neurons with zeros, and a transposed copy of w0
template <typename T>
__host__ __device__ __forceinline__ size_t adjoint_lds(int nt, int ntc, int H, int nb, unsigned char* base, AdjointLds<T>& L,
                                                       bool hm = false)
{
    size_t off = 0;
    L.coef = (T*)(base + off);  off += lds16((size_t)nt * nt * nb * KC * sizeof(T));
    const size_t tables = off;
    if (hm) H = HM_HP;
    L.acc = (T*)(base + off);
    L.w0 = (T*)(base + off);    off += lds16((size_t)nt * H * FDP * sizeof(T));
    L.w0t = (T*)(base + off);   if (hm) off += lds16((size_t)nt * HM_HPT * FDP * sizeof(T));
    L.b0 = (T*)(base + off);    off += lds16((size_t)nt * H * sizeof(T));
    L.w1 = (T*)(base + off);    off += lds16((size_t)nt * H * sizeof(T));
    L.qs = (T*)(base + off);    off += lds16((size_t)FDP * sizeof(T));
    const size_t acc_end = tables + lds16((size_t)ntc * KC * CB * sizeof(T));
    if (off < acc_end) off = acc_end;
    L.stage = (T*)(base + off); off += lds16((size_t)(CB / 64) * 64 * STP * 4 * sizeof(T));
    L.red = (double*)(base + off); off += lds16((size_t)(CB / 64) * 10 * sizeof(double));
    return off;
}

template <typename T>
struct GatherLds {
    T* stage;
    double* red;
};
template <typename T>
__host__ __device__ __forceinline__ size_t gather_lds(unsigned char* base, GatherLds<T>& L)
{
    size_t off = 0;
    L.stage = (T*)(base + off); off += lds16((size_t)(CB / 64) * 64 * STP * 4 * sizeof(T));
    L.red = (double*)(base + off); off += lds16((size_t)(CB / 64) * 9 * sizeof(double));
    return off;
}

// ---- the hidden layer of a wavefront's 64 atoms on the matrix cores (fp32) ----------------------------
// The weights depend on the atom's species, so the wavefront first groups its atoms by species: every lane gets a
// row in a table of scaled descriptors in LDS (the wavefront's own staging buffer, idle between the walks; no
// workgroup barrier is involved), each species' rows padded to a multiple of 16: at most 96 rows for up to three
// species.  Then, tile by tile (16 rows of one species), with v_mfma_f32_16x16x4f32 (D[i][j] += sum_k A[i][k] B[k][j];
// lane l holds A[l%16][l/16], B[l/16][l%16] and D[4 (l/16) + v][l%16] in register v):
//   layer 1, transposed:  H^T[n][r] = sum_k W0[n][k] Q[r][k]   (A = weights, B = descriptors), four tiles of 16
//            neurons; on the accumulators: + b0, tanh, the energy terms w1 tanh, and G = w1 (1 - tanh^2);
//   layer 2:              dE/dq[r][j] = sum_n G[r][n] W0[n][j]: the accumulators of layer 1 are already laid out
//            as the A operand of this product (lane l holds row r = l%16 and, in register v of neuron tile n0,
//            neuron n0 + 4 (l/16) + v), so the sum over the neurons simply runs in that order and G never leaves
//            the registers; B = W0[n0 + 4 (l/16) + v][j0 + l%16].
// dE/dq and the energy go back into the table row, and every lane reads its row.  Neurons beyond H and
// descriptors beyond DC are zero weights.  Reference arithmetic: nep.h:415-447.
constexpr int kHiddenDefault = 0;                 // vector ALUs unless measured otherwise
constexpr int HM_TILE = 16, HM_NT = 4;            // rows per tile; neuron tiles (H <= 64)
constexpr int HM_STRIDE = FDP;                    // floats per table row: DC descriptors, [FDP-1] the energy
constexpr int HM_ROWS = 64 * STP * 4 / HM_STRIDE; // rows the staging buffer of a wavefront holds (96)
constexpr int HM_NTC_MAX = 3;                     // 64 atoms of up to three species fit: 64 + 3 * 15 -> 96 rows
static_assert(HM_ROWS >= ((64 + HM_NTC_MAX * (HM_TILE - 1)) / HM_TILE) * HM_TILE, "staging buffer too small");

typedef float hm_f4 __attribute__((ext_vector_type(4)));

template <int NTC, int DC>
__device__ __forceinline__ void hidden_layer_mfma(const AdjointLds<float>& L, float* Q, int H, int ti, int lane,
                                                  float (&qn)[FDP], float& e_net)
{
    static_assert(DC < FDP, "the last column of a row carries the energy");
    static_assert(NTC <= HM_NTC_MAX, "too many species for the wavefront's table");
    // -- rows: species by species, inside a species by lane; ends[t] = end of species t's (padded) rows
    int row = 0, nrows = 0;
    int ends[NTC];
#pragma unroll
    for (int t = 0; t < NTC; t++) {
        const unsigned long long m = __ballot(ti == t);
        if (ti == t) row = nrows + __popcll(m & ((1ull << lane) - 1ull));
        nrows += (__popcll(m) + HM_TILE - 1) & ~(HM_TILE - 1);
        ends[t] = nrows;
    }
    __builtin_amdgcn_wave_barrier();
    {
        // rows that pad a species to a multiple of 16 are never read back; their contents only need to exist
        float* qr = Q + (size_t)row * HM_STRIDE;
#pragma unroll
        for (int j = 0; j < FDP; j += 4) *reinterpret_cast<float4*>(qr + j) = make_float4(qn[j], qn[j + 1], qn[j + 2], qn[j + 3]);
    }
    __builtin_amdgcn_wave_barrier();
    const int c = lane & 15, g = lane >> 4;
    for (int row0 = 0; row0 < nrows; row0 += HM_TILE) {
        int t = 0;                                 // species of the tile
#pragma unroll
        for (int s2 = 0; s2 + 1 < NTC; s2++) t += row0 >= ends[s2] ? 1 : 0;
        // layer 1; the sum over the descriptors runs in the order k = 6 g + kk, so that a lane's six values are
        // neighbours in memory: B = Q[row0 + c][6 g + kk], A = W0[n][6 g + kk]
        float qb[FDP / 4];
        {
            const float* qr = Q + (size_t)(row0 + c) * HM_STRIDE + 6 * g;
#pragma unroll
            for (int kk = 0; kk < FDP / 4; kk += 2) {
                const float2 v = *reinterpret_cast<const float2*>(qr + kk);
                qb[kk] = v.x; qb[kk + 1] = v.y;
            }
        }
        hm_f4 acc[HM_NT];
#pragma unroll
        for (int nt_ = 0; nt_ < HM_NT; nt_++) {
            acc[nt_] = hm_f4{0.0f, 0.0f, 0.0f, 0.0f};
            if (nt_ * HM_TILE < H) {                       // wave-uniform
                const float* wr = L.w0 + ((size_t)t * HM_HP + nt_ * HM_TILE + c) * FDP + 6 * g;
#pragma unroll
                for (int kk = 0; kk < FDP / 4; kk += 2) {
                    const float2 wa = *reinterpret_cast<const float2*>(wr + kk);
                    acc[nt_] = __builtin_amdgcn_mfma_f32_16x16x4f32(wa.x, qb[kk], acc[nt_], 0, 0, 0);
                    acc[nt_] = __builtin_amdgcn_mfma_f32_16x16x4f32(wa.y, qb[kk + 1], acc[nt_], 0, 0, 0);
                }
            }
        }
        // on the accumulators: lane (c, g), register v of tile nt_ = neuron nt_ * 16 + 4 g + v of row row0 + c
        float e = 0.0f;
#pragma unroll
        for (int nt_ = 0; nt_ < HM_NT; nt_++) {
            const float4 b0v = *reinterpret_cast<const float4*>(L.b0 + t * HM_HP + nt_ * HM_TILE + 4 * g);
            const float4 w1v = *reinterpret_cast<const float4*>(L.w1 + t * HM_HP + nt_ * HM_TILE + 4 * g);
            const float b0a[4] = {b0v.x, b0v.y, b0v.z, b0v.w}, w1a[4] = {w1v.x, w1v.y, w1v.z, w1v.w};
#pragma unroll
            for (int v = 0; v < 4; v++) {
                if (nt_ * HM_TILE + v < H) {               // wave-uniform: some lane has a neuron here
                    const float th = tanh_t(acc[nt_][v] + b0a[v]);
                    e += w1a[v] * th;
                    acc[nt_][v] = w1a[v] * (1.0f - th * th);
                } else {
                    acc[nt_][v] = 0.0f;
                }
            }
        }
        e += __shfl_xor(e, 16, 64);
        e += __shfl_xor(e, 32, 64);
        // layer 2: two tiles of 16 descriptors (j0 = 0, 16); B = W0^T[j0 + c][nt_ * 16 + 4 g + v], four neighbours
        // in the transposed table (columns beyond the table read its last, all-zero row)
        hm_f4 out[2] = {hm_f4{0.0f, 0.0f, 0.0f, 0.0f}, hm_f4{0.0f, 0.0f, 0.0f, 0.0f}};
        const float* wt0 = L.w0t + ((size_t)t * FDP + c) * HM_HPT + 4 * g;
        const float* wt1 = L.w0t + ((size_t)t * FDP + min(16 + c, FDP - 1)) * HM_HPT + 4 * g;
#pragma unroll
        for (int nt_ = 0; nt_ < HM_NT; nt_++) {
            if (nt_ * HM_TILE < H) {                       // wave-uniform
                const float4 u0 = *reinterpret_cast<const float4*>(wt0 + nt_ * HM_TILE);
                const float4 u1 = *reinterpret_cast<const float4*>(wt1 + nt_ * HM_TILE);
                const float b0a[4] = {u0.x, u0.y, u0.z, u0.w}, b1a[4] = {u1.x, u1.y, u1.z, u1.w};
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    if (nt_ * HM_TILE + v < H) {           // wave-uniform
                        out[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(acc[nt_][v], b0a[v], out[0], 0, 0, 0);
                        out[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(acc[nt_][v], b1a[v], out[1], 0, 0, 0);
                    }
                }
            }
        }
        // back into the rows (the tile's descriptors have been read): register v = row row0 + 4 g + v, column j0 + c
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int v = 0; v < 4; v++) {
            float* qr = Q + (size_t)(row0 + 4 * g + v) * HM_STRIDE;
            qr[c] = out[0][v];
            if (16 + c < FDP - 1) qr[16 + c] = out[1][v];
        }
        if (g == 0) Q[(size_t)(row0 + c) * HM_STRIDE + FDP - 1] = e;
    }
    __builtin_amdgcn_wave_barrier();
    {
        const float* qr = Q + (size_t)row * HM_STRIDE;
#pragma unroll
        for (int j = 0; j < FDP; j += 4) {
            const float4 v = *reinterpret_cast<const float4*>(qr + j);
            qn[j] = v.x; qn[j + 1] = v.y; qn[j + 2] = v.z; qn[j + 3] = v.w;
        }
    }
    __builtin_amdgcn_wave_barrier();               // the staging buffer goes back to the walks
    e_net = qn[FDP - 1];
}

// ---- kernel 1: descriptors, hidden layer, adjoints -------------------------------------------------
// HM: the hidden layer of each wavefront's 64 atoms runs on the matrix cores (fp32, at most 64 neurons and three
// species): see hidden_layer_mfma
template <typename T, int NTC, int NR, bool HM = false>
__global__ void __launch_bounds__(CB, (sizeof(T) == 4 ? 2 : 1))
nep_adjoint_kernel(const GatherArgs<T> a)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    constexpr int NB = NR + NAC, DC = NR + NAC * LC;
    static_assert(DC <= FDP, "descriptor count exceeds the padded row");
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int blk = xcd_block(blockIdx.x, gridDim.x);
    const int p = blk * CB + tid;
    const int tile = p >> 6;
    const int nt = a.ntypes, H = a.H;
    AdjointLds<T> L;
    adjoint_lds<T>(nt, NTC, H, NB, smem_raw, L, HM);
    T* const st = L.stage + (size_t)wv * 64 * STP * 4;

    for (int i = tid; i < nt * nt * NB * KC; i += CB) L.coef[i] = a.coeffs[i];
    if constexpr (HM) {
        // [species][HM_HP neurons][FDP] and its transpose [species][FDP][HM_HPT], zeros beyond H and DC
        for (int i = tid; i < nt * HM_HP * FDP; i += CB) {
            const int r = i / FDP, j = i - r * FDP, t = r / HM_HP, n = r - t * HM_HP;
            const T v = (n < H && j < DC) ? a.w0[((size_t)t * H + n) * DC + j] : (T)0;
            L.w0[i] = v;
            L.w0t[((size_t)t * FDP + j) * HM_HPT + n] = v;
        }
        for (int i = tid; i < nt * HM_HP; i += CB) {
            const int t = i / HM_HP, n = i - t * HM_HP;
            L.b0[i] = n < H ? a.b0[t * H + n] : (T)0;
            L.w1[i] = n < H ? a.w1[t * H + n] : (T)0;
        }
    } else {
        for (int i = tid; i < nt * H * FDP; i += CB) {
            const int r = i / FDP, j = i - r * FDP;
            L.w0[i] = j < DC ? a.w0[(size_t)r * DC + j] : (T)0;
        }
        for (int i = tid; i < nt * H; i += CB) { L.b0[i] = a.b0[i]; L.w1[i] = a.w1[i]; }
    }
    if (tid < FDP) L.qs[tid] = tid < DC ? (T)1 / a.q_scaler[tid] : (T)0;

    int atom, ti, n_outer, n_inner;
    const bool active = position_header<T>(a, p, atom, ti, n_outer, n_inner);
    const T rr_inv = (T)1 / a.rr, ra_inv = (T)1 / a.ra;

    T F[NTC][KC];                 // radial functions summed per neighbour species
#pragma unroll
    for (int t = 0; t < NTC; t++)
#pragma unroll
        for (int k = 0; k < KC; k++) F[t][k] = (T)0;
    T S[NAC][NLM];
#pragma unroll
    for (int n = 0; n < NAC; n++)
#pragma unroll
        for (int m = 0; m < NLM; m++) S[n][m] = (T)0;
    __syncthreads();

    // neighbours inside the angular cutoff: radial sums and angular moments
    walk_list<T, true>(a.cv, tile, lane, st, n_inner, true, [&](bool valid, T x, T y, T z, int bits) __attribute__((always_inline)) {
        const int tj = min((bits >> CL_TYPE_SHIFT) & 15, nt - 1);
        const T r = sqrt_t(x * x + y * y + z * z);
        const T rinv = (T)1 / r;
        T f[KC], df[KC];
        radial_functions<T, false>(r, rr_inv, f, df);
#pragma unroll
        for (int t = 0; t < NTC; t++) {
            const T mt = (valid && tj == t) ? (T)1 : (T)0;
#pragma unroll
            for (int k = 0; k < KC; k++) F[t][k] += mt * f[k];
        }
        radial_functions<T, false>(r, ra_inv, f, df);
        const T* c = L.coef + ((ti * nt + tj) * NB + NR) * KC;
        T bl[NLM];
        blm_values<T, LC>(x * rinv, y * rinv, z * rinv, bl);
#pragma unroll
        for (int n = 0; n < NAC; n++) {
            T c0v[4], c1v[4];
            ld4(c + n * KC, c0v);
            ld4(c + n * KC + 4, c1v);
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
    // neighbours between the cutoffs: radial sums only
    walk_list<T, true>(a.cv, tile, lane, st, n_outer, false, [&](bool valid, T x, T y, T z, int bits) __attribute__((always_inline)) {
        const int tj = min((bits >> CL_TYPE_SHIFT) & 15, nt - 1);
        const T r = sqrt_t(x * x + y * y + z * z);
        T f[KC], df[KC];
        radial_functions<T, false>(r, rr_inv, f, df);
#pragma unroll
        for (int t = 0; t < NTC; t++) {
            const T mt = (valid && tj == t) ? (T)1 : (T)0;
#pragma unroll
            for (int k = 0; k < KC; k++) F[t][k] += mt * f[k];
        }
    });

    // ---- descriptors (nepBasis.h:174-190) -------------------------------------------------------
    T q[DC];
#pragma unroll
    for (int j = 0; j < DC; j++) q[j] = (T)0;
#pragma unroll
    for (int t = 0; t < NTC; t++) {
        if (t < nt) {
            const T* c = L.coef + (ti * nt + t) * NB * KC;
#pragma unroll
            for (int n = 0; n < NR; n++) {
                T c0v[4], c1v[4];
                ld4(c + n * KC, c0v);
                ld4(c + n * KC + 4, c1v);
#pragma unroll
                for (int k = 0; k < 4; k++) q[n] += c0v[k] * F[t][k];
#pragma unroll
                for (int k = 0; k < 4; k++) q[n] += c1v[k] * F[t][4 + k];
            }
        }
    }
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
            q[NR + n * LC + (l - 1)] = acc;
        }

    // ---- hidden layer (nep.h:415-447) --------------------------------------------------------------
    T dEdq[DC];
    T e_site = active ? a.bias[ti] : (T)0;
    if constexpr (HM) {
        static_assert(std::is_same<T, float>::value, "the matrix-core hidden layer is fp32");
        float qn[FDP];
#pragma unroll
        for (int j = 0; j < FDP; j++) qn[j] = j < DC ? q[j] * L.qs[j] : 0.0f;
        float e_net = 0.0f;
        hidden_layer_mfma<NTC, DC>(L, st, H, ti, lane, qn, e_net);
        e_site += active ? e_net : 0.0f;
#pragma unroll
        for (int j = 0; j < DC; j++) dEdq[j] = qn[j] * L.qs[j];
    } else {
        T qn[DC];
#pragma unroll
        for (int j = 0; j < DC; j++) { qn[j] = q[j] * L.qs[j]; dEdq[j] = (T)0; }
        for (int pn = 0; pn < H; pn++) {
            const T* wrow = L.w0 + (size_t)(ti * H + pn) * FDP;
            T wv_[FDP];
#pragma unroll
            for (int j = 0; j < FDP; j += 4) {
                T v[4];
                ld4(wrow + j, v);
                wv_[j] = v[0]; wv_[j + 1] = v[1]; wv_[j + 2] = v[2]; wv_[j + 3] = v[3];
            }
            T h = L.b0[ti * H + pn];
#pragma unroll
            for (int j = 0; j < DC; j++) h += wv_[j] * qn[j];
            const T t = tanh_t(h);
            const T w1p = L.w1[ti * H + pn];
            e_site += active ? w1p * t : (T)0;
            const T sde = w1p * ((T)1 - t * t);
#pragma unroll
            for (int j = 0; j < DC; j++) dEdq[j] += sde * wv_[j];
        }
#pragma unroll
        for (int j = 0; j < DC; j++) dEdq[j] *= L.qs[j];
    }

    // ---- dE/dS in place of the moments (nep.h:450-466) ----------------------------------------------
#pragma unroll
    for (int n = 0; n < NAC; n++)
#pragma unroll
        for (int m = 0; m < NLM; m++) {
            const int l = m < 3 ? 1 : m < 8 ? 2 : m < 15 ? 3 : 4;
            const int mp = m - (l * l - 1);
            S[n][m] = S[n][m] * dEdq[NR + n * LC + (l - 1)] * (T)(mp == 0 ? 2.0 : 4.0) * (T)kC3B[m];
        }
    // ---- the radial coefficients contracted with dE/dq: the thread's own copy in LDS (over the network
    // tables, which every wavefront has finished with), a copy in memory for the neighbours
    __syncthreads();
#pragma unroll
    for (int t = 0; t < NTC; t++) {
        T cc[KC];
#pragma unroll
        for (int k = 0; k < KC; k++) cc[k] = (T)0;
        if (t < nt) {
            const T* c = L.coef + (ti * nt + t) * NB * KC;
#pragma unroll
            for (int n = 0; n < NR; n++) {
                T c0v[4], c1v[4];
                ld4(c + n * KC, c0v);
                ld4(c + n * KC + 4, c1v);
#pragma unroll
                for (int k = 0; k < 4; k++) { cc[k] += dEdq[n] * c0v[k]; cc[4 + k] += dEdq[n] * c1v[k]; }
            }
        }
#pragma unroll
        for (int k = 0; k < KC; k++) L.acc[(t * KC + k) * CB + tid] = cc[k];
        if (active) {
            T lo[4] = {cc[0], cc[1], cc[2], cc[3]}, hi[4] = {cc[4], cc[5], cc[6], cc[7]};
            st4(a.rcc + ((size_t)p * NTC + t) * KC, lo);
            st4(a.rcc + ((size_t)p * NTC + t) * KC + 4, hi);
        }
    }

    // ---- pairs inside the angular cutoff: g_ij = dE_i/dr_ij, radial and angular part (nep.h:468-515) ----
    T fx = (T)0, fy = (T)0, fz = (T)0;
    T vir[9];
#pragma unroll
    for (int i = 0; i < 9; i++) vir[i] = (T)0;
    if (a.force || a.want_virial) {
        const bool hand_over = a.force != nullptr;
        walk_list<T, true>(a.cv, tile, lane, st, n_inner, true, [&](bool valid, T x, T y, T z, int bits) __attribute__((always_inline)) {
            int j = bits & CL_INDEX_MASK;
            if (valid && j >= a.cv.natoms) { atomicOr(a.status, ST_BAD_NEIGHBOR); valid = false; }
            if (!valid) return;
            const int tj = min((bits >> CL_TYPE_SHIFT) & 15, nt - 1);
            // the place of this pair among the pairs that name atom j
            int place = 0;
            if (hand_over) place = atomicAdd(a.incoming + j, 1);
            const T r = sqrt_t(x * x + y * y + z * z);
            const T rinv = (T)1 / r;
            const T ux = x * rinv, uy = y * rinv, uz = z * rinv;
            T f[KC], df[KC];
            T srad;
            {
                T ck[KC];
#pragma unroll
                for (int k = 0; k < KC; k++) ck[k] = L.acc[(tj * KC + k) * CB + tid];
                srad = radial_derivative_dot<T>(r, rr_inv, ck);
            }
            radial_functions<T, true>(r, ra_inv, f, df);
            const T* ci = L.coef + ((ti * nt + tj) * NB + NR) * KC;
            T A[NLM], Ad[NLM];
#pragma unroll
            for (int m = 0; m < NLM; m++) { A[m] = (T)0; Ad[m] = (T)0; }
#pragma unroll
            for (int n = 0; n < NAC; n++) {
                T c0v[4], c1v[4];
                ld4(ci + n * KC, c0v);
                ld4(ci + n * KC + 4, c1v);
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
            const T gx = srad * ux + wx * rinv, gy = srad * uy + wy * rinv, gz = srad * uz + wz * rinv;
            if (hand_over) {
                if (place < NSLOT) {
                    const T g4[4] = {gx, gy, gz, (T)0};
                    st4(a.slots + ((size_t)place * a.cv.natoms + j) * 4, g4);
                } else {
                    unsigned long long* row = a.overflow + (size_t)j * OverflowRow<T>::WORDS;
                    // (a comparison with NaN is false)
                    if (fabs((double)gx) < a.overflow_limit && fabs((double)gy) < a.overflow_limit &&
                        fabs((double)gz) < a.overflow_limit) {
                        OverflowRow<T>::add(row, 0, gx);
                        OverflowRow<T>::add(row, 1, gy);
                        OverflowRow<T>::add(row, 2, gz);
                    } else {
                        atomicAdd(row + OverflowRow<T>::BAD, 1ull);
                    }
                }
            }
            fx += gx; fy += gy; fz += gz;
            vir[0] -= gx * x; vir[1] -= gx * y; vir[2] -= gx * z;
            vir[3] -= gy * x; vir[4] -= gy * y; vir[5] -= gy * z;
            vir[6] -= gz * x; vir[7] -= gz * y; vir[8] -= gz * z;
        });
        if (active && a.force) {
            T* fo = a.force + (size_t)atom * 3;
            fo[0] = fx; fo[1] = fy; fo[2] = fz;
        }
    }

    // ---- workgroup partial sums of the energy and of this kernel's share of the virial (fp64) ----------
    {
        double vals[10];
        vals[0] = active ? (double)e_site : 0.0;
#pragma unroll
        for (int i = 0; i < 9; i++) vals[1 + i] = active ? (double)vir[i] : 0.0;
        const int nv = a.want_virial ? 10 : 1;
#pragma unroll
        for (int i = 0; i < 10; i++)
            if (i < nv) {                          // wave-uniform
                const double v = wave_sum(vals[i]);
                if (lane == 0) L.red[wv * 10 + i] = v;
            }
        __syncthreads();
        if (tid < nv) {
            double v = 0.0;
            for (int w = 0; w < CB / 64; w++) v += L.red[w * 10 + tid];
            a.partial[(size_t)blk * 10 + tid] = v;
        }
    }
}

// ---- kernel 2: pairs between the cutoffs by gather, and the slots -----------------------------------------
template <typename T, int NTC>
__global__ void __launch_bounds__(CB)
nep_gather_kernel(const GatherArgs<T> a)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int blk = xcd_block(blockIdx.x, gridDim.x);
    const int p = blk * CB + tid;
    const int tile = p >> 6;
    const int nt = a.ntypes;
    GatherLds<T> L;
    gather_lds<T>(smem_raw, L);
    T* const st = L.stage + (size_t)wv * 64 * STP * 4;

    int atom, ti, n_outer, n_inner;
    const bool active = position_header<T>(a, p, atom, ti, n_outer, n_inner);
    const T rr_inv = (T)1 / a.rr;

    // own contracted radial coefficients, one array per neighbour species (separate arrays: a select between
    // them stays a select, where one two-dimensional array would be indexed through scratch memory)
    T cc0[KC], cc1[KC], cc2[KC], cc3[KC];
    auto load_cc = [&](int t, T (&c)[KC]) __attribute__((always_inline)) {
        T lo[4] = {(T)0, (T)0, (T)0, (T)0}, hi[4] = {(T)0, (T)0, (T)0, (T)0};
        if (active && t < NTC) { ld4(a.rcc + ((size_t)p * NTC + t) * KC, lo); ld4(a.rcc + ((size_t)p * NTC + t) * KC + 4, hi); }
#pragma unroll
        for (int k = 0; k < 4; k++) { c[k] = lo[k]; c[4 + k] = hi[k]; }
    };
    load_cc(0, cc0); load_cc(1, cc1); load_cc(2, cc2); load_cc(3, cc3);

    T fx = (T)0, fy = (T)0, fz = (T)0;
    T vir[9];
#pragma unroll
    for (int i = 0; i < 9; i++) vir[i] = (T)0;
    // g_ij - g_ji = (cc_i[t_j] + cc_j[t_i]) . f'(r) r_ij / r
    walk_list<T, true>(a.cv, tile, lane, st, n_outer, false, [&](bool valid, T x, T y, T z, int bits) __attribute__((always_inline)) {
        const int j = bits & CL_INDEX_MASK;
        if (valid && j >= a.cv.natoms) { atomicOr(a.status, ST_BAD_NEIGHBOR); valid = false; }
        if (!valid) return;                  // lanes past the end of their list issue no loads
        const int tj = min((bits >> CL_TYPE_SHIFT) & 15, nt - 1);
        T lo[4], hi[4];
        ld4(a.rcc + ((size_t)j * NTC + ti) * KC, lo);
        ld4(a.rcc + ((size_t)j * NTC + ti) * KC + 4, hi);
        const T r = sqrt_t(x * x + y * y + z * z);
        T ck[KC];
#pragma unroll
        for (int k = 0; k < KC; k++) {
            ck[k] = cc0[k];
            if (NTC > 1) ck[k] = tj == 1 ? cc1[k] : ck[k];
            if (NTC > 2) ck[k] = tj == 2 ? cc2[k] : ck[k];
            if (NTC > 3) ck[k] = tj == 3 ? cc3[k] : ck[k];
        }
#pragma unroll
        for (int k = 0; k < 4; k++) { ck[k] += lo[k]; ck[4 + k] += hi[k]; }
        const T sr = radial_derivative_dot<T>(r, rr_inv, ck) / r;
        const T gx = sr * x, gy = sr * y, gz = sr * z;
        fx += gx; fy += gy; fz += gz;
        vir[0] -= gx * x; vir[1] -= gx * y; vir[2] -= gx * z;
        vir[3] -= gy * x; vir[4] -= gy * y; vir[5] -= gy * z;
        vir[6] -= gz * x; vir[7] -= gz * y; vir[8] -= gz * z;
    });

    // what the neighbours inside the angular cutoff handed over: F_i -= sum_j g_ji
    if (p < a.cv.natoms && a.force) {
        const int n = a.incoming[p];
        a.incoming[p] = 0;                                  // the next call finds the counters at zero
        FixedSum<T> sx, sy, sz;
        double mag = 0.0;                                   // NaN or inf in a slot makes this NaN or inf
        for (int t = 0; t < min(n, NSLOT); t++) {
            T v[4];
            ld4_stream(a.slots + ((size_t)t * a.cv.natoms + p) * 4, v);        // read once
            mag += fabs((double)v[0]) + fabs((double)v[1]) + fabs((double)v[2]);
            sx.add(v[0]); sy.add(v[1]); sz.add(v[2]);
        }
        bool ok = mag < kFixedSumLimit;
        if (n > NSLOT) {
            unsigned long long* row = a.overflow + (size_t)p * OverflowRow<T>::WORDS;
            ok = ok && row[OverflowRow<T>::BAD] == 0ull;
            row[OverflowRow<T>::BAD] = 0ull;
            OverflowRow<T>::take(row, 0, sx);
            OverflowRow<T>::take(row, 1, sy);
            OverflowRow<T>::take(row, 2, sz);
        }
        if (active) {
            T* fo = a.force + (size_t)atom * 3;
            const double nan = __longlong_as_double(0x7ff8000000000000ll);
            fo[0] = (T)(ok ? (double)fo[0] + (double)fx - sx.value() : nan);
            fo[1] = (T)(ok ? (double)fo[1] + (double)fy - sy.value() : nan);
            fo[2] = (T)(ok ? (double)fo[2] + (double)fz - sz.value() : nan);
        }
    }
    // every pair between the cutoffs was met from both ends: half of this sum is their virial
    if (a.want_virial) {
        double vals[9];
#pragma unroll
        for (int i = 0; i < 9; i++) vals[i] = active ? 0.5 * (double)vir[i] : 0.0;
#pragma unroll
        for (int i = 0; i < 9; i++) {
            const double v = wave_sum(vals[i]);
            if (lane == 0) L.red[wv * 9 + i] = v;
        }
        __syncthreads();
        if (tid < 9) {
            double v = a.partial[(size_t)blk * 10 + 1 + tid];      // the adjoint kernel's share
            for (int w = 0; w < CB / 64; w++) v += L.red[w * 9 + tid];
            a.partial[(size_t)blk * 10 + 1 + tid] = v;
        }
    }
}

// Which unit runs the hidden layer: 0 vector ALUs (one thread per atom), 1 matrix cores (fp32, at most 64
// neurons).  AI2POT_NEP_HIDDEN=valu|mfma overrides the default; a2p_nep_hidden_layer_unit sets it at run time.
int g_hidden_unit = -1;
int hidden_unit()
{
    if (g_hidden_unit < 0) {
        const char* e = getenv("AI2POT_NEP_HIDDEN");
        g_hidden_unit = (e && std::string(e) == "mfma") ? 1 : (e && std::string(e) == "valu") ? 0 : kHiddenDefault;
    }
    return g_hidden_unit;
}

template <typename T, int NTC, int NR>
auto adjoint_kernel_for(bool mfma)
{
    if constexpr (std::is_same<T, float>::value && NTC <= HM_NTC_MAX) {
        if (mfma) return nep_adjoint_kernel<T, NTC, NR, true>;
    }
    return nep_adjoint_kernel<T, NTC, NR, false>;
}

template <typename T, int NTC, int NR>
int launch_gather(const GatherArgs<T>& a, int nblocks, bool pairs, hipStream_t stream)
{
    AdjointLds<T> la;
    GatherLds<T> lg;
    const bool mfma = std::is_same<T, float>::value && NTC <= HM_NTC_MAX && hidden_unit() == 1 && a.H <= HM_NT * HM_TILE;
    const size_t lds_a = adjoint_lds<T>(a.ntypes, NTC, a.H, NR + NAC, nullptr, la, mfma);
    const size_t lds_g = gather_lds<T>(nullptr, lg);
    auto ka = adjoint_kernel_for<T, NTC, NR>(mfma);
    auto kg = nep_gather_kernel<T, NTC>;
    if (lds_a > 48 * 1024)
        A2P_HIP_CHECK(hipFuncSetAttribute((const void*)ka, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_a));
    if (lds_g > 48 * 1024)
        A2P_HIP_CHECK(hipFuncSetAttribute((const void*)kg, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_g));
    prof_begin("nep_adjoint_kernel", stream);
    hipLaunchKernelGGL(ka, dim3(nblocks), dim3(CB), lds_a, stream, a);
    prof_end(stream);
    if (pairs) {
        prof_begin("nep_gather_kernel", stream);
        hipLaunchKernelGGL(kg, dim3(nblocks), dim3(CB), lds_g, stream, a);
        prof_end(stream);
    }
    A2P_HIP_CHECK(hipGetLastError());
    return A2P_OK;
}

int ntc_of(int ntypes) { return ntypes <= 1 ? 1 : ntypes == 2 ? 2 : ntypes == 3 ? 3 : 4; }

template <typename T>
size_t compact_lds_need(int n_r, int H, int ntypes)
{
    AdjointLds<T> la;
    GatherLds<T> lg;
    return std::max(adjoint_lds<T>(ntypes, ntc_of(ntypes), H, n_r + NAC, nullptr, la), gather_lds<T>(nullptr, lg));
}

bool compact_shape_ok(int K, int n_r, int n_a, int l_max, int H, int ntypes)
{
    return K == KC && (n_r == 4 || n_r == 6) && n_a == NAC && l_max == LC && ntypes >= 1 && ntypes <= 4 && H >= 1;
}

constexpr size_t kLdsLimit = 150 * 1024;

template <typename T>
int nep_efv_compact(int K, int n_r, int n_a, int l_max, int H, int ntypes, const T* coeffs, const T* w0, const T* b0,
                    const T* w1, const T* bias, const T* q_scaler, double rr, double ra, int natoms, int umax,
                    const int* types, void* compact, T* etot, T* force, T* virial, hipStream_t stream)
{
    A2P_REQUIRE(compact_shape_ok(K, n_r, n_a, l_max, H, ntypes), A2P_ERR_INVALID,
                "nep (compact lists): model shape not covered (chebyshev_size 8, n_radial 4 or 6, n_angular 4, l_max 4, "
                "at most 4 species); use the padded-list entry points");
    A2P_REQUIRE(H >= 1, A2P_ERR_INVALID, "nep: num_neurons must be positive");
    A2P_REQUIRE(compact_supported(natoms, umax), A2P_ERR_INVALID, "nep (compact lists): bad natoms / umax");
    A2P_REQUIRE(rr > 0 && ra > 0, A2P_ERR_INVALID, "nep: cutoffs must be positive");
    A2P_REQUIRE(coeffs && w0 && b0 && w1 && bias && q_scaler && types && compact && etot, A2P_ERR_INVALID,
                "nep (compact lists): null pointer");
    GatherArgs<T> a;
    a.H = H; a.ntypes = ntypes;
    a.coeffs = coeffs; a.w0 = w0; a.b0 = b0; a.w1 = w1; a.bias = bias; a.q_scaler = q_scaler;
    a.rr = (T)rr; a.ra = (T)ra;
    a.cv = compact_view<T>(compact, natoms, umax);
    a.types = types;
    a.force = force;
    a.want_virial = virial != nullptr;
    const int nblocks = ceil_div(a.cv.npad, CB);
    {
        const size_t need = compact_lds_need<T>(n_r, H, ntypes);
        A2P_REQUIRE(need <= kLdsLimit, A2P_ERR_INVALID, "nep (compact lists): %zu bytes of LDS needed (num_neurons %d)",
                    need, H);
    }
    void* ws = nullptr;
    int rc = ws_get(WS_FLAGS, 64, &ws);
    if (rc) return rc;
    a.status = (int*)ws;
    rc = ws_get(WS_PARTIAL, (size_t)nblocks * 10 * sizeof(double), &ws);
    if (rc) return rc;
    a.partial = (double*)ws;
    const bool pairs = force != nullptr || virial != nullptr;
    const size_t n_rcc = (size_t)natoms * ntc_of(ntypes) * KC, n_slots = (size_t)NSLOT * natoms * 4;
    rc = ws_get(WS_PAIR_G, (n_rcc + n_slots) * sizeof(T), &ws);
    if (rc) return rc;
    a.rcc = (T*)ws;
    a.slots = a.rcc + n_rcc;
    // spare rows | counters of claimed places: zero when allocated, and nep_gather_kernel leaves them zero
    const size_t ovf_bytes = (size_t)natoms * OverflowRow<T>::WORDS * sizeof(unsigned long long);
    rc = ws_get(WS_NEP_CLAIMS, ovf_bytes + (size_t)natoms * sizeof(int), &ws);
    if (rc) return rc;
    a.overflow = (unsigned long long*)ws;
    a.incoming = (int*)((unsigned char*)ws + ovf_bytes);
    a.overflow_limit = kFixedSumLimit / (double)umax;       // umax values of that size still sum below 2^21
    auto launch = [&](auto nr) {
        constexpr int NR = decltype(nr)::value;
        switch (ntc_of(ntypes)) {
        case 1: return launch_gather<T, 1, NR>(a, nblocks, pairs, stream);
        case 2: return launch_gather<T, 2, NR>(a, nblocks, pairs, stream);
        case 3: return launch_gather<T, 3, NR>(a, nblocks, pairs, stream);
        default: return launch_gather<T, 4, NR>(a, nblocks, pairs, stream);
        }
    };
    rc = n_r == 4 ? launch(std::integral_constant<int, 4>{}) : launch(std::integral_constant<int, 6>{});
    if (rc) {
        (void)ws_drop(WS_NEP_CLAIMS);       // a launch that failed may have left counters behind
        return rc;
    }
    return finish_energy_virial<T>(etot, virial, a.partial, 1, nblocks, stream);
}

}  // namespace
}  // namespace a2p

extern "C" {

int a2p_nep_hidden_layer_unit(int unit)
{
    const int before = a2p::hidden_unit();
    if (unit == 0 || unit == 1) a2p::g_hidden_unit = unit;
    return before;
}

int a2p_nep_efv_compact_supported(int K, int n_r, int n_a, int l_max, int H, int ntypes, int elem_size)
{
    if (!a2p::compact_shape_ok(K, n_r, n_a, l_max, H, ntypes)) return 0;
    if (elem_size == 4) return a2p::compact_lds_need<float>(n_r, H, ntypes) <= a2p::kLdsLimit;
    if (elem_size == 8) return a2p::compact_lds_need<double>(n_r, H, ntypes) <= a2p::kLdsLimit;
    return 0;
}

int a2p_nep_efv_compact_f32(int K, int n_r, int n_a, int l_max, int H, int ntypes, const float* coeffs,
                            const float* w0, const float* b0, const float* w1, const float* bias,
                            const float* q_scaler, double rr, double ra, int natoms, int umax, const int* types,
                            void* compact, float* etot, float* force, float* virial, void* stream)
{
    return a2p::nep_efv_compact<float>(K, n_r, n_a, l_max, H, ntypes, coeffs, w0, b0, w1, bias, q_scaler, rr, ra,
                                       natoms, umax, types, compact, etot, force, virial, (hipStream_t)stream);
}

int a2p_nep_efv_compact_f64(int K, int n_r, int n_a, int l_max, int H, int ntypes, const double* coeffs,
                            const double* w0, const double* b0, const double* w1, const double* bias,
                            const double* q_scaler, double rr, double ra, int natoms, int umax, const int* types,
                            void* compact, double* etot, double* force, double* virial, void* stream)
{
    return a2p::nep_efv_compact<double>(K, n_r, n_a, l_max, H, ntypes, coeffs, w0, b0, w1, bias, q_scaler, rr, ra,
                                        natoms, umax, types, compact, etot, force, virial, (hipStream_t)stream);
}
}
