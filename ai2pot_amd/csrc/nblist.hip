// Periodic neighbour list for gfx950, bit-exact to the reference's
// source/nblist/include/{structure.h, binLinkedList.h, neighborList.h}.
//
// The reference replicates the cell into an explicit supercell of (2*ceil(rcut/d_a)+1)
// images per periodic axis, bins every image atom into rcut/2 bins by head insertion and,
// per centre atom, walks 5x5x5 bins (dx outer, dz inner), each bin in descending supercell
// index.  Only image atoms that fall into the bins around the centre cell can ever be
// visited, so here the supercell is never materialised:
//   1. coords   : Cartesian coordinates; min / max of ALL image coordinates (they define
//                 the reference's bin origin) and of the centre atoms, by reduction
//   2. count    : every (atom, image) pair computes its reference bin with the reference's
//                 rounding; those inside the bin box around the centre atoms are counted
//   3. scan     : prefix sum over the box's bins (z fastest, so the five dz bins of one
//                 (dx, dy) column are contiguous)
//   4. fill     : image atoms copied into their bin segment
//   5. binsort  : each bin ordered by descending supercell index (= the head-insertion order)
//   6. lists    : one wavefront per centre atom walks the 25 (dx, dy) columns in reference
//                 order; 64 candidates are distance-tested at a time with the reference's
//                 mixed float/double arithmetic and compacted in order with a wave ballot
//                 and prefix popcount; the padded row (-1 / 0 fill) is written in the same pass
//   7. sort     : (sort = true) per atom, the same introsort + insertion sort sequence as
//                 libstdc++'s std::sort on float-rounded distances, so ties land where the
//                 reference puts them
// This translation unit is compiled with -ffp-contract=off and spells the critical
// operations with the *_rn intrinsics: no fused multiply-add may change a rounding.
#include "a2p_common.h"
#include "compact_list.h"

#include <hipcub/hipcub.hpp>

#include <climits>
#include <cmath>
#include <vector>

namespace a2p {
namespace {

constexpr double kMargin = 0.5;      // NBLIST_MARGIN, structure.h:27
constexpr double kEpsilon = 1e-3;    // EPSILON, binLinkedList.h:28
constexpr int NBL_BLOCK = 256;

__device__ __forceinline__ float add_rn(float a, float b) { return __fadd_rn(a, b); }
__device__ __forceinline__ float sub_rn(float a, float b) { return __fsub_rn(a, b); }
__device__ __forceinline__ float mul_rn(float a, float b) { return __fmul_rn(a, b); }
__device__ __forceinline__ float div_rn(float a, float b) { return __fdiv_rn(a, b); }
__device__ __forceinline__ double add_rn(double a, double b) { return __dadd_rn(a, b); }
__device__ __forceinline__ double sub_rn(double a, double b) { return __dsub_rn(a, b); }
__device__ __forceinline__ double mul_rn(double a, double b) { return __dmul_rn(a, b); }
__device__ __forceinline__ double div_rn(double a, double b) { return __ddiv_rn(a, b); }

template <typename T>
struct Grid {
    T b[3][3];        // lattice rows
    T mn[3];          // bin origin: min over all image coordinates - 0.5
    T bin_size;       // rcut / 2
    T rcut;
    double rcut2;     // std::pow(rcut, 2) evaluated in double
    int nbin[3];      // the reference's bin counts
    int rlo[3];       // bin box kept here: [rlo, rlo + rdim)
    int rdim[3];
    int img_lo[3];    // image index ranges
    int img_dim[3];
    int nimg;
    int N;
    int ext_bins;     // ceil(rcut / bin_size) = 2
    int is_cart;
    float inv_side;   // 1 / (2 ext_bins + 1), 1 / bin_size: for the pruning arithmetic of the
    float inv_bin;    // list kernel, which is approximate by design
    T keep_lo[3];     // coordinates outside [keep_lo, keep_hi] lie outside the kept bin box for sure
    T keep_hi[3];     // (the box widened by far more than the rounding of the binning)
};

// The part of the grid that follows from the extents of the coordinates.  A build that does not read the
// extents back to the host (a2p_nblist_sync_free) has a one-thread kernel derive it on the device; the other
// kernels then take these fields from device memory instead of their by-value Grid argument.
template <typename T>
struct GridDyn {
    T mn[3], keep_lo[3], keep_hi[3];
    int nbin[3], rlo[3], rdim[3];
    int nregion;
};

template <typename T>
__device__ __forceinline__ Grid<T> with_dyn(const Grid<T>& in, const GridDyn<T>* __restrict__ gd)
{
    Grid<T> g = in;
    if (gd) {
#pragma unroll
        for (int a = 0; a < 3; a++) {
            g.mn[a] = gd->mn[a]; g.keep_lo[a] = gd->keep_lo[a]; g.keep_hi[a] = gd->keep_hi[a];
            g.nbin[a] = gd->nbin[a]; g.rlo[a] = gd->rlo[a]; g.rdim[a] = gd->rdim[a];
        }
    }
    return g;
}

// image coordinate x + b0*ii + b1*jj + b2*kk, left to right (structure.h:659-676)
template <typename T>
__device__ __forceinline__ T image_coord(T x, T b0, T b1, T b2, int ii, int jj, int kk)
{
    T v = add_rn(x, mul_rn(b0, (T)ii));
    v = add_rn(v, mul_rn(b1, (T)jj));
    return add_rn(v, mul_rn(b2, (T)kk));
}

template <typename T>
__device__ __forceinline__ int bin_of(T c, T mn, T bin_size)      // binLinkedList.h:824-826
{
    return (int)floor(div_rn(sub_rn(c, mn), bin_size));
}

// ---- 1. coordinates and extents --------------------------------------------------------------
template <typename T>
__global__ void coords_minmax_kernel(const Grid<T> g, const T* __restrict__ coords, T* __restrict__ x,
                                     T* __restrict__ partial)
{
    __shared__ T sh[NBL_BLOCK / 64][12];
    const int p = blockIdx.x * NBL_BLOCK + threadIdx.x;
    T v[12];
#pragma unroll
    for (int a = 0; a < 3; a++) {
        v[a] = (T)INT_MAX; v[3 + a] = (T)INT_MIN;       // structure.h:1018-1022
        v[6 + a] = (T)INT_MAX; v[9 + a] = (T)INT_MIN;
    }
    if (p < g.N) {
        T c[3];
        if (g.is_cart) {
#pragma unroll
            for (int a = 0; a < 3; a++) c[a] = coords[(size_t)p * 3 + a];
        } else {                                         // calc_cart_coords, structure.h:561-579
            const T f0 = coords[(size_t)p * 3], f1 = coords[(size_t)p * 3 + 1], f2 = coords[(size_t)p * 3 + 2];
#pragma unroll
            for (int a = 0; a < 3; a++)
                c[a] = add_rn(add_rn(mul_rn(f0, g.b[0][a]), mul_rn(f1, g.b[1][a])), mul_rn(f2, g.b[2][a]));
        }
#pragma unroll
        for (int a = 0; a < 3; a++) {
            x[(size_t)p * 3 + a] = c[a];
            v[6 + a] = c[a];
            v[9 + a] = c[a];
        }
        // Extremes over the atom's images (structure.h:1018-1052 takes them over the whole supercell).  Rounded
        // multiplication and addition are monotone in each operand, so image_coord is monotone in each image
        // index, rising or falling with the sign of the lattice component: the extremes sit at the ends of
        // the index ranges, and two images per axis give the same values as the loop over all of them.
#pragma unroll
        for (int a = 0; a < 3; a++) {
            int lo[3], hi[3];
#pragma unroll
            for (int w = 0; w < 3; w++) {
                const int first = g.img_lo[w], last = g.img_lo[w] + g.img_dim[w] - 1;
                const bool rising = g.b[w][a] >= (T)0;
                lo[w] = rising ? first : last;
                hi[w] = rising ? last : first;
            }
            v[a] = image_coord(c[a], g.b[0][a], g.b[1][a], g.b[2][a], lo[0], lo[1], lo[2]);
            v[3 + a] = image_coord(c[a], g.b[0][a], g.b[1][a], g.b[2][a], hi[0], hi[1], hi[2]);
        }
    }
#pragma unroll
    for (int q = 0; q < 12; q++) {
        const bool is_min = (q % 6) < 3;
        T r = v[q];
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            T o = __shfl_xor(r, off, 64);
            r = is_min ? (o < r ? o : r) : (o > r ? o : r);
        }
        if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6][q] = r;
    }
    __syncthreads();
    if (threadIdx.x < 12) {
        const int q = threadIdx.x;
        const bool is_min = (q % 6) < 3;
        T r = sh[0][q];
        for (int w = 1; w < NBL_BLOCK / 64; w++) {
            T o = sh[w][q];
            r = is_min ? (o < r ? o : r) : (o > r ? o : r);
        }
        partial[(size_t)blockIdx.x * 12 + q] = r;
    }
}

// 12 wavefronts, one per extent (minima of the image coordinates, their maxima, minima and maxima
// of the centre atoms, three axes each)
template <typename T>
__global__ void minmax_finish_kernel(const T* __restrict__ partial, int nblocks, T* __restrict__ out)
{
    const int q = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const bool is_min = (q % 6) < 3;
    T r = is_min ? (T)INT_MAX : (T)INT_MIN;
    for (int k0 = lane; k0 < nblocks; k0 += 64 * 8) {
        T o[8];                                    // eight loads in flight
#pragma unroll
        for (int u = 0; u < 8; u++) o[u] = partial[(size_t)min(k0 + 64 * u, nblocks - 1) * 12 + q];
#pragma unroll
        for (int u = 0; u < 8; u++) r = is_min ? (o[u] < r ? o[u] : r) : (o[u] > r ? o[u] : r);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const T o = __shfl_xor(r, off, 64);
        r = is_min ? (o < r ? o : r) : (o > r ? o : r);
    }
    if (lane == 0) out[q] = r;
}

// ---- 1b. bin grid from the extents, on the device (builds that do not read the extents back) ----------
// The arithmetic of find_pl_info4nblist and of the bin counts (structure.h:1013-1061, binLinkedList.h:685-688) as
// the host does it in the synchronised build, in T with correctly rounded operations.  The box must fit the
// bound the host sized its launches and scratch arrays for, and its coordinates the bound the host assumed:
// otherwise (or if an extent is not finite) the box
// is made empty, so that no kernel indexes beyond the bound, and ST_GRID_BOUND is raised.
template <typename T>
__global__ void grid_setup_kernel(const Grid<T> g, const T* __restrict__ ext, GridDyn<T>* __restrict__ gd, int cap0,
                                  int cap1, int cap2, double big_bound, int* __restrict__ status)
{
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    const int cap[3] = {cap0, cap1, cap2};
    bool ok = true;
    long long nregion = 1;
    for (int a = 0; a < 3; a++) {
        const T lo = ext[a], hi = ext[3 + a];
        if (!(fabs((double)lo) < 1.0e30) || !(fabs((double)hi) < 1.0e30)) ok = false;    // NaN, infinity or absurd
        const T mn = sub_rn(lo, (T)kMargin);
        const T mx = add_rn(hi, (T)kMargin);
        const T pl = sub_rn(mx, mn);
        if (!((double)pl / (double)g.bin_size < 1.0e9)) ok = false;       // the bin counts below must fit an int
        const int nbin = (int)ceil(div_rn(pl, g.bin_size));
        const int cb_lo = (int)floor(div_rn(sub_rn(ext[6 + a], mn), g.bin_size));
        const int cb_hi = (int)floor(div_rn(sub_rn(ext[9 + a], mn), g.bin_size));
        const int rlo = max(cb_lo - g.ext_bins, 0);
        const int rhi = min(cb_hi + g.ext_bins, nbin - 1);
        int rdim = rhi - rlo + 1;
        if (rdim <= 0 || rdim > cap[a]) ok = false;
        const double big = fmax(fabs((double)mn), fabs((double)mx));
        const double slack = 1.0e-3 * (double)g.bin_size + 1.0e-5 * (big + (double)pl);
        gd->mn[a] = mn;
        gd->nbin[a] = nbin;
        gd->rlo[a] = rlo;
        gd->rdim[a] = rdim;
        gd->keep_lo[a] = (T)((double)mn + (double)rlo * (double)g.bin_size - slack);
        gd->keep_hi[a] = (T)((double)mn + (double)(rlo + rdim) * (double)g.bin_size + slack);
        // the host sized the symmetry band of the compact lists for coordinates within big_bound
        if (fmax(fabs((double)gd->keep_lo[a]), fabs((double)gd->keep_hi[a])) > big_bound) ok = false;
        nregion *= rdim > 0 ? rdim : 0;
    }
    if (!ok) {
        for (int a = 0; a < 3; a++) { gd->rdim[a] = 0; gd->keep_lo[a] = (T)1; gd->keep_hi[a] = (T)-1; }
        nregion = 0;
        atomicOr(status, ST_GRID_BOUND);
    }
    gd->nregion = (int)nregion;
}

// ---- 2 / 4. binning of (atom, image) pairs ---------------------------------------------------
// Image (i, j, k) of an atom at xp: storage index of its bin inside the box, or -1 when outside.
template <typename T>
__device__ __forceinline__ int locate(const Grid<T>& g, const T (&xp)[3], int i, int j, int k, T* c)
{
    int bin[3];
    // most images of most atoms lie far outside the box: two comparisons per axis settle them
    // before the exactly rounded divisions of the binning
#pragma unroll
    for (int a = 0; a < 3; a++) {
        c[a] = image_coord(xp[a], g.b[0][a], g.b[1][a], g.b[2][a], g.img_lo[0] + i, g.img_lo[1] + j,
                           g.img_lo[2] + k);
        if (c[a] < g.keep_lo[a] || c[a] > g.keep_hi[a]) return -1;
    }
#pragma unroll
    for (int a = 0; a < 3; a++) {
        bin[a] = bin_of(c[a], g.mn[a], g.bin_size) - g.rlo[a];
        if (bin[a] < 0 || bin[a] >= g.rdim[a]) return -1;
    }
    return (bin[0] * g.rdim[1] + bin[1]) * g.rdim[2] + bin[2];
}

// ---- image records: [x y z index], 4 values of T, the index in the bits of the fourth ------------------
template <typename T>
__device__ __forceinline__ void entry_store(T* p, T x, T y, T z, int bits);
template <>
__device__ __forceinline__ void entry_store<float>(float* p, float x, float y, float z, int bits)
{
    *reinterpret_cast<float4*>(p) = make_float4(x, y, z, __int_as_float(bits));
}
template <>
__device__ __forceinline__ void entry_store<double>(double* p, double x, double y, double z, int bits)
{
    *reinterpret_cast<double2*>(p) = make_double2(x, y);
    *reinterpret_cast<double2*>(p + 2) = make_double2(z, __longlong_as_double((long long)bits));
}
// The same, streamed past the caches (non-temporal): for the compact entries, which are written once and read by other
// kernels later; ordinary stores of this much data (1.6 GB per build of a million atoms, with the padded rows) cost the
// list kernel a quarter of its time.
template <typename T>
__device__ __forceinline__ void entry_store_stream(T* p, T x, T y, T z, int bits);
template <>
__device__ __forceinline__ void entry_store_stream<float>(float* p, float x, float y, float z, int bits)
{
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    const f32x4 v = {x, y, z, __int_as_float(bits)};
    __builtin_nontemporal_store(v, reinterpret_cast<f32x4*>(p));
}
template <>
__device__ __forceinline__ void entry_store_stream<double>(double* p, double x, double y, double z, int bits)
{
    typedef double f64x2 __attribute__((ext_vector_type(2)));
    const f64x2 lo = {x, y}, hi = {z, __longlong_as_double((long long)bits)};
    __builtin_nontemporal_store(lo, reinterpret_cast<f64x2*>(p));
    __builtin_nontemporal_store(hi, reinterpret_cast<f64x2*>(p + 2));
}

// the reverse: one 16-byte (fp32) or two 16-byte (fp64) loads
__device__ __forceinline__ void entry_load(const float* p, float& x, float& y, float& z, int& bits)
{
    const float4 v = *reinterpret_cast<const float4*>(p);
    x = v.x; y = v.y; z = v.z; bits = __float_as_int(v.w);
}
__device__ __forceinline__ void entry_load(const double* p, double& x, double& y, double& z, int& bits)
{
    const double2 v0 = *reinterpret_cast<const double2*>(p);
    const double2 v1 = *reinterpret_cast<const double2*>(p + 2);
    x = v0.x; y = v0.y; z = v1.x; bits = (int)__double_as_longlong(v1.y);
}

// One thread per atom walks its images (x outer, z inner: image m = (i * dim_y + j) * dim_z + k,
// supercell index m * N + p, structure.h:654-681).
// With split > 1 (small structures, where a thread per atom leaves most of the chip idle) a thread takes one
// x-layer of an atom's images: thread = atom * split + layer, split = img_dim[0].
template <typename T>
__global__ void count_kernel(const Grid<T> g_in, const T* __restrict__ x, int* __restrict__ counts,
                             int* __restrict__ incoming, const GridDyn<T>* __restrict__ gd,
                             const int* __restrict__ types, int* __restrict__ ilist, int* __restrict__ types_out,
                             int split)
{
    const Grid<T> g = with_dyn(g_in, gd);
    const int t = blockIdx.x * NBL_BLOCK + threadIdx.x;
    const int p = split > 1 ? t / split : t;
    if (p >= g.N) return;
    const int i0 = split > 1 ? t - p * split : 0, i1 = split > 1 ? i0 + 1 : g.img_dim[0];
    if (i0 == 0) {
        if (incoming) incoming[p] = 0;                // counted up by the list kernel
        // neighborList.h:548-553: the two outputs that do not depend on the list are written here, in atom order (the
        // list kernel may process the atoms in another order and would scatter them)
        if (ilist) { ilist[p] = p; types_out[p] = types[p]; }
    }
    const T xp[3] = {x[(size_t)p * 3], x[(size_t)p * 3 + 1], x[(size_t)p * 3 + 2]};
    for (int i = i0; i < i1; i++)
        for (int j = 0; j < g.img_dim[1]; j++)
            for (int k = 0; k < g.img_dim[2]; k++) {
                T c[3];
                const int bin = locate(g, xp, i, j, k, c);
                if (bin >= 0) atomicAdd(&counts[bin], 1);
            }
}

template <typename T>
__global__ void fill_kernel(const Grid<T> g_in, const T* __restrict__ x, const int* __restrict__ offsets,
                            int* __restrict__ cursor, T* __restrict__ s_rec,
                            const GridDyn<T>* __restrict__ gd, int split)
{
    const Grid<T> g = with_dyn(g_in, gd);
    const int t = blockIdx.x * NBL_BLOCK + threadIdx.x;
    const int p = split > 1 ? t / split : t;
    if (p >= g.N) return;
    const int i0 = split > 1 ? t - p * split : 0, i1 = split > 1 ? i0 + 1 : g.img_dim[0];
    const T xp[3] = {x[(size_t)p * 3], x[(size_t)p * 3 + 1], x[(size_t)p * 3 + 2]};
    int m = i0 * g.img_dim[1] * g.img_dim[2];
    for (int i = i0; i < i1; i++)
        for (int j = 0; j < g.img_dim[1]; j++)
            for (int k = 0; k < g.img_dim[2]; k++, m++) {
                T c[3];
                const int bin = locate(g, xp, i, j, k, c);
                if (bin < 0) continue;
                const int pos = offsets[bin] + atomicAdd(&cursor[bin], 1);
                entry_store<T>(s_rec + (size_t)pos * 4, c[0], c[1], c[2], m * g.N + p);
            }
}

// ---- 5. order inside a bin: descending supercell index (head insertion, binLinkedList.h:833) -
// Afterwards only the atom behind a supercell entry matters (neighborList.h:561), so the sorted
// indices are reduced modulo natoms here, once per entry instead of once per candidate pair.
// With `types` the species of the atom rides in the bits above CL_TYPE_SHIFT and CL_IMAGE_BIT marks the
// periodic images (compact lists: the list
// kernel then never gathers a neighbour's species).
template <typename T>
__global__ void binsort_kernel(int nbins, const int* __restrict__ offsets, T* __restrict__ s_rec, int natoms,
                               const int* __restrict__ types, const GridDyn<T>* __restrict__ gd, int central)
{
    if (gd) nbins = gd->nregion;                  // the launch covers the host's bound
    const int b = blockIdx.x * NBL_BLOCK + threadIdx.x;
    if (b >= nbins) return;
    const int beg = offsets[b], end = offsets[b + 1];
    for (int i = beg + 1; i < end; i++) {
        T kx, ky, kz;
        int key;
        entry_load(s_rec + (size_t)i * 4, kx, ky, kz, key);
        int j = i - 1;
        while (j >= beg) {
            T x, y, z;
            int idx;
            entry_load(s_rec + (size_t)j * 4, x, y, z, idx);
            if (idx >= key) break;
            entry_store<T>(s_rec + (size_t)(j + 1) * 4, x, y, z, idx);
            j--;
        }
        entry_store<T>(s_rec + (size_t)(j + 1) * 4, kx, ky, kz, key);
    }
    for (int i = beg; i < end; i++) {
        T x, y, z;
        int idx;
        entry_load(s_rec + (size_t)i * 4, x, y, z, idx);
        const int at = idx % natoms;
        // compact lists: the species, and whether this is an image outside the cell (image number != central)
        entry_store<T>(s_rec + (size_t)i * 4, x, y, z,
                       types ? at | ((types[at] & 15) << CL_TYPE_SHIFT) | (idx / natoms != central ? CL_IMAGE_BIT : 0) : at);
    }
}

// ---- processing order of the compact lists: atoms along a Morton curve through the bins ----------
__device__ __forceinline__ unsigned spread3(unsigned v)      // 10 bits -> every third bit
{
    v &= 0x3ffu;
    v = (v | (v << 16)) & 0x030000ffu;
    v = (v | (v << 8)) & 0x0300f00fu;
    v = (v | (v << 4)) & 0x030c30c3u;
    v = (v | (v << 2)) & 0x09249249u;
    return v;
}

// xs[position] = x[order[position]]: the list kernel then reads its atoms' coordinates without first
// waiting for the order; and the inverse of the order
template <typename T>
__global__ void sorted_coords_kernel(int N, const T* __restrict__ x, const int* __restrict__ order, T* __restrict__ xs,
                                     int* __restrict__ inv)
{
    const int p = blockIdx.x * NBL_BLOCK + threadIdx.x;
    if (p >= N) return;
    const int at = min(max(order[p], 0), N - 1);
    inv[at] = p;                                  // atom -> position: the index the compact entries carry
    xs[(size_t)p * 3 + 0] = x[(size_t)at * 3 + 0];
    xs[(size_t)p * 3 + 1] = x[(size_t)at * 3 + 1];
    xs[(size_t)p * 3 + 2] = x[(size_t)at * 3 + 2];
}

template <typename T>
__global__ void order_keys_kernel(const Grid<T> g_in, const T* __restrict__ x, int shift, unsigned* __restrict__ keys,
                                  int* __restrict__ vals, const GridDyn<T>* __restrict__ gd)
{
    const Grid<T> g = with_dyn(g_in, gd);
    const int p = blockIdx.x * NBL_BLOCK + threadIdx.x;
    if (p >= g.N) return;
    unsigned b[3];
#pragma unroll
    for (int a = 0; a < 3; a++) {
        const int bin = bin_of(x[(size_t)p * 3 + a], g.mn[a], g.bin_size) - g.rlo[a];
        b[a] = (unsigned)min(max(bin, 0), g.rdim[a] - 1) >> shift;
    }
    keys[p] = spread3(b[0]) | (spread3(b[1]) << 1) | (spread3(b[2]) << 2);
    vals[p] = p;
}

// squared distance as the reference forms it: differences in T, squares and sum in double,
// result rounded to T (binLinkedList.h:1008-1012, neighborList.h:318-322)
template <typename T>
__device__ __forceinline__ double dist2_double(T dx, T dy, T dz)
{
    const double a = (double)dx, b = (double)dy, c = (double)dz;
    return __dadd_rn(__dadd_rn(__dmul_rn(a, a), __dmul_rn(b, b)), __dmul_rn(c, c));
}

// row[beg .. end) = v by one wave: single elements up to the first 16-byte boundary, then
// 16-byte stores, then the tail
template <typename V>
__device__ __forceinline__ void pad_fill(V* __restrict__ row, int beg, int end, V v, int lane)
{
    constexpr int PER = 16 / (int)sizeof(V);
    const uintptr_t addr = (uintptr_t)(row + beg);
    int head = (int)(((16 - (addr & 15)) & 15) / sizeof(V));
    head = min(head, end - beg);
    if (lane < head) row[beg + lane] = v;
    const int b0 = beg + head;
    const int nvec = (end - b0) / PER;
    struct alignas(16) Vec { V e[PER]; };
    Vec vv;
#pragma unroll
    for (int i = 0; i < PER; i++) vv.e[i] = v;
    Vec* dst = reinterpret_cast<Vec*>(row + b0);
    for (int i = lane; i < nvec; i += 64) dst[i] = vv;
    const int t0 = b0 + nvec * PER;
    if (t0 + lane < end) row[t0 + lane] = v;
}

// ---- 6. per-atom lists: one wavefront per centre atom ----------------------------------------
// The reference walks the (2e+1)^3 bins around the centre's bin, dx outermost and dz innermost
// (binLinkedList.h:925-927), and appends every atom closer than rcut.  Bins are stored so that
// the dz run of a (dx, dy) column is contiguous: lane c owns column c.  A column, or the ends of
// its dz run, that lies farther from the centre atom than rcut (with a margin for the rounding
// of the binning) cannot contribute and is left out; the order of what remains is unchanged.
// The runs are then laid out back to back as a flat candidate list (in LDS: the column of every
// candidate, one byte each, next to the columns' starts and bases), which the wave scans 64
// candidates at a time; accepted candidates are appended with a ballot prefix.
// With ROWBUF the wave assembles its whole output row (accepted entries, then the -1 / 0 padding)
// in LDS and writes it with 16-byte stores, one full row of firstneigh and one of rcs; this needs
// umax % 4 == 0 and 16-byte aligned outputs.
constexpr int NBL_UNROLL = 4;
constexpr int NBL_ENT_CAP = 256;   // flat candidate list per atom (entries); longer lists search the runs

template <typename T>
inline size_t rowbuf_bytes(int umax, bool rank) { return (size_t)umax * (4 + 3 * sizeof(T) + (rank ? 4 : 0)); }

// Run of supercell entries that column `lane` of the (2e+1)^2 columns around the bin of the atom at
// c can contribute: start index and length (0 for lanes without a column or with nothing in reach).
template <typename T>
__device__ __forceinline__ void column_setup(const Grid<T>& g, const T (&c)[3], int lane,
                                             const int* __restrict__ offsets, int& start, int& len)
{
    int cb[3];
#pragma unroll
    for (int a = 0; a < 3; a++) cb[a] = bin_of(c[a], g.mn[a], g.bin_size);
    const int e = g.ext_bins, side = 2 * e + 1, nruns = side * side;
    start = 0; len = 0;
    if (lane < nruns) {
        const int lq = (int)(((float)lane + 0.5f) * g.inv_side);     // lane / side for small integers
        const int bx = cb[0] + lq - e, by = cb[1] + (lane - lq * side) - e;
        int zlo = cb[2] - e, zhi = cb[2] + e;
        // bins outside the reference's grid are skipped (binLinkedList.h:952-968); inside it the
        // box kept here covers every bin within `e` of a centre atom
        bool ok = bx >= 0 && bx < g.nbin[0] && by >= 0 && by < g.nbin[1] &&
                  bx >= g.rlo[0] && bx < g.rlo[0] + g.rdim[0] && by >= g.rlo[1] &&
                  by < g.rlo[1] + g.rdim[1];
        zlo = max(zlo, max(0, g.rlo[2]));
        zhi = min(zhi, min(g.nbin[2] - 1, g.rlo[2] + g.rdim[2] - 1));
        // geometric pruning (float is enough: the margin dwarfs its rounding): distance from the
        // atom to the column's rectangle in x and y, then the reach left for z
        {
            const float bs = (float)g.bin_size, inv_bs = g.inv_bin, rc2 = (float)g.rcut2 * 1.00001f;
            float lat2 = 0.0f;
            const int bxy[2] = {bx, by};
#pragma unroll
            for (int a = 0; a < 2; a++) {
                const float rel = (float)c[a] - (float)g.mn[a];
                const float tol = 1.0e-3f * bs + 1.0e-5f * (fabsf(rel) + fabsf((float)c[a]) + fabsf((float)g.mn[a]));
                const float lo = (float)bxy[a] * bs;
                const float d = fmaxf(fmaxf(lo - rel, rel - (lo + bs)) - tol, 0.0f);
                lat2 += d * d;
            }
            if (lat2 > rc2) ok = false;
            else {
                const float rel = (float)c[2] - (float)g.mn[2];
                const float tol = 1.0e-3f * bs + 1.0e-5f * (fabsf(rel) + fabsf((float)c[2]) + fabsf((float)g.mn[2]));
                // the hardware square root is within an ulp; the tolerance is five orders above that
                const float reach = __builtin_amdgcn_sqrtf(rc2 - lat2) + tol;
                zlo = max(zlo, (int)floorf((rel - reach) * inv_bs - 1.0e-3f));
                zhi = min(zhi, (int)floorf((rel + reach) * inv_bs + 1.0e-3f));
            }
        }
        if (ok && zlo <= zhi) {
            const int col = ((bx - g.rlo[0]) * g.rdim[1] + (by - g.rlo[1])) * g.rdim[2] - g.rlo[2];
            start = offsets[col + zlo];
            len = offsets[col + zhi + 1] - start;
        }
    }
}

constexpr int NBL_APW = 2;         // consecutive centre atoms per wavefront

// Compact lists (compact_list.h) written next to, or instead of, the padded rows.  The wavefront
// that holds a finished row in LDS sorts its entries into the two ends of the position's slots:
// beyond `split` (and within `outer`) from slot 0 upwards, within `split` from slot umax-1 downwards.
template <typename T>
struct CompactEmit {
    const int* order;   // position -> atom
    const T* xs;        // [natoms][3] Cartesian coordinates in processing order
    const int* inv;     // [natoms] atom -> position (for an order that is no permutation: leftovers in places)
    T* entries;
    int* n_outer;
    int* n_inner;
    int nch;
    T split2, outer2;   // squares of the two cutoffs
    T near_band;        // |d^2 - split2| within which the two ends of a pair may disagree about the side
    int write_rows;     // the padded outputs are wanted as well
};
// set in n_inner of a position that has an entry close to the inner cutoff, between the list kernel and
// compact_symmetry_kernel, which clears it
constexpr int CL_NEAR_FLAG = 1 << 30;

// Squared length of the vector from the atom at c to the image of atom j it sees at c + d, formed so that the two
// ends of a pair get the same bits: the difference of the two atoms' own coordinates (which changes sign exactly
// when the ends are swapped) plus the lattice shift of the image (rebuilt from its indices, which also only
// change sign).  The list's own vector d = image - c does not have this property: the image is rounded at the size
// of the coordinates, differently for the two ends.  Used to put both entries of a pair on the same side of the
// inner cutoff of the compact lists.
template <typename T>
__device__ T pair_symmetric_d2(const Grid<T>& g, const T* __restrict__ x, const T (&c)[3], T dx, T dy, T dz, int j)
{
    const T d[3] = {dx, dy, dz};
    T e[3], v[3];
    j = min(max(j, 0), g.N - 1);                     // positions come from the inverse of a caller-writable order
#pragma unroll
    for (int a = 0; a < 3; a++) {
        e[a] = sub_rn(x[(size_t)j * 3 + a], c[a]);
        v[a] = d[a] - e[a];                       // the image's shift, up to rounding
    }
    auto shift = [&](int ii, int jj, int kk, T (&s)[3]) __attribute__((always_inline)) {
#pragma unroll
        for (int a = 0; a < 3; a++)
            s[a] = add_rn(add_rn(mul_rn(g.b[0][a], (T)ii), mul_rn(g.b[1][a], (T)jj)), mul_rn(g.b[2][a], (T)kk));
    };
    T best = (T)INFINITY;
    int bi = 0, bj = 0, bk = 0;
    for (int ii = g.img_lo[0]; ii < g.img_lo[0] + g.img_dim[0]; ii++)
        for (int jj = g.img_lo[1]; jj < g.img_lo[1] + g.img_dim[1]; jj++)
            for (int kk = g.img_lo[2]; kk < g.img_lo[2] + g.img_dim[2]; kk++) {
                T s[3];
                shift(ii, jj, kk, s);
                const T q = (v[0] - s[0]) * (v[0] - s[0]) + (v[1] - s[1]) * (v[1] - s[1]) + (v[2] - s[2]) * (v[2] - s[2]);
                if (q < best) { best = q; bi = ii; bj = jj; bk = kk; }
            }
    T s[3];
    shift(bi, bj, bk, s);
    const T w0 = add_rn(e[0], s[0]), w1 = add_rn(e[1], s[1]), w2 = add_rn(e[2], s[2]);
    return add_rn(add_rn(mul_rn(w0, w0), mul_rn(w1, w1)), mul_rn(w2, w2));
}

template <typename T, bool SORT, bool ROWBUF, bool RANK, bool COMPACT = false>
__global__ void __launch_bounds__(NBL_BLOCK)
lists_kernel(const Grid<T> g_in, const T* __restrict__ x, const int* __restrict__ types,
             const int* __restrict__ offsets, const T* __restrict__ s_rec,
             int umax, int* __restrict__ ilist, int* __restrict__ numneigh, int* __restrict__ firstneigh,
             T* __restrict__ rcs, int* __restrict__ types_out, T* __restrict__ keys,
             int* __restrict__ status, int update, int* __restrict__ rank_out, int* __restrict__ incoming,
             const CompactEmit<T> ce, const GridDyn<T>* __restrict__ gd)
{
    static_assert(!COMPACT || (ROWBUF && !SORT && !RANK), "compact lists are cut from the row held in LDS");
    const Grid<T> g = with_dyn(g_in, gd);
    __shared__ int sh_start[NBL_BLOCK / 64][64];
    __shared__ int sh_base[NBL_BLOCK / 64][64];
    __shared__ unsigned char sh_col[NBL_BLOCK / 64][NBL_APW][NBL_ENT_CAP];   // column of each flat candidate
    extern __shared__ __align__(16) unsigned char sh_rows[];
    const int wv = threadIdx.x >> 6, lane = threadIdx.x & 63;
    // the wave's first position, in a scalar register: the loads of its atoms' indices and coordinates are then
    // scalar loads
    const int p0 = __builtin_amdgcn_readfirstlane((blockIdx.x * (NBL_BLOCK / 64) + wv) * NBL_APW);
    if (p0 >= g.N) return;                        // whole wave leaves together
    const int np = min(NBL_APW, g.N - p0);
    T* rb_rcs = nullptr;
    int* rb_first = nullptr;
    int* rb_rank = nullptr;
    if (ROWBUF) {
        unsigned char* mine = sh_rows + (size_t)wv * umax * (4 + 3 * sizeof(T) + (RANK ? 4 : 0));
        rb_rcs = (T*)mine;
        rb_first = (int*)(mine + (size_t)umax * 3 * sizeof(T));
        rb_rank = rb_first + umax;
    }
    // A row costs three dependent trips to memory (coordinates, column runs, candidates).  The
    // wavefront takes NBL_APW atoms: all their coordinates are loaded first, and the column runs of
    // the next atom are requested before the candidates of the current one are scanned.
    T cs[NBL_APW][3];
    int atom[NBL_APW];                            // the atom behind each of the wave's positions
#pragma unroll
    for (int a = 0; a < NBL_APW; a++) {
        const int q = min(p0 + a, g.N - 1);
        // the caller may write the order: an index outside the structure must not reach an address
        // (compact_symmetry_kernel reports it)
        atom[a] = COMPACT ? min(max(ce.order[q], 0), g.N - 1) : q;
    }
#pragma unroll
    for (int a = 0; a < NBL_APW; a++)
#pragma unroll
        for (int d = 0; d < 3; d++)
            cs[a][d] = COMPACT ? ce.xs[(size_t)min(p0 + a, g.N - 1) * 3 + d] : x[(size_t)atom[a] * 3 + d];
    const int nruns = (2 * g.ext_bins + 1) * (2 * g.ext_bins + 1);
    // With at most 32 columns per atom the wave's two atoms are set up side by side, lanes 0-31 and 32-63 (their
    // halves of sh_start / sh_base, their own flat list); with more, one after the other through the first
    // flat list, the column runs of the second requested before the candidates of the first are scanned.
    static_assert(NBL_APW == 2, "two atoms per wavefront");
    const bool paired = nruns <= 32;              // wave-uniform
    int start, len;
    int totals[NBL_APW] = {0, 0};
    if (paired) {
        const int sub = lane >> 5;
        const T csel[3] = {sub ? cs[1][0] : cs[0][0], sub ? cs[1][1] : cs[0][1], sub ? cs[1][2] : cs[0][2]};
        column_setup<T>(g, csel, lane & 31, offsets, start, len);
        if (sub >= np) len = 0;
        const int incl = wave_inclusive_scan(len);
        totals[0] = __shfl(incl, 31, 64);
        totals[1] = __shfl(incl, 63, 64) - totals[0];
        const int base = incl - len - (sub ? totals[0] : 0);
        sh_start[wv][lane] = start;
        sh_base[wv][lane] = base;
        if ((sub ? totals[1] : totals[0]) <= NBL_ENT_CAP)
            for (int k = 0; k < len; k++) sh_col[wv][sub][base + k] = (unsigned char)(lane & 31);
        __builtin_amdgcn_wave_barrier();
    } else {
        column_setup<T>(g, cs[0], lane, offsets, start, len);
    }
    const T near_band = ce.near_band;
#pragma unroll
    for (int ia = 0; ia < NBL_APW; ia++) {
    if (ia >= np) break;                          // wave-uniform
    const int pos = p0 + ia;                      // position in processing order
    const int p = atom[ia];                       // atom, row of the padded outputs
    const bool rows = !COMPACT || ce.write_rows;  // wave-uniform
    const T (&c)[3] = cs[ia];
    int nstart = 0, nlen = 0;
    if (!paired) {
        if (ia + 1 < NBL_APW && ia + 1 < np) column_setup<T>(g, cs[ia + 1 < NBL_APW ? ia + 1 : ia], lane, offsets, nstart, nlen);
        const int incl = wave_inclusive_scan(len);
        totals[ia] = __shfl(incl, 63, 64);
        const int base = incl - len;
        sh_start[wv][lane] = start;
        sh_base[wv][lane] = base;
        if (totals[ia] <= NBL_ENT_CAP)
            for (int k = 0; k < len; k++) sh_col[wv][0][base + k] = (unsigned char)lane;
        __builtin_amdgcn_wave_barrier();
    }
    const int total = totals[ia];
    const bool flat = total <= NBL_ENT_CAP;       // wave-uniform
    const int so = paired ? ia * 32 : 0;          // the atom's part of sh_start / sh_base
    const unsigned char* const cols = sh_col[wv][paired ? ia : 0];

    int cnt = 0;
    const size_t rowi = (size_t)p * umax;
    // update of an earlier result held in the same buffers: beyond the row's old length the
    // padding is already in place
    const int old_len = (update && rows) ? min(max(numneigh[p], 0), umax) : umax;
    // NBL_UNROLL chunks of 64 candidates per trip: all their loads are issued before the first is
    // used, so a typical row (100 - 250 candidates) costs one memory round trip
    for (int c0 = 0; c0 < total; c0 += 64 * NBL_UNROLL) {
        int sj[NBL_UNROLL];
        T px[NBL_UNROLL], py[NBL_UNROLL], pz[NBL_UNROLL];
#pragma unroll
        for (int u = 0; u < NBL_UNROLL; u++) {
            // no branch around the load: a lane past the end of the list reads the last candidate again and
            // drops it below, and the loads of the trip's chunks stay back to back
            const int ci = min(c0 + u * 64 + lane, total - 1);
            int ent;
            if (flat) {
                const int col = so + cols[ci];
                ent = sh_start[wv][col] + (ci - sh_base[wv][col]);
            } else {
                // last column whose base is <= ci
                int lo = 0, hi = nruns - 1;
                while (lo < hi) {
                    const int mid = (lo + hi + 1) >> 1;
                    if (sh_base[wv][so + mid] <= ci) lo = mid; else hi = mid - 1;
                }
                ent = sh_start[wv][so + lo] + (ci - sh_base[wv][so + lo]);
            }
            entry_load(s_rec + (size_t)ent * 4, px[u], py[u], pz[u], sj[u]);
        }
        // RANK: the pair's place among the pairs that name the same neighbour, claimed here so that
        // the force kernels need no atomics; the answers are collected after the chunk's last claim
        int rk[NBL_UNROLL], rs[NBL_UNROLL];
#pragma unroll
        for (int u = 0; u < NBL_UNROLL; u++) rs[u] = -1;
#pragma unroll
        for (int u = 0; u < NBL_UNROLL; u++) {
            if (c0 + u * 64 >= total) break;                           // wave-uniform
            const bool have = c0 + u * 64 + lane < total;
            const T dx = sub_rn(px[u], c[0]), dy = sub_rn(py[u], c[1]), dz = sub_rn(pz[u], c[2]);
            const double d2d = dist2_double(dx, dy, dz);
            const T d2 = (T)d2d;                                       // `CoordType relative_distance2`
            const bool in = have && ((double)d2 < g.rcut2) && ((double)d2 > kEpsilon);   // binLinkedList.h:1014-1017
            const unsigned long long mask = __ballot(in);
            const int rank = __popcll(mask & ((1ull << lane) - 1ull));
            const int slot = cnt + rank;
            if (in && slot < umax) {
                if (ROWBUF) {
                    rb_first[slot] = sj[u];
                    rb_rcs[slot * 3 + 0] = dx;
                    rb_rcs[slot * 3 + 1] = dy;
                    rb_rcs[slot * 3 + 2] = dz;
                } else {
                    firstneigh[rowi + slot] = sj[u];                   // neighborList.h:561 (already mod natoms)
                    rcs[(rowi + slot) * 3 + 0] = dx;
                    rcs[(rowi + slot) * 3 + 1] = dy;
                    rcs[(rowi + slot) * 3 + 2] = dz;
                }
                if (SORT) keys[rowi + slot] = (T)__dsqrt_rn(d2d);      // neighborList.h:318-322
                if (RANK) {
                    rk[u] = atomicAdd(&incoming[sj[u]], 1);
                    rs[u] = slot;
                }
            }
            cnt += __popcll(mask);
        }
        if (RANK) {
#pragma unroll
            for (int u = 0; u < NBL_UNROLL; u++)
                if (rs[u] >= 0) {
                    if (ROWBUF) rb_rank[rs[u]] = rk[u];
                    else rank_out[rowi + rs[u]] = rk[u];
                }
        }
    }
    if (lane == 0) {
        if (rows) numneigh[p] = cnt;             // ilist and types_out: count_kernel
        if (cnt > umax) atomicOr(status, ST_NEIGH_OVERFLOW);
    }
    // the first 64 entries of the row: their compact stores wait until the padded row has gone out (below)
    T first_dx = (T)0, first_dy = (T)0, first_dz = (T)0;
    int first_bits = 0, first_slot = -1;
    T* compact_base = nullptr;
    if (COMPACT) {
        // the row's entries, 64 at a time: class by distance, place by ballot prefix, one 16-byte
        // (fp32) store per entry; 8 consecutive slots of a position are contiguous in memory
        __builtin_amdgcn_wave_barrier();
        const int used = min(cnt, umax);
        int n_outer = 0, n_inner = 0;
        T nearest = (T)INFINITY;                  // |d^2 - split^2| of the lane's entry closest to the inner cutoff
        // slot e of this position sits at  base + (e / 8) * (64 * 8 * 4) + (e % 8) * 4  values
        T* const base = ce.entries + compact_slot_offset(ce.nch, __builtin_amdgcn_readfirstlane(pos), 0);
        compact_base = base;
        for (int e0 = 0; e0 < used; e0 += 64) {
            const int e = e0 + lane;
            const bool have = e < used;
            const int ee = have ? e : 0;
            const T dx = rb_rcs[ee * 3 + 0], dy = rb_rcs[ee * 3 + 1], dz = rb_rcs[ee * 3 + 2];
            const int word = rb_first[ee];
            // The entry names its neighbour by position in the processing order (what the force kernels index their
            // per-atom arrays with), the record and the padded row by atom: one gather per entry.  The first 64
            // entries (most rows have no more) do not wait for the answer here: they are stored after the padded
            // row.  A value of the inverse is a valid position unless the order is no permutation, which
            // compact_symmetry_kernel reports; the consumers of the entries check the index they find.
            const int bits = ce.inv[word & (CL_IMAGE_BIT - 1)] | (word & ~CL_INDEX_MASK);
            const T d2 = dx * dx + dy * dy + dz * dz;
            const bool in_outer = have && d2 <= ce.outer2;
            const bool is_inner = in_outer && d2 <= ce.split2;
            // Both entries of a pair must fall on the same side of the inner cutoff (the force kernels treat the
            // two classes by different routes), but the two ends see vectors that differ by the rounding of their
            // images (a pair of atoms in the cell itself has exactly opposite vectors).  A position with an image
            // inside a band around the cutoff several times wider than that rounding is flagged for
            // compact_symmetry_kernel, which settles such entries by a squared distance both ends form
            // bit-identically; outside the band the two ends agree anyway.
            nearest = fmin(nearest, (in_outer && (word & CL_IMAGE_BIT)) ? fabs(d2 - ce.split2) : nearest);
            const bool is_outer = in_outer && !is_inner;
            const unsigned long long mi = __ballot(is_inner), mo = __ballot(is_outer);
            const unsigned long long below = (1ull << lane) - 1ull;
            int slot = -1;
            if (is_inner) slot = umax - 1 - (n_inner + __popcll(mi & below));
            if (is_outer) slot = n_outer + __popcll(mo & below);
            if (e0 == 0) {                        // wave-uniform
                first_dx = dx; first_dy = dy; first_dz = dz; first_bits = bits; first_slot = slot;
            } else if (slot >= 0) {
                entry_store_stream<T>(base + (((unsigned)slot >> 3) << 11) + (((unsigned)slot & 7u) << 2), dx, dy, dz, bits);
            }
            n_inner += __popcll(mi);
            n_outer += __popcll(mo);
        }
        const bool any_near = __ballot(nearest <= near_band) != 0ull;
        if (lane == 0) {
            ce.n_outer[pos] = n_outer;
            ce.n_inner[pos] = n_inner | (any_near ? CL_NEAR_FLAG : 0);         // the flag: for compact_symmetry_kernel
        }
        // the padded row lists plain indices
        if (rows)
            for (int e = lane; e < used; e += 64) rb_first[e] &= CL_IMAGE_BIT - 1;
    }
    if (ROWBUF && rows) {
        __builtin_amdgcn_wave_barrier();
        const uint4* s1 = reinterpret_cast<const uint4*>(rb_first);
        uint4* d1 = reinterpret_cast<uint4*>(firstneigh + rowi);
        const int used = min(cnt, umax);
        const int live = (max(used, old_len) + 3) & ~3;               // umax is a multiple of 4
        for (int i = used + lane; i < live; i += 64) {                 // padding, neighborList.h:557, 563
            rb_first[i] = -1;
            rb_rcs[i * 3 + 0] = (T)0; rb_rcs[i * 3 + 1] = (T)0; rb_rcs[i * 3 + 2] = (T)0;
        }
        __builtin_amdgcn_wave_barrier();
        typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));    // non-temporal, as the compact entries
        for (int i = lane; i < live / 4; i += 64) __builtin_nontemporal_store(*reinterpret_cast<const u32x4*>(&s1[i]), reinterpret_cast<u32x4*>(&d1[i]));
        const uint4* s2 = reinterpret_cast<const uint4*>(rb_rcs);
        uint4* d2 = reinterpret_cast<uint4*>(rcs + rowi * 3);
        const int nv = (int)((size_t)live * 3 * sizeof(T) / 16);
        for (int i = lane; i < nv; i += 64) __builtin_nontemporal_store(*reinterpret_cast<const u32x4*>(&s2[i]), reinterpret_cast<u32x4*>(&d2[i]));
        if (RANK) {                                                    // slots past the row's end are not defined
            const uint4* s3 = reinterpret_cast<const uint4*>(rb_rank);
            uint4* d3 = reinterpret_cast<uint4*>(rank_out + rowi);
            for (int i = lane; i < (used + 3) / 4; i += 64) d3[i] = s3[i];
        }
    } else if (!ROWBUF) {
        // padding: -1 / 0 (neighborList.h:557, 563)
        const int first_pad = min(cnt, umax);
        const int last_pad = max(first_pad, old_len);
        pad_fill(firstneigh + rowi, first_pad, last_pad, -1, lane);
        pad_fill(rcs + rowi * 3, first_pad * 3, last_pad * 3, (T)0, lane);
    }
    if (COMPACT && first_slot >= 0)
        entry_store_stream<T>(compact_base + (((unsigned)first_slot >> 3) << 11) + (((unsigned)first_slot & 7u) << 2), first_dx,
                       first_dy, first_dz, first_bits);
    start = nstart;
    len = nlen;
    __builtin_amdgcn_wave_barrier();              // the LDS arrays are reused by the next atom
    }
}

// ---- 6b. compact lists: both entries of a pair on the same side of the inner cutoff ---------------------
// A wavefront looks at the flags of 64 positions and works through the flagged ones, one at a time.  It reads
// such a position's entries 64 at a time, first the class beyond the cutoff, then the class inside; an entry
// within the band takes the side its symmetric squared distance gives; entries that stay are written back in
// order (compacting in place: a write never passes the reads of its own trip), entries that change sides wait
// in LDS and are appended to their new class at the end.
template <typename T>
__global__ void __launch_bounds__(NBL_BLOCK)
compact_symmetry_kernel(const Grid<T> g_in, const GridDyn<T>* __restrict__ gd, const T* __restrict__ x,
                        const CompactEmit<T> ce, int umax, int* __restrict__ status)
{
    extern __shared__ __align__(16) unsigned char sh_move[];     // per wave: umax entries of 4 values
    const Grid<T> g = with_dyn(g_in, gd);
    const int wv = threadIdx.x >> 6, lane = threadIdx.x & 63;
    T* const mv = (T*)sh_move + (size_t)wv * umax * 4;
    const int p0 = (blockIdx.x * (NBL_BLOCK / 64) + wv) * 64;
    const int mine = p0 + lane < g.N ? ce.n_inner[p0 + lane] : 0;
    // The processing order must name every atom once: an index outside the structure (clamped where it is used) or
    // an atom named twice (then some atom has no row, and the inverse of the order holds leftovers) is reported.
    if (p0 + lane < g.N) {
        const int at = ce.order[p0 + lane];
        if ((unsigned)at >= (unsigned)g.N || ce.inv[at] != p0 + lane) atomicOr(status, ST_BAD_NEIGHBOR);
    }
    unsigned long long todo = __ballot((mine & CL_NEAR_FLAG) != 0);
    if (todo == 0ull) return;                     // whole wave
    const T band = ce.near_band;
    const unsigned long long below = (1ull << lane) - 1ull;
    for (; todo != 0ull; todo &= todo - 1ull) {
        const int pos = p0 + __builtin_ctzll(todo);
        const T c[3] = {ce.xs[(size_t)pos * 3], ce.xs[(size_t)pos * 3 + 1], ce.xs[(size_t)pos * 3 + 2]};
        const int n_outer = ce.n_outer[pos], n_inner = ce.n_inner[pos] & ~CL_NEAR_FLAG;
        T* const base = ce.entries + compact_slot_offset(ce.nch, pos, 0);
        auto slot = [&](int e) __attribute__((always_inline)) {
            return base + (((unsigned)e >> 3) << 11) + (((unsigned)e & 7u) << 2);
        };
        int kept[2] = {0, 0}, moved[2] = {0, 0};   // by the class an entry came from: 0 beyond the cutoff, 1 inside
        // entries that change sides: those from beyond the cutoff from the front of mv, the others from its back
#pragma unroll
        for (int cls = 0; cls < 2; cls++) {
            const int count = cls ? n_inner : n_outer;
            for (int e0 = 0; e0 < count; e0 += 64) {
                const int e = e0 + lane;
                const bool have = e < count;
                T dx = (T)0, dy = (T)0, dz = (T)0;
                int bits = 0;
                if (have) entry_load(slot(cls ? umax - 1 - e : e), dx, dy, dz, bits);
                const T d2 = dx * dx + dy * dy + dz * dz;
                bool inside = cls != 0;
                if (have && fabs(d2 - ce.split2) <= band)
                    inside = pair_symmetric_d2<T>(g, ce.xs, c, dx, dy, dz, bits & CL_INDEX_MASK) <= ce.split2;
                const bool stay = have && inside == (cls != 0), go = have && !stay;
                const unsigned long long ms = __ballot(stay), mg = __ballot(go);
                if (stay) {
                    const int k = kept[cls] + __popcll(ms & below);
                    entry_store<T>(slot(cls ? umax - 1 - k : k), dx, dy, dz, bits);
                }
                if (go) {
                    const int k = moved[cls] + __popcll(mg & below);
                    entry_store<T>(mv + (size_t)(cls ? umax - 1 - k : k) * 4, dx, dy, dz, bits);
                }
                kept[cls] += __popcll(ms);
                moved[cls] += __popcll(mg);
            }
        }
        __builtin_amdgcn_wave_barrier();
        // entries that came from beyond the cutoff join the class inside, and the other way round
        for (int k = lane; k < moved[0]; k += 64) {
            T dx, dy, dz;
            int bits;
            entry_load(mv + (size_t)k * 4, dx, dy, dz, bits);
            entry_store<T>(slot(umax - 1 - (kept[1] + k)), dx, dy, dz, bits);
        }
        for (int k = lane; k < moved[1]; k += 64) {
            T dx, dy, dz;
            int bits;
            entry_load(mv + (size_t)(umax - 1 - k) * 4, dx, dy, dz, bits);
            entry_store<T>(slot(kept[0] + k), dx, dy, dz, bits);
        }
        if (lane == 0) {
            ce.n_outer[pos] = kept[0] + moved[1];
            ce.n_inner[pos] = kept[1] + moved[0];
        }
        __builtin_amdgcn_wave_barrier();          // mv is reused by the wave's next position
    }
}

// ---- 7. distance sort, emulating libstdc++ std::sort(indices, cmp = d[a] < d[b]) --------------
// Introsort: median-of-three quicksort down to partitions of 16, heap sort beyond depth
// 2*floor(log2 n), then one insertion sort pass.  Only the sequence of comparisons and moves
// decides where equal keys end up, so the published algorithm is followed step by step.
template <typename T>
struct IdxSorter {
    int* v;          // index array being sorted
    const T* d;      // keys
    __device__ bool less(int a, int b) const { return d[a] < d[b]; }
    __device__ void iter_swap(int i, int j) { int t = v[i]; v[i] = v[j]; v[j] = t; }

    __device__ void move_median_to_first(int result, int a, int b, int c)
    {
        if (less(v[a], v[b])) {
            if (less(v[b], v[c])) iter_swap(result, b);
            else if (less(v[a], v[c])) iter_swap(result, c);
            else iter_swap(result, a);
        } else if (less(v[a], v[c])) iter_swap(result, a);
        else if (less(v[b], v[c])) iter_swap(result, c);
        else iter_swap(result, b);
    }
    __device__ int unguarded_partition(int first, int last, int pivot)
    {
        while (true) {
            while (less(v[first], v[pivot])) ++first;
            --last;
            while (less(v[pivot], v[last])) --last;
            if (!(first < last)) return first;
            iter_swap(first, last);
            ++first;
        }
    }
    __device__ void push_heap(int first, int hole, int top, int value)
    {
        int parent = (hole - 1) / 2;
        while (hole > top && less(v[first + parent], value)) {
            v[first + hole] = v[first + parent];
            hole = parent;
            parent = (hole - 1) / 2;
        }
        v[first + hole] = value;
    }
    __device__ void adjust_heap(int first, int hole, int len, int value)
    {
        const int top = hole;
        int child = hole;
        while (child < (len - 1) / 2) {
            child = 2 * (child + 1);
            if (less(v[first + child], v[first + (child - 1)])) child--;
            v[first + hole] = v[first + child];
            hole = child;
        }
        if ((len & 1) == 0 && child == (len - 2) / 2) {
            child = 2 * (child + 1);
            v[first + hole] = v[first + (child - 1)];
            hole = child - 1;
        }
        push_heap(first, hole, top, value);
    }
    __device__ void heap_sort(int first, int last)      // __partial_sort(first, last, last)
    {
        const int len = last - first;
        if (len >= 2) {                                  // __make_heap
            int parent = (len - 2) / 2;
            while (true) {
                int value = v[first + parent];
                adjust_heap(first, parent, len, value);
                if (parent == 0) break;
                parent--;
            }
        }
        while (last - first > 1) {                       // __sort_heap / __pop_heap
            --last;
            int value = v[last];
            v[last] = v[first];
            adjust_heap(first, 0, last - first, value);
        }
    }
    __device__ void unguarded_linear_insert(int last)
    {
        int val = v[last];
        int next = last - 1;
        while (less(val, v[next])) {
            v[last] = v[next];
            last = next;
            --next;
        }
        v[last] = val;
    }
    __device__ void insertion_sort(int first, int last)
    {
        if (first == last) return;
        for (int i = first + 1; i != last; ++i) {
            if (less(v[i], v[first])) {
                int val = v[i];
                for (int k = i; k > first; --k) v[k] = v[k - 1];   // move_backward
                v[first] = val;
            } else unguarded_linear_insert(i);
        }
    }
    __device__ void sort(int n)
    {
        if (n <= 1) return;
        int depth = 2 * (31 - __clz(n));
        // __introsort_loop, recursion on the right part turned into an explicit stack
        int stack_first[64], stack_last[64], stack_depth[64];
        int sp = 0;
        int first = 0, last = n;
        while (true) {
            while (last - first > 16) {
                if (depth == 0) { heap_sort(first, last); break; }
                --depth;
                const int mid = first + (last - first) / 2;
                move_median_to_first(first, first + 1, mid, last - 1);
                const int cut = unguarded_partition(first + 1, last, first);
                // the reference recurses into [cut, last) first, then continues with [first, cut)
                stack_first[sp] = first; stack_last[sp] = cut; stack_depth[sp] = depth; sp++;
                first = cut;
            }
            if (sp == 0) break;
            sp--;
            first = stack_first[sp]; last = stack_last[sp]; depth = stack_depth[sp];
        }
        if (n > 16) {                                    // __final_insertion_sort
            insertion_sort(0, 16);
            for (int i = 16; i < n; ++i) unguarded_linear_insert(i);
        } else insertion_sort(0, n);
    }
};

template <typename T>
__global__ void sort_rows_kernel(int N, int umax, const int* __restrict__ numneigh,
                                 const T* __restrict__ keys, int* __restrict__ order)
{
    const int p = blockIdx.x * 64 + threadIdx.x;
    if (p >= N) return;
    const int n = min(numneigh[p], umax);
    int* v = order + (size_t)p * umax;
    for (int j = 0; j < n; j++) v[j] = j;
    IdxSorter<T> s{v, keys + (size_t)p * umax};
    s.sort(n);
}

// out row = tmp row gathered through `order` (SingleNeighborListArrangement, neighborList.h:46-67)
template <typename T>
__global__ void gather_rows_kernel(int N, int umax, const int* __restrict__ numneigh,
                                   const int* __restrict__ order, const int* __restrict__ tmp_first,
                                   const T* __restrict__ tmp_rcs, int* __restrict__ firstneigh,
                                   T* __restrict__ rcs)
{
    const int p = (blockIdx.x * NBL_BLOCK + threadIdx.x) >> 6, lane = threadIdx.x & 63;
    if (p >= N) return;
    const int n = min(numneigh[p], umax);
    const size_t row = (size_t)p * umax;
    for (int s = lane; s < umax; s += 64) {
        if (s < n) {
            const int src = order[row + s];
            firstneigh[row + s] = tmp_first[row + src];
            rcs[(row + s) * 3 + 0] = tmp_rcs[(row + src) * 3 + 0];
            rcs[(row + s) * 3 + 1] = tmp_rcs[(row + src) * 3 + 1];
            rcs[(row + s) * 3 + 2] = tmp_rcs[(row + src) * 3 + 2];
        } else {
            firstneigh[row + s] = -1;
            rcs[(row + s) * 3 + 0] = (T)0;
            rcs[(row + s) * 3 + 1] = (T)0;
            rcs[(row + s) * 3 + 2] = (T)0;
        }
    }
}

__global__ void int_max_kernel(const int* __restrict__ v, int n, int* __restrict__ out)
{
    __shared__ int sh[4];
    int m = 0;
    for (int i = blockIdx.x * 256 + threadIdx.x; i < n; i += gridDim.x * 256) m = max(m, v[i]);
    m = wave_max(m);
    if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) atomicMax(out, max(max(sh[0], sh[1]), max(sh[2], sh[3])));
}

// ---- host ------------------------------------------------------------------------------------
template <typename T>
void host_cross(const T* a, const T* b, T* o)        // source/core/include/vec3Operation.h:87-93
{
    o[0] = a[1] * b[2] - a[2] * b[1];
    o[1] = a[2] * b[0] - a[0] * b[2];
    o[2] = a[0] * b[1] - a[1] * b[0];
}

template <typename T>
T host_plane_distance(const T* v, const T* n)        // structure.h:818-842, vec3Operation.h:97-104
{
    // squares and their sum in double, square root rounded to T, division and dot product in T
    T len = (T)std::sqrt((double)n[0] * (double)n[0] + (double)n[1] * (double)n[1] +
                         (double)n[2] * (double)n[2]);
    T u[3] = {(T)(n[0] / len), (T)(n[1] / len), (T)(n[2] / len)};
    T d = v[0] * u[0] + v[1] * u[1] + v[2] * u[2];
    return std::abs(d);
}

// compact lists wanted from a build: the caller's buffer (compact_list.h) and the two cutoffs
struct CompactOut {
    void* buffer;
    double split, outer;
    int keep_order;    // the buffer already holds a processing order from an earlier build: use it
};

// ---- builds that do not read the extents back (a2p_nblist_sync_free) -----------------------------------
// The synchronised build remembers, per host thread, the bin box it found for a structure (device, natoms, lattice,
// cutoff, periodicity).  With the switch on, a later build of the same structure sizes its launches and scratch
// arrays for that box plus a margin, derives the actual box on the device (grid_setup_kernel) and never waits
// for the stream; a box that outgrows the bound empties the lists and raises ST_GRID_BOUND.
struct GridBound {
    bool valid = false;
    int device = -1, N = 0, is_cart = 0, pbc[3] = {0, 0, 0};
    double lattice[9] = {0, 0, 0, 0, 0, 0, 0, 0, 0}, rcut = 0;
    int rdim[3] = {0, 0, 0};
    double big = 0;    // largest |coordinate| of the box kept by that build
};
// a few structures per host thread (two calculators used in turn keep both of their bounds), oldest replaced first
constexpr size_t kMaxBounds = 8;
thread_local std::vector<GridBound> g_bounds;
thread_local int g_sync_free = 0;

template <typename T>
int nblist_build(const T* lattice, const int* types, const T* coords, int N, double rcut_in, int umax,
                 int is_cart, const int* pbc, int sort, int* ilist, int* numneigh, int* firstneigh,
                 T* rcs, int* types_out, int* max_nn_host, hipStream_t stream, int update = 0,
                 int* rank = nullptr, int* incoming = nullptr, const CompactOut* co = nullptr)
{
    const bool want_rows = !co || (ilist || numneigh || firstneigh || rcs || types_out);
    if (co) {
        A2P_REQUIRE(co->buffer, A2P_ERR_INVALID, "nblist: null compact-list buffer");
        A2P_REQUIRE(!sort && !rank, A2P_ERR_INVALID, "nblist: compact lists come with unsorted rows and without places");
        A2P_REQUIRE(compact_supported(N, umax), A2P_ERR_INVALID,
                    "nblist: compact lists need umax %% 8 == 0 and fewer than 2^28 atoms (natoms %d, umax %d)", N, umax);
        A2P_REQUIRE(co->split > 0 && co->outer >= co->split, A2P_ERR_INVALID, "nblist: bad cutoffs for the compact lists");
        A2P_REQUIRE(rowbuf_bytes<T>(umax, false) * (NBL_BLOCK / 64) <= 32 * 1024, A2P_ERR_INVALID,
                    "nblist: umax %d too large for compact lists", umax);
        A2P_REQUIRE(!want_rows || ((uintptr_t)firstneigh % 16 == 0 && (uintptr_t)rcs % 16 == 0), A2P_ERR_INVALID,
                    "nblist: firstneigh and rcs must be 16-byte aligned");
    }
    A2P_REQUIRE((rank == nullptr) == (incoming == nullptr), A2P_ERR_INVALID,
                "nblist: rank and incoming come together");
    A2P_REQUIRE(!(rank && sort), A2P_ERR_INVALID, "nblist: places of the pairs are produced for unsorted rows only");
    A2P_REQUIRE(lattice && pbc, A2P_ERR_INVALID, "nblist: lattice and pbc must be host pointers");
    A2P_REQUIRE(N > 0, A2P_ERR_INVALID, "nblist: the structure has no atoms");   // binLinkedList.h:659
    A2P_REQUIRE(umax > 0 && rcut_in > 0, A2P_ERR_INVALID, "nblist: rcut and umax must be positive");
    A2P_REQUIRE(types && coords, A2P_ERR_INVALID, "nblist: null device pointer");
    A2P_REQUIRE(!want_rows || (ilist && numneigh && firstneigh && rcs && types_out), A2P_ERR_INVALID,
                "nblist: null device pointer (the padded outputs come all or none)");
    A2P_REQUIRE(want_rows || !max_nn_host, A2P_ERR_INVALID, "nblist: the largest neighbour count needs the padded outputs");
    A2P_REQUIRE((long long)N * umax < (1ll << 31), A2P_ERR_INVALID, "nblist: natoms*umax exceeds 2^31");

    Grid<T> g;
    g.N = N;
    g.is_cart = is_cart;
    g.rcut = (T)rcut_in;
    g.rcut2 = (double)g.rcut * (double)g.rcut;
    g.bin_size = g.rcut / 2;                                   // binLinkedList.h:664
    for (int i = 0; i < 3; i++)
        for (int j = 0; j < 3; j++) g.b[i][j] = lattice[i * 3 + j];
    T nyz[3], nxz[3], nxy[3];
    host_cross(g.b[1], g.b[2], nyz);
    host_cross(g.b[0], g.b[2], nxz);
    host_cross(g.b[0], g.b[1], nxy);
    const T dplane[3] = {host_plane_distance(g.b[0], nyz), host_plane_distance(g.b[1], nxz),
                         host_plane_distance(g.b[2], nxy)};
    long long nimg = 1;
    for (int a = 0; a < 3; a++) {
        A2P_REQUIRE(dplane[a] > 0 && std::isfinite((double)dplane[a]), A2P_ERR_INVALID,
                    "nblist: degenerate lattice");
        const int ext = (int)std::ceil(g.rcut / dplane[a]);    // binLinkedList.h:672-676
        const int scaling = pbc[a] ? ext * 2 + 1 : 1;
        g.img_dim[a] = scaling;
        g.img_lo[a] = -(scaling - 1) / 2;                      // structure.h:597-606 (odd scaling)
        nimg *= scaling;
    }
    A2P_REQUIRE(nimg * N < (1ll << 31), A2P_ERR_INVALID,
                "nblist: %lld images x %d atoms exceeds the reference's int supercell index", nimg, N);
    g.nimg = (int)nimg;
    g.ext_bins = (int)std::ceil(g.rcut / g.bin_size);          // binLinkedList.h:914-915
    A2P_REQUIRE(g.ext_bins >= 1 && g.ext_bins <= 3, A2P_ERR_INVALID, "nblist: unsupported bin stencil");
    g.inv_side = 1.0f / (float)(2 * g.ext_bins + 1);
    g.inv_bin = 1.0f / (float)g.bin_size;

    // workspace A: x[N*3] | partial[nblocks*12] | ext[12]
    const int nblocks = ceil_div(N, NBL_BLOCK);
    void* wsA = nullptr;
    size_t bytesA = ((size_t)N * 3 * (co ? 2 : 1) + (size_t)nblocks * 12 + 16) * sizeof(T) + (co ? (size_t)N * sizeof(int) : 0);
    int rc = ws_get(WS_NBL_A, bytesA, &wsA);
    if (rc) return rc;
    T* x = (T*)wsA;
    T* partial = x + (size_t)N * 3;
    T* ext_dev = partial + (size_t)nblocks * 12;
    T* xs = ext_dev + 16;                               // coordinates in processing order (compact lists)
    int* inv = (int*)(xs + (size_t)N * 3);              // ... and the inverse of the order
    void* flags = nullptr;
    rc = ws_get(WS_FLAGS, 64, &flags);
    if (rc) return rc;
    int* status = (int*)flags;

    for (int a = 0; a < 3; a++) { g.mn[a] = 0; g.nbin[a] = 0; g.rlo[a] = 0; g.rdim[a] = 0; }
    prof_begin("nbl_coords_minmax", stream);
    hipLaunchKernelGGL(coords_minmax_kernel<T>, dim3(nblocks), dim3(NBL_BLOCK), 0, stream, g, coords, x,
                       partial);
    prof_end(stream);
    prof_begin("nbl_coords_minmax", stream);
    hipLaunchKernelGGL(minmax_finish_kernel<T>, dim3(1), dim3(12 * 64), 0, stream, partial, nblocks, ext_dev);
    prof_end(stream);
    // the bin box: read back from the extents, or bounded by the box of the last synchronised build of this structure
    int device = 0;
    A2P_HIP_CHECK(hipGetDevice(&device));
    const GridBound* bound = nullptr;
    for (const GridBound& gb : g_bounds) {
        bool same = gb.valid && gb.device == device && gb.N == N && gb.is_cart == is_cart && gb.rcut == (double)g.rcut;
        for (int a = 0; a < 3 && same; a++) same = gb.pbc[a] == (pbc[a] ? 1 : 0);
        for (int q = 0; q < 9 && same; q++) same = gb.lattice[q] == (double)lattice[q];
        if (same) { bound = &gb; break; }
    }
    const bool same = bound != nullptr;
    const bool sync_free = g_sync_free && same && !max_nn_host &&
                           (long long)N * g.nimg * (long long)(4 * sizeof(T)) <= (2ll << 30);
    GridDyn<T>* gd = nullptr;
    long long nregion = 1;
    double big_coord = 0;                               // bound of the coordinates the build keeps
    if (sync_free) {
        int cap[3];
        int grow = 0;
        for (int a = 0; a < 3; a++) {
            cap[a] = bound->rdim[a] + std::max(2, bound->rdim[a] / 8);
            g.rdim[a] = cap[a];                         // host copies of the box serve launch and scratch sizes only
            nregion *= cap[a];
            grow = std::max(grow, cap[a] - bound->rdim[a]);
        }
        big_coord = bound->big + (double)(grow + 2) * (double)g.bin_size;   // the box cannot have moved further
        A2P_REQUIRE(nregion < (1ll << 30), A2P_ERR_INVALID, "nblist: %lld bins around the centre atoms", nregion);
        void* wsG = nullptr;
        rc = ws_get(WS_GRID, 256, &wsG);
        if (rc) return rc;
        gd = (GridDyn<T>*)wsG;
        hipLaunchKernelGGL(grid_setup_kernel<T>, dim3(1), dim3(64), 0, stream, g, (const T*)ext_dev, gd, cap[0], cap[1],
                           cap[2], big_coord, status);
    } else {
        T ext[12];
        A2P_HIP_CHECK(hipMemcpyAsync(ext, ext_dev, sizeof(ext), hipMemcpyDeviceToHost, stream));
        A2P_HIP_CHECK(hipStreamSynchronize(stream));

        // find_pl_info4nblist + bin counts (structure.h:1013-1061, binLinkedList.h:685-688)
        for (int a = 0; a < 3; a++) {
            A2P_REQUIRE(std::isfinite((double)ext[a]) && std::isfinite((double)ext[3 + a]), A2P_ERR_INVALID,
                        "nblist: non-finite coordinates");
            const T mn = ext[a] - (T)kMargin;
            const T mx = ext[3 + a] + (T)kMargin;
            const T pl = mx - mn;
            g.mn[a] = mn;
            g.nbin[a] = (int)std::ceil(pl / g.bin_size);
            const int cb_lo = (int)std::floor((ext[6 + a] - mn) / g.bin_size);
            const int cb_hi = (int)std::floor((ext[9 + a] - mn) / g.bin_size);
            g.rlo[a] = std::max(cb_lo - g.ext_bins, 0);
            const int rhi = std::min(cb_hi + g.ext_bins, g.nbin[a] - 1);
            g.rdim[a] = rhi - g.rlo[a] + 1;
            A2P_REQUIRE(g.rdim[a] > 0, A2P_ERR_INVALID, "nblist: empty bin box");
            {
                // a coordinate c is binned as floor((c - mn) / bin_size) in T: the slack covers the
                // rounding of that expression and of the two bounds by orders of magnitude
                const double big = std::max(std::fabs((double)mn), std::fabs((double)mx));
                const double slack = 1.0e-3 * (double)g.bin_size + 1.0e-5 * (big + (double)pl);
                g.keep_lo[a] = (T)((double)mn + (double)g.rlo[a] * (double)g.bin_size - slack);
                g.keep_hi[a] = (T)((double)mn + (double)(g.rlo[a] + g.rdim[a]) * (double)g.bin_size + slack);
            }
            nregion *= g.rdim[a];
        }
        A2P_REQUIRE(nregion < (1ll << 30), A2P_ERR_INVALID,
                    "nblist: %lld bins around the centre atoms; are the coordinates far outside the cell?",
                    nregion);
        for (int a = 0; a < 3; a++)
            big_coord = std::max(big_coord, std::max(std::fabs((double)g.keep_lo[a]), std::fabs((double)g.keep_hi[a])));
        GridBound nb;
        nb.big = big_coord;
        nb.valid = true;
        nb.device = device; nb.N = N; nb.is_cart = is_cart; nb.rcut = (double)g.rcut;
        for (int a = 0; a < 3; a++) { nb.pbc[a] = pbc[a] ? 1 : 0; nb.rdim[a] = g.rdim[a]; }
        for (int q = 0; q < 9; q++) nb.lattice[q] = (double)lattice[q];
        if (bound) {
            g_bounds[bound - g_bounds.data()] = nb;
        } else {
            if (g_bounds.size() >= kMaxBounds) g_bounds.erase(g_bounds.begin());
            g_bounds.push_back(nb);
        }
    }
    const int nb1 = (int)nregion + 1;

    // workspace B: counts[nb1] | offsets[nb1] | cursor[nb1] | scan tmp, then (after the count is
    // known) the image records s_rec[total][4], and for sort: keys[N*umax] | order[N*umax] | tmp rows
    const int ntmp = scan_tmp_ints(nb1);
    size_t ints = (size_t)nb1 * 3 + ntmp;
    void* wsB = nullptr;
    rc = ws_get(WS_NBL_B, ints * sizeof(int), &wsB);
    if (rc) return rc;
    int* counts = (int*)wsB;
    int* offsets = counts + nb1;
    int* cursor = offsets + nb1;
    int* tmp = cursor + nb1;
    rc = fill_zero2(counts, (size_t)nb1 * sizeof(int), cursor, (size_t)nb1 * sizeof(int), stream);
    if (rc) return rc;
    const dim3 pair_grid(ceil_div(N, NBL_BLOCK));
    // binning: a thread per atom, or per x-layer of an atom's images while the structure is small
    const int split = (N < 65536 && g.img_dim[0] > 1) ? g.img_dim[0] : 1;
    const dim3 image_grid(ceil_div((long long)N * split, NBL_BLOCK));
    prof_begin("nbl_count", stream);
    hipLaunchKernelGGL(count_kernel<T>, image_grid, dim3(NBL_BLOCK), 0, stream, g, x, counts, incoming,
                       (const GridDyn<T>*)gd, types, want_rows ? ilist : (int*)nullptr, types_out, split);
    prof_end(stream);
    rc = exclusive_scan_i32(counts, offsets, nb1, tmp, stream);
    if (rc) return rc;
    // Entries of the sorted image arrays.  Every (atom, image) pair can own at most one: while that
    // bound stays below 2 GiB the arrays are simply sized for it and the host never learns the count
    // (one synchronisation less per build); beyond, the count is read back.
    long long total = (long long)N * g.nimg;
    if (total * (long long)(4 * sizeof(T)) > (2ll << 30)) {
        int counted = 0;
        A2P_HIP_CHECK(hipMemcpyAsync(&counted, offsets + nregion, sizeof(int), hipMemcpyDeviceToHost, stream));
        A2P_HIP_CHECK(hipStreamSynchronize(stream));
        total = counted;
    }

    size_t sorted_bytes = (size_t)total * 4 * sizeof(T) + 256;
    size_t sort_bytes = sort ? (size_t)N * umax * (2 * sizeof(int) + 4 * sizeof(T)) + 256 : 0;
    void* wsC = nullptr;
    rc = ws_get(WS_MISC, sorted_bytes + sort_bytes, &wsC);
    if (rc) return rc;
    T* s_rec = (T*)wsC;
    char* sort_base = (char*)wsC + (sorted_bytes / 256) * 256;   // 256-byte aligned, inside the slack
    T* tmp_rcs = nullptr;
    T* keys = nullptr;
    int* order = nullptr;
    int* tmp_first = nullptr;
    if (sort) {
        tmp_rcs = (T*)sort_base;
        keys = tmp_rcs + (size_t)N * umax * 3;
        order = (int*)(keys + (size_t)N * umax);
        tmp_first = order + (size_t)N * umax;
    }

    prof_begin("nbl_fill", stream);

    hipLaunchKernelGGL(fill_kernel<T>, image_grid, dim3(NBL_BLOCK), 0, stream, g, x, offsets, cursor,
                       s_rec, (const GridDyn<T>*)gd, split);

    prof_end(stream);
    prof_begin("nbl_binsort", stream);
    hipLaunchKernelGGL(binsort_kernel<T>, dim3(ceil_div(nregion, NBL_BLOCK)), dim3(NBL_BLOCK), 0, stream,
                       (int)nregion, offsets, s_rec, g.N, co ? types : (const int*)nullptr, (const GridDyn<T>*)gd,
                       ((-g.img_lo[0]) * g.img_dim[1] + (-g.img_lo[1])) * g.img_dim[2] + (-g.img_lo[2]));
    prof_end(stream);
    CompactEmit<T> ce{};
    if (co) {
        // processing order: atoms sorted by the Morton code of their bin (ties by index: the sort is stable)
        const CompactView<T> cv = compact_view<T>(co->buffer, N, umax);
        if (!co->keep_order) {
        int maxdim = std::max(g.rdim[0], std::max(g.rdim[1], g.rdim[2]));
        int shift = 0;
        while ((maxdim >> shift) > 1024) shift++;
        int bits = 1;
        while ((1 << bits) < ((maxdim >> shift) + 1)) bits++;
        size_t tmp_bytes = 0;
        A2P_HIP_CHECK(hipcub::DeviceRadixSort::SortPairs(nullptr, tmp_bytes, (const unsigned*)nullptr, (unsigned*)nullptr,
                                                         (const int*)nullptr, (int*)nullptr, N, 0, 3 * bits, stream));
        const size_t key_bytes = (((size_t)N * sizeof(unsigned) + 255) / 256) * 256;
        void* wsD = nullptr;
        rc = ws_get(WS_CSR, 3 * key_bytes + tmp_bytes, &wsD);
        if (rc) return rc;
        unsigned* keys_in = (unsigned*)wsD;
        unsigned* keys_out = (unsigned*)((char*)wsD + key_bytes);
        int* vals_in = (int*)((char*)wsD + 2 * key_bytes);
        void* tmp_sort = (char*)wsD + 3 * key_bytes;
        prof_begin("nbl_order", stream);
        hipLaunchKernelGGL(order_keys_kernel<T>, pair_grid, dim3(NBL_BLOCK), 0, stream, g, x, shift, keys_in, vals_in,
                           (const GridDyn<T>*)gd);
        prof_end(stream);
        prof_begin("nbl_order", stream);
        A2P_HIP_CHECK(hipcub::DeviceRadixSort::SortPairs(tmp_sort, tmp_bytes, (const unsigned*)keys_in, keys_out,
                                                         (const int*)vals_in, cv.order, N, 0, 3 * bits, stream));
        prof_end(stream);
        }
        ce.order = cv.order;
        ce.entries = cv.entries;
        ce.n_outer = cv.n_outer;
        ce.n_inner = cv.n_inner;
        ce.nch = cv.nch;
        prof_begin("nbl_order", stream);
        hipLaunchKernelGGL(sorted_coords_kernel<T>, pair_grid, dim3(NBL_BLOCK), 0, stream, N, (const T*)x,
                           (const int*)cv.order, xs, inv);
        prof_end(stream);
        ce.xs = xs;
        ce.inv = inv;
        ce.split2 = (T)co->split * (T)co->split;
        ce.outer2 = (T)co->outer * (T)co->outer;
        ce.write_rows = want_rows ? 1 : 0;
        {
            // the two ends of a pair see vectors that differ by the rounding of their images (three roundings at the
            // size of the coordinates): the band is 16 such roundings wide
            const double dr = 16.0 * (sizeof(T) == 4 ? 1.1920929e-7 : 2.220446049250313e-16) * big_coord;
            ce.near_band = (T)(2.0 * co->split * dr + dr * dr);
        }
    }
    const int list_blocks = ceil_div(N, (NBL_BLOCK / 64) * NBL_APW);
    prof_begin("nbl_lists", stream);
    const size_t rows_lds = rowbuf_bytes<T>(umax, rank != nullptr) * (NBL_BLOCK / 64);
    const bool rowbuf = !sort && umax % 4 == 0 && rows_lds <= 32 * 1024 && (uintptr_t)firstneigh % 16 == 0 &&
                        (uintptr_t)rcs % 16 == 0 && (uintptr_t)rank % 16 == 0;
    if (co)
        hipLaunchKernelGGL((lists_kernel<T, false, true, false, true>), dim3(list_blocks), dim3(NBL_BLOCK), rows_lds,
                           stream, g, x, types, offsets, s_rec, umax, ilist, numneigh, firstneigh, rcs, types_out,
                           keys, status, update, nullptr, nullptr, ce, (const GridDyn<T>*)gd);
    else if (sort)
        hipLaunchKernelGGL((lists_kernel<T, true, false, false>), dim3(list_blocks), dim3(NBL_BLOCK), 0, stream, g, x,
                           types, offsets, s_rec, umax, ilist, numneigh, tmp_first, tmp_rcs, types_out, keys,
                           status, 0, nullptr, nullptr, CompactEmit<T>{}, (const GridDyn<T>*)gd);
    else if (rowbuf && rank)
        hipLaunchKernelGGL((lists_kernel<T, false, true, true>), dim3(list_blocks), dim3(NBL_BLOCK), rows_lds, stream,
                           g, x, types, offsets, s_rec, umax, ilist, numneigh, firstneigh, rcs, types_out, keys,
                           status, update, rank, incoming, CompactEmit<T>{}, (const GridDyn<T>*)gd);
    else if (rowbuf)
        hipLaunchKernelGGL((lists_kernel<T, false, true, false>), dim3(list_blocks), dim3(NBL_BLOCK), rows_lds, stream,
                           g, x, types, offsets, s_rec, umax, ilist, numneigh, firstneigh, rcs, types_out, keys,
                           status, update, nullptr, nullptr, CompactEmit<T>{}, (const GridDyn<T>*)gd);
    else if (rank)
        hipLaunchKernelGGL((lists_kernel<T, false, false, true>), dim3(list_blocks), dim3(NBL_BLOCK), 0, stream, g, x,
                           types, offsets, s_rec, umax, ilist, numneigh, firstneigh, rcs, types_out, keys,
                           status, update, rank, incoming, CompactEmit<T>{}, (const GridDyn<T>*)gd);
    else
        hipLaunchKernelGGL((lists_kernel<T, false, false, false>), dim3(list_blocks), dim3(NBL_BLOCK), 0, stream, g, x,
                           types, offsets, s_rec, umax, ilist, numneigh, firstneigh, rcs, types_out, keys,
                           status, update, nullptr, nullptr, CompactEmit<T>{}, (const GridDyn<T>*)gd);
    prof_end(stream);
    if (co) {
        prof_begin("nbl_symmetry", stream);
        hipLaunchKernelGGL(compact_symmetry_kernel<T>, dim3(ceil_div(N, NBL_BLOCK)), dim3(NBL_BLOCK), (size_t)(NBL_BLOCK / 64) * umax * 4 * sizeof(T),
                           stream, g, (const GridDyn<T>*)gd, (const T*)x, ce, umax, status);
        prof_end(stream);
    }
    if (sort) {
        prof_begin("nbl_sort_rows", stream);
        hipLaunchKernelGGL(sort_rows_kernel<T>, dim3(ceil_div(N, 64)), dim3(64), 0, stream, N, umax, numneigh,
                           keys, order);
        prof_end(stream);
        prof_begin("nbl_gather_rows", stream);
        hipLaunchKernelGGL(gather_rows_kernel<T>, dim3(ceil_div(N, NBL_BLOCK / 64)), dim3(NBL_BLOCK), 0, stream, N, umax,
                           numneigh, order, tmp_first, tmp_rcs, firstneigh, rcs);
        prof_end(stream);
    }
    A2P_HIP_CHECK(hipGetLastError());

    if (max_nn_host) {
        // largest neighbour count: block-wise maxima, one integer atomic per block
        rc = fill_zero(status + 1, sizeof(int), stream);
        if (rc) return rc;
        prof_begin("nbl_max", stream);
        hipLaunchKernelGGL(int_max_kernel, dim3(std::min(ceil_div(N, 256), 1024)), dim3(256), 0, stream,
                           numneigh, N, status + 1);
        prof_end(stream);
        int st[2] = {0, 0};
        A2P_HIP_CHECK(hipMemcpyAsync(st, status, sizeof(st), hipMemcpyDeviceToHost, stream));
        A2P_HIP_CHECK(hipStreamSynchronize(stream));
        *max_nn_host = st[1];
        if (st[1] > umax) {
            rc = fill_zero(status, sizeof(int), stream);
            if (rc) return rc;
            set_error("nblist: an atom has %d neighbours, more than umax_num_neigh_atoms = %d", st[1], umax);
            return A2P_ERR_OVERFLOW;
        }
    }
    return A2P_OK;
}

}  // namespace
}  // namespace a2p

extern "C" {

int a2p_nblist_sync_free(int on)
{
    const int before = a2p::g_sync_free;
    a2p::g_sync_free = on ? 1 : 0;
    return before;
}

int a2p_nblist_build_f32(const float* lattice, const int* types, const float* coords, int natoms,
                         double rcut, int umax, int is_cart, const int* pbc, int sort, int* ilist,
                         int* numneigh, int* firstneigh, float* rcs, int* types_out, int* max_numneigh,
                         void* stream)
{
    return a2p::nblist_build<float>(lattice, types, coords, natoms, rcut, umax, is_cart, pbc, sort, ilist,
                                    numneigh, firstneigh, rcs, types_out, max_numneigh, (hipStream_t)stream);
}

int a2p_nblist_build_f64(const double* lattice, const int* types, const double* coords, int natoms,
                         double rcut, int umax, int is_cart, const int* pbc, int sort, int* ilist,
                         int* numneigh, int* firstneigh, double* rcs, int* types_out, int* max_numneigh,
                         void* stream)
{
    return a2p::nblist_build<double>(lattice, types, coords, natoms, rcut, umax, is_cart, pbc, sort, ilist,
                                     numneigh, firstneigh, rcs, types_out, max_numneigh,
                                     (hipStream_t)stream);
}

int a2p_nblist_update_f32(const float* lattice, const int* types, const float* coords, int natoms,
                          double rcut, int umax, int is_cart, const int* pbc, int sort, int* ilist,
                          int* numneigh, int* firstneigh, float* rcs, int* types_out, int* max_numneigh,
                          void* stream)
{
    return a2p::nblist_build<float>(lattice, types, coords, natoms, rcut, umax, is_cart, pbc, sort, ilist,
                                    numneigh, firstneigh, rcs, types_out, max_numneigh, (hipStream_t)stream,
                                    1);
}

int a2p_nblist_update_f64(const double* lattice, const int* types, const double* coords, int natoms,
                          double rcut, int umax, int is_cart, const int* pbc, int sort, int* ilist,
                          int* numneigh, int* firstneigh, double* rcs, int* types_out, int* max_numneigh,
                          void* stream)
{
    return a2p::nblist_build<double>(lattice, types, coords, natoms, rcut, umax, is_cart, pbc, sort, ilist,
                                     numneigh, firstneigh, rcs, types_out, max_numneigh,
                                     (hipStream_t)stream, 1);
}

int a2p_nblist_build_ranked_f32(const float* lattice, const int* types, const float* coords, int natoms,
                                double rcut, int umax, int is_cart, const int* pbc, int update, int* ilist,
                                int* numneigh, int* firstneigh, float* rcs, int* types_out, int* rank,
                                int* incoming, int* max_numneigh, void* stream)
{
    if (!rank || !incoming) {
        a2p::set_error("nblist: rank and incoming must be device pointers");
        return A2P_ERR_INVALID;
    }
    return a2p::nblist_build<float>(lattice, types, coords, natoms, rcut, umax, is_cart, pbc, 0, ilist, numneigh,
                                    firstneigh, rcs, types_out, max_numneigh, (hipStream_t)stream, update ? 1 : 0,
                                    rank, incoming);
}

int a2p_nblist_build_ranked_f64(const double* lattice, const int* types, const double* coords, int natoms,
                                double rcut, int umax, int is_cart, const int* pbc, int update, int* ilist,
                                int* numneigh, int* firstneigh, double* rcs, int* types_out, int* rank,
                                int* incoming, int* max_numneigh, void* stream)
{
    if (!rank || !incoming) {
        a2p::set_error("nblist: rank and incoming must be device pointers");
        return A2P_ERR_INVALID;
    }
    return a2p::nblist_build<double>(lattice, types, coords, natoms, rcut, umax, is_cart, pbc, 0, ilist, numneigh,
                                     firstneigh, rcs, types_out, max_numneigh, (hipStream_t)stream, update ? 1 : 0,
                                     rank, incoming);
}

size_t a2p_nblist_compact_bytes(int natoms, int umax, int elem_size)
{
    if (!a2p::compact_supported(natoms, umax) || (elem_size != 4 && elem_size != 8)) return 0;
    return a2p::compact_layout(natoms, umax, (size_t)elem_size).bytes;
}

int a2p_nblist_build_compact_f32(const float* lattice, const int* types, const float* coords, int natoms,
                                 double rcut, int umax, int is_cart, const int* pbc, int update, double rcut_outer,
                                 double rcut_inner, int* ilist, int* numneigh, int* firstneigh, float* rcs,
                                 int* types_out, void* compact, void* stream)
{
    const a2p::CompactOut co{compact, rcut_inner, rcut_outer, (update & 2) ? 1 : 0};
    return a2p::nblist_build<float>(lattice, types, coords, natoms, rcut, umax, is_cart, pbc, 0, ilist, numneigh,
                                    firstneigh, rcs, types_out, nullptr, (hipStream_t)stream, (update & 1) ? 1 : 0, nullptr,
                                    nullptr, &co);
}

int a2p_nblist_build_compact_f64(const double* lattice, const int* types, const double* coords, int natoms,
                                 double rcut, int umax, int is_cart, const int* pbc, int update, double rcut_outer,
                                 double rcut_inner, int* ilist, int* numneigh, int* firstneigh, double* rcs,
                                 int* types_out, void* compact, void* stream)
{
    const a2p::CompactOut co{compact, rcut_inner, rcut_outer, (update & 2) ? 1 : 0};
    return a2p::nblist_build<double>(lattice, types, coords, natoms, rcut, umax, is_cart, pbc, 0, ilist, numneigh,
                                     firstneigh, rcs, types_out, nullptr, (hipStream_t)stream, (update & 1) ? 1 : 0, nullptr,
                                     nullptr, &co);
}
}
