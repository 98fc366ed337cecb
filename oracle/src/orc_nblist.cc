// TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference's periodic neighbor list,
// used by the tests, smoke() and the cpu_baseline leg of bench.py as the checker.
// It follows the reference's algorithm and, because the outputs must be bit-exact, its
// arithmetic (which operations run in T and which in double) step by step.  Citations
// are to files under the reference's source/nblist/include unless a path is given.
//
// Pinned by: the compiled reference (oracle/_ref/libref_nblist.so) on every fixture of
// tests/test_oracle_nblist.py, the reference's own assertions (max 12 neighbours at
// rcut 3.2 on MoS2, tests/test_neighborList.cc:244) and an O(N^2 * images) brute force.
#include <algorithm>
#include <climits>
#include <cmath>
#include <cstring>
#include <vector>

namespace {

const double kMargin = 0.5;     // NBLIST_MARGIN, structure.h:27
const double kEpsilon = 1e-3;   // EPSILON, binLinkedList.h:28

template <typename T>
struct SortByDistance {         // SingleNeighborListSortBasis, neighborList.h:31-43
    const T* d;
    bool operator()(int a, int b) const { return d[a] < d[b]; }
};

template <typename T>
void cross(const T* a, const T* b, T* o)      // source/core/include/vec3Operation.h:87-93
{
    o[0] = a[1] * b[2] - a[2] * b[1];
    o[1] = a[2] * b[0] - a[0] * b[2];
    o[2] = a[0] * b[1] - a[1] * b[0];
}

template <typename T>
void normalize(const T* v, T* u)              // vec3Operation.h:97-104 (squares via pow -> double)
{
    T len = std::sqrt(std::pow(v[0], 2) + std::pow(v[1], 2) + std::pow(v[2], 2));
    u[0] = v[0] / len;
    u[1] = v[1] / len;
    u[2] = v[2] / len;
}

template <typename T>
T dot(const T* a, const T* b) { return a[0] * b[0] + a[1] * b[1] + a[2] * b[2]; }   // :40-43

template <typename T>
int build(const T* lattice, const int* types, const T* coords, int n, double rcut_in, int umax,
          int is_cart, const int* pbc, int sort, int* ilist, int* numneigh, int* firstneigh, T* rcs,
          int* types_out, int* max_nn)
{
    if (n <= 0) return 2;                      // assert(num_atoms > 0), binLinkedList.h:659
    const T rcut = (T)rcut_in;
    T b[3][3];
    for (int i = 0; i < 3; i++)
        for (int j = 0; j < 3; j++) b[i][j] = lattice[i * 3 + j];

    // Structure ctor + calc_cart_coords, structure.h:300-342, 561-579
    std::vector<T> x((size_t)n * 3);
    for (int i = 0; i < n; i++) {
        if (is_cart) {
            for (int a = 0; a < 3; a++) x[i * 3 + a] = coords[i * 3 + a];
        } else {
            for (int a = 0; a < 3; a++)
                x[i * 3 + a] = coords[i * 3 + 0] * b[0][a] + coords[i * 3 + 1] * b[1][a] +
                               coords[i * 3 + 2] * b[2][a];
        }
    }

    // get_interplanar_distances, structure.h:818-842
    T vyz[3], vxz[3], vxy[3], uyz[3], uxz[3], uxy[3], dplane[3];
    cross(b[1], b[2], vyz);
    cross(b[0], b[2], vxz);
    cross(b[0], b[1], vxy);
    normalize(vyz, uyz);
    normalize(vxz, uxz);
    normalize(vxy, uxy);
    dplane[0] = std::abs(dot(b[0], uyz));
    dplane[1] = std::abs(dot(b[1], uxz));
    dplane[2] = std::abs(dot(b[2], uxy));

    // BinLinkedList ctor, binLinkedList.h:658-696
    const T bin_size = rcut / 2;
    int scaling[3];
    for (int a = 0; a < 3; a++) {
        int ext = std::ceil(rcut / dplane[a]);
        scaling[a] = pbc[a] ? ext * 2 + 1 : 1;
    }
    // make_supercell, structure.h:589-707 (scaling is always odd here)
    int lo[3], hi[3];
    for (int a = 0; a < 3; a++) {
        lo[a] = -(scaling[a] - 1) / 2;
        hi[a] = (scaling[a] - 1) / 2;
    }
    const size_t nimg = (size_t)scaling[0] * scaling[1] * scaling[2];
    const size_t nsup = nimg * n;
    if (nsup > (size_t)INT_MAX) return 3;
    std::vector<T> sx(nsup * 3);
    {
        size_t idx = 0;
        for (int ii = lo[0]; ii <= hi[0]; ii++)
            for (int jj = lo[1]; jj <= hi[1]; jj++)
                for (int kk = lo[2]; kk <= hi[2]; kk++)
                    for (int p = 0; p < n; p++) {
                        for (int a = 0; a < 3; a++)
                            sx[idx * 3 + a] = x[p * 3 + a] + b[0][a] * ii + b[1][a] * jj + b[2][a] * kk;
                        idx++;
                    }
    }
    // centre image: calc_prim_cell_idx, binLinkedList.h:468-497
    int pc[3];
    for (int a = 0; a < 3; a++) pc[a] = (scaling[a] - 1) / 2;
    const int prim_cell_idx = pc[0] + pc[1] * scaling[0] + pc[2] * scaling[0] * scaling[1];
    const size_t centre0 = (size_t)prim_cell_idx * n;

    // find_pl_info4nblist, structure.h:1013-1061
    T mn[3], mx[3], pl[3];
    for (int a = 0; a < 3; a++) {
        mn[a] = INT_MAX;
        mx[a] = INT_MIN;
    }
    for (size_t i = 0; i < nsup; i++)
        for (int a = 0; a < 3; a++) {
            T c = sx[i * 3 + a];
            if (c < mn[a]) mn[a] = c;
            if (c > mx[a]) mx[a] = c;
        }
    int nbin[3];
    for (int a = 0; a < 3; a++) {
        mn[a] -= (T)kMargin;
        mx[a] += (T)kMargin;
        pl[a] = mx[a] - mn[a];
        nbin[a] = std::ceil(pl[a] / bin_size);
    }

    // BinLinkedList::_build, binLinkedList.h:808-836 (head insertion)
    std::vector<int> heads((size_t)nbin[0] * nbin[1] * nbin[2], -1), nexts(nsup, -1);
    for (size_t i = 0; i < nsup; i++) {
        int bx = std::floor((sx[i * 3 + 0] - mn[0]) / bin_size);
        int by = std::floor((sx[i * 3 + 1] - mn[1]) / bin_size);
        int bz = std::floor((sx[i * 3 + 2] - mn[2]) / bin_size);
        size_t bin = (size_t)bx + (size_t)by * nbin[0] + (size_t)bz * nbin[0] * nbin[1];
        nexts[i] = heads[bin];
        heads[bin] = (int)i;
    }

    // get_neigh_bins + get_neigh_atoms, binLinkedList.h:900-1031; sort, neighborList.h:274-338
    const int ext_bins = std::ceil(rcut / bin_size);
    std::vector<std::vector<int>> lists(n);
    int maxn = 0;
    for (int p = 0; p < n; p++) {
        const T* c = &sx[(centre0 + p) * 3];
        int cb[3];
        for (int a = 0; a < 3; a++) cb[a] = std::floor((c[a] - mn[a]) / bin_size);
        std::vector<int>& out = lists[p];
        for (int ii = -ext_bins; ii <= ext_bins; ii++)
            for (int jj = -ext_bins; jj <= ext_bins; jj++)
                for (int kk = -ext_bins; kk <= ext_bins; kk++) {
                    int q[3] = {cb[0] + ii, cb[1] + jj, cb[2] + kk};
                    bool valid = true;
                    for (int a = 0; a < 3; a++) {
                        if (pbc[a]) q[a] = (q[a] + nbin[a]) % nbin[a];
                        if (q[a] < 0 || q[a] >= nbin[a]) valid = false;
                    }
                    if (!valid) continue;
                    size_t bin = (size_t)q[0] + (size_t)q[1] * nbin[0] + (size_t)q[2] * nbin[0] * nbin[1];
                    for (int j = heads[bin]; j != -1; j = nexts[j]) {
                        const T* nc = &sx[(size_t)j * 3];
                        T d2 = std::pow(nc[0] - c[0], 2) + std::pow(nc[1] - c[1], 2) +
                               std::pow(nc[2] - c[2], 2);
                        if ((d2 < std::pow(rcut, 2)) && (d2 > kEpsilon)) out.push_back(j);
                    }
                }
        if (sort) {
            int m = (int)out.size();
            std::vector<T> dist(m);
            std::vector<int> idx(m);
            for (int j = 0; j < m; j++) {
                const T* nc = &sx[(size_t)out[j] * 3];
                idx[j] = j;
                dist[j] = std::sqrt(std::pow(nc[0] - c[0], 2) + std::pow(nc[1] - c[1], 2) +
                                    std::pow(nc[2] - c[2], 2));
            }
            std::sort(idx.begin(), idx.end(), SortByDistance<T>{dist.data()});
            std::vector<int> arranged(m);
            for (int j = 0; j < m; j++) arranged[j] = out[idx[j]];
            out.swap(arranged);
        }
        if ((int)out.size() > maxn) maxn = (int)out.size();
    }
    *max_nn = maxn;
    if (maxn > umax) return 1;

    // find_info4mlff, neighborList.h:532-578
    std::fill(firstneigh, firstneigh + (size_t)n * umax, -1);
    std::fill(rcs, rcs + (size_t)n * umax * 3, (T)0);
    for (int p = 0; p < n; p++) {
        ilist[p] = p;
        numneigh[p] = (int)lists[p].size();
        types_out[p] = types[p];
        const T* c = &sx[(centre0 + p) * 3];
        for (int j = 0; j < numneigh[p]; j++) {
            int s = lists[p][j];
            firstneigh[(size_t)p * umax + j] = s % n;
            for (int a = 0; a < 3; a++)
                rcs[((size_t)p * umax + j) * 3 + a] = sx[(size_t)s * 3 + a] - c[a];
        }
    }
    return 0;
}

}  // namespace

extern "C" {
int orc_nblist_f32(const float* lattice, const int* types, const float* coords, int n, double rcut,
                   int umax, int is_cart, const int* pbc, int sort, int* ilist, int* numneigh,
                   int* firstneigh, float* rcs, int* types_out, int* max_nn)
{
    return build<float>(lattice, types, coords, n, rcut, umax, is_cart, pbc, sort, ilist, numneigh,
                        firstneigh, rcs, types_out, max_nn);
}
int orc_nblist_f64(const double* lattice, const int* types, const double* coords, int n, double rcut,
                   int umax, int is_cart, const int* pbc, int sort, int* ilist, int* numneigh,
                   int* firstneigh, double* rcs, int* types_out, int* max_nn)
{
    return build<double>(lattice, types, coords, n, rcut, umax, is_cart, pbc, sort, ilist, numneigh,
                         firstneigh, rcs, types_out, max_nn);
}
}
