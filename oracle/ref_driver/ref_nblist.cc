// TEST INFRASTRUCTURE ONLY. Thin extern "C" driver around the reference's own
// neighbor-list headers, compiled where they lie (REF_ROOT/source/nblist/include)
// into oracle/_ref/libref_nblist.so. Nothing of the reference is copied here; the
// driver only instantiates its templates and marshals flat arrays, doing what
// source/nblist/bind/nblist_bind.cc:35-189 does for NumPy arrays.
#include <cstring>
#include "nblist/include/neighborList.h"

namespace {
template <typename T>
int run(const T* lattice, const int* types, const T* coords, int n, double rcut, int umax,
        int is_cart, const int* pbc, int sort, int* ilist, int* numneigh, int* firstneigh,
        T* rcs, int* types_out, int* max_nn)
{
    bool pbc_xyz[3] = {pbc[0] != 0, pbc[1] != 0, pbc[2] != 0};
    ai2pot::Structure<T> structure(n, const_cast<T*>(lattice), const_cast<int*>(types),
                                   const_cast<T*>(coords), is_cart != 0);
    ai2pot::NeighborList<T> nbl(structure, (T)rcut, pbc_xyz, sort != 0);
    int mx = nbl.get_max_num_neigh_atoms();
    *max_nn = mx;
    if (mx > umax) return 1;   // the reference would overflow its output arrays here
    int inum = 0, nghost = 0;
    std::memcpy(types_out, types, sizeof(int) * n);
    nbl.find_info4mlff(inum, ilist, numneigh, firstneigh, rcs, types_out, nghost, umax);
    return 0;
}
}  // namespace

extern "C" {
int ref_nblist_f32(const float* lattice, const int* types, const float* coords, int n, double rcut,
                   int umax, int is_cart, const int* pbc, int sort, int* ilist, int* numneigh,
                   int* firstneigh, float* rcs, int* types_out, int* max_nn)
{
    return run<float>(lattice, types, coords, n, rcut, umax, is_cart, pbc, sort, ilist, numneigh,
                      firstneigh, rcs, types_out, max_nn);
}
int ref_nblist_f64(const double* lattice, const int* types, const double* coords, int n, double rcut,
                   int umax, int is_cart, const int* pbc, int sort, int* ilist, int* numneigh,
                   int* firstneigh, double* rcs, int* types_out, int* max_nn)
{
    return run<double>(lattice, types, coords, n, rcut, umax, is_cart, pbc, sort, ilist, numneigh,
                       firstneigh, rcs, types_out, max_nn);
}
}
