// TEST INFRASTRUCTURE ONLY -- CPU restatement (fp64) of the reference's short-range force
// and virial reductions and of their vector-Jacobian products, without the dense Jacobian
// the reference materialises (source/fvt/include/force_sr.h:50-124, virial_sr.h:24-51;
// backward formulas as in src/force_sr_op.cc and src/virial_sr_op.cc).
//
// Pinned by: the compiled reference (oracle/_ref/libref_fvt.so) on tiny inputs, where its
// Jacobian entries are +-1 (the property test/fromcc/test_forceSrOp.py:57-81 checks), and by
// the closed forms F_c = sum_j g_cj - sum_{(i,j): nbr(i,j)=c} g_ij, V_ab = -sum g_a r_b.
#include <cstddef>
#include <cstring>

extern "C" {

void orc_fvt_force_f64(double* force, double* grad_out, const double* grad_in, int inum,
                       const int* ilist, const int* numneigh, const int* firstneigh, int nghost,
                       int umax, const double* dei_drij)
{
    std::memset(force, 0, sizeof(double) * (inum + nghost) * 3);
    if (grad_out) std::memset(grad_out, 0, sizeof(double) * (size_t)inum * umax * 3);
    for (int ii = 0; ii < inum; ii++) {
        int c = ilist[ii];
        for (int jj = 0; jj < numneigh[ii]; jj++) {
            int j = firstneigh[(size_t)ii * umax + jj];
            for (int k = 0; k < 3; k++) {
                size_t e = ((size_t)ii * umax + jj) * 3 + k;
                force[c * 3 + k] += dei_drij[e];
                force[j * 3 + k] -= dei_drij[e];
                if (grad_out) grad_out[e] = grad_in[c * 3 + k] - grad_in[j * 3 + k];
            }
        }
    }
}

void orc_fvt_virial_f64(double* virial, double* der1, double* der2, int inum, const int* numneigh,
                        const double* rcs, int umax, const double* dei_drij)
{
    std::memset(virial, 0, sizeof(double) * 9);
    size_t n = (size_t)inum * umax;
    if (der1) std::memset(der1, 0, sizeof(double) * 9 * n);
    if (der2) std::memset(der2, 0, sizeof(double) * 9 * n);
    for (int ii = 0; ii < inum; ii++)
        for (int jj = 0; jj < numneigh[ii]; jj++) {
            size_t e = (size_t)ii * umax + jj;
            for (int a = 0; a < 3; a++)
                for (int b = 0; b < 3; b++) {
                    virial[a * 3 + b] -= dei_drij[e * 3 + a] * rcs[e * 3 + b];
                    if (der1) der1[(a * 3 + b) * n + e] -= rcs[e * 3 + b];
                    if (der2) der2[(a * 3 + b) * n + e] -= dei_drij[e * 3 + a];
                }
        }
}

}
