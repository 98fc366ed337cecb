// TEST INFRASTRUCTURE ONLY. extern "C" driver around the reference's short-range
// force / virial kernels (REF_ROOT/source/fvt/include/force_sr.h:50-124,
// virial_sr.h:24-51), built into oracle/_ref/libref_fvt.so. The reference fills a dense
// Jacobian [(inum+nghost)*3, inum*umax]; the driver allocates it, so only tiny inputs fit.
#include <cstdlib>
#include <cstring>
#include <cmath>
#include "fvt/include/force_sr.h"
#include "fvt/include/virial_sr.h"

using namespace ai2pot::fvt;

extern "C" {

// force[(inum+nghost)*3]; grad_in = dL/dforce; grad_out[inum*umax*3] = dL/d(dei_drij)
void ref_fvt_force_f64(double* force, double* grad_out, const double* grad_in, int inum,
                       const int* ilist, const int* numneigh, const int* firstneigh, int nghost,
                       int umax, const double* dei_drij)
{
    size_t nder = (size_t)(inum + nghost) * 3 * inum * umax;
    double* der = (double*)std::malloc(sizeof(double) * nder);
    ForceSr<double>::find_val_der(force, der, inum, const_cast<int*>(ilist),
                                  const_cast<int*>(numneigh), const_cast<int*>(firstneigh), nghost,
                                  umax, const_cast<double*>(dei_drij));
    if (grad_out) {
        std::memset(grad_out, 0, sizeof(double) * inum * umax * 3);
        ForceSr<double>::find_der_backward(grad_out, const_cast<double*>(grad_in), der, inum,
                                           const_cast<int*>(ilist), const_cast<int*>(numneigh),
                                           const_cast<int*>(firstneigh), nghost, umax);
    }
    std::free(der);
}

// virial[9]; der1/der2 [9, inum*umax] as the reference lays them out (may be null)
void ref_fvt_virial_f64(double* virial, double* der1, double* der2, int inum, const int* numneigh,
                        const double* rcs, int umax, const double* dei_drij)
{
    size_t nder = (size_t)9 * inum * umax;
    double* d1 = der1 ? der1 : (double*)std::malloc(sizeof(double) * nder);
    double* d2 = der2 ? der2 : (double*)std::malloc(sizeof(double) * nder);
    VirialSr<double>::find_val_der(virial, d1, d2, inum, const_cast<int*>(numneigh),
                                   const_cast<double*>(rcs), umax, const_cast<double*>(dei_drij));
    if (!der1) std::free(d1);
    if (!der2) std::free(d2);
}

}
