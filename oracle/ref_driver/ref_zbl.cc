// TEST INFRASTRUCTURE ONLY. extern "C" driver around the reference's PairZBL
// (REF_ROOT/source/descriptor/correction/include/zbl.h:331-393: add_atomic_energy_one,
// add_atomic_force_one, add_virial_one), built into oracle/_ref/libref_zbl.so.  The three member
// functions are the reference's; the loop that applies all three to every pair of a centre atom is
// this file's and mirrors the device composition (correction/gpu/include/zbl.cuh:422-500), because
// the reference's CPU GroupZBL::correct_efv has the force and virial calls commented out
// (zbl.h:523-526).
#include <cassert>      // zbl.h uses assert without including it
#include <cmath>
#include <cstddef>
#include "descriptor/correction/include/zbl.h"

using namespace ai2pot::correction;

extern "C" void ref_zbl_correct_f64(double* betot, double* bforce, double* bvirial, double rmax, double rmin,
                                    const double* cks, const double* dks, int ntypes, const int* type_map, int B,
                                    int P, int U, int nghost, const int* binum, const int* bilist,
                                    const int* bnumneigh, const int* bfirstneigh, const double* brcs,
                                    const int* btypes)
{
    const int NF = P + nghost;
    for (int b = 0; b < B; b++)
        for (int ii = 0; ii < binum[b]; ii++) {
            const size_t row = (size_t)b * P + ii;
            const int ci = bilist[row], ti = btypes[(size_t)b * NF + ci];
            for (int jj = 0; jj < bnumneigh[row]; jj++) {
                double v[3] = {brcs[(row * U + jj) * 3], brcs[(row * U + jj) * 3 + 1], brcs[(row * U + jj) * 3 + 2]};
                const double r = std::sqrt(v[0] * v[0] + v[1] * v[1] + v[2] * v[2]);
                if (r > rmax) continue;
                const int tj = btypes[(size_t)b * NF + bfirstneigh[row * U + jj]];
                PairZBL<double> pz(type_map[ti], type_map[tj], rmax, rmin,
                                   const_cast<double*>(&cks[(size_t)(ti * ntypes + tj) * 4]),
                                   const_cast<double*>(&dks[(size_t)(ti * ntypes + tj) * 4]));
                pz.add_atomic_energy_one(betot[b], r);
                pz.add_atomic_force_one(&bforce[((size_t)b * NF + ci) * 3], v);
                pz.add_virial_one(&bvirial[b * 9], v);
            }
        }
}

// GroupZBL::correct_e_sites (zbl.h:625-685) itself, structure by structure
extern "C" void ref_zbl_esites_f64(double* be_sites, double rmax, double rmin, const double* cks, const double* dks,
                                   int ntypes, const int* type_map, int B, int P, int U, int nghost, const int* binum,
                                   const int* bilist, const int* bnumneigh, const int* bfirstneigh, const double* brcs,
                                   const int* btypes)
{
    const int NF = P + nghost;
    GroupZBL<double> gz(ntypes, const_cast<int*>(type_map), const_cast<int*>(type_map), rmax, rmin,
                        const_cast<double*>(cks), const_cast<double*>(dks));
    for (int b = 0; b < B; b++)
        gz.correct_e_sites(be_sites + (size_t)b * P, binum[b], const_cast<int*>(bilist + (size_t)b * P),
                           const_cast<int*>(bnumneigh + (size_t)b * P), const_cast<int*>(bfirstneigh + (size_t)b * P * U),
                           (double (*)[3])const_cast<double*>(brcs + (size_t)b * P * U * 3),
                           const_cast<int*>(btypes + (size_t)b * NF), ntypes, const_cast<int*>(type_map), U, nghost);
}
