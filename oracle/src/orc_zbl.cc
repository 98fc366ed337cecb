// TEST INFRASTRUCTURE ONLY -- CPU restatement (fp64) of the reference's ZBL correction:
// pair formulas of source/descriptor/correction/include/zbl.h:262-395, composed per centre atom as
// correction/gpu/include/zbl.cuh:422-500 does (the reference's CPU composition, zbl.h:491-556, has
// its force and virial lines commented out, so the device code is the one that defines the result).
//
// Pinned by: the reference's own PairZBL member functions compiled from zbl.h
// (oracle/_ref/libref_zbl.so) pair by pair; finite differences of the energy for the force and the
// virial; switching-function end values (tests/test_pair_zbl.cc:75-77).
// Parity unpinned for the composition per centre atom (which atom receives the force, the halves):
// it is read off the device source, which cannot be compiled or run here, and no output of it
// ships with the reference; energy consistency (force = -dE/dx for a full list) is what checks it.
#include <cmath>
#include <cstddef>

extern "C" void orc_zbl_correct_f64(double* betot, double* bforce, double* bvirial, double rmax, double rmin,
                                    const double* cks, const double* dks, int ntypes, const int* type_map, int B,
                                    int P, int U, int nghost, const int* binum, const int* bilist,
                                    const int* bnumneigh, const int* bfirstneigh, const double* brcs,
                                    const int* btypes)
{
    const double kc = 14.399645;                                                // zbl.h:34
    const int NF = P + nghost;
    for (int b = 0; b < B; b++)
        for (int ii = 0; ii < binum[b]; ii++) {
            const size_t row = (size_t)b * P + ii;
            const int ci = bilist[row], ti = btypes[(size_t)b * NF + ci];
            const double Zi = type_map[ti];
            for (int jj = 0; jj < bnumneigh[row]; jj++) {
                const double* v = &brcs[(row * U + jj) * 3];
                const double r = std::sqrt(v[0] * v[0] + v[1] * v[1] + v[2] * v[2]);
                if (r > rmax) continue;                                         // zbl.cuh:455-456
                const int tj = btypes[(size_t)b * NF + bfirstneigh[row * U + jj]];
                const double Zj = type_map[tj];
                const double* ck = &cks[(size_t)(ti * ntypes + tj) * 4];
                const double* dk = &dks[(size_t)(ti * ntypes + tj) * 4];
                const double a = 0.46848 / (std::pow(Zi, 0.23) + std::pow(Zj, 0.23));   // zbl.h:291-318
                double phi = 0, dphi = 0;
                for (int k = 0; k < 4; k++) {
                    phi += ck[k] * std::exp(-dk[k] * r / a);
                    dphi += -ck[k] * dk[k] / a * std::exp(-dk[k] * r / a);
                }
                double sw = 1, dsw = 0;                                         // zbl.h:262-288
                if (r >= rmin) {
                    const double u = (r - rmin) / (rmax - rmin);
                    sw = u * u * u * (-6 * u * u + 15 * u - 10) + 1;
                    dsw = 1 / (rmax - rmin) * (-30 * u * u * u * u + 60 * u * u * u - 30 * u * u);
                }
                const double A = kc * Zi * Zj / r, dA = -kc * Zi * Zj / (r * r);
                const double dEdr = dA * phi * sw + A * dphi * sw + A * phi * dsw;
                if (betot) betot[b] += 0.5 * A * phi * sw;                      // zbl.h:331-339
                for (int c = 0; c < 3; c++) {
                    if (bforce) bforce[((size_t)b * NF + ci) * 3 + c] += dEdr * v[c] / r;            // zbl.h:343-365
                    if (bvirial)
                        for (int d = 0; d < 3; d++) bvirial[b * 9 + c * 3 + d] += -0.5 * v[c] * dEdr * v[d] / r;   // :369-393
                }
            }
        }
}

// Per-row ZBL energies added onto be_sites[B, P]: half of every pair energy of the row's centre atom
// (GroupZBL::correct_e_sites, zbl.h:625-685).  Pinned by that member function itself, compiled from the
// reference's header (oracle/_ref/libref_zbl.so), and by the sum rule against orc_zbl_correct_f64's energy.
extern "C" void orc_zbl_esites_f64(double* be_sites, double rmax, double rmin, const double* cks, const double* dks,
                                   int ntypes, const int* type_map, int B, int P, int U, int nghost, const int* binum,
                                   const int* bilist, const int* bnumneigh, const int* bfirstneigh, const double* brcs,
                                   const int* btypes)
{
    const double kc = 14.399645;                                                // zbl.h:34
    const int NF = P + nghost;
    for (int b = 0; b < B; b++)
        for (int ii = 0; ii < binum[b]; ii++) {
            const size_t row = (size_t)b * P + ii;
            const int ci = bilist[row], ti = btypes[(size_t)b * NF + ci];
            const double Zi = type_map[ti];
            for (int jj = 0; jj < bnumneigh[row]; jj++) {
                const double* v = &brcs[(row * U + jj) * 3];
                const double r = std::sqrt(v[0] * v[0] + v[1] * v[1] + v[2] * v[2]);
                if (r > rmax) continue;                                         // zbl.h:677-678
                const int tj = btypes[(size_t)b * NF + bfirstneigh[row * U + jj]];
                const double Zj = type_map[tj];
                const double* ck = &cks[(size_t)(ti * ntypes + tj) * 4];
                const double* dk = &dks[(size_t)(ti * ntypes + tj) * 4];
                const double a = 0.46848 / (std::pow(Zi, 0.23) + std::pow(Zj, 0.23));
                double phi = 0;
                for (int k = 0; k < 4; k++) phi += ck[k] * std::exp(-dk[k] * r / a);
                double sw = 1;
                if (r >= rmin) {
                    const double u = (r - rmin) / (rmax - rmin);
                    sw = u * u * u * (-6 * u * u + 15 * u - 10) + 1;
                }
                be_sites[row] += 0.5 * kc * Zi * Zj / r * phi * sw;             // zbl.h:331-339, 680
            }
        }
}
