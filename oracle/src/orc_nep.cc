// TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference's NEP energy / force /
// virial evaluation (radial + three-body angular descriptors, one tanh hidden layer per
// species).  Citations are to files under the reference's source/descriptor/nep/include.
// Written from the formulas, not the loop nest: the radial functions g_n(r) are contracted
// with the coefficients once per neighbour, and the solid harmonics are generated from a
// table of monomials with symbolic gradients (the reference spells every polynomial and
// gradient out by hand, nep_utilities.h:100-379).
//
// Pinned by: the compiled reference (oracle/_ref/libref_nep.so) in fp64 to 1e-12 on random
// and MoS2 inputs; the known answer E = 46.363417549065026 of the reference's own unit-test
// set-up (tests/test_nep.cc:100-255); central finite differences of E for forces and
// strain derivatives for the virial; the addition theorem (q_nl for two neighbours is a
// Legendre polynomial of the enclosed angle) in tests/test_oracle_nep.py.
#include <cmath>
#include <cstring>
#include <vector>

namespace {

// Three-body weights, nep_utilities.h:25-31.  The reference's array is a double array whose
// odd entries carry an `f` suffix; the same literals are kept so fp64 results agree.
const double C3B[24] = {
    0.238732414637843, 0.119366207318922f, 0.119366207318922f, 0.099471839432435f,
    0.596831036594608, 0.596831036594608f, 0.149207759148652f, 0.149207759148652f,
    0.139260575205408, 0.104445431404056f, 0.104445431404056f, 1.044454314040563f,
    1.044454314040563, 0.174075719006761f, 0.174075719006761f, 0.011190581936149f,
    0.223811638722978, 0.223811638722978f, 0.111905819361489f, 0.111905819361489f,
    1.566681471060845, 1.566681471060845f, 0.195835183882606f, 0.195835183882606f};

// Four- and five-body weights: the constants of the reference's unfinished draft
// (source/descriptor/ace/include/nep_descriptor.h:43-54; its accum_4b_descriptor_one / accum_5b_descriptor_one are
// declared at :109-111 and never defined).  The invariants they weight are restated below from the published NEP
// formulation; PARITY UNPINNED: no reference code evaluates them.  Pinned instead by rotation invariance,
// finite differences and the reduction to the three-body model (tests/test_oracle_nep_manybody.py).
const double C4B[5] = {-0.007499480826664, -0.134990654879954, 0.067495327439977, 0.404971964639861,
                       -0.809943929279723};
const double C5B[3] = {0.026596810706114, 0.053193621412227, 0.026596810706114};

// Un-normalised real solid harmonics b_lm (nep_utilities.h:110-203) as polynomials
// sum_t c_t x^a y^b z^c r^(2d), listed per flat index l*l-1+mp.
struct Term { double c; int a, b, c_, d; };
struct Poly { int nterm; Term t[4]; };
const Poly BLM[24] = {
    // l = 1: z, x, y
    {1, {{1, 0, 0, 1, 0}}}, {1, {{1, 1, 0, 0, 0}}}, {1, {{1, 0, 1, 0, 0}}},
    // l = 2: 3z^2 - r^2, xz, yz, x^2 - y^2, 2xy
    {2, {{3, 0, 0, 2, 0}, {-1, 0, 0, 0, 1}}}, {1, {{1, 1, 0, 1, 0}}}, {1, {{1, 0, 1, 1, 0}}},
    {2, {{1, 2, 0, 0, 0}, {-1, 0, 2, 0, 0}}}, {1, {{2, 1, 1, 0, 0}}},
    // l = 3
    {2, {{5, 0, 0, 3, 0}, {-3, 0, 0, 1, 1}}},                   // (5z^2 - 3r^2) z
    {2, {{5, 1, 0, 2, 0}, {-1, 1, 0, 0, 1}}},                   // (5z^2 - r^2) x
    {2, {{5, 0, 1, 2, 0}, {-1, 0, 1, 0, 1}}},                   // (5z^2 - r^2) y
    {2, {{1, 2, 0, 1, 0}, {-1, 0, 2, 1, 0}}},                   // (x^2 - y^2) z
    {1, {{2, 1, 1, 1, 0}}},                                     // 2xyz
    {2, {{1, 3, 0, 0, 0}, {-3, 1, 2, 0, 0}}},                   // (x^2 - 3y^2) x
    {2, {{3, 2, 1, 0, 0}, {-1, 0, 3, 0, 0}}},                   // (3x^2 - y^2) y
    // l = 4
    {3, {{35, 0, 0, 4, 0}, {-30, 0, 0, 2, 1}, {3, 0, 0, 0, 2}}},  // (35z^2 - 30r^2) z^2 + 3r^4
    {2, {{7, 1, 0, 3, 0}, {-3, 1, 0, 1, 1}}},                   // (7z^2 - 3r^2) xz
    {2, {{7, 0, 1, 3, 0}, {-3, 0, 1, 1, 1}}},                   // (7z^2 - 3r^2) yz
    {4, {{7, 2, 0, 2, 0}, {-7, 0, 2, 2, 0}, {-1, 2, 0, 0, 1}, {1, 0, 2, 0, 1}}},  // (7z^2-r^2)(x^2-y^2)
    {2, {{14, 1, 1, 2, 0}, {-2, 1, 1, 0, 1}}},                  // (7z^2 - r^2) 2xy
    {2, {{1, 3, 0, 1, 0}, {-3, 1, 2, 1, 0}}},                   // (x^2 - 3y^2) xz
    {2, {{3, 2, 1, 1, 0}, {-1, 0, 3, 1, 0}}},                   // (3x^2 - y^2) yz
    {3, {{1, 4, 0, 0, 0}, {-6, 2, 2, 0, 0}, {1, 0, 4, 0, 0}}},  // (x^2-y^2)^2 - 4x^2y^2
    {2, {{4, 3, 1, 0, 0}, {-4, 1, 3, 0, 0}}},                   // 4(x^2 - y^2) xy
};

inline double ipow(double v, int n)
{
    double o = 1;
    for (int i = 0; i < n; i++) o *= v;
    return o;
}

// The reference differentiates b_lm with r held as an independent symbol only in the sense
// that its listed gradients already include d(r^2)/dx = 2x (nep_utilities.h:206-379), i.e.
// they are the full Cartesian gradients of the polynomial in (x, y, z).
void blm_val_grad(int idx, const double* v, double r, double& val, double* grad)
{
    const Poly& p = BLM[idx];
    val = 0;
    grad[0] = grad[1] = grad[2] = 0;
    const double r2 = r * r;
    for (int t = 0; t < p.nterm; t++) {
        const Term& m = p.t[t];
        const int e[3] = {m.a, m.b, m.c_};
        double mono = ipow(v[0], e[0]) * ipow(v[1], e[1]) * ipow(v[2], e[2]);
        double rr = ipow(r2, m.d);
        val += m.c * mono * rr;
        for (int a = 0; a < 3; a++) {
            double g = 0;
            if (e[a] > 0) {
                int ee[3] = {e[0], e[1], e[2]};
                ee[a]--;
                g += e[a] * ipow(v[0], ee[0]) * ipow(v[1], ee[1]) * ipow(v[2], ee[2]) * rr;
            }
            if (m.d > 0) g += mono * m.d * ipow(r2, m.d - 1) * 2 * v[a];
            grad[a] += m.c * g;
        }
    }
}

// f_k(r) = 1/2 (T_k(x) + 1) * fc(r), x = 2 (r/rc - 1)^2 - 1, fc = 1/2 (1 + cos(pi r / rc))
// for r <= rc (basis.h:137-158, 300-332, 519-530), with d f_k / d r.
void radial_basis(int K, double rc, double r, double* f, double* df)
{
    double x = 2 * (r / rc - 1) * (r / rc - 1) - 1;
    double dxdr = 4.0 / rc * (r / rc - 1);
    double fc = 0, dfc = 0;
    if (r <= rc) {
        fc = 0.5 * (1 + std::cos(M_PI * r / rc));
        dfc = -0.5 * std::sin(M_PI * r / rc) * M_PI / rc;
    }
    std::vector<double> T(K), dT(K);
    for (int k = 0; k < K; k++) {
        if (k == 0) { T[k] = 1; dT[k] = 0; }
        else if (k == 1) { T[k] = x; dT[k] = 1; }
        else {
            T[k] = 2 * x * T[k - 1] - T[k - 2];
            dT[k] = 2 * T[k - 1] + 2 * x * dT[k - 1] - dT[k - 2];
        }
        double v = (T[k] + 1) * 0.5, dv = dT[k] * 0.5 * dxdr;
        f[k] = fc * v;
        df[k] = dfc * v + fc * dv;
    }
}

struct Model {
    int K, n_r, n_a, l_max, H, ntypes;
    const double *coeffs, *w0, *b0, *w1, *bias, *q_scaler;
    double rr, ra;
    int mb4 = 0, mb5 = 0;       // extension: a four-body (l = 2) and a five-body (l = 1) invariant per angular channel
    int num_l() const { return l_max + mb4 + mb5; }
    int D() const { return l_max == 0 ? n_r : n_r + n_a * num_l(); }
    int nlm() const { return l_max * l_max + 2 * l_max; }
};

// q_4b(s) of the l = 2 moments s[3..7] and q_5b(s) of the l = 1 moments s[0..2] of one channel, with gradients
inline double q4b_of(const double* s, double* d)
{
    const double s3 = s[3], s4 = s[4], s5 = s[5], s6 = s[6], s7 = s[7];
    if (d) {
        d[3] = 3 * C4B[0] * s3 * s3 + C4B[1] * (s4 * s4 + s5 * s5) + C4B[2] * (s6 * s6 + s7 * s7);
        d[4] = 2 * C4B[1] * s3 * s4 - 2 * C4B[3] * s6 * s4 + C4B[4] * s5 * s7;
        d[5] = 2 * C4B[1] * s3 * s5 + 2 * C4B[3] * s6 * s5 + C4B[4] * s4 * s7;
        d[6] = 2 * C4B[2] * s3 * s6 + C4B[3] * (s5 * s5 - s4 * s4);
        d[7] = 2 * C4B[2] * s3 * s7 + C4B[4] * s4 * s5;
    }
    return C4B[0] * s3 * s3 * s3 + C4B[1] * s3 * (s4 * s4 + s5 * s5) + C4B[2] * s3 * (s6 * s6 + s7 * s7) +
           C4B[3] * s6 * (s5 * s5 - s4 * s4) + C4B[4] * s4 * s5 * s7;
}
inline double q5b_of(const double* s, double* d)
{
    const double a = s[0] * s[0], b = s[1] * s[1] + s[2] * s[2];
    if (d) {
        d[0] = 4 * C5B[0] * a * s[0] + 2 * C5B[1] * s[0] * b;
        d[1] = 2 * C5B[1] * a * s[1] + 4 * C5B[2] * b * s[1];
        d[2] = 2 * C5B[1] * a * s[2] + 4 * C5B[2] * b * s[2];
    }
    return C5B[0] * a * a + C5B[1] * a * b + C5B[2] * b * b;
}

// One centre atom: descriptors q[D], moments S[n_a*nlm] (nepBasis.h:57-196).
void descriptors_of(const Model& m, int ti, int nn, const int* first, const double* rcs,
                    const int* types, double* q, double* S)
{
    const int nlm = m.nlm(), D = m.D();
    std::fill(q, q + D, 0.0);
    std::fill(S, S + m.n_a * nlm, 0.0);
    std::vector<double> fR(m.K), dfR(m.K), fA(m.K), dfA(m.K);
    for (int jj = 0; jj < nn; jj++) {
        const double* v = &rcs[jj * 3];
        double r = std::sqrt(v[0] * v[0] + v[1] * v[1] + v[2] * v[2]);
        if (r > m.rr) continue;                              // nepBasis.h:106
        int tj = types[first[jj]];
        const double* c = &m.coeffs[(size_t)(ti * m.ntypes + tj) * (m.n_r + m.n_a) * m.K];
        radial_basis(m.K, m.rr, r, fR.data(), dfR.data());
        for (int n = 0; n < m.n_r; n++)
            for (int k = 0; k < m.K; k++) q[n] += c[n * m.K + k] * fR[k];
        if (m.l_max == 0 || r > m.ra) continue;              // nepBasis.h:135
        radial_basis(m.K, m.ra, r, fA.data(), dfA.data());
        for (int n = 0; n < m.n_a; n++) {
            double g = 0;
            for (int k = 0; k < m.K; k++) g += c[(m.n_r + n) * m.K + k] * fA[k];
            for (int l = 1; l <= m.l_max; l++)
                for (int mp = 0; mp < 2 * l + 1; mp++) {
                    double bv, bg[3];
                    blm_val_grad(l * l - 1 + mp, v, r, bv, bg);
                    S[n * nlm + l * l - 1 + mp] += g * bv / ipow(r, l);
                }
        }
    }
    for (int n = 0; n < m.n_a && m.l_max > 0; n++)           // nepBasis.h:174-190
        for (int l = 1; l <= m.l_max; l++)
            for (int mp = 0; mp < 2 * l + 1; mp++) {
                double s = S[n * nlm + l * l - 1 + mp];
                q[m.n_r + n * m.num_l() + (l - 1)] += (mp == 0 ? 1 : 2) * C3B[l * l - 1 + mp] * s * s;
            }
    for (int n = 0; n < m.n_a && m.l_max > 0; n++) {
        if (m.mb4) q[m.n_r + n * m.num_l() + m.l_max] = q4b_of(&S[n * nlm], nullptr);
        if (m.mb5) q[m.n_r + n * m.num_l() + m.l_max + m.mb4] = q5b_of(&S[n * nlm], nullptr);
    }
}

template <typename T>
void efv_one(const Model& m, double& etot, double* force, double* virial, int inum, const int* ilist,
             const int* numneigh, const int* firstneigh, const T* rcsT, const int* types, int U)
{
    const int D = m.D(), nlm = m.nlm();
    std::vector<double> q(D), S(m.n_a * nlm + 1), dEdq(D), dEdS(m.n_a * nlm + 1);
    std::vector<double> fR(m.K), dfR(m.K), fA(m.K), dfA(m.K), rcs((size_t)U * 3);
    for (int ii = 0; ii < inum; ii++) {
        const int ci = ilist[ii], ti = types[ci], nn = numneigh[ii];
        const int* first = &firstneigh[(size_t)ii * U];
        for (int j = 0; j < nn * 3; j++) rcs[j] = rcsT[(size_t)ii * U * 3 + j];
        descriptors_of(m, ti, nn, first, rcs.data(), types, q.data(), S.data());

        // hidden layer, nep.h:415-447
        const double* W0 = &m.w0[(size_t)ti * m.H * D];
        double e = m.bias[ti];
        std::fill(dEdq.begin(), dEdq.end(), 0.0);
        for (int p = 0; p < m.H; p++) {
            double h = m.b0[ti * m.H + p];
            for (int k = 0; k < D; k++) h += W0[p * D + k] * q[k] / m.q_scaler[k];
            double t = std::tanh(h);
            e += m.w1[ti * m.H + p] * t;
            for (int k = 0; k < D; k++)
                dEdq[k] += m.w1[ti * m.H + p] * (1 - t * t) * W0[p * D + k] / m.q_scaler[k];
        }
        etot += e;
        // dE/dS, nep.h:450-466
        for (int n = 0; n < m.n_a && m.l_max > 0; n++)
            for (int l = 1; l <= m.l_max; l++)
                for (int mp = 0; mp < 2 * l + 1; mp++) {
                    int is = n * nlm + l * l - 1 + mp;
                    dEdS[is] = dEdq[m.n_r + n * m.num_l() + l - 1] * (mp == 0 ? 1 : 2) * 2 *
                               C3B[l * l - 1 + mp] * S[is];
                }
        for (int n = 0; n < m.n_a && m.l_max > 0; n++) {
            double d[8];
            if (m.mb4) {
                q4b_of(&S[n * nlm], d);
                for (int k = 3; k < 8; k++) dEdS[n * nlm + k] += dEdq[m.n_r + n * m.num_l() + m.l_max] * d[k];
            }
            if (m.mb5) {
                q5b_of(&S[n * nlm], d);
                for (int k = 0; k < 3; k++) dEdS[n * nlm + k] += dEdq[m.n_r + n * m.num_l() + m.l_max + m.mb4] * d[k];
            }
        }
        // pair derivatives and scatter, nep.h:468-515
        for (int jj = 0; jj < nn; jj++) {
            const double* v = &rcs[jj * 3];
            double r = std::sqrt(v[0] * v[0] + v[1] * v[1] + v[2] * v[2]);
            if (r > m.rr) continue;
            int nj = first[jj], tj = types[nj];
            const double* c = &m.coeffs[(size_t)(ti * m.ntypes + tj) * (m.n_r + m.n_a) * m.K];
            double g[3] = {0, 0, 0};
            radial_basis(m.K, m.rr, r, fR.data(), dfR.data());
            for (int n = 0; n < m.n_r; n++) {
                double dg = 0;
                for (int k = 0; k < m.K; k++) dg += c[n * m.K + k] * dfR[k];
                for (int a = 0; a < 3; a++) g[a] += dEdq[n] * dg * v[a] / r;
            }
            if (m.l_max > 0 && r <= m.ra) {
                radial_basis(m.K, m.ra, r, fA.data(), dfA.data());
                for (int n = 0; n < m.n_a; n++) {
                    double gn = 0, dgn = 0;
                    for (int k = 0; k < m.K; k++) {
                        gn += c[(m.n_r + n) * m.K + k] * fA[k];
                        dgn += c[(m.n_r + n) * m.K + k] * dfA[k];
                    }
                    for (int l = 1; l <= m.l_max; l++) {
                        double rl = ipow(r, l);
                        for (int mp = 0; mp < 2 * l + 1; mp++) {
                            double bv, bg[3];
                            blm_val_grad(l * l - 1 + mp, v, r, bv, bg);
                            double w = dEdS[n * nlm + l * l - 1 + mp];
                            for (int a = 0; a < 3; a++)
                                g[a] += w * (dgn * v[a] / r * bv / rl + gn * bg[a] / rl -
                                             gn * bv * l / (rl * r) * v[a] / r);
                        }
                    }
                }
            }
            for (int a = 0; a < 3; a++) {
                force[ci * 3 + a] += g[a];
                force[nj * 3 + a] -= g[a];
                for (int bb = 0; bb < 3; bb++) virial[a * 3 + bb] -= g[a] * v[bb];
            }
        }
    }
}

template <typename T>
void efv(T* betot, T* bforce, T* bvirial, int K, int n_r, int n_a, int l_max, int H, const T* coeffs,
         const T* w0, const T* b0, const T* w1, const T* bias, int B, int P, const int* binum,
         const int* bilist, const int* bnumneigh, const int* bfirstneigh, const T* brcs,
         const int* btypes, int ntypes, int U, int nghost, double rr, double ra, const T* q_scaler, int mb4 = 0,
         int mb5 = 0)
{
    const int D = l_max == 0 ? n_r : n_r + n_a * (l_max + mb4 + mb5);
    auto up = [](const T* p, size_t n) { return std::vector<double>(p, p + n); };
    std::vector<double> c = up(coeffs, (size_t)ntypes * ntypes * (n_r + n_a) * K),
                        W0 = up(w0, (size_t)ntypes * H * D), B0 = up(b0, (size_t)ntypes * H),
                        W1 = up(w1, (size_t)ntypes * H), bi = up(bias, ntypes), qs = up(q_scaler, D);
    // cutoffs are rounded to T first, as the reference's launcher receives them in T
    Model m{K, n_r, n_a, l_max, H, ntypes, c.data(), W0.data(), B0.data(), W1.data(), bi.data(),
            qs.data(), (double)(T)rr, (double)(T)ra};
    m.mb4 = mb4; m.mb5 = mb5;
    for (int b = 0; b < B; b++) {
        double e = 0, v[9] = {0};
        std::vector<double> f((size_t)(P + nghost) * 3, 0.0);
        efv_one<T>(m, e, f.data(), v, binum[b], &bilist[(size_t)b * P], &bnumneigh[(size_t)b * P],
                   &bfirstneigh[(size_t)b * P * U], &brcs[(size_t)b * P * U * 3],
                   &btypes[(size_t)b * (P + nghost)], U);
        betot[b] = (T)e;
        for (size_t i = 0; i < f.size(); i++) bforce[(size_t)b * (P + nghost) * 3 + i] = (T)f[i];
        for (int i = 0; i < 9; i++) bvirial[b * 9 + i] = (T)v[i];
    }
}

template <typename T>
void desc(T* bdesc, int K, int n_r, int n_a, int l_max, const T* coeffs, int B, int P,
          const int* binum, const int* bilist, const int* bnumneigh, const int* bfirstneigh,
          const T* brcs, const int* btypes, int ntypes, int U, double rr, double ra, int mb4 = 0, int mb5 = 0)
{
    const int D = l_max == 0 ? n_r : n_r + n_a * (l_max + mb4 + mb5);
    std::vector<double> c(coeffs, coeffs + (size_t)ntypes * ntypes * (n_r + n_a) * K);
    Model m{K, n_r, n_a, l_max, 0, ntypes, c.data(), nullptr, nullptr, nullptr, nullptr, nullptr,
            (double)(T)rr, (double)(T)ra};
    m.mb4 = mb4; m.mb5 = mb5;
    std::vector<double> q(D), S(n_a * m.nlm() + 1), rcs((size_t)U * 3);
    for (int b = 0; b < B; b++)
        for (int ii = 0; ii < binum[b]; ii++) {
            const size_t row = (size_t)b * P + ii;
            const int* types = &btypes[(size_t)b * P];
            int nn = bnumneigh[row];
            for (int j = 0; j < nn * 3; j++) rcs[j] = brcs[row * U * 3 + j];
            descriptors_of(m, types[bilist[row]], nn, &bfirstneigh[row * U], rcs.data(), types,
                           q.data(), S.data());
            // the reference writes row ii, not row ilist[ii] (nep.h:533-, find_descriptors)
            for (int k = 0; k < D; k++) bdesc[row * D + k] = (T)q[k];
        }
}

}  // namespace

#define ARGS_EFV(T) T* betot, T* bforce, T* bvirial, int K, int n_r, int n_a, int l_max, int H, \
    const T* coeffs, const T* w0, const T* b0, const T* w1, const T* bias, int B, int P, \
    const int* binum, const int* bilist, const int* bnumneigh, const int* bfirstneigh, \
    const T* brcs, const int* btypes, int ntypes, const int* type_map, int U, int nghost, \
    double rr, double ra, const T* q_scaler
#define PASS_EFV betot, bforce, bvirial, K, n_r, n_a, l_max, H, coeffs, w0, b0, w1, bias, B, P, \
    binum, bilist, bnumneigh, bfirstneigh, brcs, btypes, ntypes, U, nghost, rr, ra, q_scaler
#define ARGS_DESC(T) T* bdesc, int K, int n_r, int n_a, int l_max, const T* coeffs, int B, int P, \
    const int* binum, const int* bilist, const int* bnumneigh, const int* bfirstneigh, \
    const T* brcs, const int* btypes, int ntypes, const int* type_map, int U, int nghost, \
    double rr, double ra
#define PASS_DESC bdesc, K, n_r, n_a, l_max, coeffs, B, P, binum, bilist, bnumneigh, bfirstneigh, \
    brcs, btypes, ntypes, U, rr, ra

// The fp32 entry points evaluate in double on the fp32 inputs and round the results: they
// check a fp32 implementation against the exactly-rounded answer rather than against the
// reference's own fp32 rounding noise.
extern "C" {
void orc_nep_efv_f32(ARGS_EFV(float)) { efv<float>(PASS_EFV); }
void orc_nep_efv_f64(ARGS_EFV(double)) { efv<double>(PASS_EFV); }
void orc_nep_desc_f32(ARGS_DESC(float)) { desc<float>(PASS_DESC); }
void orc_nep_desc_f64(ARGS_DESC(double)) { desc<double>(PASS_DESC); }
// the extension with four- and five-body invariants (mb4, mb5 = 0 or 1); parity unpinned, see C4B above
void orc_nep_efv_mb_f32(ARGS_EFV(float), int mb4, int mb5) { efv<float>(PASS_EFV, mb4, mb5); }
void orc_nep_efv_mb_f64(ARGS_EFV(double), int mb4, int mb5) { efv<double>(PASS_EFV, mb4, mb5); }
void orc_nep_desc_mb_f32(ARGS_DESC(float), int mb4, int mb5) { desc<float>(PASS_DESC, mb4, mb5); }
void orc_nep_desc_mb_f64(ARGS_DESC(double), int mb4, int mb5) { desc<double>(PASS_DESC, mb4, mb5); }
}
