// TEST INFRASTRUCTURE ONLY -- CPU restatement (fp64) of the reference's linear Moment
// Tensor Potential: energy / force / virial and one training-loss step (forward loss,
// RMSEs and the per-structure gradients w.r.t. coeffs, linear_coeffs and type_bias).
// Citations are to files under the reference's source/descriptor/mtpr/include.
//
// The E/F/V part follows the reference's formulas (mtpBasis.h:400-534, linearMtp.h:190-352).
// The loss gradient is NOT the reference's hand-derived tangent/adjoint sweeps
// (linearMtpLoss.h:212-569): it is obtained here by forward-mode differentiation of the
// E/F/V evaluation itself with dual numbers, one parameter direction at a time, which is
// slow but independent, so an error in either derivation shows up as a mismatch.
//
// Pinned by: the compiled reference (oracle/_ref/libref_mtpr.so) to 1e-12 relative on the
// test fixtures; the reference unit test's known answer E = -0.938157350795572
// (tests/test_linearMtp.cc, efv_force_accuracy set-up); finite differences of E; switch
// function end values (tests/test_basis.cc:106-111); linearity of E in linear_coeffs.
//
// Also here, each with its own citations below: site energies / scalar moments and their
// gradient (pinned by the reference's committed outputs, the sum rule and the linear read-out);
// the backward of the legacy basis operator (reference outputs, central differences);
// the normal equations of the linear parameters and the Gram-Schmidt of the radial functions
// (reference outputs; rebuilt independently from one-hot E/F/V calls); the neural-network MTP
// (source/descriptor/nnmtp): E/F/V and site energies (reference outputs, finite differences, the
// linear limit of a small network), its training-loss gradient and site-energy gradient by
// forward-mode AD.  For the last two the reference's hand-derived backward is NOT reproduced
// by this file: it omits terms (loss: d/dcoeffs, d/dw0 of the force and virial parts) or
// mis-assigns rows (site energies: w0 / w1 for several species); the AD results are pinned by
// finite differences and by the reference where its formulas are complete (w1, type_bias,
// energy-only loss, one species).
#include <algorithm>
#include <cmath>
#include <cstring>
#include <type_traits>
#include <vector>

namespace {

// minimal dual number: value + one directional derivative
struct Dual {
    double v, d;
    Dual(double v_ = 0, double d_ = 0) : v(v_), d(d_) {}
};
inline Dual operator+(Dual a, Dual b) { return {a.v + b.v, a.d + b.d}; }
inline Dual operator-(Dual a, Dual b) { return {a.v - b.v, a.d - b.d}; }
inline Dual operator*(Dual a, Dual b) { return {a.v * b.v, a.d * b.v + a.v * b.d}; }
inline Dual operator/(Dual a, Dual b) { return {a.v / b.v, (a.d * b.v - a.v * b.d) / (b.v * b.v)}; }
inline Dual& operator+=(Dual& a, Dual b) { a = a + b; return a; }
inline Dual& operator-=(Dual& a, Dual b) { a = a - b; return a; }
inline double val(double x) { return x; }
inline double val(Dual x) { return x.v; }

struct Tables {
    int n_moms, n_basic, n_times, n_scalar, nmus;
    const int *basic, *times, *mapping;
};

// Read-out of the neural-network MTP (source/descriptor/nnmtp/include/nnMtp.h:470-507): one tanh
// layer per centre species on the shifted and scaled scalar moments, no hidden bias.
template <typename S>
struct NNReadout {
    int H;
    const S *w0, *w1;                  // w0[ntypes, H, n_scalar], w1[ntypes, H]
    const double* shift;               // [n_scalar]
};
// nnMtpUtils.h:54-71: tanh from exponentials
inline double tanh_exp(double h) { return (std::exp(h) - std::exp(-h)) / (std::exp(h) + std::exp(-h)); }
inline Dual tanh_exp(Dual h)
{
    const double th = tanh_exp(h.v);
    return {th, (1 - th * th) * h.d};
}

// f_k(r) = scaling * s(u) * T_k(x) and its r-derivative (basis.h:154-196, 351-381, 620-637)
void radial_basis(int K, double rmax, double rmin, double scaling, double r, double* f, double* df)
{
    double x = (2 * r - (rmax + rmin)) / (rmax - rmin);
    double dx = 2 / (rmax - rmin);
    double u = (r - rmin) / (rmax - rmin);
    double s = 0, ds = 0;
    if (r >= rmin && r < rmax) {
        s = u * u * u * (-6 * u * u + 15 * u - 10) + 1;
        ds = 1 / (rmax - rmin) * (-30 * u * u * u * u + 60 * u * u * u - 30 * u * u);
    }
    std::vector<double> T(K), dT(K);
    for (int k = 0; k < K; k++) {
        if (k == 0) { T[k] = 1; dT[k] = 0; }
        else if (k == 1) { T[k] = x; dT[k] = 1; }
        else {
            T[k] = 2 * x * T[k - 1] - T[k - 2];
            dT[k] = 2 * T[k - 1] + 2 * x * dT[k - 1] - dT[k - 2];
        }
        f[k] = scaling * s * T[k];
        df[k] = scaling * (ds * T[k] + s * dT[k] * dx);
    }
}

// E/F/V of one structure, generic in the scalar type of the parameters (double or Dual).
template <typename S>
void efv_one(S& etot, S* force, S* virial, int K, double scaling, const S* coeffs, const S* lin,
             const S* bias, const Tables& t, int inum, const int* ilist, const int* numneigh,
             const int* firstneigh, const double* rcs, const int* types, int ntypes, int U,
             int nforce, double rmax, double rmin, const double* q_scaler, S* e_sites = nullptr,
             S* desc = nullptr, const NNReadout<S>* net = nullptr)
{
    etot = S(0);
    for (int i = 0; i < nforce * 3; i++) force[i] = S(0);   // linearMtp.h:228-230
    for (int i = 0; i < 9; i++) virial[i] = S(0);
    int kmax = 0;
    for (int i = 0; i < t.n_basic; i++) {
        int k = t.basic[i * 4 + 1] + t.basic[i * 4 + 2] + t.basic[i * 4 + 3];
        if (k > kmax) kmax = k;
    }
    std::vector<S> M(t.n_moms), adj(t.n_moms), g(K * t.nmus), dg(K * t.nmus);
    std::vector<double> f(K), df(K), pw((kmax + 1) * 3), rp(kmax + 1);
    for (int ii = 0; ii < inum; ii++) {
        const int ci = ilist[ii], ti = types[ci], nn = numneigh[ii];
        std::fill(M.begin(), M.end(), S(0));
        // basic moments, mtpBasis.h:449-519
        for (int jj = 0; jj < nn; jj++) {
            const double* v = &rcs[((size_t)ii * U + jj) * 3];
            double r = std::sqrt(v[0] * v[0] + v[1] * v[1] + v[2] * v[2]);
            if (r > rmax) continue;
            int tj = types[firstneigh[(size_t)ii * U + jj]];
            radial_basis(K, rmax, rmin, scaling, r, f.data(), df.data());
            rp[0] = 1; pw[0] = pw[1] = pw[2] = 1;
            for (int k = 1; k <= kmax; k++) {
                rp[k] = rp[k - 1] * r;
                for (int a = 0; a < 3; a++) pw[k * 3 + a] = pw[(k - 1) * 3 + a] * v[a];
            }
            const S* c = &coeffs[(size_t)(ti * ntypes + tj) * t.nmus * K];
            for (int mu = 0; mu < t.nmus; mu++) {
                S s(0);
                for (int k = 0; k < K; k++) s += c[mu * K + k] * S(f[k]);
                g[mu] = s;
            }
            for (int i = 0; i < t.n_basic; i++) {
                const int* b = &t.basic[i * 4];
                int k = b[1] + b[2] + b[3];
                double ang = pw[b[1] * 3 + 0] * pw[b[2] * 3 + 1] * pw[b[3] * 3 + 2] / rp[k];
                M[i] += g[b[0]] * S(ang);
            }
        }
        for (int i = 0; i < t.n_times; i++) {                 // mtpBasis.h:522-528
            const int* q = &t.times[i * 4];
            M[q[3]] += S((double)q[2]) * M[q[0]] * M[q[1]];
        }
        S e = bias[ti];                                        // linearMtp.h:281-285
        std::fill(adj.begin(), adj.end(), S(0));               // linearMtp.h:292-306
        if (net) {                                             // nnMtp.h:470-507
            const S* w0 = net->w0 + (size_t)ti * net->H * t.n_scalar;
            const S* w1 = net->w1 + (size_t)ti * net->H;
            for (int p = 0; p < net->H; p++) {
                S h(0);
                for (int s = 0; s < t.n_scalar; s++)
                    h += w0[p * t.n_scalar + s] * (M[t.mapping[s]] - S(net->shift[s])) / S(q_scaler[s]);
                const S th = tanh_exp(h);
                e += w1[p] * th;
                for (int s = 0; s < t.n_scalar; s++)
                    adj[t.mapping[s]] += w1[p] * (S(1) - th * th) * w0[p * t.n_scalar + s] / S(q_scaler[s]);
            }
        } else {
            for (int s = 0; s < t.n_scalar; s++) e += lin[s] * M[t.mapping[s]] / S(q_scaler[s]);
            for (int s = 0; s < t.n_scalar; s++) adj[t.mapping[s]] = lin[s] / S(q_scaler[s]);
        }
        etot += e;
        if (e_sites) e_sites[ii] = e;                          // linearMtp.h:594-599 (row order)
        if (desc)                                              // linearMtp.h:884-885 (unscaled moments)
            for (int s = 0; s < t.n_scalar; s++) desc[(size_t)ii * t.n_scalar + s] = M[t.mapping[s]];
        for (int i = t.n_times - 1; i >= 0; i--) {
            const int* q = &t.times[i * 4];
            S w = adj[q[3]] * S((double)q[2]);
            adj[q[1]] += w * M[q[0]];
            adj[q[0]] += w * M[q[1]];
        }
        // pair derivative and scatter, linearMtp.h:308-342
        for (int jj = 0; jj < nn; jj++) {
            const double* v = &rcs[((size_t)ii * U + jj) * 3];
            double r = std::sqrt(v[0] * v[0] + v[1] * v[1] + v[2] * v[2]);
            if (r > rmax) continue;
            int nj = firstneigh[(size_t)ii * U + jj], tj = types[nj];
            radial_basis(K, rmax, rmin, scaling, r, f.data(), df.data());
            rp[0] = 1; pw[0] = pw[1] = pw[2] = 1;
            for (int k = 1; k <= kmax; k++) {
                rp[k] = rp[k - 1] * r;
                for (int a = 0; a < 3; a++) pw[k * 3 + a] = pw[(k - 1) * 3 + a] * v[a];
            }
            const S* c = &coeffs[(size_t)(ti * ntypes + tj) * t.nmus * K];
            for (int mu = 0; mu < t.nmus; mu++) {
                S s(0), ds(0);
                for (int k = 0; k < K; k++) {
                    s += c[mu * K + k] * S(f[k]);
                    ds += c[mu * K + k] * S(df[k]);
                }
                g[mu] = s;
                dg[mu] = ds;
            }
            S gr[3] = {S(0), S(0), S(0)};
            for (int i = 0; i < t.n_basic; i++) {
                const int* b = &t.basic[i * 4];
                int k = b[1] + b[2] + b[3];
                double mono = pw[b[1] * 3 + 0] * pw[b[2] * 3 + 1] * pw[b[3] * 3 + 2];
                double ang = mono / rp[k];
                for (int a = 0; a < 3; a++) {
                    double dmono = 0;
                    if (b[1 + a] > 0) {
                        int e[3] = {b[1], b[2], b[3]};
                        e[a]--;
                        dmono = b[1 + a] * pw[e[0] * 3 + 0] * pw[e[1] * 3 + 1] * pw[e[2] * 3 + 2];
                    }
                    double dang = dmono / rp[k] - k * mono / (rp[k] * r * r) * v[a];
                    gr[a] += adj[i] * (dg[b[0]] * S(ang * v[a] / r) + g[b[0]] * S(dang));
                }
            }
            for (int a = 0; a < 3; a++) {
                force[ci * 3 + a] += gr[a];
                force[nj * 3 + a] -= gr[a];
                for (int bb = 0; bb < 3; bb++) virial[a * 3 + bb] -= gr[a] * S(v[bb]);
            }
        }
    }
}

// per-structure loss, linearMtpLoss.h:138-176
template <typename S>
S loss_one(int inum, const int* ilist, double e_w, double f_w, double v_w, S etot, double e_dft,
           const S* force, const double* f_dft, const S* virial, const double* v_dft)
{
    S fl(0), vl(0);
    for (int ii = 0; ii < inum; ii++)
        for (int a = 0; a < 3; a++) {
            S d = force[ilist[ii] * 3 + a] - S(f_dft[ilist[ii] * 3 + a]);
            fl += d * d;
        }
    for (int i = 0; i < 9; i++) {
        S d = virial[i] - S(v_dft[i]);
        vl += d * d;
    }
    S de = etot - S(e_dft);
    return S(f_w / (3 * inum)) * fl + S(v_w / (9 * inum)) * vl + S(e_w / inum) * de * de;
}

}  // namespace

#define MTP_MODEL_ARGS int K, double scaling, const double* coeffs, const double* lin, \
    const double* bias, int n_moms, int n_basic, const int* basic, int n_times, const int* times, \
    int n_scalar, const int* mapping, int nmus
#define MTP_LIST_ARGS int B, int P, const int* binum, const int* bilist, const int* bnumneigh, \
    const int* bfirstneigh, const double* brcs, const int* btypes, int ntypes, \
    const int* type_map, int U, int nghost, double rmax, double rmin, const double* q_scaler

extern "C" {

void orc_mtp_efv_f64(double* betot, double* bforce, double* bvirial, MTP_MODEL_ARGS, MTP_LIST_ARGS)
{
    Tables t{n_moms, n_basic, n_times, n_scalar, nmus, basic, times, mapping};
#pragma omp parallel for schedule(dynamic)
    for (int b = 0; b < B; b++)
        efv_one<double>(betot[b], &bforce[(size_t)b * (P + nghost) * 3], &bvirial[b * 9], K, scaling,
                        coeffs, lin, bias, t, binum[b], &bilist[(size_t)b * P],
                        &bnumneigh[(size_t)b * P], &bfirstneigh[(size_t)b * P * U],
                        &brcs[(size_t)b * P * U * 3], &btypes[(size_t)b * (P + nghost)], ntypes, U,
                        P + nghost, rmax, rmin, q_scaler);
}

void orc_mtp_loss_step_f64(double* bloss, double* rmse, double* betot, double* bforce, double* bvirial,
                           double* dcoeffs, double* dlin, double* dbias, double e_w, double f_w,
                           double v_w, const double* e_dft, const double* f_dft, const double* v_dft,
                           MTP_MODEL_ARGS, MTP_LIST_ARGS)
{
    Tables t{n_moms, n_basic, n_times, n_scalar, nmus, basic, times, mapping};
    const int ncoef = ntypes * ntypes * nmus * K;
    const int npar = ncoef + n_scalar + ntypes;
    // forward values and loss
    for (int b = 0; b < B; b++) {
        efv_one<double>(betot[b], &bforce[(size_t)b * P * 3], &bvirial[b * 9], K, scaling, coeffs, lin,
                        bias, t, binum[b], &bilist[(size_t)b * P], &bnumneigh[(size_t)b * P],
                        &bfirstneigh[(size_t)b * P * U], &brcs[(size_t)b * P * U * 3],
                        &btypes[(size_t)b * P], ntypes, U, P, rmax, rmin, q_scaler);
        bloss[b] = loss_one<double>(binum[b], &bilist[(size_t)b * P], e_w, f_w, v_w, betot[b], e_dft[b],
                                    &bforce[(size_t)b * P * 3], &f_dft[(size_t)b * P * 3],
                                    &bvirial[b * 9], &v_dft[b * 9]);
    }
    // RMSEs, linearMtpLoss_cpu_launcher.h:477-527
    double es = 0, fs = 0, vs = 0;
    long nf = 0;
    for (int b = 0; b < B; b++) {
        double de = (betot[b] - e_dft[b]) / binum[b];
        es += de * de;
        for (int ii = 0; ii < binum[b]; ii++) {
            int ci = bilist[(size_t)b * P + ii];
            for (int a = 0; a < 3; a++) {
                double d = bforce[((size_t)b * P + ci) * 3 + a] - f_dft[((size_t)b * P + ci) * 3 + a];
                fs += d * d;
            }
            nf += 3;
        }
        for (int i = 0; i < 9; i++) {
            double d = (bvirial[b * 9 + i] - v_dft[b * 9 + i]) / binum[b];
            vs += d * d;
        }
    }
    rmse[0] = std::sqrt(es / B);
    rmse[1] = std::sqrt(fs / nf);
    rmse[2] = std::sqrt(vs / (9.0 * B));

    // gradient by forward-mode AD, one parameter direction per pass
#pragma omp parallel
    {
        std::vector<Dual> c(ncoef), l(n_scalar), bi(ntypes), force((size_t)P * 3), virial(9);
#pragma omp for schedule(dynamic) collapse(2)
        for (int b = 0; b < B; b++)
            for (int p = 0; p < npar; p++) {
                for (int i = 0; i < ncoef; i++) c[i] = Dual(coeffs[i], i == p);
                for (int i = 0; i < n_scalar; i++) l[i] = Dual(lin[i], ncoef + i == p);
                for (int i = 0; i < ntypes; i++) bi[i] = Dual(bias[i], ncoef + n_scalar + i == p);
                Dual e;
                efv_one<Dual>(e, force.data(), virial.data(), K, scaling, c.data(), l.data(), bi.data(),
                              t, binum[b], &bilist[(size_t)b * P], &bnumneigh[(size_t)b * P],
                              &bfirstneigh[(size_t)b * P * U], &brcs[(size_t)b * P * U * 3],
                              &btypes[(size_t)b * P], ntypes, U, P, rmax, rmin, q_scaler);
                Dual L = loss_one<Dual>(binum[b], &bilist[(size_t)b * P], e_w, f_w, v_w, e, e_dft[b],
                                        force.data(), &f_dft[(size_t)b * P * 3], virial.data(),
                                        &v_dft[b * 9]);
                if (p < ncoef) dcoeffs[(size_t)b * ncoef + p] = L.d;
                else if (p < ncoef + n_scalar) dlin[(size_t)b * n_scalar + p - ncoef] = L.d;
                else dbias[(size_t)b * ntypes + p - ncoef - n_scalar] = L.d;
            }
    }
}


// site energies e_sites[B, P] and scalar moments desc[B, P, n_scalar] (either may be null)
void orc_mtp_esites_f64(double* e_sites, double* desc, MTP_MODEL_ARGS, MTP_LIST_ARGS)
{
    Tables t{n_moms, n_basic, n_times, n_scalar, nmus, basic, times, mapping};
    for (int b = 0; b < B; b++) {
        double e;
        std::vector<double> force((size_t)(P + nghost) * 3), virial(9);
        efv_one<double>(e, force.data(), virial.data(), K, scaling, coeffs, lin, bias, t, binum[b],
                        &bilist[(size_t)b * P], &bnumneigh[(size_t)b * P], &bfirstneigh[(size_t)b * P * U],
                        &brcs[(size_t)b * P * U * 3], &btypes[(size_t)b * (P + nghost)], ntypes, U, P + nghost,
                        rmax, rmin, q_scaler, e_sites ? &e_sites[(size_t)b * P] : nullptr,
                        desc ? &desc[(size_t)b * P * n_scalar] : nullptr);
    }
}

// d/dtheta of sum_ii gout[b, ii] e_sites[b, ii] per structure, by forward-mode AD
void orc_mtp_esites_bwd_f64(double* dcoeffs, double* dlin, double* dbias, const double* gout, MTP_MODEL_ARGS,
                            MTP_LIST_ARGS)
{
    Tables t{n_moms, n_basic, n_times, n_scalar, nmus, basic, times, mapping};
    const int ncoef = ntypes * ntypes * nmus * K;
    const int npar = ncoef + n_scalar + ntypes;
#pragma omp parallel
    {
        std::vector<Dual> c(ncoef), l(n_scalar), bi(ntypes), force((size_t)(P + nghost) * 3), virial(9), es(P);
#pragma omp for schedule(dynamic) collapse(2)
        for (int b = 0; b < B; b++)
            for (int p = 0; p < npar; p++) {
                for (int i = 0; i < ncoef; i++) c[i] = Dual(coeffs[i], i == p);
                for (int i = 0; i < n_scalar; i++) l[i] = Dual(lin[i], ncoef + i == p);
                for (int i = 0; i < ntypes; i++) bi[i] = Dual(bias[i], ncoef + n_scalar + i == p);
                Dual e;
                efv_one<Dual>(e, force.data(), virial.data(), K, scaling, c.data(), l.data(), bi.data(), t,
                              binum[b], &bilist[(size_t)b * P], &bnumneigh[(size_t)b * P],
                              &bfirstneigh[(size_t)b * P * U], &brcs[(size_t)b * P * U * 3],
                              &btypes[(size_t)b * (P + nghost)], ntypes, U, P + nghost, rmax, rmin, q_scaler,
                              es.data());
                double acc = 0;
                for (int ii = 0; ii < binum[b]; ii++) acc += gout[(size_t)b * P + ii] * es[ii].d;
                if (p < ncoef) dcoeffs[(size_t)b * ncoef + p] = acc;
                else if (p < ncoef + n_scalar) dlin[(size_t)b * n_scalar + p - ncoef] = acc;
                else dbias[(size_t)b * ntypes + p - ncoef - n_scalar] = acc;
            }
    }
}

// Neural-network MTP (source/descriptor/nnmtp): E/F/V, site energies e_sites[B, P] (may be null)
// with the moments of the linear MTP at scaling 1 (nnmtp/include/mtpBasis.h differs from
// mtpr/include/mtpBasis.h only by that factor) and the tanh read-out of nnMtp.h:378-567, 648-753.
void orc_nnmtp_efv_f64(double* betot, double* bforce, double* bvirial, double* e_sites, int K, int H,
                       const double* coeffs, const double* w0, const double* w1, const double* bias, int n_moms,
                       int n_basic, const int* basic, int n_times, const int* times, int n_scalar,
                       const int* mapping, int nmus, int B, int P, const int* binum, const int* bilist,
                       const int* bnumneigh, const int* bfirstneigh, const double* brcs, const int* btypes,
                       int ntypes, const int* type_map, int U, int nghost, double rmax, double rmin,
                       const double* q_shifter, const double* q_scaler)
{
    Tables t{n_moms, n_basic, n_times, n_scalar, nmus, basic, times, mapping};
    NNReadout<double> nn{H, w0, w1, q_shifter};
    for (int b = 0; b < B; b++)
        efv_one<double>(betot[b], &bforce[(size_t)b * (P + nghost) * 3], &bvirial[b * 9], K, 1.0, coeffs, nullptr,
                        bias, t, binum[b], &bilist[(size_t)b * P], &bnumneigh[(size_t)b * P],
                        &bfirstneigh[(size_t)b * P * U], &brcs[(size_t)b * P * U * 3],
                        &btypes[(size_t)b * (P + nghost)], ntypes, U, P + nghost, rmax, rmin, q_scaler,
                        e_sites ? &e_sites[(size_t)b * P] : nullptr, nullptr, &nn);
}

// one training step of the neural-network MTP: E/F/V, per-structure loss (nnMtpLoss.h:141-181, the
// linear MTP's formula) and its gradients w.r.t. coeffs, w0, w1, type_bias by forward-mode AD
void orc_nnmtp_loss_step_f64(double* bloss, double* betot, double* bforce, double* bvirial, double* dcoeffs,
                             double* dw0, double* dw1, double* dbias, double e_w, double f_w, double v_w,
                             const double* e_dft, const double* f_dft, const double* v_dft, int K, int H,
                             const double* coeffs, const double* w0, const double* w1, const double* bias,
                             int n_moms, int n_basic, const int* basic, int n_times, const int* times,
                             int n_scalar, const int* mapping, int nmus, int B, int P, const int* binum,
                             const int* bilist, const int* bnumneigh, const int* bfirstneigh, const double* brcs,
                             const int* btypes, int ntypes, const int* type_map, int U, int nghost, double rmax,
                             double rmin, const double* q_shifter, const double* q_scaler)
{
    Tables t{n_moms, n_basic, n_times, n_scalar, nmus, basic, times, mapping};
    const int ncoef = ntypes * ntypes * nmus * K, nw0 = ntypes * H * n_scalar, nw1 = ntypes * H;
    const int npar = ncoef + nw0 + nw1 + ntypes;
    NNReadout<double> nn{H, w0, w1, q_shifter};
    for (int b = 0; b < B; b++) {
        efv_one<double>(betot[b], &bforce[(size_t)b * P * 3], &bvirial[b * 9], K, 1.0, coeffs, nullptr, bias, t,
                        binum[b], &bilist[(size_t)b * P], &bnumneigh[(size_t)b * P], &bfirstneigh[(size_t)b * P * U],
                        &brcs[(size_t)b * P * U * 3], &btypes[(size_t)b * P], ntypes, U, P, rmax, rmin, q_scaler,
                        nullptr, nullptr, &nn);
        bloss[b] = loss_one<double>(binum[b], &bilist[(size_t)b * P], e_w, f_w, v_w, betot[b], e_dft[b],
                                    &bforce[(size_t)b * P * 3], &f_dft[(size_t)b * P * 3], &bvirial[b * 9],
                                    &v_dft[b * 9]);
    }
#pragma omp parallel
    {
        std::vector<Dual> c(ncoef), a0(nw0), a1(nw1), bi(ntypes), force((size_t)P * 3), virial(9);
#pragma omp for schedule(dynamic) collapse(2)
        for (int b = 0; b < B; b++)
            for (int p = 0; p < npar; p++) {
                for (int i = 0; i < ncoef; i++) c[i] = Dual(coeffs[i], i == p);
                for (int i = 0; i < nw0; i++) a0[i] = Dual(w0[i], ncoef + i == p);
                for (int i = 0; i < nw1; i++) a1[i] = Dual(w1[i], ncoef + nw0 + i == p);
                for (int i = 0; i < ntypes; i++) bi[i] = Dual(bias[i], ncoef + nw0 + nw1 + i == p);
                NNReadout<Dual> nd{H, a0.data(), a1.data(), q_shifter};
                Dual e;
                efv_one<Dual>(e, force.data(), virial.data(), K, 1.0, c.data(), nullptr, bi.data(), t, binum[b],
                              &bilist[(size_t)b * P], &bnumneigh[(size_t)b * P], &bfirstneigh[(size_t)b * P * U],
                              &brcs[(size_t)b * P * U * 3], &btypes[(size_t)b * P], ntypes, U, P, rmax, rmin,
                              q_scaler, nullptr, nullptr, &nd);
                Dual L = loss_one<Dual>(binum[b], &bilist[(size_t)b * P], e_w, f_w, v_w, e, e_dft[b], force.data(),
                                        &f_dft[(size_t)b * P * 3], virial.data(), &v_dft[b * 9]);
                if (p < ncoef) dcoeffs[(size_t)b * ncoef + p] = L.d;
                else if (p < ncoef + nw0) dw0[(size_t)b * nw0 + p - ncoef] = L.d;
                else if (p < ncoef + nw0 + nw1) dw1[(size_t)b * nw1 + p - ncoef - nw0] = L.d;
                else dbias[(size_t)b * ntypes + p - ncoef - nw0 - nw1] = L.d;
            }
    }
}

// d/dtheta of sum_ii gout[b, ii] e_sites[b, ii] per structure for the neural-network MTP, forward-mode AD
void orc_nnmtp_esites_bwd_f64(double* dcoeffs, double* dw0, double* dw1, double* dbias, const double* gout, int K,
                              int H, const double* coeffs, const double* w0, const double* w1, const double* bias,
                              int n_moms, int n_basic, const int* basic, int n_times, const int* times,
                              int n_scalar, const int* mapping, int nmus, int B, int P, const int* binum,
                              const int* bilist, const int* bnumneigh, const int* bfirstneigh, const double* brcs,
                              const int* btypes, int ntypes, const int* type_map, int U, int nghost, double rmax,
                              double rmin, const double* q_shifter, const double* q_scaler)
{
    Tables t{n_moms, n_basic, n_times, n_scalar, nmus, basic, times, mapping};
    const int ncoef = ntypes * ntypes * nmus * K, nw0 = ntypes * H * n_scalar, nw1 = ntypes * H;
    const int npar = ncoef + nw0 + nw1 + ntypes;
#pragma omp parallel
    {
        std::vector<Dual> c(ncoef), a0(nw0), a1(nw1), bi(ntypes), force((size_t)(P + nghost) * 3), virial(9), es(P);
#pragma omp for schedule(dynamic) collapse(2)
        for (int b = 0; b < B; b++)
            for (int p = 0; p < npar; p++) {
                for (int i = 0; i < ncoef; i++) c[i] = Dual(coeffs[i], i == p);
                for (int i = 0; i < nw0; i++) a0[i] = Dual(w0[i], ncoef + i == p);
                for (int i = 0; i < nw1; i++) a1[i] = Dual(w1[i], ncoef + nw0 + i == p);
                for (int i = 0; i < ntypes; i++) bi[i] = Dual(bias[i], ncoef + nw0 + nw1 + i == p);
                NNReadout<Dual> nd{H, a0.data(), a1.data(), q_shifter};
                Dual e;
                efv_one<Dual>(e, force.data(), virial.data(), K, 1.0, c.data(), nullptr, bi.data(), t, binum[b],
                              &bilist[(size_t)b * P], &bnumneigh[(size_t)b * P], &bfirstneigh[(size_t)b * P * U],
                              &brcs[(size_t)b * P * U * 3], &btypes[(size_t)b * (P + nghost)], ntypes, U, P + nghost,
                              rmax, rmin, q_scaler, es.data(), nullptr, &nd);
                double acc = 0;
                for (int ii = 0; ii < binum[b]; ii++) acc += gout[(size_t)b * P + ii] * es[ii].d;
                if (p < ncoef) dcoeffs[(size_t)b * ncoef + p] = acc;
                else if (p < ncoef + nw0) dw0[(size_t)b * nw0 + p - ncoef] = acc;
                else if (p < ncoef + nw0 + nw1) dw1[(size_t)b * nw1 + p - ncoef - nw0] = acc;
                else dbias[(size_t)b * ntypes + p - ncoef - nw0 - nw1] = acc;
            }
    }
}

// Backward of the legacy basis operator (src/mtpBasisOp.cc:220-326): with w[B, P, n_scalar] the gradient arriving
// at the scalar moments,  drcs[b, ii, u, :] = sum_s w_s dM_s / d rcs[b, ii, u, :]  and, per structure,
// dcoeffs[b, :] = sum_ii sum_s w_s dM_s / d coeffs  (mtpBasis.h:359-394 contracts the dense derivative arrays that
// find_val_der fills; the operator adds the structures' coefficient gradients into one vector).
// The position part restates the reference's forward differentiation (mtpBasis.h:186-245 basic moments,
// :248-300 products: dense dM[moment][neighbour][3] carried through the product table in file order).  The
// coefficient part is NOT the reference's mom_ders2coeffs propagation (:255-283): it is forward-mode AD of the
// scalar moments of efv_one, one coefficient at a time.
// Pinned by: the compiled reference (oracle/_ref/libref_mtpr.so, MtpBasis::find_val_der + find_der_backward)
// on the test fixtures; central differences of the scalar moments w.r.t. every pair vector and coefficient.
void orc_mtp_basis_bwd_f64(double* drcs, double* dcoeffs, const double* w, MTP_MODEL_ARGS, MTP_LIST_ARGS)
{
    Tables t{n_moms, n_basic, n_times, n_scalar, nmus, basic, times, mapping};
    const int ncoef = ntypes * ntypes * nmus * K;
    int kmax = 0;
    for (int i = 0; i < n_basic; i++) kmax = std::max(kmax, basic[i * 4 + 1] + basic[i * 4 + 2] + basic[i * 4 + 3]);
    if (drcs) {
        std::memset(drcs, 0, sizeof(double) * (size_t)B * P * U * 3);
#pragma omp parallel
        {
            std::vector<double> M(n_moms), dM((size_t)n_moms * U * 3), f(K), df(K), pw((kmax + 1) * 3), rp(kmax + 1),
                g(nmus), dg(nmus);
#pragma omp for schedule(dynamic) collapse(2)
            for (int b = 0; b < B; b++)
                for (int ii = 0; ii < P; ii++) {
                    if (ii >= binum[b]) continue;
                    const size_t row = (size_t)b * P + ii;
                    const int* types = &btypes[(size_t)b * (P + nghost)];
                    const int ti = types[bilist[row]], nn = bnumneigh[row];
                    std::fill(M.begin(), M.end(), 0.0);
                    std::fill(dM.begin(), dM.end(), 0.0);
                    for (int jj = 0; jj < nn; jj++) {
                        const double* v = &brcs[(row * U + jj) * 3];
                        const double r = std::sqrt(v[0] * v[0] + v[1] * v[1] + v[2] * v[2]);
                        if (r > rmax) continue;
                        const int tj = types[bfirstneigh[row * U + jj]];
                        radial_basis(K, rmax, rmin, scaling, r, f.data(), df.data());
                        rp[0] = 1; pw[0] = pw[1] = pw[2] = 1;
                        for (int k = 1; k <= kmax; k++) {
                            rp[k] = rp[k - 1] * r;
                            for (int a = 0; a < 3; a++) pw[k * 3 + a] = pw[(k - 1) * 3 + a] * v[a];
                        }
                        const double* c = &coeffs[(size_t)(ti * ntypes + tj) * nmus * K];
                        for (int mu = 0; mu < nmus; mu++) {
                            g[mu] = 0; dg[mu] = 0;
                            for (int k = 0; k < K; k++) { g[mu] += c[mu * K + k] * f[k]; dg[mu] += c[mu * K + k] * df[k]; }
                        }
                        for (int i = 0; i < n_basic; i++) {
                            const int* q = &basic[i * 4];
                            const int k = q[1] + q[2] + q[3];
                            const double mono = pw[q[1] * 3 + 0] * pw[q[2] * 3 + 1] * pw[q[3] * 3 + 2];
                            M[i] += g[q[0]] * mono / rp[k];
                            for (int a = 0; a < 3; a++) {
                                double dmono = 0;
                                if (q[1 + a] > 0) {
                                    int e[3] = {q[1], q[2], q[3]};
                                    e[a]--;
                                    dmono = q[1 + a] * pw[e[0] * 3 + 0] * pw[e[1] * 3 + 1] * pw[e[2] * 3 + 2];
                                }
                                dM[((size_t)i * U + jj) * 3 + a] =
                                    (dg[q[0]] * mono / rp[k] - g[q[0]] * k * mono / (rp[k] * r)) * v[a] / r + g[q[0]] * dmono / rp[k];
                            }
                        }
                    }
                    for (int i = 0; i < n_times; i++) {
                        const int* q = &times[i * 4];
                        const double v0 = M[q[0]], v1 = M[q[1]], mult = q[2];
                        M[q[3]] += mult * v0 * v1;
                        for (int e = 0; e < nn * 3; e++)
                            dM[(size_t)q[3] * U * 3 + e] += mult * (dM[(size_t)q[0] * U * 3 + e] * v1 + v0 * dM[(size_t)q[1] * U * 3 + e]);
                    }
                    for (int s = 0; s < n_scalar; s++) {
                        const double ws = w[row * n_scalar + s];
                        for (int e = 0; e < nn * 3; e++) drcs[row * U * 3 + e] += ws * dM[(size_t)mapping[s] * U * 3 + e];
                    }
                }
        }
    }
    if (dcoeffs) {
#pragma omp parallel
        {
            std::vector<Dual> c(ncoef), l(n_scalar, Dual(1.0, 0.0)), bi(ntypes, Dual(0.0, 0.0)), force((size_t)(P + nghost) * 3),
                virial(9), desc((size_t)P * n_scalar);
            std::vector<double> ones(n_scalar, 1.0);
#pragma omp for schedule(dynamic) collapse(2)
            for (int b = 0; b < B; b++)
                for (int p = 0; p < ncoef; p++) {
                    for (int i = 0; i < ncoef; i++) c[i] = Dual(coeffs[i], i == p);
                    Dual e;
                    efv_one<Dual>(e, force.data(), virial.data(), K, scaling, c.data(), l.data(), bi.data(), t, binum[b],
                                  &bilist[(size_t)b * P], &bnumneigh[(size_t)b * P], &bfirstneigh[(size_t)b * P * U],
                                  &brcs[(size_t)b * P * U * 3], &btypes[(size_t)b * (P + nghost)], ntypes, U, P + nghost,
                                  rmax, rmin, ones.data(), nullptr, desc.data());
                    double acc = 0;
                    for (int ii = 0; ii < binum[b]; ii++)
                        for (int s = 0; s < n_scalar; s++)
                            acc += w[((size_t)b * P + ii) * n_scalar + s] * desc[(size_t)ii * n_scalar + s].d;
                    dcoeffs[(size_t)b * ncoef + p] = acc;
                }
        }
    }
}

// Normal equations of the linear parameters (linear_mtp_gram_and_cross.h:446-575): per structure the
// energy / force / virial of every parameter taken alone (:125-374, by forward differentiation of the
// scalar moments along each pair displacement), accumulated into lin_matrix[n, n] and lin_vector[n]
// (:377-443), n = n_scalar + ntypes; the residuals are the labels themselves (no ZBL part).
void orc_mtp_lin_system_f64(double* lin_matrix, double* lin_vector, double e_w, double f_w, double v_w,
                            const double* e_res, const double* f_res, const double* v_res, MTP_MODEL_ARGS,
                            MTP_LIST_ARGS)
{
    Tables t{n_moms, n_basic, n_times, n_scalar, nmus, basic, times, mapping};
    const int n = n_scalar + ntypes;
    std::fill(lin_matrix, lin_matrix + (size_t)n * n, 0.0);
    std::fill(lin_vector, lin_vector + n, 0.0);
    int kmax = 0;
    for (int i = 0; i < n_basic; i++) kmax = std::max(kmax, basic[i * 4 + 1] + basic[i * 4 + 2] + basic[i * 4 + 3]);
    std::vector<double> ec(n), fc((size_t)P * 3 * n), vc((size_t)9 * n), M(n_moms), dM(n_moms), f(K), df(K),
        pw((kmax + 1) * 3), rp(kmax + 1);
    for (int b = 0; b < B; b++) {
        std::fill(ec.begin(), ec.end(), 0.0);
        std::fill(fc.begin(), fc.end(), 0.0);
        std::fill(vc.begin(), vc.end(), 0.0);
        const int* ilist = &bilist[(size_t)b * P];
        const int* types = &btypes[(size_t)b * P];
        for (int ii = 0; ii < binum[b]; ii++) {
            const int ci = ilist[ii], ti = types[ci], nn = bnumneigh[(size_t)b * P + ii];
            const int* first = &bfirstneigh[((size_t)b * P + ii) * U];
            const double* rcs = &brcs[((size_t)b * P + ii) * U * 3];
            // moments, as efv_one
            std::fill(M.begin(), M.end(), 0.0);
            auto pair_terms = [&](int jj, double& r) {
                const double* v = &rcs[jj * 3];
                r = std::sqrt(v[0] * v[0] + v[1] * v[1] + v[2] * v[2]);
                radial_basis(K, rmax, rmin, scaling, r, f.data(), df.data());
                rp[0] = 1; pw[0] = pw[1] = pw[2] = 1;
                for (int k = 1; k <= kmax; k++) {
                    rp[k] = rp[k - 1] * r;
                    for (int a = 0; a < 3; a++) pw[k * 3 + a] = pw[(k - 1) * 3 + a] * v[a];
                }
            };
            for (int jj = 0; jj < nn; jj++) {
                double r;
                pair_terms(jj, r);
                if (r > rmax) continue;
                const double* c = &coeffs[(size_t)(ti * ntypes + types[first[jj]]) * nmus * K];
                for (int i = 0; i < n_basic; i++) {
                    const int* q = &basic[i * 4];
                    double g = 0;
                    for (int k = 0; k < K; k++) g += c[q[0] * K + k] * f[k];
                    M[i] += g * pw[q[1] * 3] * pw[q[2] * 3 + 1] * pw[q[3] * 3 + 2] / rp[q[1] + q[2] + q[3]];
                }
            }
            for (int i = 0; i < n_times; i++) {
                const int* q = &times[i * 4];
                M[q[3]] += q[2] * M[q[0]] * M[q[1]];
            }
            ec[n_scalar + ti] += 1.0;                                          // :248-255
            for (int s = 0; s < n_scalar; s++) ec[s] += M[mapping[s]] / q_scaler[s];
            // derivative of every moment along each component of each pair displacement, :258-352
            for (int jj = 0; jj < nn; jj++) {
                double r;
                pair_terms(jj, r);
                if (r > rmax) continue;
                const int nj = first[jj];
                const double* v = &rcs[jj * 3];
                const double* c = &coeffs[(size_t)(ti * ntypes + types[nj]) * nmus * K];
                for (int a = 0; a < 3; a++) {
                    std::fill(dM.begin(), dM.end(), 0.0);
                    for (int i = 0; i < n_basic; i++) {
                        const int* q = &basic[i * 4];
                        const int kk = q[1] + q[2] + q[3];
                        double g = 0, dg = 0;
                        for (int k = 0; k < K; k++) { g += c[q[0] * K + k] * f[k]; dg += c[q[0] * K + k] * df[k]; }
                        const double mono = pw[q[1] * 3] * pw[q[2] * 3 + 1] * pw[q[3] * 3 + 2];
                        double dmono = 0;
                        if (q[1 + a] > 0) {
                            int e[3] = {q[1], q[2], q[3]};
                            e[a]--;
                            dmono = q[1 + a] * pw[e[0] * 3] * pw[e[1] * 3 + 1] * pw[e[2] * 3 + 2];
                        }
                        dM[i] = dg * v[a] / r * mono / rp[kk] + g * dmono / rp[kk] -
                                g * mono * kk / (rp[kk] * r * r) * v[a];
                    }
                    for (int i = 0; i < n_times; i++) {
                        const int* q = &times[i * 4];
                        dM[q[3]] += q[2] * (dM[q[0]] * M[q[1]] + M[q[0]] * dM[q[1]]);
                    }
                    for (int s = 0; s < n_scalar; s++) {
                        const double d = dM[mapping[s]] / q_scaler[s];
                        fc[((size_t)ci * 3 + a) * n + s] += d;
                        fc[((size_t)nj * 3 + a) * n + s] -= d;
                        for (int bb = 0; bb < 3; bb++) vc[(size_t)(a * 3 + bb) * n + s] -= d * v[bb];
                    }
                }
            }
        }
        // accumulation, :377-443 (upper triangle, mirrored at the end)
        for (int k1 = 0; k1 < n; k1++) {
            for (int k2 = k1; k2 < n; k2++) lin_matrix[(size_t)k1 * n + k2] += e_w * ec[k1] * ec[k2];
            lin_vector[k1] += e_w * e_res[b] * ec[k1];
        }
        for (int ii = 0; ii < binum[b]; ii++) {
            const int ci = ilist[ii];
            for (int a = 0; a < 3; a++) {
                const double* row = &fc[((size_t)ci * 3 + a) * n];
                for (int k1 = 0; k1 < n; k1++) {
                    for (int k2 = k1; k2 < n; k2++) lin_matrix[(size_t)k1 * n + k2] += f_w * row[k1] * row[k2];
                    lin_vector[k1] += f_w * f_res[((size_t)b * P + ci) * 3 + a] * row[k1];
                }
            }
        }
        for (int ab = 0; ab < 9; ab++) {
            const double* row = &vc[(size_t)ab * n];
            for (int k1 = 0; k1 < n; k1++) {
                for (int k2 = k1; k2 < n; k2++) lin_matrix[(size_t)k1 * n + k2] += v_w * row[k1] * row[k2];
                lin_vector[k1] += v_w * v_res[b * 9 + ab] * row[k1];
            }
        }
    }
    for (int k1 = 0; k1 < n; k1++)
        for (int k2 = k1 + 1; k2 < n; k2++) lin_matrix[(size_t)k2 * n + k1] = lin_matrix[(size_t)k1 * n + k2];
}

// schmidt_orth.h:38-116
void orc_mtp_schmidt_orth_f64(double* out, int ntypes, int nmus, int K, const double* in)
{
    const int np = ntypes * ntypes;
    for (int i = 0; i < np * nmus * K; i++) out[i] = in[i];
    auto at = [&](int pr, int mu, int xi) -> double& { return out[(pr * nmus + mu) * K + xi]; };
    for (int k1 = 0; k1 < nmus; k1++) {
        for (int k2 = 0; k2 < k1; k2++) {
            double norm2 = 0, scal = 0;
            for (int pr = 0; pr < np; pr++)
                for (int xi = 0; xi < K; xi++) { norm2 += at(pr, k2, xi) * at(pr, k2, xi); scal += at(pr, k1, xi) * at(pr, k2, xi); }
            for (int pr = 0; pr < np; pr++)
                for (int xi = 0; xi < K; xi++) at(pr, k1, xi) -= at(pr, k2, xi) * scal / norm2;
        }
        double norm2 = 1e-10;
        for (int pr = 0; pr < np; pr++)
            for (int xi = 0; xi < K; xi++) norm2 += at(pr, k1, xi) * at(pr, k1, xi);
        const double norm = std::sqrt(norm2);
        for (int pr = 0; pr < np; pr++)
            for (int xi = 0; xi < K; xi++) at(pr, k1, xi) /= norm;
    }
}
}
