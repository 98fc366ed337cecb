// Contraction plan of a linear Moment Tensor Potential level: the reference's tables
// (alpha_index_basic / alpha_index_times / alpha_moment_mapping, parsed from NN.almtp by
// source/descriptor/mtpr/src/mtpParam.cc:82-214) re-ordered on the host for parallel
// execution and kept resident on the device.
//
// The reference executes `times` sequentially: M[dst] += mult * M[m0] * M[m1] in file order
// (include/mtpBasis.h:522-528) and the adjoint sweep in reverse order
// (include/linearMtp.h:295-306).  Here every moment gets a dependency level (basic moments
// are level 0, a product is one above its deepest factor); moments of one level are
// independent, so one lane computes one moment as a gather over its terms:
//   forward : M[dst]  = sum_t mult_t * M[m0_t] * M[m1_t]             levels ascending
//   reverse : adj[m] += sum_t mult_t * adj[dst_t] * M[other_t]       levels descending
// The plan is valid only if no product is read before its last contribution in file order;
// plan creation verifies this.
#pragma once
#include <vector>

namespace a2p {

struct MtpPlanDevice {
    // sizes
    int n_moms, n_basic, n_times, n_scalar, nmus, kmax;
    int n_levels;              // number of product levels (>= 0)
    // device arrays
    const int* basic;          // [n_basic*4]  (mu, a, b, c)
    const int* mu_begin;       // [nmus+1]     basics are grouped by mu: run of each mu
    const int* mapping;        // [n_scalar]
    // forward gather: level l covers dst slots [f_level[l], f_level[l+1])
    const int* f_level;        // [n_levels+1]
    const int* f_dst;          // [n_fdst]
    const int* f_begin;        // [n_fdst+1] -> terms
    const int* f_m0;           // [n_times]
    const int* f_m1;           // [n_times]
    const double* f_mult;      // [n_times]
    // reverse gather: sources by level, level l covers [r_level[l], r_level[l+1]),
    // processed from the last level (deepest factors' consumers first) to level 0
    const int* r_level;        // [n_levels+1]  index l = level of the SOURCE moment
    const int* r_src;          // [n_rsrc]
    const int* r_begin;        // [n_rsrc+1]
    const int* r_dst;          // [2*n_times]
    const int* r_other;        // [2*n_times]
    const double* r_mult;      // [2*n_times]
};

struct MtpPlan {
    MtpPlanDevice d;
    void* device_block = nullptr;   // one allocation holding all arrays
    int device = 0;
};

}  // namespace a2p
