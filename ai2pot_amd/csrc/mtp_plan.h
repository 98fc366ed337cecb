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
#include <hip/hip_runtime.h>
#include <vector>

namespace a2p {

constexpr int MTP_SLOT_CAP = 16;
// The sweeps fetch the words of a slot MTP_DEPTH_STEP at a time; the depth of a group of slots is a multiple of it.
constexpr int MTP_DEPTH_STEP = 2;

struct MtpPlanDevice {
    // sizes
    int n_moms, n_basic, n_times, n_scalar, nmus, kmax;
    int n_levels;              // number of product levels (>= 0)
    // device arrays
    const int* basic;          // [n_basic*4]  (mu, a, b, c)
    const int* mu_begin;       // [nmus+1]     basics are grouped by mu: run of each mu
    const int* mapping;        // [n_scalar]
    // forward gather.  A slot holds up to MTP_SLOT_CAP terms of one destination moment; a longer
    // list is cut into consecutive slots (pieces), so that no lane walks a long list alone; the pieces of a
    // list lie in one group of 64 slots and the wavefront that walks the group adds their partial sums with
    // shuffles (f_multi[group] doubling steps: lists are sorted by length, so only a level's first groups hold cut lists).  Slots are grouped 64 at a time; level l covers slots
    // [f_level[l], f_level[l+1]) (whole groups; [f_level[l], f_lend[l]) without the padding slots).  The terms of a group are stored
    // interleaved and padded with zero terms to the group's depth (a multiple of MTP_DEPTH_STEP): term k of slot s is
    // f_terms[f_gbase[s >> 6] + k * 64 + (s & 63)], k < f_gdepth[s >> 6], so the 64 lanes that walk
    // a group read consecutive words and share the trip count.  A term packs x = 8 m0 | 8 m1 << 16 (byte offsets
    // into an array of doubles), y = multiplicity.
    const int* f_level;        // [n_levels+1]
    const int* f_lend;         // [n_levels+1]
    const int* f_multi;        // [n_fslots/64] doubling steps that add up the pieces of the group's longest list (0: none is cut)
    const int* f_dst;          // [n_fslots]   destination in the first piece of a list (-1 elsewhere and in padding)
    const int* f_rem;          // [n_fslots]   pieces of the same list behind this one
    const int* f_gbase;        // [n_fslots/64]
    const int* f_gdepth;       // [n_fslots/64]
    const int2* f_terms;
    // reverse gather, same layout: sources by level (index l = level of the SOURCE moment),
    // processed from the last level to level 0; a term packs x = 8 dst | 8 other << 16, y = mult
    const int* r_level;        // [n_levels+1]
    const int* r_lend;         // [n_levels+1]
    const int* r_multi;        // [n_rslots/64]
    const int* r_src;          // [n_rslots]
    const int* r_rem;          // [n_rslots]
    const int* r_gbase;        // [n_rslots/64]
    const int* r_gdepth;       // [n_rslots/64]
    const int2* r_terms;
    int max_level_slots;       // most slots of any level (forward or reverse)
    // Monomial walk of the pair-derivative pass.  The monomials x^a y^b z^c, a + b + c <= kmax, are numbered
    // q = row_base(a, b) + c; the adjoints of the basic moments are gathered into a dense array
    // AD[q][nmp] (mu fastest, nmp = nmus rounded up to even, zero where no basic moment has that
    // (mu, a, b, c)), so that a lane that owns one neighbour can walk a row (a, b), c = 0 .. kmax-a-b,
    // with z^c by recurrence and the adjoints as uniform reads.
    int nq, nmp, nrows;
    const int* rows;           // [nrows] a | b << 8 | row_base << 16, longest rows first
    const int* dense_pos;      // [n_basic] entry of each basic moment
    int dense_unique;          // no two basic moments share an entry (the usual case: a plain scatter fills AD)
    const int* dense_src;      // [nq*nmp] basic moment behind the entry, -1 none, -2 several (dense_off/items)
    const int* dense_off;      // [nq*nmp+1]
    const int* dense_items;    // [n_basic] basic moments ordered by dense entry
    // The one-hot adjoints of all scalar moments at once (linear-solver components).  A node (s, m) is moment m as an
    // ancestor of scalar moment s: mapping[s] itself, or a factor of a product among its ancestors.  The adjoint
    // sweeps of all read-outs e_s together are one reverse gather over the nodes, laid out like the reverse gather
    // above (a term packs x = 8 node(dst) | 8 other << 16 with `other` a moment, y = mult; x_src names the node).
    // The basic ancestors of a scalar moment form a list of words node | basic << 16; lists are sorted by length, cut into
    // pieces of at most MTP_SLOT_CAP words, and dealt to slots, 64 slots a group, the pieces of a list in neighbouring
    // slots of one group (the wavefront adds their sums with shuffles, x_bsteps doubling steps).  A group's words are
    // stored interleaved and padded to the group's depth with node x_nodes, whose adjoint is always zero: word k of
    // slot q is x_bwords[x_bbase[q >> 6] + k * 64 + (q & 63)].
    // The scalar moments are dealt to batches whose nodes fit the kernel's LDS budget (MtpPlan::xbatches); the fields
    // below are those of the batch a launch works on (x_root is -1 for the scalar moments of other batches).
    int x_nodes, x_slots;
    const int* x_root;         // [n_scalar] node (s, mapping[s])
    const int* x_seed;         // [x_slots]  scalar moment, in the slot of its list's first piece; -1 elsewhere
    const int* x_brem;         // [x_slots]  pieces of the same list behind this one
    const int* x_level;        // [n_levels+1]
    const int* x_multi;        // [n_xslots/64]
    const int* x_src;          // [n_xslots]
    const int* x_rem;          // [n_xslots]
    const int* x_gbase;        // [n_xslots/64]
    const int* x_gdepth;       // [n_xslots/64]
    const int2* x_terms;
    const int* x_bbase;        // [x_slots/64]
    const int* x_bdepth;       // [x_slots/64]
    const int* x_bsteps;       // [x_slots/64]
    const int* x_bwords;
};

// one batch of scalar moments of the components kernel: the x_ fields of MtpPlanDevice
struct MtpXBatch {
    int nodes, slots;
    const int *root, *seed, *level, *multi, *src, *rem, *gbase, *gdepth;
    const int2* terms;
    const int *bbase, *bdepth, *bsteps, *brem, *bwords;
};

struct MtpPlan {
    MtpPlanDevice d;
    std::vector<MtpXBatch> xbatches;   // empty: a scalar moment has too many ancestors (components pass by pass)
    void* device_block = nullptr;   // one allocation holding all arrays
    int device = 0;
};

}  // namespace a2p
