/* libai2pot_hip.so -- C ABI of the MI355X (gfx950) energy / force / virial hot path.
 *
 * Every entry point takes plain pointers and sizes.  Unless a parameter is documented as
 * "host", pointers are DEVICE pointers on the current HIP device; the caller owns every
 * input and output buffer.  Work is enqueued on `stream` (a hipStream_t passed as void*;
 * NULL = the default stream) and, unless stated otherwise, the call returns without
 * synchronising.  Scratch memory is a per-device workspace the library grows on demand
 * (steady-state calls allocate nothing).  Return value: A2P_OK or an A2P_ERR_* code; the
 * message of the last error on the calling thread is returned by a2p_last_error().
 *
 * "Reference" below is lhycms/AI2Pot; paths are relative to its root.
 */
#ifndef AI2POT_HIP_H
#define AI2POT_HIP_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define A2P_OK 0
#define A2P_ERR_INVALID 1   /* argument violates the contract (message says which)          */
#define A2P_ERR_HIP 2       /* a HIP runtime call failed                                     */
#define A2P_ERR_OVERFLOW 3  /* a neighbour count exceeds the row capacity umax               */
#define A2P_ERR_INPUT 4     /* device-side input check failed (bad neighbour / type index)   */
#define A2P_ERR_SEGMENT 5   /* an atom is named by more pairs than its reduction segment holds */
#define A2P_ERR_GRID 6      /* sync-free neighbour-list build: the bin box outgrew the bound of the last synchronised build */

const char* a2p_last_error(void);

/* Version of this ABI (bumped on incompatible change). */
int a2p_abi_version(void);

/* The per-device workspace (no counterpart in the reference, whose operators allocate their
 * scratch per call, e.g. source/descriptor/nep/include/nep.h:391-392).  It grows to what the
 * largest call so far needed and is then reused, so the library's work on ONE device must not
 * overlap in time.  Calls on one stream never do; when a call arrives on another stream than the
 * library's previous launch on that device, the library synchronises the device first (a stream
 * under graph capture is left alone; calls from several host threads at once are not supported).
 * Different devices are independent.  a2p_workspace_bytes returns what the library holds on the current device;
 * a2p_workspace_release synchronises the device and frees it (the next call allocates again). */
size_t a2p_workspace_bytes(void);
int a2p_workspace_release(void);
/* Counts the times a workspace buffer was freed or replaced by a larger one (any device).  A captured
 * HIP graph holds raw pointers into the workspace: record the value at capture and replay only while
 * it is unchanged (a larger call or a2p_workspace_release in between invalidates the graph). */
unsigned long long a2p_workspace_generation(void);

/* Reads and clears the device status word that kernels set when an input violates the
 * contract (neighbour index outside [0, natoms_pad+nghost), type index outside
 * [0, ntypes), numneigh > umax, more pairs naming one atom than its reduction segment holds).
 * Synchronises `stream`.  Returns A2P_OK, A2P_ERR_INPUT, A2P_ERR_OVERFLOW, A2P_ERR_SEGMENT or A2P_ERR_GRID.  The reference has no such check: it asserts or overflows
 * (source/nblist/include/neighborList.h:550, commented-out assert). */
int a2p_check_status(void* stream);

/* Per-kernel timing for benchmarks (no counterpart in the reference, which leaves timing to
 * commented-out std::chrono calls, interface/lammps/AI2POT/pair_ai2pot.cpp:392-442).  While
 * enabled, every kernel launch of the library is bracketed by HIP events on its stream.
 * a2p_profile_report synchronises the device and writes one line per kernel label,
 * "<label> <launch count> <total milliseconds>\n", into buf (truncated to buflen), then
 * clears the records. */
void a2p_profile_enable(int on);
int a2p_profile_report(char* buf, size_t buflen);
/* Restricts the timing to the kernel labels of a comma-separated list ("nep_stage_kernel,nbl_lists");
 * NULL or "" times every kernel again.  Two events per launch cost a few microseconds each, which a
 * step of fifteen launches feels: a benchmark times only the kernels it reports on. */
void a2p_profile_select(const char* labels);

/* ------------------------------------------------------------------------------------------
 * NEP energy / force / virial -- replaces the compute of torch.ops.nep.nepToEFVOp /
 * nepToEFOp / nepToDescriptorsOp (source/descriptor/nep/bind/nep_bind.cc:26-135, 278-311;
 * source/descriptor/nep/src/nepOp.cc:947-1284 -> include/nep_cpu_launcher.h:186-255 ->
 * include/nep.h:320-529, include/nepBasis.h:57-196).
 *
 * Model: coeffs[ntypes][ntypes][n_radial+n_angular][K], w0[ntypes][H][D], b0[ntypes][H],
 * w1[ntypes][H], type_bias[ntypes], q_scaler[D], D = n_radial + n_angular*l_max.
 * Batch (the 7-tensor contract): binum[B], bilist[B][P], bnumneigh[B][P],
 * bfirstneigh[B][P][U], brcs[B][P][U][3] (r_j - r_i), btypes[B][P+nghost] (type indices).
 * Outputs (each may be NULL to skip): etot[B], force[B][P+nghost][3], virial[B][9]
 * (row-major a*3+b, V = -sum g_a r_b), descriptors[B][P][D].  Outputs are overwritten: etot,
 * force (rows of padded atoms and ghosts included) and virial need no initialisation, every
 * element is written; of descriptors only the rows below binum[b] are.
 * Sign convention as the reference: force[i] += dE_i/dr_ij, force[j] -= dE_i/dr_ij.
 * ------------------------------------------------------------------------------------------ */
int a2p_nep_efv_f32(int chebyshev_size, int n_radial, int n_angular, int l_max, int num_neurons,
                    int ntypes, const float* coeffs, const float* w0, const float* b0,
                    const float* w1, const float* type_bias, const float* q_scaler,
                    double rmax_radial, double rmax_angular, int batch, int natoms_pad, int umax,
                    int nghost, const int* binum, const int* bilist, const int* bnumneigh,
                    const int* bfirstneigh, const float* brcs, const int* btypes, float* etot,
                    float* force, float* virial, float* descriptors, void* stream);

int a2p_nep_efv_f64(int chebyshev_size, int n_radial, int n_angular, int l_max, int num_neurons,
                    int ntypes, const double* coeffs, const double* w0, const double* b0,
                    const double* w1, const double* type_bias, const double* q_scaler,
                    double rmax_radial, double rmax_angular, int batch, int natoms_pad, int umax,
                    int nghost, const int* binum, const int* bilist, const int* bnumneigh,
                    const int* bfirstneigh, const double* brcs, const int* btypes, double* etot,
                    double* force, double* virial, double* descriptors, void* stream);

/* E/F/V calls that keep the places of the pairs in their targets' reduction segments from call to
 * call (no counterpart in the reference, which adds forces with atomics, nep.h:498-513).  The fast
 * NEP kernels give every pair (row, slot) an entry in the segment of the neighbour it names and
 * claim it with one integer atomic per pair and call.  A caller that uses a list for several
 * steps (molecular dynamics with a skin) owns two buffers for that list,
 *   rank[batch][natoms_pad][umax]      index of the pair among the pairs naming the same neighbour
 *   incoming[batch][natoms_pad+nghost] number of pairs naming each atom,
 * and passes ranks_valid = 0 on the first call for a list (the call records the places it claims)
 * and 1 on the following calls (they claim nothing: a third of the staging kernel's time).
 * Otherwise the calls equal a2p_nep_efv_*: the results do not depend on the ranks (the sums over a
 * segment are exact) and are bit-identical.  Kernels that have no use for ranks leave the buffers
 * alone.  a2p_pair_ranks fills the two buffers from the list alone. */
int a2p_pair_ranks(int batch, int natoms_pad, int umax, int nghost, const int* binum, const int* bnumneigh,
                   const int* bfirstneigh, int* rank, int* incoming, void* stream);

/* Reduction segments for lists that are not symmetric (no counterpart in the reference, which adds
 * forces with atomics, nep.h:498-513).  The fast NEP / MTP kernels store the derivative of every
 * pair into a segment owned by the neighbour it names, umax entries per atom: a list built with one
 * cutoff names an atom no more often than its own row is long.  Half lists, or ghosts that collect
 * the pairs of several rows (LAMMPS domains), can exceed that: the kernels then flag the call
 * (a2p_check_status returns A2P_ERR_SEGMENT; the forces of that call are incomplete) and the caller
 * repeats it with larger segments:
 *   a2p_pair_incoming_max   largest number of pairs naming one atom (HOST int out; synchronises),
 *   a2p_pair_segment_capacity(c)  segments of max(c, umax) entries for the following calls of the
 *                           CALLING THREAD (0 = back to umax); returns the previous setting.
 * The operator libraries and ai2pot_amd.ops do this by themselves unless validation is switched off. */
int a2p_pair_incoming_max(int batch, int natoms_pad, int umax, int nghost, const int* binum, const int* bnumneigh,
                          const int* bfirstneigh, int* max_incoming, void* stream);
int a2p_pair_segment_capacity(int capacity);

int a2p_nep_efv_ranked_f32(int chebyshev_size, int n_radial, int n_angular, int l_max, int num_neurons,
                           int ntypes, const float* coeffs, const float* w0, const float* b0,
                           const float* w1, const float* type_bias, const float* q_scaler,
                           double rmax_radial, double rmax_angular, int batch, int natoms_pad, int umax,
                           int nghost, const int* binum, const int* bilist, const int* bnumneigh,
                           const int* bfirstneigh, const float* brcs, const int* btypes, int* rank,
                           int* incoming, int ranks_valid, float* etot, float* force, float* virial,
                           float* descriptors, void* stream);

int a2p_nep_efv_ranked_f64(int chebyshev_size, int n_radial, int n_angular, int l_max, int num_neurons,
                           int ntypes, const double* coeffs, const double* w0, const double* b0,
                           const double* w1, const double* type_bias, const double* q_scaler,
                           double rmax_radial, double rmax_angular, int batch, int natoms_pad, int umax,
                           int nghost, const int* binum, const int* bilist, const int* bnumneigh,
                           const int* bfirstneigh, const double* brcs, const int* btypes, int* rank,
                           int* incoming, int ranks_valid, double* etot, double* force, double* virial,
                           double* descriptors, void* stream);

/* ------------------------------------------------------------------------------------------
 * Neighbour list -- replaces the compute of the CPython module function
 * nblist.find_info4mlff(lattice, types, coords, rcut, umax, is_cart, pbc_xyz, sort)
 * (source/nblist/bind/nblist_bind.cc:35-189 -> source/nblist/include/structure.h,
 * binLinkedList.h:658-696, 808-836, 900-1031, neighborList.h:274-338, 532-578).
 *
 * lattice[9] (rows) and pbc[3] are HOST pointers; types[natoms], coords[natoms][3] and all
 * outputs are device pointers: ilist[natoms], numneigh[natoms], firstneigh[natoms][umax]
 * (-1 padded, indices modulo natoms), rcs[natoms][umax][3] (r_j - r_i, 0 padded),
 * types_out[natoms].  Results are bit-identical to the reference's, in both sort modes.
 * The call synchronises `stream` once (the extents are read back to size the bin grid), and a
 * second time only when natoms times the number of periodic images exceeds 2 GiB of scratch
 * (the count of kept images is then read back instead of bounded).  max_numneigh (HOST int, may be NULL): when given, the call synchronises once
 * more, stores the largest neighbour count and returns A2P_ERR_OVERFLOW if it exceeds umax
 * (rows are then truncated, never overrun; the reference overruns, neighborList.h:550).
 * When NULL the check is left to a2p_check_status.
 * ------------------------------------------------------------------------------------------ */
int a2p_nblist_build_f32(const float* lattice, const int* types, const float* coords, int natoms,
                         double rcut, int umax, int is_cart, const int* pbc, int sort, int* ilist,
                         int* numneigh, int* firstneigh, float* rcs, int* types_out, int* max_numneigh,
                         void* stream);

int a2p_nblist_build_f64(const double* lattice, const int* types, const double* coords, int natoms,
                         double rcut, int umax, int is_cart, const int* pbc, int sort, int* ilist,
                         int* numneigh, int* firstneigh, double* rcs, int* types_out, int* max_numneigh,
                         void* stream);

/* Rebuild into buffers that already hold a list.  Same arguments and results as
 * a2p_nblist_build_*, for a caller that keeps its list buffers between steps (molecular
 * dynamics; the reference allocates fresh arrays per call, nblist_bind.cc:95-134, so it has no
 * counterpart of the distinction).  Contract: numneigh, firstneigh and rcs hold the unmodified
 * result of an earlier a2p_nblist_build_* or a2p_nblist_update_* call with the same natoms and
 * umax.  With sort = 0 a row is then written only up to the longer of its old and new lengths:
 * the -1 / 0 padding beyond is already in place, which saves three quarters of the writes at
 * umax = 200 and 48 neighbours.  With sort = 1 the call is the same as a2p_nblist_build_*. */
int a2p_nblist_update_f32(const float* lattice, const int* types, const float* coords, int natoms,
                          double rcut, int umax, int is_cart, const int* pbc, int sort, int* ilist,
                          int* numneigh, int* firstneigh, float* rcs, int* types_out, int* max_numneigh,
                          void* stream);

int a2p_nblist_update_f64(const double* lattice, const int* types, const double* coords, int natoms,
                          double rcut, int umax, int is_cart, const int* pbc, int sort, int* ilist,
                          int* numneigh, int* firstneigh, double* rcs, int* types_out, int* max_numneigh,
                          void* stream);

/* The list together with the places of its pairs (no counterpart in the reference; for callers
 * that go on to a2p_nep_efv_ranked_* with ranks_valid = 1, which then needs no atomics).  Rows are
 * unsorted (the sort = 0 result of a2p_nblist_build_*, bit for bit).  update = 0 / 1 chooses
 * between the contracts of a2p_nblist_build_* and a2p_nblist_update_*.  rank[natoms, umax] and
 * incoming[natoms] (DEVICE int32) are filled as a2p_pair_ranks fills them: rank[i, k] is the
 * place of pair (i, k) among the pairs that name the same neighbour, incoming[j] their number;
 * slots past a row's end are undefined. */
int a2p_nblist_build_ranked_f32(const float* lattice, const int* types, const float* coords, int natoms,
                                double rcut, int umax, int is_cart, const int* pbc, int update, int* ilist,
                                int* numneigh, int* firstneigh, float* rcs, int* types_out, int* rank,
                                int* incoming, int* max_numneigh, void* stream);

int a2p_nblist_build_ranked_f64(const double* lattice, const int* types, const double* coords, int natoms,
                                double rcut, int umax, int is_cart, const int* pbc, int update, int* ilist,
                                int* numneigh, int* firstneigh, double* rcs, int* types_out, int* rank,
                                int* incoming, int* max_numneigh, void* stream);

/* ------------------------------------------------------------------------------------------
 * Device-resident step: compact neighbour lists + NEP E/F/V on them.  Together the two calls
 * replace the reference's inference pair  nblist.find_info4mlff(...)  ->  torch.ops.nep.nepToEFVOp(...)
 * (ai2pot/utils/usepot.py:76-97, ai2pot/models/nep/nep.py:298-357) for ONE periodic structure
 * without ghosts, when positions stay on the device.  No counterpart of the list format exists in
 * the reference (its only format is the padded arrays of neighborList.h:532-578).
 *
 * a2p_nblist_build_compact_*: the build of a2p_nblist_build_* / a2p_nblist_update_* (sort = 0;
 * update as there) that ALSO cuts every row into the caller's `compact` buffer of
 * a2p_nblist_compact_bytes(natoms, umax, sizeof(T)) bytes: atoms in Morton order of their bins,
 * per atom the neighbours with r <= rcut_outer as 16-byte (fp32) entries [r_j - r_i, position |
 * species << 28] (position: the neighbour's place in that order, which is what the force kernels index
 * their per-atom arrays with), those with r <= rcut_inner kept apart from the rest (the radial and angular
 * cutoffs of the model; rcut_inner <= rcut_outer <= rcut).  update: bit 0 as for a2p_nblist_update_*
 * (the padded outputs hold an earlier result), bit 1 = keep the processing order that an earlier
 * build left in `compact` (it is a locality hint; atoms that moved a little are still well ordered)
 * instead of sorting again.  The order is the first array of the buffer, int32[natoms], position ->
 * atom; a caller whose atoms are already ordered in space may write the identity (or any permutation
 * of the atoms) there and set bit 1 from the first build on.  The array is not checked: it must hold
 * every index 0 .. natoms-1 once (an index outside that range is an access outside the buffers).  The five padded outputs are written,
 * bit-identical to a2p_nblist_build_*, when they are given; pass all five NULL to skip them.
 * Needs umax % 8 == 0, natoms < 2^27, species < 16, 16-byte aligned firstneigh / rcs.
 *
 * a2p_nep_efv_compact_*: energy, forces and virial of the structure from that buffer.  The list
 * names every pair from both ends, so F_i = sum_j (g_ij - g_ji) (nep.h:468-515 scatters the same terms).
 * For a pair inside the angular cutoff atom i evaluates g_ij once, adds it to its own force and hands it
 * to atom j through a 16-byte slot whose place it claims with an integer atomic; atom j sums its slots
 * in fixed point, so the result does not depend on the order of the claims: bit-reproducible.  For a pair
 * between the cutoffs g_ij - g_ji is evaluated by both ends from 32 gathered bytes of the other's
 * adjoints: nothing stored per pair.  The slots (32 per atom, 16 or 32 bytes each) live in the library's
 * workspace; an atom named by more than 32 pairs inside the angular cutoff receives the rest through a
 * spare row of 64-bit integers in the same fixed point, added to with integer atomics: bit-reproducible as
 * well.  The fixed point holds sums of magnitudes below 2^21 eV/A: when the magnitudes handed to one atom
 * through its slots add up to more, or one value sent to a spare row reaches 2^21 / umax, that atom's
 * force is NaN.  The counters of claimed places and the spare rows are zero between calls (the second
 * kernel clears what it read), so a call launches no fill kernel.
 * Model shapes: chebyshev_size 8, n_radial 4 or 6,
 * n_angular 4, l_max 4, at most 4 species (A2P_ERR_INVALID otherwise: use a2p_nep_efv_*).
 * types[natoms] are the type indices the list was built with.  etot[1] is required; force[natoms][3]
 * and virial[9] may be NULL.
 * ------------------------------------------------------------------------------------------ */
size_t a2p_nblist_compact_bytes(int natoms, int umax, int elem_size);   /* 0: not available for these sizes */

/* Neighbour-list builds without a host synchronisation (no counterpart in the reference, whose list build runs on
 * the host).  Every a2p_nblist_* build reads twelve coordinate extents back to size its bin grid, which makes the
 * host wait for the stream once per build and keeps the build out of HIP graphs.  a2p_nblist_sync_free(1) switches
 * that off for the calling host thread (returns the previous setting): a build of a structure this thread has built
 * before with the switch off or on (same device, natoms, lattice, cutoff, periodicity, coordinate kind) then sizes
 * its launches and scratch arrays for the bin box of that synchronised build plus a margin (an eighth, at least two
 * bins, per axis), derives the actual grid on the device and returns without waiting; results are bit-identical.  If
 * the atoms have spread beyond that bound (or a coordinate is not finite) the build leaves every list empty and
 * raises a status bit: a2p_check_status returns A2P_ERR_GRID, and the caller builds again with the switch off, which
 * also renews the bound.  Builds that ask for max_numneigh, or whose image arrays would exceed 2 GiB, synchronise as
 * before.  After one eager call in this mode the build can be captured into a HIP graph together with the operators
 * that consume the list. */
int a2p_nblist_sync_free(int on);

/* Which unit evaluates the per-species network (nep.h:415-447) inside a2p_nep_efv_compact_f32: 0 = the vector
 * ALUs, one thread per atom; 1 = the matrix cores (v_mfma_f32_16x16x4f32): the 64 atoms of a wavefront are grouped
 * by species in LDS and both layers run as [16 x 24] x [24 x 64] and [16 x 64] x [64 x 24] products per tile of 16
 * atoms, fp32 in and out (num_neurons <= 64, at most three species; larger models and fp64 stay on the vector
 * ALUs).  Returns the previous setting; any other argument only queries.  The environment variable
 * AI2POT_NEP_HIDDEN=valu|mfma sets the initial value.  Process-wide. */
int a2p_nep_hidden_layer_unit(int unit);

/* 1 when a2p_nep_efv_compact_* covers the model (shape as above, tables fit in LDS), else 0 */
int a2p_nep_efv_compact_supported(int chebyshev_size, int n_radial, int n_angular, int l_max, int num_neurons,
                                  int ntypes, int elem_size);

int a2p_nblist_build_compact_f32(const float* lattice, const int* types, const float* coords, int natoms,
                                 double rcut, int umax, int is_cart, const int* pbc, int update, double rcut_outer,
                                 double rcut_inner, int* ilist, int* numneigh, int* firstneigh, float* rcs,
                                 int* types_out, void* compact, void* stream);

int a2p_nblist_build_compact_f64(const double* lattice, const int* types, const double* coords, int natoms,
                                 double rcut, int umax, int is_cart, const int* pbc, int update, double rcut_outer,
                                 double rcut_inner, int* ilist, int* numneigh, int* firstneigh, double* rcs,
                                 int* types_out, void* compact, void* stream);

int a2p_nep_efv_compact_f32(int chebyshev_size, int n_radial, int n_angular, int l_max, int num_neurons, int ntypes,
                            const float* coeffs, const float* w0, const float* b0, const float* w1,
                            const float* type_bias, const float* q_scaler, double rmax_radial, double rmax_angular,
                            int natoms, int umax, const int* types, void* compact, float* etot, float* force,
                            float* virial, void* stream);

int a2p_nep_efv_compact_f64(int chebyshev_size, int n_radial, int n_angular, int l_max, int num_neurons, int ntypes,
                            const double* coeffs, const double* w0, const double* b0, const double* w1,
                            const double* type_bias, const double* q_scaler, double rmax_radial, double rmax_angular,
                            int natoms, int umax, const int* types, void* compact, double* etot, double* force,
                            double* virial, void* stream);

/* ------------------------------------------------------------------------------------------
 * Linear Moment Tensor Potential.
 *
 * a2p_mtp_plan_create takes the three HOST tables the reference's mtpParamOp returns
 * (source/descriptor/mtpr/src/mtpParamOp.cc:25-63, parsed from NN.almtp by
 * src/mtpParam.cc:82-214): alpha_index_basic[n_basic][4] = (mu, a, b, c),
 * alpha_index_times[n_times][4] = (m0, m1, mult, dst), alpha_moment_mapping[n_scalar];
 * it validates them, orders the products by dependency level and keeps the result on the
 * current device.  The handle is passed to the calls below and freed by
 * a2p_mtp_plan_destroy.  Levels whose moment vector does not fit LDS (above 24) are refused.
 *
 * a2p_mtp_efv_* replaces the compute of torch.ops.mtpr.linearMtpToEFVOp / linearMtpToEFOp
 * (source/descriptor/mtpr/bind/mtpr_bind.cc:333-457; src/linearMtpOp.cc:2834-3180 ->
 * include/linearMtp_cpu_launcher.h:128-203 -> include/linearMtp.h:190-352,
 * include/mtpBasis.h:400-534).  coeffs[ntypes][ntypes][nmus][K], linear_coeffs[n_scalar],
 * type_bias[ntypes], q_scaler[n_scalar]; batch and outputs as for a2p_nep_efv_*.
 *
 * a2p_mtp_loss_* replaces the compute of torch.ops.mtpr.linearMtpToLossOp, forward and
 * backward (mtpr_bind.cc:189-261; src/linearMtpOp.cc:621-1181, 1184-1765 ->
 * include/linearMtpLoss.h:138-176, 212-569, include/linearMtpLoss_cpu_launcher.h:151-194,
 * 233-337, 477-527).  Labels e_dft[B], f_dft[B][P][3], v_dft[B][9].  Outputs: bloss[B],
 * rmse[3] = (e, f, v) (may be NULL), the model's etot[B], force[B][P][3], virial[B][9]
 * (required), and the per-structure gradients dcoeffs[B][ntypes*ntypes*nmus*K],
 * dlinear[B][n_scalar], dbias[B][ntypes] (all three NULL = forward only).  The reference's
 * backward then returns grad_output[B] @ these matrices (linearMtpOp.cc:1740-1742); that
 * product is left to the caller.  nghost must be 0 for the loss, as in the reference
 * (linearMtpLoss_cpu_launcher.h:174, 285 index forces with stride natoms_pad).
 * ------------------------------------------------------------------------------------------ */
int a2p_mtp_plan_create(int n_moms, int n_basic, const int* basic, int n_times, const int* times,
                        int n_scalar, const int* mapping, void** plan);
int a2p_mtp_plan_destroy(void* plan);

int a2p_mtp_efv_f64(void* plan, int chebyshev_size, double scaling, const double* coeffs,
                    const double* linear_coeffs, const double* type_bias, int nmus, int ntypes,
                    const double* q_scaler, double rmax, double rmin, int batch, int natoms_pad, int umax,
                    int nghost, const int* binum, const int* bilist, const int* bnumneigh,
                    const int* bfirstneigh, const double* brcs, const int* btypes, double* etot,
                    double* force, double* virial, void* stream);

int a2p_mtp_efv_f32(void* plan, int chebyshev_size, double scaling, const float* coeffs,
                    const float* linear_coeffs, const float* type_bias, int nmus, int ntypes,
                    const float* q_scaler, double rmax, double rmin, int batch, int natoms_pad, int umax,
                    int nghost, const int* binum, const int* bilist, const int* bnumneigh,
                    const int* bfirstneigh, const float* brcs, const int* btypes, float* etot,
                    float* force, float* virial, void* stream);

int a2p_mtp_loss_f64(void* plan, double e_weight, double f_weight, double v_weight, const double* e_dft,
                     const double* f_dft, const double* v_dft, int chebyshev_size, double scaling,
                     const double* coeffs, const double* linear_coeffs, const double* type_bias, int nmus,
                     int ntypes, const double* q_scaler, double rmax, double rmin, int batch,
                     int natoms_pad, int umax, const int* binum, const int* bilist, const int* bnumneigh,
                     const int* bfirstneigh, const double* brcs, const int* btypes, double* bloss,
                     double* rmse, double* etot, double* force, double* virial, double* dcoeffs,
                     double* dlinear, double* dbias, void* stream);

int a2p_mtp_loss_f32(void* plan, double e_weight, double f_weight, double v_weight, const float* e_dft,
                     const float* f_dft, const float* v_dft, int chebyshev_size, double scaling,
                     const float* coeffs, const float* linear_coeffs, const float* type_bias, int nmus,
                     int ntypes, const float* q_scaler, double rmax, double rmin, int batch, int natoms_pad,
                     int umax, const int* binum, const int* bilist, const int* bnumneigh,
                     const int* bfirstneigh, const float* brcs, const int* btypes, float* bloss,
                     float* rmse, float* etot, float* force, float* virial, float* dcoeffs, float* dlinear,
                     float* dbias, void* stream);

/* ------------------------------------------------------------------------------------------
 * Linear-MTP site energies and scalar moments -- replaces the compute of
 * torch.ops.mtpr.linearMtpToEsitesOp (forward and backward) and linearMtpToDescriptorsOp
 * (source/descriptor/mtpr/bind/mtpr_bind.cc:459-569; src/linearMtpOp.cc:3589-4240;
 *  include/linearMtp.h:514-611 find_e_sites, :616-818 find_e_sites_backward, :821-890
 *  find_descriptors).
 * a2p_mtp_esites_*: e_sites[B, P] (row order, bias + sum_s lin[s] M[map[s]] / q_scaler[s]; may be
 * NULL) and descriptors[B, P, n_scalar] = M[map[s]] (unscaled; may be NULL); padded rows are zero.
 * a2p_mtp_esites_bwd_*: per-structure  sum_ii grad_e_sites[b, ii] * d e_sites[b, ii] / d theta  into
 * dcoeffs[B, ncoef], dlinear[B, n_scalar], dbias[B, ntypes] (any may be NULL); the operator's
 * backward sums them over the batch (linearMtpOp.cc:4002-4005).
 * ------------------------------------------------------------------------------------------ */
int a2p_mtp_esites_f64(void* plan, int chebyshev_size, double scaling, const double* coeffs,
                       const double* linear_coeffs, const double* type_bias, int nmus, int ntypes,
                       const double* q_scaler, double rmax, double rmin, int batch, int natoms_pad, int umax,
                       int nghost, const int* binum, const int* bilist, const int* bnumneigh,
                       const int* bfirstneigh, const double* brcs, const int* btypes, double* e_sites,
                       double* descriptors, void* stream);
int a2p_mtp_esites_f32(void* plan, int chebyshev_size, double scaling, const float* coeffs,
                       const float* linear_coeffs, const float* type_bias, int nmus, int ntypes,
                       const float* q_scaler, double rmax, double rmin, int batch, int natoms_pad, int umax,
                       int nghost, const int* binum, const int* bilist, const int* bnumneigh,
                       const int* bfirstneigh, const float* brcs, const int* btypes, float* e_sites,
                       float* descriptors, void* stream);
int a2p_mtp_esites_bwd_f64(void* plan, int chebyshev_size, double scaling, const double* coeffs,
                           const double* linear_coeffs, const double* type_bias, int nmus, int ntypes,
                           const double* q_scaler, double rmax, double rmin, int batch, int natoms_pad, int umax,
                           int nghost, const int* binum, const int* bilist, const int* bnumneigh,
                           const int* bfirstneigh, const double* brcs, const int* btypes,
                           const double* grad_e_sites, double* dcoeffs, double* dlinear, double* dbias,
                           void* stream);
int a2p_mtp_esites_bwd_f32(void* plan, int chebyshev_size, double scaling, const float* coeffs,
                           const float* linear_coeffs, const float* type_bias, int nmus, int ntypes,
                           const float* q_scaler, double rmax, double rmin, int batch, int natoms_pad, int umax,
                           int nghost, const int* binum, const int* bilist, const int* bnumneigh,
                           const int* bfirstneigh, const float* brcs, const int* btypes,
                           const float* grad_e_sites, float* dcoeffs, float* dlinear, float* dbias,
                           void* stream);

/* ------------------------------------------------------------------------------------------
 * Legacy basis operator -- replaces the compute of torch.ops.mtpr.mtpBasisOp, forward and backward
 * (source/descriptor/mtpr/bind/mtpr_bind.cc:140-187; src/mtpBasisOp.cc:28-218 forward, :220-326 backward;
 *  include/mtpBasis.h:107-356 MtpBasis::find_val_der, :359-394 find_der_backward).
 * Forward: the operator's output, the scalar moments M[map[s]] of every row, is what
 * a2p_mtp_esites_* writes to `descriptors` (e_sites NULL).  The reference's forward also fills two dense
 * arrays for its backward, dM_s/d rcs [B, P, S, umax, 3] and dM_s/d coeffs [B, P, S, ncoef]; here nothing
 * is kept between the passes.
 * a2p_mtp_basis_bwd_*: with w = grad_desc[B, P, S] (the gradient arriving at the forward output),
 *   drcs[b, ii, u, :] = sum_s w[b, ii, s] dM_s / d rcs[b, ii, u, :]      [B, P, umax, 3], zero beyond each row
 *   dcoeffs[b, :]     = sum_ii sum_s w[b, ii, s] dM_s / d coeffs          [B, ncoef]
 * (either may be NULL); the operator's backward sums dcoeffs over the batch (mtpBasis.h:389-393 adds every
 * structure into one vector).  Rows beyond binum and neighbours beyond rmax contribute nothing.
 * ------------------------------------------------------------------------------------------ */
int a2p_mtp_basis_bwd_f64(void* plan, int chebyshev_size, double scaling, const double* coeffs, int nmus,
                          int ntypes, double rmax, double rmin, int batch, int natoms_pad, int umax, int nghost,
                          const int* binum, const int* bilist, const int* bnumneigh, const int* bfirstneigh,
                          const double* brcs, const int* btypes, const double* grad_desc, double* drcs,
                          double* dcoeffs, void* stream);
int a2p_mtp_basis_bwd_f32(void* plan, int chebyshev_size, double scaling, const float* coeffs, int nmus,
                          int ntypes, double rmax, double rmin, int batch, int natoms_pad, int umax, int nghost,
                          const int* binum, const int* bilist, const int* bnumneigh, const int* bfirstneigh,
                          const float* brcs, const int* btypes, const float* grad_desc, float* drcs,
                          float* dcoeffs, void* stream);

/* ------------------------------------------------------------------------------------------
 * EXTENSION without a counterpart in the reference -- NEP energy / force / virial with four- and five-body
 * descriptors.  The reference's operators have radial and three-body descriptors only
 * (source/descriptor/nep/bind/nep_bind.cc:81-105, include/nep_utilities.h:39-49); its unfinished draft
 * source/descriptor/ace/include/nep_descriptor.h holds the weights C4B / C5B (:43-54) and declares
 * accum_4b_descriptor_one / accum_5b_descriptor_one (:109-111) without defining them.  PARITY UNPINNED: there is
 * no reference result to compare with; the entry points are checked by rotation invariance, finite differences of
 * the energy and the reduction to a2p_nep_efv_* when both terms are off.
 * Arguments as a2p_nep_efv_*, plus l_4body (0 or 2: one invariant per angular channel, cubic in its l = 2 moments)
 * and l_5body (0 or 1: one invariant, quartic in its l = 1 moments).  Descriptors of a channel are ordered
 * l = 1 .. l_max, four-body, five-body: D = n_radial + n_angular * (l_max + [l_4body > 0] + [l_5body > 0]), which
 * is the row length of w0 and q_scaler and of desc.
 * ------------------------------------------------------------------------------------------ */
int a2p_nep_efv_manybody_f32(int chebyshev_size, int n_radial, int n_angular, int l_max, int l_4body, int l_5body,
                             int num_neurons, int ntypes, const float* coeffs, const float* w0, const float* b0,
                             const float* w1, const float* type_bias, const float* q_scaler, double rmax_radial,
                             double rmax_angular, int batch, int natoms_pad, int umax, int nghost, const int* binum,
                             const int* bilist, const int* bnumneigh, const int* bfirstneigh, const float* brcs,
                             const int* btypes, float* etot, float* force, float* virial, float* desc, void* stream);
int a2p_nep_efv_manybody_f64(int chebyshev_size, int n_radial, int n_angular, int l_max, int l_4body, int l_5body,
                             int num_neurons, int ntypes, const double* coeffs, const double* w0, const double* b0,
                             const double* w1, const double* type_bias, const double* q_scaler, double rmax_radial,
                             double rmax_angular, int batch, int natoms_pad, int umax, int nghost, const int* binum,
                             const int* bilist, const int* bnumneigh, const int* bfirstneigh, const double* brcs,
                             const int* btypes, double* etot, double* force, double* virial, double* desc,
                             void* stream);

/* ------------------------------------------------------------------------------------------
 * ZBL short-range correction -- the part of every E/F/V operator that its zbl_rmax > 0 argument
 * switches on (source/descriptor/correction/include/zbl.h:262-395 pair formulas;
 *  correction/gpu/include/zbl.cuh:422-620 composition per centre atom;
 *  e.g. src/nepOp.cc:1086-1110, src/linearMtpOp.cc:2975-3000 call sites).
 * ADDS onto etot[B], force[B, P+nghost, 3] and virial[B, 9] (any may be NULL), which normally hold the
 * model's result: 0.5 E_pair per ordered pair to the energy, dE_pair/dr * r_vec / r to the force of
 * the centre atom only (a full list supplies the other half; ghosts receive nothing), and
 * -0.5 r_a dE_pair/dr r_b / r to the virial.  zbl_cks / zbl_dks: [ntypes, ntypes, 4] (device);
 * type_map: atomic numbers [ntypes] (device int32).
 * Parity: the pair formulas equal the reference's PairZBL member functions; the composition per centre atom
 * follows the reference's device source only (its CPU correct_efv has the force and virial calls commented
 * out): PARITY UNPINNED by a run of the reference.
 * ------------------------------------------------------------------------------------------ */
int a2p_zbl_correct_f64(double zbl_rmax, double zbl_rmin, const double* zbl_cks, const double* zbl_dks, int ntypes,
                        const int* type_map, int batch, int natoms_pad, int umax, int nghost, const int* binum,
                        const int* bilist, const int* bnumneigh, const int* bfirstneigh, const double* brcs,
                        const int* btypes, double* etot, double* force, double* virial, void* stream);
int a2p_zbl_correct_f32(double zbl_rmax, double zbl_rmin, const float* zbl_cks, const float* zbl_dks, int ntypes,
                        const int* type_map, int batch, int natoms_pad, int umax, int nghost, const int* binum,
                        const int* bilist, const int* bnumneigh, const int* bfirstneigh, const float* brcs,
                        const int* btypes, float* etot, float* force, float* virial, void* stream);
/* The same correction for the site-energy operators (GroupZBL::correct_e_sites, zbl.h:625-685, called by
 * src/linearMtpOp.cc:3662-3683 and the NN-MTP twin): ADDS to be_sites[B, natoms_pad] the row's sum of 0.5 E_pair
 * over its pairs with r <= zbl_rmax.  The reference's CPU operators call it BEFORE find_e_sites, which then assigns
 * its rows (linearMtp.h:598), so their output does not contain the term; here it is added to the model's rows, so
 * that the site energies sum to the energy the E/F/V operators give. */
int a2p_zbl_esites_f64(double zbl_rmax, double zbl_rmin, const double* zbl_cks, const double* zbl_dks, int ntypes,
                       const int* type_map, int batch, int natoms_pad, int umax, int nghost, const int* binum,
                       const int* bilist, const int* bnumneigh, const int* bfirstneigh, const double* brcs,
                       const int* btypes, double* be_sites, void* stream);
int a2p_zbl_esites_f32(double zbl_rmax, double zbl_rmin, const float* zbl_cks, const float* zbl_dks, int ntypes,
                       const int* type_map, int batch, int natoms_pad, int umax, int nghost, const int* binum,
                       const int* bilist, const int* bnumneigh, const int* bfirstneigh, const float* brcs,
                       const int* btypes, float* be_sites, void* stream);

/* ------------------------------------------------------------------------------------------
 * Linear solver support of the linear MTP -- replaces the compute of torch.ops.mtpr.LinMatrixLinVectorOp
 * and torch.ops.mtpr.CoeffsSchmidtOrthOp (source/descriptor/mtpr/bind/mtpr_bind.cc:38-131;
 *  include/linear_mtp_gram_and_cross.h:125-374 components, :377-443 accumulation, :446-575 launcher;
 *  include/schmidt_orth.h:38-116).
 * a2p_mtp_lin_components_*: with n = n_scalar + ntypes, per structure the energy ecomp[B, n], force
 * fcomp[B, P, 3, n] and virial vcomp[B, 9, n] of every linear parameter taken alone (column s: scalar
 * moment s over q_scaler[s]; column n_scalar + t: the species count in the energy, zero elsewhere).
 * The normal equations of the reference,
 *   lin_matrix = sum_b e_w E_b^T E_b + f_w F_b^T F_b + v_w V_b^T V_b,   lin_vector = the same against the residuals,
 * are plain GEMMs over these arrays and are left to the caller's BLAS (the bind library uses torch's).
 * nghost is 0, as the reference's force_components has natoms_pad rows.
 * All columns come from one pass over the atoms: the adjoint of column s is non-zero on the ancestors of scalar
 * moment s only, so the adjoints of all columns together are one gather about as long as an ordinary adjoint sweep
 * (the reference differentiates every moment along every pair displacement instead).  The call reads one integer back
 * (the number of pairs, to size its pair buffer: pairs * 3 * n_scalar values in the library's workspace, 0.4 GB for
 * 8192 atoms of 21 neighbours at level 16, 2 GB for 8192 atoms of 35 neighbours at level 20), so it cannot be captured in
 * a HIP graph.  a2p_mtp_components_route(0) switches to one energy / force / virial
 * pass per scalar moment; both routes agree to rounding.
 * a2p_mtp_components_route returns the previous setting (1 = one pass, the default; 0 = pass per column); any other
 * argument only queries.  The environment variable AI2POT_MTP_COMPONENTS=nodes|passes sets the initial value.
 * a2p_mtp_schmidt_orth_*: Gram-Schmidt over the nmus radial functions, each the vector of its
 * ntypes^2 * chebyshev_size coefficients; orth_coeffs must not alias coeffs.
 * ------------------------------------------------------------------------------------------ */
int a2p_mtp_lin_components_f64(void* plan, int chebyshev_size, double scaling, const double* coeffs, int nmus,
                               int ntypes, const double* q_scaler, double rmax, double rmin, int batch,
                               int natoms_pad, int umax, const int* binum, const int* bilist, const int* bnumneigh,
                               const int* bfirstneigh, const double* brcs, const int* btypes, double* ecomp,
                               double* fcomp, double* vcomp, void* stream);
int a2p_mtp_lin_components_f32(void* plan, int chebyshev_size, double scaling, const float* coeffs, int nmus,
                               int ntypes, const float* q_scaler, double rmax, double rmin, int batch,
                               int natoms_pad, int umax, const int* binum, const int* bilist, const int* bnumneigh,
                               const int* bfirstneigh, const float* brcs, const int* btypes, float* ecomp,
                               float* fcomp, float* vcomp, void* stream);
int a2p_mtp_components_route(int route);
int a2p_mtp_schmidt_orth_f64(int ntypes, int nmus, int chebyshev_size, const double* coeffs, double* orth_coeffs,
                             void* stream);
int a2p_mtp_schmidt_orth_f32(int ntypes, int nmus, int chebyshev_size, const float* coeffs, float* orth_coeffs,
                             void* stream);

/* ------------------------------------------------------------------------------------------
 * Neural-network MTP: energy, force, virial and site energies -- replaces the compute of
 * torch.ops.nnmtp.nnMtpToEFVOp / nnMtpToEFOp / nnMtpToEsitesOp (forward)
 * (source/descriptor/nnmtp/bind/nnmtp_bind.cc:193-322, 370-430; src/nnMtpOp.cc:2785-3190;
 *  include/nnMtp.h:378-567 find_efv, :648-753 find_e_sites).  The moments are those of the linear
 * MTP at scaling 1 (nnmtp/include/mtpBasis.h), so `plan` comes from a2p_mtp_plan_create; the
 * read-out is one tanh layer per centre species without hidden bias:
 *   e_i = type_bias[t] + sum_p w1[t,p] tanh( sum_k w0[t,p,k] (M_k - q_shifter[k]) / q_scaler[k] ).
 * w0[ntypes, num_neurons, n_scalar], w1[ntypes, num_neurons].  Outputs as a2p_mtp_efv_*; e_sites[B, P]
 * in row order (may be NULL); with etot, force and virial all NULL only the site energies are
 * computed.  nnMtpToDescriptorsOp is a2p_mtp_esites_* with scaling 1 (nnMtp.h:570-645).
 * ------------------------------------------------------------------------------------------ */
int a2p_nnmtp_efv_f64(void* plan, int chebyshev_size, int num_neurons, const double* coeffs, const double* w0,
                      const double* w1, const double* type_bias, int nmus, int ntypes, const double* q_shifter,
                      const double* q_scaler, double rmax, double rmin, int batch, int natoms_pad, int umax,
                      int nghost, const int* binum, const int* bilist, const int* bnumneigh,
                      const int* bfirstneigh, const double* brcs, const int* btypes, double* etot, double* force,
                      double* virial, double* e_sites, void* stream);
int a2p_nnmtp_efv_f32(void* plan, int chebyshev_size, int num_neurons, const float* coeffs, const float* w0,
                      const float* w1, const float* type_bias, int nmus, int ntypes, const float* q_shifter,
                      const float* q_scaler, double rmax, double rmin, int batch, int natoms_pad, int umax,
                      int nghost, const int* binum, const int* bilist, const int* bnumneigh,
                      const int* bfirstneigh, const float* brcs, const int* btypes, float* etot, float* force,
                      float* virial, float* e_sites, void* stream);

/* Backward of nnMtpToEsitesOp (src/nnMtpOp.cc:4170-4330; include/nnMtp.h:756-990 find_e_sites_backward):
 * per structure  sum_ii grad_e_sites[b, ii] * d e_sites[b, ii] / d theta  into dcoeffs[B, ntypes^2 nmus K],
 * dw0[B, ntypes H S], dw1[B, ntypes H], dbias[B, ntypes] (any may be NULL); the operator sums them over the batch. */
int a2p_nnmtp_esites_bwd_f64(void* plan, int chebyshev_size, int num_neurons, const double* coeffs,
                             const double* w0, const double* w1, const double* type_bias, int nmus, int ntypes,
                             const double* q_shifter, const double* q_scaler, double rmax, double rmin, int batch,
                             int natoms_pad, int umax, int nghost, const int* binum, const int* bilist,
                             const int* bnumneigh, const int* bfirstneigh, const double* brcs, const int* btypes,
                             const double* grad_e_sites, double* dcoeffs, double* dw0, double* dw1, double* dbias,
                             void* stream);
int a2p_nnmtp_esites_bwd_f32(void* plan, int chebyshev_size, int num_neurons, const float* coeffs, const float* w0,
                             const float* w1, const float* type_bias, int nmus, int ntypes, const float* q_shifter,
                             const float* q_scaler, double rmax, double rmin, int batch, int natoms_pad, int umax,
                             int nghost, const int* binum, const int* bilist, const int* bnumneigh,
                             const int* bfirstneigh, const float* brcs, const int* btypes,
                             const float* grad_e_sites, float* dcoeffs, float* dw0, float* dw1, float* dbias,
                             void* stream);

/* ------------------------------------------------------------------------------------------
 * Neural-network MTP training loss, forward and analytic backward -- replaces the compute of
 * torch.ops.nnmtp.nnMtpToLossOp and nnMtpToEFLossOp
 * (source/descriptor/nnmtp/bind/nnmtp_bind.cc:43-191; src/nnMtpOp.cc:569-2780;
 *  include/nnMtpLoss.h:141-181 loss, :216-610 and :612-994 backward).
 * Per structure  loss = e_w/N (E-E0)^2 + f_w/(3N) sum |F-F0|^2 + v_w/(9N) sum (V-V0)^2;
 * nnMtpToEFLossOp is the same call with v_weight = 0 (v_dft still has to point at B*9 values).
 * Outputs (device): bloss[B]; the model's etot[B], force[B,P,3], virial[B,9]; per-structure
 * gradients dcoeffs[B, ntypes^2 nmus K], dw0[B, ntypes H S], dw1[B, ntypes H], dbias[B, ntypes] (any
 * may be NULL; all NULL skips the backward kernels).  The operator's backward multiplies them by
 * grad_output[B] (nnMtpOp.cc:2748-2780).  nghost is 0, as in the reference's loss launchers.
 * exact_gradient = 0 evaluates the reference's backward formulas; these omit, for the force and
 * virial terms, the dependence of dE/dM on the moments in d/dcoeffs (nnMtpLoss.h:497-529) and the
 * off-diagonal part of the pre-activation tangent in d/dw0 (:560-585), so they are not the
 * derivative of the loss.  exact_gradient = 1 returns the complete derivative.
 * ------------------------------------------------------------------------------------------ */
int a2p_nnmtp_loss_f64(void* plan, double e_weight, double f_weight, double v_weight, const double* e_dft,
                       const double* f_dft, const double* v_dft, int chebyshev_size, int num_neurons,
                       const double* coeffs, const double* w0, const double* w1, const double* type_bias, int nmus,
                       int ntypes, const double* q_shifter, const double* q_scaler, double rmax, double rmin,
                       int batch, int natoms_pad, int umax, const int* binum, const int* bilist,
                       const int* bnumneigh, const int* bfirstneigh, const double* brcs, const int* btypes,
                       double* bloss, double* etot, double* force, double* virial, double* dcoeffs, double* dw0,
                       double* dw1, double* dbias, int exact_gradient, void* stream);
int a2p_nnmtp_loss_f32(void* plan, double e_weight, double f_weight, double v_weight, const float* e_dft,
                       const float* f_dft, const float* v_dft, int chebyshev_size, int num_neurons,
                       const float* coeffs, const float* w0, const float* w1, const float* type_bias, int nmus,
                       int ntypes, const float* q_shifter, const float* q_scaler, double rmax, double rmin,
                       int batch, int natoms_pad, int umax, const int* binum, const int* bilist,
                       const int* bnumneigh, const int* bfirstneigh, const float* brcs, const int* btypes,
                       float* bloss, float* etot, float* force, float* virial, float* dcoeffs, float* dw0,
                       float* dw1, float* dbias, int exact_gradient, void* stream);

/* ------------------------------------------------------------------------------------------
 * NEP training loss, forward and analytic backward -- replaces the compute of
 * torch.ops.nep.nepToLossOp and torch.ops.nep.nepToEFLossOp
 * (source/descriptor/nep/bind/nep_bind.cc:136-276; src/nepOp.cc:2359-3484;
 *  include/nepLoss.h:139-209 loss, :213-745 and :752-1298 backward;
 *  include/nepLoss_cpu_launcher.h:31-163, 167-330 launchers, :333-406 RMSEs).
 * Per structure  loss = e_w/N (E-E0)^2 + f_w/(3N) sum |F-F0|^2 + v_w/(9N) sum (V-V0)^2;
 * nepToEFLossOp is the same call with v_weight = 0 (v_dft still has to point at B*9 values).
 * Outputs (device): bloss[B]; rmse[3] = (E per atom, F per component, V per component: the
 * virial one is not divided by the atom count, unlike the MTP operator); the model's
 * etot[B], force[B,P,3], virial[B,9]; and per-structure gradients dcoeffs[B, ntypes^2 (n_r+n_a) K],
 * dw0[B, ntypes H D], db0[B, ntypes H], dw1[B, ntypes H], dbias[B, ntypes] (any may be NULL;
 * all NULL skips the backward kernels).  The operator's backward multiplies them by
 * grad_output[B] (nepOp.cc:2901-2960).  nghost is 0, as in the reference's loss launchers,
 * which index forces with stride natoms_pad.
 * ------------------------------------------------------------------------------------------ */
int a2p_nep_loss_f64(double e_weight, double f_weight, double v_weight, const double* e_dft, const double* f_dft,
                     const double* v_dft, int chebyshev_size, int n_radial_basis, int n_angular_basis, int l_max,
                     int num_neurons, int ntypes, const double* coeffs, const double* w0, const double* b0,
                     const double* w1, const double* type_bias, const double* q_scaler, double rmax_radial,
                     double rmax_angular, int batch, int natoms_pad, int umax, const int* binum, const int* bilist,
                     const int* bnumneigh, const int* bfirstneigh, const double* brcs, const int* btypes,
                     double* bloss, double* rmse, double* etot, double* force, double* virial, double* dcoeffs,
                     double* dw0, double* db0, double* dw1, double* dbias, void* stream);
int a2p_nep_loss_f32(double e_weight, double f_weight, double v_weight, const float* e_dft, const float* f_dft,
                     const float* v_dft, int chebyshev_size, int n_radial_basis, int n_angular_basis, int l_max,
                     int num_neurons, int ntypes, const float* coeffs, const float* w0, const float* b0,
                     const float* w1, const float* type_bias, const float* q_scaler, double rmax_radial,
                     double rmax_angular, int batch, int natoms_pad, int umax, const int* binum, const int* bilist,
                     const int* bnumneigh, const int* bfirstneigh, const float* brcs, const int* btypes,
                     float* bloss, float* rmse, float* etot, float* force, float* virial, float* dcoeffs,
                     float* dw0, float* db0, float* dw1, float* dbias, void* stream);

/* ------------------------------------------------------------------------------------------
 * Short-range force / virial from per-pair derivatives -- replaces the compute of
 * torch.ops.fvt.ForceSrOp and torch.ops.fvt.VirialSrOp, forward and backward
 * (source/fvt/bind/fvt_sr_op_bind.cc:9-46; src/force_sr_op.cc:11-179, src/virial_sr_op.cc:10-164
 * -> include/force_sr.h:50-124, include/virial_sr.h:24-51).
 * dei_drij[B][nlocal][umax][3]; force[B][nlocal+nghost][3]; virial[B][9]; rows ii < binum[b]
 * (force) or all nlocal rows (virial, as the reference) and slots s < bnumneigh[b][ii] count.
 *   force_fwd : force[c] = sum_s dei[ii,s] - sum_{pairs with neighbour c} dei   (c = bilist[ii])
 *   force_bwd : grad_dei[ii,s,k] = grad_force[c,k] - grad_force[j,k], zero on padding
 *   virial_fwd: virial[a*3+b] = - sum dei[ii,s,a] rcs[ii,s,b]
 *   virial_bwd: grad_dei[ii,s,a] = - sum_b grad_virial[a*3+b] rcs[ii,s,b];
 *               grad_rcs[ii,s,b] = - sum_a grad_virial[a*3+b] dei[ii,s,a]   (either may be NULL)
 * The dense Jacobians the reference builds are never formed.
 * ------------------------------------------------------------------------------------------ */
int a2p_fvt_force_fwd_f32(int batch, int nlocal, int umax, int nghost, const int* binum, const int* bilist,
                          const int* bnumneigh, const int* bfirstneigh, const float* dei_drij, float* force,
                          void* stream);
int a2p_fvt_force_fwd_f64(int batch, int nlocal, int umax, int nghost, const int* binum, const int* bilist,
                          const int* bnumneigh, const int* bfirstneigh, const double* dei_drij, double* force,
                          void* stream);
int a2p_fvt_force_bwd_f32(int batch, int nlocal, int umax, int nghost, const int* binum, const int* bilist,
                          const int* bnumneigh, const int* bfirstneigh, const float* grad_force,
                          float* grad_dei, void* stream);
int a2p_fvt_force_bwd_f64(int batch, int nlocal, int umax, int nghost, const int* binum, const int* bilist,
                          const int* bnumneigh, const int* bfirstneigh, const double* grad_force,
                          double* grad_dei, void* stream);
int a2p_fvt_virial_fwd_f32(int batch, int nlocal, int umax, const int* bnumneigh, const float* rcs,
                           const float* dei_drij, float* virial, void* stream);
int a2p_fvt_virial_fwd_f64(int batch, int nlocal, int umax, const int* bnumneigh, const double* rcs,
                           const double* dei_drij, double* virial, void* stream);
/* a2p_fvt_virial_fwd_f32 for callers that cannot allocate device memory (code under HIP graph
 * capture, serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same
 * arguments, same kernels and bit-identical results, but the row partial sums go to a buffer that is
 * part of the library's image (4.5 MiB per GPU the library runs on, held until the process ends)
 * instead of the growable workspace, and the call never allocates or frees anything: no hipMalloc,
 * no hipFree, no event creation.  Limit: batch * nlocal <= 65536 rows; more returns A2P_ERR_INVALID.
 * All calls on one GPU share the buffer, so calls that overlap in time on one GPU (two streams, two
 * host threads) race; order them on one stream or with events. */
int a2p_fvt_virial_fwd_noalloc_f32(int batch, int nlocal, int umax, const int* bnumneigh, const float* rcs,
                                   const float* dei_drij, float* virial, void* stream);
int a2p_fvt_virial_bwd_f32(int batch, int nlocal, int umax, const int* bnumneigh, const float* rcs,
                           const float* dei_drij, const float* grad_virial, float* grad_dei, float* grad_rcs,
                           void* stream);
int a2p_fvt_virial_bwd_f64(int batch, int nlocal, int umax, const int* bnumneigh, const double* rcs,
                           const double* dei_drij, const double* grad_virial, double* grad_dei,
                           double* grad_rcs, void* stream);

#ifdef __cplusplus
}
#endif
#endif
