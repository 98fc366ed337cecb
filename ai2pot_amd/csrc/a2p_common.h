// Internal helpers shared by the HIP translation units of libai2pot_hip.so:
// error reporting, a per-device growable workspace, launch checks and wave-level
// primitives for 64-wide wavefronts (gfx950).
#pragma once
#include <hip/hip_runtime.h>
#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <cstdarg>
#include <string>

#include "../../include/ai2pot_hip.h"

namespace a2p {

// ---- error state (thread local, read back through a2p_last_error) ---------------------
void set_error(const char* fmt, ...);
const char* last_error();

#define A2P_HIP_CHECK(expr)                                                              \
    do {                                                                                 \
        hipError_t e_ = (expr);                                                          \
        if (e_ != hipSuccess) {                                                          \
            a2p::set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_),        \
                           __FILE__, __LINE__);                                          \
            return A2P_ERR_HIP;                                                          \
        }                                                                                \
    } while (0)

#define A2P_REQUIRE(cond, code, ...)                                                     \
    do {                                                                                 \
        if (!(cond)) {                                                                   \
            a2p::set_error(__VA_ARGS__);                                                 \
            return code;                                                                 \
        }                                                                                \
    } while (0)

// ---- workspace: a few named device buffers per device, grown on demand -----------------
enum WsSlot {
    WS_PAIR_G = 0,     // per-pair derivative buffer [rows, U, 3]
    WS_CSR,            // counts / offsets / cursors / incoming pair ids
    WS_PARTIAL,        // per-block partial sums (energy, virial, loss terms)
    WS_NBL_A,          // neighbor-list: images, bins
    WS_NBL_B,
    WS_MTP,            // MTP per-atom scratch
    WS_FLAGS,          // device-side status words
    WS_MISC,
    WS_GRID,           // neighbor-list: the bin grid derived on the device (builds without read-back)
    WS_NEP_CLAIMS,     // NEP on compact lists: counters of claimed places and spare rows; zero between calls
    WS_NSLOTS
};
// Returns a device pointer valid until the next ws_get on the same slot with a larger size.
// Growth synchronises the device (hipFree); steady-state calls do not allocate.
// WS_FLAGS and WS_NEP_CLAIMS are zero-filled when they are allocated; their users leave them zero.
int ws_get(int slot, size_t bytes, void** out);
int ws_drop(int slot); // synchronises the device and frees one buffer of the current device (its contents are suspect)
size_t ws_bytes();     // held on the current device
int ws_release();      // synchronises the device, frees the current device's buffers

// Device status word bits written by kernels when inputs violate the contract.
enum StatusBits {
    ST_BAD_NEIGHBOR = 1,   // neighbour index outside [0, natoms_pad + nghost)
    ST_BAD_TYPE = 2,       // type index outside [0, ntypes)
    ST_NEIGH_OVERFLOW = 4, // numneigh larger than the row capacity
    ST_SEG_OVERFLOW = 8,   // more pairs name one atom than its reduction segment holds (a list that is not symmetric)
    ST_GRID_BOUND = 16,    // neighbour list built without reading the extents back: the bin box outgrew its bound
};

inline int ceil_div(long long a, long long b) { return (int)((a + b - 1) / b); }

// ---- optional per-kernel timing with HIP events on the launching stream --------------------
// While profiling is enabled (a2p_profile_enable), a ProfScope around a launch records an
// event before and after it on `stream`; a2p_profile_report resolves them into per-label
// totals.  Disabled (the default) it costs one branch.
void prof_begin(const char* label, hipStream_t stream);
void prof_end(hipStream_t stream);
// Orders this library's work across streams of a device (device synchronisation when the stream changes; a stream
// under capture is left alone).  prof_begin calls it; entry points that launch without prof_begin call it first.
int enter_stream(hipStream_t stream);
struct ProfScope {
    hipStream_t s;
    ProfScope(const char* label, hipStream_t stream) : s(stream) { prof_begin(label, stream); }
    ~ProfScope() { prof_end(s); }
};

// ---- wave64 primitives -------------------------------------------------------------------
__device__ __forceinline__ int lane_id() { return (int)(threadIdx.x & 63); }

template <typename T>
__device__ __forceinline__ T wave_sum(T v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

template <typename T>
__device__ __forceinline__ T wave_max(T v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        T o = __shfl_xor(v, off, 64);
        v = o > v ? o : v;
    }
    return v;
}

__device__ __forceinline__ long long shfl_xor_ll(long long v, int off)
{
    int lo = __shfl_xor((int)(v & 0xffffffffll), off, 64);
    int hi = __shfl_xor((int)(v >> 32), off, 64);
    return ((long long)hi << 32) | (unsigned int)lo;
}

// inclusive prefix sum across the 64 lanes of a wave: shifts by 1, 2, 4, 8 inside each row of
// 16 lanes, then the last lane of row 0 / 2 is added to row 1 / 3 and lane 31 to rows 2 and 3
__device__ __forceinline__ int wave_inclusive_scan(int v)
{
    v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, true);    // row_shr:1
    v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, true);    // row_shr:2
    v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, true);    // row_shr:4
    v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, true);    // row_shr:8
    v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);   // row_bcast:15 -> rows 1, 3
    v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);   // row_bcast:31 -> rows 2, 3
    return v;
}

// ---- shared device routines (pair_reduce.hip) --------------------------------------------
// Deterministic reduction of per-pair derivatives g[row, slot, 3] onto atoms:
//   force[b, j] = own[b, j] - sum over pairs (row, slot) of structure b whose neighbour is j.
// `force` must already hold the `own` part (zero for atoms without a row).  Integer atomics
// build the incoming lists; the floating-point sums are order-independent (terms rounded to a
// common quantum chosen from the per-target maximum, then added exactly), so results are
// reproducible run to run.
template <typename T>
int pair_reduce(T* force, const T* pair_g, int B, int P, int U, int nghost, const int* binum,
                const int* bnumneigh, const int* bfirstneigh, hipStream_t stream);

// The same reduction for a producer that stores each pair derivative straight into its
// target's segment, without the intermediate [row, slot, 3] array:
//   pair_csr_begin   counts the incoming pairs per target and scans them into segment offsets;
//                    with_rank: every valid pair (row, slot) also gets rank[row*U + slot], its
//                    place inside its target's segment (-1 for an index out of range);
//   the producer     stores seg_g[pos*3 .. pos*3+2] at  pos = offsets[t] + rank[row*U + slot]
//                    for EVERY valid pair (zeros where the derivative vanishes), or, without
//                    ranks, claims  pos = offsets[t] + atomicAdd(&cursor[t], 1)  and may skip pairs;
//   pair_csr_finish  sums the filled part of every segment onto `force` as above.
// Capacity of the fixed reduction segments: umax unless the calling thread asked for more with
// a2p_pair_segment_capacity (lists in which an atom is named by more pairs than a row holds).
int pair_segment_capacity(int U);
// pair_fixed_begin skips counting: every target owns a segment of fixed capacity seg_cap (umax by default)
// (a cutoff-built list sends an atom no more pairs than its own row could hold); the producer
// claims  rank = atomicAdd(&cursor[t], 1),  stores at  pos = t*seg_cap + rank  when rank < seg_cap
// and otherwise raises ST_SEG_OVERFLOW and stores at the spare entry n*seg_cap.
struct PairCsr {
    int* counts;
    int* offsets;
    int* cursor;
    int* rank;      // [B*P, U] or null
    void* seg_g;
    int n;          // B * (P + nghost) targets
    int seg_cap;    // > 0: fixed-capacity segments (offsets, counts and rank are null)
};
template <typename T>
int pair_csr_begin(PairCsr* csr, bool with_rank, int B, int P, int U, int nghost, const int* binum,
                   const int* bnumneigh, const int* bfirstneigh, hipStream_t stream);
// also_zero / also_bytes: a second range cleared by the same launch that clears the cursors
// (the force array of the caller, as a rule)
template <typename T>
int pair_fixed_begin(PairCsr* csr, int B, int P, int U, int nghost, hipStream_t stream, void* also_zero = nullptr,
                     size_t also_bytes = 0, int* cursor_ext = nullptr, bool cursor_final = false);
// cursor_ext (optional): the caller's array takes the place of the cursors, so that the counts
// survive the call; cursor_final: it already holds the final counts (every pair's place is known
// from an earlier call), so it is neither zeroed nor written.

// rank[B, P, U] = index of pair (row, slot) among the pairs naming the same neighbour (-1 for an
// index out of range), incoming[B, P+nghost] = number of pairs naming each atom.
int pair_ranks(int B, int P, int U, int nghost, const int* binum, const int* bnumneigh, const int* bfirstneigh,
               int* rank, int* incoming, hipStream_t stream);
// With etot or virial given, the same launch also sums the energy / virial partials
// (finish_energy_virial's work, in workgroups of its own behind those of the segments).
template <typename T>
int pair_csr_finish(T* force, const PairCsr& csr, hipStream_t stream, T* etot = nullptr, T* virial = nullptr,
                    const double* partial = nullptr, int B = 0, int nblocks = 0);

// out[b*out_stride + c] = sum over blocks of partial[(b*nblocks + block)*src_stride + c], c < ncomp,
// with a fixed summation tree (fp64).  timed = false: the launch is never bracketed by timing events
// (which are created on first use), for the callers that must not allocate.
template <typename T>
int finish_partials(T* out, const double* partial, int B, int nblocks, int ncomp, int src_stride,
                    int out_stride, hipStream_t stream, bool timed = true);

// One workgroup of 256 threads: component c (0 energy, 1..9 virial) of structure b from
// partial[(b*nblocks + block)*10 + c], summed over the blocks by a fixed tree (fp64).
template <typename T>
__device__ __forceinline__ void finish_ev_body(T* etot, T* virial, const double* partial, int nblocks, int b, int c,
                                               double* sh)
{
    if (c == 0 ? etot == nullptr : virial == nullptr) return;      // uniform over the workgroup
    const double* src = partial + ((size_t)b * nblocks) * 10 + c;
    double acc = 0.0;
    for (int k = threadIdx.x; k < nblocks; k += 256) acc += src[(size_t)k * 10];
    sh[threadIdx.x] = acc;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
        if ((int)threadIdx.x < s) sh[threadIdx.x] += sh[threadIdx.x + s];
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        if (c == 0) etot[b] = (T)sh[0];
        else virial[(size_t)b * 9 + c - 1] = (T)sh[0];
    }
}

// etot[b] and virial[b*9 + c] from partial[(b*nblocks + block)*10 + (0 | 1 + c)], one launch; either
// output may be null.
template <typename T>
int finish_energy_virial(T* etot, T* virial, const double* partial, int B, int nblocks, hipStream_t stream);

int fill_zero(void* ptr, size_t bytes, hipStream_t stream);
int fill_zero2(void* ptr, size_t bytes, void* ptr2, size_t bytes2, hipStream_t stream);   // two ranges, one launch

// out[i] = in[0] + ... + in[i-1] for i < n (out must not alias in); tmp holds
// scan_tmp_ints(n) ints, and tmp[ceil(n/2048)] receives the total.
int scan_tmp_ints(int n);
int exclusive_scan_i32(const int* in, int* out, int n, int* tmp, hipStream_t stream);

}  // namespace a2p
