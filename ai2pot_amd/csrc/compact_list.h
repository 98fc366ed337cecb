// Compact neighbour lists in processing order: what the neighbour-list kernel hands to the NEP
// gather kernels when both run inside this library (no counterpart in the reference, whose only
// list format is the padded [natoms, umax] arrays of source/nblist/include/neighborList.h:532-578).
//
// Atoms are processed in a space-filling order: position p handles atom order[p].  64 consecutive
// positions form a tile (one wavefront).  A position owns umax entry slots of 4 values each,
// [x y z bits], bits = neighbour's position in the processing order | neighbour species << 28.  Neighbours beyond the inner
// (angular) cutoff fill the slots from 0 upwards, neighbours inside it from umax-1 downwards;
// neighbours beyond the outer (radial) cutoff are left out.  The slots are stored in chunks of 8:
//     slot e of position p  ->  entry ((tile * NCH + e / 8) * 64 + p % 64) * 8 + e % 8,   NCH = umax / 8
// so the wavefront that builds one position's list writes 128-byte pieces, and the wavefront that
// consumes a tile reads chunk c of all its 64 positions as one contiguous 8 KiB block (fp32).
// One device buffer holds everything:  order[Npad] | n_outer[Npad] | n_inner[Npad] | entries,
// Npad = natoms rounded up to a multiple of 64, the entries 256-byte aligned.
#pragma once
#include <hip/hip_runtime.h>
#include <cstddef>
#include <cstdint>

namespace a2p {

constexpr int CL_TILE = 64;            // positions per tile
constexpr int CL_CHUNK = 8;            // slots per chunk
constexpr int CL_TYPE_SHIFT = 28;      // bits = position | species << 28
constexpr int CL_INDEX_MASK = (1 << CL_TYPE_SHIFT) - 1;
// Inside the list build only: set in the index word of a neighbour that is a periodic image (not the atom in
// the cell itself); finished entries do not carry it.  Atom indices therefore stay below 2^27.
constexpr int CL_IMAGE_BIT = 1 << 27;

struct CompactLayout {
    int natoms, umax, npad, nch, ntiles;
    size_t off_order, off_outer, off_inner, off_entries, bytes;
};

inline bool compact_supported(int natoms, int umax)
{
    return natoms > 0 && natoms < CL_IMAGE_BIT && umax >= CL_CHUNK && umax % CL_CHUNK == 0;
}

inline CompactLayout compact_layout(int natoms, int umax, size_t elem)
{
    CompactLayout L;
    L.natoms = natoms;
    L.umax = umax;
    L.ntiles = (natoms + CL_TILE - 1) / CL_TILE;
    L.npad = L.ntiles * CL_TILE;
    L.nch = umax / CL_CHUNK;
    L.off_order = 0;
    L.off_outer = (size_t)L.npad * sizeof(int);
    L.off_inner = 2 * (size_t)L.npad * sizeof(int);
    L.off_entries = ((3 * (size_t)L.npad * sizeof(int) + 255) / 256) * 256;
    L.bytes = L.off_entries + (size_t)L.npad * umax * 4 * elem;
    return L;
}

// Device-side view of the buffer
template <typename T>
struct CompactView {
    int natoms, umax, npad, nch;
    int* order;       // [npad] atom handled at each position (positions >= natoms: undefined)
    int* n_outer;     // [npad] neighbours between the two cutoffs (slots 0 .. n_outer-1)
    int* n_inner;     // [npad] neighbours inside the inner cutoff (slots umax-1 .. umax-n_inner)
    T* entries;       // 4 values per slot
};

template <typename T>
inline CompactView<T> compact_view(void* buffer, int natoms, int umax)
{
    const CompactLayout L = compact_layout(natoms, umax, sizeof(T));
    CompactView<T> v;
    v.natoms = natoms; v.umax = umax; v.npad = L.npad; v.nch = L.nch;
    v.order = (int*)((char*)buffer + L.off_order);
    v.n_outer = (int*)((char*)buffer + L.off_outer);
    v.n_inner = (int*)((char*)buffer + L.off_inner);
    v.entries = (T*)((char*)buffer + L.off_entries);
    return v;
}

// first value of chunk `c` of tile `tile` (64 positions x 8 slots x 4 values follow contiguously)
template <typename T>
__host__ __device__ __forceinline__ size_t compact_chunk_offset(int nch, int tile, int c)
{
    return ((size_t)tile * nch + c) * (CL_TILE * CL_CHUNK * 4);
}

// first value of slot e of position p
__host__ __device__ __forceinline__ size_t compact_slot_offset(int nch, int p, int e)
{
    return ((((size_t)(p >> 6) * nch + (e >> 3)) * CL_TILE + (p & 63)) * CL_CHUNK + (e & 7)) * 4;
}

}  // namespace a2p
