// Deterministic neighbour-pair reduction: every pair (row, slot) of a structure holds a
// derivative g = dE_row/dr_(row,slot); atom j receives  -sum of g over the pairs whose
// neighbour is j  on top of the sum over its own row that the producing kernel stored.
//
// Steps (all on `stream`):
//   1. count  : integer histogram of neighbour indices            (HBM: reads valid firstneigh)
//   2. scan   : exclusive prefix sum -> segment offsets
//   3. fill   : pair derivatives copied into their target's segment (position by integer
//               atomic; the order inside a segment is therefore arbitrary)
//   4. reduce : per target, order-independent sum: every term is converted to 64-bit fixed
//               point against the segment's largest magnitude, integers are added (exact,
//               associative), the total is converted back.  The result is identical for
//               any arrival order, so the output is bit-reproducible run to run; the
//               conversion error per term is below 2^-37 (fp32 inputs) / 2^-52 (fp64 inputs)
//               of the largest term, i.e. below the rounding error of a floating sum.
// No floating-point atomics are used.
#include "a2p_common.h"

namespace a2p {

namespace {

constexpr int SCAN_BLOCK = 256;
constexpr int SCAN_ITEMS = 8;   // items per thread
constexpr int SCAN_TILE = SCAN_BLOCK * SCAN_ITEMS;

__global__ void count_kernel(int* __restrict__ counts, int* __restrict__ rank, int B, int P, int U, int NF,
                             const int* __restrict__ binum, const int* __restrict__ bnumneigh,
                             const int* __restrict__ bfirstneigh, int* __restrict__ status)
{
    // one wave per row; lanes stride the valid slots (coalesced over the row).  With `rank` the
    // pair also learns its place inside its target's segment.
    const int wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int lane = threadIdx.x & 63;
    if (wave >= B * P) return;
    const int b = wave / P, ii = wave - b * P;
    if (ii >= binum[b]) return;
    int nn = bnumneigh[wave];
    if (nn > U) {
        if (lane == 0) atomicOr(status, ST_NEIGH_OVERFLOW);
        nn = U;
    }
    const int* row = bfirstneigh + (size_t)wave * U;
    for (int s = lane; s < nn; s += 64) {
        int j = row[s];
        if ((unsigned)j >= (unsigned)NF) {
            atomicOr(status, ST_BAD_NEIGHBOR);
            if (rank) rank[(size_t)wave * U + s] = -1;
            continue;
        }
        if (rank) rank[(size_t)wave * U + s] = atomicAdd(&counts[(size_t)b * NF + j], 1);
        else atomicAdd(&counts[(size_t)b * NF + j], 1);
    }
}

// ---- three-phase exclusive scan over int32 ------------------------------------------------
__global__ void scan_tile_sums(const int* __restrict__ in, int* __restrict__ tile_sums, int n)
{
    __shared__ int sh[SCAN_BLOCK / 64];
    const size_t base = (size_t)blockIdx.x * SCAN_TILE;
    int acc = 0;
#pragma unroll
    for (int k = 0; k < SCAN_ITEMS; k++) {
        size_t i = base + (size_t)threadIdx.x * SCAN_ITEMS + k;
        if (i < (size_t)n) acc += in[i];
    }
    acc = wave_sum(acc);
    if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        int t = 0;
        for (int w = 0; w < SCAN_BLOCK / 64; w++) t += sh[w];
        tile_sums[blockIdx.x] = t;
    }
}

// single block: exclusive scan of the tile sums (ntiles is small: n / 2048)
__global__ void scan_tile_offsets(int* __restrict__ tile_sums, int ntiles, int* __restrict__ total)
{
    __shared__ int sh[1024 / 64];
    __shared__ int carry_sh;
    if (threadIdx.x == 0) carry_sh = 0;
    __syncthreads();
    for (int base = 0; base < ntiles; base += 1024) {
        int i = base + threadIdx.x;
        int v = i < ntiles ? tile_sums[i] : 0;
        int incl = wave_inclusive_scan(v);
        if ((threadIdx.x & 63) == 63) sh[threadIdx.x >> 6] = incl;
        __syncthreads();
        int wave_off = 0;
        for (int w = 0; w < (int)(threadIdx.x >> 6); w++) wave_off += sh[w];
        int carry = carry_sh;
        if (i < ntiles) tile_sums[i] = carry + wave_off + incl - v;
        __syncthreads();
        if (threadIdx.x == 1023) carry_sh = carry + wave_off + incl;
        __syncthreads();
    }
    if (threadIdx.x == 0) *total = carry_sh;
}

__global__ void scan_apply(const int* __restrict__ in, int* __restrict__ out,
                           const int* __restrict__ tile_offsets, int n)
{
    __shared__ int sh[SCAN_BLOCK / 64];
    const size_t base = (size_t)blockIdx.x * SCAN_TILE + (size_t)threadIdx.x * SCAN_ITEMS;
    int v[SCAN_ITEMS];
    int acc = 0;
#pragma unroll
    for (int k = 0; k < SCAN_ITEMS; k++) {
        size_t i = base + k;
        v[k] = i < (size_t)n ? in[i] : 0;
        acc += v[k];
    }
    int incl = wave_inclusive_scan(acc);
    if ((threadIdx.x & 63) == 63) sh[threadIdx.x >> 6] = incl;
    __syncthreads();
    int off = tile_offsets[blockIdx.x] + incl - acc;
    for (int w = 0; w < (int)(threadIdx.x >> 6); w++) off += sh[w];
#pragma unroll
    for (int k = 0; k < SCAN_ITEMS; k++) {
        size_t i = base + k;
        if (i < (size_t)n) out[i] = off;
        off += v[k];
    }
}

template <typename T>
__global__ void fill_kernel(T* __restrict__ seg_g, int* __restrict__ cursor,
                            const int* __restrict__ offsets, const T* __restrict__ pair_g, int B,
                            int P, int U, int NF, const int* __restrict__ binum,
                            const int* __restrict__ bnumneigh, const int* __restrict__ bfirstneigh)
{
    const int wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int lane = threadIdx.x & 63;
    if (wave >= B * P) return;
    const int b = wave / P, ii = wave - b * P;
    if (ii >= binum[b]) return;
    int nn = min(bnumneigh[wave], U);
    const int* row = bfirstneigh + (size_t)wave * U;
    const T* grow = pair_g + (size_t)wave * U * 3;
    for (int s = lane; s < nn; s += 64) {
        int j = row[s];
        if ((unsigned)j >= (unsigned)NF) continue;
        size_t t = (size_t)b * NF + j;
        int pos = offsets[t] + atomicAdd(&cursor[t], 1);
        seg_g[(size_t)pos * 3 + 0] = grow[s * 3 + 0];
        seg_g[(size_t)pos * 3 + 1] = grow[s * 3 + 1];
        seg_g[(size_t)pos * 3 + 2] = grow[s * 3 + 2];
    }
}

// 16 lanes per target atom.  Workgroups from `reduce_blocks` on sum the energy / virial partials
// instead (one component of one structure each), which saves small systems a launch.
template <typename T>
__global__ void reduce_kernel(T* __restrict__ force, const T* __restrict__ seg_g,
                              const int* __restrict__ offsets, const int* __restrict__ counts, int NT,
                              int seg_cap, int reduce_blocks, T* __restrict__ etot, T* __restrict__ virial,
                              const double* __restrict__ partial, int nblocks)
{
    if ((int)blockIdx.x >= reduce_blocks) {
        __shared__ double sh[256];
        const int id = (int)blockIdx.x - reduce_blocks;
        finish_ev_body<T>(etot, virial, partial, nblocks, id / 10, id % 10, sh);
        return;
    }
    const int gid = blockIdx.x * blockDim.x + threadIdx.x;
    const int t = gid >> 4;
    const int sub = gid & 15;
    const bool live = t < NT;
    // seg_cap > 0: segments of fixed capacity, target t owns entries [t*seg_cap, (t+1)*seg_cap)
    const int beg = !live ? 0 : seg_cap > 0 ? t * seg_cap : offsets[t];
    const int cnt = !live ? 0 : seg_cap > 0 ? min(counts[t], seg_cap) : counts[t];
    if constexpr (sizeof(T) == 4) {
        // fp32 segments: every value is rounded to a multiple of 2^q, q chosen from the segment's
        // largest magnitude and its length so that any partial sum of the rounded values fits the
        // 53 bits of a double: the additions are then exact in whatever order they happen.  The
        // first four entries of every lane stay in registers between the two passes.
        float gx[4], gy[4], gz[4];
        float mf = 0.0f;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const int e = sub + 16 * k;
            gx[k] = 0.0f; gy[k] = 0.0f; gz[k] = 0.0f;
            if (e < cnt) {
                const float* g = seg_g + (size_t)(beg + e) * 3;
                gx[k] = g[0]; gy[k] = g[1]; gz[k] = g[2];
            }
            mf = fmaxf(mf, fmaxf(fabsf(gx[k]), fmaxf(fabsf(gy[k]), fabsf(gz[k]))));
            // fmaxf drops a NaN operand: keep it
            if (gx[k] != gx[k] || gy[k] != gy[k] || gz[k] != gz[k]) mf = NAN;
        }
        for (int e = sub + 64; e < cnt; e += 16) {
            const float* g = seg_g + (size_t)(beg + e) * 3;
            const float a0 = g[0], a1 = g[1], a2 = g[2];
            if (!(mf != mf)) mf = fmaxf(mf, fmaxf(fabsf(a0), fmaxf(fabsf(a1), fabsf(a2))));
            if (a0 != a0 || a1 != a1 || a2 != a2) mf = NAN;
        }
#pragma unroll
        for (int off = 8; off > 0; off >>= 1) {
            const float o = __shfl_xor(mf, off, 64);
            mf = (mf != mf || o != o) ? NAN : fmaxf(mf, o);
        }
        if (cnt == 0) return;               // uniform over the 16 lanes of a target
        const bool finite = mf < 3.0e38f && mf == mf;
        double s0 = 0.0, s1 = 0.0, s2 = 0.0;
        const bool any = finite && mf > 0.0f;
        if (any) {
            // |v| < 2^(ex+1), fewer than 2^hb of them: sums stay below 2^(ex+1+hb), so q = ex + hb - 52;
            // (v + C) - C with C = 1.5 * 2^(52+q) rounds v to a multiple of 2^q (needs hb >= 2)
            const int hb = max(32 - __clz(cnt), 2);
            const double C = ldexp(1.5, ilogbf(mf) + hb);
#pragma unroll
            for (int k = 0; k < 4; k++) {
                s0 += ((double)gx[k] + C) - C;
                s1 += ((double)gy[k] + C) - C;
                s2 += ((double)gz[k] + C) - C;
            }
            for (int e = sub + 64; e < cnt; e += 16) {
                const float* g = seg_g + (size_t)(beg + e) * 3;
                s0 += ((double)g[0] + C) - C;
                s1 += ((double)g[1] + C) - C;
                s2 += ((double)g[2] + C) - C;
            }
        }
#pragma unroll
        for (int off = 8; off > 0; off >>= 1) {
            s0 += __shfl_xor(s0, off, 64);
            s1 += __shfl_xor(s1, off, 64);
            s2 += __shfl_xor(s2, off, 64);
        }
        if (sub == 0) {
            T* f = force + (size_t)t * 3;
            if (!finite) {
                f[0] = f[1] = f[2] = (T)NAN;
            } else if (any) {
                f[0] = (T)((double)f[0] - s0);
                f[1] = (T)((double)f[1] - s1);
                f[2] = (T)((double)f[2] - s2);
            }
        }
        return;
    }
    // pass 1: largest magnitude of the segment
    double m = 0.0;
    for (int e = sub; e < cnt; e += 16) {
        const T* g = seg_g + (size_t)(beg + e) * 3;
        m = fmax(m, fmax(fabs((double)g[0]), fmax(fabs((double)g[1]), fabs((double)g[2]))));
    }
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) m = fmax(m, __shfl_xor(m, off, 64));
    if (cnt == 0) return;               // uniform over the 16 lanes of a target
    long long s0 = 0, s1 = 0, s2 = 0;
    double scale = 0.0;
    const bool finite = m < 1.0e300 && m == m;
    if (m < 1.0e-280) m = 0.0;          // nothing but (sub)normal dust: contributes zero
    if (m > 0.0 && finite) {
        int bits = 61 - (32 - __clz(cnt));          // head-room for cnt additions
        scale = ldexp(1.0, bits - 1 - ilogb(m));
        for (int e = sub; e < cnt; e += 16) {
            const T* g = seg_g + (size_t)(beg + e) * 3;
            s0 += __double2ll_rn((double)g[0] * scale);
            s1 += __double2ll_rn((double)g[1] * scale);
            s2 += __double2ll_rn((double)g[2] * scale);
        }
    }
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) {
        s0 += shfl_xor_ll(s0, off);
        s1 += shfl_xor_ll(s1, off);
        s2 += shfl_xor_ll(s2, off);
    }
    if (sub == 0) {
        T* f = force + (size_t)t * 3;
        if (!finite) {
            f[0] = f[1] = f[2] = (T)NAN;
        } else if (m > 0.0) {
            f[0] = (T)((double)f[0] - (double)s0 / scale);
            f[1] = (T)((double)f[1] - (double)s1 / scale);
            f[2] = (T)((double)f[2] - (double)s2 / scale);
        }
    }
}

}  // namespace

int scan_tmp_ints(int n) { return ceil_div(n, SCAN_TILE) + 8; }

int exclusive_scan_i32(const int* in, int* out, int n, int* tmp, hipStream_t stream)
{
    if (n <= 0) return A2P_OK;
    const int ntiles = ceil_div(n, SCAN_TILE);
    prof_begin("scan", stream);
    hipLaunchKernelGGL(scan_tile_sums, dim3(ntiles), dim3(SCAN_BLOCK), 0, stream, in, tmp, n);
    prof_end(stream);
    prof_begin("scan", stream);
    hipLaunchKernelGGL(scan_tile_offsets, dim3(1), dim3(1024), 0, stream, tmp, ntiles, tmp + ntiles);
    prof_end(stream);
    prof_begin("scan", stream);
    hipLaunchKernelGGL(scan_apply, dim3(ntiles), dim3(SCAN_BLOCK), 0, stream, in, out, tmp, n);
    prof_end(stream);
    A2P_HIP_CHECK(hipGetLastError());
    return A2P_OK;
}

template <typename T>
int pair_csr_begin(PairCsr* csr, bool with_rank, int B, int P, int U, int nghost, const int* binum,
                   const int* bnumneigh, const int* bfirstneigh, hipStream_t stream)
{
    const int NF = P + nghost;
    const long long NT = (long long)B * NF;
    const long long rows = (long long)B * P;
    A2P_REQUIRE(NT < (1ll << 31) - SCAN_TILE && rows * U < (1ll << 31), A2P_ERR_INVALID,
                "pair_reduce: batch too large for 32-bit pair indexing");
    const int n = (int)NT;
    const int ntiles = ceil_div(n, SCAN_TILE);
    // workspace: counts[n] | offsets[n] | cursor[n] | tile[ntiles] | total[1] | seg_g[rows*U*3] | rank[rows*U]
    size_t ints = (size_t)n * 3 + ntiles + 8;
    size_t bytes = ((ints * sizeof(int) + 255) / 256) * 256;
    size_t seg_bytes = (((size_t)rows * U * 3 * sizeof(T) + 255) / 256) * 256;
    size_t rank_bytes = with_rank ? (size_t)rows * U * sizeof(int) : 0;
    void* ws = nullptr;
    int rc = ws_get(WS_CSR, bytes + seg_bytes + rank_bytes, &ws);
    if (rc) return rc;
    void* flags = nullptr;
    rc = ws_get(WS_FLAGS, 64, &flags);
    if (rc) return rc;
    csr->n = n;
    csr->seg_cap = 0;
    csr->counts = (int*)ws;
    csr->offsets = csr->counts + n;
    csr->cursor = csr->offsets + n;
    int* tiles = csr->cursor + n;
    csr->seg_g = (void*)((char*)ws + bytes);
    csr->rank = with_rank ? (int*)((char*)ws + bytes + seg_bytes) : nullptr;

    // counts and cursor are adjacent and start at zero (offsets is fully overwritten)
    rc = fill_zero(csr->counts, (size_t)n * sizeof(int), stream);
    if (rc) return rc;
    rc = fill_zero(csr->cursor, (size_t)n * sizeof(int), stream);
    if (rc) return rc;

    const int wave_blocks = ceil_div(rows * 64, 256);
    prof_begin("reduce_count", stream);
    hipLaunchKernelGGL(count_kernel, dim3(wave_blocks), dim3(256), 0, stream, csr->counts, csr->rank, B, P,
                       U, NF, binum, bnumneigh, bfirstneigh, (int*)flags);
    prof_end(stream);
    return exclusive_scan_i32(csr->counts, csr->offsets, n, tiles, stream);
}

static thread_local int g_seg_capacity = 0;

int pair_segment_capacity(int U) { return g_seg_capacity > U ? g_seg_capacity : U; }

template <typename T>
int pair_fixed_begin(PairCsr* csr, int B, int P, int U_rows, int nghost, hipStream_t stream, void* also_zero,
                     size_t also_bytes, int* cursor_ext, bool cursor_final)
{
    const int U = pair_segment_capacity(U_rows);
    const long long NT = (long long)B * (P + nghost);
    A2P_REQUIRE(NT * U + 1 < (1ll << 31), A2P_ERR_INVALID,
                "pair_reduce: (natoms_pad + nghost) * segment capacity exceeds 32-bit pair indexing");
    const int n = (int)NT;
    // workspace: cursor[n] | seg_g[(n*U + 1) * 3]   (the last entry takes what overflows)
    size_t bytes = (((size_t)n * sizeof(int) + 255) / 256) * 256;
    size_t seg_bytes = ((size_t)n * U + 1) * 3 * sizeof(T);
    void* ws = nullptr;
    int rc = ws_get(WS_CSR, bytes + seg_bytes, &ws);
    if (rc) return rc;
    csr->n = n;
    csr->seg_cap = U;
    csr->counts = nullptr;
    csr->offsets = nullptr;
    csr->rank = nullptr;
    csr->cursor = (int*)ws;
    csr->seg_g = (void*)((char*)ws + bytes);
    if (cursor_ext) csr->cursor = cursor_ext;            // the caller keeps the counts
    if (cursor_ext && cursor_final)                      // ... and they are final: every pair's place is known
        return fill_zero(also_zero, also_bytes, stream);
    return fill_zero2(csr->cursor, (size_t)n * sizeof(int), also_zero, also_bytes, stream);
}

int pair_ranks(int B, int P, int U, int nghost, const int* binum, const int* bnumneigh, const int* bfirstneigh,
               int* rank, int* incoming, hipStream_t stream)
{
    A2P_REQUIRE(B >= 0 && P >= 0 && U >= 1 && nghost >= 0, A2P_ERR_INVALID, "pair_ranks: bad shape");
    A2P_REQUIRE(binum && bnumneigh && bfirstneigh && rank && incoming, A2P_ERR_INVALID, "pair_ranks: null pointer");
    if (B == 0 || P == 0) return A2P_OK;
    const int NF = P + nghost;
    void* flags = nullptr;
    int rc = ws_get(WS_FLAGS, 64, &flags);
    if (rc) return rc;
    rc = fill_zero(incoming, (size_t)B * NF * sizeof(int), stream);
    if (rc) return rc;
    prof_begin("pair_ranks", stream);
    hipLaunchKernelGGL(count_kernel, dim3(ceil_div((long long)B * P * 64, 256)), dim3(256), 0, stream, incoming, rank,
                       B, P, U, NF, binum, bnumneigh, bfirstneigh, (int*)flags);
    prof_end(stream);
    A2P_HIP_CHECK(hipGetLastError());
    return A2P_OK;
}

template <typename T>
int pair_csr_finish(T* force, const PairCsr& csr, hipStream_t stream, T* etot, T* virial, const double* partial,
                    int B, int nblocks)
{
    // with ranks every counted pair has its place in the segment; otherwise the cursor holds
    // how many entries were filled
    const int reduce_blocks = ceil_div((long long)csr.n * 16, 256);
    const int ev_blocks = (etot || virial) ? 10 * B : 0;
    prof_begin("reduce_sum", stream);
    hipLaunchKernelGGL(reduce_kernel<T>, dim3(reduce_blocks + ev_blocks), dim3(256), 0, stream,
                       force, (const T*)csr.seg_g, csr.offsets, csr.rank ? csr.counts : csr.cursor, csr.n,
                       csr.seg_cap, reduce_blocks, etot, virial, partial, nblocks);
    prof_end(stream);
    A2P_HIP_CHECK(hipGetLastError());
    return A2P_OK;
}

template <typename T>
int pair_reduce(T* force, const T* pair_g, int B, int P, int U, int nghost, const int* binum,
                const int* bnumneigh, const int* bfirstneigh, hipStream_t stream)
{
    PairCsr csr;
    int rc = pair_csr_begin<T>(&csr, false, B, P, U, nghost, binum, bnumneigh, bfirstneigh, stream);
    if (rc) return rc;
    const long long rows = (long long)B * P;
    const int wave_blocks = ceil_div(rows * 64, 256);
    prof_begin("reduce_fill", stream);
    hipLaunchKernelGGL(fill_kernel<T>, dim3(wave_blocks), dim3(256), 0, stream, (T*)csr.seg_g, csr.cursor,
                       csr.offsets, pair_g, B, P, U, P + nghost, binum, bnumneigh, bfirstneigh);
    prof_end(stream);
    return pair_csr_finish<T>(force, csr, stream);
}

template int pair_csr_begin<float>(PairCsr*, bool, int, int, int, int, const int*, const int*, const int*, hipStream_t);
template int pair_csr_begin<double>(PairCsr*, bool, int, int, int, int, const int*, const int*, const int*, hipStream_t);
template int pair_fixed_begin<float>(PairCsr*, int, int, int, int, hipStream_t, void*, size_t, int*, bool);
template int pair_fixed_begin<double>(PairCsr*, int, int, int, int, hipStream_t, void*, size_t, int*, bool);
template int pair_csr_finish<float>(float*, const PairCsr&, hipStream_t, float*, float*, const double*, int, int);
template int pair_csr_finish<double>(double*, const PairCsr&, hipStream_t, double*, double*, const double*, int, int);
template int pair_reduce<float>(float*, const float*, int, int, int, int, const int*, const int*,
                                const int*, hipStream_t);
template int pair_reduce<double>(double*, const double*, int, int, int, int, const int*, const int*,
                                 const int*, hipStream_t);

}  // namespace a2p

// largest number of pairs naming one atom: counts (the histogram of a2p_pair_ranks without the ranks), then the maximum
__global__ void incoming_max_kernel(const int* __restrict__ v, int n, int* __restrict__ out)
{
    __shared__ int sh[4];
    int m = 0;
    for (int i = blockIdx.x * 256 + threadIdx.x; i < n; i += gridDim.x * 256) m = max(m, v[i]);
    m = a2p::wave_max(m);
    if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) atomicMax(out, max(max(sh[0], sh[1]), max(sh[2], sh[3])));
}

extern "C" int a2p_pair_segment_capacity(int capacity)
{
    const int old = a2p::g_seg_capacity;
    a2p::g_seg_capacity = capacity > 0 ? capacity : 0;
    return old;
}

extern "C" int a2p_pair_incoming_max(int batch, int natoms_pad, int umax, int nghost, const int* binum,
                                     const int* bnumneigh, const int* bfirstneigh, int* max_incoming, void* stream_)
{
    using namespace a2p;
    hipStream_t stream = (hipStream_t)stream_;
    A2P_REQUIRE(batch >= 0 && natoms_pad >= 0 && umax >= 1 && nghost >= 0, A2P_ERR_INVALID, "pair_incoming_max: bad shape");
    A2P_REQUIRE(binum && bnumneigh && bfirstneigh && max_incoming, A2P_ERR_INVALID, "pair_incoming_max: null pointer");
    *max_incoming = 0;
    if (batch == 0 || natoms_pad == 0) return A2P_OK;
    int rc = enter_stream(stream);
    if (rc) return rc;
    const int NF = natoms_pad + nghost;
    const size_t n = (size_t)batch * NF;
    void* ws = nullptr;
    rc = ws_get(WS_CSR, (n + 64) * sizeof(int), &ws);
    if (rc) return rc;
    void* flags = nullptr;
    rc = ws_get(WS_FLAGS, 64, &flags);
    if (rc) return rc;
    int* counts = (int*)ws;
    rc = fill_zero(counts, (n + 64) * sizeof(int), stream);
    if (rc) return rc;
    hipLaunchKernelGGL(count_kernel, dim3(ceil_div((long long)batch * natoms_pad * 64, 256)), dim3(256), 0, stream, counts,
                       (int*)nullptr, batch, natoms_pad, umax, NF, binum, bnumneigh, bfirstneigh, (int*)flags);
    hipLaunchKernelGGL(incoming_max_kernel, dim3(std::min(ceil_div((long long)n, 256), 1024)), dim3(256), 0, stream,
                       (const int*)counts, (int)n, counts + n);
    A2P_HIP_CHECK(hipGetLastError());
    A2P_HIP_CHECK(hipMemcpyAsync(max_incoming, counts + n, sizeof(int), hipMemcpyDeviceToHost, stream));
    A2P_HIP_CHECK(hipStreamSynchronize(stream));
    return A2P_OK;
}

extern "C" int a2p_pair_ranks(int batch, int natoms_pad, int umax, int nghost, const int* binum, const int* bnumneigh,
                              const int* bfirstneigh, int* rank, int* incoming, void* stream)
{
    return a2p::pair_ranks(batch, natoms_pad, umax, nghost, binum, bnumneigh, bfirstneigh, rank, incoming,
                           (hipStream_t)stream);
}
