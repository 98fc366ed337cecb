// Error state, per-device workspace and small utility kernels of libai2pot_hip.so.
#include "a2p_common.h"

#include <mutex>
#include <string>
#include <vector>

namespace a2p {

static thread_local std::string g_err;

void set_error(const char* fmt, ...)
{
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_err = buf;
}

const char* last_error() { return g_err.c_str(); }

namespace {
struct Buf {
    void* ptr = nullptr;
    size_t bytes = 0;
};
struct DeviceWs {
    Buf slot[WS_NSLOTS];
};
std::mutex g_ws_mutex;
std::vector<DeviceWs> g_ws;
unsigned long long g_ws_generation = 0;   // bumped whenever a buffer is freed or replaced
}  // namespace

int ws_get(int slot, size_t bytes, void** out)
{
    int dev = 0;
    A2P_HIP_CHECK(hipGetDevice(&dev));
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    if ((int)g_ws.size() <= dev) g_ws.resize(dev + 1);
    Buf& b = g_ws[dev].slot[slot];
    if (bytes > b.bytes) {
        if (b.ptr) {
            A2P_HIP_CHECK(hipFree(b.ptr));          // synchronises: no kernel still uses it
            g_ws_generation++;                      // ... but a captured graph may still name it
        }
        b.ptr = nullptr;
        b.bytes = 0;
        size_t want = bytes + bytes / 8 + 256;      // head-room so small growth does not realloc
        A2P_HIP_CHECK(hipMalloc(&b.ptr, want));
        b.bytes = want;
        if (slot == WS_FLAGS || slot == WS_NEP_CLAIMS) A2P_HIP_CHECK(hipMemset(b.ptr, 0, want));
    }
    *out = b.ptr;
    return A2P_OK;
}

int ws_drop(int slot)
{
    int dev = 0;
    A2P_HIP_CHECK(hipGetDevice(&dev));
    A2P_HIP_CHECK(hipDeviceSynchronize());
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    if ((int)g_ws.size() <= dev) return A2P_OK;
    Buf& b = g_ws[dev].slot[slot];
    if (b.ptr) {
        A2P_HIP_CHECK(hipFree(b.ptr));
        g_ws_generation++;
    }
    b.ptr = nullptr;
    b.bytes = 0;
    return A2P_OK;
}

size_t ws_bytes()
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 0;
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    if ((int)g_ws.size() <= dev) return 0;
    size_t total = 0;
    for (const Buf& b : g_ws[dev].slot) total += b.bytes;
    return total;
}

int ws_release()
{
    int dev = 0;
    A2P_HIP_CHECK(hipGetDevice(&dev));
    A2P_HIP_CHECK(hipDeviceSynchronize());          // no kernel of any stream still uses the buffers
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    if ((int)g_ws.size() <= dev) return A2P_OK;
    for (Buf& b : g_ws[dev].slot) {
        if (b.ptr) A2P_HIP_CHECK(hipFree(b.ptr));
        b.ptr = nullptr;
        b.bytes = 0;
    }
    g_ws_generation++;
    return A2P_OK;
}

// ---- per-kernel timing ---------------------------------------------------------------------
namespace {
struct ProfRec {
    const char* label;
    hipEvent_t start, stop;
};
bool g_prof_on = false;
std::mutex g_prof_mutex;
std::vector<ProfRec> g_prof_recs;
thread_local hipEvent_t g_prof_pending_stop = nullptr;
std::string g_prof_select;                 // ",label,label,": only these are timed; empty: all
std::vector<hipEvent_t> g_prof_pool;       // events of reported records, reused (one device's)
int g_prof_pool_dev = -1;

bool prof_event(hipEvent_t* e)
{
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess) return false;
    if (dev != g_prof_pool_dev) {
        for (hipEvent_t old : g_prof_pool) (void)hipEventDestroy(old);
        g_prof_pool.clear();
        g_prof_pool_dev = dev;
    }
    if (!g_prof_pool.empty()) {
        *e = g_prof_pool.back();
        g_prof_pool.pop_back();
        return true;
    }
    return hipEventCreate(e) == hipSuccess;
}
}  // namespace

// The workspace is shared by every call on a device, so work of this library on two streams must not overlap.
// Every launch passes through prof_begin, which calls enter_stream: when the stream differs from the one the
// previous launch on this device used, the device is synchronised first (callers that keep to one stream never
// pay for it).  Entry points whose launches are not bracketed by prof_begin call enter_stream themselves.  A
// stream that is being captured is left alone: a capture keeps to itself, and its replays are ordered by whoever
// launches them.
namespace {
std::mutex g_stream_mutex;
std::vector<hipStream_t> g_last_stream;
std::vector<char> g_have_stream;
}  // namespace

int enter_stream(hipStream_t stream)
{
    int dev = 0;
    A2P_HIP_CHECK(hipGetDevice(&dev));
    std::lock_guard<std::mutex> lock(g_stream_mutex);
    if ((int)g_last_stream.size() <= dev) { g_last_stream.resize(dev + 1, nullptr); g_have_stream.resize(dev + 1, 0); }
    if (g_have_stream[dev] && g_last_stream[dev] == stream) return A2P_OK;
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &st) != hipSuccess) { (void)hipGetLastError(); return A2P_OK; }
    if (st != hipStreamCaptureStatusNone) return A2P_OK;
    if (g_have_stream[dev]) A2P_HIP_CHECK(hipDeviceSynchronize());
    g_last_stream[dev] = stream;
    g_have_stream[dev] = 1;
    return A2P_OK;
}

void prof_begin(const char* label, hipStream_t stream)
{
    (void)enter_stream(stream);        // a failed synchronisation stays pending and fails the call's own check
    if (!g_prof_on) return;
    std::lock_guard<std::mutex> lock(g_prof_mutex);
    if (!g_prof_select.empty() && g_prof_select.find("," + std::string(label) + ",") == std::string::npos) return;
    ProfRec r{label, nullptr, nullptr};
    if (!prof_event(&r.start) || !prof_event(&r.stop)) return;
    (void)hipEventRecord(r.start, stream);
    g_prof_pending_stop = r.stop;
    g_prof_recs.push_back(r);
}

void prof_end(hipStream_t stream)
{
    if (!g_prof_on || !g_prof_pending_stop) return;
    (void)hipEventRecord(g_prof_pending_stop, stream);
    g_prof_pending_stop = nullptr;
}

__global__ void fill_zero_kernel(uint32_t* p, size_t nwords)
{
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < nwords; i += stride) p[i] = 0u;
}

__global__ void fill_zero2_kernel(uint32_t* p, size_t nwords, uint32_t* q, size_t mwords)
{
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t k = i; k < nwords; k += stride) p[k] = 0u;
    for (size_t k = i; k < mwords; k += stride) q[k] = 0u;
}

int fill_zero2(void* ptr, size_t bytes, void* ptr2, size_t bytes2, hipStream_t stream)
{
    if (bytes == 0) return fill_zero(ptr2, bytes2, stream);
    if (bytes2 == 0) return fill_zero(ptr, bytes, stream);
    A2P_REQUIRE(bytes % 4 == 0 && bytes2 % 4 == 0, A2P_ERR_INVALID, "fill_zero: size not a multiple of 4");
    const size_t nwords = bytes / 4, mwords = bytes2 / 4;
    const int blocks = (int)std::min<size_t>((std::max(nwords, mwords) + 255) / 256, 256 * 32);
    prof_begin("fill_zero", stream);
    hipLaunchKernelGGL(fill_zero2_kernel, dim3(blocks), dim3(256), 0, stream, (uint32_t*)ptr, nwords,
                       (uint32_t*)ptr2, mwords);
    prof_end(stream);
    A2P_HIP_CHECK(hipGetLastError());
    return A2P_OK;
}

int fill_zero(void* ptr, size_t bytes, hipStream_t stream)
{
    if (bytes == 0) return A2P_OK;
    A2P_REQUIRE(bytes % 4 == 0, A2P_ERR_INVALID, "fill_zero: size not a multiple of 4");
    size_t nwords = bytes / 4;
    int blocks = (int)std::min<size_t>((nwords + 255) / 256, 256 * 32);
    prof_begin("fill_zero", stream);
    hipLaunchKernelGGL(fill_zero_kernel, dim3(blocks), dim3(256), 0, stream, (uint32_t*)ptr, nwords);
    prof_end(stream);
    A2P_HIP_CHECK(hipGetLastError());
    return A2P_OK;
}

// One block per (structure, component): sums the per-block partials in block order.
template <typename T>
__global__ void finish_partials_kernel(T* out, const double* partial, int nblocks, int src_stride,
                                       int out_stride)
{
    __shared__ double sh[256];
    const int b = blockIdx.y, c = blockIdx.x;
    const double* src = partial + ((size_t)b * nblocks) * src_stride + c;
    // fixed assignment of blocks to threads, fixed tree: the result does not depend on timing
    double acc = 0.0;
    for (int k = threadIdx.x; k < nblocks; k += 256) acc += src[(size_t)k * src_stride];
    sh[threadIdx.x] = acc;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
        if ((int)threadIdx.x < s) sh[threadIdx.x] += sh[threadIdx.x + s];
        __syncthreads();
    }
    if (threadIdx.x == 0) out[(size_t)b * out_stride + c] = (T)sh[0];
}

template <typename T>
int finish_partials(T* out, const double* partial, int B, int nblocks, int ncomp, int src_stride,
                    int out_stride, hipStream_t stream, bool timed)
{
    if (timed) prof_begin("finish_partials", stream);
    hipLaunchKernelGGL(finish_partials_kernel<T>, dim3(ncomp, B), dim3(256), 0, stream, out, partial,
                       nblocks, src_stride, out_stride);
    if (timed) prof_end(stream);
    A2P_HIP_CHECK(hipGetLastError());
    return A2P_OK;
}
// Energy (component 0) and virial (components 1-9) of partial[.., 10] in one launch; either output
// may be null.  Same summation per component as finish_partials.
template <typename T>
__global__ void finish_ev_kernel(T* etot, T* virial, const double* partial, int nblocks)
{
    __shared__ double sh[256];
    finish_ev_body<T>(etot, virial, partial, nblocks, blockIdx.y, blockIdx.x, sh);
}

template <typename T>
int finish_energy_virial(T* etot, T* virial, const double* partial, int B, int nblocks, hipStream_t stream)
{
    if (!etot && !virial) return A2P_OK;
    prof_begin("finish_partials", stream);
    hipLaunchKernelGGL(finish_ev_kernel<T>, dim3(10, B), dim3(256), 0, stream, etot, virial, partial, nblocks);
    prof_end(stream);
    A2P_HIP_CHECK(hipGetLastError());
    return A2P_OK;
}
template int finish_energy_virial<float>(float*, float*, const double*, int, int, hipStream_t);
template int finish_energy_virial<double>(double*, double*, const double*, int, int, hipStream_t);
template int finish_partials<float>(float*, const double*, int, int, int, int, int, hipStream_t, bool);
template int finish_partials<double>(double*, const double*, int, int, int, int, int, hipStream_t, bool);

}  // namespace a2p

extern "C" {

const char* a2p_last_error(void) { return a2p::last_error(); }

int a2p_abi_version(void) { return 1; }

size_t a2p_workspace_bytes(void) { return a2p::ws_bytes(); }

int a2p_workspace_release(void) { return a2p::ws_release(); }

unsigned long long a2p_workspace_generation(void)
{
    std::lock_guard<std::mutex> lock(a2p::g_ws_mutex);
    return a2p::g_ws_generation;
}

void a2p_profile_enable(int on)
{
    std::lock_guard<std::mutex> lock(a2p::g_prof_mutex);
    a2p::g_prof_on = on != 0;
}

void a2p_profile_select(const char* labels)
{
    std::lock_guard<std::mutex> lock(a2p::g_prof_mutex);
    a2p::g_prof_select.clear();
    if (labels && labels[0]) a2p::g_prof_select = "," + std::string(labels) + ",";
}

int a2p_profile_report(char* buf, size_t buflen)
{
    A2P_HIP_CHECK(hipDeviceSynchronize());
    std::lock_guard<std::mutex> lock(a2p::g_prof_mutex);
    struct Acc { const char* label; double ms; long count; };
    std::vector<Acc> acc;
    for (auto& r : a2p::g_prof_recs) {
        float ms = 0.f;
        if (hipEventElapsedTime(&ms, r.start, r.stop) == hipSuccess) {
            bool found = false;
            for (auto& a : acc)
                if (std::string(a.label) == r.label) { a.ms += ms; a.count++; found = true; break; }
            if (!found) acc.push_back({r.label, (double)ms, 1});
        }
        int dev = -1;
        if (hipGetDevice(&dev) == hipSuccess && dev == a2p::g_prof_pool_dev && a2p::g_prof_pool.size() < 4096) {
            a2p::g_prof_pool.push_back(r.start);
            a2p::g_prof_pool.push_back(r.stop);
        } else {
            (void)hipEventDestroy(r.start);
            (void)hipEventDestroy(r.stop);
        }
    }
    a2p::g_prof_recs.clear();
    size_t used = 0;
    if (buf && buflen) buf[0] = 0;
    for (auto& a : acc) {
        int n = snprintf(buf + used, used < buflen ? buflen - used : 0, "%s %ld %.6f\n", a.label, a.count, a.ms);
        if (n < 0 || used + (size_t)n >= buflen) break;
        used += (size_t)n;
    }
    return A2P_OK;
}

int a2p_check_status(void* stream_)
{
    hipStream_t stream = (hipStream_t)stream_;
    void* flags = nullptr;
    int rc = a2p::ws_get(a2p::WS_FLAGS, 64, &flags);
    if (rc) return rc;
    int host = 0;
    A2P_HIP_CHECK(hipMemcpyAsync(&host, flags, sizeof(int), hipMemcpyDeviceToHost, stream));
    A2P_HIP_CHECK(hipStreamSynchronize(stream));
    if (host == 0) return A2P_OK;
    rc = a2p::fill_zero(flags, 64, stream);
    if (rc) return rc;
    A2P_HIP_CHECK(hipStreamSynchronize(stream));
    if (host & a2p::ST_SEG_OVERFLOW) {
        a2p::set_error("an atom is named by more pairs than its reduction segment holds (the list is not symmetric, or "
                       "ghosts collect the pairs of several rows): forces of this call are incomplete; call again after "
                       "a2p_pair_segment_capacity(a2p_pair_incoming_max(...))");
        return A2P_ERR_SEGMENT;
    }
    if (host & a2p::ST_GRID_BOUND) {
        a2p::set_error("neighbour list: the bin box around the atoms outgrew the bound taken from the last synchronised "
                       "build (or the coordinates are not finite); the lists of this build are empty: build again "
                       "after a2p_nblist_sync_free(0)");
        return A2P_ERR_GRID;
    }
    if (host & a2p::ST_NEIGH_OVERFLOW) {
        a2p::set_error("a neighbour count exceeds umax_num_neigh_atoms");
        return A2P_ERR_OVERFLOW;
    }
    a2p::set_error("device-side input check failed:%s%s",
                   (host & a2p::ST_BAD_NEIGHBOR) ? " neighbour index outside [0, natoms_pad+nghost)" : "",
                   (host & a2p::ST_BAD_TYPE) ? " type index outside [0, ntypes)" : "");
    return A2P_ERR_INPUT;
}
}
