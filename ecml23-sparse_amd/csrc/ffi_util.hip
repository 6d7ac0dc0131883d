// Small helpers: workspace pool, device properties, matrix transpose.
#include "ffi_internal.h"
#include "ffi_lds_tile.h"

#include <algorithm>
#include <deque>
#include <mutex>
#include <vector>

namespace ffi {
namespace {

struct WsEntry {
    int device;
    hipStream_t stream;
    int slot;
    void* ptr;
    size_t bytes;
};
std::mutex g_ws_mutex;
std::vector<WsEntry> g_ws;

struct StreamMutex {
    int device;
    hipStream_t stream;
    std::recursive_mutex mutex;
    StreamMutex(int d, hipStream_t s) : device(d), stream(s) {}
};
std::mutex g_stream_mutexes_guard;
std::deque<StreamMutex> g_stream_mutexes;      // a deque: entries are never moved or removed

constexpr int kTrTile = 32;

// 32x32 tiles through LDS (padded), coalesced on both sides.
__global__ __launch_bounds__(kTrTile * 8) void transpose_kernel(const float* __restrict__ src,
                                                                 float* __restrict__ dst, int rows, int cols, int src_ld,
                                                                 int dst_ld) {
    __shared__ float tile[kTrTile][kTrTile + 1];
    const int c0 = blockIdx.x * kTrTile, r0 = blockIdx.y * kTrTile;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    for (int i = ty; i < kTrTile; i += 8) {
        const int r = r0 + i, c = c0 + tx;
        tile[i][tx] = (r < rows && c < cols) ? src[(size_t)r * src_ld + c] : 0.f;
    }
    __syncthreads();
    for (int i = ty; i < kTrTile; i += 8) {
        const int c = c0 + i, r = r0 + tx;
        if (r < rows && c < cols) dst[(size_t)c * dst_ld + r] = tile[tx][i];
    }
}

}  // namespace

StreamCall::StreamCall(hipStream_t s) : mutex_(nullptr) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess) { (void)hipGetLastError(); return; }   // the call itself will report the missing device
    std::recursive_mutex* m = nullptr;
    {
        std::lock_guard<std::mutex> lock(g_stream_mutexes_guard);
        for (StreamMutex& e : g_stream_mutexes)
            if (e.device == dev && e.stream == s) m = &e.mutex;
        if (!m) {
            g_stream_mutexes.emplace_back(dev, s);
            m = &g_stream_mutexes.back().mutex;
        }
    }
    m->lock();
    mutex_ = m;
}

StreamCall::~StreamCall() {
    if (mutex_) static_cast<std::recursive_mutex*>(mutex_)->unlock();
}

int device_cu_count() {
    static int cached[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    if (cached[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cached[dev] = n;
    }
    return cached[dev];
}

int workspace_get(hipStream_t s, int slot, size_t bytes, void** out) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess) return FFI_ERR_NO_DEVICE;
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    for (WsEntry& e : g_ws) {
        if (e.device == dev && e.stream == s && e.slot == slot) {
            if (e.bytes < bytes) {
                // the old buffer may still be in use by work queued on this stream
                FFI_HIP_TRY(hipStreamSynchronize(s));
                (void)hipFree(e.ptr);
                e.ptr = nullptr; e.bytes = 0;
                if (hipMalloc(&e.ptr, bytes) != hipSuccess) { (void)hipGetLastError(); return FFI_ERR_OUT_OF_MEMORY; }
                e.bytes = bytes;
            }
            *out = e.ptr;
            return FFI_OK;
        }
    }
    WsEntry e{dev, s, slot, nullptr, 0};
    const size_t want = std::max<size_t>(bytes, 256);
    if (hipMalloc(&e.ptr, want) != hipSuccess) { (void)hipGetLastError(); return FFI_ERR_OUT_OF_MEMORY; }
    e.bytes = want;
    g_ws.push_back(e);
    *out = e.ptr;
    return FFI_OK;
}

void workspace_clear(int device) {
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    for (size_t i = 0; i < g_ws.size();) {
        if (g_ws[i].device == device) {
            (void)hipFree(g_ws[i].ptr);
            g_ws.erase(g_ws.begin() + i);
        } else {
            ++i;
        }
    }
}

size_t workspace_bytes(int device) {
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    size_t total = 0;
    for (const WsEntry& e : g_ws)
        if (e.device == device) total += e.bytes;
    return total;
}

int launch_transpose(const float* src, float* dst, int rows, int cols, hipStream_t s, int src_ld, int dst_ld) {
    dim3 grid((cols + kTrTile - 1) / kTrTile, (rows + kTrTile - 1) / kTrTile);
    if (grid.y > 65535u) return FFI_ERR_TOO_LARGE;
    hipLaunchKernelGGL(transpose_kernel, grid, dim3(kTrTile * 8), 0, s, src, dst, rows, cols, src_ld > 0 ? src_ld : cols,
                       dst_ld > 0 ? dst_ld : rows);
    FFI_HIP_TRY(hipGetLastError());
    return FFI_OK;
}

}  // namespace ffi
