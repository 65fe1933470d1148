// Copies between pageable host arrays (what a ctypes caller hands over: numpy buffers) and device memory.
//
// hipMemcpy on pageable memory moves the bytes through a bounce buffer on one thread; at N = 1M, D = 100, K = 32 the
// 656 MB of a call took 38 ms that way, more than half the time of the build itself.  Here a few host threads each
// take a contiguous slice of the array and move it in pieces through their own pair of pinned buffers
// (hipHostMalloc; registering the caller's memory is not an option) on their own stream: the memcpy into / out of
// the pinned buffer of one piece overlaps the DMA of the previous one, and the threads overlap each other.
// The pinned buffers are kept for the next call; rsfk_release_workspace() frees them.
#include "rsfk_common.hpp"
#include "forest.hpp"
#include <algorithm>
#include <atomic>
#include <cstring>
#include <mutex>
#include <thread>
#include <vector>

namespace rsfk {

namespace {

constexpr int kCopyThreads = 4;
constexpr size_t kPiece = (size_t)8 << 20;          // bytes per pinned buffer
constexpr size_t kSmall = (size_t)4 << 20;          // below this a plain hipMemcpy is used

struct Lane {
    void* pinned[2] = {nullptr, nullptr};
    hipStream_t stream = nullptr;
    hipEvent_t done[2] = {nullptr, nullptr};
};

struct Lanes {
    std::mutex mu;
    int device = -1;
    Lane lane[kCopyThreads];
    bool ready = false;
};

Lanes& lanes()
{
    static Lanes l;
    return l;
}

void free_lanes_locked(Lanes& L)
{
    for (Lane& a : L.lane) {
        for (int i = 0; i < 2; ++i) {
            if (a.pinned[i]) (void)hipHostFree(a.pinned[i]);
            if (a.done[i]) (void)hipEventDestroy(a.done[i]);
            a.pinned[i] = nullptr;
            a.done[i] = nullptr;
        }
        if (a.stream) (void)hipStreamDestroy(a.stream);
        a.stream = nullptr;
    }
    L.ready = false;
    L.device = -1;
}

int make_lanes_locked(Lanes& L, int dev)
{
    if (L.ready && L.device == dev) return 0;
    free_lanes_locked(L);
    for (Lane& a : L.lane) {
        RSFK_HIP(hipStreamCreateWithFlags(&a.stream, hipStreamNonBlocking));
        for (int i = 0; i < 2; ++i) {
            RSFK_HIP(hipHostMalloc(&a.pinned[i], kPiece));
            RSFK_HIP(hipEventCreateWithFlags(&a.done[i], hipEventDisableTiming));
        }
    }
    L.device = dev;
    L.ready = true;
    return 0;
}

// one thread's slice: [begin, end) of the array, to_device or back
void run_slice(Lane& a, int dev, char* dev_ptr, char* host_ptr, size_t begin, size_t end, bool to_device, std::atomic<int>& err)
{
    if (hipSetDevice(dev) != hipSuccess) { err = 1; return; }
    size_t off[2] = {0, 0}, len[2] = {0, 0};
    int n = 0;
    for (size_t at = begin; at < end && !err; at += kPiece, ++n) {
        const int b = n & 1;
        const size_t bytes = std::min(kPiece, end - at);
        if (n >= 2) {
            // the piece that used this buffer two steps ago
            if (hipEventSynchronize(a.done[b]) != hipSuccess) { err = 1; return; }
            if (!to_device) std::memcpy(host_ptr + off[b], a.pinned[b], len[b]);
        }
        off[b] = at;
        len[b] = bytes;
        if (to_device) {
            std::memcpy(a.pinned[b], host_ptr + at, bytes);
            if (hipMemcpyAsync(dev_ptr + at, a.pinned[b], bytes, hipMemcpyHostToDevice, a.stream) != hipSuccess) { err = 1; return; }
        } else {
            if (hipMemcpyAsync(a.pinned[b], dev_ptr + at, bytes, hipMemcpyDeviceToHost, a.stream) != hipSuccess) { err = 1; return; }
        }
        if (hipEventRecord(a.done[b], a.stream) != hipSuccess) { err = 1; return; }
    }
    // drain: the last (up to) two pieces
    for (int k = std::max(0, n - 2); k < n && !err; ++k) {
        const int b = k & 1;
        if (hipEventSynchronize(a.done[b]) != hipSuccess) { err = 1; return; }
        if (!to_device) std::memcpy(host_ptr + off[b], a.pinned[b], len[b]);
    }
}

int staged_copy(void* dev_ptr, void* host_ptr, size_t bytes, bool to_device)
{
    if (bytes == 0) return 0;
    if (bytes < kSmall) {
        if (to_device) RSFK_HIP(hipMemcpy(dev_ptr, host_ptr, bytes, hipMemcpyHostToDevice));
        else RSFK_HIP(hipMemcpy(host_ptr, dev_ptr, bytes, hipMemcpyDeviceToHost));
        return 0;
    }
    int dev = 0;
    RSFK_HIP(hipGetDevice(&dev));
    Lanes& L = lanes();
    std::lock_guard<std::mutex> lock(L.mu);            // one staged copy at a time
    if (make_lanes_locked(L, dev)) return 1;
    // what the device was asked to do before must be done when the copies on the other streams touch the memory
    RSFK_HIP(hipDeviceSynchronize());
    std::atomic<int> err{0};
    const size_t per = ((bytes + kCopyThreads - 1) / kCopyThreads + 255) & ~(size_t)255;
    std::vector<std::thread> th;
    for (int t = 0; t < kCopyThreads; ++t) {
        const size_t b = std::min(bytes, per * t), e = std::min(bytes, per * (t + 1));
        if (b >= e) break;
        th.emplace_back(run_slice, std::ref(L.lane[t]), dev, static_cast<char*>(dev_ptr), static_cast<char*>(host_ptr), b, e,
                        to_device, std::ref(err));
    }
    for (auto& t : th) t.join();
    RSFK_CHECK(err == 0, "copy between host and device failed");
    return 0;
}

}  // namespace

int copy_to_device(void* dev_ptr, const void* host_ptr, size_t bytes)
{
    return staged_copy(dev_ptr, const_cast<void*>(host_ptr), bytes, true);
}

int copy_to_host(void* host_ptr, const void* dev_ptr, size_t bytes)
{
    return staged_copy(const_cast<void*>(dev_ptr), host_ptr, bytes, false);
}

void release_copy_buffers()
{
    Lanes& L = lanes();
    std::lock_guard<std::mutex> lock(L.mu);
    free_lanes_locked(L);
}

}  // namespace rsfk
