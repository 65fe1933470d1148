// Device memory for the working buffers of a call (permutations, screening copies, exploration workspace).
//
// hipMalloc / hipFree of a few hundred megabytes cost tens to hundreds of microseconds each and a call needs
// about thirty of them, so blocks are kept after use and handed out again to the next call that asks for the
// same size on the same device (a build repeated with the same shapes allocates nothing).  Idle blocks are
// capped at RSFK_WORKSPACE_POOL_MB megabytes (default: a quarter of the device memory, at most 16 GiB; 0 keeps
// nothing); rsfk_release_workspace() returns all of them to the driver.
// The reference allocates and frees inside every tree level (src/rsfk.cu:640-1180).
#include "rsfk_common.hpp"
#include <algorithm>
#include <cstdlib>
#include <map>
#include <mutex>
#include <vector>

namespace rsfk {

namespace {

struct Pool {
    std::mutex mu;
    std::multimap<std::pair<int, size_t>, void*> idle;     // (device, bytes) -> block
    std::map<void*, std::pair<int, size_t>> live;           // blocks handed out
    size_t idle_bytes = 0;
    size_t idle_cap = 0;                                    // set on first use
    bool cap_known = false;
};

// most idle bytes the pool keeps (asked of the device once)
size_t idle_cap_locked(Pool& P)
{
    if (!P.cap_known) {
        P.cap_known = true;
        size_t free_b = 0, total_b = 0;
        P.idle_cap = (size_t)4 << 30;
        if (hipMemGetInfo(&free_b, &total_b) == hipSuccess) P.idle_cap = std::min<size_t>(total_b / 4, (size_t)16 << 30);
        const char* e = std::getenv("RSFK_WORKSPACE_POOL_MB");
        if (e && *e) P.idle_cap = (size_t)std::max(0ll, std::atoll(e)) << 20;
    }
    return P.idle_cap;
}

Pool& pool()
{
    static Pool p;
    return p;
}

}  // namespace

namespace {
// must: a block the caller cannot do without (idle blocks are given back to make room, the error text is set);
// otherwise one plain attempt that leaves the pool and the error text alone
int ws_alloc_impl(void** out, size_t bytes, bool must)
{
    *out = nullptr;
    if (bytes == 0) bytes = 1;
    bytes = (bytes + 255) & ~(size_t)255;
    int dev = 0;
    RSFK_HIP(hipGetDevice(&dev));
    Pool& P = pool();
    {
        std::lock_guard<std::mutex> lock(P.mu);
        auto it = P.idle.find({dev, bytes});
        if (it != P.idle.end()) {
            *out = it->second;
            P.idle.erase(it);
            P.idle_bytes -= bytes;
            P.live[*out] = {dev, bytes};
            return 0;
        }
    }
    void* p = nullptr;
    hipError_t e = hipMalloc(&p, bytes);
    if (e != hipSuccess && !must) {
        (void)hipGetLastError();
        return 1;
    }
    if (e != hipSuccess) {
        // give the idle blocks back and try once more
        (void)hipGetLastError();
        ws_release_all();
        e = hipMalloc(&p, bytes);
    }
    if (e != hipSuccess) {
        (void)hipGetLastError();
        set_last_error(std::string("out of device memory (") + std::to_string(bytes) + " bytes): " + hipGetErrorString(e));
        return 1;
    }
    std::lock_guard<std::mutex> lock(P.mu);
    P.live[p] = {dev, bytes};
    *out = p;
    return 0;
}
}  // namespace

int ws_alloc(void** out, size_t bytes) { return ws_alloc_impl(out, bytes, true); }

// A block the caller can do without (it only makes something faster): nonzero, with nothing else changed, when the
// device does not have the room.
int ws_try_alloc(void** out, size_t bytes) { return ws_alloc_impl(out, bytes, false); }

// The caller has made sure that no work that uses the block is still running.
void ws_free(void* p)
{
    if (!p) return;
    Pool& P = pool();
    std::pair<int, size_t> key;
    {
        std::lock_guard<std::mutex> lock(P.mu);
        auto it = P.live.find(p);
        if (it == P.live.end()) {           // not ours
            (void)hipFree(p);
            return;
        }
        key = it->second;
        P.live.erase(it);
        if (P.idle_bytes + key.second <= idle_cap_locked(P)) {
            P.idle.insert({key, p});
            P.idle_bytes += key.second;
            return;
        }
    }
    (void)hipFree(p);
}

void ws_release_all()
{
    Pool& P = pool();
    std::vector<void*> blocks;
    {
        std::lock_guard<std::mutex> lock(P.mu);
        for (auto& kv : P.idle) blocks.push_back(kv.second);
        P.idle.clear();
        P.idle_bytes = 0;
    }
    for (void* b : blocks) (void)hipFree(b);
}

}  // namespace rsfk
