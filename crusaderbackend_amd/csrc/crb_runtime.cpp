// Host-side runtime pieces of the C ABI: per-thread error text, HIP status translation and the
// lazily grown device scratch arenas used for split-K partial sums.
#include <cstdarg>
#include <cstdio>
#include <map>
#include <mutex>
#include <utility>

#include "crb_common.h"

namespace crb {

static thread_local char g_err[512] = "";

int fail(int st, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return st;
}

int check_hip(hipError_t e, const char *what) {
    if (e == hipSuccess) return CRB_OK;
    return fail(CRB_EHIP, "%s: %s", what, hipGetErrorString(e));
}

int check_launch(const char *what) { return check_hip(hipGetLastError(), what); }

// One arena per (device, stream): work queued on one stream never shares partial-sum scratch with work on another, so
// calls on different streams may overlap. (The reference itself is single-device and single-stream: Tensor::instantiate
// pins deviceId 0, seblas/tensor/Tensor.cu:358.) An arena grows geometrically and is kept until crb_release_workspace.
struct Arena {
    void *ptr = nullptr;
    size_t bytes = 0;
};
static std::mutex g_arena_mu;
static std::map<std::pair<int, hipStream_t>, Arena> g_arenas;

void *arena_get(size_t bytes, hipStream_t stream) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
    }
    std::lock_guard<std::mutex> lk(g_arena_mu);
    Arena &a = g_arenas[std::make_pair(dev, stream)];
    if (bytes <= a.bytes) return a.ptr;
    if (a.ptr) {
        // work already queued on the old block (all of it on this stream) must finish before it is returned to the allocator
        (void)hipStreamSynchronize(stream);
        (void)hipFree(a.ptr);
        a = Arena();
    }
    const size_t want = bytes < (size_t(8) << 20) ? (size_t(8) << 20) : bytes + bytes / 2;
    void *p = nullptr;
    if (hipMalloc(&p, want) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
    }
    a.ptr = p;
    a.bytes = want;
    return p;
}

void arena_release() {
    std::lock_guard<std::mutex> lk(g_arena_mu);
    if (g_arenas.empty()) return;
    int cur = 0;
    (void)hipGetDevice(&cur);
    for (auto &kv : g_arenas) {
        if (!kv.second.ptr) continue;
        (void)hipSetDevice(kv.first.first);
        (void)hipDeviceSynchronize();
        (void)hipFree(kv.second.ptr);
    }
    (void)hipSetDevice(cur);
    g_arenas.clear();
}

}  // namespace crb

extern "C" {

int crb_abi_version(void) { return 1000; }

const char *crb_last_error_string(void) { return crb::g_err; }

void crb_release_workspace(void) { crb::arena_release(); }

}  // extern "C"
