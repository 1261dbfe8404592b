// Host-side runtime pieces of the C ABI: per-thread error text, HIP status translation and the
// lazily grown device scratch arena used for split-K partial sums.
#include <cstdarg>
#include <cstdio>
#include <mutex>

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

// One arena per process (the reference is single-device: Tensor::instantiate pins deviceId 0,
// seblas/tensor/Tensor.cu:358). Grows geometrically; never shrinks until released.
static std::mutex g_arena_mu;
static void *g_arena = nullptr;
static size_t g_arena_bytes = 0;

void *arena_get(size_t bytes) {
    std::lock_guard<std::mutex> lk(g_arena_mu);
    if (bytes <= g_arena_bytes) return g_arena;
    if (g_arena) {
        // work already queued on the old block must finish before it is returned to the allocator
        (void)hipDeviceSynchronize();
        (void)hipFree(g_arena);
        g_arena = nullptr;
        g_arena_bytes = 0;
    }
    size_t want = bytes < (size_t(8) << 20) ? (size_t(8) << 20) : bytes + bytes / 2;
    void *p = nullptr;
    if (hipMalloc(&p, want) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
    }
    g_arena = p;
    g_arena_bytes = want;
    return g_arena;
}

void arena_release() {
    std::lock_guard<std::mutex> lk(g_arena_mu);
    if (g_arena) {
        (void)hipDeviceSynchronize();
        (void)hipFree(g_arena);
    }
    g_arena = nullptr;
    g_arena_bytes = 0;
}

}  // namespace crb

extern "C" {

int crb_abi_version(void) { return 1000; }

const char *crb_last_error_string(void) { return crb::g_err; }

void crb_release_workspace(void) { crb::arena_release(); }

}  // extern "C"
