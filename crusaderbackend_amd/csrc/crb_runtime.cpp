// Host-side runtime pieces of the C ABI: per-thread error text, HIP status translation and the
// lazily grown device scratch arenas used for split-K partial sums.
#include <cstdarg>
#include <cstdio>
#include <map>
#include <mutex>
#include <utility>
#include <vector>

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

// Split scratch (partial sums of contractions cut along K) comes from, in this order:
//   1. the calling thread's scratch scope, if one is open (an entry point that must not allocate opens one over a block
//      it owns: every nested request is then served from that block or refused);
//   2. the block the caller bound to this (device, stream) with crb_bind_workspace: served or refused, never grown;
//   3. the library's own arena of this (device, stream), grown with hipMalloc on first use or when a call needs more.
// One arena per (device, stream): work queued on one stream never shares partial-sum scratch with work on another, so
// calls on different streams may overlap. (The reference itself is single-device and single-stream: Tensor::instantiate
// pins deviceId 0, seblas/tensor/Tensor.cu:358.) A block an arena has outgrown may still be named by work in flight or
// by a recorded graph, so it is kept on a retired list until crb_release_workspace instead of being freed on growth.
struct Arena {
    void *ptr = nullptr;
    size_t bytes = 0;
    bool bound = false;  // caller-owned (crb_bind_workspace): never freed, never grown
};
static std::mutex g_arena_mu;
static std::map<std::pair<int, hipStream_t>, Arena> g_arenas;
static std::vector<std::pair<int, void *>> g_retired;  // (device, block)

static thread_local void *g_scope_ptr = nullptr;
static thread_local size_t g_scope_bytes = 0;
static thread_local size_t g_scope_used = 0;  // bytes of the open scope already handed out

ScratchScope::ScratchScope(void *ptr, size_t bytes) : prev_ptr(g_scope_ptr), prev_bytes(g_scope_bytes), prev_used(g_scope_used) {
    g_scope_ptr = ptr, g_scope_bytes = bytes, g_scope_used = 0;
}
ScratchScope::~ScratchScope() { g_scope_ptr = prev_ptr, g_scope_bytes = prev_bytes, g_scope_used = prev_used; }

int scratch_get(size_t bytes, hipStream_t stream, const char *what, void **out) {
    *out = nullptr;
    if (g_scope_ptr) {
        // every request inside one scope gets a block of its own (256-byte steps), so two requests of one call never alias
        const size_t at = (g_scope_used + 255) & ~size_t(255);
        if (at > g_scope_bytes || bytes > g_scope_bytes - at)
            return fail(CRB_EWORKSPACE, "%s: needs %zu bytes of scratch, the buffer this call may use holds %zu (%zu already in use)",
                        what, bytes, g_scope_bytes, at);
        *out = static_cast<char *>(g_scope_ptr) + at;
        g_scope_used = at + bytes;
        return CRB_OK;
    }
    int dev = 0;
    if (hipError_t e = hipGetDevice(&dev)) return check_hip(e, what);
    std::lock_guard<std::mutex> lk(g_arena_mu);
    Arena &a = g_arenas[std::make_pair(dev, stream)];
    if (a.bound) {
        if (bytes > a.bytes)
            return fail(CRB_EWORKSPACE, "%s: needs %zu bytes of scratch, the workspace bound to this stream holds %zu", what, bytes, a.bytes);
        *out = a.ptr;
        return CRB_OK;
    }
    if (bytes <= a.bytes) {
        *out = a.ptr;
        return CRB_OK;
    }
    // growing means hipMalloc, which a stream capture cannot record
    // (a capture query that fails — the legacy stream while another stream captures in global mode — counts as capturing)
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &cap) != hipSuccess) {
        (void)hipGetLastError();
        cap = hipStreamCaptureStatusActive;
    }
    if (cap != hipStreamCaptureStatusNone)
        return fail(CRB_EWORKSPACE,
                    "%s: needs %zu bytes of scratch while the stream is being captured; bind a workspace to the stream "
                    "(crb_bind_workspace) or run the call once before capturing", what, bytes);
    if (a.ptr) g_retired.emplace_back(dev, a.ptr);
    a = Arena();
    const size_t want = bytes < (size_t(8) << 20) ? (size_t(8) << 20) : bytes + bytes / 2;
    void *p = nullptr;
    if (hipError_t e = hipMalloc(&p, want)) {
        (void)hipGetLastError();
        return fail(CRB_EHIP, "%s: cannot allocate %zu bytes of split scratch: %s", what, want, hipGetErrorString(e));
    }
    a.ptr = p;
    a.bytes = want;
    *out = p;
    return CRB_OK;
}

int scratch_bind(void *ptr, size_t bytes, hipStream_t stream) {
    int dev = 0;
    if (hipError_t e = hipGetDevice(&dev)) return check_hip(e, "crb_bind_workspace");
    std::lock_guard<std::mutex> lk(g_arena_mu);
    Arena &a = g_arenas[std::make_pair(dev, stream)];
    if (a.ptr && !a.bound) g_retired.emplace_back(dev, a.ptr);  // the library's own block: freed by crb_release_workspace
    a = Arena();
    if (ptr) a.ptr = ptr, a.bytes = bytes, a.bound = true;
    return CRB_OK;
}

void arena_release() {
    std::lock_guard<std::mutex> lk(g_arena_mu);
    int cur = 0;
    (void)hipGetDevice(&cur);
    for (auto it = g_arenas.begin(); it != g_arenas.end();) {
        if (it->second.bound) {  // caller-owned blocks stay bound
            ++it;
            continue;
        }
        if (it->second.ptr) g_retired.emplace_back(it->first.first, it->second.ptr);
        it = g_arenas.erase(it);
    }
    for (auto &r : g_retired) {
        (void)hipSetDevice(r.first);
        (void)hipDeviceSynchronize();
        (void)hipFree(r.second);
    }
    if (!g_retired.empty()) (void)hipSetDevice(cur);
    g_retired.clear();
}

}  // namespace crb

extern "C" {

int crb_abi_version(void) { return 1000; }

const char *crb_last_error_string(void) { return crb::g_err; }

void crb_release_workspace(void) { crb::arena_release(); }

int crb_bind_workspace(void *workspace, size_t workspace_bytes, void *stream) {
    if (workspace && (reinterpret_cast<uintptr_t>(workspace) & 255u))
        return crb::fail(CRB_EWORKSPACE, "crb_bind_workspace: workspace is not 256-byte aligned");
    if (workspace && !workspace_bytes) return crb::fail(CRB_EWORKSPACE, "crb_bind_workspace: empty workspace");
    return crb::scratch_bind(workspace, workspace_bytes, hipStream_t(stream));
}

}  // extern "C"
