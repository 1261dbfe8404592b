// Shared host/device helpers for the gfx950 seblas kernels: status plumbing, exact uint32
// division by a runtime constant, launch-geometry helpers.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/crusader_hip.h"

namespace crb {

typedef uint32_t u32;

// Records `msg` as the calling thread's last error and returns `st`.
int fail(int st, const char *fmt, ...);
// Checks a HIP return code / the sticky launch error; returns CRB_OK or CRB_EHIP (message recorded).
int check_hip(hipError_t e, const char *what);
int check_launch(const char *what);

// Device scratch for partial sums (`bytes` > 0) of a call queued on `stream` of the current device: the calling thread's
// open ScratchScope, else the workspace bound to the stream, else the library's lazily grown arena of that stream. A block
// stays valid for work queued on that stream until crb_release_workspace. Returns CRB_OK and the block, or an error
// (CRB_EWORKSPACE: the scope / bound workspace is too small, or growth was needed during a stream capture; CRB_EHIP:
// allocation failed).
int scratch_get(size_t bytes, hipStream_t stream, const char *what, void **out);
template <class T>
inline int scratch_get(size_t bytes, hipStream_t stream, const char *what, T **out) {
    void *p = nullptr;
    const int st = scratch_get(bytes, stream, what, &p);
    *out = static_cast<T *>(p);
    return st;
}
int scratch_bind(void *ptr, size_t bytes, hipStream_t stream);
void arena_release();
// While alive, every scratch_get of this thread is served from [ptr, ptr + bytes) or refused; nothing is allocated.
// Requests inside one scope get consecutive blocks (256-byte steps), never the same memory twice.
struct ScratchScope {
    ScratchScope(void *ptr, size_t bytes);
    ~ScratchScope();
    ScratchScope(const ScratchScope &) = delete;
    ScratchScope &operator=(const ScratchScope &) = delete;
  private:
    void *prev_ptr;
    size_t prev_bytes, prev_used;
};

// Exact floor(n / d) for any n, d in [1, 2^32): round-up magic multiply (Granlund-Montgomery).
// q = (t + ((n - t) >> s1)) >> s2 with t = mulhi(m, n).
struct FastDiv {
    u32 d, m, s1, s2;
    __host__ __device__ FastDiv() : d(1), m(1), s1(0), s2(0) {}
    explicit FastDiv(u32 div) { init(div); }
    void init(u32 div) {
        d = div ? div : 1;
        u32 l = 0;
        while (l < 32 && (uint64_t(1) << l) < d) ++l;
        uint64_t two_l = uint64_t(1) << l;
        m = u32(((two_l - d) << 32) / d + 1);
        s1 = l < 1 ? l : 1;
        s2 = l > 0 ? l - 1 : 0;
    }
    __host__ __device__ __forceinline__ u32 div(u32 n) const {
#if defined(__HIP_DEVICE_COMPILE__)
        u32 t = __umulhi(m, n);
#else
        u32 t = u32((uint64_t(m) * n) >> 32);
#endif
        return (t + ((n - t) >> s1)) >> s2;
    }
    __host__ __device__ __forceinline__ void divmod(u32 n, u32 &q, u32 &r) const {
        q = div(n);
        r = n - q * d;
    }
};

static inline u32 ceil_div(u32 a, u32 b) { return (a + b - 1) / b; }

}  // namespace crb
