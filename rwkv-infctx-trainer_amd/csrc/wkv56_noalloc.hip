// WKV5 / WKV6 forward for callers that cannot allocate and have no workspace to hand in (code under HIP graph
// capture, serving loops, harnesses that forbid hipMalloc): the piece summaries of the time-parallel split, the one
// scratch buffer the blocked forward needs, live in a file-scope device array of the library instead of a caller's
// workspace.  Every GPU the library runs on holds its own copy of the array until the process ends.  All calls on
// one GPU share that GPU's array: calls that overlap in time on one GPU race on it.  Nothing in it has to start at
// zero (every summary is written before it is read within a call).
#include "common.h"

namespace wkv {
namespace chunked {

// 16 MiB per GPU; no checkpoints are kept (forward only).
constexpr size_t STATIC_SCRATCH_BYTES = (size_t)16 << 20;
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];
// The array's address on the current device (each GPU has its own copy of the array at its own address).
static hipError_t static_scratch_address(void **out) {
    static void *ptrs[64] = {nullptr};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= 64) return hipErrorInvalidDevice;
    void *p = __atomic_load_n(&ptrs[dev], __ATOMIC_ACQUIRE);
    if (!p) {
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        __atomic_store_n(&ptrs[dev], p, __ATOMIC_RELEASE);
    }
    *out = p;
    return hipSuccess;
}
// what wkv_init() does for this entry point: the array's address on the current device, so that the first call has
// no set-up left to do (a first call inside a stream capture)
hipError_t init_static_scratch() {
    void *p = nullptr;
    return static_scratch_address(&p);
}
// returns hipErrorOutOfMemory when the plan's summaries do not fit the array
hipError_t forward_static_launch(hipStream_t s, bool per_token, bool w16, int B, int Tlen, int C, int H, const void *r, const void *k,
                                 const void *v, const void *w, const float *u, const float *s_in, void *y, float *s_out,
                                 int floor_decay) {
    const GroupPlan gp = plan_groups(B * H, Tlen);
    if (part_bytes(B * H, gp) > STATIC_SCRATCH_BYTES) return hipErrorOutOfMemory;
    void *ptr = nullptr;
    if (gp.b.nseg > 1) {
        hipError_t e = static_scratch_address(&ptr);
        if (e != hipSuccess) return e;
    }
    return forward_launch(s, per_token, w16, B, Tlen, C, H, r, k, v, w, u, s_in, y, s_out, nullptr, (float *)ptr, gp, floor_decay);
}

}  // namespace chunked
}  // namespace wkv
