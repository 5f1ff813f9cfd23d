// Shared device helpers: storage types, conversions, vector loads/stores.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <vector>
#include <algorithm>
#include <cstdlib>

namespace wkv {

constexpr int HEAD = 64;                    // key size == value size of one head
constexpr float LOG_W_FLOOR = -5.298317366548036f;   // ln 0.005

struct bf16 { uint16_t bits; };
struct f16 { _Float16 h; };

__device__ __forceinline__ float to_float(float x) { return x; }
__device__ __forceinline__ float to_float(bf16 x) { return __uint_as_float((uint32_t)x.bits << 16); }
__device__ __forceinline__ float to_float(f16 x) { return (float)x.h; }

// fp32 -> bf16, round to nearest even (one v_cvt_pk_bf16_f32 on gfx950)
__device__ __forceinline__ uint16_t bf16_bits(float f) { return __builtin_bit_cast(uint16_t, (__bf16)f); }
__device__ __forceinline__ uint32_t bf16_pack2(float lo, float hi) {      // lo in bits 0..15
    typedef float f2 __attribute__((ext_vector_type(2)));
    typedef __bf16 h2 __attribute__((ext_vector_type(2)));
    const f2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, h2));
}

template <class T> __device__ __forceinline__ T from_float(float f);
template <> __device__ __forceinline__ float from_float<float>(float f) { return f; }
template <> __device__ __forceinline__ bf16 from_float<bf16>(float f) { return bf16{bf16_bits(f)}; }
template <> __device__ __forceinline__ f16 from_float<f16>(float f) { return f16{(_Float16)f}; }

// four consecutive elements <-> four floats (p must be aligned to 4 elements)
__device__ __forceinline__ void load4(const float *p, float (&o)[4]) {
    float4 x = *reinterpret_cast<const float4 *>(p);
    o[0] = x.x; o[1] = x.y; o[2] = x.z; o[3] = x.w;
}
__device__ __forceinline__ void load4(const bf16 *p, float (&o)[4]) {
    uint2 x = *reinterpret_cast<const uint2 *>(p);
    o[0] = __uint_as_float(x.x << 16); o[1] = __uint_as_float(x.x & 0xffff0000u);
    o[2] = __uint_as_float(x.y << 16); o[3] = __uint_as_float(x.y & 0xffff0000u);
}
__device__ __forceinline__ void load4(const f16 *p, float (&o)[4]) {
    typedef _Float16 h4 __attribute__((ext_vector_type(4)));
    h4 x = *reinterpret_cast<const h4 *>(p);
    o[0] = (float)x[0]; o[1] = (float)x[1]; o[2] = (float)x[2]; o[3] = (float)x[3];
}
__device__ __forceinline__ void store4(float *p, const float (&o)[4]) {
    *reinterpret_cast<float4 *>(p) = make_float4(o[0], o[1], o[2], o[3]);
}
__device__ __forceinline__ void store4(bf16 *p, const float (&o)[4]) {
    uint2 x;
    x.x = bf16_pack2(o[0], o[1]);
    x.y = bf16_pack2(o[2], o[3]);
    *reinterpret_cast<uint2 *>(p) = x;
}
__device__ __forceinline__ void store4(f16 *p, const float (&o)[4]) {
    typedef _Float16 h4 __attribute__((ext_vector_type(4)));
    h4 x = {(_Float16)o[0], (_Float16)o[1], (_Float16)o[2], (_Float16)o[3]};
    *reinterpret_cast<h4 *>(p) = x;
}

// log of the decay from the raw parameter: -exp(x), optionally bounded below
__device__ __forceinline__ float log_decay(float x, bool floor_decay, bool *floored = nullptr) {
    float l = -__expf(x);
    bool f = floor_decay && (l < LOG_W_FLOOR);
    if (floored) *floored = f;
    return f ? LOG_W_FLOOR : l;
}

// The blocked kernels keep log w in base-2 units: -exp(x) log2(e) = -2^(x log2(e) + log2(log2(e))), so that
// every later exponential is the bare hardware instruction.
constexpr float LOG2E = 1.4426950408889634f, LN2 = 0.6931471805599453f, LOG2_LOG2E = 0.5287663729448977f;
constexpr float LOG2_W_FLOOR = -7.643856189774724f;   // log2 0.005
__device__ __forceinline__ float exp2_fast(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float log2_decay(float x, bool floor_decay) {
    const float l = -exp2_fast(fmaf(x, LOG2E, LOG2_LOG2E));
    return (floor_decay && l < LOG2_W_FLOOR) ? LOG2_W_FLOOR : l;
}

// Workgroup barrier that waits for this wavefront's LDS traffic only: __syncthreads() would also wait for every
// global load in flight, i.e. for the prefetch the barrier is meant to overlap with.
__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// ---- optional timing of one kernel with caller-owned HIP events (wkv_profile_events)
enum KernelId {
    KID_NONE = 0, KID_REC_FORWARD = 1, KID_REC_BACKWARD = 2, KID_V4_FORWARD = 3, KID_V4_BACKWARD = 4,
    KID_CHUNK_FORWARD = 10, KID_CHUNK_BACKWARD = 11
};
struct ProfileSlot {
    int id = KID_NONE;
    std::vector<hipEvent_t> start, stop;
    size_t used = 0;
};
inline ProfileSlot &profile_slot() { static ProfileSlot p; return p; }
inline void prof_begin(int id, hipStream_t s) {
    ProfileSlot &p = profile_slot();
    if (p.id == id && p.used < p.start.size()) (void)hipEventRecord(p.start[p.used], s);
}
inline void prof_end(int id, hipStream_t s) {
    ProfileSlot &p = profile_slot();
    if (p.id == id && p.used < p.start.size()) { (void)hipEventRecord(p.stop[p.used], s); p.used++; }
}

// Set-up that belongs to a device (a kernel's raised LDS limit is a property of the code object loaded on that
// device): runs `setup` the first time it is asked for the current device and hands back what it returned from then on.
struct PerDevice {
    hipError_t status[64];
    PerDevice() { std::fill(status, status + 64, hipErrorNotReady); }
    template <class F> hipError_t once(F setup) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) { (void)hipGetLastError(); return setup(); }
        if (status[dev] == hipErrorNotReady) status[dev] = setup();
        return status[dev];
    }
};

// sum per-batch partials: in (B, n) -> out (n); fixed order, so repeatable
static __global__ void sum_over_batch(int B, int n, const float *__restrict__ in, float *__restrict__ out) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float s = 0.f;
    for (int b = 0; b < B; b++) s += in[(size_t)b * n + i];
    out[i] = s;
}

// Compute units of the current device (256 on MI355X; also the answer when no device can be asked, as in a
// workspace query made on a machine without one).
inline int cu_count() {
    static int cached[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) { (void)hipGetLastError(); return 256; }
    if (cached[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) { (void)hipGetLastError(); n = 256; }
        cached[dev] = n;
    }
    return cached[dev];
}

}  // namespace wkv
