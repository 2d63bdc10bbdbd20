// common.hpp — helpers shared by the gfx950 kernels and the C-ABI layer of libinpc_hip.so.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <mutex>

#include "../../include/inpc_hip.h"

namespace inpc {

// ------------------------------------------------------------------------------------------------
// host side: error reporting and launches
// ------------------------------------------------------------------------------------------------
void set_error(const char* fmt, ...);
int fail(int code, const char* fmt, ...);

// Optional per-launch timing (HIP events on the launch stream), see inpc_timing_enable().
void timing_begin(const char* name, hipStream_t stream);
void timing_end(hipStream_t stream);
bool timing_enabled();   // for the calling thread

// A second stream for work that does not depend on what the caller's stream is doing at the moment, with the two
// events that tie it to that stream: `fork` is recorded on the caller's stream and awaited by `stream`, `join` the
// other way round. Every (device, caller's stream) pair has a lane of its own, so callers on different streams
// never meet on one, and a capture of the caller's stream takes along a stream nobody else uses. Created on
// first use (non-blocking, default priority) and kept until the process ends; nullptr when there is none and
// `may_create` is false (a stream that is being captured gets no new lane), when it cannot be created, when the
// process already keeps kMaxSideLanes of them, or when the lane's stream is in a capture that the caller's stream is
// not part of (left over from a capture that was abandoned): the caller then keeps the work on its own stream.
// Two host threads that enqueue on one stream share its lane: fork under `mutex`.
struct SideLane {
    hipStream_t stream;
    hipEvent_t fork, join;
    std::mutex mutex;
};
constexpr int kMaxSideLanes = 256;
SideLane* side_lane(hipStream_t owner, bool owner_is_capturing);

#define INPC_HIP_CHECK(expr)                                                                        \
    do {                                                                                            \
        hipError_t _e = (expr);                                                                     \
        if (_e != hipSuccess)                                                                       \
            return ::inpc::fail(INPC_E_HIP, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e),  \
                                __FILE__, __LINE__);                                                \
    } while (0)

// Launch `kernel<<<grid, block, 0, stream>>>(args...)`, bracketed by timing events when enabled,
// and turn a launch failure into an INPC_E_HIP return.
#define INPC_LAUNCH(name, kernel, grid, block, stream, ...)                                         \
    do {                                                                                            \
        ::inpc::timing_begin(name, stream);                                                         \
        hipLaunchKernelGGL(kernel, grid, block, 0, stream, __VA_ARGS__);                            \
        ::inpc::timing_end(stream);                                                                 \
        hipError_t _e = hipGetLastError();                                                          \
        if (_e != hipSuccess)                                                                       \
            return ::inpc::fail(INPC_E_HIP, "launch of %s failed: %s", name, hipGetErrorString(_e)); \
    } while (0)

inline uint32_t div_up(uint32_t a, uint32_t b) { return (a + b - 1) / b; }
inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

inline int bit_length(uint32_t n) {
    int b = 0;
    while (n) {
        ++b;
        n >>= 1;
    }
    return b;
}

// Fill `n` 32-bit words with `value` (a kernel, not hipMemsetAsync, so that callers may capture
// the stream into a graph).
int fill_u32(void* dst, uint32_t value, size_t n_words, hipStream_t stream);

// Number of blocks of `threads` threads of `kernel` (static LDS only) that the current device holds at once.
int resident_blocks(const void* kernel, int threads, uint32_t& blocks);

// ------------------------------------------------------------------------------------------------
// device side
// ------------------------------------------------------------------------------------------------
constexpr int kWave = 64;

// The dynamic LDS of a launch as an array `name` of `type` (16-byte aligned).
#ifndef INPC_DYNAMIC_LDS
#define INPC_DYNAMIC_LDS(type, name) extern __shared__ __align__(16) type name[]
#endif

// Plain per-thread arithmetic that the tests also run on the host (geometry.hpp, the generators below).
#define INPC_HD __host__ __device__ __forceinline__

INPC_HD uint32_t float_bits_of(float f) { return __builtin_bit_cast(uint32_t, f); }
INPC_HD float float_of_bits(uint32_t u) { return __builtin_bit_cast(float, u); }

// Clamp to [0, 1] (the device's saturate; finite input on either side).
INPC_HD float saturate01(float v) {
#if defined(__HIP_DEVICE_COMPILE__)
    return __saturatef(v);
#else
    return v < 0.0f ? 0.0f : (v > 1.0f ? 1.0f : v);
#endif
}

// Orders the LDS traffic of one wave: everything issued before is visible to every lane after.
__device__ __forceinline__ void wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

__device__ __forceinline__ uint32_t lane_id() { return __lane_id(); }

// Number of set bits of `mask` below the calling lane.
__device__ __forceinline__ uint32_t mask_rank(uint64_t mask) {
    return __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
}

// One row of the affine world-to-camera transform, evaluated left to right without fused
// multiply-add (this translation unit is compiled with -ffp-contract=off).
INPC_HD float affine_row(const float4 r, float x, float y, float z) {
    return ((r.x * x + r.y * y) + r.z * z) + r.w;
}

struct Camera {
    float width, height, fx, fy, cx, cy, near_plane, far_plane;
};

inline Camera to_device_camera(const inpc_camera& c) {
    return Camera{(float)c.width, (float)c.height, c.focal_x, c.focal_y, c.center_x, c.center_y, c.near_plane,
                  c.far_plane};
}

// ---- PCG32 (XSH-RR 64/32) -----------------------------------------------------------------------
constexpr uint64_t kPcgMult = 0x5851f42d4c957f2dULL;

struct Pcg32 {
    uint64_t state, inc;
};

__host__ __device__ __forceinline__ uint32_t pcg_next(Pcg32& r) {
    const uint64_t old = r.state;
    r.state = old * kPcgMult + r.inc;
    const uint32_t xs = (uint32_t)(((old >> 18u) ^ old) >> 27u);
    const uint32_t rot = (uint32_t)(old >> 59u);
    return (xs >> rot) | (xs << ((~rot + 1u) & 31u));
}

__device__ __forceinline__ float pcg_float(Pcg32& r) {
    return __uint_as_float((pcg_next(r) >> 9) | 0x3f800000u) - 1.0f;
}

// The generator stepped `delta` times is state -> mult * state + plus (Brown's jump-ahead).
struct PcgJump {
    uint64_t mult, plus;
};

__host__ __device__ __forceinline__ PcgJump pcg_jump(uint64_t inc, uint64_t delta) {
    uint64_t cur_mult = kPcgMult, cur_plus = inc, acc_mult = 1u, acc_plus = 0u;
    while (delta > 0) {
        if (delta & 1) {
            acc_mult *= cur_mult;
            acc_plus = acc_plus * cur_mult + cur_plus;
        }
        cur_plus = (cur_mult + 1) * cur_plus;
        cur_mult *= cur_mult;
        delta >>= 1;
    }
    return PcgJump{acc_mult, acc_plus};
}

__host__ __device__ __forceinline__ uint64_t pcg_apply(const PcgJump& j, uint64_t state) {
    return j.mult * state + j.plus;
}

// ---- decoupled look-back --------------------------------------------------------------------------
// A status word is {2 flag bits, 30 value bits}. A block must only ever wait on blocks that are running: every
// kernel with a look-back hands its tiles out through an atomic ticket, taken when a block starts a tile, so a
// tile that is waited for has always been taken by a block that was running then, whatever else occupies the GPU
// (other streams, other kernels). The grids are sized to what fits the GPU at once, so a block takes many tiles
// and the tickets stay few. The wait is bounded all the same and raises the error flag instead of spinning forever.
constexpr uint32_t kFlagAggregate = 1u << 30;
constexpr uint32_t kFlagInclusive = 2u << 30;
constexpr uint32_t kValueMask = (1u << 30) - 1u;
constexpr uint32_t kSpinLimit = 1u << 22;

// Status words carry their payload themselves and no other memory is handed over between blocks of
// one launch, so relaxed agent-scope accesses suffice. (Acquire / release at agent scope would make every
// access write back or invalidate the whole L2 of its XCD.)
__device__ __forceinline__ void status_store(uint32_t* p, uint32_t v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ uint32_t status_load(const uint32_t* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Exclusive prefix of one value per block over blocks 0..bid-1, walked by a whole wave: the 64 lanes look at 64
// predecessors at a time; publishes this block's aggregate first and its inclusive prefix at the end. Every lane of
// the calling wave must enter; all get the result.
__device__ __forceinline__ uint32_t lookback_exclusive_wave(uint32_t* status, uint32_t bid, uint32_t aggregate,
                                                            uint32_t* error_flag) {
    const uint32_t lane = lane_id();
    if (lane == 0) status_store(status + bid, (bid == 0 ? kFlagInclusive : kFlagAggregate) | aggregate);
    if (bid == 0) return 0u;
    uint32_t exclusive = 0u, spins = 0u;
    int64_t window = (int64_t)bid - 1;  // lane l looks at block window - l
    for (;;) {
        const int64_t p = window - (int64_t)lane;
        const uint32_t word = p >= 0 ? status_load(status + p) : kFlagInclusive;  // before block 0: nothing
        const uint64_t ready = __ballot((word & ~kValueMask) != 0u);
        const uint64_t inclusive = __ballot((word & kFlagInclusive) != 0u);
        const uint32_t last = inclusive ? (uint32_t)__builtin_ctzll(inclusive) : 63u;  // walk ends at this lane
        const uint64_t needed = last == 63u ? ~0ull : ((2ull << last) - 1ull);
        if ((ready & needed) == needed) {
            uint32_t v = lane <= last ? (word & kValueMask) : 0u;
            for (int s = 32; s > 0; s >>= 1) v += __shfl_xor(v, s, 64);
            exclusive += v;
            if (inclusive) break;
            window -= 64;
        } else {
            if (++spins > kSpinLimit) {
                if (lane == 0) atomicOr(error_flag, 1u);
                break;
            }
            __builtin_amdgcn_s_sleep(2);
        }
    }
    if (lane == 0) status_store(status + bid, kFlagInclusive | ((exclusive + aggregate) & kValueMask));
    return exclusive;
}

}  // namespace inpc
