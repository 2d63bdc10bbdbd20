// hip/hip_runtime.h of the tests' SIMT simulator: what the library's sources use of HIP, for a plain C++ compiler.
// Kernels run on the CPU through sim::launch (sim.hpp); "device" pointers are host pointers; streams do nothing
// (every launch has run when the call returns) and an event is the host's clock when it is recorded.
// TEST INFRASTRUCTURE ONLY, never part of the product's build.
#pragma once

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <chrono>
#include <cstring>

#include "../sim.hpp"

#define INPC_SIM 1

// ---- qualifiers --------------------------------------------------------------------------------------------------
#define __global__
#define __device__
#define __host__
#define __forceinline__ inline __attribute__((always_inline))
#define __launch_bounds__(...)
// __shared__ variables are statics gathered in one section of the library, which sim::launch fills with a byte
// pattern before every block: LDS holds nothing a block can count on. (One launch at a time per process.)
#define __shared__ static __attribute__((section("sim_lds")))
extern "C" char __start_sim_lds[], __stop_sim_lds[];
#define __align__(n) __attribute__((aligned(n)))

// ---- vector types ------------------------------------------------------------------------------------------------
struct alignas(8) float2 { float x, y; };
struct alignas(16) float4 { float x, y, z, w; };
struct alignas(8) uint2 { uint32_t x, y; };
struct alignas(16) uint4 { uint32_t x, y, z, w; };
struct alignas(8) int2 { int x, y; };
inline float2 make_float2(float x, float y) { return float2{x, y}; }
inline float4 make_float4(float x, float y, float z, float w) { return float4{x, y, z, w}; }
inline uint2 make_uint2(uint32_t x, uint32_t y) { return uint2{x, y}; }
inline uint4 make_uint4(uint32_t x, uint32_t y, uint32_t z, uint32_t w) { return uint4{x, y, z, w}; }
using dim3 = sim::Dim3;

#define threadIdx (sim::detail::thread_idx())
#define blockIdx (sim::block().block_idx)
#define blockDim (sim::block().block_dim)
#define gridDim (sim::block().grid_dim)

namespace sim {
namespace detail {
inline Dim3 thread_idx() {
    const Block& b = block();
    const uint32_t t = fiber().tid;
    return Dim3(t % b.block_dim.x, (t / b.block_dim.x) % b.block_dim.y, t / (b.block_dim.x * b.block_dim.y));
}
template <typename T>
inline uint64_t to_bits(T v) {
    static_assert(sizeof(T) <= 8, "meeting points carry at most 8 bytes");
    uint64_t u = 0;
    std::memcpy(&u, &v, sizeof(T));
    return u;
}
template <typename T>
inline T from_bits(uint64_t u) {
    T v;
    std::memcpy(&v, &u, sizeof(T));
    return v;
}
// value of `source` lane if it took part, else `fallback`
template <typename T>
inline T pick(const uint64_t* slots, uint64_t members, int source, T fallback) {
    if (source < 0 || source > 63 || !((members >> source) & 1ull)) return fallback;
    return from_bits<T>(slots[source]);
}
}  // namespace detail

inline void* dynamic_lds() { return block().dynamic_lds; }
}  // namespace sim

// extern __shared__ arrays: the launch's dynamic LDS
#define INPC_DYNAMIC_LDS(type, name) type* name = (type*)sim::dynamic_lds()

// ---- block and wave operations -------------------------------------------------------------------------------------
inline void __syncthreads() { sim::meet_block(0, nullptr); }
inline int __syncthreads_count(int pred) {
    const uint64_t* masks;
    const uint64_t* v = sim::meet_block(pred ? 1u : 0u, &masks);
    int n = 0;
    for (uint32_t t = 0; t < sim::block().n_threads; ++t)
        if ((masks[t >> 6] >> (t & 63u)) & 1ull) n += (int)v[t];
    return n;
}
inline int __syncthreads_or(int pred) { return __syncthreads_count(pred) != 0; }
inline int __syncthreads_and(int pred) {
    const uint64_t* masks;
    const uint64_t* v = sim::meet_block(pred ? 1u : 0u, &masks);
    for (uint32_t t = 0; t < sim::block().n_threads; ++t)
        if (((masks[t >> 6] >> (t & 63u)) & 1ull) && !v[t]) return 0;
    return 1;
}
inline uint32_t __lane_id() { return sim::lane(); }
inline unsigned long long __ballot(int pred) {
    uint64_t members;
    const uint64_t* v = sim::meet_wave(pred ? 1u : 0u, &members);
    unsigned long long out = 0;
    for (int l = 0; l < 64; ++l)
        if (((members >> l) & 1ull) && v[l]) out |= 1ull << l;
    return out;
}
template <typename T>
inline T __shfl(T value, int source, int width = 64) {
    uint64_t members;
    const uint64_t* v = sim::meet_wave(sim::detail::to_bits(value), &members);
    const int lane = (int)sim::lane();
    const int src = (lane & ~(width - 1)) + (source & (width - 1));
    return sim::detail::pick<T>(v, members, src, value);
}
template <typename T>
inline T __shfl_xor(T value, int mask, int width = 64) {
    uint64_t members;
    const uint64_t* v = sim::meet_wave(sim::detail::to_bits(value), &members);
    const int src = (int)sim::lane() ^ mask;
    return sim::detail::pick<T>(v, members, src, value);
}
template <typename T>
inline T __shfl_up(T value, unsigned delta, int width = 64) {
    uint64_t members;
    const uint64_t* v = sim::meet_wave(sim::detail::to_bits(value), &members);
    const int lane = (int)sim::lane();
    const int src = lane - (int)delta;
    if (src < (lane & ~(width - 1))) return value;
    return sim::detail::pick<T>(v, members, src, value);
}
template <typename T>
inline T __shfl_down(T value, unsigned delta, int width = 64) {
    uint64_t members;
    const uint64_t* v = sim::meet_wave(sim::detail::to_bits(value), &members);
    const int lane = (int)sim::lane();
    const int src = lane + (int)delta;
    if (src > (lane | (width - 1))) return value;
    return sim::detail::pick<T>(v, members, src, value);
}

// DPP: lane i of a wave takes the value of another lane, chosen by `ctrl`; a lane whose source does not exist or
// took no part, or whose row / bank is masked out, keeps `old` (bound_ctrl = false). Controls as on gfx9: 0x00-0xFF
// quad_perm, 0x101-0x10F row_shl, 0x111-0x11F row_shr, 0x121-0x12F row_ror, 0x130 wave_shl:1, 0x138 wave_shr:1,
// 0x140 row_mirror, 0x141 row_half_mirror, 0x142 row_bcast:15, 0x143 row_bcast:31.
inline int sim_update_dpp(int old, int src, int ctrl, int row_mask, int bank_mask, bool bound_ctrl) {
    uint64_t members;
    const uint64_t* v = sim::meet_wave(sim::detail::to_bits(src), &members);
    const int lane = (int)sim::lane();
    const int row = lane >> 4, in_row = lane & 15;
    if (!((row_mask >> row) & 1) || !((bank_mask >> (in_row >> 2)) & 1)) return old;
    int source = -1;
    if (ctrl >= 0x00 && ctrl <= 0xFF) {
        source = (lane & ~3) + ((ctrl >> (2 * (lane & 3))) & 3);
    } else if (ctrl >= 0x101 && ctrl <= 0x10F) {
        const int s = in_row + (ctrl & 15);
        source = s <= 15 ? (lane & ~15) + s : -1;
    } else if (ctrl >= 0x111 && ctrl <= 0x11F) {
        const int s = in_row - (ctrl & 15);
        source = s >= 0 ? (lane & ~15) + s : -1;
    } else if (ctrl >= 0x121 && ctrl <= 0x12F) {
        source = (lane & ~15) + ((in_row - (ctrl & 15)) & 15);
    } else if (ctrl == 0x130) {
        source = lane < 63 ? lane + 1 : -1;
    } else if (ctrl == 0x138) {
        source = lane > 0 ? lane - 1 : -1;
    } else if (ctrl == 0x140) {
        source = (lane & ~15) + (15 - in_row);
    } else if (ctrl == 0x141) {
        source = (lane & ~7) + (7 - (lane & 7));
    } else if (ctrl == 0x142) {
        source = row > 0 ? (row - 1) * 16 + 15 : -1;
    } else if (ctrl == 0x143) {
        source = row > 1 ? 31 : -1;
    } else {
        std::fprintf(stderr, "sim: DPP control 0x%x is not modelled\n", ctrl);
        std::abort();
    }
    if (source < 0 || !((members >> source) & 1ull)) return bound_ctrl ? 0 : old;
    return sim::detail::from_bits<int>(v[source]);
}
#define __builtin_amdgcn_update_dpp(old, src, ctrl, row_mask, bank_mask, bound_ctrl) \
    sim_update_dpp((old), (src), (ctrl), (row_mask), (bank_mask), (bound_ctrl))
inline int sim_readlane(int value, int source) {
    uint64_t members;
    const uint64_t* v = sim::meet_wave(sim::detail::to_bits(value), &members);
    return sim::detail::pick<int>(v, members, source, value);
}
#define __builtin_amdgcn_readlane(value, source) sim_readlane((value), (source))
inline uint32_t sim_mbcnt_lo(uint32_t mask, uint32_t base) {
    const uint32_t lane = sim::lane();
    const uint32_t below = lane >= 32 ? 0xFFFFFFFFu : ((1u << lane) - 1u);
    return base + (uint32_t)__builtin_popcount(mask & below);
}
inline uint32_t sim_mbcnt_hi(uint32_t mask, uint32_t base) {
    const uint32_t lane = sim::lane();
    const uint32_t below = lane <= 32 ? 0u : ((1u << (lane - 32)) - 1u);
    return base + (uint32_t)__builtin_popcount(mask & below);
}
#define __builtin_amdgcn_mbcnt_lo(mask, base) sim_mbcnt_lo((mask), (base))
#define __builtin_amdgcn_mbcnt_hi(mask, base) sim_mbcnt_hi((mask), (base))
#define __builtin_amdgcn_fence(order, scope) ((void)0)
#define __builtin_amdgcn_wave_barrier() ((void)sim::meet_wave(0, nullptr))
#define __builtin_amdgcn_s_sleep(n) ((void)0)
#define __builtin_amdgcn_rcpf(x) (1.0f / (x))
#define __builtin_amdgcn_sqrtf(x) (std::sqrt((float)(x)))

// ---- atomics: one fiber runs at a time -------------------------------------------------------------------------------
template <typename T>
inline T atomicAdd(T* p, T v) { const T old = *p; *p = old + v; return old; }
inline unsigned long long atomicAdd(unsigned long long* p, unsigned long long v) { const auto old = *p; *p = old + v; return old; }
template <typename T>
inline T atomicOr(T* p, T v) { const T old = *p; *p = old | v; return old; }
template <typename T>
inline T atomicAnd(T* p, T v) { const T old = *p; *p = old & v; return old; }
template <typename T>
inline T atomicMin(T* p, T v) { const T old = *p; *p = old < v ? old : v; return old; }
template <typename T>
inline T atomicMax(T* p, T v) { const T old = *p; *p = old > v ? old : v; return old; }
#define __HIP_MEMORY_SCOPE_AGENT 0
#define __hip_atomic_load(p, order, scope) (*(p))
#define __hip_atomic_store(p, v, order, scope) (*(p) = (v))

// ---- scalar device functions ---------------------------------------------------------------------------------------
inline uint32_t __float_as_uint(float f) { uint32_t u; std::memcpy(&u, &f, 4); return u; }
inline int __float_as_int(float f) { int u; std::memcpy(&u, &f, 4); return u; }
inline float __uint_as_float(uint32_t u) { float f; std::memcpy(&f, &u, 4); return f; }
inline float __int_as_float(int u) { float f; std::memcpy(&f, &u, 4); return f; }
inline int __popc(uint32_t v) { return __builtin_popcount(v); }
inline int __popcll(unsigned long long v) { return __builtin_popcountll(v); }
inline int __ffs(uint32_t v) { return __builtin_ffs((int)v); }
inline int __clz(uint32_t v) { return v ? __builtin_clz(v) : 32; }
inline float __saturatef(float v) { return v < 0.0f ? 0.0f : (v > 1.0f ? 1.0f : (v == v ? v : 0.0f)); }
inline float rsqrtf(float v) { return 1.0f / std::sqrt(v); }
inline float __expf(float v) { return std::exp(v); }
inline int __float2int_rn(float v) { return (int)std::nearbyint(v); }
inline uint32_t min(uint32_t a, uint32_t b) { return a < b ? a : b; }
inline uint32_t max(uint32_t a, uint32_t b) { return a > b ? a : b; }
inline int min(int a, int b) { return a < b ? a : b; }
inline int max(int a, int b) { return a > b ? a : b; }
inline size_t min(size_t a, size_t b) { return a < b ? a : b; }
inline size_t max(size_t a, size_t b) { return a > b ? a : b; }
inline uint64_t min(unsigned long long a, unsigned long long b) { return a < b ? a : b; }

// ---- runtime API ---------------------------------------------------------------------------------------------------
typedef int hipError_t;
constexpr hipError_t hipSuccess = 0;
typedef void* hipStream_t;
typedef void* hipEvent_t;
enum hipStreamCaptureStatus { hipStreamCaptureStatusNone = 0, hipStreamCaptureStatusActive = 1 };
enum hipMemcpyKind { hipMemcpyHostToDevice = 1, hipMemcpyDeviceToHost = 2, hipMemcpyDeviceToDevice = 3 };
enum hipDeviceAttribute_t { hipDeviceAttributeMultiprocessorCount = 1 };
enum hipFuncAttribute { hipFuncAttributeMaxDynamicSharedMemorySize = 1 };
constexpr unsigned hipStreamNonBlocking = 1, hipEventDisableTiming = 2;
inline const char* hipGetErrorString(hipError_t) { return "simulated HIP runtime"; }
inline hipError_t hipGetLastError() { return hipSuccess; }
inline hipError_t hipGetDevice(int* d) { *d = 0; return hipSuccess; }
inline hipError_t hipStreamSynchronize(hipStream_t) { return hipSuccess; }
inline hipError_t hipStreamIsCapturing(hipStream_t, hipStreamCaptureStatus* s) { *s = hipStreamCaptureStatusNone; return hipSuccess; }
inline hipError_t hipStreamCreateWithFlags(hipStream_t* s, unsigned) { *s = (hipStream_t)0x1; return hipSuccess; }
inline hipError_t hipStreamDestroy(hipStream_t) { return hipSuccess; }
inline hipError_t hipStreamWaitEvent(hipStream_t, hipEvent_t, unsigned) { return hipSuccess; }
// an event is the host's clock at the moment it is recorded: launches run to completion inside the launch call
inline hipError_t hipEventCreate(hipEvent_t* e) { *e = new double(0.0); return hipSuccess; }
inline hipError_t hipEventCreateWithFlags(hipEvent_t* e, unsigned) { return hipEventCreate(e); }
inline hipError_t hipEventDestroy(hipEvent_t e) { delete (double*)e; return hipSuccess; }
inline hipError_t hipEventRecord(hipEvent_t e, hipStream_t) {
    *(double*)e = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now().time_since_epoch()).count();
    return hipSuccess;
}
inline hipError_t hipEventSynchronize(hipEvent_t) { return hipSuccess; }
inline hipError_t hipEventElapsedTime(float* ms, hipEvent_t start, hipEvent_t stop) {
    *ms = (float)(*(double*)stop - *(double*)start);
    return hipSuccess;
}
inline hipError_t hipMemcpyAsync(void* dst, const void* src, size_t bytes, hipMemcpyKind, hipStream_t) { std::memcpy(dst, src, bytes); return hipSuccess; }
inline hipError_t hipMemsetAsync(void* dst, int value, size_t bytes, hipStream_t) { std::memset(dst, value, bytes); return hipSuccess; }
inline hipError_t hipDeviceGetAttribute(int* v, hipDeviceAttribute_t, int) { *v = 2; return hipSuccess; }
template <typename F>
inline hipError_t hipOccupancyMaxActiveBlocksPerMultiprocessor(int* n, F, int, size_t) { *n = 1; return hipSuccess; }
inline hipError_t hipFuncSetAttribute(const void*, hipFuncAttribute, int) { return hipSuccess; }
#define HIP_SYMBOL(x) (x)
template <typename T>
inline hipError_t hipGetSymbolAddress(void** p, T& symbol) { *p = (void*)&symbol; return hipSuccess; }

#define hipLaunchKernelGGL(kernel, grid, block, lds, stream, ...) \
    sim::launch((grid), (block), (size_t)(lds), [&]() { kernel(__VA_ARGS__); })
