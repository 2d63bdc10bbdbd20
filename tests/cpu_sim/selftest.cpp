// selftest.cpp — small kernels that check the simulator itself (tests/test_sim_selftest.py): what its wave and block
// operations return, against their definitions stated independently in the test, and that a hand-off between lanes
// without a barrier gives results that depend on the order in which the threads are resumed (INPC_SIM_ORDER), while
// the same hand-off with a barrier does not. Compiled with the simulator's stand-in for hip/hip_runtime.h only.
#include <hip/hip_runtime.h>

namespace {

__global__ void k_handoff(uint32_t* out, int with_barrier) {
    __shared__ uint32_t s_value[256];
    const uint32_t t = threadIdx.x;
    s_value[t] = 0u;
    __syncthreads();
    s_value[t] = 3u * t + 1u;
    if (with_barrier) __syncthreads();
    out[blockIdx.x * 256u + t] = s_value[255u - t];   // the value of a thread at the other end of the block
}

// inclusive sum over the wave from row shifts and the two row broadcasts, the way scan kernels on this hardware do it
__device__ uint32_t dpp(uint32_t old, uint32_t v, int ctrl, int row_mask) {
    return (uint32_t)__builtin_amdgcn_update_dpp((int)old, (int)v, ctrl, row_mask, 0xf, false);
}
__global__ void k_wave_ops(const uint32_t* in, uint32_t* scan, uint64_t* ballots, uint32_t* shuffled, uint32_t* quads,
                           uint32_t* counted) {
    const uint32_t t = threadIdx.x, lane = t & 63u;
    uint32_t v = in[t];
    uint32_t s = v;
    s += dpp(0u, s, 0x111, 0xf);
    s += dpp(0u, s, 0x112, 0xf);
    s += dpp(0u, s, 0x114, 0xf);
    s += dpp(0u, s, 0x118, 0xf);
    s += dpp(0u, s, 0x142, 0xa);
    s += dpp(0u, s, 0x143, 0xc);
    scan[t] = s;
    const unsigned long long b = __ballot((v & 1u) != 0u);
    if (lane == 0u) ballots[t >> 6] = b;
    shuffled[t] = __shfl(v, (int)((lane * 7u + 3u) & 63u), 64) + 1000u * __shfl_xor(v, 5, 64) + 1000000u * __shfl_up(v, 2u, 64);
    quads[t] = dpp(77u, v, 0xB1, 0xf) + 100000u * dpp(77u, v, 0x138, 0xf);   // neighbours swapped; the lane in front
    // block-wide counts with threads that have left: thread t leaves before the barrier when t % 5 == 0
    if (t % 5u == 0u) return;
    const int n = __syncthreads_count((v & 2u) != 0u);
    const int any = __syncthreads_or(v == 0xFFFFFFFFu);
    const int all = __syncthreads_and((v & 0x80000000u) == 0u);
    counted[t] = (uint32_t)n + 10000u * (uint32_t)any + 100000u * (uint32_t)all;
}

__global__ void k_atomics(uint32_t* counter, uint32_t* slots, float* total) {
    __shared__ uint32_t s_counter;
    if (threadIdx.x == 0) s_counter = 0u;
    __syncthreads();
    const uint32_t mine = atomicAdd(&s_counter, 1u);   // a ticket per thread: every value below 128 exactly once
    slots[blockIdx.x * 128u + mine] += 1u;
    atomicAdd(counter, threadIdx.x);
    atomicMax(counter + 1, blockIdx.x * 128u + threadIdx.x);
    atomicAdd(total, 0.5f);
}

}  // namespace

extern "C" {

int selftest_handoff(uint32_t* out, int with_barrier) {
    hipLaunchKernelGGL(k_handoff, dim3(3), dim3(256), 0, nullptr, out, with_barrier);
    return 0;
}

int selftest_wave_ops(const uint32_t* in, uint32_t* scan, uint64_t* ballots, uint32_t* shuffled, uint32_t* quads,
                      uint32_t* counted) {
    hipLaunchKernelGGL(k_wave_ops, dim3(1), dim3(192), 0, nullptr, in, scan, ballots, shuffled, quads, counted);
    return 0;
}

int selftest_atomics(uint32_t* counter, uint32_t* slots, float* total) {
    hipLaunchKernelGGL(k_atomics, dim3(5), dim3(128), 0, nullptr, counter, slots, total);
    return 0;
}

}  // extern "C"
