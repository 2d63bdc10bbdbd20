// sim.cpp — fibers and meeting points of the SIMT simulator (see sim.hpp). x86-64 only.
#include "sim.hpp"

#include <cstdlib>
#include <cstring>
#include <utility>

#include <cstdio>

// The section that holds every __shared__ variable of the library this file is linked into (hip/hip_runtime.h); the
// linker provides its bounds. Weak: a library without __shared__ variables has no such section.
extern "C" char __start_sim_lds[] __attribute__((weak));
extern "C" char __stop_sim_lds[] __attribute__((weak));

namespace sim {

namespace {
thread_local Block* g_block = nullptr;
thread_local Fiber* g_fiber = nullptr;
constexpr size_t kStackBytes = 256 * 1024;

// Saves the callee-saved registers on the current stack, stores the stack pointer in *from, switches to `to`.
extern "C" void sim_switch(void** from, void* to);
asm(R"(
.text
.globl sim_switch
.type sim_switch,@function
sim_switch:
    pushq %rbp
    pushq %rbx
    pushq %r12
    pushq %r13
    pushq %r14
    pushq %r15
    subq $8, %rsp
    stmxcsr (%rsp)
    fnstcw 4(%rsp)
    movq %rsp, (%rdi)
    movq %rsi, %rsp
    ldmxcsr (%rsp)
    fldcw 4(%rsp)
    addq $8, %rsp
    popq %r15
    popq %r14
    popq %r13
    popq %r12
    popq %rbx
    popq %rbp
    ret
.size sim_switch,.-sim_switch
)");

void fiber_main() {
    Block& b = *g_block;
    Fiber& f = *g_fiber;
    b.body();
    f.done = true;
    b.progress = true;
    // a fiber that ends no longer takes part in meetings: the others may be waiting for exactly that
    b.block_meeting.alive -= 1;
    b.waves[f.tid >> 6].alive -= 1;
    sim_switch(&f.sp, b.scheduler_sp);
    std::fprintf(stderr, "sim: a finished fiber was resumed\n");
    std::abort();
}

void prepare(Fiber& f) {
    if (!f.stack) f.stack = (char*)std::aligned_alloc(64, kStackBytes);
    // initial frame for sim_switch: mxcsr / x87 control word, six callee-saved registers, return address
    uintptr_t top = ((uintptr_t)f.stack + kStackBytes) & ~(uintptr_t)63;
    uint64_t* sp = (uint64_t*)top;
    *--sp = 0;                       // alignment: at fiber_main's entry rsp + 8 must be a multiple of 16
    *--sp = (uint64_t)&fiber_main;   // return address of the first switch
    for (int i = 0; i < 6; ++i) *--sp = 0;
    uint32_t mxcsr, fpcw = 0;
    asm volatile("stmxcsr %0" : "=m"(mxcsr));
    asm volatile("fnstcw %0" : "=m"(*(uint16_t*)&fpcw));
    *--sp = ((uint64_t)fpcw << 32) | mxcsr;
    f.sp = sp;
}

const uint64_t* meet(Meeting& m, uint64_t& my_gen, uint32_t index, uint64_t value) {
    Block& b = *g_block;
    const uint64_t g = my_gen;
    const int p = (int)(g & 1u);
    if (m.arrived[p] == 0) std::memset(m.present[p], 0, sizeof(m.present[p]));
    m.slot[p][index] = value;
    m.present[p][index >> 6] |= 1ull << (index & 63u);
    m.arrived[p] += 1;
    b.progress = true;
    while (m.completed < g + 1) {
        if (m.arrived[p] >= m.alive) {
            std::memcpy(m.mask[p], m.present[p], sizeof(m.present[p]));
            m.completed = g + 1;
            m.arrived[p] = 0;
            b.progress = true;
            break;
        }
        yield();
    }
    my_gen = g + 1;
    return m.slot[p];
}
}  // namespace

Block& block() { return *g_block; }
Fiber& fiber() { return *g_fiber; }

void yield() {
    Fiber& f = *g_fiber;
    sim_switch(&f.sp, g_block->scheduler_sp);
}

const uint64_t* meet_wave(uint64_t value, uint64_t* members) {
    Fiber& f = *g_fiber;
    Meeting& m = g_block->waves[f.tid >> 6];
    const int p = (int)(f.wave_gen & 1u);
    const uint64_t* slots = meet(m, f.wave_gen, f.tid & 63u, value);
    if (members) *members = m.mask[p][0];
    return slots;
}

const uint64_t* meet_block(uint64_t value, const uint64_t** members) {
    Fiber& f = *g_fiber;
    Meeting& m = g_block->block_meeting;
    const int p = (int)(f.block_gen & 1u);
    const uint64_t* slots = meet(m, f.block_gen, f.tid, value);
    if (members) *members = m.mask[p];
    return slots;
}

// The order in which the scheduler resumes the fibers of a block between meeting points. Nothing a kernel computes may
// depend on it: lanes that hand data to each other through memory have a meeting point (a barrier) in between. The
// environment variable INPC_SIM_ORDER picks it: "forward" (thread 0 first, the default), "reverse", or "shuffle" (a new
// pseudo-random order for every sweep); a kernel that relies on its lanes running in step or in thread order gives
// different results under different orders.
namespace {
enum class Order { kForward, kReverse, kShuffle };
Order thread_order() {
    static const Order order = [] {
        const char* v = std::getenv("INPC_SIM_ORDER");
        if (v && std::strcmp(v, "reverse") == 0) return Order::kReverse;
        if (v && std::strcmp(v, "shuffle") == 0) return Order::kShuffle;
        return Order::kForward;
    }();
    return order;
}

// The byte that fills LDS before every block: 0xCD, or INPC_SIM_LDS_BYTE (a number) to see that no result depends on it.
int lds_pattern() {
    static const int pattern = [] {
        const char* v = std::getenv("INPC_SIM_LDS_BYTE");
        return v ? (int)(std::strtol(v, nullptr, 0) & 0xFF) : 0xCD;
    }();
    return pattern;
}

void next_order(std::vector<uint32_t>& order, uint32_t n) {
    static thread_local uint64_t state = 0x9E3779B97F4A7C15ull;
    const Order mode = thread_order();
    if (order.size() != n || mode == Order::kShuffle) {
        order.resize(n);
        for (uint32_t i = 0; i < n; ++i) order[i] = mode == Order::kReverse ? n - 1u - i : i;
    }
    if (mode == Order::kShuffle)
        for (uint32_t i = n; i > 1; --i) {
            state = state * 6364136223846793005ull + 1442695040888963407ull;
            std::swap(order[i - 1], order[(uint32_t)((state >> 33) % i)]);
        }
}
}  // namespace

void launch(Dim3 grid, Dim3 block_dim, size_t dynamic_lds_bytes, std::function<void()> body) {
    const uint32_t n_threads = block_dim.x * block_dim.y * block_dim.z;
    if (n_threads == 0 || n_threads > (uint32_t)kMaxThreads) {
        std::fprintf(stderr, "sim: %u threads per block\n", n_threads);
        std::abort();
    }
    static thread_local Block b;   // the stacks are kept from launch to launch
    Block* outer_block = g_block;
    Fiber* outer_fiber = g_fiber;
    g_block = &b;
    b.block_dim = block_dim;
    b.grid_dim = grid;
    b.n_threads = n_threads;
    if (b.fibers.size() < n_threads) b.fibers.resize(n_threads);
    b.waves.resize((n_threads + 63) / 64);
    if (b.dynamic_lds_bytes != dynamic_lds_bytes || !b.dynamic_lds) {
        std::free(b.dynamic_lds);
        void* p = nullptr;
        if (posix_memalign(&p, 64, dynamic_lds_bytes ? dynamic_lds_bytes : 1) != 0) std::abort();
        b.dynamic_lds = (char*)p;
        b.dynamic_lds_bytes = dynamic_lds_bytes;
    }
    b.body = std::move(body);
    static thread_local std::vector<uint32_t> order;
    const bool blocks_reversed = thread_order() != Order::kForward;
    for (uint32_t iz = 0; iz < grid.z; ++iz)
        for (uint32_t iy = 0; iy < grid.y; ++iy)
            for (uint32_t ix = 0; ix < grid.x; ++ix) {
                // the blocks of a grid may run in any order: with the threads' order the blocks' is turned round too
                const uint32_t bx = blocks_reversed ? grid.x - 1u - ix : ix, by = blocks_reversed ? grid.y - 1u - iy : iy,
                               bz = blocks_reversed ? grid.z - 1u - iz : iz;
                b.block_idx = Dim3(bx, by, bz);
                // LDS holds what the block before left there, or anything: a kernel that counts on zeros shows up
                std::memset(b.dynamic_lds, lds_pattern(), b.dynamic_lds_bytes);
                if (__start_sim_lds && __stop_sim_lds > __start_sim_lds)
                    std::memset(__start_sim_lds, lds_pattern(), (size_t)(__stop_sim_lds - __start_sim_lds));
                b.block_meeting = Meeting{};
                b.block_meeting.alive = n_threads;
                for (size_t w = 0; w < b.waves.size(); ++w) {
                    b.waves[w] = Meeting{};
                    b.waves[w].alive = std::min<uint32_t>(64u, n_threads - (uint32_t)w * 64u);
                }
                for (uint32_t t = 0; t < n_threads; ++t) {
                    Fiber& f = b.fibers[t];
                    f.done = false;
                    f.tid = t;
                    f.wave_gen = f.block_gen = 0;
                    prepare(f);
                }
                uint32_t left = n_threads;
                while (left) {
                    b.progress = false;
                    left = 0;
                    next_order(order, n_threads);
                    for (uint32_t k = 0; k < n_threads; ++k) {
                        const uint32_t t = order[k];
                        Fiber& f = b.fibers[t];
                        if (f.done) continue;
                        g_fiber = &f;
                        sim_switch(&b.scheduler_sp, f.sp);
                        if (!f.done) ++left;
                    }
                    if (left && !b.progress) {
                        std::fprintf(stderr, "sim: deadlock in block (%u,%u,%u): %u fibers wait at meeting points "
                                             "that not all live fibers of their wave or block reach\n", bx, by, bz, left);
                        std::abort();
                    }
                }
            }
    g_block = outer_block;
    g_fiber = outer_fiber;
}

}  // namespace sim
