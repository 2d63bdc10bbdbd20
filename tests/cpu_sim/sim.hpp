// sim.hpp — a small SIMT simulator for the tests: runs a __global__ function of the library on the CPU, one block after
// the other, every thread of a block as a fiber of its own (all fibers of a block in one OS thread, so nothing races).
// Wave-level operations (ballot, shuffles, DPP, wave barriers) and block barriers are meeting points: a fiber that
// reaches one waits there until all live fibers of its wave (block) have reached it, then all of them take their
// results. Between meeting points the fibers of a wave run one after the other, not in lockstep: code that hands data
// from lane to lane through memory has to have a wave barrier in between, as the kernels do. The order in which the
// fibers of a block (and the blocks of a grid) are resumed is the environment variable INPC_SIM_ORDER's: forward, reverse
// or shuffle; the tests must pass under all three.
// TEST INFRASTRUCTURE ONLY: it exists so that the kernels' logic can be run against the oracle where there is no GPU.
#pragma once

#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <vector>

namespace sim {

constexpr int kWave = 64;
constexpr int kMaxThreads = 1024;

struct Dim3 {
    uint32_t x, y, z;
    constexpr Dim3(uint32_t x_ = 1, uint32_t y_ = 1, uint32_t z_ = 1) : x(x_), y(y_), z(z_) {}
};

struct Fiber {
    void* sp = nullptr;          // saved stack pointer while the fiber is switched out
    char* stack = nullptr;
    bool done = false;
    uint32_t tid = 0;            // thread index in the block
    uint64_t wave_gen = 0;       // meeting points of its wave / of the block it has passed
    uint64_t block_gen = 0;
};

// One group of fibers that meet: a wave or the whole block.
struct Meeting {
    uint64_t slot[2][kMaxThreads];   // what every member brought, by generation parity
    uint64_t present[2][kMaxThreads / 64];
    uint64_t mask[2][kMaxThreads / 64];   // members present when the generation completed
    uint32_t arrived[2] = {0, 0};
    uint64_t completed = 0;
    uint32_t alive = 0;
};

struct Block {
    Dim3 block_idx, block_dim, grid_dim;
    uint32_t n_threads = 0;
    std::vector<Fiber> fibers;
    Meeting block_meeting;
    std::vector<Meeting> waves;
    char* dynamic_lds = nullptr;        // 64-byte aligned, exactly as many bytes as the launch asked for (so that a
    size_t dynamic_lds_bytes = 0;       // sanitizer sees an access behind them)
    void* scheduler_sp = nullptr;
    std::function<void()> body;
    bool progress = false;
};

Block& block();            // of the calling fiber
Fiber& fiber();
void yield();              // back to the scheduler; returns when the fiber is resumed

// Runs `body` once per thread of every block of the grid.
void launch(Dim3 grid, Dim3 block_dim, size_t dynamic_lds_bytes, std::function<void()> body);

// The calling fiber brings `value` to the next meeting point of its wave (block) and waits for the others.
// Returns the values of all members (indexed by lane / by thread); `members` receives who was there.
const uint64_t* meet_wave(uint64_t value, uint64_t* members);
const uint64_t* meet_block(uint64_t value, const uint64_t** members);

inline uint32_t lane() { return fiber().tid & 63u; }

}  // namespace sim
