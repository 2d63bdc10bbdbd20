// runtime.hip — error reporting, per-launch timing hooks, fill kernel, PCG32 host helpers.
#include <algorithm>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "common.hpp"

namespace inpc {

namespace {
thread_local char g_error[512] = "";

struct TimingEntry {
    const char* name;
    hipEvent_t start, stop;
};
thread_local bool g_timing_on = false;
thread_local std::vector<TimingEntry> g_timing_entries;
thread_local std::vector<hipEvent_t> g_event_pool;
thread_local TimingEntry g_open{nullptr, nullptr, nullptr};

hipEvent_t take_event() {
    if (!g_event_pool.empty()) {
        hipEvent_t e = g_event_pool.back();
        g_event_pool.pop_back();
        return e;
    }
    hipEvent_t e = nullptr;
    if (hipEventCreate(&e) != hipSuccess) return nullptr;
    return e;
}
}  // namespace

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}

bool timing_enabled() { return g_timing_on; }

namespace {
struct LaneEntry {
    int device;
    hipStream_t owner;
    SideLane lane;
};
std::mutex g_lane_mutex;
std::vector<std::unique_ptr<LaneEntry>> g_lanes;   // entries never move or go away: callers keep pointers to them
}  // namespace

// Which lane, if any, a forward pass on `owner` may use: the decision of side_lane() without the HIP calls.
//   existing:           a lane for (device, owner) exists
//   owner_is_capturing: the caller's stream is being captured into a graph
//   lane_is_capturing:  the lane's stream is (only asked when a lane exists)
//   n_lanes:            lanes the process keeps
enum class LaneChoice : int { kUse = 0, kCreate = 1, kNone = 2 };
LaneChoice choose_lane(bool existing, bool owner_is_capturing, bool lane_is_capturing, int n_lanes) {
    if (existing) {
        // between two calls the lane's stream is idle and outside any capture: each call joins it back into the
        // caller's stream before it returns. A lane that still captures although its owner does not belongs to a
        // capture that was abandoned half-way; it is left alone.
        if (lane_is_capturing && !owner_is_capturing) return LaneChoice::kNone;
        return LaneChoice::kUse;
    }
    if (owner_is_capturing) return LaneChoice::kNone;   // creating a stream is no operation for a capture
    if (n_lanes >= kMaxSideLanes) return LaneChoice::kNone;
    return LaneChoice::kCreate;
}

SideLane* side_lane(hipStream_t owner, bool owner_is_capturing) {
    int device = -1;
    if (hipGetDevice(&device) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(g_lane_mutex);
    LaneEntry* found = nullptr;
    for (auto& e : g_lanes)
        if (e->device == device && e->owner == owner) found = e.get();
    bool lane_is_capturing = false;
    if (found) {
        hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(found->lane.stream, &status) != hipSuccess) {
            (void)hipGetLastError();
            return nullptr;
        }
        lane_is_capturing = status != hipStreamCaptureStatusNone;
    }
    switch (choose_lane(found != nullptr, owner_is_capturing, lane_is_capturing, (int)g_lanes.size())) {
        case LaneChoice::kUse: return &found->lane;
        case LaneChoice::kNone: return nullptr;
        case LaneChoice::kCreate: break;
    }
    auto entry = std::make_unique<LaneEntry>();
    entry->device = device;
    entry->owner = owner;
    SideLane& lane = entry->lane;
    lane.stream = nullptr;
    lane.fork = lane.join = nullptr;
    // no timing data in the events: they only order the two streams
    if (hipStreamCreateWithFlags(&lane.stream, hipStreamNonBlocking) != hipSuccess ||
        hipEventCreateWithFlags(&lane.fork, hipEventDisableTiming) != hipSuccess ||
        hipEventCreateWithFlags(&lane.join, hipEventDisableTiming) != hipSuccess) {
        (void)hipGetLastError();   // the failure is handled here: the caller works without the lane
        if (lane.fork) (void)hipEventDestroy(lane.fork);
        if (lane.stream) (void)hipStreamDestroy(lane.stream);
        return nullptr;
    }
    g_lanes.push_back(std::move(entry));
    return &g_lanes.back()->lane;
}

void timing_begin(const char* name, hipStream_t stream) {
    if (!g_timing_on) return;
    g_open.name = name;
    g_open.start = take_event();
    g_open.stop = take_event();
    if (g_open.start) (void)hipEventRecord(g_open.start, stream);
}

void timing_end(hipStream_t stream) {
    if (!g_timing_on || !g_open.name) return;
    if (g_open.stop) (void)hipEventRecord(g_open.stop, stream);
    g_timing_entries.push_back(g_open);
    g_open = TimingEntry{nullptr, nullptr, nullptr};
}

__global__ void __launch_bounds__(256) k_fill_u32(uint32_t* dst, uint32_t value, size_t n) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) dst[i] = value;
}

int fill_u32(void* dst, uint32_t value, size_t n_words, hipStream_t stream) {
    if (n_words == 0) return INPC_OK;
    const uint32_t blocks = (uint32_t)std::min<size_t>((n_words + 255) / 256, 8192);
    INPC_LAUNCH("fill_u32", k_fill_u32, dim3(blocks), dim3(256), stream, (uint32_t*)dst, value, n_words);
    return INPC_OK;
}

int resident_blocks(const void* kernel, int threads, uint32_t& blocks) {
    // asked on every launch of a resident grid: remembered per (device, kernel, block size)
    struct Entry {
        int device;
        const void* kernel;
        int threads;
        uint32_t blocks;
    };
    static std::mutex lock;
    static std::vector<Entry> known;
    int device = 0;
    INPC_HIP_CHECK(hipGetDevice(&device));
    {
        std::lock_guard<std::mutex> guard(lock);
        for (const Entry& e : known)
            if (e.device == device && e.kernel == kernel && e.threads == threads) {
                blocks = e.blocks;
                return INPC_OK;
            }
    }
    int per_cu = 0, cus = 0;
    INPC_HIP_CHECK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device));
    INPC_HIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, threads, 0));
    if (per_cu < 1 || cus < 1) return fail(INPC_E_HIP, "occupancy query returned %d blocks on %d compute units", per_cu, cus);
    blocks = (uint32_t)per_cu * (uint32_t)cus;
    std::lock_guard<std::mutex> guard(lock);
    known.push_back(Entry{device, kernel, threads, blocks});
    return INPC_OK;
}

// Plain streaming copy, 16 bytes per lane: the yardstick for profiler byte counters.
__global__ void __launch_bounds__(256) k_copy_u128(const uint4* __restrict__ src, uint4* __restrict__ dst, size_t n) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) dst[i] = src[i];
}

}  // namespace inpc

extern "C" {

int inpc_calibration_copy(const void* src, void* dst, size_t bytes, void* stream) {
    using namespace inpc;
    if (!src || !dst) return fail(INPC_E_INVALID_ARGUMENT, "calibration_copy: null pointer");
    if (bytes % 16 != 0 || ((uintptr_t)src | (uintptr_t)dst) % 16 != 0)
        return fail(INPC_E_INVALID_ARGUMENT, "calibration_copy: pointers and size must be multiples of 16 bytes");
    if (bytes == 0) return INPC_OK;
    const size_t n = bytes / 16;
    const uint32_t blocks = (uint32_t)std::min<size_t>((n + 255) / 256, 16384);
    INPC_LAUNCH("calibration_copy", k_copy_u128, dim3(blocks), dim3(256), (hipStream_t)stream, (const uint4*)src,
                (uint4*)dst, n);
    return INPC_OK;
}

const char* inpc_last_error(void) { return inpc::g_error; }

int inpc_abi_version(void) { return 4; }

int inpc_side_stream_policy(int existing, int stream_is_capturing, int second_is_capturing, int n_kept) {
    return (int)inpc::choose_lane(existing != 0, stream_is_capturing != 0, second_is_capturing != 0, n_kept);
}

void inpc_timing_enable(int on) {
    inpc::g_timing_on = on != 0;
    if (!on) {
        for (auto& e : inpc::g_timing_entries) {
            inpc::g_event_pool.push_back(e.start);
            inpc::g_event_pool.push_back(e.stop);
        }
        inpc::g_timing_entries.clear();
    }
}

int inpc_timing_collect(inpc_timing_record* out, int capacity) {
    int n = 0;
    for (auto& e : inpc::g_timing_entries) {
        float ms = 0.0f;
        if (e.start && e.stop && hipEventSynchronize(e.stop) == hipSuccess &&
            hipEventElapsedTime(&ms, e.start, e.stop) == hipSuccess) {
            if (n < capacity) {
                out[n].name = e.name;
                out[n].ms = ms;
                ++n;
            }
        }
        if (e.start) inpc::g_event_pool.push_back(e.start);
        if (e.stop) inpc::g_event_pool.push_back(e.stop);
    }
    inpc::g_timing_entries.clear();
    return n;
}

void inpc_pcg32_seed(uint64_t rng[2], uint64_t initstate, uint64_t initseq) {
    inpc::Pcg32 r;
    r.state = 0u;
    r.inc = (initseq << 1u) | 1u;
    inpc::pcg_next(r);
    r.state += initstate;
    inpc::pcg_next(r);
    rng[0] = r.state;
    rng[1] = r.inc;
}

uint32_t inpc_pcg32_next_uint(uint64_t rng[2]) {
    inpc::Pcg32 r{rng[0], rng[1]};
    const uint32_t v = inpc::pcg_next(r);
    rng[0] = r.state;
    return v;
}

float inpc_pcg32_next_float(uint64_t rng[2]) {
    union {
        uint32_t u;
        float f;
    } x;
    x.u = (inpc_pcg32_next_uint(rng) >> 9) | 0x3f800000u;
    return x.f - 1.0f;
}

void inpc_pcg32_advance(uint64_t rng[2], int64_t delta) {
    const inpc::PcgJump j = inpc::pcg_jump(rng[1], (uint64_t)delta);
    rng[0] = inpc::pcg_apply(j, rng[0]);
}

}  // extern "C"
