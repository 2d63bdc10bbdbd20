// radix.hpp — device-wide stable LSD radix sort of (key, value) pairs for gfx950.
//
// Replaces the two cub::DeviceRadixSort::SortPairs calls of the reference
// (B/rasterization/src/bilinear/forward.cu:91-98,132-139). One digit pass = one kernel:
//   - the digit histograms of all passes are accumulated by the kernel that produces the keys
//     (radix::hist_add / hist_flush), so keys are not read an extra time;
//   - a block ranks its 4096 keys stably (per-wave ballot matching, 64-wide), stages them through
//     LDS so that every digit leaves the block as one contiguous run, and finds its global offsets
//     with a decoupled look-back over per-(block, digit) status words.
// The grid is resident as a whole and walks over the tiles in order, so look-back only waits on running blocks.
#pragma once

#include "common.hpp"

namespace inpc {
namespace radix {

// Digits of up to 8 bits. (9-bit digits save a pass on 27-bit depth keys, but a pass then leaves the block in runs
// of 8 keys instead of 32 and takes a third longer: measured 3 x 88 us against 4 x 66 us.)
constexpr int kMaxBits = 8;
constexpr int kRadix = 1 << kMaxBits;
constexpr int kBlock = kRadix;          // thread d owns digit d
constexpr int kWaves = kBlock / kWave;
constexpr int kItems = 4096 / kRadix;
constexpr int kTile = kBlock * kItems;  // keys per block
constexpr int kMaxPasses = 4;
static_assert(kMaxBits * kMaxPasses >= 32, "every 32-bit key must fit the passes");
constexpr uint32_t kInvalidKey = 0xFFFFFFFFu;

struct PassPlan {
    int n_passes;
    int shift[kMaxPasses];
    int bits[kMaxPasses];
};

// Split `total_bits` key bits into the fewest passes of at most kMaxBits bits, as evenly as possible.
inline PassPlan make_plan(int total_bits) {
    PassPlan p{};
    if (total_bits < 1) total_bits = 1;
    p.n_passes = (total_bits + kMaxBits - 1) / kMaxBits;
    const int base = total_bits / p.n_passes, rem = total_bits % p.n_passes;
    int shift = 0;
    for (int i = 0; i < p.n_passes; ++i) {
        p.bits[i] = base + (i < rem ? 1 : 0);
        p.shift[i] = shift;
        shift += p.bits[i];
    }
    return p;
}

struct DevicePlan {
    int n_passes;
    int shift[kMaxPasses];
    uint32_t mask[kMaxPasses];
};

inline DevicePlan to_device_plan(const PassPlan& p) {
    DevicePlan d{};
    d.n_passes = p.n_passes;
    for (int i = 0; i < p.n_passes; ++i) {
        d.shift[i] = p.shift[i];
        d.mask[i] = (1u << p.bits[i]) - 1u;
    }
    return d;
}

// ---- histogram helpers for the key-producing kernels -------------------------------------------------
// s_hist is uint32_t[n_passes * kRadix] in LDS, zeroed by the caller.
__device__ __forceinline__ void hist_add(uint32_t* s_hist, const DevicePlan& plan, uint32_t key) {
    for (int p = 0; p < plan.n_passes; ++p) atomicAdd(&s_hist[p * kRadix + ((key >> plan.shift[p]) & plan.mask[p])], 1u);
}

__device__ __forceinline__ void hist_flush(const uint32_t* s_hist, const DevicePlan& plan, uint32_t* g_hist) {
    for (int i = threadIdx.x; i < plan.n_passes * kRadix; i += blockDim.x) {
        const uint32_t c = s_hist[i];
        if (c) atomicAdd(&g_hist[i], c);
    }
}

// Exclusive scan of each kRadix-bin histogram (one block per pass).
__global__ void __launch_bounds__(kRadix) k_digit_bases(const uint32_t* __restrict__ hist, uint32_t* __restrict__ bases) {
    __shared__ uint32_t s_wave[kRadix / kWave];
    const uint32_t d = threadIdx.x, lane = d & 63u, wave = d >> 6;
    const uint32_t v = hist[blockIdx.x * kRadix + d];
    uint32_t incl = v;
#pragma unroll
    for (int s = 1; s < 64; s <<= 1) {
        const uint32_t up = __shfl_up(incl, s, 64);
        if (lane >= (uint32_t)s) incl += up;
    }
    if (lane == 63) s_wave[wave] = incl;
    __syncthreads();
    uint32_t base = 0;
    for (uint32_t w = 0; w < wave; ++w) base += s_wave[w];
    bases[blockIdx.x * kRadix + d] = base + incl - v;
}

// How the first pass of a sort treats its input.
enum FirstPass : int {
    kPlain = 0,        // n keys (n on the device), all valid
    kSkipInvalid = 1,  // n_max keys (n on the host); keys equal to kInvalidKey are dropped, which compacts
                       // the drawn points for free
};

// One digit pass. FIRST: n comes from the host and keys equal to kInvalidKey are dropped.
// Order of work inside a block: load -> digit histogram (LDS atomics) -> publish the aggregates -> stable
// ranking -> look-back walk -> LDS staging -> coalesced write. Publishing before the expensive ranking means
// that, by the time a block walks back, its predecessors' aggregates are already there.
template <typename KeyT, bool FIRST>
__global__ void __launch_bounds__(kBlock)
    k_scatter(const KeyT* __restrict__ keys_in, const uint32_t* __restrict__ vals_in, KeyT* __restrict__ keys_out,
              uint32_t* __restrict__ vals_out, const uint32_t* __restrict__ n_dev, uint32_t n_host, int shift,
              uint32_t digit_mask, int bits, const uint32_t* __restrict__ digit_base, uint32_t* status,
              uint32_t* error_flag) {
    __shared__ uint32_t s_cnt[kWaves][kRadix];
    __shared__ uint32_t s_hist[kRadix];
    __shared__ uint32_t s_local_base[kRadix];
    __shared__ uint32_t s_global[kRadix];
    __shared__ KeyT s_keys[kTile];
    __shared__ uint32_t s_vals[kTile];
    __shared__ uint32_t s_wave[kWaves];
    __shared__ uint32_t s_bid;

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    uint32_t n = n_host;
    if (!FIRST) n = min(n_host, *n_dev);
    // A block takes its tiles from a ticket counter, in order: a tile waits (look-back) only for tiles in front of
    // it, and each of those was taken by a block that was running when it took it. So nothing ever waits for a
    // block that has not started, whatever else occupies the GPU; the grid only needs as many blocks as fit.
    uint32_t* ticket = status + (size_t)((n_host + kTile - 1u) / kTile) * kRadix;
    for (;;) {
    if (tid == 0) s_bid = atomicAdd(ticket, 1u);
    __syncthreads();
    const uint32_t bid = s_bid;
    const uint64_t tile_base = (uint64_t)bid * kTile;
    if (tile_base >= n) break;
    for (int i = tid; i < kWaves * kRadix; i += kBlock) (&s_cnt[0][0])[i] = 0u;
    s_hist[tid] = 0u;
    __syncthreads();

    KeyT key[kItems];
    uint32_t val[kItems];
    uint32_t valid_bits = 0;
    const uint64_t wave_base = tile_base + (uint64_t)wave * (kItems * kWave);
#pragma unroll
    for (int r = 0; r < kItems; ++r) {
        const uint64_t idx = wave_base + (uint64_t)r * kWave + lane;
        bool valid = idx < n;
        KeyT k = 0;
        if (valid) k = keys_in[idx];
        if (FIRST) valid = valid && ((uint32_t)k != kInvalidKey);
        val[r] = valid ? vals_in[idx] : 0u;
        key[r] = k;
        if (valid) valid_bits |= 1u << r;
    }
#pragma unroll
    for (int r = 0; r < kItems; ++r)
        if (valid_bits & (1u << r)) atomicAdd(&s_hist[((uint32_t)key[r] >> shift) & digit_mask], 1u);
    __syncthreads();
    // thread d owns digit d: block total, publish, position of the digit's run inside the block
    const uint32_t total = s_hist[tid];
    if (tid <= digit_mask) lookback_publish(status + tid, kRadix, bid, total);
    uint32_t incl = total;
#pragma unroll
    for (int s = 1; s < 64; s <<= 1) {
        const uint32_t up = __shfl_up(incl, s, 64);
        if (lane >= (uint32_t)s) incl += up;
    }
    if (lane == 63) s_wave[wave] = incl;

    // stable rank of every key among the keys of its wave with the same digit
    uint32_t rank[kItems];
#pragma unroll
    for (int r = 0; r < kItems; ++r) {
        const bool valid = (valid_bits >> r) & 1u;
        const uint32_t d = ((uint32_t)key[r] >> shift) & digit_mask;
        uint64_t peers = __ballot(valid);
        for (int b = 0; b < bits; ++b) {
            const bool bit = (d >> b) & 1u;
            const uint64_t set = __ballot(valid && bit);
            peers &= bit ? set : ~set;
        }
        rank[r] = 0;
        if (valid) {
            const uint32_t before = s_cnt[wave][d];
            rank[r] = before + mask_rank(peers);
            if (lane == 63u - (uint32_t)__clzll((long long)peers)) s_cnt[wave][d] = before + (uint32_t)__popcll(peers);
        }
        __builtin_amdgcn_wave_barrier();
    }
    __syncthreads();

    // per-wave offsets inside the digit's run, block-level exclusive scan over the digits
    {
        uint32_t run = 0;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            const uint32_t c = s_cnt[w][tid];
            s_cnt[w][tid] = run;
            run += c;
        }
    }
    uint32_t wave_off = 0, block_total = 0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
        const uint32_t c = s_wave[w];
        if ((uint32_t)w < wave) wave_off += c;
        block_total += c;
    }
    const uint32_t local_base = wave_off + incl - total;
    s_local_base[tid] = local_base;
    if (tid <= digit_mask) {  // one look-back per digit in use
        const uint32_t exclusive = lookback_walk(status + tid, kRadix, bid, total, error_flag);
        s_global[tid] = digit_base[tid] + exclusive - local_base;
    }
    __syncthreads();

#pragma unroll
    for (int r = 0; r < kItems; ++r) {
        if (valid_bits & (1u << r)) {
            const uint32_t d = ((uint32_t)key[r] >> shift) & digit_mask;
            const uint32_t pos = s_local_base[d] + s_cnt[wave][d] + rank[r];
            s_keys[pos] = key[r];
            s_vals[pos] = val[r];
        }
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < kItems; ++j) {
        const uint32_t idx = j * kBlock + tid;
        if (idx < block_total) {
            const KeyT k = s_keys[idx];
            const uint32_t d = ((uint32_t)k >> shift) & digit_mask;
            const uint32_t out = s_global[d] + idx;
            keys_out[out] = k;
            vals_out[out] = s_vals[idx];
        }
    }
    __syncthreads();   // the LDS arrays are reused by the next tile
    }
}

// Status words one pass needs for up to n_max keys: a word per (tile, digit), then the pass's ticket counter.
inline size_t status_words(uint32_t n_max) { return (size_t)div_up(n_max, kTile) * kRadix + kRadix; }

// Enqueue every pass of a sort. Buffers ping-pong: pass 0 reads keys_a / vals_a, the result ends in the
// a-buffers when the pass count is even, else in the b-buffers.
// hist: n_passes*256 filled histograms; bases: same size scratch; status: n_passes*status_words(n_max)
// zeroed words.
template <typename KeyT>
int sort_pairs(const PassPlan& plan, FirstPass first, KeyT* keys_a, uint32_t* vals_a, KeyT* keys_b,
               uint32_t* vals_b, const uint32_t* n_dev, uint32_t n_max, const uint32_t* hist, uint32_t* bases,
               uint32_t* status, uint32_t* error_flag, hipStream_t stream, const char* name) {
    if (n_max == 0) return INPC_OK;
    INPC_LAUNCH("radix_digit_bases", k_digit_bases, dim3(plan.n_passes), dim3(kRadix), stream, hist, bases);
    uint32_t resident_first = 0, resident_rest = 0;
    int rc = resident_blocks((const void*)k_scatter<KeyT, true>, kBlock, resident_first);
    if (rc != INPC_OK) return rc;
    rc = resident_blocks((const void*)k_scatter<KeyT, false>, kBlock, resident_rest);
    if (rc != INPC_OK) return rc;
    const uint32_t tiles = div_up(n_max, kTile);
    const size_t words = status_words(n_max);
    KeyT* kin = keys_a;
    uint32_t* vin = vals_a;
    KeyT* kout = keys_b;
    uint32_t* vout = vals_b;
    for (int p = 0; p < plan.n_passes; ++p) {
        const uint32_t mask = (1u << plan.bits[p]) - 1u;
        if (p == 0 && first == kSkipInvalid) {
            INPC_LAUNCH(name, (k_scatter<KeyT, true>), dim3(std::min(tiles, resident_first)), dim3(kBlock), stream, (const KeyT*)kin,
                        (const uint32_t*)vin, kout, vout, n_dev, n_max, plan.shift[p], mask, plan.bits[p],
                        (const uint32_t*)(bases + p * kRadix), status + p * words, error_flag);
        } else {
            INPC_LAUNCH(name, (k_scatter<KeyT, false>), dim3(std::min(tiles, resident_rest)), dim3(kBlock), stream, (const KeyT*)kin,
                        (const uint32_t*)vin, kout, vout, n_dev, n_max, plan.shift[p], mask, plan.bits[p],
                        (const uint32_t*)(bases + p * kRadix), status + p * words, error_flag);
        }
        std::swap(kin, kout);
        std::swap(vin, vout);
    }
    return INPC_OK;
}

}  // namespace radix
}  // namespace inpc
