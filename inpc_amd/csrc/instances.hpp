// instances.hpp — depth-ordered points -> per-tile instance lists in depth order, without a global sort.
// Included by raster.hip after the binning helpers.
//
// The reference expands every depth-sorted point into one (tile, point) instance per touched tile
// (B/rasterization/src/bilinear/kernels.cu:186-220) and then sorts all instances by tile with a stable radix
// sort (forward.cu:132-139), which leaves every tile's instances in depth order. The result is a stable
// distribution of a sequence over tiles, and that needs no device-wide sort:
//   k_inst_count   the depth-ordered points are cut into kChunks contiguous chunks; per (chunk, tile) count the
//                  instances (LDS histogram)                                   -> table[chunk][tile]
//   k_bin_offsets  per tile: exclusive prefix over the chunks                  (shared with the record binning)
//   k_bin_scan     exclusive scan over the tiles = [begin, end) of every tile  (kernels.cu:222-239)
//   k_inst_emit    a block walks its chunk in order: a few thousand instances at a time are expanded into LDS,
//                  sorted there by tile (stable, two digit passes, nothing leaves the CU), and every tile's run
//                  is appended at the tile's cursor (tile start + chunks in front + what the block wrote so far).
// Every instance is written exactly once, to its final place, in runs of consecutive addresses.
#pragma once

namespace instances {

#ifndef INPC_INST_CHUNKS
#define INPC_INST_CHUNKS 1024
#endif
constexpr int kChunks = INPC_INST_CHUNKS;  // contiguous chunks of the depth-ordered points, one block each
#ifndef INPC_EMIT_THREADS
#define INPC_EMIT_THREADS 512
#endif
constexpr int kEmitThreads = INPC_EMIT_THREADS;
#ifndef INPC_EMIT_ITEMS
#define INPC_EMIT_ITEMS 4
#endif
constexpr int kEmitItems = INPC_EMIT_ITEMS;                          // points per thread and sub-chunk
constexpr int kEmitPoints = kEmitThreads * kEmitItems;  // points per sub-chunk
#ifndef INPC_EMIT_STAGE
#define INPC_EMIT_STAGE 3072
#endif
constexpr int kStage = INPC_EMIT_STAGE;                 // instances sorted in LDS at a time
constexpr int kStageItems = kStage / kEmitThreads;      // per thread
constexpr int kSortWaves = kEmitThreads / kWave;
constexpr int kDigits = 256;                            // the LDS digit passes take at most 8 bits (16-bit tile keys)
static_assert(kEmitThreads >= kDigits, "thread d owns digit d in the LDS digit passes");
static_assert(kStage % kEmitThreads == 0 && kEmitItems % 4 == 0, "whole rows per thread, 16-byte loads of the sort values");
constexpr uint32_t kNoPoint = 0xFFFFFFFFu;

__host__ __device__ inline uint32_t chunk_size(uint32_t n) {
    const uint32_t per = (n + kChunks - 1) / kChunks;
    return (per + 255u) / 256u * 256u;  // a multiple of 16 keeps the 64-byte loads of k_inst_emit aligned
}

// Tile of the first instance of the point behind sort value `val` (record slot << 2 | span bits).
__device__ __forceinline__ uint32_t first_tile(uint32_t val, const uint32_t* __restrict__ bin_start,
                                               const uint16_t* __restrict__ coarse) {
    const uint32_t slot = val >> 2, b = slot >> kCoarseShift;
    return tile_of_slot(bin_start, coarse[b], (uint32_t)coarse[b + 1] + 1u, slot);
}

__global__ void __launch_bounds__(kBinThreads)
    k_inst_count(const uint32_t* __restrict__ depth_order, const uint32_t* __restrict__ bin_start,
                 const uint16_t* __restrict__ coarse, const uint32_t* __restrict__ counters, uint32_t* __restrict__ table,
                 uint32_t n_points, uint32_t gw, uint32_t n_tiles) {
    extern __shared__ uint32_t s_count[];
    for (uint32_t t = threadIdx.x; t < n_tiles; t += kBinThreads) s_count[t] = 0u;
    __syncthreads();
    const uint32_t n_visible = min(counters[kCntVisible], n_points);
    const uint32_t chunk = chunk_size(n_points);
    const uint32_t begin = min(blockIdx.x * chunk, n_visible), end = min(begin + chunk, n_visible);
    constexpr int kUnroll = 4;   // points per thread and round: the dependent loads of the tile search overlap
    for (uint32_t base = begin; base < end; base += kUnroll * kBinThreads) {
        uint32_t val[kUnroll], lo[kUnroll], hi[kUnroll];
        bool live[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const uint32_t i = base + u * kBinThreads + threadIdx.x;
            live[u] = i < end;
            val[u] = depth_order[live[u] ? i : begin];
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const uint32_t b = (val[u] >> 2) >> kCoarseShift;
            lo[u] = coarse[b];
            hi[u] = (uint32_t)coarse[b + 1] + 1u;
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            if (!live[u]) continue;
            const uint32_t tile0 = tile_of_slot(bin_start, lo[u], hi[u], val[u] >> 2);
            const uint32_t nx = (val[u] & 1u) + 1u, ny = ((val[u] >> 1) & 1u) + 1u;
            for (uint32_t dy = 0; dy < ny; ++dy)
                for (uint32_t dx = 0; dx < nx; ++dx) atomicAdd(&s_count[tile0 + dy * gw + dx], 1u);
        }
    }
    __syncthreads();
    uint32_t* row = table + (size_t)blockIdx.x * n_tiles;
    for (uint32_t t = threadIdx.x; t < n_tiles; t += kBinThreads) row[t] = s_count[t];
}

// ranges[t] = [start[t], start[t + 1]); tiles without instances keep (0, 0) as in the reference (forward.cu:52).
__global__ void __launch_bounds__(kBlock) k_ranges_from_starts(const uint32_t* __restrict__ start, uint2* __restrict__ ranges,
                                                               uint32_t n_tiles) {
    const uint32_t t = blockIdx.x * kBlock + threadIdx.x;
    if (t >= n_tiles) return;
    const uint32_t b = start[t], e = start[t + 1];
    ranges[t] = b == e ? make_uint2(0u, 0u) : make_uint2(b, e);
}

// One stable digit pass over s_key / s_val [0, n) in LDS. Element (wave w, row r, lane l) = w * kStageItems * 64 +
// r * 64 + l, so a wave's elements are consecutive and the per-wave ranking by ballots is stable.
__device__ __forceinline__ void lds_digit_pass(uint16_t* s_key, uint32_t* s_val, uint32_t n, int shift, int bits,
                                               uint32_t (*s_cnt)[kDigits], uint32_t* s_base) {
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t digit_mask = (1u << bits) - 1u;
    for (uint32_t i = tid; i < kSortWaves * kDigits; i += kEmitThreads) (&s_cnt[0][0])[i] = 0u;
    uint32_t key[kStageItems], val[kStageItems], rank[kStageItems];
    uint32_t valid_bits = 0;
#pragma unroll
    for (int r = 0; r < kStageItems; ++r) {
        const uint32_t idx = wave * (kStageItems * kWave) + r * kWave + lane;
        key[r] = 0u;
        val[r] = 0u;
        if (idx < n) {
            key[r] = s_key[idx];
            val[r] = s_val[idx];
            valid_bits |= 1u << r;
        }
    }
    __syncthreads();  // counters are zero, every element is in registers
#pragma unroll
    for (int r = 0; r < kStageItems; ++r) {
        const bool valid = (valid_bits >> r) & 1u;
        const uint32_t d = (key[r] >> shift) & digit_mask;
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
    // thread d: offsets of the waves inside digit d's run, then the start of the run
    uint32_t total = 0;
    if (tid <= digit_mask) {
#pragma unroll
        for (int w = 0; w < kSortWaves; ++w) {
            const uint32_t c = s_cnt[w][tid];
            s_cnt[w][tid] = total;
            total += c;
        }
    }
    uint32_t incl = total;
#pragma unroll
    for (int s = 1; s < 64; s <<= 1) {
        const uint32_t up = __shfl_up(incl, s, 64);
        if (lane >= (uint32_t)s) incl += up;
    }
    __shared__ uint32_t s_wave_total[kSortWaves];
    if (lane == 63u) s_wave_total[wave] = incl;
    __syncthreads();
    uint32_t wave_off = 0;
#pragma unroll
    for (int w = 0; w < kSortWaves; ++w)
        if ((uint32_t)w < wave) wave_off += s_wave_total[w];
    if (tid < (uint32_t)kDigits) s_base[tid] = wave_off + incl - total;   // one entry per digit, not per thread
    __syncthreads();
#pragma unroll
    for (int r = 0; r < kStageItems; ++r) {
        if ((valid_bits >> r) & 1u) {
            const uint32_t d = (key[r] >> shift) & digit_mask;
            const uint32_t dst = s_base[d] + s_cnt[wave][d] + rank[r];
            s_key[dst] = (uint16_t)key[r];
            s_val[dst] = val[r];
        }
    }
    __syncthreads();
}

__global__ void __launch_bounds__(kEmitThreads)
    k_inst_emit(const uint32_t* __restrict__ depth_order, const uint32_t* __restrict__ bin_start,
                const uint16_t* __restrict__ coarse, const uint32_t* __restrict__ counters,
                const uint32_t* __restrict__ table, const uint32_t* __restrict__ inst_start,
                uint16_t* __restrict__ inst_keys, uint32_t* __restrict__ inst_slots, uint32_t n_points, uint32_t gw,
                uint32_t n_tiles, int key_bits) {
    extern __shared__ uint32_t s_cursor[];  // n_tiles: where the next instance of every tile goes
    __shared__ uint16_t s_key[kStage];
    __shared__ uint32_t s_val[kStage];
    __shared__ uint16_t s_first[kStage];    // index of the first element of the element's tile run
    __shared__ uint32_t s_cnt[kSortWaves][kDigits];
    __shared__ uint32_t s_base[kDigits];
    __shared__ uint32_t s_scan[kSortWaves];
    __shared__ int s_carry[kSortWaves];
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    {
        const uint32_t* row = table + (size_t)blockIdx.x * n_tiles;
        for (uint32_t t = tid; t < n_tiles; t += kEmitThreads) s_cursor[t] = inst_start[t] + row[t];
    }
    __syncthreads();
    const uint32_t n_visible = min(counters[kCntVisible], n_points);
    const uint32_t chunk = chunk_size(n_points);
    const uint32_t begin = min(blockIdx.x * chunk, n_visible), end = min(begin + chunk, n_visible);
    const int bits_low = (key_bits + 1) / 2, bits_high = key_bits - bits_low;

    for (uint32_t sub = begin; sub < end; sub += kEmitPoints) {
        // ---- this thread's points of the sub-chunk: sort value, first tile, number of instances
        const uint32_t first = sub + tid * kEmitItems;
        uint32_t val[kEmitItems];
        if (first + kEmitItems <= end) {
            const uint4* src = (const uint4*)(depth_order + first);  // sub and first are multiples of 16
#pragma unroll
            for (int q = 0; q < kEmitItems / 4; ++q) {
                const uint4 v = src[q];
                val[4 * q] = v.x;
                val[4 * q + 1] = v.y;
                val[4 * q + 2] = v.z;
                val[4 * q + 3] = v.w;
            }
        } else {
#pragma unroll
            for (int j = 0; j < kEmitItems; ++j) val[j] = first + j < end ? depth_order[first + j] : kNoPoint;
        }
        uint16_t tile0[kEmitItems];
        uint32_t mine = 0;
#pragma unroll
        for (int j = 0; j < kEmitItems; ++j) {
            tile0[j] = 0;
            if (val[j] != kNoPoint) {
                tile0[j] = (uint16_t)first_tile(val[j], bin_start, coarse);
                mine += ((val[j] & 1u) + 1u) * (((val[j] >> 1) & 1u) + 1u);
            }
        }
        // block exclusive scan of `mine`: position of the thread's first instance inside the sub-chunk
        uint32_t incl = mine;
#pragma unroll
        for (int s = 1; s < 64; s <<= 1) {
            const uint32_t up = __shfl_up(incl, s, 64);
            if (lane >= (uint32_t)s) incl += up;
        }
        if (lane == 63u) s_scan[wave] = incl;
        __syncthreads();
        uint32_t wave_off = 0, sub_total = 0;
#pragma unroll
        for (int w = 0; w < kSortWaves; ++w) {
            const uint32_t c = s_scan[w];
            if ((uint32_t)w < wave) wave_off += c;
            sub_total += c;
        }
        const uint32_t local_first = wave_off + incl - mine;

        for (uint32_t round = 0; round < sub_total; round += kStage) {
            const uint32_t n_round = min((uint32_t)kStage, sub_total - round);
            // ---- expand into LDS, in depth order (row-major over the touched tiles of a point)
            uint32_t local = local_first;
#pragma unroll
            for (int j = 0; j < kEmitItems; ++j) {
                if (val[j] == kNoPoint) continue;
                const uint32_t slot = val[j] >> 2, nx = (val[j] & 1u) + 1u, ny = ((val[j] >> 1) & 1u) + 1u;
                for (uint32_t dy = 0; dy < ny; ++dy)
                    for (uint32_t dx = 0; dx < nx; ++dx) {
                        const uint32_t at = local - round;  // wraps below the round: fails the test as well
                        if (at < (uint32_t)kStage) {
                            s_key[at] = (uint16_t)(tile0[j] + dy * gw + dx);
                            s_val[at] = slot;
                        }
                        ++local;
                    }
            }
            __syncthreads();
            // ---- stable sort by tile inside LDS
            lds_digit_pass(s_key, s_val, n_round, 0, bits_low, s_cnt, s_base);
            if (bits_high > 0) lds_digit_pass(s_key, s_val, n_round, bits_low, bits_high, s_cnt, s_base);
            // ---- start of every element's tile run: running maximum of the run heads' indices
            {
                const uint32_t e0 = tid * kStageItems;  // this thread: elements e0 .. e0 + kStageItems - 1
                int last_head = -1;
                int head_at[kStageItems];
#pragma unroll
                for (int r = 0; r < kStageItems; ++r) {
                    const uint32_t e = e0 + r;
                    head_at[r] = -1;
                    if (e < n_round && (e == 0u || s_key[e - 1] != s_key[e])) head_at[r] = (int)e;
                    last_head = max(last_head, head_at[r]);
                }
                int scan = last_head;
#pragma unroll
                for (int s = 1; s < 64; s <<= 1) {
                    const int up = __shfl_up(scan, s, 64);
                    if (lane >= (uint32_t)s) scan = max(scan, up);
                }
                if (lane == 63u) s_carry[wave] = scan;
                __syncthreads();
                int carry = __shfl_up(scan, 1, 64);
                if (lane == 0u) carry = -1;
#pragma unroll
                for (int w = 0; w < kSortWaves; ++w)
                    if ((uint32_t)w < wave) carry = max(carry, s_carry[w]);
#pragma unroll
                for (int r = 0; r < kStageItems; ++r) {
                    const uint32_t e = e0 + r;
                    carry = max(carry, head_at[r]);
                    if (e < n_round) s_first[e] = (uint16_t)carry;
                }
            }
            __syncthreads();
            // ---- append every run at its tile's cursor
            for (uint32_t e = tid; e < n_round; e += kEmitThreads) {
                const uint32_t t = s_key[e];
                const uint32_t pos = s_cursor[t] + (e - (uint32_t)s_first[e]);
                inst_keys[pos] = (uint16_t)t;
                inst_slots[pos] = s_val[e];
            }
            __syncthreads();
            for (uint32_t e = tid; e < n_round; e += kEmitThreads) {
                const uint32_t t = s_key[e];
                if (e + 1u == n_round || s_key[e + 1] != t) s_cursor[t] += e - (uint32_t)s_first[e] + 1u;  // one tail per run
            }
            __syncthreads();
        }
    }
}

}  // namespace instances
