// tilesort.hpp — per-tile depth sort of the binned instances, inside LDS. Included by raster.hip.
//
// The reference sorts all drawn points by depth with one device-wide radix sort, expands them into
// (tile, point) instances and sorts those by tile with a second, stable device-wide sort
// (B/rasterization/src/bilinear/forward.cu:91-141): the result is, for every tile, its instances ordered by
// (depth bits, compaction order). With points compacted in ascending point index that is the order
// (tile, depth bits, point index), and it can be had without any device-wide sort: the preprocess pass drops a
// (depth key, point index) pair per instance into the bin of its tile, and one block per tile sorts its bin.
//
//   elements   u64 = depth key << 32 | point index: the order wanted is plain ascending u64 order
//   in LDS     least-significant-digit radix sort, 4-bit digits, over the key bits. A thread owns kPer
//              consecutive elements and counts their digits in sixteen 4-bit fields of one 64-bit register; the
//              16 x kThreads counts are scanned in digit-major order, which is a stable ranking. Digits
//              that are the same for all elements of the tile are skipped (the depths of one tile mostly share
//              their leading bits).
//   ties       elements with equal keys come out in the order they were binned, which is arbitrary: a few
//              ties are put right in place (rank by point index inside the run of equal keys); a tile with
//              many is sorted again over all 64 bits.
//   big tiles  more elements than fit LDS: runs of kCap elements are sorted as above and written back, then
//              merged pairwise through global memory (rank of an element = its place in its own run + the
//              number of smaller elements in the partner run, by binary search on the full 64 bits).
#pragma once

namespace tilesort {

constexpr int kThreads = 512;
constexpr int kWaves = kThreads / kWave;
constexpr int kMaxPer = 7;                  // elements per thread: 1, 3, 5 or 7 (odd: conflict-free LDS rows)
constexpr int kCap = kThreads * kMaxPer;    // elements sorted in LDS at a time
constexpr int kDigits = 16;
constexpr uint64_t kPad = ~0ull;            // sorts behind every element
constexpr uint32_t kFewTies = 16;           // threads with tied elements up to which ties are fixed in place

struct Shared {
    uint64_t buf[2][kCap];
    alignas(16) uint16_t count[kDigits * kThreads];   // [digit][thread], scanned in this order
    uint32_t wave_sum[kWaves];
    uint32_t bits_or[2], bits_and[2];                 // over the tile's elements: [0] point index, [1] key
};
constexpr size_t kSharedBytes = sizeof(Shared);

__device__ __forceinline__ uint32_t hi32(uint64_t v) { return (uint32_t)(v >> 32); }
__device__ __forceinline__ uint32_t lo32(uint64_t v) { return (uint32_t)v; }

__device__ __forceinline__ uint32_t wave_inclusive_u32(uint32_t v) {
    v += blend::dpp_take<blend::kDppRowShr1, 0xf>(0u, v);
    v += blend::dpp_take<blend::kDppRowShr2, 0xf>(0u, v);
    v += blend::dpp_take<blend::kDppRowShr4, 0xf>(0u, v);
    v += blend::dpp_take<blend::kDppRowShr8, 0xf>(0u, v);
    v += blend::dpp_take<blend::kDppRowBcast15, 0xa>(0u, v);
    v += blend::dpp_take<blend::kDppRowBcast31, 0xc>(0u, v);
    return v;
}

// One stable counting pass on the 4-bit digit at bit `shift`, from sh.buf[src] to sh.buf[1 - src]. All
// kThreads threads call it; kPer * kThreads elements (padding included) take part. Ends with a barrier.
template <int kPer>
__device__ __forceinline__ void digit_pass(Shared& sh, int src, int shift) {
    const uint32_t t = threadIdx.x, lane = t & 63u, wave = t >> 6;
    const uint64_t* from = sh.buf[src];
    uint64_t* to = sh.buf[1 - src];
    uint64_t v[kPer];
    uint64_t fields = 0ull;   // sixteen 4-bit counters: kPer <= 15 elements per thread cannot overflow one
#pragma unroll
    for (int e = 0; e < kPer; ++e) {
        v[e] = from[t * kPer + e];
        fields += 1ull << (4u * (uint32_t)((v[e] >> shift) & 15ull));
    }
#pragma unroll
    for (int d = 0; d < kDigits; ++d) sh.count[d * kThreads + t] = (uint16_t)((fields >> (4 * d)) & 15ull);
    __syncthreads();
    // exclusive scan of the 16 * kThreads counts in storage order; thread t owns entries [16 t, 16 t + 16)
    uint4* mine = (uint4*)(sh.count + 16u * t);
    uint4 a = mine[0], b = mine[1];
    uint32_t w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};   // two counts per word
    uint32_t sum = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) sum += (w[i] & 0xFFFFu) + (w[i] >> 16);
    const uint32_t incl = wave_inclusive_u32(sum);
    if (lane == 63u) sh.wave_sum[wave] = incl;
    __syncthreads();
    uint32_t run = incl - sum;
#pragma unroll
    for (int k = 0; k < kWaves; ++k) run += (uint32_t)k < wave ? sh.wave_sum[k] : 0u;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const uint32_t c0 = w[i] & 0xFFFFu, c1 = w[i] >> 16;
        w[i] = run | ((run + c0) << 16);
        run += c0 + c1;
    }
    mine[0] = make_uint4(w[0], w[1], w[2], w[3]);
    mine[1] = make_uint4(w[4], w[5], w[6], w[7]);
    __syncthreads();
    uint64_t seen = 0ull;     // how many of this thread's earlier elements had the same digit
#pragma unroll
    for (int e = 0; e < kPer; ++e) {
        const uint32_t d = (uint32_t)((v[e] >> shift) & 15ull);
        const uint32_t at = (uint32_t)sh.count[d * kThreads + t] + (uint32_t)((seen >> (4u * d)) & 15ull);
        seen += 1ull << (4u * d);
        to[at] = v[e];
    }
    __syncthreads();
}

// Sorts the n <= kPer * kThreads elements in sh.buf[0] ascending as u64 (the slots behind them hold kPad);
// returns the buffer that holds the result. All threads call it.
template <int kPer>
__device__ int sort_run(Shared& sh, uint32_t n, int key_bits) {
    const uint32_t t = threadIdx.x, lane = t & 63u;
    // bits that differ between the elements
    {
        uint32_t or_lo = 0u, or_hi = 0u, and_lo = ~0u, and_hi = ~0u;
#pragma unroll
        for (int e = 0; e < kPer; ++e) {
            const uint32_t p = t * kPer + e;
            if (p < n) {
                const uint64_t v = sh.buf[0][p];
                or_lo |= lo32(v);
                or_hi |= hi32(v);
                and_lo &= lo32(v);
                and_hi &= hi32(v);
            }
        }
        for (int s = 32; s > 0; s >>= 1) {
            or_lo |= __shfl_xor(or_lo, s, 64);
            or_hi |= __shfl_xor(or_hi, s, 64);
            and_lo &= __shfl_xor(and_lo, s, 64);
            and_hi &= __shfl_xor(and_hi, s, 64);
        }
        if (t < 2) {
            sh.bits_or[t] = 0u;
            sh.bits_and[t] = ~0u;
        }
        __syncthreads();
        if (lane == 0u) {
            atomicOr(&sh.bits_or[0], or_lo);
            atomicOr(&sh.bits_or[1], or_hi);
            atomicAnd(&sh.bits_and[0], and_lo);
            atomicAnd(&sh.bits_and[1], and_hi);
        }
        __syncthreads();
    }
    const uint32_t vary_lo = sh.bits_or[0] ^ sh.bits_and[0], vary_hi = sh.bits_or[1] ^ sh.bits_and[1];
    int cur = 0;
    auto key_passes = [&]() {
        for (int shift = 0; shift < key_bits; shift += 4)
            if ((vary_hi >> shift) & 15u) {
                digit_pass<kPer>(sh, cur, 32 + shift);
                cur ^= 1;
            }
    };
    key_passes();
    // elements with equal keys stand in the order they were binned; the order wanted is by point index
    bool tied[kPer];
    bool any = false;
    {
        const uint64_t* b = sh.buf[cur];
#pragma unroll
        for (int e = 0; e < kPer; ++e) {
            const uint32_t p = t * kPer + e;
            tied[e] = false;
            if (p < n) {
                const uint32_t key = hi32(b[p]);
                tied[e] = (p > 0u && hi32(b[p - 1u]) == key) || (p + 1u < n && hi32(b[p + 1u]) == key);
            }
            any = any || tied[e];
        }
    }
    const uint32_t threads_tied = (uint32_t)__syncthreads_count(any);
    if (threads_tied == 0u) return cur;
    if (threads_tied <= kFewTies) {
        // few ties (runs of at most kFewTies * kPer elements): every tied element finds its run and its rank in it
        const uint64_t* b = sh.buf[cur];
        uint64_t* to = sh.buf[cur ^ 1];
#pragma unroll
        for (int e = 0; e < kPer; ++e) {
            const uint32_t p = t * kPer + e;
            const uint64_t v = b[p];
            uint32_t at = p;
            if (tied[e]) {
                const uint32_t key = hi32(v);
                uint32_t first = p, last = p + 1u;
                while (first > 0u && hi32(b[first - 1u]) == key) --first;
                while (last < n && hi32(b[last]) == key) ++last;
                uint32_t smaller = 0;
                for (uint32_t q = first; q < last; ++q) smaller += lo32(b[q]) < lo32(v) ? 1u : 0u;
                at = first + smaller;
            }
            to[at] = v;
        }
        __syncthreads();
        return cur ^ 1;
    }
    // many ties: sort over all 64 bits, least significant digit first
    for (int shift = 0; shift < 32; shift += 4)
        if ((vary_lo >> shift) & 15u) {
            digit_pass<kPer>(sh, cur, shift);
            cur ^= 1;
        }
    key_passes();
    return cur;
}

// Loads `n` elements from `src` into sh.buf[0], pads, sorts; returns the buffer holding the result.
__device__ __forceinline__ int load_and_sort(Shared& sh, const uint64_t* __restrict__ src, uint32_t n, int key_bits) {
    const uint32_t t = threadIdx.x;
    const uint32_t per = (n + kThreads - 1u) / kThreads;            // 1 .. kMaxPer
    const uint32_t padded = (per <= 1u ? 1u : per <= 3u ? 3u : per <= 5u ? 5u : 7u) * kThreads;
    for (uint32_t p = t; p < padded; p += kThreads) sh.buf[0][p] = p < n ? src[p] : kPad;
    __syncthreads();
    if (per <= 1u) return sort_run<1>(sh, n, key_bits);
    if (per <= 3u) return sort_run<3>(sh, n, key_bits);
    if (per <= 5u) return sort_run<5>(sh, n, key_bits);
    return sort_run<7>(sh, n, key_bits);
}

// One block per tile, longest bins first. pairs[begin .. end) of a tile are its elements in no particular order;
// afterwards points[begin .. end) holds their point indices in ascending element order. `pairs` and `scratch`
// (same size) are clobbered for tiles with more than kCap elements.
__global__ void __launch_bounds__(kThreads)
    k_tile_sort(const uint2* __restrict__ ranges, const uint32_t* __restrict__ tile_order, uint64_t* pairs,
                uint64_t* scratch, uint32_t* __restrict__ points, int key_bits) {
    extern __shared__ __align__(16) unsigned char s_raw[];
    Shared& sh = *reinterpret_cast<Shared*>(s_raw);
    const uint32_t t = threadIdx.x;
    const uint2 range = ranges[tile_order[blockIdx.x]];
    const uint32_t begin = range.x, n = range.y - range.x;
    if (n == 0u) return;
    if (n <= (uint32_t)kCap) {
        const int res = load_and_sort(sh, pairs + begin, n, key_bits);
        for (uint32_t p = t; p < n; p += kThreads) points[begin + p] = lo32(sh.buf[res][p]);
        return;
    }
    // runs of kCap elements, each sorted in LDS and written back in place
    for (uint32_t first = 0; first < n; first += kCap) {
        const uint32_t len = min((uint32_t)kCap, n - first);
        const int res = load_and_sort(sh, pairs + begin + first, len, key_bits);
        for (uint32_t p = t; p < len; p += kThreads) pairs[begin + first + p] = sh.buf[res][p];
        __syncthreads();
    }
    // pairwise merges; the global stores of a level are visible to the whole block behind the barrier
    uint64_t* from = pairs + begin;
    uint64_t* to = scratch + begin;
    for (uint32_t width = kCap; width < n; width <<= 1) {
        constexpr int kAhead = 4;   // independent searches per thread
        for (uint32_t base = 0; base < n; base += kAhead * kThreads) {
            uint64_t v[kAhead];
            uint32_t lo[kAhead], hi[kAhead];   // the part of the partner run still searched
#pragma unroll
            for (int u = 0; u < kAhead; ++u) {
                const uint32_t p = base + u * kThreads + t;
                lo[u] = hi[u] = 0u;
                v[u] = 0ull;
                if (p < n) {
                    v[u] = from[p];
                    const uint32_t run = p / width, left = (run & ~1u) * width;
                    const uint32_t mid = min(left + width, n), right_end = min(left + 2u * width, n);
                    lo[u] = (run & 1u) ? left : mid;
                    hi[u] = (run & 1u) ? mid : right_end;
                }
            }
            bool busy = true;
            while (busy) {
                busy = false;
#pragma unroll
                for (int u = 0; u < kAhead; ++u)
                    if (lo[u] < hi[u]) {
                        const uint32_t mid = (lo[u] + hi[u]) >> 1;
                        if (from[mid] < v[u]) lo[u] = mid + 1u;
                        else hi[u] = mid;
                        busy = busy || lo[u] < hi[u];
                    }
            }
#pragma unroll
            for (int u = 0; u < kAhead; ++u) {
                const uint32_t p = base + u * kThreads + t;
                if (p < n) {
                    const uint32_t run = p / width, left = (run & ~1u) * width;
                    const uint32_t mid = min(left + width, n);
                    // lo[u]: first element of the partner run that is not smaller than v
                    const uint32_t smaller = (run & 1u) ? lo[u] - left : lo[u] - mid;
                    const uint32_t own = (run & 1u) ? p - mid : p - left;
                    to[left + own + smaller] = v[u];
                }
            }
        }
        __syncthreads();
        uint64_t* swap = from;
        from = to;
        to = swap;
    }
    for (uint32_t p = t; p < n; p += kThreads) points[begin + p] = lo32(from[p]);
}

}  // namespace tilesort
