// A stable least-significant-digit radix sort of (32-bit key, 32-bit value) pairs, eight bits a pass: what index_add_
// orders its sources with (equal destinations keep ascending source order, so the sums are added as the reference's
// walk adds them).  A pass is three launches: per-block digit counts, one exclusive scan over (digit, block) - which
// the scatter does itself when the blocks are few - and a scatter in which every block walks its chunk again in 256-element groups - inside a group an element's place among
// the elements of its digit is a count of the lower lanes of its wave that hold the same digit (eight ballots) plus
// the counts of the waves before it, and a running count per digit carries from group to group.
#pragma once
#include <cstddef>
#include <cstdint>

#include "mxh.hpp"

namespace mxh {

constexpr int RS_THREADS = 256;
constexpr int RS_BINS = 256;
constexpr uint32_t RS_SCAN_IN_SCATTER = 64;   // up to this many blocks the scatter scans the counts itself
constexpr uint32_t RS_MAX_BLOCKS = 2048;       // (the scan is one work-group over RS_BINS * blocks counts)

struct RsPlan {
    uint32_t blocks, chunk;      // every block sorts `chunk` consecutive elements (a multiple of RS_THREADS)
};
inline RsPlan rs_plan(size_t n) {
    RsPlan p;
    // (measured on an embedding gradient's sort: for 65536 pairs chunks of 1024 are best - 64 blocks, which still scan
    // the counts themselves -, 8192-16384 for 2^20; smaller chunks scatter a block's elements over too many short runs)
    size_t chunk = 1024;
    while (chunk < 4096 && (n + chunk - 1) / chunk > RS_SCAN_IN_SCATTER) chunk *= 2;
    if (n >= (1u << 19)) chunk = 8192;
    while ((n + chunk - 1) / chunk > RS_MAX_BLOCKS) chunk *= 2;
    p.chunk = (uint32_t)chunk;
    p.blocks = (uint32_t)((n + chunk - 1) / chunk);
    return p;
}
// bytes of workspace a sort of n pairs needs (the counts of one pass)
inline size_t rs_workspace_bytes(size_t n) { return (size_t)RS_BINS * rs_plan(n).blocks * sizeof(uint32_t); }

__global__ __launch_bounds__(RS_THREADS) void rs_count_kernel(const uint32_t* __restrict__ keys, uint32_t n, uint32_t shift, uint32_t chunk,
                                                              uint32_t blocks, uint32_t* __restrict__ counts) {
    __shared__ uint32_t bins[RS_BINS];
    bins[threadIdx.x] = 0;
    __syncthreads();
    const uint32_t beg = blockIdx.x * chunk, end = n - beg < chunk ? n : beg + chunk;
    for (uint32_t i = beg + threadIdx.x; i < end; i += RS_THREADS) atomicAdd(&bins[(keys[i] >> shift) & (RS_BINS - 1)], 1u);
    __syncthreads();
    counts[(size_t)threadIdx.x * blocks + blockIdx.x] = bins[threadIdx.x];      // digit-major: the order the scan walks
}

// counts[0 .. total) -> the sum of everything before each entry, by one work-group
constexpr int RS_SCAN_THREADS = 1024;
__global__ __launch_bounds__(RS_SCAN_THREADS) void rs_scan_kernel(uint32_t* __restrict__ counts, uint32_t total) {
    __shared__ uint32_t part[RS_SCAN_THREADS];
    const uint32_t per = (total + RS_SCAN_THREADS - 1) / RS_SCAN_THREADS;
    const uint32_t beg = threadIdx.x * per < total ? threadIdx.x * per : total, end = total - beg < per ? total : beg + per;
    uint32_t sum = 0;
    for (uint32_t i = beg; i < end; ++i) sum += counts[i];
    part[threadIdx.x] = sum;
    __syncthreads();
    // the threads' sums to their exclusive prefixes: thread 0 alone (1024 additions)
    if (threadIdx.x == 0) {
        uint32_t run = 0;
        for (int t = 0; t < RS_SCAN_THREADS; ++t) {
            const uint32_t mine = part[t];
            part[t] = run;
            run += mine;
        }
    }
    __syncthreads();
    uint32_t run = part[threadIdx.x];
    for (uint32_t i = beg; i < end; ++i) {
        const uint32_t mine = counts[i];
        counts[i] = run;
        run += mine;
    }
}

__global__ __launch_bounds__(RS_THREADS) void rs_scatter_kernel(const uint32_t* __restrict__ keys_in, const uint32_t* __restrict__ vals_in,
                                                                uint32_t* __restrict__ keys_out, uint32_t* __restrict__ vals_out, uint32_t n,
                                                                uint32_t shift, uint32_t chunk, uint32_t blocks,
                                                                const uint32_t* __restrict__ offsets, bool scanned) {
    constexpr int WAVES = RS_THREADS / WAVE;
    __shared__ uint32_t next[RS_BINS];                 // where the block's next element of each digit goes
    __shared__ uint32_t wave_count[WAVES][RS_BINS];    // a group's elements per wave and digit, then their first places
    const unsigned tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;
    if (scanned) {
        next[tid] = offsets[(size_t)tid * blocks + blockIdx.x];
    } else {
        // few blocks: `offsets` still holds the counts, and every block works out its own places from them (digit tid:
        // the elements of lower digits anywhere, plus this digit's in the blocks before) - one launch less per pass
        uint32_t before = 0, all = 0;
        for (uint32_t b = 0; b < blocks; ++b) {
            const uint32_t c = offsets[(size_t)tid * blocks + b];
            before += b < blockIdx.x ? c : 0u;
            all += c;
        }
        uint32_t* scan = &wave_count[0][0];            // (free until the first group)
        scan[tid] = all;
        __syncthreads();
        for (int d = 1; d < RS_BINS; d *= 2) {          // inclusive prefix over the digits
            const uint32_t add = tid >= (unsigned)d ? scan[tid - d] : 0u;
            __syncthreads();
            scan[tid] += add;
            __syncthreads();
        }
        next[tid] = scan[tid] - all + before;
        __syncthreads();
    }
    const uint32_t beg = blockIdx.x * chunk, end = n - beg < chunk ? n : beg + chunk;
    for (uint32_t group = beg; group < end; group += RS_THREADS) {
#pragma unroll
        for (int w = 0; w < WAVES; ++w) wave_count[w][tid] = 0;
        __syncthreads();
        const uint32_t i = group + tid;
        const bool valid = i < end;
        const uint32_t key = valid ? keys_in[i] : 0u;
        const uint32_t digit = (key >> shift) & (RS_BINS - 1);
        // the lanes of this wave that hold the same digit
        unsigned long long peers = __ballot(valid);
#pragma unroll
        for (int b = 0; b < 8; ++b) {
            const unsigned long long has = __ballot(valid && ((digit >> b) & 1u));
            peers &= ((digit >> b) & 1u) ? has : ~has;
        }
        const uint32_t before = (uint32_t)__popcll(peers & ((1ull << lane) - 1ull));
        if (valid && before == 0) wave_count[wave][digit] = (uint32_t)__popcll(peers);
        __syncthreads();
        {
            // digit `tid`: the waves' counts to the first place of each wave's elements, and the running place moves on
            uint32_t run = next[tid];
#pragma unroll
            for (int w = 0; w < WAVES; ++w) {
                const uint32_t mine = wave_count[w][tid];
                wave_count[w][tid] = run;
                run += mine;
            }
            next[tid] = run;
        }
        __syncthreads();
        if (valid) {
            const uint32_t at = wave_count[wave][digit] + before;
            keys_out[at] = key;
            vals_out[at] = vals_in[i];
        }
        __syncthreads();
    }
}

// Sorts n pairs by the low `bits` bits of their keys.  The two buffer pairs are used in turn; returns true when the
// result is in (keys_b, vals_b), false when it is in (keys_a, vals_a).  `counts`: rs_workspace_bytes(n) bytes.
inline bool radix_sort_pairs_u32(uint32_t* keys_a, uint32_t* vals_a, uint32_t* keys_b, uint32_t* vals_b, size_t n, unsigned bits, uint32_t* counts,
                                 hipStream_t s) {
    const RsPlan p = rs_plan(n);
    bool in_b = false;
    for (unsigned shift = 0; shift < bits; shift += 8) {
        const uint32_t *ki = in_b ? keys_b : keys_a, *vi = in_b ? vals_b : vals_a;
        uint32_t *ko = in_b ? keys_a : keys_b, *vo = in_b ? vals_a : vals_b;
        hipLaunchKernelGGL(rs_count_kernel, dim3(p.blocks), dim3(RS_THREADS), 0, s, ki, (uint32_t)n, shift, p.chunk, p.blocks, counts);
        const bool scan_launch = p.blocks > RS_SCAN_IN_SCATTER;
        if (scan_launch) hipLaunchKernelGGL(rs_scan_kernel, dim3(1), dim3(RS_SCAN_THREADS), 0, s, counts, (uint32_t)(RS_BINS * p.blocks));
        hipLaunchKernelGGL(rs_scatter_kernel, dim3(p.blocks), dim3(RS_THREADS), 0, s, ki, vi, ko, vo, (uint32_t)n, shift, p.chunk, p.blocks, counts,
                           scan_launch);
        in_b = !in_b;
    }
    return in_b;
}

}  // namespace mxh
