// gfx950 device code, part of apk_kernels.hip (one translation unit, one code object): greedy pick over rows of logits.
#pragma once

// Greedy pick over rows of logits: the LAST maximum under f32::total_cmp, i.e. Rust's
// (0..n).max_by(total_cmp) of Model::forward_greedy (model/decode.rs:628-630): ties go to
// the higher index.  A row is split over `parts` workgroups; each folds its slice into a
// (key << 32 | index) word and merges it with an atomic max into best[row]; the last
// workgroup of a row (counted next to it) writes out[row] and re-arms both words.
// scratch: one 128-byte line per row (word 0: running best, word 1: arrivals), so the
// atomics of different rows never share a cache line.
// The fold costs three integer operations per logit: non-negative floats order as signed integers of their bits
// and negative ones in reverse, so a lane keeps the signed maximum and minimum of its raw tiles, picks the maximum
// if it is non-negative and the minimum otherwise (the lane's largest value under total_cmp either way), and finds
// the pick's position with one more sweep over the registers, in index order, so that the last of equal values
// wins.  (A 64-bit (key, index) compare per logit was ten operations and showed next to the stream: 8.7 us against
// 8.0 us for 64 x 151 936 logits before the merge.)
extern "C" __global__ __launch_bounds__(1024) void apk_argmax_rows(const float* logits, uint64_t n, int parts,
                                                                  unsigned long long* scratch, uint32_t* out) {
    __shared__ unsigned long long wbest[16];
    const uint32_t row = blockIdx.x / parts, part = blockIdx.x % parts;
    unsigned long long* best = scratch + (uint64_t)row * 16;
    uint32_t* done = (uint32_t*)(best + 1);
    const float* lr = logits + (uint64_t)row * n;
    unsigned long long b = 0;
    uint64_t lo, hi;
    if ((n & 3) == 0) {  // rows are 16-byte aligned: 16-byte tiles, 4 loads in flight per lane
        const uint64_t ntile = n >> 2, per = (ntile + parts - 1) / parts;
        lo = (uint64_t)part * per;
        hi = min(lo + per, ntile);
        const u32x4* lt = (const u32x4*)lr;
        for (uint64_t i0 = lo + threadIdx.x; i0 < hi; i0 += 4 * blockDim.x) {
            u32x4 t[4];
#pragma unroll
            for (int j = 0; j < 4; j++) {  // a tile past the end re-reads the lane's first tile (valid logits of this part)
                const uint64_t i = i0 + (uint64_t)j * blockDim.x;
                t[j] = __builtin_nontemporal_load(lt + (i < hi ? i : i0));
            }
            int32_t imax = INT32_MIN, imin = INT32_MAX;
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const int32_t r = (int32_t)t[j][e];
                    imax = max(imax, r);
                    imin = min(imin, r);
                }
            const int32_t pick = imax >= 0 ? imax : imin;
            uint32_t slot = 0;
#pragma unroll
            for (int j = 0; j < 4; j++) {  // a re-read tile repeats an earlier index: it must not shadow a later one
                const bool live = i0 + (uint64_t)j * blockDim.x < hi;
#pragma unroll
                for (int e = 0; e < 4; e++) slot = live && (int32_t)t[j][e] == pick ? (uint32_t)(4 * j + e) : slot;
            }
            const uint64_t idx = 4 * (i0 + (uint64_t)(slot >> 2) * blockDim.x) + (slot & 3);
            const unsigned long long cand = ((unsigned long long)total_order_key(__builtin_bit_cast(float, pick)) << 32) | idx;
            b = cand > b ? cand : b;  // equal keys: the higher index is the larger word
        }
    } else {
        const uint64_t per = (n + parts - 1) / parts;
        lo = (uint64_t)part * per;
        hi = min(lo + per, n);
        for (uint64_t i = lo + threadIdx.x; i < hi; i += blockDim.x) {
            const unsigned long long cand = ((unsigned long long)total_order_key(lr[i]) << 32) | (unsigned long long)i;
            b = cand > b ? cand : b;
        }
    }
    b = wave_max_u64(b);
    if ((threadIdx.x & 63) == 0) wbest[threadIdx.x >> 6] = b;
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < (int)(blockDim.x >> 6); w++) b = wbest[w] > b ? wbest[w] : b;
        // No device-scope fence (it would write back the whole L2): the arrival count is made
        // data-dependent on the returned value of the max, so the max is performed first; the
        // last arrival therefore sees every max of the row.
        const unsigned long long prev = atomicMax(best, b);
        uint32_t inc = 1u;
        asm volatile("" : "+v"(inc) : "v"((uint32_t)prev));
        if (atomicAdd(done, inc) == (uint32_t)parts - 1u) {  // last workgroup of the row
            const unsigned long long win = atomicExch(best, 0ull);
            out[row] = (uint32_t)(win & 0xffffffffull);
            atomicExch(done, 0u);
        }
    }
}

// Zero fill of 8-byte words (the scratch lines of apk_argmax_rows_noalloc ahead of its launch: a fill kernel, not a
// memset, so that the call can sit inside a recording).
extern "C" __global__ __launch_bounds__(256) void apk_zero_u64(unsigned long long* p, uint64_t n) {
    const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0ull;
}
