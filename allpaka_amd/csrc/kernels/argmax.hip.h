// gfx950 device code, part of apk_kernels.hip (one translation unit, one code object): greedy pick over rows of logits.
#pragma once

// Greedy pick over rows of logits: the LAST maximum under f32::total_cmp, i.e. Rust's
// (0..n).max_by(total_cmp) of Model::forward_greedy (model/decode.rs:628-630): ties go to
// the higher index.  A row is split over `parts` workgroups; each folds its slice into a
// (key << 32 | index) word and merges it with an atomic max into best[row]; the last
// workgroup of a row (counted next to it) writes out[row] and re-arms both words.
// scratch: one 128-byte line per row (word 0: running best, word 1: arrivals), so the
// atomics of different rows never share a cache line.
extern "C" __global__ __launch_bounds__(256) void apk_argmax_rows(const float* logits, uint64_t n, int parts,
                                                                 unsigned long long* scratch, uint32_t* out) {
    __shared__ unsigned long long wbest[4];
    const uint32_t row = blockIdx.x / parts, part = blockIdx.x % parts;
    unsigned long long* best = scratch + (uint64_t)row * 16;
    uint32_t* done = (uint32_t*)(best + 1);
    const float* lr = logits + (uint64_t)row * n;
    unsigned long long b = 0;
    auto fold = [&](float v, uint64_t i) {
        const unsigned long long cand = ((unsigned long long)total_order_key(v) << 32) | (unsigned long long)i;
        b = cand > b ? cand : b;  // equal keys: the higher index is the larger word
    };
    uint64_t lo, hi;
    if ((n & 3) == 0) {  // rows are 16-byte aligned: 16-byte tiles, 4 loads in flight per lane
        const uint64_t ntile = n >> 2, per = (ntile + parts - 1) / parts;
        lo = (uint64_t)part * per;
        hi = min(lo + per, ntile);
        const f32x4* lt = (const f32x4*)lr;
        for (uint64_t i0 = lo + threadIdx.x; i0 < hi; i0 += 4 * blockDim.x) {
            f32x4 t[4];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const uint64_t i = i0 + (uint64_t)j * blockDim.x;
                t[j] = __builtin_nontemporal_load(lt + (i < hi ? i : i0));
            }
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const uint64_t i = i0 + (uint64_t)j * blockDim.x;
                if (i < hi) {
                    fold(t[j].x, 4 * i);
                    fold(t[j].y, 4 * i + 1);
                    fold(t[j].z, 4 * i + 2);
                    fold(t[j].w, 4 * i + 3);
                }
            }
        }
    } else {
        const uint64_t per = (n + parts - 1) / parts;
        lo = (uint64_t)part * per;
        hi = min(lo + per, n);
        for (uint64_t i = lo + threadIdx.x; i < hi; i += blockDim.x) fold(lr[i], i);
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
