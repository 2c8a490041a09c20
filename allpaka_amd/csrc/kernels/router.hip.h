// gfx950 device code, part of apk_kernels.hip (one translation unit, one code object): MoE router: softmax / sigmoid + top-k.
#pragma once

// =========================================================================
// MoE router: per token softmax (or sigmoid) over n_expert <= 64*EPL logits, top-k
// by descending selection score with the LOWER INDEX winning ties, winners
// renormalised (moe.rs:524-594).  One wave per token; lane l holds experts
// l, l+64, l+128, ... (EPL of them).  For softmax without bias the selection runs on the
// raw logits (same order as the probabilities, no dependence on exp rounding).
// =========================================================================
DEV float wave_sum_f32(float v) { return group_sum<64>(v); }
// One token by one wave: lane r < k ends up with the r-th best expert and its final weight.
template <int EPL>  // experts per lane: the wave covers 64*EPL experts
DEV void route_token(const float* lr, const float* bias, int n_expert, int k, int norm, float scale, int sigmoid, int lane,
                     uint32_t& pick_id, float& pick_w) {
    float lg[EPL], score[EPL];
    uint32_t key[EPL];
    float mx = -INFINITY;
    float raw[EPL];
#pragma unroll
    for (int j = 0; j < EPL; j++) raw[j] = lr[min(lane + 64 * j, n_expert - 1)];  // every load in flight, no branch
#pragma unroll
    for (int j = 0; j < EPL; j++) {
        const int e = lane + 64 * j;
        lg[j] = e < n_expert ? raw[j] : -INFINITY;
        if (e < n_expert) mx = fmaxf(mx, lg[j]);
    }
    if (!sigmoid) {
        mx = wave_max_f32(mx);
        float sum = 0.0f;
#pragma unroll
        for (int j = 0; j < EPL; j++) {
            const int e = lane + 64 * j;
            score[j] = e < n_expert ? expf(lg[j] - mx) : 0.0f;
            sum += score[j];
        }
        sum = wave_sum_f32(sum);
        const float inv = 1.0f / sum;
#pragma unroll
        for (int j = 0; j < EPL; j++) score[j] *= inv;
    } else {
#pragma unroll
        for (int j = 0; j < EPL; j++) score[j] = 1.0f / (1.0f + expf(-lg[j]));
    }
    const bool on_logits = !sigmoid && bias == nullptr;
#pragma unroll
    for (int j = 0; j < EPL; j++) {
        const int e = lane + 64 * j;
        float sel = on_logits ? lg[j] : (bias != nullptr && e < n_expert ? score[j] + bias[e] : score[j]);
        key[j] = total_order_key(sel);
    }
    uint32_t taken = 0;
#pragma unroll
    for (int j = 0; j < EPL; j++)
        if (lane + 64 * j >= n_expert) taken |= 1u << j;
    uint32_t my_id = 0;
    float my_score = 0.0f, total = 0.0f;
    for (int r = 0; r < k; r++) {
        // the best key still in play: per lane, then across the wave (32-bit DPP maximum) ...
        uint32_t lbest = 0;
#pragma unroll
        for (int j = 0; j < EPL; j++)
            if (!(taken & (1u << j))) lbest = key[j] > lbest ? key[j] : lbest;
        const uint32_t best = wave_max_u32(lbest);
        // ... and its lowest index: expert = lane + 64*j, so the first slot j with a match holds it,
        // at the lowest matching lane (k <= n_expert: some valid slot is always left, and only valid,
        // untaken slots can match)
        int slot = -1, owner = 0;
        if constexpr (EPL <= 4) {
#pragma unroll
            for (int j = 0; j < EPL; j++) {
                const uint64_t mask = __ballot(!(taken & (1u << j)) && key[j] == best);
                if (slot < 0 && mask != 0) {  // uniform
                    slot = j;
                    owner = __builtin_ctzll(mask);
                }
            }
        } else {  // many slots per lane: each lane's lowest matching index, then a wave minimum
            uint32_t cand = 0;  // ~index, so that the maximum is the lowest index; 0 = no match
#pragma unroll
            for (int j = EPL - 1; j >= 0; j--)
                if (!(taken & (1u << j)) && key[j] == best) cand = ~(uint32_t)(lane + 64 * j);
            const uint32_t win = ~wave_max_u32(cand);
            owner = (int)(win & 63u);
            slot = (int)(win >> 6);
        }
        const uint32_t e = (uint32_t)owner + 64u * (uint32_t)slot;
        float s = 0.0f;
#pragma unroll
        for (int j = 0; j < EPL; j++) s = slot == j ? score[j] : s;  // selects, not an indexed (scratch) read
        if (lane == owner) taken |= 1u << slot;
        s = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, s), owner));
        total += s;  // best-first sequential f32 sum, as the reference's iterator sum
        if (lane == r) {
            my_id = e;
            my_score = s;
        }
    }
    const float w = (norm && total > 0.0f) ? my_score / total : (norm ? 1.0f / (float)k : my_score);
    pick_id = my_id;
    pick_w = w * scale;
}
template <int EPL>
DEV void route_topk_body(const float* logits, const float* bias, int rows, int n_expert, int k, int norm, float scale,
                         int sigmoid, uint32_t* ids, float* wout) {
    const int lane = threadIdx.x & 63;
    const uint64_t t = (uint64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (t >= (uint64_t)rows) return;  // whole wave exits together
    uint32_t id;
    float w;
    route_token<EPL>(logits + t * (uint64_t)n_expert, bias, n_expert, k, norm, scale, sigmoid, lane, id, w);
    if (lane < k) {
        ids[t * (uint64_t)k + lane] = id;
        wout[t * (uint64_t)k + lane] = w;
    }
}

extern "C" __global__ __launch_bounds__(256) void apk_route_topk(const float* logits, const float* bias, int rows,
                                                                int n_expert, int k, int norm, float scale,
                                                                int sigmoid, uint32_t* ids, float* wout) {
    route_topk_body<4>(logits, bias, rows, n_expert, k, norm, scale, sigmoid, ids, wout);
}
// narrow routers: one or two experts per lane (a round of the selection costs per slot held)
extern "C" __global__ __launch_bounds__(256) void apk_route_topk_e64(const float* logits, const float* bias, int rows,
                                                                    int n_expert, int k, int norm, float scale,
                                                                    int sigmoid, uint32_t* ids, float* wout) {
    route_topk_body<1>(logits, bias, rows, n_expert, k, norm, scale, sigmoid, ids, wout);
}
extern "C" __global__ __launch_bounds__(256) void apk_route_topk_e128(const float* logits, const float* bias, int rows,
                                                                     int n_expert, int k, int norm, float scale,
                                                                     int sigmoid, uint32_t* ids, float* wout) {
    route_topk_body<2>(logits, bias, rows, n_expert, k, norm, scale, sigmoid, ids, wout);
}
// routers wider than 256 experts (the reference's heap path, moe.rs:536-545): up to 1024
extern "C" __global__ __launch_bounds__(256) void apk_route_topk_wide(const float* logits, const float* bias, int rows,
                                                                     int n_expert, int k, int norm, float scale,
                                                                     int sigmoid, uint32_t* ids, float* wout) {
    route_topk_body<16>(logits, bias, rows, n_expert, k, norm, scale, sigmoid, ids, wout);
}
