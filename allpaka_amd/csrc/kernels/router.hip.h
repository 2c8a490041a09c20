// gfx950 device code, part of apk_kernels.hip (one translation unit, one code object): MoE router: softmax / sigmoid + top-k.
#pragma once

// =========================================================================
// MoE router: per token softmax (sigmoid == 1: sigmoid; 2: the row holds the scores already) over n_expert <= 64*EPL logits, top-k
// by descending selection score with the LOWER INDEX winning ties, winners
// renormalised (moe.rs:524-594).  One wave per token; lane l holds experts
// l, l+64, l+128, ... (EPL of them).
// The scores are the reference's bit for bit, so that the selection -- which the reference makes on the scores, not
// on the logits (moe.rs:552-582) -- picks the same experts in the same order also where two distinct logits round
// to one score (logits closer than an ulp of logit - max, or of the score: then the lower index wins there and
// here), and the weights are the reference's bit for bit as well:
//   * exp is glibc's expf (the libm symbol Rust's f32::exp lowers to on linux-gnu), restated below;
//   * the softmax denominator is summed one score after the other in index order, as activation.rs:5-16 does,
//     not as a tree over lanes; 1/sum and score/total are IEEE divisions.
// =========================================================================
// glibc's expf (sysdeps/ieee754/flt-32/e_expf.c, glibc >= 2.27: exp(x) = 2^(k/32) * 2^(r/32) with a 32-entry
// table and a cubic in double precision, one rounding to float).  The same restatement in C agrees with the host's
// libm (glibc 2.35) on every one of 4.8e8 inputs, with and without contraction of its three multiply-adds.
static __device__ const uint64_t kExp2fTab[32] = {
    0x3ff0000000000000, 0x3fefd9b0d3158574, 0x3fefb5586cf9890f, 0x3fef9301d0125b51, 0x3fef72b83c7d517b, 0x3fef54873168b9aa,
    0x3fef387a6e756238, 0x3fef1e9df51fdee1, 0x3fef06fe0a31b715, 0x3feef1a7373aa9cb, 0x3feedea64c123422, 0x3feece086061892d,
    0x3feebfdad5362a27, 0x3feeb42b569d4f82, 0x3feeab07dd485429, 0x3feea47eb03a5585, 0x3feea09e667f3bcd, 0x3fee9f75e8ec5f74,
    0x3feea11473eb0187, 0x3feea589994cce13, 0x3feeace5422aa0db, 0x3feeb737b0cdc5e5, 0x3feec49182a3f090, 0x3feed503b23e255d,
    0x3feee89f995ad3ad, 0x3feeff76f2fb5e47, 0x3fef199bdd85529c, 0x3fef3720dcef9069, 0x3fef5818dcfba487, 0x3fef7c97337b9b5f,
    0x3fefa4afa2a490da, 0x3fefd0765b6e4540};
// tab: kExp2fTab[lane & 31], fetched by the caller next to its first loads; the entry a lane needs comes from the lane
// that holds it (a cross-lane read, so the lookup adds no memory round trip after the logits have arrived).  Called by
// every lane of the wave together: the special cases are selects after the common path, not branches around it.
DEV float expf_ref(float x, uint64_t tab) {
    const uint32_t ux = __builtin_bit_cast(uint32_t, x);
    const uint32_t abstop = (ux >> 20) & 0x7ffu;
    const double z = (0x1.71547652b82fep+0 * 32) * (double)x;
    double kd = z + 0x1.8p+52;  // round to nearest integer in the low mantissa bits
    const uint64_t ki = __builtin_bit_cast(uint64_t, kd);
    kd -= 0x1.8p+52;
    const double r = z - kd;
    const int src = (int)(ki & 31);
    const uint64_t t = ((uint64_t)(uint32_t)__shfl((int)(uint32_t)(tab >> 32), src, 64) << 32) | (uint32_t)__shfl((int)(uint32_t)tab, src, 64);
    const double sc = __builtin_bit_cast(double, t + (ki << 47));
    const double p = (0x1.c6af84b912394p-5 / 32 / 32 / 32) * r + (0x1.ebfce50fac4f3p-3 / 32 / 32);
    const double y = p * (r * r) + ((0x1.62e42ff0c52d6p-1 / 32) * r + 1.0);
    float res = (float)(y * sc);
    if (abstop >= (0x42b00000u >> 20)) {  // |x| >= 88 or NaN
        if (ux == 0xff800000u) res = 0.0f;                     // -inf
        else if (abstop >= (0x7f800000u >> 20)) res = x + x;    // +inf, NaN
        else if (x > 0x1.62e42ep6f) res = INFINITY;             // overflow
        else if (x < -0x1.9fe368p6f) res = 0.0f;                // underflow to zero
    }
    return res;
}

// One token by one wave: lane r < k ends up with the r-th best expert and its final weight.
// lds: 64*EPL floats of the wave's own (the scores in index order, for the one-after-the-other sum).
template <int EPL>  // experts per lane: the wave covers 64*EPL experts
DEV void route_token(const float* lr, const float* bias, int n_expert, int k, int norm, float scale, int sigmoid, int lane,
                     uint32_t& pick_id, float& pick_w, float* lds) {
    float lg[EPL], score[EPL];
    uint32_t key[EPL];
    float mx = -INFINITY;
    float raw[EPL];
    const uint64_t tab = kExp2fTab[lane & 31];  // this lane's entry of the exp table, in flight with the logits
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
#pragma unroll
        for (int j = 0; j < EPL; j++) {
            const int e = lane + 64 * j;
            const float ex = expf_ref(lg[j] - mx, tab);  // every lane: lanes past n_expert hold -inf and get 0
            score[j] = e < n_expert ? ex : 0.0f;
            if constexpr (EPL > 4) lds[e] = score[j];
        }
        // in index order, every lane the same chain of additions.  Up to 256 experts the scores come out of the lanes'
        // registers one by one (scores past n_expert are +0 and change nothing); wider routers walk the wave's own
        // copy in LDS (a wave's LDS operations complete in order; the wave barrier pins the compiler's order).
        float sum = 0.0f;
        if constexpr (EPL > 4) __builtin_amdgcn_wave_barrier();  // the walk below reads what other lanes stored above
        if constexpr (EPL <= 4) {
#pragma unroll
            for (int j = 0; j < EPL; j++)
#pragma unroll
                for (int l = 0; l < 64; l++)
                    sum += __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, score[j]), l));
        } else {
            for (int e = 0; e < n_expert; e++) sum += lds[e];
        }
        const float inv = 1.0f / sum;
#pragma unroll
        for (int j = 0; j < EPL; j++) score[j] *= inv;
    } else if (sigmoid == 1) {
#pragma unroll
        for (int j = 0; j < EPL; j++) score[j] = 1.0f / (1.0f + expf_ref(-lg[j], tab));
    } else {  // the inputs are the scores already: route(probs, k) of the softmaxed row (moe.rs:623-658)
#pragma unroll
        for (int j = 0; j < EPL; j++) score[j] = lane + 64 * j < n_expert ? lg[j] : 0.0f;
    }
#pragma unroll
    for (int j = 0; j < EPL; j++) {  // the selection value: the score, plus the expert's bias where the model has one
        const int e = lane + 64 * j;
        const float sel = bias != nullptr && e < n_expert ? score[j] + bias[e] : score[j];
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
    __shared__ float s_scores[4][EPL > 4 ? 64 * EPL : 1];
    const int lane = threadIdx.x & 63;
    const uint64_t t = (uint64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (t >= (uint64_t)rows) return;  // whole wave exits together
    uint32_t id;
    float w;
    route_token<EPL>(logits + t * (uint64_t)n_expert, bias, n_expert, k, norm, scale, sigmoid, lane, id, w, s_scores[threadIdx.x >> 6]);
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
