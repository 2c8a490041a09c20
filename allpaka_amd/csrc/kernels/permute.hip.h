// gfx950 device code, part of apk_kernels.hip (one translation unit, one code object): token -> expert grouping, gather / scatter of rows, the calibration copy.
#pragma once

// =========================================================================
// Token -> expert grouping (moe.rs:229-271, prefill.rs:624-675), deterministic:
// rows of an expert are in ascending token order, exactly the CPU order.
// One workgroup per expert, no global atomics and no scratch memory:
//   pass A  every workgroup histograms all rows*k picks in LDS (integer LDS
//           atomics: the counts are order-independent) and derives its own
//           row0 = sum of counts of lower experts and its index among the
//           non-empty experts;
//   pass B  walks the tokens in order, ranks the tokens that picked this expert
//           with a ballot/popcount scan and writes tok[], hit_row[], hit_w[].
// A token's hit list is ordered by ascending expert id: the slot of this expert
// in it is the number of the token's picks with a smaller id.
// =========================================================================
#define APK_PERMUTE_THREADS 512
extern "C" __global__ __launch_bounds__(APK_PERMUTE_THREADS) void apk_moe_permute(
    const uint32_t* ids, const float* w, int rows, int k, int n_expert, uint32_t* table, uint32_t* n_used_out,
    uint32_t* tok, uint32_t* tok_off, uint32_t* hit_row, float* hit_w, uint32_t* fault) {
    __shared__ uint32_t hist[1024];
    __shared__ uint32_t wave_tot[APK_PERMUTE_THREADS / 64], wave_used[APK_PERMUTE_THREADS / 64];
    __shared__ uint32_t s_row0, s_used;
    const int e = blockIdx.x;
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    for (int i = tid; i < n_expert; i += blockDim.x) hist[i] = 0;
    __syncthreads();
    const int total = rows * k;
    auto count = [&](uint32_t id) {
        if (id < (uint32_t)n_expert) atomicAdd(&hist[id], 1u);
        else if (e == 0) atomicOr(fault, APK_FAULT_EXPERT_RANGE);
    };
    {   // 16-byte loads, four in flight per lane (the ids sit in L2; one dependent load per
        // pick would serialise a hit latency per iteration)
        const int nvec = total >> 2;
        const u32x4* ids4 = (const u32x4*)ids;
        for (int base = 0; base < nvec; base += 4 * blockDim.x) {
            u32x4 v[4];
#pragma unroll
            for (int j = 0; j < 4; j++) v[j] = ids4[min(base + tid + j * (int)blockDim.x, nvec - 1)];
#pragma unroll
            for (int j = 0; j < 4; j++)
                if (base + tid + j * (int)blockDim.x < nvec) {
                    count(v[j].x);
                    count(v[j].y);
                    count(v[j].z);
                    count(v[j].w);
                }
        }
        for (int i = (nvec << 2) + tid; i < total; i += blockDim.x) count(ids[i]);
    }
    __syncthreads();
    {  // row0 = picks of lower experts, s_used = non-empty lower experts: a workgroup sum, not a serial walk
        uint32_t r0 = 0, used = 0;
        for (int i = tid; i < e; i += blockDim.x) {
            r0 += hist[i];
            used += hist[i] != 0;
        }
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            r0 += __shfl_xor(r0, o, 64);
            used += __shfl_xor(used, o, 64);
        }
        if (lane == 0) {
            wave_tot[wv] = r0;
            wave_used[wv] = used;
        }
        __syncthreads();
        if (tid == 0) {
            uint32_t a = 0, b = 0;
            for (int i = 0; i < (int)(blockDim.x >> 6); i++) {
                a += wave_tot[i];
                b += wave_used[i];
            }
            s_row0 = a;
            s_used = b;
        }
    }
    __syncthreads();
    const uint32_t row0 = s_row0, mine = hist[e];
    if (e == 0)
        for (int t = tid; t <= rows; t += blockDim.x) tok_off[t] = (uint32_t)t * (uint32_t)k;
    if (tid == 0) {
        if (mine) {
            table[3 * s_used] = (uint32_t)e;
            table[3 * s_used + 1] = row0;
            table[3 * s_used + 2] = mine;
        }
        if (e == n_expert - 1) *n_used_out = s_used + (mine != 0);
    }
    if (mine == 0) return;  // uniform for the workgroup
    uint32_t running = 0;
    for (int base = 0; base < rows; base += blockDim.x) {
        const int t = base + tid;
        int j_hit = -1, slot = 0;
        if (t < rows) {
            const uint32_t* mine_ids = ids + (uint64_t)t * k;
            int j = 0;
            if ((k & 3) == 0) {  // rows of picks are 16-byte aligned: two tiles in flight
                for (; j + 8 <= k; j += 8) {
                    const u32x4 a = *(const u32x4*)(mine_ids + j), b = *(const u32x4*)(mine_ids + j + 4);
                    const uint32_t v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
                    for (int i = 0; i < 8; i++) {
                        if (v[i] == (uint32_t)e && j_hit < 0) j_hit = j + i;
                        slot += v[i] < (uint32_t)e;
                    }
                }
            }
            for (; j < k; j++) {
                const uint32_t id = mine_ids[j];
                if (id == (uint32_t)e && j_hit < 0) j_hit = j;
                slot += id < (uint32_t)e;
            }
        }
        const bool flag = j_hit >= 0;
        const uint64_t mask = __ballot(flag);
        const uint32_t in_wave = (uint32_t)__popcll(mask & ((1ull << lane) - 1ull));
        if (lane == 0) wave_tot[wv] = (uint32_t)__popcll(mask);
        __syncthreads();
        uint32_t before = 0, all = 0;
        for (int i = 0; i < (int)(blockDim.x >> 6); i++) {
            const uint32_t c = wave_tot[i];
            before += i < wv ? c : 0;
            all += c;
        }
        if (flag) {
            const uint32_t r = row0 + running + before + in_wave;
            tok[r] = (uint32_t)t;
            hit_row[(uint64_t)t * k + slot] = r;
            hit_w[(uint64_t)t * k + slot] = w[(uint64_t)t * k + j_hit];
        }
        running += all;
        __syncthreads();
    }
}

// Router and grouping of a decode-sized batch as ONE launch (at most 16 tokens): the two kernels above
// cost a launch each and the second waits for the first, which is most of their time at these sizes
// (1 token, 128 experts, top-8: 7.8 us as two launches, 4.8 us as one; from about 24 tokens on the two
// launches are ahead).  One workgroup of 16 waves, a token per wave (the same arithmetic as
// apk_route_topk); the picks stay in LDS, an expert's tokens are a bit mask in LDS (bit t set when token
// t picked it: LDS integer atomics, order-independent), and the grouping falls out of popcounts -- rows
// of an expert = bits of its mask, row0 = prefix sum over lower experts, a token's row inside its expert
// = bits below the token's.  Same outputs as apk_route_topk followed by apk_moe_permute, bit for bit.
#define APK_FUSED_ROUTE_TOKENS 16
template <int EPL>
DEV void route_group_small_body(const float* logits, const float* bias, int rows, int n_expert, int k, int norm, float scale,
                                int sigmoid, uint32_t* ids, float* wout, uint32_t* table, uint32_t* n_used_out, uint32_t* tok,
                                uint32_t* tok_off, uint32_t* hit_row, float* hit_w) {
    __shared__ uint32_t mask[1024];
    __shared__ uint32_t s_row0[1024];
    __shared__ uint32_t s_ids[APK_FUSED_ROUTE_TOKENS * 64];
    __shared__ float s_w[APK_FUSED_ROUTE_TOKENS * 64];
    __shared__ uint32_t wave_cnt[16], wave_used[16];
    __shared__ float s_scores[APK_FUSED_ROUTE_TOKENS][EPL > 4 ? 64 * EPL : 1];
    // the widest router (1024 experts) keeps 16 tokens x 1024 scores here: 80 KiB of LDS with the tables above, more
    // than the 64 KiB of earlier parts of the family -- this code object is built for gfx950 (160 KiB per workgroup) only
    static_assert(sizeof(mask) + sizeof(s_row0) + sizeof(s_ids) + sizeof(s_w) + sizeof(wave_cnt) + sizeof(wave_used) +
                      sizeof(s_scores) <= 160 * 1024, "LDS budget of a gfx950 workgroup");
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    if (tid < n_expert) mask[tid] = 0u;
    __syncthreads();
    if (wv < rows) {  // uniform per wave: wave wv routes token wv
        uint32_t id;
        float w;
        route_token<EPL>(logits + (uint64_t)wv * n_expert, bias, n_expert, k, norm, scale, sigmoid, lane, id, w, s_scores[wv]);
        if (lane < k) {
            ids[wv * k + lane] = id;
            wout[wv * k + lane] = w;
            s_ids[wv * k + lane] = id;
            s_w[wv * k + lane] = w;
            atomicOr(&mask[id], 1u << wv);
        }
    }
    __syncthreads();
    {   // per expert: rows, then exclusive sums of the rows and of the non-empty experts below it
        const uint32_t cnt = tid < n_expert ? (uint32_t)__popc(mask[tid]) : 0u;
        uint32_t inc = cnt, used = cnt != 0;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const uint32_t a = __shfl_up(inc, o, 64), b = __shfl_up(used, o, 64);
            if (lane >= o) {
                inc += a;
                used += b;
            }
        }
        if (lane == 63) {
            wave_cnt[wv] = inc;
            wave_used[wv] = used;
        }
        __syncthreads();
        uint32_t base = 0, ubase = 0, all_used = 0;
        for (int i = 0; i < 16; i++) {
            base += i < wv ? wave_cnt[i] : 0u;
            ubase += i < wv ? wave_used[i] : 0u;
            all_used += wave_used[i];
        }
        const uint32_t row0 = base + inc - cnt, uidx = ubase + used - (cnt != 0);
        if (tid < n_expert) {
            s_row0[tid] = row0;
            if (cnt) {
                table[3 * uidx] = (uint32_t)tid;
                table[3 * uidx + 1] = row0;
                table[3 * uidx + 2] = cnt;
            }
        }
        if (tid == 0) *n_used_out = all_used;
    }
    __syncthreads();
    if (tid <= rows) tok_off[tid] = (uint32_t)tid * (uint32_t)k;
    if (tid < rows * k) {
        const int t = tid / k;
        const uint32_t e = s_ids[tid];
        const uint32_t r = s_row0[e] + (uint32_t)__popc(mask[e] & ((1u << t) - 1u));
        int slot = 0;  // the token's hits are listed by ascending expert
        for (int j = 0; j < k; j++) slot += s_ids[t * k + j] < e;
        tok[r] = (uint32_t)t;
        hit_row[t * k + slot] = r;
        hit_w[t * k + slot] = s_w[tid];
    }
}
#define APK_ROUTE_GROUP_SMALL(NAME, EPL)                                                                                 \
    extern "C" __global__ __launch_bounds__(1024) void NAME(                                                             \
        const float* logits, const float* bias, int rows, int n_expert, int k, int norm, float scale, int sigmoid,       \
        uint32_t* ids, float* wout, uint32_t* table, uint32_t* n_used_out, uint32_t* tok, uint32_t* tok_off,            \
        uint32_t* hit_row, float* hit_w) {                                                                               \
        route_group_small_body<EPL>(logits, bias, rows, n_expert, k, norm, scale, sigmoid, ids, wout, table, n_used_out, \
                                    tok, tok_off, hit_row, hit_w);                                                       \
    }
APK_ROUTE_GROUP_SMALL(apk_route_group_small_e64, 1)
APK_ROUTE_GROUP_SMALL(apk_route_group_small_e128, 2)
APK_ROUTE_GROUP_SMALL(apk_route_group_small_e256, 4)
APK_ROUTE_GROUP_SMALL(apk_route_group_small_e1024, 16)

// The same grouping for large batches, as two launches.  In the single launch above every
// workgroup walks all rows*k picks, which is fastest up to a couple of thousand tokens and
// grows linearly beyond.  Here the tokens are cut into parts of APK_PART_TOKENS:
//   apk_moe_count  one workgroup per part histograms the part's picks (LDS integer atomics:
//                  order-independent) into counts[part][expert];
//   apk_moe_rank   one workgroup per (expert, part): row0 of the expert and the rows of the
//                  expert in earlier parts come from counts (sums, no atomics), then the part's
//                  tokens are ranked in token order with the same ballot scan.
// Same outputs, bit for bit: the order inside an expert is still ascending token order.
#define APK_PART_TOKENS 1024
extern "C" __global__ __launch_bounds__(APK_PERMUTE_THREADS) void apk_moe_count(const uint32_t* ids, int rows, int k,
                                                                                int n_expert, uint32_t* counts,
                                                                                uint32_t* fault) {
    __shared__ uint32_t hist[1024];
    const int part = blockIdx.x, tid = threadIdx.x;
    for (int i = tid; i < n_expert; i += blockDim.x) hist[i] = 0;
    __syncthreads();
    const int t0 = part * APK_PART_TOKENS, t1 = min(rows, t0 + APK_PART_TOKENS);
    const uint32_t* p0 = ids + (uint64_t)t0 * k;
    const int total = (t1 - t0) * k;
    bool bad = false;
    for (int base = 0; base < total; base += 4 * (int)blockDim.x) {  // four picks in flight per lane
        uint32_t v[4];
#pragma unroll
        for (int j = 0; j < 4; j++) v[j] = p0[min(base + j * (int)blockDim.x + tid, total - 1)];
#pragma unroll
        for (int j = 0; j < 4; j++)
            if (base + j * (int)blockDim.x + tid < total) {
                if (v[j] < (uint32_t)n_expert) atomicAdd(&hist[v[j]], 1u);
                else bad = true;
            }
    }
    if (bad) atomicOr(fault, APK_FAULT_EXPERT_RANGE);
    __syncthreads();
    for (int i = tid; i < n_expert; i += blockDim.x) counts[(uint64_t)part * n_expert + i] = hist[i];
}

extern "C" __global__ __launch_bounds__(APK_PERMUTE_THREADS) void apk_moe_rank(
    const uint32_t* ids, const float* w, int rows, int k, int n_expert, int parts, const uint32_t* counts, uint32_t* table,
    uint32_t* n_used_out, uint32_t* tok, uint32_t* tok_off, uint32_t* hit_row, float* hit_w) {
    __shared__ uint32_t wave_a[APK_PERMUTE_THREADS / 64], wave_b[APK_PERMUTE_THREADS / 64], wave_tot[APK_PERMUTE_THREADS / 64];
    __shared__ uint32_t s_row0, s_used;
    const int e = blockIdx.x / parts, part = blockIdx.x - e * parts;
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6, nwv = (int)(blockDim.x >> 6);
    {  // rows of lower experts (all parts) and how many of them are non-empty
        uint32_t r0 = 0, used = 0;
        for (int i = tid; i < e; i += blockDim.x) {
            uint32_t c = 0;
            for (int q = 0; q < parts; q++) c += counts[(uint64_t)q * n_expert + i];
            r0 += c;
            used += c != 0;
        }
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            r0 += __shfl_xor(r0, o, 64);
            used += __shfl_xor(used, o, 64);
        }
        if (lane == 0) {
            wave_a[wv] = r0;
            wave_b[wv] = used;
        }
        __syncthreads();
        if (tid == 0) {
            uint32_t a = 0, b = 0;
            for (int i = 0; i < nwv; i++) {
                a += wave_a[i];
                b += wave_b[i];
            }
            s_row0 = a;
            s_used = b;
        }
        __syncthreads();
    }
    uint32_t before = 0, mine_total = 0;  // this expert's rows in earlier parts / in all parts (uniform)
    for (int q = 0; q < parts; q++) {
        const uint32_t c = counts[(uint64_t)q * n_expert + e];
        before += q < part ? c : 0u;
        mine_total += c;
    }
    const uint32_t mine = counts[(uint64_t)part * n_expert + e];
    const int t0 = part * APK_PART_TOKENS, t1 = min(rows, t0 + APK_PART_TOKENS);
    if (e == 0) {
        for (int t = t0 + tid; t < t1; t += blockDim.x) tok_off[t] = (uint32_t)t * (uint32_t)k;
        if (part == parts - 1 && tid == 0) tok_off[rows] = (uint32_t)rows * (uint32_t)k;
    }
    if (part == 0 && tid == 0) {
        if (mine_total) {
            table[3 * s_used] = (uint32_t)e;
            table[3 * s_used + 1] = s_row0;
            table[3 * s_used + 2] = mine_total;
        }
        if (e == n_expert - 1) *n_used_out = s_used + (mine_total != 0);
    }
    if (mine == 0) return;  // uniform for the workgroup
    uint32_t running = s_row0 + before;
    for (int base = t0; base < t1; base += blockDim.x) {
        const int t = base + tid;
        int j_hit = -1, slot = 0;
        if (t < t1) {
            const uint32_t* mine_ids = ids + (uint64_t)t * k;
            int j = 0;
            if ((k & 3) == 0) {
                for (; j + 8 <= k; j += 8) {
                    const u32x4 a = *(const u32x4*)(mine_ids + j), b = *(const u32x4*)(mine_ids + j + 4);
                    const uint32_t v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
                    for (int i = 0; i < 8; i++) {
                        if (v[i] == (uint32_t)e && j_hit < 0) j_hit = j + i;
                        slot += v[i] < (uint32_t)e;
                    }
                }
            }
            for (; j < k; j++) {
                const uint32_t id = mine_ids[j];
                if (id == (uint32_t)e && j_hit < 0) j_hit = j;
                slot += id < (uint32_t)e;
            }
        }
        const bool flag = j_hit >= 0;
        const uint64_t mask = __ballot(flag);
        const uint32_t in_wave = (uint32_t)__popcll(mask & ((1ull << lane) - 1ull));
        if (lane == 0) wave_tot[wv] = (uint32_t)__popcll(mask);
        __syncthreads();
        uint32_t bef = 0, all = 0;
        for (int i = 0; i < nwv; i++) {
            const uint32_t c = wave_tot[i];
            bef += i < wv ? c : 0;
            all += c;
        }
        if (flag) {
            const uint32_t r = running + bef + in_wave;
            tok[r] = (uint32_t)t;
            hit_row[(uint64_t)t * k + slot] = r;
            hit_w[(uint64_t)t * k + slot] = w[(uint64_t)t * k + j_hit];
        }
        running += all;
        __syncthreads();
    }
}

// Gathered activations in tok order (moe.rs:348-352): dst[r,:] = src[tok[r],:].
// Every source row is wanted k times, by destination rows that lie far apart (one per expert that the
// token picked).  Taken in destination order the k reads of a row come from any of the 8 XCDs, each with
// an L2 of its own, and the row crosses the fabric up to 8 times (T=4096, 2048 f32 columns: 75 us).  Here
// workgroup b runs on XCD b % 8 and takes, of the 32 destination rows of group b / 8, those whose SOURCE
// row number is b % 8 modulo 8: a source row is then only ever read through one L2, which holds that
// XCD's eighth of the source for batches of a few thousand tokens (53 us; the token-side scatter 44 us).
#define APK_GATHER_GROUP 32
extern "C" __global__ __launch_bounds__(256) void apk_gather_rows(const u32x4* src, const uint32_t* tok,
                                                                 uint32_t src_rows, uint32_t total_rows, int row_vecs,
                                                                 u32x4* dst, uint32_t* fault) {
    const uint32_t xcd = blockIdx.x & 7u, r0 = (blockIdx.x >> 3) * APK_GATHER_GROUP;
    const int lane = threadIdx.x & 63;
    const uint32_t r = r0 + (uint32_t)lane;
    const bool mine_to_check = lane < APK_GATHER_GROUP && r < total_rows;
    const uint32_t t = mine_to_check ? tok[r] : 0u;
    const bool mine = mine_to_check && (t & 7u) == xcd;
    if (__ballot(mine && t >= src_rows) != 0 && threadIdx.x == 0) atomicOr(fault, APK_FAULT_ROW_RANGE);
    uint64_t m = __ballot(mine && t < src_rows);  // the same in every wave of the workgroup
    while (m) {
        const int j = __builtin_ctzll(m);
        m &= m - 1;
        const u32x4* sp = src + (uint64_t)__shfl(t, j, 64) * row_vecs;
        u32x4* dp = dst + (uint64_t)(r0 + (uint32_t)j) * row_vecs;
        for (int c = threadIdx.x; c < row_vecs; c += blockDim.x) nt_store(sp[c], dp + c);
    }
}

// The same permutation driven from the token side: dst[hit_row[t*k + j], :] = src[t, :]
// for the k hits of token t (the CSR lists of apk_moe_permute).  Each source row is read
// from HBM once and written k times; the gather form above re-reads it from every XCD's
// own L2 (8 XCDs, 8 fills of the same row through the fabric).
// One workgroup per (token, slice of 256*TPT tiles, hit): TPT loads and TPT stores per lane and
// the wave is gone -- a write-heavy launch runs faster the shorter its waves are (a workgroup
// that kept a token's tiles and stored them k times took 62 us where this takes 50 us, for
// 302 MB; a plain copy of as many bytes 48 us).  The k workgroups that share a source slice are
// consecutive on one XCD (workgroup b is started on XCD b % 8), so k - 1 of the k loads hit
// that XCD's L2; without that order the launch takes 76 us.
template <int TPT>
DEV void scatter_rows_body(const u32x4* src, const uint32_t* hit_row, uint32_t k, uint32_t total_rows, int row_vecs,
                           u32x4* dst, uint32_t* fault, uint32_t items, uint32_t slices) {
    const uint32_t b = blockIdx.x, xcd = b & 7u, m = b >> 3;
    const uint32_t item = xcd + 8u * (m / k), j = m % k;
    if (item >= items) return;  // uniform
    const uint32_t t = item / slices, s = item - t * slices;
    const uint32_t r = hit_row[(uint64_t)t * k + j];
    const u32x4* sp = src + (uint64_t)t * row_vecs;
    u32x4 a[TPT];
    int c[TPT];
#pragma unroll
    for (int i = 0; i < TPT; i++) {
        c[i] = (int)((s * TPT + i) * 256u + threadIdx.x);
        a[i] = sp[min(c[i], row_vecs - 1)];  // not nontemporal: the next k - 1 workgroups want it in L2
    }
    if (r >= total_rows) {  // uniform
        if (threadIdx.x == 0 && s == 0) atomicOr(fault, APK_FAULT_ROW_RANGE);
        return;
    }
    u32x4* dp = dst + (uint64_t)r * row_vecs;
#pragma unroll
    for (int i = 0; i < TPT; i++)
        if (c[i] < row_vecs) nt_store(a[i], dp + c[i]);
}
extern "C" __global__ __launch_bounds__(256) void apk_scatter_rows_t1(const u32x4* src, const uint32_t* hit_row, uint32_t k,
                                                                     uint32_t total_rows, int row_vecs, u32x4* dst,
                                                                     uint32_t* fault, uint32_t items, uint32_t slices) {
    scatter_rows_body<1>(src, hit_row, k, total_rows, row_vecs, dst, fault, items, slices);
}
extern "C" __global__ __launch_bounds__(256) void apk_scatter_rows_t2(const u32x4* src, const uint32_t* hit_row, uint32_t k,
                                                                     uint32_t total_rows, int row_vecs, u32x4* dst,
                                                                     uint32_t* fault, uint32_t items, uint32_t slices) {
    scatter_rows_body<2>(src, hit_row, k, total_rows, row_vecs, dst, fault, items, slices);
}

// Reference stream for bandwidth calibration: dst = src, one 16-byte tile per lane.
extern "C" __global__ __launch_bounds__(256) void apk_copy(const u32x4* src, u32x4* dst, uint64_t nvec) {
    const uint64_t c = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (c < nvec) wt_store(__builtin_nontemporal_load(src + c), dst + c);
}

// The shared expert of GLM-style MoE layers in the per-token hit lists (model/prefill.rs:621-635, flattened :658-675):
// every token gets one more hit, after its routed ones, of weight 1 at flat row total_rows + token -- the shared FFN's
// rows sit right after the experts' rows.  Any CSR in, the lengthened CSR out (tok_off_out[t] = tok_off[t] + t).
extern "C" __global__ __launch_bounds__(256) void apk_moe_shared_hits(const uint32_t* tok_off, const uint32_t* hit_row,
                                                                     const float* hit_w, uint32_t rows, uint32_t total_rows,
                                                                     uint32_t* tok_off_out, uint32_t* hit_row_out,
                                                                     float* hit_w_out) {
    const uint32_t t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t > rows) return;
    const uint32_t h0 = tok_off[t];
    tok_off_out[t] = h0 + t;
    if (t == rows) return;
    const uint32_t h1 = tok_off[t + 1];
    for (uint32_t i = h0; i < h1; i++) {
        hit_row_out[i + t] = hit_row[i];
        hit_w_out[i + t] = hit_w[i];
    }
    hit_row_out[h1 + t] = total_rows + t;
    hit_w_out[h1 + t] = 1.0f;
}
