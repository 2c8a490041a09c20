// gfx950 device code, part of apk_kernels.hip (one translation unit, one code object): per-head QK-norm + RoPE, K/V cache store, layer prologue, rotary table.
#pragma once

// =========================================================================
// Per-head QK-norm + NeoX RoPE, in place on q [rows, n_q*HD] and k [rows, n_kv*HD]
// (caller loop attention.rs:131-165: rmsnorm(head, w, eps) then the NeoX
// rotation with the row's [sin, cos] table, rope.rs:70-81).
// Lane mapping: a lane holds one 16-byte tile of the first half of a head and
// the tile of its NeoX partners in the second half (EPL = 8 fp16 / 4 f32
// elements each), so the rotation needs no cross-lane traffic, every global
// access is a full 16-byte tile and the LPH = HD/2/EPL lanes of a head cover
// contiguous runs.  A wave owns (row, q or k, group of HPW consecutive heads), HPW = 64/LPH
// heads, and makes ONE pass (about 2-4 KB of heads): one tensor per wave means one norm weight
// per wave and no per-element selects.  Longer waves were measured and dropped: two or four
// passes per wave hold more registers per resident byte and lose 2-8 % over 1024..8192 rows, and
// a wave that carries a row's 64 q heads in 8 passes lives as long as the whole launch, so that a
// batch a few rows beyond one resident round (2061 rows instead of 2048) takes 15 % longer;
// short waves fill in evenly.  (ITERQ stays a template parameter of the item; every kernel sets 1.)
// Wave order: workgroups take items in plain index order, which the dispatcher deals round the eight
// chiplets (XCDs, an L2 each).  The 9 waves that share a row's sin/cos line (64 + 8 heads of 128) so sit on 4-5
// chiplets and the 1 MB table of 2048 rows is fetched 4.6 times: +5 % on the kernel's HBM reads (FETCH_SIZE).
// Giving each chiplet rows of its own removes those reads (FETCH_SIZE then +0.3 %) and was measured slower all the
// same: 13.7 us (rows dealt c, c + 8, ...) and 14.2 us (eight contiguous shares) against 13.5 us in plain order for
// 2048 rows, three runs each on one machine -- the chip moving through memory as one front is worth more than
// the 3.7 MB.  Plain order stays.
// Arithmetic: the reference's, for both activation types (see `headstat`): f64 statistics,
// (x as f64 * scale) as f32 * w, then the four products and two sums of the rotation,
// not contracted.  fp16 results are that f32 result rounded once.
// =========================================================================
// KV = true (k items only): the rotated k tiles are also narrowed to fp16 into the cache row
// kc, and the same tiles of the row's v are narrowed into vc (KvCache::store_at,
// crates/allpaka-model/src/kv.rs:682-697: k and v rows as f16 at pos*kv_dim).
// PAIRS = false: NeoX pairs (i, i + HD/2), one from each of the lane's two tiles; the lane's [sin, cos]
// entries are l*EPL .. l*EPL+EPL-1.  PAIRS = true: adjacent pairs (2i, 2i+1) (RopeStyle::Norm, rope.rs:52-64,
// the Llama-family layout, chosen per model in attention.rs:62-67), both inside one tile; the lane's
// entries are the EPL/2 pairs of each of its two tiles.  Same loads, same bytes, same statistics.
// Partial rotary (rot < HD channels rotate, the rest is normalised and passes through, rope.rs:52-81): the
// table row then has rot/2 entries.  With adjacent pairs a whole tile either rotates or does not (rot is a
// multiple of the tile); with NeoX pairs (i, i + rot/2) the first rot/2/EPL lanes of a head take the partner
// tiles at i and i + rot/2, the others two consecutive tiles of the tail.  rot == HD is the layout above.
// BIAS = true: the projection biases of models that carry them (attention.rs:125-129: add_bias_rows on q, k and
// v right in front of this loop; loader.rs:519-523) are added as the tiles are widened: bias [nheads*HD] f32 for the
// item's tensor (NULL: none); with the cache store, vbias is added to the row's v, which is written back (vout)
// as well as narrowed into the cache.
// NORM = false: neither tensor has a norm weight (the Llama / Qwen2 families: biases or not, then the rotation):
// no statistics, no weight tiles -- the launch then runs at the speed of a plain copy of the same bytes.
// The per-head statistics of this op, for both activation types: the reference's own operations
// (norm.rs:115-187) -- the sum of squares in f64, scale = 1/sqrt(mean + eps) in f64, (x as f64 * scale) as f32 -- so
// that an fp16 result is the reference's f32 result rounded once (a rotated output a*cos - b*sin can nearly cancel,
// and an f32-level difference in the normalised inputs is then many ulps of the fp16 result).  f32 rows take the
// IEEE square root and division; fp16 rows take two f64 Newton steps from the hardware rsq (1e-16 of
// sqrt-then-divide, a third of the instructions), which no fp16 result can show.
template <typename T> struct rotstat : stat<float> {};
template <> struct rotstat<f16_t> : stat<float> {
    DEV double rscale(double ss, int n, float eps) {
        const double v = ss / (double)n + (double)eps;  // n a power of two known at compile time: a multiplication
        double y = (double)__builtin_amdgcn_rsqf((float)v);
        y = y * __builtin_fma(-0.5 * v, y * y, 1.5);
        return y * __builtin_fma(-0.5 * v, y * y, 1.5);
    }
};

// LDSC = true: the wave copies the row's [sin, cos] entries (rot floats) and its tensor's norm weight (HD floats)
// into 2*HD floats of LDS of its own (lmem) and reads the lane's entries back pass by pass, right where they are
// used, instead of holding them in 2-4 registers per element from the first load on.  With fp16 tiles that is the
// difference between 84 and 63 registers, i.e. between 5 and 8 resident waves per SIMD, and this kernel's speed
// follows its resident waves (the arithmetic of a pass is not free next to the stream).  Nothing is shared between
// waves: no barrier, only the wave's own LDS counter.
template <typename T, int HD, int ITER, bool KV = false, bool PAIRS = false, bool BIAS = false, bool NORM = true, bool LDSC = false, bool FULL = false>
DEV void qk_item(T* base, int nheads, int g, const float* w, const float* trow, float eps, int l, int sub, int rot,
                 f16_t* kc = nullptr, const float* bias = nullptr, float* lmem = nullptr) {
    constexpr int EPL = io<T>::VEC;   // elements per lane per half
    constexpr int HALF = HD / 2;
    constexpr int LPH = HALF / EPL;   // lanes per head
    constexpr int HPW = 64 / LPH;     // heads per wave pass
    // the lane's two tiles inside a head, whether each rotates, and where its [sin, cos] floats start
    int off_a, off_b, sc_a, sc_b;
    bool rot_a, rot_b;
    if constexpr (FULL) {  // rot == HD, known at compile time: every tile rotates, no selects below
        rot_a = rot_b = true;
        off_a = EPL * l;
        off_b = HALF + EPL * l;
        sc_a = PAIRS ? off_a : 2 * EPL * l;
        sc_b = PAIRS ? off_b : sc_a + EPL;
        rot = HD;
    } else if constexpr (PAIRS) {
        off_a = EPL * l;
        off_b = HALF + EPL * l;
        rot_a = off_a < rot;
        rot_b = off_b < rot;
        sc_a = rot_a ? off_a : 0;
        sc_b = rot_b ? off_b : 0;
    } else {
        const int lr = (rot >> 1) / EPL;  // lanes of a head that hold rotating pairs
        rot_a = rot_b = l < lr;
        off_a = rot_a ? EPL * l : rot + 2 * EPL * (l - lr);
        off_b = rot_a ? (rot >> 1) + EPL * l : off_a + EPL;
        sc_a = rot_a ? 2 * EPL * l : 0;
        sc_b = sc_a + EPL;
    }
    // Loads return in issue order, so the small cached ones go first and the first pass
    // can start as soon as its own two tiles arrive.  No branch, no conversion here: a
    // lane of a pass beyond the last head re-reads the last head and stores nothing.
    float sc[2 * EPL], wa[EPL], wb[EPL];
    constexpr int NST = (HD + 127) / 128;  // 8-byte pieces per lane of a staged array
    f32x2 st_sc[LDSC ? NST : 1], st_w[LDSC ? NST : 1];
    if constexpr (LDSC) {
        const int lane = sub * LPH + l;
#pragma unroll
        for (int j = 0; j < NST; j++) {  // a piece past the end re-reads the last one and is not written
            const int i = 2 * lane + 128 * j;
            st_sc[j] = *(const f32x2*)(trow + min(i, rot - 2));
            if constexpr (NORM) st_w[j] = *(const f32x2*)(w + min(i, HD - 2));
        }
    } else {
#pragma unroll
        for (int i = 0; i < EPL; i += 4) {  // a tile that does not rotate reads the row's first entries and ignores them
            io<float>::load(trow + sc_a + i, sc + i);
            io<float>::load(trow + sc_b + i, sc + EPL + i);
        }
        if constexpr (NORM) {
#pragma unroll
            for (int i = 0; i < EPL; i += 4) {
                io<float>::load(w + off_a + i, wa + i);
                io<float>::load(w + off_b + i, wb + i);
            }
        }
    }
    typename io<T>::raw_t araw[ITER], braw[ITER];
    float ba[BIAS ? ITER : 1][EPL], bb[BIAS ? ITER : 1][EPL];
    // head of pass `it` and its element offset: recomputed where needed (a few integer
    // operations) rather than kept in registers across the loads
    const int hh_first = g * ITER * HPW + sub;
    auto head_off = [&](int it) { return min(hh_first + it * HPW, nheads - 1) * HD; };
#pragma unroll
    for (int it = 0; it < ITER; it++) {
        const int off = head_off(it);
        __builtin_amdgcn_sched_barrier(0);  // loads stay in program order (returns are in order)
        if constexpr (BIAS) {  // uniform branches: a tensor has a bias or it has none
            if (bias) {
#pragma unroll
                for (int i = 0; i < EPL; i += 4) {
                    io<float>::load(bias + off + off_a + i, ba[it] + i);
                    io<float>::load(bias + off + off_b + i, bb[it] + i);
                }
            }
        }
        araw[it] = io<T>::ldraw_nt(base + off + off_a);
        braw[it] = io<T>::ldraw_nt(base + off + off_b);
    }
    __builtin_amdgcn_sched_barrier(0);  // every load above; all uses below
    if constexpr (LDSC) {
        const int lane = sub * LPH + l;
#pragma unroll
        for (int j = 0; j < NST; j++) {
            const int i = 2 * lane + 128 * j;
            if (i < rot) *(f32x2*)(lmem + i) = st_sc[j];
            if constexpr (NORM) {
                if (i < HD) *(f32x2*)(lmem + HD + i) = st_w[j];
            }
        }
        // other lanes of this wave read these entries back below: the wave barrier keeps the compiler from moving
        // those reads above the writes (it emits no instruction; a wave's LDS operations complete in order)
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int it = 0; it < ITER; it++) {
        float a[EPL], b[EPL], oa[EPL], ob[EPL];
        io<T>::widen(araw[it], a);
        io<T>::widen(braw[it], b);
        if constexpr (BIAS) {
            if (bias) {
#pragma unroll
                for (int i = 0; i < EPL; i++) {
                    a[i] += ba[it][i];
                    b[i] += bb[it][i];
                }
            }
        }
        double scale = 0;
        if constexpr (NORM) {
            double ss = 0;
#pragma unroll
            for (int i = 0; i < EPL; i++) {
                ss = rotstat<T>::sq(ss, a[i]);
                ss = rotstat<T>::sq(ss, b[i]);
            }
            ss = group_sum<LPH>(ss);
            scale = rotstat<T>::rscale(ss, HD, eps);
        }
        if constexpr (LDSC) {  // the lane's entries, back from the wave's LDS (a tile that does not rotate reads the first entries)
#pragma unroll
            for (int i = 0; i < EPL; i += 4) {
                io<float>::load(lmem + sc_a + i, sc + i);
                io<float>::load(lmem + sc_b + i, sc + EPL + i);
            }
            if constexpr (NORM) {
#pragma unroll
                for (int i = 0; i < EPL; i += 4) {
                    io<float>::load(lmem + HD + off_a + i, wa + i);
                    io<float>::load(lmem + HD + off_b + i, wb + i);
                }
            }
        }
        if constexpr (PAIRS) {
#pragma unroll
            for (int i = 0; i < EPL; i++) {
                if constexpr (NORM) {
                    a[i] = rotstat<T>::apply(a[i], scale, wa[i]);
                    b[i] = rotstat<T>::apply(b[i], scale, wb[i]);
                }
            }
#pragma unroll
            for (int m = 0; m < EPL / 2; m++) {  // sc[0 .. EPL): the pairs of tile a, sc[EPL .. 2 EPL): of tile b
                const float sa = sc[2 * m], ca = sc[2 * m + 1], sb = sc[EPL + 2 * m], cb = sc[EPL + 2 * m + 1];
                oa[2 * m] = FULL || rot_a ? a[2 * m] * ca - a[2 * m + 1] * sa : a[2 * m];
                oa[2 * m + 1] = FULL || rot_a ? a[2 * m] * sa + a[2 * m + 1] * ca : a[2 * m + 1];
                ob[2 * m] = FULL || rot_b ? b[2 * m] * cb - b[2 * m + 1] * sb : b[2 * m];
                ob[2 * m + 1] = FULL || rot_b ? b[2 * m] * sb + b[2 * m + 1] * cb : b[2 * m + 1];
            }
        } else {
#pragma unroll
            for (int i = 0; i < EPL; i++) {
                float x = a[i], y = b[i];
                if constexpr (NORM) {
                    x = rotstat<T>::apply(x, scale, wa[i]);
                    y = rotstat<T>::apply(y, scale, wb[i]);
                }
                const float s = sc[2 * i], c = sc[2 * i + 1];
                oa[i] = FULL || rot_a ? x * c - y * s : x;  // not contracted: the reference's four products and two sums
                ob[i] = FULL || rot_a ? x * s + y * c : y;
            }
        }
        const bool live = hh_first + it * HPW < nheads;
        const int off = head_off(it);
        if (live) {
            io<T>::store_wt(base + off + off_a, oa);
            io<T>::store_wt(base + off + off_b, ob);
        }
        if constexpr (KV) {
            if (live && kc != nullptr) {  // kc == nullptr: cache position out of range, the row's cache store is skipped
                store_f16_tile<T>(kc + off + off_a, oa);
                store_f16_tile<T>(kc + off + off_b, ob);
            }
        }
        __builtin_amdgcn_sched_barrier(0);  // pass by pass: pass it+1 waits only for its own tiles
    }
}

// The v half of the cache store, waves of its own (a pure stream: short, few registers, so the k waves stay as light
// as the q waves): a wave narrows HPW heads of the row's v into the cache row vc (two 16-byte tiles per lane, each
// instruction a contiguous run); with a bias, v + v_bias is written back to v as well.
template <typename T, int HD, bool BIAS>
DEV void v_item(T* vrow, int nheads, int g, f16_t* vc, const float* vbias, int lane) {
    constexpr int EPL = io<T>::VEC, HPW = 64 / (HD / 2 / EPL);
    const int total = nheads * HD, start = g * HPW * HD;
    typename io<T>::raw_t raw[2];
    float bv[BIAS ? 2 : 1][EPL];
    int off[2];
#pragma unroll
    for (int j = 0; j < 2; j++) {
        off[j] = start + (lane + 64 * j) * EPL;
        const int oc = min(off[j], total - EPL);  // a lane past the last head re-reads the last tile and stores nothing
        if constexpr (BIAS) {
            if (vbias) {
#pragma unroll
                for (int i = 0; i < EPL; i += 4) io<float>::load(vbias + oc + i, bv[j] + i);
            }
        }
        raw[j] = io<T>::ldraw_nt(vrow + oc);
    }
#pragma unroll
    for (int j = 0; j < 2; j++) {
        float v[EPL];
        io<T>::widen(raw[j], v);
        if (off[j] < total) {
            if constexpr (BIAS) {
                if (vbias) {
#pragma unroll
                    for (int i = 0; i < EPL; i++) v[i] += bv[j][i];
                    io<T>::store_wt(vrow + off[j], v);
                }
            }
            if (vc != nullptr) store_f16_tile<T>(vc + off[j], v);
        }
    }
}

// BLOCK: the workgroup size the host launches (the wave's LDS slot is its index in the workgroup).
template <typename T, int HD, int ITERQ, bool KV = false, bool PAIRS = false, bool BIAS = false, bool NORM = true, bool LDSC = false, int BLOCK = 256>
DEV void qknorm_rope_body(T* q, T* k, const float* qw, const float* kw, const float* rope, int rows, int n_q, int n_kv,
                          float eps, int rot, uint32_t vblock, T* v = nullptr, const uint32_t* cache_pos = nullptr,
                          f16_t* k_cache = nullptr, f16_t* v_cache = nullptr, uint32_t capacity = 0,
                          uint32_t* fault = nullptr, const float* qb = nullptr, const float* kb = nullptr,
                          const float* vb = nullptr) {
    constexpr int LPH = HD / 2 / io<T>::VEC, HPW = 64 / LPH;
    __shared__ __attribute__((aligned(16))) float lds_consts[LDSC ? BLOCK / 64 : 1][LDSC ? 2 * HD : 4];
    float* lmem = LDSC ? lds_consts[threadIdx.x >> 6] : nullptr;
    const int lane = threadIdx.x & 63;
    const int l = lane % LPH, sub = lane / LPH;
    const uint32_t gq = (n_q + HPW * ITERQ - 1) / (HPW * ITERQ), gk = (n_kv + HPW - 1) / HPW;
    // The k items first, then (with the cache store) the v items, then the q items.  The wave's index is a scalar
    // (the host keeps the number of waves below 2^32): the row and group come from scalar arithmetic.
    const uint32_t wid = __builtin_amdgcn_readfirstlane(vblock * (blockDim.x >> 6) + (threadIdx.x >> 6));
    const uint32_t nq_items = (uint32_t)rows * gq, nk_items = (uint32_t)rows * gk, nv_items = KV ? nk_items : 0;
    if (wid >= nq_items + nk_items + nv_items) return;  // whole wave
    // Two facts of the launch choose among four instances of the item: whether this tensor has a norm weight (a model
    // may norm q and not k) and whether the whole head rotates (no per-lane selects then).  Uniform branches.
    const bool full = rot == HD;
    const uint64_t kv_dim = (uint64_t)n_kv * HD;
    if (wid >= nk_items + nv_items) {
        const uint32_t w1 = wid - nk_items - nv_items, row = w1 / gq;
        T* base = q + (uint64_t)row * n_q * HD;
        const float* trow = rope + (uint64_t)row * rot;
        const int g = (int)(w1 - row * gq);
#define APK_QK_Q(N, F) qk_item<T, HD, ITERQ, false, PAIRS, BIAS, N, LDSC, F>(base, n_q, g, qw, trow, eps, l, sub, rot, nullptr, qb, lmem)
        if (NORM && qw) { if (full) APK_QK_Q(NORM, true); else APK_QK_Q(NORM, false); }
        else { if (full) APK_QK_Q(false, true); else APK_QK_Q(false, false); }
#undef APK_QK_Q
    } else if (wid < nk_items) {
        const uint32_t row = wid / gk;
        const int g = (int)(wid - row * gk);
        T* base = k + row * kv_dim;
        const float* trow = rope + (uint64_t)row * rot;
        f16_t* kc = nullptr;
        if constexpr (KV) {
            const uint32_t pos = cache_pos[row];
            const bool ok = pos < capacity;
            if (!ok && lane == 0 && g == 0) atomicOr(fault, APK_FAULT_CACHE_RANGE);
            kc = ok ? k_cache + pos * kv_dim : nullptr;  // nullptr: the row's cache store is skipped
        }
#define APK_QK_K(N, F) qk_item<T, HD, 1, KV, PAIRS, BIAS, N, LDSC, F>(base, n_kv, g, kw, trow, eps, l, sub, rot, kc, kb, lmem)
        if (NORM && kw) { if (full) APK_QK_K(NORM, true); else APK_QK_K(NORM, false); }
        else { if (full) APK_QK_K(false, true); else APK_QK_K(false, false); }
#undef APK_QK_K
    } else {
        if constexpr (KV) {
            const uint32_t w2 = wid - nk_items, row = w2 / gk;
            const uint32_t pos = cache_pos[row];
            v_item<T, HD, BIAS>(v + row * kv_dim, n_kv, (int)(w2 - row * gk), pos < capacity ? v_cache + pos * kv_dim : nullptr, vb, lane);
        }
    }
}
// fp16 tiles: one pass per wave, constants in LDS, workgroups of two waves, up to 64 registers (8 waves per SIMD);
// f32 tiles: one pass per wave, constants in registers, workgroups of four waves.
template <typename T> struct qk_shape { static constexpr bool LDSC = false; static constexpr int BLOCK = 256; };
template <> struct qk_shape<f16_t> { static constexpr bool LDSC = true; static constexpr int BLOCK = 128; };
// Resident waves per SIMD the compiler is to allow for: every fp16 variant is built for 6 (up to 85 registers; the
// plain and the cache-store kernels come out at 62-71, i.e. 7-8 resident waves, none spills), the f32 variants for 4.
#define APK_QK_OCC(T, W16) __launch_bounds__(qk_shape<T>::BLOCK) __attribute__((amdgpu_waves_per_eu(sizeof(T) == 2 ? W16 : 4)))
// One kernel per (norm or not, pairing, cache store, biases, type, head size).  PFX: apk_qknorm_rope
// (a norm weight for q and / or k) or apk_rope (none for either); PN: pairs_ or nothing.  The argument lists are the
// same with and without norm weights (qw, kw are then NULL and unused).
#define APK_QK_PLAIN(PFX, NORM, T, TN, HD, ITER, PAIRS, PN)                                                        \
    extern "C" __global__ APK_QK_OCC(T, 6) void PFX##_##PN##TN##_hd##HD##_i##ITER(                                    \
        T* q, T* k, const float* qw, const float* kw, const float* rope, int rows, int n_q, int n_kv, float eps, int rot) { \
        qknorm_rope_body<T, HD, ITER, false, PAIRS, false, NORM, qk_shape<T>::LDSC, qk_shape<T>::BLOCK>(q, k, qw, kw, rope, rows, n_q, n_kv, eps, rot, blockIdx.x); \
    }
// The same with the K/V cache store fused in: rotated k and the row's v narrowed to fp16
// at cache row cache_pos[row] (one launch instead of QK-norm+RoPE, then two narrowing copies).
#define APK_QK_KV(PFX, NORM, T, TN, HD, ITER, PAIRS, PN)                                                           \
    extern "C" __global__ APK_QK_OCC(T, 6) void PFX##_##PN##kv_##TN##_hd##HD##_i##ITER(                               \
        T* q, T* k, const T* v, const float* qw, const float* kw, const float* rope, const uint32_t* cache_pos,   \
        f16_t* k_cache, f16_t* v_cache, uint32_t capacity, int rows, int n_q, int n_kv, float eps, uint32_t* fault, int rot) { \
        qknorm_rope_body<T, HD, ITER, true, PAIRS, false, NORM, qk_shape<T>::LDSC, qk_shape<T>::BLOCK>(q, k, qw, kw, rope, rows, n_q, n_kv, eps, rot, blockIdx.x, (T*)v, \
                                                                cache_pos, k_cache, v_cache, capacity, fault);    \
    }
// With the projection biases.  Without the cache store v is not touched here; with it, v + v_bias is written back
// to v and narrowed into the cache.
#define APK_QK_BIAS(PFX, NORM, T, TN, HD, ITER, PAIRS, PN)                                                         \
    extern "C" __global__ APK_QK_OCC(T, 6) void PFX##_##PN##bias_##TN##_hd##HD##_i##ITER(                             \
        T* q, T* k, const float* qw, const float* kw, const float* rope, int rows, int n_q, int n_kv, float eps, int rot, \
        const float* qb, const float* kb) {                                                                       \
        qknorm_rope_body<T, HD, ITER, false, PAIRS, true, NORM, qk_shape<T>::LDSC, qk_shape<T>::BLOCK>(q, k, qw, kw, rope, rows, n_q, n_kv, eps, rot, blockIdx.x, nullptr, \
                                                                nullptr, nullptr, nullptr, 0, nullptr, qb, kb, nullptr); \
    }                                                                                                             \
    extern "C" __global__ APK_QK_OCC(T, 6) void PFX##_##PN##kv_bias_##TN##_hd##HD##_i##ITER(                          \
        T* q, T* k, T* v, const float* qw, const float* kw, const float* rope, const uint32_t* cache_pos,         \
        f16_t* k_cache, f16_t* v_cache, uint32_t capacity, int rows, int n_q, int n_kv, float eps, uint32_t* fault, int rot, \
        const float* qb, const float* kb, const float* vb) {                                                      \
        qknorm_rope_body<T, HD, ITER, true, PAIRS, true, NORM, qk_shape<T>::LDSC, qk_shape<T>::BLOCK>(q, k, qw, kw, rope, rows, n_q, n_kv, eps, rot, blockIdx.x, v, \
                                                               cache_pos, k_cache, v_cache, capacity, fault, qb, kb, vb); \
    }
#define APK_QK_FAMILY(PFX, NORM, T, TN, HD, ITER)                                                                  \
    APK_QK_PLAIN(PFX, NORM, T, TN, HD, ITER, false, ) APK_QK_PLAIN(PFX, NORM, T, TN, HD, ITER, true, pairs_)       \
    APK_QK_KV(PFX, NORM, T, TN, HD, ITER, false, ) APK_QK_KV(PFX, NORM, T, TN, HD, ITER, true, pairs_)             \
    APK_QK_BIAS(PFX, NORM, T, TN, HD, ITER, false, ) APK_QK_BIAS(PFX, NORM, T, TN, HD, ITER, true, pairs_)
// one pass per wave for both types (measured)
#define APK_QK_SIZES(PFX, NORM)                                                                                    \
    APK_QK_FAMILY(PFX, NORM, float, f32, 64, 1) APK_QK_FAMILY(PFX, NORM, float, f32, 128, 1) APK_QK_FAMILY(PFX, NORM, float, f32, 256, 1) \
    APK_QK_FAMILY(PFX, NORM, f16_t, f16, 64, 1) APK_QK_FAMILY(PFX, NORM, f16_t, f16, 128, 1) APK_QK_FAMILY(PFX, NORM, f16_t, f16, 256, 1)
APK_QK_SIZES(apk_qknorm_rope, true)
APK_QK_SIZES(apk_rope, false)
// Any other head geometry: head_dim not 64/128/256, a rotary table that covers only the
// leading rot_half pairs of a head (partial rotary: channels >= 2*rot_half are normalised
// and pass through, rope.rs:52-81), or the adjacent-pair style (RopeStyle::Norm, pairs
// (2i, 2i+1), rope.rs:52-64; chosen per model in attention.rs:62-67).  A wave per head,
// element-wise; same arithmetic as the tiled kernels minus the coefficient folding.
template <typename T>
DEV void qknorm_rope_generic_body(T* q, T* k, const float* qw, const float* kw, const float* rope, int rows, int n_q,
                                  int n_kv, int hd, int rot_half, int norm_style, float eps, const float* qb, const float* kb) {
    typedef typename headstat<T>::acc_t acc_t;
    const int lane = threadIdx.x & 63;
    const uint64_t wid = ((uint64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const uint64_t heads = (uint64_t)n_q + n_kv;
    if (wid >= (uint64_t)rows * heads) return;  // whole wave
    const uint64_t row = wid / heads;
    const int hh = (int)(wid % heads);
    const bool isq = hh < n_q;
    T* x = isq ? q + (row * n_q + hh) * (uint64_t)hd : k + (row * n_kv + (hh - n_q)) * (uint64_t)hd;
    const float* w = isq ? qw : kw;
    const float* bias = isq ? qb : kb;  // the projection bias of this head's channels, or none
    if (bias) bias += (uint64_t)(isq ? hh : hh - n_q) * hd;
    auto ld = [&](int i) { return bias ? (float)x[i] + bias[i] : (float)x[i]; };
    const float* t = rope + row * (uint64_t)rot_half * 2;
    typename headstat<T>::scale_t scale{};
    if (w) {
        acc_t ss = 0;
        for (int i = lane; i < hd; i += 64) ss = headstat<T>::sq(ss, ld(i));
        ss = group_sum<64>(ss);  // every lane's loads are consumed here, before any store below
        scale = headstat<T>::rscale(ss, hd, eps);
    }
    for (int i = lane; i < rot_half; i += 64) {
        const int ia = norm_style ? 2 * i : i, ib = norm_style ? 2 * i + 1 : i + rot_half;
        float a = ld(ia), b = ld(ib);
        if (w) {
            a = headstat<T>::apply(a, scale, w[ia]);
            b = headstat<T>::apply(b, scale, w[ib]);
        }
        const float sn = t[2 * i], cs = t[2 * i + 1];
        x[ia] = (T)(a * cs - b * sn);
        x[ib] = (T)(a * sn + b * cs);
    }
    if (w) {
        for (int i = 2 * rot_half + lane; i < hd; i += 64) x[i] = (T)headstat<T>::apply(ld(i), scale, w[i]);
    } else if (bias) {
        for (int i = 2 * rot_half + lane; i < hd; i += 64) x[i] = (T)ld(i);
    }
}
extern "C" __global__ __launch_bounds__(256) void apk_qknorm_rope_generic_f32(
    float* q, float* k, const float* qw, const float* kw, const float* rope, int rows, int n_q, int n_kv, int hd,
    int rot_half, int norm_style, float eps, const float* qb, const float* kb) {
    qknorm_rope_generic_body<float>(q, k, qw, kw, rope, rows, n_q, n_kv, hd, rot_half, norm_style, eps, qb, kb);
}
extern "C" __global__ __launch_bounds__(256) void apk_qknorm_rope_generic_f16(
    f16_t* q, f16_t* k, const float* qw, const float* kw, const float* rope, int rows, int n_q, int n_kv, int hd,
    int rot_half, int norm_style, float eps, const float* qb, const float* kb) {
    qknorm_rope_generic_body<f16_t>(q, k, qw, kw, rope, rows, n_q, n_kv, hd, rot_half, norm_style, eps, qb, kb);
}

// The same step with the rotary angles taken from the rows' positions inside the kernel, for a decode-sized batch:
// [sin, cos] of pair i of a row is sincos((pos[row] as f32) * inv_freq[i]) (rope.rs:18-22), evaluated in double and
// rounded once, exactly what apk_rope_table writes -- so the launch equals apk_rope_table followed by the op on that
// table, without the table (the reference's rmsnorm_rope_freq_dpos / rmsnorm_rope_store_freq_dpos,
// gpu/cuda/kernels.rs:577-671, which read d_pos and inv_freq in the kernel so that one recorded graph serves every
// token).  A wave per head, element-wise, any head geometry and either pairing; with k_cache / v_cache the rotated k
// heads and the row's v heads are also narrowed to fp16 into cache row pos[row] (KvCache::store_at, kv.rs:682-697).
// The double-precision sine and cosine make a wave long; the host takes this kernel for up to 64 rows, where the
// launch, not the arithmetic, is the cost.
template <typename T>
DEV void qknorm_rope_pos_body(T* q, T* k, const T* v, const float* qw, const float* kw, const uint32_t* pos,
                              const float* inv_freq, f16_t* k_cache, f16_t* v_cache, uint32_t capacity, int rows, int n_q,
                              int n_kv, int hd, int rot_half, int norm_style, float eps, uint32_t* fault) {
    typedef typename headstat<T>::acc_t acc_t;
    const int lane = threadIdx.x & 63;
    const uint64_t wid = ((uint64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const uint64_t heads = (uint64_t)n_q + n_kv + (v_cache ? n_kv : 0);
    if (wid >= (uint64_t)rows * heads) return;  // whole wave
    const uint64_t row = wid / heads;
    const int hh = (int)(wid % heads);
    const uint32_t p = pos[row];
    const uint64_t kv_dim = (uint64_t)n_kv * hd;
    const bool cache_ok = p < capacity;  // uniform per row
    if (hh >= n_q + n_kv) {  // a v head: narrowed into the cache as it is
        const int vh = hh - n_q - n_kv;
        if (!cache_ok) return;
        const T* src = v + row * kv_dim + (uint64_t)vh * hd;
        f16_t* dst = v_cache + p * kv_dim + (uint64_t)vh * hd;
        for (int i = lane; i < hd; i += 64) dst[i] = (f16_t)(float)src[i];
        return;
    }
    const bool isq = hh < n_q;
    T* x = isq ? q + (row * n_q + hh) * (uint64_t)hd : k + row * kv_dim + (uint64_t)(hh - n_q) * hd;
    const float* w = isq ? qw : kw;
    f16_t* kc = nullptr;
    if (!isq && k_cache) {
        if (!cache_ok && lane == 0 && hh == n_q) atomicOr(fault, APK_FAULT_CACHE_RANGE);
        kc = cache_ok ? k_cache + p * kv_dim + (uint64_t)(hh - n_q) * hd : nullptr;
    }
    typename headstat<T>::scale_t scale{};
    if (w) {
        acc_t ss = 0;
        for (int i = lane; i < hd; i += 64) ss = headstat<T>::sq(ss, (float)x[i]);
        ss = group_sum<64>(ss);  // every lane's loads are consumed here, before any store below
        scale = headstat<T>::rscale(ss, hd, eps);
    }
    const float posf = (float)p;
    for (int i = lane; i < rot_half; i += 64) {
        const int ia = norm_style ? 2 * i : i, ib = norm_style ? 2 * i + 1 : i + rot_half;
        float a = (float)x[ia], b = (float)x[ib];
        if (w) {
            a = headstat<T>::apply(a, scale, w[ia]);
            b = headstat<T>::apply(b, scale, w[ib]);
        }
        double sd, cd;
        sincos((double)(posf * inv_freq[i]), &sd, &cd);  // one f32 rounding of the angle, as the reference
        const float sn = (float)sd, cs = (float)cd;
        const T oa = (T)(a * cs - b * sn), ob = (T)(a * sn + b * cs);
        x[ia] = oa;
        x[ib] = ob;
        if (kc) {
            kc[ia] = (f16_t)(float)oa;
            kc[ib] = (f16_t)(float)ob;
        }
    }
    for (int i = 2 * rot_half + lane; i < hd; i += 64) {  // channels past the rotary width: normalised, not rotated
        const T o = w ? (T)headstat<T>::apply((float)x[i], scale, w[i]) : x[i];
        if (w) x[i] = o;
        if (kc) kc[i] = (f16_t)(float)o;
    }
}
extern "C" __global__ __launch_bounds__(256) void apk_qknorm_rope_pos_f32(
    float* q, float* k, const float* v, const float* qw, const float* kw, const uint32_t* pos, const float* inv_freq,
    f16_t* k_cache, f16_t* v_cache, uint32_t capacity, int rows, int n_q, int n_kv, int hd, int rot_half, int norm_style,
    float eps, uint32_t* fault) {
    qknorm_rope_pos_body<float>(q, k, v, qw, kw, pos, inv_freq, k_cache, v_cache, capacity, rows, n_q, n_kv, hd, rot_half,
                                norm_style, eps, fault);
}
extern "C" __global__ __launch_bounds__(256) void apk_qknorm_rope_pos_f16(
    f16_t* q, f16_t* k, const f16_t* v, const float* qw, const float* kw, const uint32_t* pos, const float* inv_freq,
    f16_t* k_cache, f16_t* v_cache, uint32_t capacity, int rows, int n_q, int n_kv, int hd, int rot_half, int norm_style,
    float eps, uint32_t* fault) {
    qknorm_rope_pos_body<f16_t>(q, k, v, qw, kw, pos, inv_freq, k_cache, v_cache, capacity, rows, n_q, n_kv, hd, rot_half,
                                norm_style, eps, fault);
}

// Layer prologue for small decode batches: the residual add + RMSNorm of the hidden
// rows and the QK-norm + RoPE of the q/k rows as ONE launch.  They are two independent
// jobs sharing a grid (workgroups [0, rows) normalise one hidden row each, the rest
// own 8-head groups of q/k); in a layer a QKV projection sits between them, so this
// removes a launch, not a pass over memory.  One tile per lane (NCH = 1), one pass per
// wave (ITER = 1): the shapes where launch latency, not bandwidth, is the cost.
#define APK_PROLOGUE(T, TN, HD)                                                                                   \
    extern "C" __global__ __launch_bounds__(1024) void apk_layer_prologue_##TN##_hd##HD(                         \
        T* x, const T* delta, T* h, const float* gamma, int n, T* q, T* k, const float* qw, const float* kw,     \
        const float* rope, int rows, int n_q, int n_kv, float eps) {                                             \
        if (blockIdx.x < (uint32_t)rows) add_rmsnorm_body<T, 1>(x, delta, h, gamma, n, eps, blockIdx.x);         \
        else qknorm_rope_body<T, HD, 1>(q, k, qw, kw, rope, rows, n_q, n_kv, eps, HD, blockIdx.x - (uint32_t)rows);  \
    }
APK_PROLOGUE(float, f32, 64) APK_PROLOGUE(float, f32, 128) APK_PROLOGUE(float, f32, 256)
APK_PROLOGUE(f16_t, f16, 64) APK_PROLOGUE(f16_t, f16, 128) APK_PROLOGUE(f16_t, f16, 256)

// RoPE table rows from per-row positions (rope.rs:18-22, session.rs:34-50):
// table[r][i] = [sin, cos]((pos[r] as f32) * inv_freq[i]).  One f32 rounding of
// the angle, as the reference; then sine and cosine of that f32 angle in double
// precision, rounded once to f32: the correctly rounded values, which is what the
// reference's libm returns in all but rare cases -- a 2-ulp sincosf here would
// show as 1e-5 in rotated outputs that nearly cancel.  (The table is rows*half
// values: the cost of the double evaluation does not register.)
extern "C" __global__ __launch_bounds__(256) void apk_rope_table(const uint32_t* pos, const float* inv_freq, int rows,
                                                                int half, float* table) {
    const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (uint64_t)rows * half) return;
    const float ang = (float)pos[i / half] * inv_freq[i % half];
    double s, c;
    sincos((double)ang, &s, &c);
    table[2 * i] = (float)s;
    table[2 * i + 1] = (float)c;
}
