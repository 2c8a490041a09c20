// gfx950 device code, part of apk_kernels.hip (one translation unit, one code object): embedding rows: dequant + gather, all ten formats.
#pragma once

// =========================================================================
// Embedding rows: out[t, :] = dequant(table row ids[t])   (quantmat/mod.rs:75-89)
// The dequant is fused into the gather; the id is read on the device.
// An id >= vocab raises APK_FAULT_TOKEN_RANGE and leaves its row untouched.
// =========================================================================
// Q4_K (dequant.rs:211-231): 144-byte super-block = d, dmin (f16), 12 packed
// scale bytes, 128 quant bytes -> 256 outputs.  d*sc, dmin*mn, (d*sc)*q and the
// subtraction are four separately rounded f32 operations.
// One workgroup per output row; 8 lanes share a super-block and are laid out so
// that EVERY store instruction writes one full, contiguous 128-byte line per
// super-block (partial-line streaming stores cost more than 2x here):
//   fp16 out: store k (0..3) of lane L covers outputs [64k + 8L, +8): sub-block
//             2k + L/4, i.e. quant bytes qs[32k + 8(L%4), +8), low nibbles for
//             L < 4 and high nibbles for L >= 4;
//   f32 out : store k (0..7) of lane L covers outputs [32k + 4L, +4): sub-block k,
//             quant bytes qs[32(k/2) + 4L, +4), low nibbles for even k.
DEV void k4_scale_min(const u32x4 hdr, int s, float& sc, float& mn) {
    // the 12 packed bytes are hdr.y, hdr.z, hdr.w (little endian); scale_min_k4, allpaka-dtype lib.rs:382-390
    auto byte_at = [&](int i) -> uint32_t {
        uint32_t w = i < 4 ? hdr.y : (i < 8 ? hdr.z : hdr.w);
        return (w >> (8 * (i & 3))) & 0xffu;
    };
    uint32_t a, b;
    if (s < 4) {
        a = byte_at(s) & 63u;
        b = byte_at(s + 4) & 63u;
    } else {
        a = (byte_at(s + 4) & 0xfu) | ((byte_at(s - 4) >> 6) << 4);
        b = (byte_at(s + 4) >> 4) | ((byte_at(s) >> 6) << 4);
    }
    sc = (float)a;
    mn = (float)b;
}

// The embedding multiplier of models that scale their token embeddings (`*v *= embed_scale`
// after the dequant, only when it is not 1: model/prefill.rs:107-109, model/decode.rs:427-429).
template <int N> DEV void embed_scale(float* v, float scale) {
    // compared as bits: as floats the compiler drops the test (v * 1.0f == v) and multiplies every time
    if (__builtin_bit_cast(uint32_t, scale) != 0x3f800000u) {
#pragma unroll
        for (int i = 0; i < N; i++) v[i] *= scale;
    }
}

template <typename TO>
DEV void embed_q4k_body(const uint8_t* table, uint32_t vocab, int n_in, const uint32_t* ids, TO* out, uint32_t* fault,
                        float scale, uint32_t row0) {
    const int nsb = n_in / 256;
    const uint64_t t = blockIdx.x;
    const uint32_t id = ids ? ids[t] : row0 + (uint32_t)t;  // no id list: the rows row0, row0 + 1, ...
    if (id >= vocab) {
        if (threadIdx.x == 0) atomicOr(fault, APK_FAULT_TOKEN_RANGE);
        return;
    }
    const uint8_t* row = table + (uint64_t)id * ((uint64_t)nsb * 144);
    TO* orow = out + t * (uint64_t)n_in;
    for (int rem = threadIdx.x; rem < nsb * 8; rem += blockDim.x) {
        const int sb = rem >> 3, L = rem & 7;
        const uint8_t* blk = row + (uint64_t)sb * 144;
        const u32x4 hdr = *(const u32x4*)blk;
        const float d = h2f(hdr.x & 0xffffu), dmin = h2f(hdr.x >> 16);
        if constexpr (sizeof(TO) == 2) {
            u32x2 qs[4];
#pragma unroll
            for (int k = 0; k < 4; k++) qs[k] = *(const u32x2*)(blk + 16 + k * 32 + (L & 3) * 8);
            const int hi = L >> 2;
#pragma unroll
            for (int k = 0; k < 4; k++) {
                float sc, mn;
                k4_scale_min(hdr, 2 * k + hi, sc, mn);
                const float dl = d * sc, ml = dmin * mn;
                float v[8];
#pragma unroll
                for (int w = 0; w < 2; w++)
#pragma unroll
                    for (int b = 0; b < 4; b++) {
                        const uint32_t byte = (qs[k][w] >> (8 * b)) & 0xffu;
                        const uint32_t qv = hi ? (byte >> 4) : (byte & 0xfu);
                        v[4 * w + b] = dl * (float)qv - ml;
                    }
                embed_scale<8>(v, scale);
                io<f16_t>::store_nt((f16_t*)orow + (uint64_t)sb * 256 + k * 64 + L * 8, v);
            }
        } else {
            uint32_t qs[4];
#pragma unroll
            for (int pr = 0; pr < 4; pr++) qs[pr] = *(const uint32_t*)(blk + 16 + pr * 32 + L * 4);
#pragma unroll
            for (int k = 0; k < 8; k++) {
                float sc, mn;
                k4_scale_min(hdr, k, sc, mn);
                const float dl = d * sc, ml = dmin * mn;
                float v[4];
#pragma unroll
                for (int b = 0; b < 4; b++) {
                    const uint32_t byte = (qs[k >> 1] >> (8 * b)) & 0xffu;
                    const uint32_t qv = (k & 1) ? (byte >> 4) : (byte & 0xfu);
                    v[b] = dl * (float)qv - ml;
                }
                embed_scale<4>(v, scale);
                io<float>::store_nt((float*)orow + (uint64_t)sb * 256 + k * 32 + L * 4, v);
            }
        }
    }
}
extern "C" __global__ __launch_bounds__(256) void apk_embed_q4k_f32(const uint8_t* table, uint32_t vocab, int n_in,
                                                                   const uint32_t* ids, float* out, uint32_t* fault,
                                                                   float scale, uint32_t row0) {
    embed_q4k_body<float>(table, vocab, n_in, ids, out, fault, scale, row0);
}
extern "C" __global__ __launch_bounds__(256) void apk_embed_q4k_f16(const uint8_t* table, uint32_t vocab, int n_in,
                                                                   const uint32_t* ids, f16_t* out, uint32_t* fault,
                                                                   float scale, uint32_t row0) {
    embed_q4k_body<f16_t>(table, vocab, n_in, ids, out, fault, scale, row0);
}

// ---- formats decoded straight from global memory -------------------------------------
// A lane owns one 16-byte output tile (N = 8 fp16 / 4 f32 consecutive outputs): it reads what
// the tile needs -- the block's scale fields and its own N quants -- with a few small loads
// (2-byte-aligned vector loads where blocks are only 2-byte aligned: the hardware takes
// unaligned global addresses), and consecutive lanes write consecutive tiles: no staging, no
// barrier, every store instruction covers whole lines.  Tiles are numbered across the batch.
typedef u32x2 __attribute__((aligned(2))) u32x2_a2;
typedef uint32_t __attribute__((aligned(2))) u32_a2;
template <int N> struct qbytes;  // N consecutive bytes at a 2-byte-aligned address
template <> struct qbytes<8> {
    u32x2 v;
    DEV qbytes<8> at(const uint8_t* p) { return qbytes<8>{*(const u32x2_a2*)p}; }
    DEV uint32_t byte(const qbytes<8>& q, int i) { return (q.v[i >> 2] >> (8 * (i & 3))) & 0xffu; }
    DEV uint32_t word(const qbytes<8>& q, int w) { return q.v[w]; }  // bytes 4w .. 4w+3
};
template <> struct qbytes<4> {
    uint32_t v;
    DEV qbytes<4> at(const uint8_t* p) { return qbytes<4>{*(const u32_a2*)p}; }
    DEV uint32_t byte(const qbytes<4>& q, int i) { return (q.v >> (8 * i)) & 0xffu; }
    DEV uint32_t word(const qbytes<4>& q, int) { return q.v; }
};
// The four bytes of a word as floats (each a single byte-to-float conversion of the hardware).
DEV void bytes_to_f32(uint32_t w, float* f) {
    f[0] = (float)(w & 0xffu);
    f[1] = (float)((w >> 8) & 0xffu);
    f[2] = (float)((w >> 16) & 0xffu);
    f[3] = (float)(w >> 24);
}
template <int FMT> struct dqd;  // tile<N>(row, e0, o): outputs e0 .. e0+N-1 of the row, e0 a multiple of N
template <> struct dqd<3> {     // Q8_0 (dequant.rs:94-126): 34-byte block = f16 scale + 32 int8; out = d * q
    static constexpr int BE = 32, BB = 34;
    template <int N> DEV void tile(const uint8_t* row, uint32_t e0, float* o) {
        const uint8_t* b = row + (uint64_t)(e0 >> 5) * 34;
        const float d = h2f(*(const uint16_t*)b);
        const qbytes<N> q = qbytes<N>::at(b + 2 + (e0 & 31u));
#pragma unroll
        for (int i = 0; i < N; i++) o[i] = d * (float)(int8_t)qbytes<N>::byte(q, i);
    }
};
template <> struct dqd<6> {  // Q5_0 (dequant.rs:131-141): d, qh (32 fifth bits), qs[16]; out = d * ((nibble | bit << 4) - 16)
    static constexpr int BE = 32, BB = 22;
    template <int N> DEV void tile(const uint8_t* row, uint32_t e0, float* o) {
        const uint8_t* b = row + (uint64_t)(e0 >> 5) * 22;
        const int e = (int)(e0 & 31u);
        const float d = h2f(*(const uint16_t*)b);
        const uint32_t qh = *(const u32_a2*)(b + 2);
        const qbytes<N> qs = qbytes<N>::at(b + 6 + (e & 15));
#pragma unroll
        for (int i = 0; i < N; i++) {
            const uint32_t byte = qbytes<N>::byte(qs, i);
            const uint32_t nib = e < 16 ? (byte & 0xfu) : (byte >> 4);
            const uint32_t hb = (qh >> (e + i)) & 1u;
            o[i] = d * (float)((int)(nib | (hb << 4)) - 16);
        }
    }
};
template <> struct dqd<4> {  // Q2_K (dequant.rs:150-174): scales[16] qs[64] d dmin; out = (d*sc)*q - dmin*mn
    static constexpr int BE = 256, BB = 84;
    template <int N> DEV void tile(const uint8_t* row, uint32_t e0, float* o) {
        const uint8_t* b = row + (uint64_t)(e0 >> 8) * 84;
        const int e = (int)(e0 & 255u), half = e >> 7, r = e & 127, si = r >> 5, within = r & 31, group = within >> 4,
                  l0 = within & 15;
        const uint32_t sc = b[half * 8 + si * 2 + group];
        const uint32_t dd = *(const u32_a2*)(b + 80);
        const float dl = h2f(dd & 0xffffu) * (float)(sc & 0xfu), ml = h2f(dd >> 16) * (float)(sc >> 4);
        const qbytes<N> qs = qbytes<N>::at(b + 16 + half * 32 + group * 16 + l0);
#pragma unroll
        for (int w = 0; w < N / 4; w++) {  // four 2-bit quants at a time, in the bytes of one word
            float f[4];
            bytes_to_f32((qbytes<N>::word(qs, w) >> (2 * si)) & 0x03030303u, f);
#pragma unroll
            for (int i = 0; i < 4; i++) o[4 * w + i] = dl * f[i] - ml;
        }
    }
};
template <> struct dqd<5> {  // Q3_K (dequant.rs:176-204; scales: allpaka-dtype lib.rs:395-422): hmask[32] qs[64] scales[12] d
    static constexpr int BE = 256, BB = 110;
    template <int N> DEV void tile(const uint8_t* row, uint32_t e0, float* o) {
        const uint8_t* b = row + (uint64_t)(e0 >> 8) * 110;
        const int e = (int)(e0 & 255u), half = e >> 7, r = e & 127, si = r >> 5, within = r & 31, group = within >> 4,
                  l0 = within & 15;
        const int is = half * 8 + si * 2 + group;
        const uint8_t* pk = b + 96;
        const uint32_t lo = is < 8 ? (pk[is] & 0xfu) : (uint32_t)(pk[is - 8] >> 4);
        const uint32_t hi = (pk[8 + (is & 3)] >> (2 * (is >> 2))) & 3u;
        const float dl = h2f(*(const uint16_t*)(b + 108)) * (float)((int)(int8_t)(lo | (hi << 4)) - 32);
        const int idx0 = group * 16 + l0;
        const qbytes<N> hm = qbytes<N>::at(b + idx0);
        const qbytes<N> qs = qbytes<N>::at(b + 32 + half * 32 + idx0);
        // four quants at a time, in the bytes of one word: the two low bits | the mask bit << 2 = 0 .. 7, which is
        // the reference's (low bits - (mask bit ? 0 : 4)) plus 4
        const int mbit = half * 4 + si;
#pragma unroll
        for (int w = 0; w < N / 4; w++) {
            const uint32_t low = (qbytes<N>::word(qs, w) >> (2 * si)) & 0x03030303u;
            const uint32_t top = (qbytes<N>::word(hm, w) >> mbit) & 0x01010101u;
            float f[4];
            bytes_to_f32(low | (top << 2), f);
#pragma unroll
            for (int i = 0; i < 4; i++) o[4 * w + i] = dl * (f[i] - 4.0f);
        }
    }
};
template <> struct dqd<1> {  // Q5_K (dequant.rs:238-263): d dmin scales[12] qh[32] qs[128]; out = (d*sc)*(q4 + 16*bit) - dmin*mn
    static constexpr int BE = 256, BB = 176;
    template <int N> DEV void tile(const uint8_t* row, uint32_t e0, float* o) {
        const uint8_t* b = row + (uint64_t)(e0 >> 8) * 176;  // 176 = 11 * 16: blocks are 16-byte aligned
        const int e = (int)(e0 & 255u), pair = e >> 6, r = e & 63, hn = r >> 5, l0 = r & 31, sub = 2 * pair + hn;
        const u32x4 hdr = *(const u32x4*)b;  // d, dmin and the 12 packed scale bytes, as in Q4_K
        const qbytes<N> qs = qbytes<N>::at(b + 48 + pair * 32 + l0);
        const qbytes<N> qh = qbytes<N>::at(b + 16 + l0);
        float sc, mn;
        k4_scale_min(hdr, sub, sc, mn);
        const float dsc = h2f(hdr.x & 0xffffu) * sc, dm = h2f(hdr.x >> 16) * mn;
#pragma unroll
        for (int w = 0; w < N / 4; w++) {  // four quants at a time, in the bytes of one word: nibble | fifth bit << 4
            const uint32_t lo = qbytes<N>::word(qs, w);
            const uint32_t nib = (hn ? lo >> 4 : lo) & 0x0f0f0f0fu;
            const uint32_t top = (qbytes<N>::word(qh, w) >> sub) & 0x01010101u;
            float f[4];
            bytes_to_f32(nib | (top << 4), f);
#pragma unroll
            for (int i = 0; i < 4; i++) o[4 * w + i] = dsc * f[i] - dm;
        }
    }
};
template <> struct dqd<2> {  // Q6_K (dequant.rs:271-295): ql[128] qh[64] scales[16] d; out = (d * scale) * q
    static constexpr int BE = 256, BB = 210;
    template <int N> DEV void tile(const uint8_t* row, uint32_t e0, float* o) {
        const uint8_t* b = row + (uint64_t)(e0 >> 8) * 210;
        const int e = (int)(e0 & 255u), half = e >> 7, r = e & 127, quarter = r >> 5, l0 = r & 31, is = l0 >> 4;
        const qbytes<N> ql = qbytes<N>::at(b + half * 64 + (quarter & 1) * 32 + l0);
        const qbytes<N> qh = qbytes<N>::at(b + 128 + half * 32 + l0);
        const float sc = (float)(int8_t)b[192 + half * 8 + is + 2 * quarter];
        const float dl = h2f(*(const uint16_t*)(b + 208)) * sc;
        // four quants at a time, in the bytes of one word: low nibbles | high bit pairs << 4 = 0 .. 63; the
        // reference's (q as i8 - 32) as f32 is that byte as a float minus 32 (both exact)
#pragma unroll
        for (int w = 0; w < N / 4; w++) {
            const uint32_t lo = qbytes<N>::word(ql, w);
            const uint32_t nib = (quarter < 2 ? lo : lo >> 4) & 0x0f0f0f0fu;
            const uint32_t q4 = nib | (((qbytes<N>::word(qh, w) >> (2 * quarter)) & 0x03030303u) << 4);
            float f[4];
            bytes_to_f32(q4, f);
#pragma unroll
            for (int i = 0; i < 4; i++) o[4 * w + i] = dl * (f[i] - 32.0f);
        }
    }
};
template <> struct dqd<8> {  // F32
    static constexpr int BE = 1, BB = 4;
    template <int N> DEV void tile(const uint8_t* row, uint32_t e0, float* o) {
#pragma unroll
        for (int i = 0; i < N; i += 4) io<float>::load_nt((const float*)(row + 4 * (uint64_t)e0) + i, o + i);
    }
};
#define APK_EMBED_UNR 4  // tiles per lane: the quants of all of them in flight before the first store
// Workgroup w serves row w / chunks, tiles [chunk * blockDim * UNR, +blockDim * UNR) of it: the row
// number and the token id are uniform for the workgroup (scalar loads, no per-lane division).
template <int FMT, typename TO>
DEV void embed_direct_body(const uint8_t* table, uint32_t vocab, int n_in, const uint32_t* ids, uint32_t chunks, TO* out,
                           uint32_t* fault, float scale, uint32_t row0) {
    constexpr int OPT = io<TO>::VEC;  // outputs per tile
    const uint32_t tiles_per_row = (uint32_t)n_in / OPT;
    const uint32_t t = blockIdx.x / chunks, chunk = blockIdx.x - t * chunks;
    const uint32_t id = ids ? ids[t] : row0 + (uint32_t)t;  // no id list: the rows row0, row0 + 1, ...
    if (id >= vocab) {  // uniform
        if (threadIdx.x == 0 && chunk == 0) atomicOr(fault, APK_FAULT_TOKEN_RANGE);
        return;
    }
    const uint8_t* row = table + (uint64_t)id * ((uint64_t)(n_in / dqd<FMT>::BE) * dqd<FMT>::BB);
    const uint32_t first = chunk * (blockDim.x * APK_EMBED_UNR) + threadIdx.x;
    float o[APK_EMBED_UNR][OPT];
#pragma unroll
    for (int u = 0; u < APK_EMBED_UNR; u++) {
        // a lane past the end of the row re-reads its last tile and stores nothing
        const uint32_t tile = min(first + (uint32_t)u * blockDim.x, tiles_per_row - 1u);
        dqd<FMT>::template tile<OPT>(row, tile * OPT, o[u]);
    }
    TO* orow = out + (uint64_t)t * n_in;
#pragma unroll
    for (int u = 0; u < APK_EMBED_UNR; u++) {
        const uint32_t tile = first + (uint32_t)u * blockDim.x;
        if (tile < tiles_per_row) {
            embed_scale<OPT>(o[u], scale);
            io<TO>::store_nt(orow + (uint64_t)tile * OPT, o[u]);
        }
    }
}
// The same for the 256-element super-block formats, with the lane layout of the Q4_K kernel: 8
// lanes per super-block, lane L owning tiles 8k + L of it (k = 0 .. 3 for fp16 output, 0 .. 7 for
// f32): the super-block's header and scale fields are fetched once per lane for all its tiles
// (the compiler merges the identical loads), and for every k the 8 lanes write one whole line.
// Super-blocks are numbered across the batch (lane j of the launch serves super-block j / 8, of row (j / 8) / nsb), so
// that a row whose super-blocks do not fill whole waves (5120 columns: 160 lanes) leaves no lane idle: the row
// number and the token id are per lane (one division; the id loads of a wave hit one or two words).
template <int FMT, typename TO>
DEV void embed_direct_sb_body(const uint8_t* __restrict__ table, uint32_t vocab, int n_in, const uint32_t* __restrict__ ids,
                              uint32_t rows, TO* __restrict__ out, uint32_t* fault, float scale, uint32_t row0) {
    constexpr int OPT = io<TO>::VEC, K = 256 / OPT / 8;
    const uint32_t nsb = (uint32_t)n_in / 256;
    const uint64_t j = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const uint32_t L = (uint32_t)j & 7u;
    const uint32_t total = rows * nsb;  // the host keeps the batch's super-blocks below 2^32
    const bool inside = (j >> 3) < total;
    const uint32_t sbc = inside ? (uint32_t)(j >> 3) : total - 1u;  // a lane past the last super-block re-reads it and stores nothing
    const uint32_t t = sbc / nsb, sb = sbc - t * nsb;
    const uint32_t id = ids ? ids[t] : row0 + t;  // no id list: the rows row0, row0 + 1, ...
    const bool ok = id < vocab;
    if (!ok && inside && sb == 0 && L == 0) atomicOr(fault, APK_FAULT_TOKEN_RANGE);
    const uint8_t* row = table + (uint64_t)(ok ? id : 0u) * ((uint64_t)nsb * dqd<FMT>::BB);  // a bad id reads row 0 and stores nothing
    float o[K][OPT];
#pragma unroll
    for (int k = 0; k < K; k++) dqd<FMT>::template tile<OPT>(row, sb * 256u + (8u * k + L) * OPT, o[k]);
    if (!inside || !ok) return;
    TO* orow = out + (uint64_t)t * n_in + (uint64_t)sb * 256;
#pragma unroll
    for (int k = 0; k < K; k++) {
        embed_scale<OPT>(o[k], scale);
        io<TO>::store_nt(orow + (8 * k + L) * OPT, o[k]);
    }
}
#define APK_EMBED_DIRECT_SB(NAME, FMT)                                                                                   \
    extern "C" __global__ __launch_bounds__(256) void apk_embed_##NAME##_f32(                                            \
        const uint8_t* table, uint32_t vocab, int n_in, const uint32_t* ids, uint32_t rows, float* out, uint32_t* fault, \
        float scale, uint32_t row0) {                                                                                    \
        embed_direct_sb_body<FMT, float>(table, vocab, n_in, ids, rows, out, fault, scale, row0);                        \
    }                                                                                                                    \
    extern "C" __global__ __launch_bounds__(256) void apk_embed_##NAME##_f16(                                            \
        const uint8_t* table, uint32_t vocab, int n_in, const uint32_t* ids, uint32_t rows, f16_t* out, uint32_t* fault, \
        float scale, uint32_t row0) {                                                                                    \
        embed_direct_sb_body<FMT, f16_t>(table, vocab, n_in, ids, rows, out, fault, scale, row0);                        \
    }
APK_EMBED_DIRECT_SB(q6k, 2) APK_EMBED_DIRECT_SB(q5k, 1) APK_EMBED_DIRECT_SB(q2k, 4) APK_EMBED_DIRECT_SB(q3k, 5)

#define APK_EMBED_DIRECT(NAME, FMT)                                                                                      \
    extern "C" __global__ __launch_bounds__(256) void apk_embed_##NAME##_f32(                                            \
        const uint8_t* table, uint32_t vocab, int n_in, const uint32_t* ids, uint32_t chunks, float* out, uint32_t* fault, \
        float scale, uint32_t row0) {                                                                                    \
        embed_direct_body<FMT, float>(table, vocab, n_in, ids, chunks, out, fault, scale, row0);                         \
    }                                                                                                                    \
    extern "C" __global__ __launch_bounds__(256) void apk_embed_##NAME##_f16(                                            \
        const uint8_t* table, uint32_t vocab, int n_in, const uint32_t* ids, uint32_t chunks, f16_t* out, uint32_t* fault, \
        float scale, uint32_t row0) {                                                                                    \
        embed_direct_body<FMT, f16_t>(table, vocab, n_in, ids, chunks, out, fault, scale, row0);                         \
    }
APK_EMBED_DIRECT(q8_0, 3) APK_EMBED_DIRECT(q5_0, 6) APK_EMBED_DIRECT(f32, 8)

// ---- the other GGUF formats of the unified dequant codes (gpu/common.rs:47-61) -------
// One element decoder per format, a restatement of its block function in
// crates/allpaka-gguf/src/dequant.rs with the same operation order (bit-exact), reading
// the block's bytes from LDS.  `e` is the element index inside the block.
DEV float lds_f16(const uint8_t* p) { return h2f(*(const uint16_t*)p); }  // blocks are 2-byte aligned

template <int FMT> struct dq;
template <> struct dq<7> {  // F16
    static constexpr int BE = 1, BB = 2;
    DEV float elem(const uint8_t* b, int) { return lds_f16(b); }
};
template <> struct dq<9> {  // BF16, allpaka-dtype lib.rs:188-190
    static constexpr int BE = 1, BB = 2;
    DEV float elem(const uint8_t* b, int) { return __builtin_bit_cast(float, (uint32_t)(*(const uint16_t*)b) << 16); }
};
// One workgroup per row: the row's bytes are staged in LDS with 16-byte loads (from the
// aligned address at or below the row start; rows of these formats are not 16-byte
// multiples), then each lane decodes one 16-byte output tile per pass, consecutive lanes
// writing consecutive tiles.
template <int FMT, typename TO>
DEV void embed_staged_body(const uint8_t* table, uint64_t table_bytes, uint32_t vocab, int n_in, const uint32_t* ids,
                           TO* out, uint32_t* fault, float scale, uint32_t row0) {
    extern __shared__ __attribute__((aligned(16))) uint8_t stage[];
    constexpr int OPT = io<TO>::VEC, BE = dq<FMT>::BE, BB = dq<FMT>::BB;
    const uint64_t t = blockIdx.x;
    const uint32_t id = ids ? ids[t] : row0 + (uint32_t)t;  // no id list: the rows row0, row0 + 1, ...
    if (id >= vocab) {
        if (threadIdx.x == 0) atomicOr(fault, APK_FAULT_TOKEN_RANGE);
        return;
    }
    const uint64_t row_bytes = (uint64_t)(n_in / BE) * BB;
    const uint64_t start = (uint64_t)id * row_bytes;
    const uint64_t astart = start & ~(uint64_t)15;  // table base is 16-byte aligned
    const int mis = (int)(start - astart);
    const int nvec = (int)((mis + row_bytes + 15) / 16);
    for (int i = threadIdx.x; i < nvec; i += blockDim.x) {
        const uint64_t off = astart + (uint64_t)i * 16;
        u32x4 v;
        if (off + 16 <= table_bytes) {
            v = __builtin_nontemporal_load((const u32x4*)(table + off));
        } else {  // last tile of the last row: stay inside the table
            uint32_t w[4] = {0, 0, 0, 0};
            for (int b = 0; b < 16; b++)
                if (off + b < table_bytes) w[b >> 2] |= (uint32_t)table[off + b] << (8 * (b & 3));
            v = u32x4{w[0], w[1], w[2], w[3]};
        }
        *(u32x4*)(stage + i * 16) = v;
    }
    __syncthreads();
    const int ntiles = n_in / OPT;  // the host admits only n_in that are whole tiles
    for (int g = threadIdx.x; g < ntiles; g += blockDim.x) {
        const int e0 = g * OPT;
        float o[OPT];
#pragma unroll
        for (int i = 0; i < OPT; i++) {
            const int e = e0 + i;
            o[i] = dq<FMT>::elem(stage + mis + (e / BE) * BB, e % BE);
        }
        embed_scale<OPT>(o, scale);
        io<TO>::store_nt(out + t * (uint64_t)n_in + e0, o);
    }
}
#define APK_EMBED_GEN(NAME, FMT)                                                                                         \
    extern "C" __global__ __launch_bounds__(256) void apk_embed_##NAME##_f32(                                            \
        const uint8_t* table, uint64_t table_bytes, uint32_t vocab, int n_in, const uint32_t* ids, float* out,           \
        uint32_t* fault, float scale, uint32_t row0) {                                                                   \
        embed_staged_body<FMT, float>(table, table_bytes, vocab, n_in, ids, out, fault, scale, row0);                    \
    }                                                                                                                    \
    extern "C" __global__ __launch_bounds__(256) void apk_embed_##NAME##_f16(                                            \
        const uint8_t* table, uint64_t table_bytes, uint32_t vocab, int n_in, const uint32_t* ids, f16_t* out,           \
        uint32_t* fault, float scale, uint32_t row0) {                                                                   \
        embed_staged_body<FMT, f16_t>(table, table_bytes, vocab, n_in, ids, out, fault, scale, row0);                    \
    }
APK_EMBED_GEN(f16, 7) APK_EMBED_GEN(bf16, 9)  // (measured faster staged than decoded in place)
