// gfx950 device code, part of apk_kernels.hip (one translation unit, one code object): types, 16-byte tile loads and stores, wave reductions.
#pragma once

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16_t;
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

#define DEV static __device__ __forceinline__

// Fault bits raised through the context's device status word.
#define APK_FAULT_TOKEN_RANGE 1u   // embedding id >= vocab
#define APK_FAULT_EXPERT_RANGE 2u  // routed expert id >= n_expert
#define APK_FAULT_ROW_RANGE 4u     // gather index >= source rows
#define APK_FAULT_CACHE_RANGE 8u   // KV-cache position >= capacity

DEV float h2f(uint32_t bits16) { return (float)__builtin_bit_cast(f16_t, (uint16_t)bits16); }

// ----------------------------------------------------------- 16-byte tile IO
// Two kinds of streaming store.  nt_store: non-temporal (the compiler's builtin).  wt_store: non-temporal and written
// through at device scope (the sc1 bit).  An nt-only store leaves its line dirty in the XCD's L2, and what a launch
// left dirty is written back when the kernel ends, after its last wave; a written-through store has nothing left to
// write back but completes later, and a wave holds its registers until its stores complete.  Measured per kernel:
// short waves at full occupancy gain (one-tile-per-lane copy of 75 MB in place: 13.9 -> 12.9 us; SwiGLU on
// [8192 x 768] f32: 14.0 -> 13.65; QK-norm + RoPE: 13.8 -> 13.5), long waves at low occupancy lose (add + RMSNorm with
// a wave per row: 14.4 -> 16.4; the embedding gathers 5.3 -> 5.7), so each kernel family names the kind it takes.
// The compiler has no builtin for the bit, so the instruction is written out; the s_nop covers the two wait
// states this part needs between a store of more than 8 bytes and a VALU write to its data registers, which the
// compiler cannot insert for an instruction it does not see.  No kernel reads back what it stores this way, so the
// statement needs no memory clobber (the stored value depends on every load it must follow).
DEV void wt_store(u32x4 v, void* p) { asm volatile("global_store_dwordx4 %0, %1, off sc1 nt\n\ts_nop 1" ::"v"(p), "v"(v)); }
DEV void wt_store(f32x4 v, void* p) { wt_store(__builtin_bit_cast(u32x4, v), p); }
DEV void wt_store(u32x2 v, void* p) { asm volatile("global_store_dwordx2 %0, %1, off sc1 nt" ::"v"(p), "v"(v)); }
DEV void nt_store(u32x4 v, void* p) { __builtin_nontemporal_store(v, (u32x4*)p); }
DEV void nt_store(f32x4 v, void* p) { __builtin_nontemporal_store(v, (f32x4*)p); }
DEV void nt_store(u32x2 v, void* p) { __builtin_nontemporal_store(v, (u32x2*)p); }
template <typename T> struct io;
template <> struct io<float> {
    static constexpr int VEC = 4;
    typedef f32x4 raw_t;  // a tile as loaded: kept raw until all loads of a lane are in flight
    DEV raw_t ldraw_nt(const float* p) { return __builtin_nontemporal_load((const f32x4*)p); }
    DEV raw_t zero() { return f32x4{0.f, 0.f, 0.f, 0.f}; }
    DEV void widen(raw_t t, float* v) { v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w; }
    DEV void load(const float* p, float* v) {
        f32x4 t = *(const f32x4*)p;
        v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
    }
    DEV void load_nt(const float* p, float* v) {
        f32x4 t = __builtin_nontemporal_load((const f32x4*)p);
        v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
    }
    DEV void store(float* p, const float* v) {
        f32x4 t = {v[0], v[1], v[2], v[3]};
        *(f32x4*)p = t;
    }
    DEV void store_nt(float* p, const float* v) {
        f32x4 t = {v[0], v[1], v[2], v[3]};
        nt_store(t, p);
    }
    DEV void store_wt(float* p, const float* v) {
        f32x4 t = {v[0], v[1], v[2], v[3]};
        wt_store(t, p);
    }
};
template <> struct io<f16_t> {
    static constexpr int VEC = 8;
    typedef u32x4 raw_t;
    DEV raw_t ldraw_nt(const f16_t* p) { return __builtin_nontemporal_load((const u32x4*)p); }
    DEV raw_t zero() { return u32x4{0u, 0u, 0u, 0u}; }
    DEV void widen(raw_t t, float* v) { unpack(t, v); }
    DEV void unpack(u32x4 t, float* v) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            v[2 * i] = h2f(t[i] & 0xffffu);
            v[2 * i + 1] = h2f(t[i] >> 16);
        }
    }
    DEV u32x4 pack(const float* v) {  // v_cvt_pk_f16_f32: two RNE conversions per instruction
        u32x4 t;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            f32x2 p = {v[2 * i], v[2 * i + 1]};
            t[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(p, f16x2));
        }
        return t;
    }
    DEV void load(const f16_t* p, float* v) { unpack(*(const u32x4*)p, v); }
    DEV void load_nt(const f16_t* p, float* v) { unpack(__builtin_nontemporal_load((const u32x4*)p), v); }
    DEV void store(f16_t* p, const float* v) { *(u32x4*)p = pack(v); }
    DEV void store_nt(f16_t* p, const float* v) { nt_store(pack(v), p); }
    DEV void store_wt(f16_t* p, const float* v) { wt_store(pack(v), p); }
};

// ------------------------------------------------------- wave reductions (DPP)
// Butterfly exchanges inside a 16-lane row as DPP modifiers (no LDS round trip):
// lane^1 and lane^2 by quad permutes, then row_half_mirror (i <-> 7-i) and row_mirror
// (i <-> 15-i): after step s every lane of a 2^s group holds the group's reduction, so
// mirroring pairs each lane with one of the other half-group.  Across rows: readlane.
#define DPP_XOR1 0xB1         // quad_perm:[1,0,3,2]
#define DPP_XOR2 0x4E         // quad_perm:[2,3,0,1]
#define DPP_HALF_MIRROR 0x141 // row_half_mirror
#define DPP_MIRROR 0x140      // row_mirror
template <int CTRL> DEV float dpp_f32(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
template <int CTRL> DEV double dpp_f64(double v) {
    const uint64_t b = __builtin_bit_cast(uint64_t, v);
    const uint32_t lo = (uint32_t)__builtin_amdgcn_mov_dpp((int)(uint32_t)b, CTRL, 0xf, 0xf, true);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_mov_dpp((int)(uint32_t)(b >> 32), CTRL, 0xf, 0xf, true);
    return __builtin_bit_cast(double, ((uint64_t)hi << 32) | lo);
}
template <int CTRL> DEV uint64_t dpp_u64(uint64_t b) {
    const uint32_t lo = (uint32_t)__builtin_amdgcn_mov_dpp((int)(uint32_t)b, CTRL, 0xf, 0xf, true);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_mov_dpp((int)(uint32_t)(b >> 32), CTRL, 0xf, 0xf, true);
    return ((uint64_t)hi << 32) | lo;
}
DEV float dpp_step(float v, int s) {
    return s == 0 ? dpp_f32<DPP_XOR1>(v) : s == 1 ? dpp_f32<DPP_XOR2>(v) : s == 2 ? dpp_f32<DPP_HALF_MIRROR>(v) : dpp_f32<DPP_MIRROR>(v);
}
DEV double dpp_step(double v, int s) {
    return s == 0 ? dpp_f64<DPP_XOR1>(v) : s == 1 ? dpp_f64<DPP_XOR2>(v) : s == 2 ? dpp_f64<DPP_HALF_MIRROR>(v) : dpp_f64<DPP_MIRROR>(v);
}
// The value of lane `lane` (a constant) as a wave-uniform scalar: v_readlane, no LDS round trip.
template <int LANE> DEV float lane_value(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), LANE));
}
template <int LANE> DEV double lane_value(double v) {
    const uint64_t b = __builtin_bit_cast(uint64_t, v);
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)b, LANE);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(b >> 32), LANE);
    return __builtin_bit_cast(double, ((uint64_t)hi << 32) | lo);
}
// Sum over aligned groups of WIDTH lanes (4, 8, 16, 32 or 64); every lane gets the sum.
// Inside a 16-lane row: DPP butterflies.  Across the four rows: each row's sum read as a scalar
// and added as (row0 + row1) + (row2 + row3), the value the xor-16 / xor-32 butterfly gives
// every lane, without its two LDS-crossbar round trips.
template <int WIDTH, typename A> DEV A group_sum(A v) {
#pragma unroll
    for (int s = 0; s < 4; s++)
        if ((1 << (s + 1)) <= WIDTH) v += dpp_step(v, s);
    if constexpr (WIDTH >= 32) {
        const A lo = lane_value<0>(v) + lane_value<16>(v), hi = lane_value<32>(v) + lane_value<48>(v);
        if constexpr (WIDTH >= 64) v = lo + hi;
        else v = (threadIdx.x & 32) ? hi : lo;
    }
    return v;
}

DEV float wave_max_f32(float v) {
#pragma unroll
    for (int s = 0; s < 4; s++) v = fmaxf(v, dpp_step(v, s));
    return fmaxf(fmaxf(lane_value<0>(v), lane_value<16>(v)), fmaxf(lane_value<32>(v), lane_value<48>(v)));
}

// One tile of activations narrowed to fp16 (RNE) for the KV cache: 16 bytes from an
// fp16 tile, 8 bytes from an f32 tile.
template <typename T> DEV void store_f16_tile(f16_t* p, const float* v);
template <> __device__ __forceinline__ void store_f16_tile<f16_t>(f16_t* p, const float* v) { io<f16_t>::store_wt(p, v); }
template <> __device__ __forceinline__ void store_f16_tile<float>(f16_t* p, const float* v) {
    f32x2 lo = {v[0], v[1]}, hi = {v[2], v[3]};
    u32x2 t = {__builtin_bit_cast(uint32_t, __builtin_convertvector(lo, f16x2)),
               __builtin_bit_cast(uint32_t, __builtin_convertvector(hi, f16x2))};
    wt_store(t, p);
}


DEV uint32_t total_order_key(float f) {  // f32::total_cmp as an unsigned key
    int32_t b = __builtin_bit_cast(int32_t, f);
    b ^= (int32_t)(((uint32_t)(b >> 31)) >> 1);
    return (uint32_t)b ^ 0x80000000u;
}
DEV uint32_t dpp_u32(uint32_t v, int s) {
    return s == 0   ? (uint32_t)__builtin_amdgcn_mov_dpp((int)v, DPP_XOR1, 0xf, 0xf, true)
           : s == 1 ? (uint32_t)__builtin_amdgcn_mov_dpp((int)v, DPP_XOR2, 0xf, 0xf, true)
           : s == 2 ? (uint32_t)__builtin_amdgcn_mov_dpp((int)v, DPP_HALF_MIRROR, 0xf, 0xf, true)
                    : (uint32_t)__builtin_amdgcn_mov_dpp((int)v, DPP_MIRROR, 0xf, 0xf, true);
}
DEV uint32_t wave_max_u32(uint32_t v) {  // every lane gets the maximum (a wave-uniform value)
#pragma unroll
    for (int s = 0; s < 4; s++) {
        const uint32_t o = dpp_u32(v, s);
        v = o > v ? o : v;
    }
    const uint32_t a = (uint32_t)__builtin_amdgcn_readlane((int)v, 0), b = (uint32_t)__builtin_amdgcn_readlane((int)v, 16),
                   c = (uint32_t)__builtin_amdgcn_readlane((int)v, 32), d = (uint32_t)__builtin_amdgcn_readlane((int)v, 48);
    const uint32_t ab = a > b ? a : b, cd = c > d ? c : d;
    return ab > cd ? ab : cd;
}
DEV uint64_t max_u64(uint64_t a, uint64_t b) { return a > b ? a : b; }
DEV uint64_t wave_max_u64(uint64_t v) {  // every lane gets the maximum
    v = max_u64(v, dpp_u64<DPP_XOR1>(v));
    v = max_u64(v, dpp_u64<DPP_XOR2>(v));
    v = max_u64(v, dpp_u64<DPP_HALF_MIRROR>(v));
    v = max_u64(v, dpp_u64<DPP_MIRROR>(v));  // uniform inside each 16-lane row
    uint64_t r = 0;
#pragma unroll
    for (int row = 0; row < 4; row++) {
        const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)v, row * 16);
        const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(v >> 32), row * 16);
        r = max_u64(r, ((uint64_t)hi << 32) | lo);
    }
    return r;
}
