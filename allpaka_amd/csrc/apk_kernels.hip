// gfx950 (CDNA4, MI355X) device code for allpaka's fused per-layer ops.
//
// Built with `hipcc --genco --offload-arch=gfx950 -ffp-contract=off` into one
// code object that the host library embeds and loads with hipModuleLoadData.
// Every kernel here is HBM-bound: wave64, 128-bit global accesses, DPP/shuffle
// reductions inside a wave, LDS only for cross-wave sums and byte staging.
// No MFMA: nothing on this path is a contraction.
//
// Arithmetic contract (what the CPU reference computes, op for op):
//   * -ffp-contract=off for the whole file: a*b-c stays two rounded f32 ops,
//     as in the reference's Rust (dequant.rs:221-228, rope.rs:75-80).
//   * RMS statistics are accumulated and applied in f64 (norm.rs:115-187):
//     out = ((x as f64 * scale) as f32) * w.
//   * fp16 activations (a storage form the reference does not have) are
//     widened to f32 on load and rounded once (RNE) on store.
#include <hip/hip_runtime.h>
#include <stdint.h>

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
        __builtin_nontemporal_store(t, (f32x4*)p);
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
    DEV void store_nt(f16_t* p, const float* v) { __builtin_nontemporal_store(pack(v), (u32x4*)p); }
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
template <> __device__ __forceinline__ void store_f16_tile<f16_t>(f16_t* p, const float* v) { io<f16_t>::store_nt(p, v); }
template <> __device__ __forceinline__ void store_f16_tile<float>(f16_t* p, const float* v) {
    f32x2 lo = {v[0], v[1]}, hi = {v[2], v[3]};
    u32x2 t = {__builtin_bit_cast(uint32_t, __builtin_convertvector(lo, f16x2)),
               __builtin_bit_cast(uint32_t, __builtin_convertvector(hi, f16x2))};
    __builtin_nontemporal_store(t, (u32x2*)p);
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

// =========================================================================
// SwiGLU: gate[i] = silu(gate[i]) * up[i], silu(x) = x / (1 + exp(-x))
// (activation.rs:19-22, :116-119).  Pure stream: 2 reads + 1 write / element.
// =========================================================================
template <typename T> DEV float silu_mul(float g, float u);
// f32 activations: exp(-g) by Cody-Waite reduction around the hardware exp2 (log2(e) carried in
// two parts, so the reduced argument is exact to the last bit: about 1 ulp over the whole range,
// where a bare exp2(-g*log2e) loses |g| ulps), then the hardware reciprocal (1 ulp): the result is
// within a few ulp of the reference's g / (1 + exp(-g)) * u -- 1e-6 of the 1e-5 bar -- at a third
// of the instructions of libm expf + IEEE division, which at 32 per element no longer hid behind
// the stream.
template <> __device__ __forceinline__ float silu_mul<float>(float g, float u) {
    const float L2E_HI = 1.44269502162933349609375f, L2E_LO = 1.925963033500011e-08f;  // hi + lo = log2(e)
    const float n = fminf(fmaxf(-g, -104.0f), 89.0f);  // beyond: e underflows to 0 / overflows to inf anyway
    const float k = __builtin_rintf(n * L2E_HI);
    float r = __builtin_fmaf(n, L2E_HI, -k);
    r = __builtin_fmaf(n, L2E_LO, r);
    const float e = __builtin_amdgcn_ldexpf(__builtin_amdgcn_exp2f(r), (int)k);
    // the hardware reciprocal flushes subnormal results: keep 1/(1+e) normal for e up to FLT_MAX by
    // taking it of (1+e) * 2^-32 and applying the 2^-32 after the multiplication by g (all exact)
    const float sc = e > 0x1p96f ? 0x1p-32f : 1.0f;
    return g * __builtin_amdgcn_rcpf((1.0f + e) * sc) * sc * u;  // NaN in g still gives NaN
}
// fp16 activations: the result is rounded to 11 bits, so the hardware exp2 /
// rcp approximations (about 1 ulp of f32 each) are far inside the 2-ulp-of-fp16
// budget and keep the kernel under its ALU ceiling.
template <> __device__ __forceinline__ float silu_mul<f16_t>(float g, float u) {
    float e = __builtin_amdgcn_exp2f(g * -1.4426950408889634f);
    return g * __builtin_amdgcn_rcpf(1.0f + e) * u;
}

template <typename T, int UNR> DEV void swiglu_body(T* gate, const T* up, uint64_t n) {
    constexpr int VEC = io<T>::VEC;
    const uint64_t nvec = n / VEC;
    const uint64_t base = (uint64_t)blockIdx.x * (blockDim.x * UNR) + threadIdx.x;
    float g[UNR][VEC], u[UNR][VEC];
#pragma unroll
    for (int j = 0; j < UNR; j++) {
        uint64_t c = base + (uint64_t)j * blockDim.x;
        if (c < nvec) {
            io<T>::load_nt(gate + c * VEC, g[j]);
            io<T>::load_nt(up + c * VEC, u[j]);
        }
    }
#pragma unroll
    for (int j = 0; j < UNR; j++) {
        uint64_t c = base + (uint64_t)j * blockDim.x;
        if (c < nvec) {
#pragma unroll
            for (int i = 0; i < VEC; i++) g[j][i] = silu_mul<T>(g[j][i], u[j][i]);
            io<T>::store_nt(gate + c * VEC, g[j]);
        }
    }
    // ragged tail (n not a multiple of the 16-byte tile): last block, scalar
    if (blockIdx.x == gridDim.x - 1) {
        for (uint64_t i = nvec * VEC + threadIdx.x; i < n; i += blockDim.x)
            gate[i] = (T)silu_mul<T>((float)gate[i], (float)up[i]);
    }
}
#define APK_SWIGLU_UNR 1  // measured: 1 tile per lane streams best (most waves in flight)
extern "C" __global__ __launch_bounds__(256) void apk_swiglu_f32(float* gate, const float* up, uint64_t n) {
    swiglu_body<float, APK_SWIGLU_UNR>(gate, up, n);
}
extern "C" __global__ __launch_bounds__(256) void apk_swiglu_f16(f16_t* gate, const f16_t* up, uint64_t n) {
    swiglu_body<f16_t, APK_SWIGLU_UNR>(gate, up, n);
}

// Residual add on its own: a[i] += b[i] (ops::add_assign_slice, blas.rs:105-178), for the
// places where no norm follows.  One 16-byte tile per lane, a scalar tail for ragged n.
template <typename T> DEV void add_assign_body(T* a, const T* b, uint64_t n) {
    constexpr int VEC = io<T>::VEC;
    const uint64_t nvec = n / VEC, c = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (c < nvec) {
        float x[VEC], y[VEC];
        io<T>::load_nt(a + c * VEC, x);
        io<T>::load_nt(b + c * VEC, y);
#pragma unroll
        for (int i = 0; i < VEC; i++) x[i] += y[i];
        io<T>::store_nt(a + c * VEC, x);
    }
    if (blockIdx.x == gridDim.x - 1)
        for (uint64_t i = nvec * VEC + threadIdx.x; i < n; i += blockDim.x) a[i] = (T)((float)a[i] + (float)b[i]);
}
extern "C" __global__ __launch_bounds__(256) void apk_add_assign_f32(float* a, const float* b, uint64_t n) {
    add_assign_body<float>(a, b, n);
}
extern "C" __global__ __launch_bounds__(256) void apk_add_assign_f16(f16_t* a, const f16_t* b, uint64_t n) {
    add_assign_body<f16_t>(a, b, n);
}

// Softmax over rows in place (ops::softmax, activation.rs:5-16): max, exp(v - max), sum,
// times 1/sum.  A wave per row, any row length; the sum runs in lane order, not index order.
extern "C" __global__ __launch_bounds__(256) void apk_softmax_rows(float* x, int rows, int n) {
    const int lane = threadIdx.x & 63;
    const uint64_t r = ((uint64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    if (r >= (uint64_t)rows) return;  // whole wave
    float* row = x + r * (uint64_t)n;
    float mx = -INFINITY;
    for (int i = lane; i < n; i += 64) mx = fmaxf(mx, row[i]);
    mx = wave_max_f32(mx);
    float sum = 0.0f;
    for (int i = lane; i < n; i += 64) {
        const float e = expf(row[i] - mx);
        row[i] = e;
        sum += e;
    }
    sum = group_sum<64>(sum);
    const float inv = 1.0f / sum;
    for (int i = lane; i < n; i += 64) row[i] *= inv;  // each lane re-reads only what it wrote
}

// =========================================================================
// Residual add + RMSNorm over rows (blas.rs:105-178 then norm.rs:193-269):
//   x' = x + delta  (written back when delta != null)
//   h  = ((x' as f64 * scale) as f32) * gamma,  scale = 1/sqrt(mean(x'^2)+eps)
// One workgroup of W waves per row; each lane keeps its NCH 16-byte tiles of
// the row in registers between the sum of squares and the scaling pass, so the
// row is read from HBM once.  The host picks W so that every row of a large
// batch is resident at once (W = 1: a wave per row, no LDS, no barrier).
// f32 activations: statistics and scaling in f64, exactly the reference's
// operations.  fp16 activations: the output keeps 11 bits and nothing here cancels
// (h = x * scale * gamma), so f32 statistics (8-element partial sums, then a tree),
// the hardware rsq and two f32 multiplies differ from the reference's f32 result by
// parts in 1e7: after the one rounding to fp16 the result is the reference's in all but
// about 4 in 100 000 elements, and 1 ulp of fp16 away in those.
// =========================================================================
template <typename T> struct stat;
template <> struct stat<float> {
    typedef double acc_t;
    typedef double scale_t;
    DEV double sq(double a, float v) { return __builtin_fma((double)v, (double)v, a); }
    DEV double wave_sum(double v) { return group_sum<64>(v); }
    DEV double rscale(double ss, int n, float eps) { return 1.0 / sqrt(ss / (double)n + (double)eps); }
    DEV float apply(float v, double scale, float g) { return (float)((double)v * scale) * g; }
};
template <> struct stat<f16_t> {
    typedef float acc_t;
    typedef float scale_t;
    DEV float sq(float a, float v) { return __builtin_fmaf(v, v, a); }
    DEV float wave_sum(float v) { return group_sum<64>(v); }
    DEV float rscale(float ss, int n, float eps) { return __builtin_amdgcn_rsqf(ss * (1.0f / (float)n) + eps); }
    DEV float apply(float v, float scale, float g) { return v * scale * g; }
};
// The per-head norm in front of a rotation is another matter: a rotated output a*cos - b*sin can
// nearly cancel, and an f32-level difference in the normalised inputs is then many ulps of the
// fp16 result.  There fp16 activations get the reference's values themselves, at a third of the
// double-precision work, so that the result is the reference's f32 result rounded once to fp16:
//   * the sum of squares in f64, as the reference;
//   * 1/sqrt(mean + eps) by two Newton steps in f64 from the f32 hardware rsq (agrees with the
//     reference's sqrt-then-divide to about 1e-16);
//   * (x as f64 * scale) as f32 as an error-free f32 product with scale = hi + lo:
//     p = fl(x*hi), e = x*hi - p (exact, one fma), result = fl(p + fl(e + x*lo)): the
//     correctly rounded product unless it lies within 2^-48 of a rounding boundary.
template <typename T> struct headstat : stat<T> {};
template <> struct headstat<f16_t> {
    typedef double acc_t;
    struct scale_t { float hi, lo; };
    DEV double sq(double a, float v) { return __builtin_fma((double)v, (double)v, a); }
    DEV scale_t rscale(double ss, int n, float eps) {
        const double v = ss / (double)n + (double)eps;  // n a power of two known at compile time: a multiplication
        double y = (double)__builtin_amdgcn_rsqf((float)v);
        y = y * __builtin_fma(-0.5 * v, y * y, 1.5);
        y = y * __builtin_fma(-0.5 * v, y * y, 1.5);
        const float hi = (float)y;
        return scale_t{hi, (float)(y - (double)hi)};
    }
    DEV float apply(float v, scale_t s, float g) {
        const float p = v * s.hi;
        return (p + __builtin_fmaf(v, s.lo, __builtin_fmaf(v, s.hi, -p))) * g;
    }
};

template <typename T, int NCH, bool HAS_DELTA>
DEV void add_rmsnorm_impl(T* x, const T* delta, T* h, const float* gamma, int n, float eps, uint32_t vblock,
                          uint32_t rows_per_block, uint32_t rows) {
    constexpr int VEC = io<T>::VEC;
    typedef typename stat<T>::acc_t acc_t;
    __shared__ acc_t part[16];
    const int nchunks = n / VEC;
    // Two shapes of workgroup: all its waves share one row (rows_per_block == 1: few long rows), or
    // every wave has a row of its own (a wave covers the row with NCH tiles per lane; the workgroup
    // only bundles 4 such waves, which the host asks for where rows come in their thousands).
    const bool own_row = rows_per_block > 1;  // uniform
    const uint32_t tid = own_row ? (threadIdx.x & 63u) : threadIdx.x, stride = own_row ? 64u : blockDim.x;
    const uint64_t row = own_row ? (uint64_t)vblock * rows_per_block + (threadIdx.x >> 6) : vblock;
    if (own_row && row >= rows) return;  // whole wave
    T* xr = x + row * (uint64_t)n;
    T* hr = h + row * (uint64_t)n;
    const T* dr = HAS_DELTA ? delta + row * (uint64_t)n : nullptr;

    // Every load of the lane is issued before the first use: no branch and no
    // conversion in this loop (a lane past the end of the row re-reads the last tile).
    // With one or two tiles per lane (decode-sized batches: many waves per row, the kernel is a
    // chain of latencies, not a stream) the norm weights are fetched here too, so that nothing is
    // loaded after the cross-wave reduction; with more tiles they are read after it (they sit in
    // L2, the other resident waves cover the latency, and the registers go to the row instead).
    constexpr bool PRE_GAMMA = NCH <= 2;
    typename io<T>::raw_t xraw[NCH], draw[NCH];
    float gpre[PRE_GAMMA ? NCH : 1][VEC];
    if constexpr (PRE_GAMMA) {
#pragma unroll
        for (int j = 0; j < NCH; j++) {
            const int c = min((int)(tid + j * stride), nchunks - 1);
#pragma unroll
            for (int q = 0; q < VEC; q += 4) io<float>::load(gamma + c * VEC + q, gpre[j] + q);
        }
    }
#pragma unroll
    for (int j = 0; j < NCH; j++) {
        const int c = min((int)(tid + j * stride), nchunks - 1);
        xraw[j] = io<T>::ldraw_nt(xr + c * VEC);
        if constexpr (HAS_DELTA) draw[j] = io<T>::ldraw_nt(dr + c * VEC);
    }
    __builtin_amdgcn_sched_barrier(0);  // keep every load above; all uses below
    float v[NCH][VEC];
    acc_t ss = 0;
#pragma unroll
    for (int j = 0; j < NCH; j++) {
        const int c = tid + j * stride;
        io<T>::widen(xraw[j], v[j]);
        if constexpr (HAS_DELTA) {
            float d[VEC];
            io<T>::widen(draw[j], d);
#pragma unroll
            for (int i = 0; i < VEC; i++) v[j][i] = v[j][i] + d[i];
            if (c < nchunks) io<T>::store(xr + c * VEC, v[j]);
        }
        acc_t s8 = 0;
#pragma unroll
        for (int i = 0; i < VEC; i++) s8 = stat<T>::sq(s8, v[j][i]);
        ss += c < nchunks ? s8 : (acc_t)0;
    }
    ss = stat<T>::wave_sum(ss);
    const int nwaves = own_row ? 1 : (int)((blockDim.x + 63) >> 6);
    if (nwaves > 1) {
        if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = ss;
        __syncthreads();
        ss = 0;
        for (int w = 0; w < nwaves; w++) ss += part[w];
    }
    const typename stat<T>::scale_t scale = stat<T>::rscale(ss, n, eps);
#pragma unroll
    for (int j = 0; j < NCH; j++) {
        const int c = tid + j * stride;
        if (c < nchunks) {
            float g[VEC], o[VEC];
            if constexpr (PRE_GAMMA) {
#pragma unroll
                for (int i = 0; i < VEC; i++) g[i] = gpre[j][i];
            } else {
#pragma unroll
                for (int q = 0; q < VEC; q += 4) io<float>::load(gamma + c * VEC + q, g + q);
            }
#pragma unroll
            for (int i = 0; i < VEC; i++) o[i] = stat<T>::apply(v[j][i], scale, g[i]);
            io<T>::store_nt(hr + c * VEC, o);
        }
    }
}
template <typename T, int NCH>
DEV void add_rmsnorm_body(T* x, const T* delta, T* h, const float* gamma, int n, float eps, uint32_t vblock,
                          uint32_t rows_per_block = 1, uint32_t rows = 0) {
    if (delta) add_rmsnorm_impl<T, NCH, true>(x, delta, h, gamma, n, eps, vblock, rows_per_block, rows);   // uniform for the launch
    else add_rmsnorm_impl<T, NCH, false>(x, delta, h, gamma, n, eps, vblock, rows_per_block, rows);
}
// Short rows (at most 32 tiles: 256 fp16 / 128 f32 elements, e.g. one head): LPR lanes per row,
// 64/LPR rows per wave, one tile per lane, the statistics reduced inside the LPR-lane group --
// a wave per row would leave most lanes idle.
template <typename T, int LPR>
DEV void add_rmsnorm_small_body(T* x, const T* delta, T* h, const float* gamma, int n, uint32_t rows, float eps) {
    constexpr int VEC = io<T>::VEC;
    typedef typename stat<T>::acc_t acc_t;
    const int nchunks = n / VEC;
    const uint32_t lane = threadIdx.x & 63u, l = lane % LPR;
    const uint64_t row = ((uint64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)) * (64 / LPR) + lane / LPR;
    const bool live = row < rows && (int)l < nchunks;
    const uint64_t off = min(row, (uint64_t)rows - 1) * (uint64_t)n + (uint64_t)min((int)l, nchunks - 1) * VEC;  // clamped: read, not used
    float g[VEC], v[VEC];
#pragma unroll
    for (int q = 0; q < VEC; q += 4) io<float>::load(gamma + min((int)l, nchunks - 1) * VEC + q, g + q);
    io<T>::load_nt(x + off, v);
    if (delta) {
        float d[VEC];
        io<T>::load_nt(delta + off, d);
#pragma unroll
        for (int i = 0; i < VEC; i++) v[i] = v[i] + d[i];
        if (live) io<T>::store(x + off, v);
    }
    acc_t ss = 0;
    if (live) {
#pragma unroll
        for (int i = 0; i < VEC; i++) ss = stat<T>::sq(ss, v[i]);
    }
    ss = group_sum<LPR>(ss);
    const typename stat<T>::scale_t scale = stat<T>::rscale(ss, n, eps);
    if (live) {
        float o[VEC];
#pragma unroll
        for (int i = 0; i < VEC; i++) o[i] = stat<T>::apply(v[i], scale, g[i]);
        io<T>::store_nt(h + off, o);
    }
}
#define APK_ADDNORM_SMALL(T, TN, LPR)                                                                              \
    extern "C" __global__ __launch_bounds__(256) void apk_add_rmsnorm_small_##TN##_l##LPR(                         \
        T* x, const T* delta, T* h, const float* gamma, int n, uint32_t rows, float eps) {                         \
        add_rmsnorm_small_body<T, LPR>(x, delta, h, gamma, n, rows, eps);                                          \
    }
APK_ADDNORM_SMALL(float, f32, 4) APK_ADDNORM_SMALL(float, f32, 8) APK_ADDNORM_SMALL(float, f32, 16) APK_ADDNORM_SMALL(float, f32, 32)
APK_ADDNORM_SMALL(f16_t, f16, 4) APK_ADDNORM_SMALL(f16_t, f16, 8) APK_ADDNORM_SMALL(f16_t, f16, 16) APK_ADDNORM_SMALL(f16_t, f16, 32)

// Rows whose length is not a whole number of 16-byte tiles (so rows are not 16-byte aligned
// either), or longer than the tiled kernels keep in registers: one element per lane per step,
// two passes over the row.  The first pass only accumulates the statistics of x + delta; the
// second recomputes the sum, writes it back and normalises the unrounded value -- for fp16 rows
// the norm must see the f32 sum, not its fp16 rounding.  Correctness path for odd shapes (the
// reference's 2- and 6-element unit tests, rows beyond 20 480 elements), not a fast one.
template <typename T>
DEV void add_rmsnorm_loop_body(T* x, const T* delta, T* h, const float* gamma, int n, float eps) {
    typedef typename stat<T>::acc_t acc_t;
    __shared__ acc_t part[4];
    const uint64_t row = blockIdx.x;
    T* xr = x + row * (uint64_t)n;
    T* hr = h + row * (uint64_t)n;
    const T* dr = delta ? delta + row * (uint64_t)n : nullptr;
    acc_t ss = 0;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        float v = (float)xr[i];
        if (dr) v = v + (float)dr[i];
        ss = stat<T>::sq(ss, v);
    }
    ss = stat<T>::wave_sum(ss);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = ss;
    __syncthreads();
    ss = 0;
    for (int w = 0; w < (int)(blockDim.x >> 6); w++) ss += part[w];
    const typename stat<T>::scale_t scale = stat<T>::rscale(ss, n, eps);
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        float v = (float)xr[i];
        if (dr) {
            v = v + (float)dr[i];
            xr[i] = (T)v;
        }
        hr[i] = (T)stat<T>::apply(v, scale, gamma[i]);
    }
}
extern "C" __global__ __launch_bounds__(256) void apk_add_rmsnorm_ragged_f32(float* x, const float* delta, float* h,
                                                                            const float* gamma, int n, float eps) {
    add_rmsnorm_loop_body<float>(x, delta, h, gamma, n, eps);
}
extern "C" __global__ __launch_bounds__(256) void apk_add_rmsnorm_ragged_f16(f16_t* x, const f16_t* delta, f16_t* h,
                                                                            const float* gamma, int n, float eps) {
    add_rmsnorm_loop_body<f16_t>(x, delta, h, gamma, n, eps);
}

// The launch bound is the largest workgroup the host uses with that tile count
// (it also caps the registers the compiler may take: 512 / (bound/64/4) per lane).
#define APK_ADDNORM(T, TN, NCH, MAXT)                                                                        \
    extern "C" __global__ __launch_bounds__(MAXT) void apk_add_rmsnorm_##TN##_c##NCH(                        \
        T* x, const T* delta, T* h, const float* gamma, int n, float eps, uint32_t rows_per_block, uint32_t rows) { \
        add_rmsnorm_body<T, NCH>(x, delta, h, gamma, n, eps, blockIdx.x, rows_per_block, rows);              \
    }
#define APK_ADDNORM_ALL(T, TN)                                                                                   \
    APK_ADDNORM(T, TN, 1, 1024) APK_ADDNORM(T, TN, 2, 1024) APK_ADDNORM(T, TN, 3, 512) APK_ADDNORM(T, TN, 4, 512) \
    APK_ADDNORM(T, TN, 5, 256) APK_ADDNORM(T, TN, 6, 256) APK_ADDNORM(T, TN, 8, 256) APK_ADDNORM(T, TN, 10, 256)  \
    APK_ADDNORM(T, TN, 12, 256) APK_ADDNORM(T, TN, 16, 256) APK_ADDNORM(T, TN, 20, 256)
APK_ADDNORM_ALL(float, f32)
APK_ADDNORM_ALL(f16_t, f16)

// =========================================================================
// MoE combine + residual add + the next RMSNorm, one pass per token row
// (moe.rs:298-333 then decode.rs:775 / prefill.rs:308-314):
//   out = 0; for each hit of the token, in CSR order: out = fma(down[hit_row], hit_w, out)
//   (ops::add_scaled_slice, blas.rs:25-102, x86 arm: one rounding per hit);
//   x += out;  h = rmsnorm(x) * gamma  (skipped when h is null).
// Same row layout as add+RMSNorm: W waves per row, NCH tiles per lane; the k
// expert rows of a token are fetched HB hits at a time, all in flight together.
// =========================================================================
template <typename T, int NCH, int HB>
DEV void combine_add_rmsnorm_body(T* x, const T* flat, const uint32_t* tok_off, const uint32_t* hit_row,
                                  const float* hit_w, uint32_t total_rows, T* h, const float* gamma, int n, float eps,
                                  uint32_t* fault) {
    constexpr int VEC = io<T>::VEC;
    typedef typename stat<T>::acc_t acc_t;
    __shared__ acc_t part[16];
    const int nchunks = n / VEC;
    const uint64_t row = blockIdx.x;
    T* xr = x + row * (uint64_t)n;
    const uint32_t h0 = tok_off[row], h1 = tok_off[row + 1];
    int cidx[NCH];
    typename io<T>::raw_t xraw[NCH];
#pragma unroll
    for (int j = 0; j < NCH; j++) {
        cidx[j] = min((int)(threadIdx.x + j * blockDim.x), nchunks - 1);
        xraw[j] = io<T>::ldraw_nt(xr + cidx[j] * VEC);
    }
    float acc[NCH][VEC];
#pragma unroll
    for (int j = 0; j < NCH; j++)
#pragma unroll
        for (int i = 0; i < VEC; i++) acc[j][i] = 0.0f;
    // HB hits at a time: their row numbers and weights first (uniform for the workgroup), then
    // every tile of all HB expert rows in flight at once, then the multiply-adds in hit order (the
    // order is the contract: one rounding per hit).  Slots past the token's last hit re-read its
    // last row (a cache hit) and add nothing.
    for (uint32_t kb = h0; kb < h1; kb += HB) {
        uint32_t r[HB];
        float w[HB];
        bool use[HB];
        bool bad = false;
#pragma unroll
        for (int j = 0; j < HB; j++) {
            const uint32_t kk = min(kb + (uint32_t)j, h1 - 1u);
            r[j] = hit_row[kk];
            w[j] = hit_w[kk];
            const bool in_range = r[j] < total_rows;
            use[j] = kb + (uint32_t)j < h1 && in_range;
            bad |= !in_range;
            r[j] = in_range ? r[j] : 0u;
        }
        if (bad && threadIdx.x == 0) atomicOr(fault, APK_FAULT_ROW_RANGE);
        typename io<T>::raw_t d[HB][NCH];
#pragma unroll
        for (int j = 0; j < HB; j++)
#pragma unroll
            for (int c = 0; c < NCH; c++) d[j][c] = io<T>::ldraw_nt(flat + (uint64_t)r[j] * n + cidx[c] * VEC);
        __builtin_amdgcn_sched_barrier(0);  // every load above, every use below
#pragma unroll
        for (int j = 0; j < HB; j++) {
            if (use[j]) {  // uniform
#pragma unroll
                for (int c = 0; c < NCH; c++) {
                    float a[VEC];
                    io<T>::widen(d[j][c], a);
#pragma unroll
                    for (int i = 0; i < VEC; i++) acc[c][i] = __builtin_fmaf(a[i], w[j], acc[c][i]);
                }
            }
        }
    }
    float v[NCH][VEC];
    acc_t ss = 0;
#pragma unroll
    for (int j = 0; j < NCH; j++) {
        const int c = threadIdx.x + j * blockDim.x;
        io<T>::widen(xraw[j], v[j]);
#pragma unroll
        for (int i = 0; i < VEC; i++) v[j][i] = v[j][i] + acc[j][i];
        if (c < nchunks) io<T>::store(xr + c * VEC, v[j]);
        acc_t s8 = 0;
#pragma unroll
        for (int i = 0; i < VEC; i++) s8 = stat<T>::sq(s8, v[j][i]);
        ss += c < nchunks ? s8 : (acc_t)0;
    }
    if (h == nullptr) return;  // uniform: combine + residual only
    ss = stat<T>::wave_sum(ss);
    const int nwaves = (blockDim.x + 63) >> 6;
    if (nwaves > 1) {
        if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = ss;
        __syncthreads();
        ss = 0;
        for (int w = 0; w < nwaves; w++) ss += part[w];
    }
    const typename stat<T>::scale_t scale = stat<T>::rscale(ss, n, eps);
    T* hr = h + row * (uint64_t)n;
#pragma unroll
    for (int j = 0; j < NCH; j++) {
        const int c = threadIdx.x + j * blockDim.x;
        if (c < nchunks) {
            float g[VEC], o[VEC];
#pragma unroll
            for (int q = 0; q < VEC; q += 4) io<float>::load(gamma + c * VEC + q, g + q);
#pragma unroll
            for (int i = 0; i < VEC; i++) o[i] = stat<T>::apply(v[j][i], scale, g[i]);
            io<T>::store_nt(hr + c * VEC, o);
        }
    }
}
// 4 hits in flight: with 4 tiles per lane that is 16 loads per lane, the register budget of a
// 1024-thread workgroup (8 hits in flight with 2 tiles per lane measured slower).
#define APK_COMBINE(T, TN, NCH)                                                                                        \
    extern "C" __global__ __launch_bounds__(1024) void apk_combine_add_rmsnorm_##TN##_c##NCH(                         \
        T* x, const T* flat, const uint32_t* tok_off, const uint32_t* hit_row, const float* hit_w, uint32_t total_rows, \
        T* h, const float* gamma, int n, float eps, uint32_t* fault) {                                                 \
        combine_add_rmsnorm_body<T, NCH, 4>(x, flat, tok_off, hit_row, hit_w, total_rows, h, gamma, n, eps, fault);    \
    }
APK_COMBINE(float, f32, 1) APK_COMBINE(float, f32, 2) APK_COMBINE(float, f32, 4)
APK_COMBINE(f16_t, f16, 1) APK_COMBINE(f16_t, f16, 2) APK_COMBINE(f16_t, f16, 4)

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

// =========================================================================
// Per-head QK-norm + NeoX RoPE, in place on q [rows, n_q*HD] and k [rows, n_kv*HD]
// (caller loop attention.rs:131-165: rmsnorm(head, w, eps) then the NeoX
// rotation with the row's [sin, cos] table, rope.rs:70-81).
// Lane mapping: a lane holds one 16-byte tile of the first half of a head and
// the tile of its NeoX partners in the second half (EPL = 8 fp16 / 4 f32
// elements each), so the rotation needs no cross-lane traffic, every global
// access is a full 16-byte tile and the LPH = HD/2/EPL lanes of a head cover
// contiguous runs.  A wave owns (row, q or k, group of HPW*ITER consecutive
// heads), HPW = 64/LPH heads per pass: one tensor per wave means one norm
// weight per wave and no per-element selects; the row's [sin, cos] tile and
// the weight are loaded once and reused over ITER passes (q: ITERQ passes,
// k: 1 pass -- under GQA k has few heads).  Waves are kept short (ITERQ 1 or 2, about
// 4 KB of heads each): a wave that carries a row's 64 q heads in 8 passes lives as long as
// the whole launch, and a batch a few rows beyond one resident round of such waves
// (2061 rows instead of 2048) then takes 15 % longer; short waves fill in evenly.
// Arithmetic: the reference's, for both activation types (see `headstat`): f64 statistics,
// (x as f64 * scale) as f32 * w, then the four products and two sums of the rotation,
// not contracted.  fp16 results are that f32 result rounded once.
// =========================================================================
// KV = true (k items only): the rotated k tiles are also narrowed to fp16 into the cache row
// kc, and the same tiles of the row's v are narrowed into vc (KvCache::store_at,
// crates/allpaka-model/src/kv.rs:682-697: k and v rows as f16 at pos*kv_dim).
template <typename T, int HD, int ITER, bool KV = false>
DEV void qk_item(T* base, int nheads, int g, const float* w, const float* trow, float eps, int l, int sub,
                 f16_t* kc = nullptr, const T* vrow = nullptr, f16_t* vc = nullptr) {
    constexpr int EPL = io<T>::VEC;   // elements per lane per half
    constexpr int HALF = HD / 2;
    constexpr int LPH = HALF / EPL;   // lanes per head
    constexpr int HPW = 64 / LPH;     // heads per wave pass
    typedef typename headstat<T>::acc_t acc_t;
    // Loads return in issue order, so the small cached ones go first and the first pass
    // can start as soon as its own two tiles arrive.  No branch, no conversion here: a
    // lane of a pass beyond the last head re-reads the last head and stores nothing; a
    // missing norm weight is read from the [sin, cos] tile instead and never used.
    float sc[2 * EPL], wa[EPL], wb[EPL];
#pragma unroll
    for (int i = 0; i < 2 * EPL; i += 4) io<float>::load(trow + 2 * EPL * l + i, sc + i);
    const float* wp = w ? w : trow;
#pragma unroll
    for (int i = 0; i < EPL; i += 4) {
        io<float>::load(wp + EPL * l + i, wa + i);
        io<float>::load(wp + HALF + EPL * l + i, wb + i);
    }
    typename io<T>::raw_t araw[ITER], braw[ITER], varaw[ITER], vbraw[ITER];
    // head of pass `it` and its element offset: recomputed where needed (a few integer
    // operations) rather than kept in registers across the loads
    const int hh_first = g * ITER * HPW + sub;
    auto head_off = [&](int it) { return min(hh_first + it * HPW, nheads - 1) * HD + EPL * l; };
#pragma unroll
    for (int it = 0; it < ITER; it++) {
        const int off = head_off(it);
        __builtin_amdgcn_sched_barrier(0);  // loads stay in program order (returns are in order)
        araw[it] = io<T>::ldraw_nt(base + off);
        braw[it] = io<T>::ldraw_nt(base + off + HALF);
        if constexpr (KV) {
            varaw[it] = io<T>::ldraw_nt(vrow + off);
            vbraw[it] = io<T>::ldraw_nt(vrow + off + HALF);
        }
    }
    __builtin_amdgcn_sched_barrier(0);  // every load above; all uses below
    const bool normed = w != nullptr;  // uniform for the wave
#pragma unroll
    for (int it = 0; it < ITER; it++) {
        float a[EPL], b[EPL], oa[EPL], ob[EPL];
        io<T>::widen(araw[it], a);
        io<T>::widen(braw[it], b);
        acc_t ss = 0;
#pragma unroll
        for (int i = 0; i < EPL; i++) {
            ss = headstat<T>::sq(ss, a[i]);
            ss = headstat<T>::sq(ss, b[i]);
        }
        ss = group_sum<LPH>(ss);
        const typename headstat<T>::scale_t scale = headstat<T>::rscale(ss, HD, eps);
#pragma unroll
        for (int i = 0; i < EPL; i++) {
            float x = a[i], y = b[i];
            if (normed) {
                x = headstat<T>::apply(x, scale, wa[i]);
                y = headstat<T>::apply(y, scale, wb[i]);
            }
            const float s = sc[2 * i], c = sc[2 * i + 1];
            oa[i] = x * c - y * s;  // not contracted: the reference's four products and two sums
            ob[i] = x * s + y * c;
        }
        const bool live = hh_first + it * HPW < nheads;
        const int off = head_off(it);
        if (live) {
            io<T>::store_nt(base + off, oa);
            io<T>::store_nt(base + off + HALF, ob);
        }
        if constexpr (KV) {
            if (live && kc != nullptr) {  // kc == nullptr: cache position out of range, row skipped
                float va[EPL], vb[EPL];
                io<T>::widen(varaw[it], va);
                io<T>::widen(vbraw[it], vb);
                store_f16_tile<T>(kc + off, oa);
                store_f16_tile<T>(kc + off + HALF, ob);
                store_f16_tile<T>(vc + off, va);
                store_f16_tile<T>(vc + off + HALF, vb);
            }
        }
        __builtin_amdgcn_sched_barrier(0);  // pass by pass: pass it+1 waits only for its own tiles
    }
}

template <typename T, int HD, int ITERQ, bool KV = false>
DEV void qknorm_rope_body(T* q, T* k, const float* qw, const float* kw, const float* rope, int rows, int n_q, int n_kv,
                          float eps, uint32_t vblock, const T* v = nullptr, const uint32_t* cache_pos = nullptr,
                          f16_t* k_cache = nullptr, f16_t* v_cache = nullptr, uint32_t capacity = 0,
                          uint32_t* fault = nullptr) {
    constexpr int LPH = HD / 2 / io<T>::VEC, HPW = 64 / LPH;
    const int lane = threadIdx.x & 63;
    const int l = lane % LPH, sub = lane / LPH;
    const int gq = (n_q + HPW * ITERQ - 1) / (HPW * ITERQ), gk = (n_kv + HPW - 1) / HPW;
    // all q items first (the longer ones, up to two passes), then the k items, one pass each
    const uint64_t wid = ((uint64_t)vblock * blockDim.x + threadIdx.x) >> 6;
    const uint64_t nq_items = (uint64_t)rows * gq;
    if (wid >= nq_items + (uint64_t)rows * gk) return;  // whole wave
    if (wid < nq_items) {
        const uint64_t row = wid / gq;
        qk_item<T, HD, ITERQ>(q + row * (uint64_t)n_q * HD, n_q, (int)(wid % gq), qw, rope + row * HD, eps, l, sub);
    } else {
        const uint64_t w2 = wid - nq_items, row = w2 / gk;
        const uint64_t kv_dim = (uint64_t)n_kv * HD;
        if constexpr (KV) {
            const uint32_t pos = cache_pos[row];
            const bool ok = pos < capacity;
            if (!ok && lane == 0 && w2 % gk == 0) atomicOr(fault, APK_FAULT_CACHE_RANGE);
            qk_item<T, HD, 1, true>(k + row * kv_dim, n_kv, (int)(w2 % gk), kw, rope + row * HD, eps, l, sub,
                                    ok ? k_cache + pos * kv_dim : nullptr, v + row * kv_dim,
                                    ok ? v_cache + pos * kv_dim : nullptr);
        } else {
            qk_item<T, HD, 1>(k + row * kv_dim, n_kv, (int)(w2 % gk), kw, rope + row * HD, eps, l, sub);
        }
    }
}
// At most 128 VGPRs (at least 4 waves per SIMD).
#define APK_QK_OCC __attribute__((amdgpu_waves_per_eu(4)))
#define APK_QKROPE(T, TN, HD, ITER)                                                                          \
    extern "C" __global__ __launch_bounds__(256) APK_QK_OCC void apk_qknorm_rope_##TN##_hd##HD##_i##ITER(   \
        T* q, T* k, const float* qw, const float* kw, const float* rope, int rows, int n_q, int n_kv, float eps) { \
        qknorm_rope_body<T, HD, ITER>(q, k, qw, kw, rope, rows, n_q, n_kv, eps, blockIdx.x);                  \
    }
#define APK_QKROPE_ALL(T, TN)                                                                                          \
    APK_QKROPE(T, TN, 64, 1) APK_QKROPE(T, TN, 64, 2) APK_QKROPE(T, TN, 128, 1) APK_QKROPE(T, TN, 128, 2)              \
    APK_QKROPE(T, TN, 256, 1) APK_QKROPE(T, TN, 256, 2)
APK_QKROPE_ALL(float, f32)
APK_QKROPE_ALL(f16_t, f16)

// The same with the K/V cache store fused in: rotated k and the row's v narrowed to fp16
// at cache row cache_pos[row] (one launch instead of QK-norm+RoPE, then two narrowing copies).
#define APK_QKROPE_KV(T, TN, HD, ITER)                                                                            \
    extern "C" __global__ __launch_bounds__(256) APK_QK_OCC void apk_qknorm_rope_kv_##TN##_hd##HD##_i##ITER(     \
        T* q, T* k, const T* v, const float* qw, const float* kw, const float* rope, const uint32_t* cache_pos,  \
        f16_t* k_cache, f16_t* v_cache, uint32_t capacity, int rows, int n_q, int n_kv, float eps, uint32_t* fault) { \
        qknorm_rope_body<T, HD, ITER, true>(q, k, qw, kw, rope, rows, n_q, n_kv, eps, blockIdx.x, v, cache_pos,   \
                                            k_cache, v_cache, capacity, fault);                                   \
    }
#define APK_QKROPE_KV_ALL(T, TN)                                                                                       \
    APK_QKROPE_KV(T, TN, 64, 1) APK_QKROPE_KV(T, TN, 64, 2) APK_QKROPE_KV(T, TN, 128, 1) APK_QKROPE_KV(T, TN, 128, 2)  \
    APK_QKROPE_KV(T, TN, 256, 1) APK_QKROPE_KV(T, TN, 256, 2)
APK_QKROPE_KV_ALL(float, f32)
APK_QKROPE_KV_ALL(f16_t, f16)

// Any other head geometry: head_dim not 64/128/256, a rotary table that covers only the
// leading rot_half pairs of a head (partial rotary: channels >= 2*rot_half are normalised
// and pass through, rope.rs:52-81), or the adjacent-pair style (RopeStyle::Norm, pairs
// (2i, 2i+1), rope.rs:52-64; chosen per model in attention.rs:62-67).  A wave per head,
// element-wise; same arithmetic as the tiled kernels minus the coefficient folding.
template <typename T>
DEV void qknorm_rope_generic_body(T* q, T* k, const float* qw, const float* kw, const float* rope, int rows, int n_q,
                                  int n_kv, int hd, int rot_half, int norm_style, float eps) {
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
    const float* t = rope + row * (uint64_t)rot_half * 2;
    typename headstat<T>::scale_t scale{};
    if (w) {
        acc_t ss = 0;
        for (int i = lane; i < hd; i += 64) ss = headstat<T>::sq(ss, (float)x[i]);
        ss = group_sum<64>(ss);  // every lane's loads are consumed here, before any store below
        scale = headstat<T>::rscale(ss, hd, eps);
    }
    for (int i = lane; i < rot_half; i += 64) {
        const int ia = norm_style ? 2 * i : i, ib = norm_style ? 2 * i + 1 : i + rot_half;
        float a = (float)x[ia], b = (float)x[ib];
        if (w) {
            a = headstat<T>::apply(a, scale, w[ia]);
            b = headstat<T>::apply(b, scale, w[ib]);
        }
        const float sn = t[2 * i], cs = t[2 * i + 1];
        x[ia] = (T)(a * cs - b * sn);
        x[ib] = (T)(a * sn + b * cs);
    }
    if (w)
        for (int i = 2 * rot_half + lane; i < hd; i += 64) x[i] = (T)headstat<T>::apply((float)x[i], scale, w[i]);
}
extern "C" __global__ __launch_bounds__(256) void apk_qknorm_rope_generic_f32(
    float* q, float* k, const float* qw, const float* kw, const float* rope, int rows, int n_q, int n_kv, int hd,
    int rot_half, int norm_style, float eps) {
    qknorm_rope_generic_body<float>(q, k, qw, kw, rope, rows, n_q, n_kv, hd, rot_half, norm_style, eps);
}
extern "C" __global__ __launch_bounds__(256) void apk_qknorm_rope_generic_f16(
    f16_t* q, f16_t* k, const float* qw, const float* kw, const float* rope, int rows, int n_q, int n_kv, int hd,
    int rot_half, int norm_style, float eps) {
    qknorm_rope_generic_body<f16_t>(q, k, qw, kw, rope, rows, n_q, n_kv, hd, rot_half, norm_style, eps);
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
        else qknorm_rope_body<T, HD, 1>(q, k, qw, kw, rope, rows, n_q, n_kv, eps, blockIdx.x - (uint32_t)rows);  \
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
    if (scale != 1.0f) {
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
};
template <> struct qbytes<4> {
    uint32_t v;
    DEV qbytes<4> at(const uint8_t* p) { return qbytes<4>{*(const u32_a2*)p}; }
    DEV uint32_t byte(const qbytes<4>& q, int i) { return (q.v >> (8 * i)) & 0xffu; }
};
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
        for (int i = 0; i < N; i++) o[i] = dl * (float)((qbytes<N>::byte(qs, i) >> (2 * si)) & 3u) - ml;
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
        const uint32_t m = 1u << (half * 4 + si);
#pragma unroll
        for (int i = 0; i < N; i++) {
            const int quant = (int)((qbytes<N>::byte(qs, i) >> (2 * si)) & 3u) - ((qbytes<N>::byte(hm, i) & m) ? 0 : 4);
            o[i] = dl * (float)quant;
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
        for (int i = 0; i < N; i++) {
            const uint32_t byte = qbytes<N>::byte(qs, i);
            const uint32_t q4 = hn ? (byte >> 4) : (byte & 0xfu);
            const uint32_t hb = (qbytes<N>::byte(qh, i) >> sub) & 1u;
            o[i] = dsc * (float)(q4 + 16u * hb) - dm;
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
#pragma unroll
        for (int i = 0; i < N; i++) {
            const uint32_t lo = qbytes<N>::byte(ql, i);
            const uint32_t nib = quarter < 2 ? (lo & 0xfu) : (lo >> 4);
            const int qv = (int)(nib | (((qbytes<N>::byte(qh, i) >> (2 * quarter)) & 3u) << 4)) - 32;
            o[i] = dl * (float)qv;
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
template <int FMT, typename TO>
DEV void embed_direct_sb_body(const uint8_t* __restrict__ table, uint32_t vocab, int n_in, const uint32_t* __restrict__ ids,
                              uint32_t chunks, TO* __restrict__ out, uint32_t* fault, float scale, uint32_t row0) {
    constexpr int OPT = io<TO>::VEC, K = 256 / OPT / 8;
    const uint32_t t = blockIdx.x / chunks, chunk = blockIdx.x - t * chunks;
    const uint32_t id = ids ? ids[t] : row0 + (uint32_t)t;  // no id list: the rows row0, row0 + 1, ...
    if (id >= vocab) {  // uniform
        if (threadIdx.x == 0 && chunk == 0) atomicOr(fault, APK_FAULT_TOKEN_RANGE);
        return;
    }
    const uint32_t nsb = (uint32_t)n_in / 256;
    const uint32_t j = chunk * blockDim.x + threadIdx.x, L = j & 7u;
    const bool live = (j >> 3) < nsb;
    const uint32_t sb = min(j >> 3, nsb - 1u);  // a lane past the last super-block re-reads it and stores nothing
    const uint8_t* row = table + (uint64_t)id * ((uint64_t)nsb * dqd<FMT>::BB);
    float o[K][OPT];
#pragma unroll
    for (int k = 0; k < K; k++) dqd<FMT>::template tile<OPT>(row, sb * 256u + (8u * k + L) * OPT, o[k]);
    if (!live) return;
    TO* orow = out + (uint64_t)t * n_in + (uint64_t)sb * 256;
#pragma unroll
    for (int k = 0; k < K; k++) {
        embed_scale<OPT>(o[k], scale);
        io<TO>::store_nt(orow + (8 * k + L) * OPT, o[k]);
    }
}
#define APK_EMBED_DIRECT_SB(NAME, FMT)                                                                                   \
    extern "C" __global__ __launch_bounds__(256) void apk_embed_##NAME##_f32(                                            \
        const uint8_t* table, uint32_t vocab, int n_in, const uint32_t* ids, uint32_t chunks, float* out, uint32_t* fault, \
        float scale, uint32_t row0) {                                                                                    \
        embed_direct_sb_body<FMT, float>(table, vocab, n_in, ids, chunks, out, fault, scale, row0);                      \
    }                                                                                                                    \
    extern "C" __global__ __launch_bounds__(256) void apk_embed_##NAME##_f16(                                            \
        const uint8_t* table, uint32_t vocab, int n_in, const uint32_t* ids, uint32_t chunks, f16_t* out, uint32_t* fault, \
        float scale, uint32_t row0) {                                                                                    \
        embed_direct_sb_body<FMT, f16_t>(table, vocab, n_in, ids, chunks, out, fault, scale, row0);                      \
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
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    if (tid < n_expert) mask[tid] = 0u;
    __syncthreads();
    if (wv < rows) {  // uniform per wave: wave wv routes token wv
        uint32_t id;
        float w;
        route_token<EPL>(logits + (uint64_t)wv * n_expert, bias, n_expert, k, norm, scale, sigmoid, lane, id, w);
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
        for (int c = threadIdx.x; c < row_vecs; c += blockDim.x) __builtin_nontemporal_store(sp[c], dp + c);
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
        if (c[i] < row_vecs) __builtin_nontemporal_store(a[i], dp + c[i]);
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
    if (c < nvec) __builtin_nontemporal_store(__builtin_nontemporal_load(src + c), dst + c);
}
