// gfx950 device code, part of apk_kernels.hip (one translation unit, one code object): SwiGLU, GeGLU, residual add, row softmax.
#pragma once

// =========================================================================
// SwiGLU: gate[i] = silu(gate[i]) * up[i], silu(x) = x / (1 + exp(-x))
// (activation.rs:19-22, :116-119).  Pure stream: 2 reads + 1 write / element.
// =========================================================================
// Both gates are g * sigmoid(a) * u: a = g for SiLU; for the tanh GELU of GeGLU (activation.rs:44-51)
// 0.5 g (1 + tanh z) = g * sigmoid(2z), z = sqrt(2/pi) g (1 + 0.044715 g^2) -- the form without the
// cancellation of 1 + tanh z for negative z (there the reference's own f32 result carries the rounding of
// its tanh, up to a few 1e-5 relative; this one stays within a few ulp of the exact value).
template <typename T> DEV float sigmoid_gate(float g, float a, float u);
// f32 activations: exp(-g) by Cody-Waite reduction around the hardware exp2 (log2(e) carried in
// two parts, so the reduced argument is exact to the last bit: about 1 ulp over the whole range,
// where a bare exp2(-g*log2e) loses |g| ulps), then the hardware reciprocal (1 ulp): the result is
// within a few ulp of the reference's g / (1 + exp(-g)) * u -- 1e-6 of the 1e-5 bar -- at a third
// of the instructions of libm expf + IEEE division, which at 32 per element no longer hid behind
// the stream.
template <> __device__ __forceinline__ float sigmoid_gate<float>(float g, float a, float u) {
    const float L2E_HI = 1.44269502162933349609375f, L2E_LO = 1.925963033500011e-08f;  // hi + lo = log2(e)
    const float n = fminf(fmaxf(-a, -104.0f), 89.0f);  // beyond: e underflows to 0 / overflows to inf anyway
    const float k = __builtin_rintf(n * L2E_HI);
    float r = __builtin_fmaf(n, L2E_HI, -k);
    r = __builtin_fmaf(n, L2E_LO, r);
    const float e = __builtin_amdgcn_ldexpf(__builtin_amdgcn_exp2f(r), (int)k);
    // the hardware reciprocal flushes subnormal results: keep 1/(1+e) normal for e up to FLT_MAX by
    // taking it of (1+e) * 2^-32 and applying the 2^-32 after the multiplication by g (all exact)
    const float sc = e > 0x1p96f ? 0x1p-32f : 1.0f;
    return g * __builtin_amdgcn_rcpf((1.0f + e) * sc) * sc * u;  // NaN in g still gives NaN (a is a function of g)
}
// fp16 activations: the result is rounded to 11 bits, so the hardware exp2 /
// rcp approximations (about 1 ulp of f32 each) are far inside the 2-ulp-of-fp16
// budget and keep the kernel under its ALU ceiling.
template <> __device__ __forceinline__ float sigmoid_gate<f16_t>(float g, float a, float u) {
    float e = __builtin_amdgcn_exp2f(a * -1.4426950408889634f);
    return g * __builtin_amdgcn_rcpf(1.0f + e) * u;
}
template <typename T, bool GELU> DEV float gate_mul(float g, float u) {
    if constexpr (GELU) return sigmoid_gate<T>(g, 2.0f * (0.7978846f * g * (1.0f + 0.044715f * g * g)), u);
    else return sigmoid_gate<T>(g, g, u);
}

template <typename T, int UNR, bool GELU = false> DEV void swiglu_body(T* gate, const T* up, uint64_t n) {
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
            for (int i = 0; i < VEC; i++) g[j][i] = gate_mul<T, GELU>(g[j][i], u[j][i]);
            io<T>::store_wt(gate + c * VEC, g[j]);
        }
    }
    // ragged tail (n not a multiple of the 16-byte tile): last block, scalar
    if (blockIdx.x == gridDim.x - 1) {
        for (uint64_t i = nvec * VEC + threadIdx.x; i < n; i += blockDim.x)
            gate[i] = (T)gate_mul<T, GELU>((float)gate[i], (float)up[i]);
    }
}
#define APK_SWIGLU_UNR 1  // measured: 1 tile per lane streams best (most waves in flight)
extern "C" __global__ __launch_bounds__(256) void apk_swiglu_f32(float* gate, const float* up, uint64_t n) {
    swiglu_body<float, APK_SWIGLU_UNR>(gate, up, n);
}
extern "C" __global__ __launch_bounds__(256) void apk_swiglu_f16(f16_t* gate, const f16_t* up, uint64_t n) {
    swiglu_body<f16_t, APK_SWIGLU_UNR>(gate, up, n);
}
// GeGLU with the tanh GELU, the FFN gate of the Gemma family: gate[i] = gelu_tanh(gate[i]) * up[i].
extern "C" __global__ __launch_bounds__(256) void apk_geglu_tanh_f32(float* gate, const float* up, uint64_t n) {
    swiglu_body<float, APK_SWIGLU_UNR, true>(gate, up, n);
}
extern "C" __global__ __launch_bounds__(256) void apk_geglu_tanh_f16(f16_t* gate, const f16_t* up, uint64_t n) {
    swiglu_body<f16_t, APK_SWIGLU_UNR, true>(gate, up, n);
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
        io<T>::store_wt(a + c * VEC, x);
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

// Scaled accumulate on its own: dst[i] = fma(src[i], scale, dst[i]) (ops::add_scaled_slice, blas.rs:25-102: one fused
// multiply-add per element on both of the reference's SIMD arms, and `mul_add` in their tails), the step the decode
// MoE combine repeats per picked expert (moe.rs:500-509).  fp16 rows: the f32 fma, rounded once.
template <typename T> DEV void add_scaled_body(T* dst, const T* src, uint64_t n, float scale) {
    constexpr int VEC = io<T>::VEC;
    const uint64_t nvec = n / VEC, c = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (c < nvec) {
        float x[VEC], y[VEC];
        io<T>::load_nt(dst + c * VEC, x);
        io<T>::load_nt(src + c * VEC, y);
#pragma unroll
        for (int i = 0; i < VEC; i++) x[i] = __builtin_fmaf(y[i], scale, x[i]);
        io<T>::store_wt(dst + c * VEC, x);
    }
    if (blockIdx.x == gridDim.x - 1)
        for (uint64_t i = nvec * VEC + threadIdx.x; i < n; i += blockDim.x) dst[i] = (T)__builtin_fmaf((float)src[i], scale, (float)dst[i]);
}
extern "C" __global__ __launch_bounds__(256) void apk_add_scaled_f32(float* dst, const float* src, uint64_t n, float scale) {
    add_scaled_body<float>(dst, src, n, scale);
}
extern "C" __global__ __launch_bounds__(256) void apk_add_scaled_f16(f16_t* dst, const f16_t* src, uint64_t n, float scale) {
    add_scaled_body<f16_t>(dst, src, n, scale);
}

// A per-row bias: x[r][i] += bias[i] (add_bias_rows, crates/allpaka-model/src/model/loader.rs:519-523: the
// projection biases of attention.rs:125-129).  Whole 16-byte tiles where the row length allows, else per element.
template <typename T> DEV void add_bias_rows_body(T* x, const float* bias, uint64_t rows, uint32_t n) {
    constexpr int VEC = io<T>::VEC;
    const uint64_t c = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (n % VEC == 0) {  // uniform
        const uint32_t tiles = n / VEC;
        if (c >= rows * tiles) return;
        const uint32_t col = (uint32_t)(c % tiles) * VEC;
        float v[VEC], b[VEC];
        io<T>::load_nt(x + c * VEC, v);
#pragma unroll
        for (int q = 0; q < VEC; q += 4) io<float>::load(bias + col + q, b + q);
#pragma unroll
        for (int i = 0; i < VEC; i++) v[i] += b[i];
        io<T>::store_wt(x + c * VEC, v);
    } else {
        if (c >= rows * n) return;
        x[c] = (T)((float)x[c] + bias[c % n]);
    }
}
extern "C" __global__ __launch_bounds__(256) void apk_add_bias_rows_f32(float* x, const float* bias, uint64_t rows, uint32_t n) {
    add_bias_rows_body<float>(x, bias, rows, n);
}
extern "C" __global__ __launch_bounds__(256) void apk_add_bias_rows_f16(f16_t* x, const float* bias, uint64_t rows, uint32_t n) {
    add_bias_rows_body<f16_t>(x, bias, rows, n);
}

// Activation type conversion between the reference's f32 and the fp16 storage form (allpaka_dtype::f32_to_f16 /
// f16_to_f32 over slices, crates/allpaka-dtype/src/lib.rs:129-184; the reference's CUDA cast_f32_to_f16 /
// cast_f16_to_f32, gpu/cuda/kernels.rs:448, :3625).  The hardware conversions are the reference's for every finite
// value, infinities and subnormals (round to nearest even; overflow to infinity); NaNs are patched to the reference's
// bits: narrowing gives the canonical quiet NaN sign | 0x7e00, widening keeps the payload (frac << 13) and does not
// quiet a signalling NaN.
DEV uint16_t narrow_ref(float x) {
    const uint32_t b = __builtin_bit_cast(uint32_t, x);
    if ((b & 0x7fffffffu) > 0x7f800000u) return (uint16_t)(((b >> 16) & 0x8000u) | 0x7e00u);
    return __builtin_bit_cast(uint16_t, (f16_t)x);
}
DEV float widen_ref(uint16_t h) {
    if ((h & 0x7c00u) == 0x7c00u && (h & 0x3ffu))
        return __builtin_bit_cast(float, ((uint32_t)(h & 0x8000u) << 16) | 0x7f800000u | ((uint32_t)(h & 0x3ffu) << 13));
    return (float)__builtin_bit_cast(f16_t, h);
}
// Four elements per lane and step (a 16-byte f32 tile against 8 bytes of fp16), two steps a workgroup apart: every
// load and store instruction of a wave covers one contiguous run (two adjacent tiles per lane measured 15 % slower).
extern "C" __global__ __launch_bounds__(256) void apk_cast_f32_f16(const float* src, uint16_t* dst, uint64_t n) {
    const uint64_t nq = n / 4, c0 = (uint64_t)blockIdx.x * (2 * blockDim.x) + threadIdx.x, c1 = c0 + blockDim.x;
    f32x4 a, b;
    if (c0 < nq) a = __builtin_nontemporal_load((const f32x4*)src + c0);
    if (c1 < nq) b = __builtin_nontemporal_load((const f32x4*)src + c1);
    if (c0 < nq) {
        const u32x2 o = {narrow_ref(a.x) | (uint32_t)narrow_ref(a.y) << 16, narrow_ref(a.z) | (uint32_t)narrow_ref(a.w) << 16};
        wt_store(o, (u32x2*)dst + c0);
    }
    if (c1 < nq) {
        const u32x2 o = {narrow_ref(b.x) | (uint32_t)narrow_ref(b.y) << 16, narrow_ref(b.z) | (uint32_t)narrow_ref(b.w) << 16};
        wt_store(o, (u32x2*)dst + c1);
    }
    if (blockIdx.x == gridDim.x - 1)
        for (uint64_t i = nq * 4 + threadIdx.x; i < n; i += blockDim.x) dst[i] = narrow_ref(src[i]);
}
extern "C" __global__ __launch_bounds__(256) void apk_cast_f16_f32(const uint16_t* src, float* dst, uint64_t n) {
    const uint64_t nq = n / 4, c0 = (uint64_t)blockIdx.x * (2 * blockDim.x) + threadIdx.x, c1 = c0 + blockDim.x;
    u32x2 a, b;
    if (c0 < nq) a = __builtin_nontemporal_load((const u32x2*)src + c0);
    if (c1 < nq) b = __builtin_nontemporal_load((const u32x2*)src + c1);
    if (c0 < nq) {
        const f32x4 o = {widen_ref((uint16_t)a.x), widen_ref((uint16_t)(a.x >> 16)), widen_ref((uint16_t)a.y), widen_ref((uint16_t)(a.y >> 16))};
        wt_store(o, (f32x4*)dst + c0);
    }
    if (c1 < nq) {
        const f32x4 o = {widen_ref((uint16_t)b.x), widen_ref((uint16_t)(b.x >> 16)), widen_ref((uint16_t)b.y), widen_ref((uint16_t)(b.y >> 16))};
        wt_store(o, (f32x4*)dst + c1);
    }
    if (blockIdx.x == gridDim.x - 1)
        for (uint64_t i = nq * 4 + threadIdx.x; i < n; i += blockDim.x) dst[i] = widen_ref(src[i]);
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
