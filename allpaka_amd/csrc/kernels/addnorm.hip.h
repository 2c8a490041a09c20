// gfx950 device code, part of apk_kernels.hip (one translation unit, one code object): residual add + RMSNorm over rows.
#pragma once

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

// POST (with a delta): the delta is normalised first, x' = x + rmsnorm(delta) * post_gamma -- the sandwich
// norm of the Gemma family (ops::rmsnorm on the projected row, then add_assign_slice: model/decode.rs:581-584,
// :771-775; the reference's CUDA rmsnorm_add_f32, gpu/cuda/kernels.rs:376-406) -- one more reduction over the
// row's delta tiles, which are in registers already; the delta itself is left as it was.
template <typename T, int NCH, bool HAS_DELTA, bool POST = false>
DEV void add_rmsnorm_impl(T* x, const T* delta, T* h, const float* gamma, int n, float eps, uint32_t vblock,
                          uint32_t rows_per_block, uint32_t rows, const float* post_gamma = nullptr) {
    constexpr int VEC = io<T>::VEC;
    typedef typename stat<T>::acc_t acc_t;
    __shared__ acc_t part[16];
    typedef typename headstat<T>::acc_t dacc_t;  // the delta's norm feeds an addition that can cancel: the reference's values
    __shared__ dacc_t part_d[POST ? 16 : 1];
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
    typename headstat<T>::scale_t dscale{};
    if constexpr (POST) {  // the delta's own statistics
        dacc_t sd = 0;
#pragma unroll
        for (int j = 0; j < NCH; j++) {
            const int c = tid + j * stride;
            float d[VEC];
            io<T>::widen(draw[j], d);
            dacc_t s8 = 0;
#pragma unroll
            for (int i = 0; i < VEC; i++) s8 = headstat<T>::sq(s8, d[i]);
            sd += c < nchunks ? s8 : (dacc_t)0;
        }
        sd = group_sum<64>(sd);
        if (!own_row && blockDim.x > 64) {
            if ((threadIdx.x & 63) == 0) part_d[threadIdx.x >> 6] = sd;
            __syncthreads();
            sd = 0;
            for (int w = 0; w < (int)((blockDim.x + 63) >> 6); w++) sd += part_d[w];
        }
        dscale = headstat<T>::rscale(sd, n, eps);
    }
    acc_t ss = 0;
#pragma unroll
    for (int j = 0; j < NCH; j++) {
        const int c = tid + j * stride;
        io<T>::widen(xraw[j], v[j]);
        if constexpr (HAS_DELTA) {
            float d[VEC];
            io<T>::widen(draw[j], d);
            if constexpr (POST) {
                float pg[VEC];
                const int cc = min(c, nchunks - 1);
#pragma unroll
                for (int q = 0; q < VEC; q += 4) io<float>::load(post_gamma + cc * VEC + q, pg + q);
#pragma unroll
                for (int i = 0; i < VEC; i++) d[i] = headstat<T>::apply(d[i], dscale, pg[i]);
                if constexpr (sizeof(T) == 2) {  // the reference's projected row is an activation: rounded to the storage type
                    // The f32 product is pinned in a register first: left alone the compiler folds "* post_gamma" and
                    // the conversion into one mixed-precision fma that rounds the exact product once to fp16, which
                    // differs from the f32 product rounded to fp16 wherever that product lands on an fp16 tie.
#pragma unroll
                    for (int i = 0; i < VEC; i++) {
                        float r = d[i];
                        asm volatile("" : "+v"(r));
                        d[i] = (float)(T)r;
                    }
                }
            }
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
#define APK_POSTNORM(T, TN, NCH, MAXT)                                                                       \
    extern "C" __global__ __launch_bounds__(MAXT) void apk_postnorm_add_rmsnorm_##TN##_c##NCH(               \
        T* x, const T* delta, T* h, const float* gamma, int n, float eps, uint32_t rows_per_block, uint32_t rows, \
        const float* post_gamma) {                                                                           \
        add_rmsnorm_impl<T, NCH, true, true>(x, delta, h, gamma, n, eps, blockIdx.x, rows_per_block, rows, post_gamma); \
    }
#define APK_ADDNORM_ALL(T, TN)                                                                                   \
    APK_ADDNORM(T, TN, 1, 1024) APK_ADDNORM(T, TN, 2, 1024) APK_ADDNORM(T, TN, 3, 512) APK_ADDNORM(T, TN, 4, 512) \
    APK_ADDNORM(T, TN, 5, 256) APK_ADDNORM(T, TN, 6, 256) APK_ADDNORM(T, TN, 8, 256) APK_ADDNORM(T, TN, 10, 256)  \
    APK_ADDNORM(T, TN, 12, 256) APK_ADDNORM(T, TN, 16, 256) APK_ADDNORM(T, TN, 20, 256)                          \
    APK_POSTNORM(T, TN, 1, 1024) APK_POSTNORM(T, TN, 2, 1024) APK_POSTNORM(T, TN, 3, 512) APK_POSTNORM(T, TN, 4, 512) \
    APK_POSTNORM(T, TN, 5, 256) APK_POSTNORM(T, TN, 6, 256) APK_POSTNORM(T, TN, 8, 256) APK_POSTNORM(T, TN, 10, 256) \
    APK_POSTNORM(T, TN, 12, 256) APK_POSTNORM(T, TN, 16, 256) APK_POSTNORM(T, TN, 20, 256)
APK_ADDNORM_ALL(float, f32)
APK_ADDNORM_ALL(f16_t, f16)
