// gfx950 device code, part of apk_kernels.hip (one translation unit, one code object): MoE combine + residual add + next RMSNorm.
#pragma once

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
                                  uint32_t* fault, uint32_t uniform_k) {
    constexpr int VEC = io<T>::VEC;
    typedef typename stat<T>::acc_t acc_t;
    __shared__ acc_t part[16];
    const int nchunks = n / VEC;
    const uint64_t row = blockIdx.x;
    T* xr = x + row * (uint64_t)n;
    // The token's hits.  Without a tok_off list every token has uniform_k hits (a routed layer without a shared
    // expert: the list would read row * k), and the first dependent load of the chain tok_off -> hit_row -> rows is gone.
    uint32_t h0, h1;
    if (tok_off) {
        h0 = tok_off[row];
        h1 = tok_off[row + 1];
    } else {
        h0 = (uint32_t)row * uniform_k;
        h1 = h0 + uniform_k;
    }
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
    // last row (a cache hit) and add nothing.  The row numbers and weights of the first 2*HB hits (a token's eight
    // experts) are fetched together up front, so the second batch of rows does not wait for a second index fetch.
    auto fetch = [&](uint32_t kb, uint32_t* r, float* w, bool* use) {
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
    };
    auto batch = [&](const uint32_t* r, const float* w, const bool* use) {
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
    };
    if (h1 > h0) {  // uniform
        uint32_t r0[HB], r1[HB];
        float w0[HB], w1[HB];
        bool u0[HB], u1[HB];
        fetch(h0, r0, w0, u0);
        const bool second = h1 - h0 > (uint32_t)HB;
        if (second) fetch(h0 + HB, r1, w1, u1);
        batch(r0, w0, u0);
        if (second) batch(r1, w1, u1);
        for (uint32_t kb = h0 + 2 * HB; kb < h1; kb += HB) {
            fetch(kb, r0, w0, u0);
            batch(r0, w0, u0);
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
        T* h, const float* gamma, int n, float eps, uint32_t* fault, uint32_t uniform_k) {                             \
        combine_add_rmsnorm_body<T, NCH, 4>(x, flat, tok_off, hit_row, hit_w, total_rows, h, gamma, n, eps, fault, uniform_k); \
    }
APK_COMBINE(float, f32, 1) APK_COMBINE(float, f32, 2) APK_COMBINE(float, f32, 4)
APK_COMBINE(f16_t, f16, 1) APK_COMBINE(f16_t, f16, 2) APK_COMBINE(f16_t, f16, 4)
