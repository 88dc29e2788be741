// Matvec bodies driven by a row trait (ojk_rows.h, ojk_iq_grid_rows.h): raw rows of a block format against f32
// activations, shared by the code objects that hold such formats.  A trait W gives the lane map of one wave step
// and load / dot for the lane's fragment of a block.
#pragma once
#include "ojk_common.h"

enum { ST_SET = 0, ST_ACCUM = 1, ST_BIAS = 2 };

template <int MODE>
__device__ __forceinline__ void store_row(float* y, const float* bs, uint n, float v) {
    if (MODE == ST_SET) y[n] = v;
    else if (MODE == ST_ACCUM) y[n] += v;
    else y[n] = v + bs[n];
}

template <class W, int R, int MODE>
__device__ __forceinline__ void gemv_nat_iq4_body(const float* __restrict__ x, const uchar* __restrict__ w,
                                                  float* __restrict__ y, const float* __restrict__ bs,
                                                  uint K, uint N) {
    const uint lane = threadIdx.x & 63u;
    const uint row0 = (blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)) * R;
    if (row0 >= N) return;
    const uint nu = W::units(K);
    const size_t rb = (size_t)nu * W::BYTES;
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = 0.0f;
    for (uint u = W::unit_of(lane); u < nu; u += W::STEP) {
        typename W::Frag f[R];
#pragma unroll
        for (int r = 0; r < R; r++) f[r] = W::load(w + (size_t)min(row0 + r, N - 1u) * rb, u, lane);
        const float* xp = x + (size_t)u * W::x_unit(0) + W::x_off(lane);
        const float4 x0 = *(const float4*)xp, x1 = *(const float4*)(xp + W::XGAP);
        const float xsum = sum4(x0) + sum4(x1);      // for the formats with an offset or a minimum
#pragma unroll
        for (int r = 0; r < R; r++) acc[r] += W::dot(f[r], lane, x0, x1, xsum);
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
        float s = wave_sum(acc[r]);
        if (lane == 0 && row0 + r < N) store_row<MODE>(y, bs, row0 + r, s);
    }
}

template <class W, int MT>
__device__ __forceinline__ void gemv_nat_iq4_m_body(const float* __restrict__ x, const uchar* __restrict__ w,
                                                    float* __restrict__ y, uint K, uint N, uint M, uint ACC) {
    const uint lane = threadIdx.x & 63u;
    const uint row = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (row >= N) return;
    const uint nu = W::units(K);
    const uchar* wr = w + (size_t)row * nu * W::BYTES;
    for (uint m0 = 0; m0 < M; m0 += MT) {
        float acc[MT];
#pragma unroll
        for (int i = 0; i < MT; i++) acc[i] = 0.0f;
        for (uint u = W::unit_of(lane); u < nu; u += W::STEP) {
            const typename W::Frag f = W::load(wr, u, lane);
#pragma unroll
            for (int i = 0; i < MT; i++) {
                const uint m = min(m0 + i, M - 1u);
                const float* xp = x + (size_t)m * K + (size_t)u * W::x_unit(0) + W::x_off(lane);
                const float4 x0 = *(const float4*)xp, x1 = *(const float4*)(xp + W::XGAP);
                acc[i] += W::dot(f, lane, x0, x1, sum4(x0) + sum4(x1));
            }
        }
#pragma unroll
        for (int i = 0; i < MT; i++) {
            float s = wave_sum(acc[i]);
            if (lane == 0 && m0 + i < M) {
                float* o = y + (size_t)(m0 + i) * N + row;
                *o = ACC ? *o + s : s;
            }
        }
    }
}

// Many rows (an output head): a 4-bit row is an eighth of the bytes of the f32 activations it meets, so
// a wave that fetches its activation fragments again for every few rows is bound by those loads, not
// by HBM (2.7 TB/s at 128256 x 4096).  Here rows are grid-stride and the wave keeps its share of x —
// 8 floats per lane and step, NS steps — in registers for the whole launch; out-of-range steps hold
// zeros and repeat the last block.   gemv_nat_iq4{nl,xs}_px(x, w, y, K, N), K <= 4096 (64 floats of x per
// lane; twice that would halve the resident waves).
template <class W, int NS>
__device__ __forceinline__ void gemv_nat_iq4_px_body(const float* __restrict__ x, const uchar* __restrict__ w,
                                                     float* __restrict__ y, uint K, uint N) {
    const uint lane = threadIdx.x & 63u;
    const uint nu = W::units(K);
    const size_t rb = (size_t)nu * W::BYTES;
    float4 xr[NS][2];
    float xsum[NS];
    uint uc[NS];
#pragma unroll
    for (int s = 0; s < NS; s++) {
        const uint u = W::unit_of(lane) + (uint)s * W::STEP;
        uc[s] = min(u, nu - 1u);
        xr[s][0] = xr[s][1] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        if (u < nu) {
            const float* xp = x + (size_t)u * W::x_unit(0) + W::x_off(lane);
            xr[s][0] = *(const float4*)xp;
            xr[s][1] = *(const float4*)(xp + W::XGAP);
        }
        xsum[s] = sum4(xr[s][0]) + sum4(xr[s][1]);
    }
    const uint nwaves = gridDim.x * (blockDim.x >> 6);
    for (uint row0 = (blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)) * 2u; row0 < N; row0 += nwaves * 2u) {
        const uchar* r0 = w + (size_t)row0 * rb;
        const uchar* r1 = w + (size_t)min(row0 + 1u, N - 1u) * rb;
        float a0 = 0.0f, a1 = 0.0f;
#pragma unroll
        for (int s = 0; s < NS; s++) {
            const typename W::Frag f0 = W::load(r0, uc[s], lane), f1 = W::load(r1, uc[s], lane);
            a0 += W::dot(f0, lane, xr[s][0], xr[s][1], xsum[s]);
            a1 += W::dot(f1, lane, xr[s][0], xr[s][1], xsum[s]);
        }
        a0 = wave_sum(a0);
        a1 = wave_sum(a1);
        if (lane == 0) {
            y[row0] = a0;
            if (row0 + 1u < N) y[row0 + 1u] = a1;
        }
    }
}

// The head form with a lane per 32-weight group: lane l of step s owns group l + 64 s of the row (its 16 code bytes in
// one load where the group-per-four-lanes map above issues four narrow ones — the address unit of the vector memory
// path takes a wave-wide load about as long whatever its width, and bounds those launches) and keeps the group's 32
// activations, and their sum, in registers.  A trait T gives row_bytes(K) and dot32(row, group, x[8], xsum): the
// group's term with its scale.  K <= 4096 (two steps).
template <class T>
__device__ __forceinline__ void gemv_nat_sub32_px_body(const float* __restrict__ x, const uchar* __restrict__ w,
                                                       float* __restrict__ y, uint K, uint N) {
    constexpr int NS = 2;
    const uint lane = threadIdx.x & 63u, nsub = K >> 5;
    const size_t rb = T::row_bytes(K);
    float4 xr[NS][8];
    float xsum[NS];
    uint sc[NS];
#pragma unroll
    for (int s = 0; s < NS; s++) {
        const uint sub = lane + 64u * (uint)s;
        sc[s] = min(sub, nsub - 1u);
        float t = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            xr[s][j] = sub < nsub ? *(const float4*)(x + (size_t)sub * 32u + 4u * (uint)j) : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            t += (xr[s][j].x + xr[s][j].y) + (xr[s][j].z + xr[s][j].w);
        }
        xsum[s] = t;
    }
    const uint nwaves = gridDim.x * (blockDim.x >> 6);
    for (uint row0 = (blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)) * 2u; row0 < N; row0 += nwaves * 2u) {
        const uchar* r0 = w + (size_t)row0 * rb;
        const uchar* r1 = w + (size_t)min(row0 + 1u, N - 1u) * rb;
        float a0 = 0.0f, a1 = 0.0f;
#pragma unroll
        for (int s = 0; s < NS; s++) {
            a0 += T::dot32(r0, sc[s], xr[s], xsum[s]);
            a1 += T::dot32(r1, sc[s], xr[s], xsum[s]);
        }
        a0 = wave_sum(a0);
        a1 = wave_sum(a1);
        if (lane == 0) {
            y[row0] = a0;
            if (row0 + 1u < N) y[row0 + 1u] = a1;
        }
    }
}
#define GEMV_NAT_SUB32_PX(FMT, T)                                                                          \
    extern "C" __global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4, 4)))           \
    gemv_nat_##FMT##_px(const float* x, const uchar* w, float* y, uint K, uint N) {                        \
        gemv_nat_sub32_px_body<T>(x, w, y, K, N); }

#define GEMV_NAT_IQ4_PX(FMT, W)                                                                            \
    extern "C" __global__ void __launch_bounds__(256) gemv_nat_##FMT##_px(                                 \
        const float* x, const uchar* w, float* y, uint K, uint N) {                                        \
        gemv_nat_iq4_px_body<W, 8>(x, w, y, K, N); }

// The reference's entry set of one format: gemv_nat_<fmt>{,_r1,_r2,_accum,_bias,_m}, over gemv_nat_<fmt>_body<R, MODE>
// and gemv_nat_<fmt>_m_body<MT>.
#define GEMV_NAT_ENTRIES(FMT)                                                                              \
    extern "C" __global__ void __launch_bounds__(256) gemv_nat_##FMT##_r1(                                 \
        const float* x, const uchar* w, float* y, uint K, uint N) {                                        \
        gemv_nat_##FMT##_body<1, ST_SET>(x, w, y, nullptr, K, N); }                                        \
    extern "C" __global__ void __launch_bounds__(256) gemv_nat_##FMT##_r2(                                 \
        const float* x, const uchar* w, float* y, uint K, uint N) {                                        \
        gemv_nat_##FMT##_body<2, ST_SET>(x, w, y, nullptr, K, N); }                                        \
    extern "C" __global__ void __launch_bounds__(256) gemv_nat_##FMT(                                      \
        const float* x, const uchar* w, float* y, uint K, uint N) {                                        \
        gemv_nat_##FMT##_body<4, ST_SET>(x, w, y, nullptr, K, N); }                                        \
    extern "C" __global__ void __launch_bounds__(256) gemv_nat_##FMT##_accum(                              \
        const float* x, const uchar* w, float* y, uint K, uint N) {                                        \
        gemv_nat_##FMT##_body<4, ST_ACCUM>(x, w, y, nullptr, K, N); }                                      \
    extern "C" __global__ void __launch_bounds__(256) gemv_nat_##FMT##_bias(                               \
        const float* x, const uchar* w, float* y, const float* bs, uint K, uint N) {                       \
        gemv_nat_##FMT##_body<4, ST_BIAS>(x, w, y, bs, K, N); }                                            \
    extern "C" __global__ void __launch_bounds__(256) gemv_nat_##FMT##_m(                                  \
        const float* x, const uchar* w, float* y, uint K, uint N, uint M, uint ACC) {                      \
        if (M <= 2) gemv_nat_##FMT##_m_body<2>(x, w, y, K, N, M, ACC);                                     \
        else gemv_nat_##FMT##_m_body<4>(x, w, y, K, N, M, ACC); }

