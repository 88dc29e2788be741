// Family "iq_grid": the grid-codebook GGUF formats — IQ2_XXS (iq2xxs), IQ2_XS (iq2xs), IQ2_S (iq2s), IQ3_XXS (iq3xxs),
// IQ3_S (iq3s), IQ1_S (iq1s), IQ1_M (iq1m) — decoded and multiplied as the file stores them.
//
//   dequant_<fmt>_f16(w, out, nblocks)                      bit-exact with crates/ojas-formats/src/gguf.rs:840-1041
//   gemv_nat_<fmt>{,_r1,_r2,_accum,_bias}(x, w, y[, bs], K, N)     f32 activations, the entry set of the reference's
//   gemv_nat_<fmt>_m(x, w, y, K, N, M, ACC)                        format table (crates/ojas-core/src/quant_src.rs:104-110);
//   gemv_nat_<fmt>_px(x, w, y, K, N)                               on the CPU path dot_iq2xxs / dot_iq3xxs / dot_iq2s /
//                                                                  dot_iq3s (crates/ojas-cpu/src/cpu_math.rs:728-757, :884-941, :1023-1052)
//   gemv_q8k_<fmt>{,_r1,_r2,_wide,_accum,_bias}(xq, xs, w, y[, bs], K, N)   <fmt> = iq2xxs, iq3xxs: int8 activations
//   gemv_q8k_<fmt>_m(xq, xs, w, y, K, N, M, ACC)                   (quant_q8k), integer dots per 32 weights, one
//                                                                  multiply per sub-block: dot_iq2xxs_q8k / dot_iq3xxs_q8k
//                                                                  (cpu_math.rs:1057-1128), what matvec_kq runs for these two
//
// In the decoders and the f32 matvecs of few rows one lane decodes one group of eight weights (ojk_iq_grid_rows.h); the
// matvec bodies are the trait-driven ones the other raw-row formats use (ojk_rowdot.h).  The int8 matvecs and the head
// form (_px) of IQ2_XXS / IQ2_S / IQ3_XXS / IQ3_S give a lane a whole 32-weight sub-block (vals32).  The matvec
// workgroups expand their codebook, and the sign masks, into LDS first (1 to 16 KB); the decoders, eight blocks per
// workgroup, read the packed table in place.
#include "ojk_iq_grid_rows.h"
#include "ojk_rowdot.h"

// ------------------------------------------------------------------ decoders
// 32 threads per block, a thread writes its group's eight values (16 bytes).  dl * (value + delta) is exact in
// f32 and rounded once to f16; the products are explicit so that nothing fuses into a differently rounded form.
template <class G>
__device__ __forceinline__ void dequant_grid_body(const uchar* __restrict__ w, ushort* __restrict__ out, uint nblocks) {
    const size_t tid = (size_t)blockIdx.x * 256u + threadIdx.x;
    const size_t b = tid >> 5;
    if (b >= nblocks) return;
    const uint t = (uint)tid & 31u;
    const IqgFrag f = G::template decode<false>(w + b * G::BYTES, t);
    const float v[8] = {sb0(f.w0), sb1(f.w0), sb2(f.w0), sb3(f.w0), sb0(f.w1), sb1(f.w1), sb2(f.w1), sb3(f.w1)};
    uint o[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        float lo = __fmul_rn(f.dl, __fadd_rn(v[2 * i], f.delta)), hi = __fmul_rn(f.dl, __fadd_rn(v[2 * i + 1], f.delta));
        asm volatile("" : "+v"(lo), "+v"(hi));      // keep "multiply, then convert" two roundings
        o[i] = (uint)__half_as_ushort(__float2half_rn(lo)) | ((uint)__half_as_ushort(__float2half_rn(hi)) << 16);
    }
    *(uint4*)(out + b * 256u + t * 8u) = make_uint4(o[0], o[1], o[2], o[3]);
}

#define IQ_GRID_DEQUANT(FMT, G)                                                                             \
    extern "C" __global__ void __launch_bounds__(256) dequant_##FMT##_f16(                                  \
        const uchar* w, ushort* out, uint nblocks) { dequant_grid_body<G>(w, out, nblocks); }
IQ_GRID_DEQUANT(iq2xxs, Iq2xxsG)
IQ_GRID_DEQUANT(iq2xs, Iq2xsG)
IQ_GRID_DEQUANT(iq2s, Iq2sG)
IQ_GRID_DEQUANT(iq3xxs, Iq3xxsG)
IQ_GRID_DEQUANT(iq3s, Iq3sG)
IQ_GRID_DEQUANT(iq1s, Iq1sG)
IQ_GRID_DEQUANT(iq1m, Iq1mG)

// ------------------------------------------------------------------ f32 activations
#define IQ_GRID_NAT(FMT, W)                                                                                 \
    template <int R, int MODE>                                                                              \
    __device__ __forceinline__ void gemv_nat_##FMT##_body(const float* x, const uchar* w, float* y,         \
                                                          const float* bs, uint K, uint N) {                \
        W::init();                                                                                          \
        __syncthreads();                                                                                    \
        gemv_nat_iq4_body<W, R, MODE>(x, w, y, bs, K, N); }                                                 \
    template <int MT>                                                                                       \
    __device__ __forceinline__ void gemv_nat_##FMT##_m_body(const float* x, const uchar* w, float* y,       \
                                                            uint K, uint N, uint M, uint ACC) {             \
        W::init();                                                                                          \
        __syncthreads();                                                                                    \
        gemv_nat_iq4_m_body<W, MT>(x, w, y, K, N, M, ACC); }                                                \
    GEMV_NAT_ENTRIES(FMT)                                                                                   \
    extern "C" __global__ void __launch_bounds__(256) gemv_nat_##FMT##_px(                                  \
        const float* x, const uchar* w, float* y, uint K, uint N) {                                         \
        W::init();                                                                                          \
        __syncthreads();                                                                                    \
        gemv_nat_iq4_px_body<W, 8>(x, w, y, K, N); }
// An output head of IQ2_XXS / IQ2_S / IQ3_XXS / IQ3_S rows: a lane per 32-weight sub-block (eight lanes a block, eight
// blocks a step, a sub-block's bytes in two to four loads, entries and sign masks from LDS), rows grid-stride two at a
// time, the lane's 32 activations of each of its (at most two) steps in registers.  A lane's term is
// dl0 (w . x over its first sixteen) + dl1 (... second sixteen): per weight a fifth of the load instructions of the
// group-per-lane form and half of its vector arithmetic.  K <= 4096.
template <class G>
__device__ __forceinline__ void gemv_nat_grid32_px_body(const float* __restrict__ x, const uchar* __restrict__ w,
                                                        float* __restrict__ y, uint K, uint N) {
    G::init();
    G::signs_init();
    __syncthreads();
    constexpr int NS = 2;
    const uint lane = threadIdx.x & 63u, ib = lane & 7u;
    const uint nu = K >> 8;
    const size_t rb = (size_t)nu * G::BYTES;
    float4 xr[NS][8];
    uint uc[NS];
#pragma unroll
    for (int s = 0; s < NS; s++) {
        const uint u = (lane >> 3) + 8u * (uint)s;
        uc[s] = min(u, nu - 1u);
#pragma unroll
        for (int j = 0; j < 8; j++)
            xr[s][j] = u < nu ? *(const float4*)(x + (size_t)u * 256u + ib * 32u + 4u * (uint)j) : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    }
    const uint nwaves = gridDim.x * (blockDim.x >> 6);
    for (uint row0 = (blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)) * 2u; row0 < N; row0 += nwaves * 2u) {
        const uchar* rp[2] = {w + (size_t)row0 * rb, w + (size_t)min(row0 + 1u, N - 1u) * rb};
        float acc[2] = {0.0f, 0.0f};
#pragma unroll
        for (int s = 0; s < NS; s++)
#pragma unroll
            for (int r = 0; r < 2; r++) {
                uint wv[8];
                float dl0, dl1;
                G::vals32(rp[r] + (size_t)uc[s] * G::BYTES, ib, wv, dl0, dl1);
                float h[2];
#pragma unroll
                for (int hh = 0; hh < 2; hh++) {
                    float a = 0.0f;
#pragma unroll
                    for (int j = 4 * hh; j < 4 * hh + 4; j++) {
                        a = fmaf(sb0(wv[j]), xr[s][j].x, a);
                        a = fmaf(sb1(wv[j]), xr[s][j].y, a);
                        a = fmaf(sb2(wv[j]), xr[s][j].z, a);
                        a = fmaf(sb3(wv[j]), xr[s][j].w, a);
                    }
                    h[hh] = a;
                }
                acc[r] += dl0 * h[0] + dl1 * h[1];
            }
        const float a0 = wave_sum(acc[0]), a1 = wave_sum(acc[1]);
        if (lane == 0) {
            y[row0] = a0;
            if (row0 + 1u < N) y[row0 + 1u] = a1;
        }
    }
}
#define IQ_GRID_NAT32(FMT, W, G)                                                                            \
    template <int R, int MODE>                                                                              \
    __device__ __forceinline__ void gemv_nat_##FMT##_body(const float* x, const uchar* w, float* y,         \
                                                          const float* bs, uint K, uint N) {                \
        W::init();                                                                                          \
        __syncthreads();                                                                                    \
        gemv_nat_iq4_body<W, R, MODE>(x, w, y, bs, K, N); }                                                 \
    template <int MT>                                                                                       \
    __device__ __forceinline__ void gemv_nat_##FMT##_m_body(const float* x, const uchar* w, float* y,       \
                                                            uint K, uint N, uint M, uint ACC) {             \
        W::init();                                                                                          \
        __syncthreads();                                                                                    \
        gemv_nat_iq4_m_body<W, MT>(x, w, y, K, N, M, ACC); }                                                \
    GEMV_NAT_ENTRIES(FMT)                                                                                   \
    extern "C" __global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4, 4))) gemv_nat_##FMT##_px( \
        const float* x, const uchar* w, float* y, uint K, uint N) {                                         \
        gemv_nat_grid32_px_body<G>(x, w, y, K, N); }
IQ_GRID_NAT32(iq2xxs, Iq2xxsW, Iq2xxsG)
IQ_GRID_NAT(iq2xs, Iq2xsW)
IQ_GRID_NAT32(iq2s, Iq2sW, Iq2sG)
IQ_GRID_NAT32(iq3xxs, Iq3xxsW, Iq3xxsG)
IQ_GRID_NAT32(iq3s, Iq3sW, Iq3sG)
IQ_GRID_NAT(iq1s, Iq1sW)
IQ_GRID_NAT(iq1m, Iq1mW)

// ------------------------------------------------------------------ int8 activations (IQ2_XXS, IQ3_XXS)
// y[n] = sum over blocks b of d * xs[b] * sum over sub-blocks g of scale_g * idot32(w_g, xq_g).  A lane per 32-weight
// sub-block: eight lanes a block, eight blocks (2048 weights) a step, the sub-block's eight bytes (IQ3_XXS: twelve) in
// one or two loads, codebook entries and sign masks from LDS.  A lane's term is xs (d scale idot32) — the CPU's
// per-sub-block product, the integer dot exact — and the terms meet in another order than the CPU's (1e-7 of the
// result).  (A lane per group of eight weights, as the f32 entries below the head form have it, took five narrow loads
// per eight weights: 94 us on a 128256 x 4096 head against 42.)
template <class G, int R, int MODE>
__device__ __forceinline__ void gemv_q8k_grid32_body(const signed char* __restrict__ xq, const float* __restrict__ xs,
                                                     const uchar* __restrict__ w, float* __restrict__ y,
                                                     const float* __restrict__ bs, uint K, uint N) {
    G::init();
    G::signs_init();
    __syncthreads();
    const uint lane = threadIdx.x & 63u, ib = lane & 7u;
    const uint row0 = (blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)) * R;
    if (row0 >= N) return;
    const uint nu = K >> 8;
    const size_t rb = (size_t)nu * G::BYTES;
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = 0.0f;
    for (uint u = lane >> 3; u < nu; u += 8u) {
        const uint4 qa = *(const uint4*)(xq + (size_t)u * 256u + ib * 32u), qb = *(const uint4*)(xq + (size_t)u * 256u + ib * 32u + 16u);
        const uint q[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
        const float s = xs[u];
#pragma unroll
        for (int r = 0; r < R; r++) {
            uint wv[8];
            float dl0, dl1;
            G::vals32(w + (size_t)min(row0 + r, N - 1u) * rb + (size_t)u * G::BYTES, ib, wv, dl0, dl1);
            int isum = 0;
#pragma unroll
            for (int j = 0; j < 8; j++) isum = dot4_i8(wv[j], q[j], isum);
            acc[r] += s * (dl0 * (float)isum);          // IQ2_XXS, IQ3_XXS: one scale per sub-block
        }
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
        const float v = wave_sum(acc[r]);
        if (lane == 0 && row0 + r < N) store_row<MODE>(y, bs, row0 + r, v);
    }
}

template <class G, int MT>
__device__ __forceinline__ void gemv_q8k_grid_m_body(const signed char* __restrict__ xq, const float* __restrict__ xs,
                                                     const uchar* __restrict__ w, float* __restrict__ y, uint K, uint N,
                                                     uint M, uint ACC) {
    G::init();
    __syncthreads();
    const uint lane = threadIdx.x & 63u, t = lane & 31u;
    const uint row = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (row >= N) return;
    const uint nu = K >> 8;
    const uchar* wr = w + (size_t)row * nu * G::BYTES;
    for (uint m0 = 0; m0 < M; m0 += MT) {
        float acc[MT];
#pragma unroll
        for (int i = 0; i < MT; i++) acc[i] = 0.0f;
        for (uint u = lane >> 5; u < nu; u += 2u) {
            const IqgFrag f = G::template decode<true>(wr + (size_t)u * G::BYTES, t);
#pragma unroll
            for (int i = 0; i < MT; i++) {
                const uint m = min(m0 + i, M - 1u);
                const uint2 q = *(const uint2*)(xq + (size_t)m * K + (size_t)u * 256u + t * 8u);
                acc[i] += f.dl * xs[(size_t)m * nu + u] * (float)dot4_i8(f.w1, q.y, dot4_i8(f.w0, q.x, 0));
            }
        }
#pragma unroll
        for (int i = 0; i < MT; i++) {
            const float v = wave_sum(acc[i]);
            if (lane == 0 && m0 + i < M) {
                float* o = y + (size_t)(m0 + i) * N + row;
                *o = ACC ? *o + v : v;
            }
        }
    }
}

#define IQ_GRID_Q8K(FMT, G)                                                                                          \
    extern "C" __global__ void __launch_bounds__(256) gemv_q8k_##FMT##_r1(                                           \
        const signed char* xq, const float* xs, const uchar* w, float* y, uint K, uint N) {                          \
        gemv_q8k_grid32_body<G, 1, ST_SET>(xq, xs, w, y, nullptr, K, N); }                                             \
    extern "C" __global__ void __launch_bounds__(256) gemv_q8k_##FMT##_r2(                                           \
        const signed char* xq, const float* xs, const uchar* w, float* y, uint K, uint N) {                          \
        gemv_q8k_grid32_body<G, 2, ST_SET>(xq, xs, w, y, nullptr, K, N); }                                             \
    extern "C" __global__ void __launch_bounds__(256) gemv_q8k_##FMT##_wide(                                         \
        const signed char* xq, const float* xs, const uchar* w, float* y, uint K, uint N) {                          \
        gemv_q8k_grid32_body<G, 2, ST_SET>(xq, xs, w, y, nullptr, K, N); }                                             \
    extern "C" __global__ void __launch_bounds__(256) gemv_q8k_##FMT(                                                \
        const signed char* xq, const float* xs, const uchar* w, float* y, uint K, uint N) {                          \
        gemv_q8k_grid32_body<G, 4, ST_SET>(xq, xs, w, y, nullptr, K, N); }                                             \
    extern "C" __global__ void __launch_bounds__(256) gemv_q8k_##FMT##_accum(                                        \
        const signed char* xq, const float* xs, const uchar* w, float* y, uint K, uint N) {                          \
        gemv_q8k_grid32_body<G, 1, ST_ACCUM>(xq, xs, w, y, nullptr, K, N); }                                           \
    extern "C" __global__ void __launch_bounds__(256) gemv_q8k_##FMT##_bias(                                         \
        const signed char* xq, const float* xs, const uchar* w, float* y, const float* bs, uint K, uint N) {         \
        gemv_q8k_grid32_body<G, 1, ST_BIAS>(xq, xs, w, y, bs, K, N); }                                                 \
    extern "C" __global__ void __launch_bounds__(256) gemv_q8k_##FMT##_m(                                            \
        const signed char* xq, const float* xs, const uchar* w, float* y, uint K, uint N, uint M, uint ACC) {        \
        if (M <= 2) gemv_q8k_grid_m_body<G, 2>(xq, xs, w, y, K, N, M, ACC);                                          \
        else gemv_q8k_grid_m_body<G, 4>(xq, xs, w, y, K, N, M, ACC); }
IQ_GRID_Q8K(iq2xxs, Iq2xxsG)
IQ_GRID_Q8K(iq3xxs, Iq3xxsG)
