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
// One lane decodes one group of eight weights (ojk_iq_grid_rows.h); the matvec bodies are the trait-driven ones the
// other raw-row formats use (ojk_rowdot.h).  The matvec workgroups expand their codebook into LDS first (1 to 16 KB);
// the decoders, eight blocks per workgroup, read the packed table in place.
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
IQ_GRID_NAT(iq2xxs, Iq2xxsW)
IQ_GRID_NAT(iq2xs, Iq2xsW)
IQ_GRID_NAT(iq2s, Iq2sW)
IQ_GRID_NAT(iq3xxs, Iq3xxsW)
IQ_GRID_NAT(iq3s, Iq3sW)
IQ_GRID_NAT(iq1s, Iq1sW)
IQ_GRID_NAT(iq1m, Iq1mW)

// ------------------------------------------------------------------ int8 activations (IQ2_XXS, IQ3_XXS)
// y[n] = sum over blocks b of d * xs[b] * sum over sub-blocks g of scale_g * idot32(w_g, xq_g): the lane's share is
// (d * scale_g) * xs[b] * idot8 of its group, the integer dot exact, the rest a few f32 roundings in another order
// than the CPU's per-sub-block sums (1e-7 of the result).
template <class G, int R, int MODE>
__device__ __forceinline__ void gemv_q8k_grid_body(const signed char* __restrict__ xq, const float* __restrict__ xs,
                                                   const uchar* __restrict__ w, float* __restrict__ y,
                                                   const float* __restrict__ bs, uint K, uint N) {
    G::init();
    __syncthreads();
    const uint lane = threadIdx.x & 63u, t = lane & 31u;
    const uint row0 = (blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)) * R;
    if (row0 >= N) return;
    const uint nu = K >> 8;
    const size_t rb = (size_t)nu * G::BYTES;
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = 0.0f;
    for (uint u = lane >> 5; u < nu; u += 2u) {
        IqgFrag f[R];
#pragma unroll
        for (int r = 0; r < R; r++) f[r] = G::template decode<true>(w + (size_t)min(row0 + r, N - 1u) * rb + (size_t)u * G::BYTES, t);
        const uint2 q = *(const uint2*)(xq + (size_t)u * 256u + t * 8u);
        const float s = xs[u];
#pragma unroll
        for (int r = 0; r < R; r++)
            acc[r] += f[r].dl * s * (float)dot4_i8(f[r].w1, q.y, dot4_i8(f[r].w0, q.x, 0));
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
        gemv_q8k_grid_body<G, 1, ST_SET>(xq, xs, w, y, nullptr, K, N); }                                             \
    extern "C" __global__ void __launch_bounds__(256) gemv_q8k_##FMT##_r2(                                           \
        const signed char* xq, const float* xs, const uchar* w, float* y, uint K, uint N) {                          \
        gemv_q8k_grid_body<G, 2, ST_SET>(xq, xs, w, y, nullptr, K, N); }                                             \
    extern "C" __global__ void __launch_bounds__(256) gemv_q8k_##FMT##_wide(                                         \
        const signed char* xq, const float* xs, const uchar* w, float* y, uint K, uint N) {                          \
        gemv_q8k_grid_body<G, 2, ST_SET>(xq, xs, w, y, nullptr, K, N); }                                             \
    extern "C" __global__ void __launch_bounds__(256) gemv_q8k_##FMT(                                                \
        const signed char* xq, const float* xs, const uchar* w, float* y, uint K, uint N) {                          \
        gemv_q8k_grid_body<G, 4, ST_SET>(xq, xs, w, y, nullptr, K, N); }                                             \
    extern "C" __global__ void __launch_bounds__(256) gemv_q8k_##FMT##_accum(                                        \
        const signed char* xq, const float* xs, const uchar* w, float* y, uint K, uint N) {                          \
        gemv_q8k_grid_body<G, 1, ST_ACCUM>(xq, xs, w, y, nullptr, K, N); }                                           \
    extern "C" __global__ void __launch_bounds__(256) gemv_q8k_##FMT##_bias(                                         \
        const signed char* xq, const float* xs, const uchar* w, float* y, const float* bs, uint K, uint N) {         \
        gemv_q8k_grid_body<G, 1, ST_BIAS>(xq, xs, w, y, bs, K, N); }                                                 \
    extern "C" __global__ void __launch_bounds__(256) gemv_q8k_##FMT##_m(                                            \
        const signed char* xq, const float* xs, const uchar* w, float* y, uint K, uint N, uint M, uint ACC) {        \
        if (M <= 2) gemv_q8k_grid_m_body<G, 2>(xq, xs, w, y, K, N, M, ACC);                                          \
        else gemv_q8k_grid_m_body<G, 4>(xq, xs, w, y, K, N, M, ACC); }
IQ_GRID_Q8K(iq2xxs, Iq2xxsG)
IQ_GRID_Q8K(iq3xxs, Iq3xxsG)
