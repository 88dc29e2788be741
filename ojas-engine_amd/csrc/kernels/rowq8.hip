// Family "rowq8": the row-int8 matmul of the reference's CPU models — weights requantized at load
// time to int8 with one f32 scale per row, activations quantized per whole vector, integer dots,
//   y[t][n] = bias[n] + ((float)(sum_k qw[n][k] * qx[t][k]) * sw[n]) * sx[t]
// (crates/ojas-cpu/src/cpu_math.rs:14-23 `W::Q8`, :174-179 `quant_row_i8`, :187-289 `matmul`,
// :404-415 `dot_i8`; the load-time requantization crates/ojas-formats/src/quant.rs:16-39).
//
//   rows_q8_from_f16(w16, q, scale, K, N)        grid N, block 256: q = clamp(round(w / sv)), sv = amax/127
//   quant_rows_i8(x, q, scale, K, M)             grid M, block 256: q = clamp(round(x * (1/s))), s = amax/127
//   matmul_q8row(xq, sx, wq, sw, y, K, N, M)             grid ceil(N/4), block 256: one wave per row,
//   matmul_q8row_bias(xq, sx, wq, sw, y, bs, K, N, M)    the row read once per 8 tokens
//
// The integer sum is exact, and the three f32 operations of the epilogue are rounded one by one in
// the reference's order (the file is compiled with contraction off), so results are bit-identical
// to the CPU path's.  K must be a multiple of 16.
#include "ojk_common.h"

// amax over a row by all 256 threads of the workgroup
__device__ __forceinline__ float block_amax(float a, float* sh) {
    a = wave_max(a);
    if ((threadIdx.x & 63u) == 0) sh[threadIdx.x >> 6] = a;
    __syncthreads();
    return fmaxf(fmaxf(sh[0], sh[1]), fmaxf(sh[2], sh[3]));
}

extern "C" __global__ void __launch_bounds__(256)
rows_q8_from_f16(const ushort* __restrict__ w16, signed char* __restrict__ q, float* __restrict__ scale, uint K, uint N) {
    __shared__ float sh[4];
    const uint r = blockIdx.x, tid = threadIdx.x;
    const ushort* row = w16 + (size_t)r * K;
    float a = 0.0f;
    for (uint c = tid; c < K; c += 256u) a = fmaxf(a, fabsf(f16_bits_to_f32(row[c])));
    const float amax = block_amax(a, sh);
    const float sv = amax > 0.0f ? __fdiv_rn(amax, 127.0f) : 1.0f;
    if (tid == 0) scale[r] = sv;
    for (uint c = tid; c < K; c += 256u) {
        float v = roundf(__fdiv_rn(f16_bits_to_f32(row[c]), sv));
        q[(size_t)r * K + c] = (signed char)(int)sat127(v);
    }
}

extern "C" __global__ void __launch_bounds__(256)
quant_rows_i8(const float* __restrict__ x, signed char* __restrict__ q, float* __restrict__ scale, uint K, uint M) {
    __shared__ float sh[4];
    const uint r = blockIdx.x, tid = threadIdx.x;
    const float* row = x + (size_t)r * K;
    float a = 0.0f;
    for (uint c = tid; c < K; c += 256u) a = fmaxf(a, fabsf(row[c]));
    const float amax = block_amax(a, sh);
    const float s = amax > 0.0f ? __fdiv_rn(amax, 127.0f) : 1.0f;
    const float inv = __fdiv_rn(1.0f, s);
    if (tid == 0) scale[r] = s;
    for (uint c = tid; c < K; c += 256u) {
        float v = roundf(__fmul_rn(row[c], inv));
        q[(size_t)r * K + c] = (signed char)(int)sat127(v);
    }
}

template <bool BIAS>
__device__ __forceinline__ void matmul_q8row_body(const signed char* __restrict__ xq, const float* __restrict__ sx,
                                                  const signed char* __restrict__ wq, const float* __restrict__ sw,
                                                  float* __restrict__ y, const float* __restrict__ bs, uint K, uint N,
                                                  uint M) {
    constexpr int MT = 8;
    const uint lane = threadIdx.x & 63u;
    const uint row = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (row >= N) return;
    const signed char* wrow = wq + (size_t)row * K;
    const float s_w = sw[row], b = BIAS ? bs[row] : 0.0f;
    for (uint m0 = 0; m0 < M; m0 += MT) {
        int acc[MT];
#pragma unroll
        for (int t = 0; t < MT; t++) acc[t] = 0;
        for (uint k = lane * 16u; k < K; k += 1024u) {
            const uint4 wv = *(const uint4*)(wrow + k);
#pragma unroll
            for (int t = 0; t < MT; t++) {
                const uint m = min(m0 + t, M - 1u);
                const uint4 xv = *(const uint4*)(xq + (size_t)m * K + k);
                acc[t] = dot4_i8(wv.x, xv.x, acc[t]);
                acc[t] = dot4_i8(wv.y, xv.y, acc[t]);
                acc[t] = dot4_i8(wv.z, xv.z, acc[t]);
                acc[t] = dot4_i8(wv.w, xv.w, acc[t]);
            }
        }
#pragma unroll
        for (int t = 0; t < MT; t++) {
            const int s = wave_sum_i32(acc[t]);
            if (lane == 0 && m0 + t < M)
                y[(size_t)(m0 + t) * N + row] = __fadd_rn(b, __fmul_rn(__fmul_rn((float)s, s_w), sx[m0 + t]));
        }
    }
}

extern "C" __global__ void __launch_bounds__(256)
matmul_q8row(const signed char* xq, const float* sx, const signed char* wq, const float* sw, float* y, uint K, uint N,
             uint M) {
    matmul_q8row_body<false>(xq, sx, wq, sw, y, nullptr, K, N, M);
}
extern "C" __global__ void __launch_bounds__(256)
matmul_q8row_bias(const signed char* xq, const float* sx, const signed char* wq, const float* sw, float* y,
                  const float* bs, uint K, uint N, uint M) {
    matmul_q8row_body<true>(xq, sx, wq, sw, y, bs, K, N, M);
}
