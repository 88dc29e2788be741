// Family "q80_dp4a": GGUF block_q8_0 rows (34 bytes per 32 weights: an f16 scale, 32 int8) read as the file
// stores them, against activations quantized to int8 per 32 values, integer dots: the reference's GPU decode
// path for Q8_0 models and its fusions (crates/ojas-cuda/src/kernels/gemv_q8.rs:152-260; the quantizer
// crates/ojas-cuda/src/kernels/gemv.rs:33-52).  Names, arguments and arithmetic are the reference's:
//
//   quantize_q8_1(x, q8, d8, d8sum, K)                         per block of 32: d8 = amax / 127,
//                                                              q = clamp(rn(x * (1 / d8)), -127, 127), d8sum = d8 * sum q
//   gemv_q80_dp4a(w, q8, d8, y, K, N)                          y[n]  = dot(n)
//   gemv_q80_dp4a_bias(w, q8, d8, y, bias, K, N)               y[n]  = dot(n) + bias[n]
//   gemv_q80_dp4a_accum(w, q8, d8, y, K, N)                    y[n] += dot(n)
//   qkv_q80_dp4a(wq, wk, wv, q8, d8, q, k, v, bias, K, Nq, Nkv)   Nq + 2 Nkv rows of three tensors in one launch,
//                                                              bias[Nq + 2 Nkv] added (the reference accepts a null
//                                                              bias; a launch through this library passes zeros)
//   ffn_gu_q80_dp4a(wg, wu, q8, d8, out, K, N, act)            out[n] = act(gate(n)) * up(n); act 0 SiLU, 1 GELU
//   dot(n) = sum over blocks b and quarters s of  dw[n][b] * d8[b] * (float) idot8(w[n][b][8 s ..], q8[32 b + 8 s ..])
//
// Launches: quantize_q8_1 grid [ceil(K / 256)] x 256 (the reference: one 32-lane warp per block; here a 64-wide
// wave holds two blocks, the reductions stay inside 32 lanes); the matvecs grid [ceil(rows / 8)] x 256, two rows
// per wave (ffn_gu: grid [ceil(N / 4)], a wave's two streams are the gate and up rows of one output).
//
// CDNA4 plan.  As in the reference four lanes share a block, so a wave covers 16 consecutive blocks, 544
// contiguous bytes, per step, and a row's 8-byte weight pieces (2 bytes past a 34-byte boundary: even, seldom
// dword aligned) load as two dwords each.  A step's loads for both streams are issued before its dots; four
// steps are unrolled so that 4 KB per wave are on their way.  v_dot4_i32_i8 does the integer work: two
// instructions per 8 weights against 16 fused multiply-adds and 8 conversions on the f32-activation path.
#include "ojk_common.h"

// Metal's ffn_act as the reference's GPU kernels carry it (crates/ojas-cuda/src/kernels/gemv_q8.rs:20-28):
// act 1 = GELU, tanh form, its argument clamped to +-30; otherwise SiLU.
__device__ __forceinline__ float q80_ffn_act(float g, uint act) {
    if (act == 1u) {
        float inner = 0.7978845608f * (g + 0.044715f * g * g * g);
        inner = fminf(fmaxf(inner, -30.0f), 30.0f);
        return 0.5f * g * (1.0f + tanhf(inner));
    }
    return g / (1.0f + expf(-g));
}

extern "C" __global__ void __launch_bounds__(256)
quantize_q8_1(const float* __restrict__ x, signed char* __restrict__ q8, float* __restrict__ d8, float* __restrict__ d8sum,
              uint K) {
    const uint i = blockIdx.x * 256u + threadIdx.x;
    const bool on = i < K;
    const float v = on ? x[i] : 0.0f;
    float a = fabsf(v);
    a = fmaxf(a, dpp_f32<OJK_DPP_QUAD_XOR1>(a));
    a = fmaxf(a, dpp_f32<OJK_DPP_QUAD_XOR2>(a));
    a = fmaxf(a, dpp_f32<OJK_DPP_ROW_HALF_MIRROR>(a));
    a = fmaxf(a, dpp_f32<OJK_DPP_ROW_MIRROR>(a));
    a = fmaxf(a, __shfl_xor(a, 16, 64));
    const float d = __fdiv_rn(a, 127.0f);
    const float id = d > 0.0f ? __fdiv_rn(1.0f, d) : 0.0f;
    const float qf = sat127(rintf(__fmul_rn(v, id)));      // a NaN product (0 * inf) is code 0, as __float2int_rn gives
    float s = qf;
    s += dpp_f32<OJK_DPP_QUAD_XOR1>(s);
    s += dpp_f32<OJK_DPP_QUAD_XOR2>(s);
    s += dpp_f32<OJK_DPP_ROW_HALF_MIRROR>(s);
    s += dpp_f32<OJK_DPP_ROW_MIRROR>(s);
    s += __shfl_xor(s, 16, 64);                            // whole numbers up to 32 * 127: exact in any order
    if (on) {
        q8[i] = (signed char)(int)qf;
        if ((threadIdx.x & 31u) == 0u) {
            d8[i >> 5] = d;
            d8sum[i >> 5] = __fmul_rn(d, s);
        }
    }
}

// Two weight streams (rows r0, r1: any two rows of block_q8_0, possibly of different tensors) against one
// quantized activation vector; every lane returns both row sums.
__device__ __forceinline__ void q80_two_rows(const uchar* __restrict__ r0, const uchar* __restrict__ r1,
                                             const signed char* __restrict__ q8, const float* __restrict__ d8, uint nblk,
                                             float& s0, float& s1) {
    const uint lane = threadIdx.x & 63u, sub = lane & 3u, b0 = lane >> 2;
    float a0 = 0.0f, a1 = 0.0f;
    for (uint base = 0; base < nblk; base += 64u) {
        u32x2_a2 w0[4], w1[4];
        ushort h0[4], h1[4];
        uint2 xq[4];
        float dx[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const uint blk = min(base + 16u * (uint)u + b0, nblk - 1u);      // steps past the row's end repeat its last block
            const size_t o = (size_t)blk * 34u;
            h0[u] = *(const ushort*)(r0 + o);
            w0[u] = *(const u32x2_a2*)(r0 + o + 2u + sub * 8u);
            h1[u] = *(const ushort*)(r1 + o);
            w1[u] = *(const u32x2_a2*)(r1 + o + 2u + sub * 8u);
            xq[u] = *(const uint2*)(q8 + (size_t)blk * 32u + sub * 8u);
            dx[u] = d8[blk];
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const bool on = base + 16u * (uint)u + b0 < nblk;
            int i0 = dot4_i8(w0[u].x, xq[u].x, 0), i1 = dot4_i8(w1[u].x, xq[u].x, 0);
            i0 = dot4_i8(w0[u].y, xq[u].y, i0);
            i1 = dot4_i8(w1[u].y, xq[u].y, i1);
            const float t0 = f16_bits_to_f32(h0[u]) * dx[u] * (float)i0, t1 = f16_bits_to_f32(h1[u]) * dx[u] * (float)i1;
            a0 += on ? t0 : 0.0f;
            a1 += on ? t1 : 0.0f;
        }
    }
    s0 = wave_sum(a0);
    s1 = wave_sum(a1);
}

template <int MODE>   // 0 store, 1 + bias, 2 accumulate
__device__ __forceinline__ void gemv_q80_dp4a_body(const uchar* __restrict__ w, const signed char* __restrict__ q8,
                                                   const float* __restrict__ d8, float* __restrict__ y,
                                                   const float* __restrict__ bias, uint K, uint N) {
    const uint n0 = (blockIdx.x * 4u + (threadIdx.x >> 6)) * 2u;
    if (n0 >= N) return;
    const uint nblk = K >> 5, n1 = min(n0 + 1u, N - 1u);
    const size_t rb = (size_t)nblk * 34u;
    float s0, s1;
    q80_two_rows(w + (size_t)n0 * rb, w + (size_t)n1 * rb, q8, d8, nblk, s0, s1);
    if ((threadIdx.x & 63u) == 0u) {
        y[n0] = MODE == 1 ? s0 + bias[n0] : MODE == 2 ? y[n0] + s0 : s0;
        if (n0 + 1u < N) y[n1] = MODE == 1 ? s1 + bias[n1] : MODE == 2 ? y[n1] + s1 : s1;
    }
}
extern "C" __global__ void __launch_bounds__(256)
gemv_q80_dp4a(const uchar* w, const signed char* q8, const float* d8, float* y, uint K, uint N) {
    gemv_q80_dp4a_body<0>(w, q8, d8, y, nullptr, K, N);
}
extern "C" __global__ void __launch_bounds__(256)
gemv_q80_dp4a_bias(const uchar* w, const signed char* q8, const float* d8, float* y, const float* bias, uint K, uint N) {
    gemv_q80_dp4a_body<1>(w, q8, d8, y, bias, K, N);
}
extern "C" __global__ void __launch_bounds__(256)
gemv_q80_dp4a_accum(const uchar* w, const signed char* q8, const float* d8, float* y, uint K, uint N) {
    gemv_q80_dp4a_body<2>(w, q8, d8, y, nullptr, K, N);
}

extern "C" __global__ void __launch_bounds__(256)
qkv_q80_dp4a(const uchar* wq_, const uchar* wk_, const uchar* wv_, const signed char* q8, const float* d8, float* q,
             float* k, float* v, const float* bias, uint K, uint Nq, uint Nkv) {
    const uint total = Nq + 2u * Nkv;
    const uint n0 = (blockIdx.x * 4u + (threadIdx.x >> 6)) * 2u;
    if (n0 >= total) return;
    const uint nblk = K >> 5;
    const size_t rb = (size_t)nblk * 34u;
    const uchar* rows[2];
    float* outs[2];
    uint at[2];
#pragma unroll
    for (int r = 0; r < 2; r++) {
        const uint n = min(n0 + (uint)r, total - 1u);
        at[r] = n;
        if (n < Nq) { rows[r] = wq_ + (size_t)n * rb; outs[r] = q + n; }
        else if (n < Nq + Nkv) { rows[r] = wk_ + (size_t)(n - Nq) * rb; outs[r] = k + (n - Nq); }
        else { rows[r] = wv_ + (size_t)(n - Nq - Nkv) * rb; outs[r] = v + (n - Nq - Nkv); }
    }
    float s0, s1;
    q80_two_rows(rows[0], rows[1], q8, d8, nblk, s0, s1);
    if ((threadIdx.x & 63u) == 0u) {
        *outs[0] = s0 + bias[at[0]];
        if (n0 + 1u < total) *outs[1] = s1 + bias[at[1]];
    }
}

extern "C" __global__ void __launch_bounds__(256)
ffn_gu_q80_dp4a(const uchar* wg, const uchar* wu, const signed char* q8, const float* d8, float* out, uint K, uint N,
                uint act) {
    const uint n = blockIdx.x * 4u + (threadIdx.x >> 6);
    if (n >= N) return;
    const uint nblk = K >> 5;
    const size_t rb = (size_t)nblk * 34u;
    float g, u;
    q80_two_rows(wg + (size_t)n * rb, wu + (size_t)n * rb, q8, d8, nblk, g, u);
    if ((threadIdx.x & 63u) == 0u) out[n] = q80_ffn_act(g, act) * u;
}
