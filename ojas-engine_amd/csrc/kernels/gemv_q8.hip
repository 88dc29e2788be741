// Family "gemv_q8": the reference GPU decoder's row-int8 matvecs under their own names and argument order
// (crates/ojas-cuda/src/kernels/gemv_q8.rs:48-152) — a row is K plain int8 values with one f32 scale per output row
// (not GGUF's block_q8_0), activations are f32:
//     y[n] = scale[n] * sum_k (float) w[n][k] * x[k].
//
//   gemv_q8{,_accum}(x, w, y, scale, K, N)          any grid of workgroups of 1 .. 16 waves; rows grid-stride
//   gemv_q8_bias(x, w, y, scale, bias, K, N)
//   gemv_q8_ksplit(x, w, y, scale, K, N)            grid [N]: one row per workgroup, its waves splitting K
//   ffn_gu_q8(x, wg, wu, out, sg, su, K, N, act)    out[n] = act(gate[n]) * up[n]; act 0 SiLU, 1 GELU (tanh form, clamped)
//   qkv_q8(x, wq, wk, wv, yq, yk, yv, sq, sk, sv, bq, bk, bv, K, Nq, Nkv)      biases may be null
//   embed_q8(table, scale, out, token, D)           out[i] = (float) table[token][i] * scale[token]
// K is a multiple of 4, as in the reference.
//
// CDNA4 plan.  The launches are bound by the weight bytes (one per weight).  A wave owns two rows at a time and walks
// them in 16-byte pieces, lane l pieces l, l + 64, ...: 1 KB per row and load instruction, fully coalesced.  The
// activations are staged once per workgroup in LDS (up to 16384 floats; longer vectors are read from global memory)
// and the workgroup walks rows blockIdx.x, + gridDim.x, ..., so the staging is paid once per many rows.  Rows whose
// length is not a multiple of 16 are only 4-byte aligned: they are walked dword by dword.  Two vector instructions per
// weight (a sign-extending convert and a fused multiply-add) against 1 byte from HBM: at 6 TB/s a quarter of the issue
// slots.  Sums are per lane over its pieces in ascending k, then the wave tree of wave_sum: the reference's warp does
// the same with 32 lanes, so results agree to rounding (its own tests ask for 1e-4 .. 1e-3 relative,
// crates/ojas-cuda/tests/conformance.rs:271-336).
#include "ojk_common.h"

#define GQ8_XMAX 16384u          // floats of x a workgroup stages (64 KB)

__device__ __forceinline__ float gq8_sb(uint v, int b) { return (float)(signed char)(v >> (8 * b)); }
__device__ __forceinline__ float gq8_dot4(uint w, float4 x, float acc) {
    acc = fmaf(gq8_sb(w, 0), x.x, acc);
    acc = fmaf(gq8_sb(w, 1), x.y, acc);
    acc = fmaf(gq8_sb(w, 2), x.z, acc);
    return fmaf(gq8_sb(w, 3), x.w, acc);
}

// x into LDS by the whole workgroup (float4 per thread and step); returns where the dots read x from
__device__ __forceinline__ const float* gq8_stage_x(const float* __restrict__ x, uint K, float* lds) {
    if (K > GQ8_XMAX) return x;
    for (uint i = threadIdx.x; i < (K >> 2); i += blockDim.x) ((float4*)lds)[i] = ((const float4*)x)[i];
    __syncthreads();
    return lds;
}

// The lane's share of R rows' dots with x (xs: LDS or global): pieces of 16 weights when the rows are 16-byte aligned
// (K % 16 == 0), dwords otherwise and for the tail.
template <int R>
__device__ __forceinline__ void gq8_rows_dot(const signed char* const (&row)[R], const float* xs, uint K, uint lane,
                                             float (&acc)[R]) {
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = 0.0f;
    uint k4 = lane;                      // next dword of the lane in the dword walk
    if ((K & 15u) == 0u) {
        const uint K16 = K >> 4;
        for (uint p = lane; p < K16; p += 64u) {
            uint4 w[R];
#pragma unroll
            for (int r = 0; r < R; r++) w[r] = ((const uint4*)row[r])[p];
            const float4 x0 = ((const float4*)xs)[4u * p], x1 = ((const float4*)xs)[4u * p + 1u];
            const float4 x2 = ((const float4*)xs)[4u * p + 2u], x3 = ((const float4*)xs)[4u * p + 3u];
#pragma unroll
            for (int r = 0; r < R; r++) {
                acc[r] = gq8_dot4(w[r].x, x0, acc[r]);
                acc[r] = gq8_dot4(w[r].y, x1, acc[r]);
                acc[r] = gq8_dot4(w[r].z, x2, acc[r]);
                acc[r] = gq8_dot4(w[r].w, x3, acc[r]);
            }
        }
        return;
    }
    for (; k4 < (K >> 2); k4 += 64u) {
        const float4 xv = ((const float4*)xs)[k4];
#pragma unroll
        for (int r = 0; r < R; r++) acc[r] = gq8_dot4(((const uint*)row[r])[k4], xv, acc[r]);
    }
}

// MODE 0: y = s * dot; 1: y += s * dot; 2: y = s * dot + bias
template <int MODE>
__device__ __forceinline__ void gemv_q8_body(const float* __restrict__ x, const signed char* __restrict__ w,
                                             float* __restrict__ y, const float* __restrict__ scale,
                                             const float* __restrict__ bias, uint K, uint N, float* lds) {
    const float* xs = gq8_stage_x(x, K, lds);
    const uint lane = threadIdx.x & 63u, nw = blockDim.x >> 6, wave = threadIdx.x >> 6;
    for (uint n0 = (blockIdx.x * nw + wave) * 2u; n0 < N; n0 += gridDim.x * nw * 2u) {
        const uint n1 = min(n0 + 1u, N - 1u);
        const signed char* const rows[2] = {w + (size_t)n0 * K, w + (size_t)n1 * K};
        float acc[2];
        gq8_rows_dot<2>(rows, xs, K, lane, acc);
        const float t = wave_sum2(acc[0], acc[1], lane);       // lane 0: row n0, lane 1: row n0 + 1
        const uint n = n0 + lane;
        if (lane < 2u && n < N) {
            const float v = t * scale[n];
            y[n] = MODE == 1 ? y[n] + v : MODE == 2 ? v + bias[n] : v;
        }
    }
}

extern "C" __global__ void __launch_bounds__(1024)
gemv_q8(const float* x, const signed char* w, float* y, const float* scale, uint K, uint N) {
    __shared__ __attribute__((aligned(16))) float lds_x[GQ8_XMAX];
    gemv_q8_body<0>(x, w, y, scale, nullptr, K, N, lds_x);
}
extern "C" __global__ void __launch_bounds__(1024)
gemv_q8_accum(const float* x, const signed char* w, float* y, const float* scale, uint K, uint N) {
    __shared__ __attribute__((aligned(16))) float lds_x[GQ8_XMAX];
    gemv_q8_body<1>(x, w, y, scale, nullptr, K, N, lds_x);
}
extern "C" __global__ void __launch_bounds__(1024)
gemv_q8_bias(const float* x, const signed char* w, float* y, const float* scale, const float* bias, uint K, uint N) {
    __shared__ __attribute__((aligned(16))) float lds_x[GQ8_XMAX];
    gemv_q8_body<2>(x, w, y, scale, bias, K, N, lds_x);
}

// One row per workgroup, its waves taking the 16-byte pieces (or dwords) wave, wave + waves, ...; partial sums meet in
// LDS and are added in wave order.  For long K and few rows, where a wave per row pair leaves most of the chip idle.
extern "C" __global__ void __launch_bounds__(1024)
gemv_q8_ksplit(const float* x, const signed char* w, float* y, const float* scale, uint K, uint N) {
    __shared__ float part[16];
    const uint lane = threadIdx.x & 63u, nw = blockDim.x >> 6, wave = threadIdx.x >> 6, n = blockIdx.x;
    if (n >= N) return;
    const signed char* row = w + (size_t)n * K;
    float p = 0.0f;
    if ((K & 15u) == 0u) {
        for (uint q = wave * 64u + lane; q < (K >> 4); q += nw * 64u) {
            const uint4 wv = ((const uint4*)row)[q];
            p = gq8_dot4(wv.x, ((const float4*)x)[4u * q], p);
            p = gq8_dot4(wv.y, ((const float4*)x)[4u * q + 1u], p);
            p = gq8_dot4(wv.z, ((const float4*)x)[4u * q + 2u], p);
            p = gq8_dot4(wv.w, ((const float4*)x)[4u * q + 3u], p);
        }
    } else {
        for (uint q = wave * 64u + lane; q < (K >> 2); q += nw * 64u) p = gq8_dot4(((const uint*)row)[q], ((const float4*)x)[q], p);
    }
    p = wave_sum(p);
    if (lane == 0u) part[wave] = p;
    __syncthreads();
    if (threadIdx.x == 0u) {
        float s = 0.0f;
        for (uint i = 0; i < nw; i++) s += part[i];
        y[n] = s * scale[n];
    }
}

// The reference GPU path's activation (crates/ojas-cuda/src/kernels/gemv_q8.rs:21-29): GELU's tanh argument clamped to
// +-30, SiLU otherwise.
__device__ __forceinline__ float gq8_act(float g, uint act) {
    if (act == 1u) {
        float inner = 0.7978845608f * (g + 0.044715f * g * g * g);
        inner = fminf(fmaxf(inner, -30.0f), 30.0f);
        return 0.5f * g * (1.0f + tanhf(inner));
    }
    return g / (1.0f + expf(-g));
}

// gate and up rows of one output read side by side, one pass over x
extern "C" __global__ void __launch_bounds__(1024)
ffn_gu_q8(const float* x, const signed char* wg, const signed char* wu, float* out, const float* sg, const float* su,
          uint K, uint N, uint act) {
    __shared__ __attribute__((aligned(16))) float lds_x[GQ8_XMAX];
    const float* xs = gq8_stage_x(x, K, lds_x);
    const uint lane = threadIdx.x & 63u, nw = blockDim.x >> 6, wave = threadIdx.x >> 6;
    for (uint n = blockIdx.x * nw + wave; n < N; n += gridDim.x * nw) {
        const signed char* const rows[2] = {wg + (size_t)n * K, wu + (size_t)n * K};
        float acc[2];
        gq8_rows_dot<2>(rows, xs, K, lane, acc);
        const float t = wave_sum2(acc[0], acc[1], lane);       // lane 0: gate, lane 1: up
        const float up = dpp_f32<OJK_DPP_QUAD_XOR1>(t);
        if (lane == 0u) out[n] = gq8_act(t * sg[n], act) * (up * su[n]);
    }
}

// q, k and v rows as one launch: row n of Nq + 2 Nkv picks its tensor
extern "C" __global__ void __launch_bounds__(1024)
qkv_q8(const float* x, const signed char* wq, const signed char* wk, const signed char* wv, float* yq, float* yk, float* yv,
       const float* sq, const float* sk, const float* sv, const float* bq, const float* bk, const float* bv,
       uint K, uint Nq, uint Nkv) {
    __shared__ __attribute__((aligned(16))) float lds_x[GQ8_XMAX];
    const float* xs = gq8_stage_x(x, K, lds_x);
    const uint lane = threadIdx.x & 63u, nw = blockDim.x >> 6, wave = threadIdx.x >> 6;
    const uint total = Nq + 2u * Nkv;
    for (uint n0 = (blockIdx.x * nw + wave) * 2u; n0 < total; n0 += gridDim.x * nw * 2u) {
        const signed char* rows[2];
        const float* sc[2];
        const float* bs[2];
        float* yo[2];
#pragma unroll
        for (int r = 0; r < 2; r++) {
            const uint n = min(n0 + (uint)r, total - 1u);
            const uint t = n < Nq ? 0u : n < Nq + Nkv ? 1u : 2u, i = n - (t == 0u ? 0u : t == 1u ? Nq : Nq + Nkv);
            rows[r] = (t == 0u ? wq : t == 1u ? wk : wv) + (size_t)i * K;
            sc[r] = (t == 0u ? sq : t == 1u ? sk : sv) + i;
            const float* b = t == 0u ? bq : t == 1u ? bk : bv;
            bs[r] = b ? b + i : nullptr;
            yo[r] = (t == 0u ? yq : t == 1u ? yk : yv) + i;
        }
        const signed char* const rr[2] = {rows[0], rows[1]};
        float acc[2];
        gq8_rows_dot<2>(rr, xs, K, lane, acc);
        const float t = wave_sum2(acc[0], acc[1], lane);
        if (lane < 2u && n0 + lane < total) {
            const uint r = lane;
            const float* b = r ? bs[1] : bs[0];
            *(r ? yo[1] : yo[0]) = t * *(r ? sc[1] : sc[0]) + (b ? *b : 0.0f);
        }
    }
}

extern "C" __global__ void __launch_bounds__(256)
embed_q8(const signed char* table, const float* scale, float* out, uint token, uint D) {
    const signed char* row = table + (size_t)token * D;
    const float s = scale[token];
    for (uint i = blockIdx.x * blockDim.x + threadIdx.x; i < D; i += gridDim.x * blockDim.x) out[i] = (float)row[i] * s;
}

// Per-token activation quantizer of the reference's batched int8 GEMM (crates/ojas-cuda/src/kernels/gemv.rs:57-74):
//   quantize_q8_pertoken(x, q8, d8, K)     grid [M]: one workgroup per token
// d = max|x| / 127, q = clamp(rint(x * (1 / d)), -127, 127) (round half to even; 0 when the token is all zeros),
// d8[token] = d.  Every operation rounded on its own, as written: the codes are the reference's bit for bit.
extern "C" __global__ void __launch_bounds__(256)
quantize_q8_pertoken(const float* __restrict__ x, signed char* __restrict__ q8, float* __restrict__ d8, uint K) {
    __shared__ float sh[16];
    const uint tok = blockIdx.x, tid = threadIdx.x, nw = blockDim.x >> 6;
    const float* xr = x + (size_t)tok * K;
    signed char* qr = q8 + (size_t)tok * K;
    float a = 0.0f;
    for (uint i = tid; i < K; i += blockDim.x) a = fmaxf(a, fabsf(xr[i]));
    a = wave_max(a);
    if ((tid & 63u) == 0u) sh[tid >> 6] = a;
    __syncthreads();
    float amax = sh[0];
    for (uint i = 1; i < nw; i++) amax = fmaxf(amax, sh[i]);
    const float d = __fdiv_rn(amax, 127.0f);
    const float id = d > 0.0f ? __fdiv_rn(1.0f, d) : 0.0f;
    for (uint i = tid; i < K; i += blockDim.x) {
        const int qi = max(-127, min(127, __float2int_rn(__fmul_rn(xr[i], id))));
        qr[i] = (signed char)qi;
    }
    if (tid == 0u) d8[tok] = d;
}
