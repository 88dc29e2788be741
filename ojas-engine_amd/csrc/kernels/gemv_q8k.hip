// Family "gemv_q8k": the CPU reference's own arithmetic for K-quant rows on the GPU —
// activations quantized to int8 per 256-superblock ("Q8_K-flavoured"), integer dots against the
// raw 4/6-bit codes, f32 scale algebra per super-block.
//
// Reference: crates/ojas-cpu/src/cpu_math.rs:539-563 (quant_q8k), :609-635 (dot_q4k),
// :674-722 (dot_q6k), :1145-1189 (matvec_kq).
//
//   quantize_q8k{,_bf16}(x, q, scales, K, M)             grid (ceil(K/256), M), block 256
//   gemv_q8k_<fmt>(xq, xs, w, y, K, N)                        4 rows per wave
//   gemv_q8k_<fmt>{_accum,_bias}(xq, xs, w, y[, bs], K, N)    1 row per wave (residual-sized N)
//   gemv_q8k_<fmt>_r1 / _r2 (same arguments)                  1 / 2 rows per wave
//   gemv_q8k_<fmt>_wide (same arguments)                      2 rows per wave; the entry the op
//                                                             seam uses for output-head sized N
//   gemv_q8k_<fmt>_m(xq, xs, w, y, K, N, M, ACC)          y[M][N], one weight pass per MT tokens
//
// Integer sums are exact, so  sum_j sc_j*idot_j  and  sum_j m_j*bsum_j  are formed in int32 and
// converted once; they equal the reference's sequential f32 sums whenever those are exact
// (always for the min term; for the scale term unless |sum| >= 2^24, where the reference itself
// rounds).  The per-row f32 accumulation over super-blocks runs in a different order than the
// reference's (lanes own different super-blocks), which moves the last ulp only.
#include "ojk_common.h"
#include "ojk_q4k_dot.h"
#include "ojk_act.h"
#include "ojk_q6k_mfma.h"

// ------------------------------------------------------------------ activation quantizer
// A workgroup per 256-value segment, as the grid has always been; its first wave does the work, four consecutive
// values a lane (one 16- or 8-byte load, the maximum across the wave, one 4-byte store of codes), and the other waves
// leave at once.  (A value per thread — four partial maxima through LDS, a barrier, 1-byte stores — ran at 2.3-2.6 TB/s
// on prefill-sized batches.)
// FLAT (`quantize_q8k{,_bf16}_w`, grid [ceil(segments / 4)]): a segment per wave, four per workgroup, segments numbered
// token-major — for batches of many short rows, where a workgroup per segment is mostly launch overhead.
template <bool BF16, bool FLAT = false>
__device__ __forceinline__ void quantize_q8k_body(const void* __restrict__ xv, signed char* __restrict__ q,
                                                  float* __restrict__ scales, uint K, uint M) {
    const uint nsb = (K + 255u) >> 8, lane = threadIdx.x & 63u;
    uint sb, m;
    if (FLAT) {
        const uint seg = blockIdx.x * 4u + (threadIdx.x >> 6);
        if (seg >= nsb * M) return;
        m = seg / nsb;
        sb = seg - m * nsb;
    } else {
        if (threadIdx.x >= 64u) return;
        sb = blockIdx.x;
        m = blockIdx.y;
    }
    const uint i = sb * 256u + 4u * lane;
    float v[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (BF16) {
        const ushort* p = (const ushort*)xv + (size_t)m * K + i;
        if (i + 3u < K && ((size_t)p & 7u) == 0) {
            const uint2 t = *(const uint2*)p;
            v[0] = bf16_bits_to_f32(t.x & 0xFFFFu); v[1] = bf16_bits_to_f32(t.x >> 16);
            v[2] = bf16_bits_to_f32(t.y & 0xFFFFu); v[3] = bf16_bits_to_f32(t.y >> 16);
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++) if (i + (uint)j < K) v[j] = bf16_bits_to_f32(p[j]);
        }
    } else {
        const float* p = (const float*)xv + (size_t)m * K + i;
        if (i + 3u < K && ((size_t)p & 15u) == 0) {
            const float4 t = *(const float4*)p;
            v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++) if (i + (uint)j < K) v[j] = p[j];
        }
    }
    const float mx = wave_max(fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3]))));
    // scale = amax/127 (1 when the segment is all zero); q = clamp(round_half_away(v * (1/scale)))
    const float scale = mx > 0.0f ? __fdiv_rn(mx, 127.0f) : 1.0f;
    const float inv = __fdiv_rn(1.0f, scale);
    uint packed = 0u;
#pragma unroll
    for (int j = 0; j < 4; j++) packed |= ((uint)(int)sat127(roundf(__fmul_rn(v[j], inv))) & 0xFFu) << (8 * j);
    // the padded tail of a ragged last segment is written as zero
    *(uint*)(q + ((size_t)m * nsb + sb) * 256u + 4u * lane) = packed;
    if (lane == 0) scales[(size_t)m * nsb + sb] = scale;
}

extern "C" __global__ void __launch_bounds__(256)
quantize_q8k(const float* x, signed char* q, float* scales, uint K, uint M) {
    quantize_q8k_body<false>(x, q, scales, K, M);
}
extern "C" __global__ void __launch_bounds__(256)
quantize_q8k_bf16(const ushort* x, signed char* q, float* scales, uint K, uint M) {
    quantize_q8k_body<true>(x, q, scales, K, M);
}
extern "C" __global__ void __launch_bounds__(256)
quantize_q8k_w(const float* x, signed char* q, float* scales, uint K, uint M) {
    quantize_q8k_body<false, true>(x, q, scales, K, M);
}
extern "C" __global__ void __launch_bounds__(256)
quantize_q8k_bf16_w(const ushort* x, signed char* q, float* scales, uint K, uint M) {
    quantize_q8k_body<true, true>(x, q, scales, K, M);
}

// ------------------------------------------------------------------ store modes
enum { ST_SET = 0, ST_ACCUM = 1, ST_BIAS = 2 };

template <int MODE>
__device__ __forceinline__ void store_row(float* y, const float* bs, uint n, float v) {
    if (MODE == ST_SET) y[n] = v;
    else if (MODE == ST_ACCUM) y[n] += v;
    else y[n] = v + bs[n];
}
// The value an accumulate / bias store adds, fetched when the wave starts instead of after its
// last reduction (a dependent load at the tail of every wave otherwise).
template <int MODE>
__device__ __forceinline__ float store_addend(const float* y, const float* bs, uint n) {
    return MODE == ST_ACCUM ? y[n] : MODE == ST_BIAS ? bs[n] : 0.0f;
}
template <int MODE>
__device__ __forceinline__ void store_row_with(float* y, uint n, float v, float addend) {
    y[n] = MODE == ST_SET ? v : MODE == ST_ACCUM ? addend + v : v + addend;
}

// ------------------------------------------------------------------ Q4_K (lane dot: ojk_q4k_dot.h)
template <int R, int MODE>
__device__ __forceinline__ void gemv_q8k_q4k_body(const signed char* __restrict__ xq, const float* __restrict__ xs,
                                                  const uchar* __restrict__ w, float* __restrict__ y,
                                                  const float* __restrict__ bs, uint K, uint N) {
    const uint lane = threadIdx.x & 63u;
    // (the wave's rows are the same in every lane: said so, the row addresses are scalar arithmetic and the loads take
    // a scalar base plus a 32-bit lane offset instead of 64-bit multiplies per lane)
    const uint row0 = (uint)__builtin_amdgcn_readfirstlane((int)((blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)) * R));
    if (row0 >= N) return;
    const uint nsb = K >> 8, g = lane >> 3, l = lane & 7u, c = l >> 1;
    float acc[R], add[R];
    const uchar* wrow[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        acc[r] = 0.0f;
        add[r] = store_addend<MODE>(y, bs, min(row0 + r, N - 1u));
        wrow[r] = w + (size_t)min(row0 + r, N - 1u) * nsb * Q4K_BYTES;
    }
    for (uint sb = g; sb < nsb; sb += 8u) {
        uint4 hdr[R], qs[R];
        const uint off = __umul24(sb, Q4K_BYTES);
#pragma unroll
        for (int r = 0; r < R; r++) {
            hdr[r] = *(const uint4*)(wrow[r] + off);
            qs[r] = *(const uint4*)(wrow[r] + (off + 16u + l * 16u));
        }
        Q4kFrag f = q4k_load_frag(xq, xs, sb, l);
#pragma unroll
        for (int r = 0; r < R; r++) acc[r] += q4k_lane_dot(hdr[r], qs[r], c, f);
    }
    if (R == 2 && MODE == ST_SET) {         // the wave's two sums in one pass (wave_sum's additions, in its order)
        const float t = wave_sum2(acc[0], acc[R - 1], lane);
        if (lane < 2u && row0 + lane < N) y[row0 + lane] = t;
        return;
    }
    if (R == 4 && MODE == ST_SET) {
        const float t = wave_sum4(acc[0], acc[1 % R], acc[2 % R], acc[3 % R], lane);
        if (lane < 4u && row0 + lane < N) y[row0 + lane] = t;
        return;
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
        float t = wave_sum(acc[r]);
        if (lane == 0 && row0 + r < N) store_row_with<MODE>(y, row0 + r, t, add[r]);
    }
}

#define GEMV_Q8K_ENTRIES(FMT, BODY)                                                                          \
    extern "C" __global__ void __launch_bounds__(256) gemv_q8k_##FMT##_r1(                                   \
        const signed char* xq, const float* xs, const uchar* w, float* y, uint K, uint N) {                  \
        BODY<1, ST_SET>(xq, xs, w, y, nullptr, K, N); }                                                      \
    extern "C" __global__ void __launch_bounds__(256) gemv_q8k_##FMT##_r2(                                   \
        const signed char* xq, const float* xs, const uchar* w, float* y, uint K, uint N) {                  \
        BODY<2, ST_SET>(xq, xs, w, y, nullptr, K, N); }                                                      \
    extern "C" __global__ void __launch_bounds__(256) gemv_q8k_##FMT##_wide(                                 \
        const signed char* xq, const float* xs, const uchar* w, float* y, uint K, uint N) {                  \
        BODY<2, ST_SET>(xq, xs, w, y, nullptr, K, N); }                                                      \
    extern "C" __global__ void __launch_bounds__(256) gemv_q8k_##FMT(                                        \
        const signed char* xq, const float* xs, const uchar* w, float* y, uint K, uint N) {                  \
        BODY<4, ST_SET>(xq, xs, w, y, nullptr, K, N); }                                                      \
    extern "C" __global__ void __launch_bounds__(256) gemv_q8k_##FMT##_accum(                                \
        const signed char* xq, const float* xs, const uchar* w, float* y, uint K, uint N) {                  \
        BODY<1, ST_ACCUM>(xq, xs, w, y, nullptr, K, N); }                                                    \
    extern "C" __global__ void __launch_bounds__(256) gemv_q8k_##FMT##_bias(                                 \
        const signed char* xq, const float* xs, const uchar* w, float* y, const float* bs, uint K, uint N) { \
        BODY<1, ST_BIAS>(xq, xs, w, y, bs, K, N); }

GEMV_Q8K_ENTRIES(q4k, gemv_q8k_q4k_body)

// ------------------------------------------------------------------ Q5_K
// The Q4_K lane map on 176-byte super-blocks: {f16 d, f16 dmin, scales[12], qh[32], qs[128]}.
// The fifth bit of weight l of sub-block j is bit j of qh[l] (crates/ojas-cpu/src/cpu_math.rs:638-670),
// so a lane adds 16 * dot(bit plane, x) to each of its two nibble dots: the 16 qh bytes it needs
// are those at the positions of its 16 quant bytes within the 32-byte chunk.
template <int R, int MODE>
__device__ __forceinline__ void gemv_q8k_q5k_body(const signed char* __restrict__ xq, const float* __restrict__ xs,
                                                  const uchar* __restrict__ w, float* __restrict__ y,
                                                  const float* __restrict__ bs, uint K, uint N) {
    const uint lane = threadIdx.x & 63u;
    const uint row0 = (blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)) * R;
    if (row0 >= N) return;
    const uint nsb = K >> 8, g = lane >> 3, l = lane & 7u, c = l >> 1;
    float acc[R], add[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        acc[r] = 0.0f;
        add[r] = store_addend<MODE>(y, bs, min(row0 + r, N - 1u));
    }
    for (uint sb = g; sb < nsb; sb += 8u) {
        uint4 hdr[R], qs[R], qh[R];
#pragma unroll
        for (int r = 0; r < R; r++) {
            const uchar* blk = w + ((size_t)min(row0 + r, N - 1u) * nsb + sb) * Q5K_BYTES;
            hdr[r] = *(const uint4*)blk;
            qh[r] = *(const uint4*)(blk + 16u + (l & 1u) * 16u);
            qs[r] = *(const uint4*)(blk + 48u + l * 16u);
        }
        Q4kFrag f = q4k_load_frag(xq, xs, sb, l);
#pragma unroll
        for (int r = 0; r < R; r++) acc[r] += q5k_lane_dot(hdr[r], qs[r], qh[r], c, f);
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
        float t = wave_sum(acc[r]);
        if (lane == 0 && row0 + r < N) store_row_with<MODE>(y, row0 + r, t, add[r]);
    }
}

GEMV_Q8K_ENTRIES(q5k, gemv_q8k_q5k_body)

template <int MT>
__device__ __forceinline__ void gemv_q8k_q5k_m_body(const signed char* __restrict__ xq, const float* __restrict__ xs,
                                                    const uchar* __restrict__ w, float* __restrict__ y,
                                                    uint K, uint N, uint M, uint ACC) {
    const uint lane = threadIdx.x & 63u;
    const uint row = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (row >= N) return;
    const uint nsb = K >> 8, g = lane >> 3, l = lane & 7u, c = l >> 1;
    for (uint m0 = 0; m0 < M; m0 += MT) {
        float acc[MT];
#pragma unroll
        for (int t = 0; t < MT; t++) acc[t] = 0.0f;
        for (uint sb = g; sb < nsb; sb += 8u) {
            const uchar* blk = w + ((size_t)row * nsb + sb) * Q5K_BYTES;
            const uint4 hdr = *(const uint4*)blk, qh = *(const uint4*)(blk + 16u + (l & 1u) * 16u);
            const uint4 qs = *(const uint4*)(blk + 48u + l * 16u);
#pragma unroll
            for (int t = 0; t < MT; t++) {
                uint m = min(m0 + t, M - 1u);
                Q4kFrag f = q4k_load_frag(xq + (size_t)m * nsb * 256u, xs + (size_t)m * nsb, sb, l);
                acc[t] += q5k_lane_dot(hdr, qs, qh, c, f);
            }
        }
#pragma unroll
        for (int t = 0; t < MT; t++) {
            float s = wave_sum(acc[t]);
            if (lane == 0 && m0 + t < M) {
                float* o = y + (size_t)(m0 + t) * N + row;
                *o = ACC ? *o + s : s;
            }
        }
    }
}

extern "C" __global__ void __launch_bounds__(256)
gemv_q8k_q5k_m(const signed char* xq, const float* xs, const uchar* w, float* y, uint K, uint N, uint M, uint ACC) {
    if (M <= 2) gemv_q8k_q5k_m_body<2>(xq, xs, w, y, K, N, M, ACC);
    else if (M <= 4) gemv_q8k_q5k_m_body<4>(xq, xs, w, y, K, N, M, ACC);
    else gemv_q8k_q5k_m_body<8>(xq, xs, w, y, K, N, M, ACC);
}

// ---- several projections of one activation in one launch -------------------------------------
//   gemv_q8k_q4k_x4_{r1,r2}(xq, xs, w0, w1, w2, w3, y0, y1, y2, y3, K, E0, E1, E2, E3)
// Up to four weight tensors (separate allocations, all K wide) share the quantized activation:
// global row r belongs to tensor i when E(i-1) <= r < E(i), E being the running row totals.
// The counterpart of the reference's fused q/k/v and gate/up launches
// (crates/ojas-core/src/kernels/gemv_q8.rs:229-260), which likewise take one pointer per
// projection.  Each row runs exactly the single-tensor arithmetic, so results are bit-identical
// to separate launches; what is saved is a dispatch and a DRAM round trip per projection.
struct X4Row {
    const uchar* w;
    float* y;
};

template <int R>
__device__ __forceinline__ void gemv_q8k_q4k_x4_body(const signed char* __restrict__ xq, const float* __restrict__ xs,
                                                     const uchar* w0, const uchar* w1, const uchar* w2,
                                                     const uchar* w3, float* y0, float* y1, float* y2, float* y3,
                                                     uint K, uint E0, uint E1, uint E2, uint E3) {
    const uint lane = threadIdx.x & 63u;
    const uint row0 = (blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)) * R;
    if (row0 >= E3) return;
    const uint nsb = K >> 8, g = lane >> 3, l = lane & 7u, c = l >> 1;
    X4Row rw[R];
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        const uint gr = min(row0 + r, E3 - 1u);
        const uchar* w;
        float* y;
        uint lr;
        if (gr < E0) { w = w0; y = y0; lr = gr; }
        else if (gr < E1) { w = w1; y = y1; lr = gr - E0; }
        else if (gr < E2) { w = w2; y = y2; lr = gr - E1; }
        else { w = w3; y = y3; lr = gr - E2; }
        rw[r].w = w + (size_t)lr * nsb * Q4K_BYTES;
        rw[r].y = y + lr;
        acc[r] = 0.0f;
    }
    for (uint sb = g; sb < nsb; sb += 8u) {
        uint4 hdr[R], qs[R];
#pragma unroll
        for (int r = 0; r < R; r++) {
            const uchar* blk = rw[r].w + (size_t)sb * Q4K_BYTES;
            hdr[r] = *(const uint4*)blk;
            qs[r] = *(const uint4*)(blk + 16u + l * 16u);
        }
        Q4kFrag f = q4k_load_frag(xq, xs, sb, l);
#pragma unroll
        for (int r = 0; r < R; r++) acc[r] += q4k_lane_dot(hdr[r], qs[r], c, f);
    }
    if (R == 2) {       // both sums in one pass
        const float t = wave_sum2(acc[0], acc[R - 1], lane);
        if (lane < 2u && row0 + lane < E3) *(lane ? rw[R - 1].y : rw[0].y) = t;
        return;
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
        float t = wave_sum(acc[r]);
        if (lane == 0 && row0 + r < E3) *rw[r].y = t;
    }
}

extern "C" __global__ void __launch_bounds__(256)
gemv_q8k_q4k_x4_r1(const signed char* xq, const float* xs, const uchar* w0, const uchar* w1, const uchar* w2,
                   const uchar* w3, float* y0, float* y1, float* y2, float* y3, uint K, uint E0, uint E1, uint E2,
                   uint E3) {
    gemv_q8k_q4k_x4_body<1>(xq, xs, w0, w1, w2, w3, y0, y1, y2, y3, K, E0, E1, E2, E3);
}
extern "C" __global__ void __launch_bounds__(256)
gemv_q8k_q4k_x4_r2(const signed char* xq, const float* xs, const uchar* w0, const uchar* w1, const uchar* w2,
                   const uchar* w3, float* y0, float* y1, float* y2, float* y3, uint K, uint E0, uint E1, uint E2,
                   uint E3) {
    gemv_q8k_q4k_x4_body<2>(xq, xs, w0, w1, w2, w3, y0, y1, y2, y3, K, E0, E1, E2, E3);
}

// ---- gate and up projections with the activation function in one launch -----------------------
//   ffn_gu_q8k_q4k(xq, xs, wg, wu, out, K, N, ACT)     out[n] = act(Wg[n] . x) * (Wu[n] . x)
// ACT 0 = SiLU  g / (1 + exp(-g))  (crates/ojas-cpu/src/cpu_math.rs:486), 1 = GELU, tanh form
// (:497-501).  The reference's decode path fuses the same three steps
// (`ffn_gu_q80_dp4a`, crates/ojas-cuda/src/kernels/gemv_q8.rs:246-260); each dot is the
// single-tensor arithmetic of gemv_q8k_q4k.

extern "C" __global__ void __launch_bounds__(256)
ffn_gu_q8k_q4k(const signed char* __restrict__ xq, const float* __restrict__ xs, const uchar* __restrict__ wg,
               const uchar* __restrict__ wu, float* __restrict__ out, uint K, uint N, uint ACT) {
    constexpr int R = 1;   // one row per wave (two weight streams): K is short, so more, lighter waves win
    const uint lane = threadIdx.x & 63u;
    const uint row0 = (blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)) * R;
    if (row0 >= N) return;
    const uint nsb = K >> 8, g = lane >> 3, l = lane & 7u, c = l >> 1;
    float ag[R], au[R];
#pragma unroll
    for (int r = 0; r < R; r++) ag[r] = au[r] = 0.0f;
    for (uint sb = g; sb < nsb; sb += 8u) {
        uint4 hg[R], qg[R], hu[R], qu[R];
#pragma unroll
        for (int r = 0; r < R; r++) {
            const size_t o = ((size_t)min(row0 + r, N - 1u) * nsb + sb) * Q4K_BYTES;
            hg[r] = *(const uint4*)(wg + o); qg[r] = *(const uint4*)(wg + o + 16u + l * 16u);
            hu[r] = *(const uint4*)(wu + o); qu[r] = *(const uint4*)(wu + o + 16u + l * 16u);
        }
        Q4kFrag f = q4k_load_frag(xq, xs, sb, l);
#pragma unroll
        for (int r = 0; r < R; r++) {
            ag[r] += q4k_lane_dot(hg[r], qg[r], c, f);
            au[r] += q4k_lane_dot(hu[r], qu[r], c, f);
        }
    }
    {   // the gate and the up sum in one pass: lane 0 ends with the gate sum, lane 1 with the up sum
        const float t = wave_sum2(ag[0], au[0], lane);
        const float su = dpp_f32<OJK_DPP_QUAD_XOR1>(t);
        if (lane == 0 && row0 < N) out[row0] = ffn_act(t, ACT) * su;
    }
}

// ---- RMS norm and activation quantizer in one launch --------------------------------------------
//   rmsnorm_q8k(x, gamma, q, scales, xn, K, M, EPS_BITS, WRITE_XN)    grid M, block 256 or 1024, K <= 16384
// xn = x * (1 / sqrt(mean(x^2) + eps)) * gamma  (crates/ojas-cpu/src/cpu_math.rs:456-460), then
// quant_q8k(xn) (:539-563) without a trip through memory: a decode layer's projections read the
// normalized vector only through its quantized form.  The mean of squares is summed in f64 and
// rounded once; the reference sums in f32 in index order, so `inv` may differ in its last bit.
// The order of the f64 sum does not depend on the block size: a lane adds the squares of its four values of a
// 256-value segment (in index order), the segment's 64 lane sums meet as wave_sum_f64 adds them, and so do the segment
// sums (segment i in lane i).  A wave owns segments w, w + waves, ...: with sixteen waves, one each up to K = 4096.
extern "C" __global__ void __launch_bounds__(1024)
rmsnorm_q8k(const float* __restrict__ x, const float* __restrict__ gamma, signed char* __restrict__ q,
            float* __restrict__ scales, float* __restrict__ xn, uint K, uint M, uint EPS_BITS, uint WRITE_XN) {
    __shared__ double part[64];
    const uint m = blockIdx.x, tid = threadIdx.x, lane = tid & 63u;
    const uint wave = (uint)__builtin_amdgcn_readfirstlane((int)(tid >> 6)), nw = blockDim.x >> 6;
    const uint nsb = (K + 255u) >> 8;
    const float* row = x + (size_t)m * K;
    const bool vec = (K & 3u) == 0 && (((size_t)row | (size_t)gamma) & 15u) == 0;   // 128-bit loads
    auto load4 = [&](const float* p, uint i0, float (&o)[4]) {
        if (vec && i0 + 3u < K) {
            const float4 t = *(const float4*)(p + i0);
            o[0] = t.x; o[1] = t.y; o[2] = t.z; o[3] = t.w;
        } else {
#pragma unroll
            for (int e = 0; e < 4; e++) o[e] = i0 + e < K ? p[i0 + e] : 0.0f;
        }
    };
    // the wave's first four segments stay in registers between the two passes (all of them up to 4 x waves x 256 values)
    float kv[4][4], kg[4][4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const uint seg = wave + nw * (uint)j;
        if (seg < nsb) {
            load4(row, seg * 256u + lane * 4u, kv[j]);      // past the row: zeros
            load4(gamma, seg * 256u + lane * 4u, kg[j]);
        }
    }
    for (uint seg = wave, j = 0; seg < nsb; seg += nw, j++) {
        float v[4];
        if (j < 4u) {
#pragma unroll
            for (int e = 0; e < 4; e++) v[e] = j == 0 ? kv[0][e] : j == 1 ? kv[1][e] : j == 2 ? kv[2][e] : kv[3][e];
        } else {
            load4(row, seg * 256u + lane * 4u, v);
        }
        double ss = (double)v[0] * (double)v[0];
        ss += (double)v[1] * (double)v[1];
        ss += (double)v[2] * (double)v[2];
        ss += (double)v[3] * (double)v[3];
        ss = wave_sum_f64(ss);      // the segment's 64 lane sums
        if (lane == 0) part[seg] = ss;
    }
    __syncthreads();
    const double total = tree_sum_f64(part, nsb, lane);
    const float mean = (float)(total / (double)K);
    const float inv = __fdiv_rn(1.0f, __fsqrt_rn(__fadd_rn(mean, __uint_as_float(EPS_BITS))));
    for (uint seg = wave, j = 0; seg < nsb; seg += nw, j++) {
        const uint i0 = seg * 256u + lane * 4u;
        float v[4], gm[4], t[4];
        if (j < 4u) {
#pragma unroll
            for (int e = 0; e < 4; e++) {
                v[e] = j == 0 ? kv[0][e] : j == 1 ? kv[1][e] : j == 2 ? kv[2][e] : kv[3][e];
                gm[e] = j == 0 ? kg[0][e] : j == 1 ? kg[1][e] : j == 2 ? kg[2][e] : kg[3][e];
            }
        } else {
            load4(row, i0, v);      // second read: from the cache
            load4(gamma, i0, gm);
        }
#pragma unroll
        for (int e = 0; e < 4; e++) t[e] = i0 + e < K ? __fmul_rn(__fmul_rn(v[e], inv), gm[e]) : 0.0f;
        const float a = wave_max(fmaxf(fmaxf(fabsf(t[0]), fabsf(t[1])), fmaxf(fabsf(t[2]), fabsf(t[3]))));
        const float scale = a > 0.0f ? __fdiv_rn(a, 127.0f) : 1.0f;
        const float is = __fdiv_rn(1.0f, scale);
        uint packed = 0;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int qi = (int)sat127(roundf(__fmul_rn(t[e], is)));
            packed |= (uint)(qi & 0xFF) << (8 * e);
            if (WRITE_XN && i0 + e < K) xn[(size_t)m * K + i0 + e] = t[e];
        }
        *(uint*)(q + ((size_t)m * nsb + seg) * 256u + lane * 4u) = packed;
        if (lane == 0) scales[(size_t)m * nsb + seg] = scale;
    }
}

// ---- the same matvec with the activation quantizer folded in ---------------------------------
//   gemv_fq8k_q4k_{r1,r2,wide}(x, w, y, K, N, NRB)      x: f32[K], K <= 16384
// A decode step is a chain of few-microsecond launches, each costing a dispatch and a DRAM round
// trip; quantizing in a launch of its own doubles that chain.  Here every workgroup quantizes x
// itself into LDS — the same arithmetic as quantize_q8k, so results are bit-identical to the
// two-launch form — after its first weight loads are already in flight, so the quantization
// hides under their latency; it then walks NRB rows (a multiple of 4R, chosen by the host so
// that the repeated quantization stays a small share of the work).  LDS segments are 288 bytes
// apart: the 16-byte fragment reads of 16 consecutive lanes then fall in distinct banks.
#define FQ_SEG 288u
#define FQ_MAX_K 16384u

template <int R>
__device__ __forceinline__ void gemv_fq8k_q4k_body(const float* __restrict__ x, const uchar* __restrict__ w,
                                                   float* __restrict__ y, uint K, uint N, uint NRB) {
    __shared__ __attribute__((aligned(16))) signed char sx[(FQ_MAX_K / 256u) * FQ_SEG];
    __shared__ float ss[FQ_MAX_K / 256u];
    const uint tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint nsb = K >> 8, g = lane >> 3, l = lane & 7u, c = l >> 1;
    const uint row_end = min((blockIdx.x + 1u) * NRB, N);
    uint row0 = blockIdx.x * NRB + wave * R;
    // first step's weights: issued before anything else
    uint4 hdr[R], qs[R];
    {
        const uint sb = min(g, nsb - 1u);
#pragma unroll
        for (int r = 0; r < R; r++) {
            uint row = min(row0 + r, N - 1u);
            const uchar* blk = w + ((size_t)row * nsb + sb) * Q4K_BYTES;
            hdr[r] = *(const uint4*)blk;
            qs[r] = *(const uint4*)(blk + 16u + l * 16u);
        }
    }
    // quantize x: wave `wave` owns segments wave, wave+4, ...; a lane holds 4 consecutive values
    for (uint seg = wave; seg < nsb; seg += 4u) {
        float4 v = *(const float4*)(x + (size_t)seg * 256u + lane * 4u);
        float a = wave_max(fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
        float scale = a > 0.0f ? __fdiv_rn(a, 127.0f) : 1.0f;
        float inv = __fdiv_rn(1.0f, scale);
        int q0 = (int)sat127(roundf(__fmul_rn(v.x, inv)));
        int q1 = (int)sat127(roundf(__fmul_rn(v.y, inv)));
        int q2 = (int)sat127(roundf(__fmul_rn(v.z, inv)));
        int q3 = (int)sat127(roundf(__fmul_rn(v.w, inv)));
        *(uint*)(sx + seg * FQ_SEG + lane * 4u) =
            (uint)(q0 & 0xFF) | ((uint)(q1 & 0xFF) << 8) | ((uint)(q2 & 0xFF) << 16) | ((uint)(q3 & 0xFF) << 24);
        if (lane == 0) ss[seg] = scale;
    }
    __syncthreads();
    bool first = true;
    for (; row0 < row_end; row0 += 4u * R) {
        float acc[R];
#pragma unroll
        for (int r = 0; r < R; r++) acc[r] = 0.0f;
        for (uint sb = g; sb < nsb; sb += 8u) {
            if (!(first && sb == g)) {
#pragma unroll
                for (int r = 0; r < R; r++) {
                    uint row = min(row0 + r, N - 1u);
                    const uchar* blk = w + ((size_t)row * nsb + sb) * Q4K_BYTES;
                    hdr[r] = *(const uint4*)blk;
                    qs[r] = *(const uint4*)(blk + 16u + l * 16u);
                }
            }
            Q4kFrag f;
            const signed char* p = sx + sb * FQ_SEG + c * 64u + (l & 1u) * 16u;
            f.xl = *(const uint4*)p;
            f.xh = *(const uint4*)(p + 32);
            f.bl = bytesum4(f.xl);
            f.bh = bytesum4(f.xh);
            f.sx = ss[sb];
#pragma unroll
            for (int r = 0; r < R; r++) acc[r] += q4k_lane_dot(hdr[r], qs[r], c, f);
        }
        first = false;
#pragma unroll
        for (int r = 0; r < R; r++) {
            float t = wave_sum(acc[r]);
            if (lane == 0 && row0 + r < row_end) y[row0 + r] = t;
        }
    }
}

extern "C" __global__ void __launch_bounds__(256)
gemv_fq8k_q4k_r1(const float* x, const uchar* w, float* y, uint K, uint N, uint NRB) {
    gemv_fq8k_q4k_body<1>(x, w, y, K, N, NRB);
}
extern "C" __global__ void __launch_bounds__(256)
gemv_fq8k_q4k_r2(const float* x, const uchar* w, float* y, uint K, uint N, uint NRB) {
    gemv_fq8k_q4k_body<2>(x, w, y, K, N, NRB);
}
extern "C" __global__ void __launch_bounds__(256)
gemv_fq8k_q4k_wide(const float* x, const uchar* w, float* y, uint K, uint N, uint NRB) {
    gemv_fq8k_q4k_body<2>(x, w, y, K, N, NRB);
}

// ---- the folded quantizer over up to four tensors ----------------------------------------------
//   gemv_fq8k_q4k_x4_{r1,r2}(x, w0, w1, w2, w3, y0, y1, y2, y3, K, E0, E1, E2, E3, NRB, ACC)     x: f32[K], K <= 16384
// One launch per stage of a decode layer: the stage's f32 activations are quantized by every workgroup into LDS (the
// arithmetic of quantize_q8k: results are bit-identical to quantizer + matvec launches) and multiplied with up to four
// weight tensors that share them (q/k/v, gate/up; a single tensor passes E0 = E1 = E2 = E3).  ACC adds onto y (the
// residual).  Vector memory operations return in order, so the activations are requested FIRST and the workgroup's
// first weights second: the quantization then runs while those weights are still on their way instead of queueing
// behind them.  A workgroup (256, 512 or 1024 threads) walks NRB rows, its waves R at a time.  The quantization is
// about 110 vector instructions per segment and wave — as much as the dot products of twenty rows for K = 4096 — and
// every workgroup repeats it, so the launch wants few, large workgroups: one or two per CU.
template <int R>
__device__ __forceinline__ void gemv_fq8k_q4k_x4_body(const float* __restrict__ x, const uchar* w0, const uchar* w1,
                                                      const uchar* w2, const uchar* w3, float* y0, float* y1, float* y2,
                                                      float* y3, uint K, uint E0, uint E1, uint E2, uint E3, uint NRB,
                                                      uint ACC) {
    __shared__ __attribute__((aligned(16))) signed char sx[(FQ_MAX_K / 256u) * FQ_SEG];
    __shared__ float ss[FQ_MAX_K / 256u];
    const uint tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, nw = blockDim.x >> 6;
    const uint nsb = K >> 8, g = lane >> 3, l = lane & 7u, c = l >> 1;
    const uint row_end = min((blockIdx.x + 1u) * NRB, E3);
    uint row0 = blockIdx.x * NRB + wave * R;
    // row r0 + r of the stacked tensors -> its block bytes and its output
    auto locate = [&](uint r0, X4Row (&rw)[R]) {
#pragma unroll
        for (int r = 0; r < R; r++) {
            const uint gr = min(r0 + r, E3 - 1u);
            const uchar* w;
            float* y;
            uint lr;
            if (gr < E0) { w = w0; y = y0; lr = gr; }
            else if (gr < E1) { w = w1; y = y1; lr = gr - E0; }
            else if (gr < E2) { w = w2; y = y2; lr = gr - E1; }
            else { w = w3; y = y3; lr = gr - E2; }
            rw[r].w = w + (size_t)lr * nsb * Q4K_BYTES;
            rw[r].y = y + lr;
        }
    };
    auto fetch = [&](const X4Row (&rw)[R], uint sb, uint4 (&hdr)[R], uint4 (&qs)[R]) {
        const uint sbc = min(sb, nsb - 1u);
#pragma unroll
        for (int r = 0; r < R; r++) {
            const uchar* blk = rw[r].w + (size_t)sbc * Q4K_BYTES;
            hdr[r] = *(const uint4*)blk;
            qs[r] = *(const uint4*)(blk + 16u + l * 16u);
        }
    };
    // 1. the activations, four segments per wave at a time (wave `wave` owns segments wave, wave + nw, ...; a lane
    //    holds 4 consecutive values), the first batch requested before anything else
    constexpr int NB = 4;
    float4 v[NB];
#pragma unroll
    for (int i = 0; i < NB; i++) {
        const uint seg = wave + nw * (uint)i;
        v[i] = *(const float4*)(x + (size_t)min(seg, nsb - 1u) * 256u + lane * 4u);
    }
    __builtin_amdgcn_sched_barrier(0);
    // 2. the first step's weights
    X4Row rwc[R], rwn[R];
    uint4 hc[R], qc[R], hn[R], qn[R];
    locate(row0, rwc);
    fetch(rwc, g, hc, qc);
    __builtin_amdgcn_sched_barrier(0);
    // 3. quantize into LDS
    for (uint s0 = 0; s0 < nsb; s0 += nw * NB) {
#pragma unroll
        for (int i = 0; i < NB; i++) {
            const uint seg = s0 + wave + nw * (uint)i;
            const float4 t = v[i];
            // the next batch's request goes out as soon as the register is free
            const uint nseg = seg + nw * NB;
            if (s0 + nw * NB < nsb) v[i] = *(const float4*)(x + (size_t)min(nseg, nsb - 1u) * 256u + lane * 4u);
            if (seg < nsb) {
                float a = wave_max(fmaxf(fmaxf(fabsf(t.x), fabsf(t.y)), fmaxf(fabsf(t.z), fabsf(t.w))));
                float scale = a > 0.0f ? __fdiv_rn(a, 127.0f) : 1.0f;
                float inv = __fdiv_rn(1.0f, scale);
                int q0 = (int)sat127(roundf(__fmul_rn(t.x, inv)));
                int q1 = (int)sat127(roundf(__fmul_rn(t.y, inv)));
                int q2 = (int)sat127(roundf(__fmul_rn(t.z, inv)));
                int q3 = (int)sat127(roundf(__fmul_rn(t.w, inv)));
                *(uint*)(sx + seg * FQ_SEG + lane * 4u) =
                    (uint)(q0 & 0xFF) | ((uint)(q1 & 0xFF) << 8) | ((uint)(q2 & 0xFF) << 16) | ((uint)(q3 & 0xFF) << 24);
                if (lane == 0) ss[seg] = scale;
            }
        }
    }
    __syncthreads();
    // 4. the rows: one stream of (row group, super-block step) units, the next unit's weights requested before the
    //    current one is multiplied
    float acc[R], add[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        acc[r] = 0.0f;
        add[r] = (ACC && row0 < row_end) ? *rwc[r].y : 0.0f;
    }
    uint sb = g;
    while (row0 < row_end) {
        uint nsb_next = sb + 8u, nrow = row0;
        const bool last = nsb_next >= nsb + g;    // (sb - g) + 8 >= nsb: this was the group's last step
        if (last) { nsb_next = g; nrow = row0 + nw * R; }
        if (last) locate(nrow, rwn);
        else {
#pragma unroll
            for (int r = 0; r < R; r++) rwn[r] = rwc[r];
        }
        if (nrow < row_end) fetch(rwn, nsb_next, hn, qn);
        if (sb < nsb) {
            Q4kFrag f;
            const signed char* p = sx + sb * FQ_SEG + c * 64u + (l & 1u) * 16u;
            f.xl = *(const uint4*)p;
            f.xh = *(const uint4*)(p + 32);
            f.bl = bytesum4(f.xl);
            f.bh = bytesum4(f.xh);
            f.sx = ss[sb];
#pragma unroll
            for (int r = 0; r < R; r++) acc[r] += q4k_lane_dot(hc[r], qc[r], c, f);
        }
        if (last) {
#pragma unroll
            for (int r = 0; r < R; r++) {
                float t = R == 2 ? 0.0f : wave_sum(acc[r]);
                if (R == 2 && r == 0) {     // both sums in one pass; lane r holds row r's
                    const float t2 = wave_sum2(acc[0], acc[R - 1], lane);
                    if (lane < 2u && row0 + lane < row_end) *(lane ? rwc[R - 1].y : rwc[0].y) = ACC ? (lane ? add[R - 1] : add[0]) + t2 : t2;
                }
                if (R != 2 && lane == 0 && row0 + r < row_end) *rwc[r].y = ACC ? add[r] + t : t;
                acc[r] = 0.0f;
                add[r] = (ACC && nrow < row_end) ? *rwn[r].y : 0.0f;
            }
        }
#pragma unroll
        for (int r = 0; r < R; r++) { rwc[r] = rwn[r]; hc[r] = hn[r]; qc[r] = qn[r]; }
        sb = nsb_next;
        row0 = nrow;
    }
}

extern "C" __global__ void __launch_bounds__(1024)
gemv_fq8k_q4k_x4_r1(const float* x, const uchar* w0, const uchar* w1, const uchar* w2, const uchar* w3, float* y0, float* y1,
                    float* y2, float* y3, uint K, uint E0, uint E1, uint E2, uint E3, uint NRB, uint ACC) {
    gemv_fq8k_q4k_x4_body<1>(x, w0, w1, w2, w3, y0, y1, y2, y3, K, E0, E1, E2, E3, NRB, ACC);
}
extern "C" __global__ void __launch_bounds__(1024)
gemv_fq8k_q4k_x4_r2(const float* x, const uchar* w0, const uchar* w1, const uchar* w2, const uchar* w3, float* y0, float* y1,
                    float* y2, float* y3, uint K, uint E0, uint E1, uint E2, uint E3, uint NRB, uint ACC) {
    gemv_fq8k_q4k_x4_body<2>(x, w0, w1, w2, w3, y0, y1, y2, y3, K, E0, E1, E2, E3, NRB, ACC);
}

// Batched form: y[M][N] (+)= quantized x[M][K] . W^T.  One wave per row; the row's weights are
// read and unpacked once per tile of MT tokens.
template <int MT>
__device__ __forceinline__ void gemv_q8k_q4k_m_body(const signed char* __restrict__ xq, const float* __restrict__ xs,
                                                    const uchar* __restrict__ w, float* __restrict__ y,
                                                    uint K, uint N, uint M, uint ACC) {
    const uint lane = threadIdx.x & 63u;
    const uint row = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (row >= N) return;
    const uint nsb = K >> 8, g = lane >> 3, l = lane & 7u, c = l >> 1;
    for (uint m0 = 0; m0 < M; m0 += MT) {
        float acc[MT];
#pragma unroll
        for (int t = 0; t < MT; t++) acc[t] = 0.0f;
        for (uint sb = g; sb < nsb; sb += 8u) {
            const uchar* blk = w + ((size_t)row * nsb + sb) * Q4K_BYTES;
            uint4 hdr = *(const uint4*)blk;
            uint4 qs = *(const uint4*)(blk + 16u + l * 16u);
#pragma unroll
            for (int t = 0; t < MT; t++) {
                uint m = min(m0 + t, M - 1u);
                Q4kFrag f = q4k_load_frag(xq + (size_t)m * nsb * 256u, xs + (size_t)m * nsb, sb, l);
                acc[t] += q4k_lane_dot(hdr, qs, c, f);
            }
        }
#pragma unroll
        for (int t = 0; t < MT; t++) {
            float s = wave_sum(acc[t]);
            if (lane == 0 && m0 + t < M) {
                float* o = y + (size_t)(m0 + t) * N + row;
                *o = ACC ? *o + s : s;
            }
        }
    }
}

extern "C" __global__ void __launch_bounds__(256)
gemv_q8k_q4k_m(const signed char* xq, const float* xs, const uchar* w, float* y, uint K, uint N, uint M, uint ACC) {
    if (M <= 2) gemv_q8k_q4k_m_body<2>(xq, xs, w, y, K, N, M, ACC);
    else if (M <= 4) gemv_q8k_q4k_m_body<4>(xq, xs, w, y, K, N, M, ACC);
    else gemv_q8k_q4k_m_body<8>(xq, xs, w, y, K, N, M, ACC);
}

// ------------------------------------------------------------------ Q6_K
// Four lanes share a super-block and a wave walks sixteen per step.  Lane u = lane % 4 owns, in
// half hf = u / 2, the sixteen positions l0..l0+15 (l0 = 16 (u % 2)) of each of the four
// quarters: three 16-byte loads (two of ql, one of qh) give 64 six-bit codes, each quarter
// under one int8 sub-scale sc[8 hf + 2 q + u % 2].
struct Q6kX {          // a lane's share of the activations of one super-block
    uint4 x[4];        // 16 int8 per quarter
    int xs[4];         // their sums (for the -32 offset of the codes)
    float sx;
};

__device__ __forceinline__ Q6kX q6k_load_x(const signed char* xq, const float* xs, uint sb, uint hf, uint l0) {
    Q6kX f;
    const signed char* p = xq + (size_t)sb * 256u + hf * 128u + l0;
#pragma unroll
    for (int q = 0; q < 4; q++) {
        f.x[q] = *(const uint4*)(p + 32 * q);
        int t = dot4_i8(f.x[q].x, 0x01010101u, 0);
        t = dot4_i8(f.x[q].y, 0x01010101u, t);
        t = dot4_i8(f.x[q].z, 0x01010101u, t);
        f.xs[q] = dot4_i8(f.x[q].w, 0x01010101u, t);
    }
    f.sx = xs[sb];
    return f;
}

struct Q6kW {          // a lane's share of one super-block of one row
    u32x4_a2 qa, qb, qh;  // ql[l0..], ql[32 + l0..], qh[l0..] of the lane's half
    uint sc4;          // the four sub-scales, one per byte
    uint d16;
};

__device__ __forceinline__ Q6kW q6k_load_w(const uchar* blk, uint hf, uint l0) {
    Q6kW r;
    r.qa = *(const u32x4_a2*)(blk + hf * 64u + l0);
    r.qb = *(const u32x4_a2*)(blk + hf * 64u + 32u + l0);
    r.qh = *(const u32x4_a2*)(blk + 128u + hf * 32u + l0);
    u32x2_a2 s = *(const u32x2_a2*)(blk + 192u + hf * 8u);
    // bytes is, is+2, is+4, is+6 of the half's 8 sub-scales -> one per byte of sc4
    const uint is = l0 >> 4;
    const uint a = s.x >> (8u * is), b = s.y >> (8u * is);
    r.sc4 = (a & 0xFFu) | ((a >> 8) & 0xFF00u) | ((b & 0xFFu) << 16) | ((b << 8) & 0xFF000000u);
    r.d16 = *(const ushort*)(blk + 208u);
    return r;
}

// the 16 codes (0..63) of quarter Q as four dwords
template <int Q>
__device__ __forceinline__ void q6k_codes(const Q6kW& r, uint (&w)[4]) {
    const uint M4 = 0x0F0F0F0Fu, H2 = 0x30303030u;
    const uint ql[4] = {Q & 1 ? r.qb.x : r.qa.x, Q & 1 ? r.qb.y : r.qa.y, Q & 1 ? r.qb.z : r.qa.z, Q & 1 ? r.qb.w : r.qa.w};
    const uint qh[4] = {r.qh.x, r.qh.y, r.qh.z, r.qh.w};
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const uint lo = Q < 2 ? ql[j] & M4 : (ql[j] >> 4) & M4;
        const uint hi = Q == 0 ? (qh[j] << 4) & H2 : Q == 1 ? (qh[j] << 2) & H2 : Q == 2 ? qh[j] & H2 : (qh[j] >> 2) & H2;
        w[j] = lo | hi;
    }
}

__device__ __forceinline__ int dot16(const uint (&w)[4], const uint4& x) {
    int t = dot4_i8(w[0], x.x, 0);
    t = dot4_i8(w[1], x.y, t);
    t = dot4_i8(w[2], x.z, t);
    return dot4_i8(w[3], x.w, t);
}

__device__ __forceinline__ float q6k_lane_dot(const Q6kW& r, const Q6kX& f) {
    uint w[4];
    q6k_codes<0>(r, w); const int i0 = dot16(w, f.x[0]) - 32 * f.xs[0];
    q6k_codes<1>(r, w); const int i1 = dot16(w, f.x[1]) - 32 * f.xs[1];
    q6k_codes<2>(r, w); const int i2 = dot16(w, f.x[2]) - 32 * f.xs[2];
    q6k_codes<3>(r, w); const int i3 = dot16(w, f.x[3]) - 32 * f.xs[3];
    const int s0 = (int)(signed char)(r.sc4), s1 = (int)(signed char)(r.sc4 >> 8);
    const int s2 = (int)(signed char)(r.sc4 >> 16), s3 = (int)r.sc4 >> 24;
    const int isum = s0 * i0 + s1 * i1 + s2 * i2 + s3 * i3;
    return f.sx * f16_bits_to_f32(r.d16) * (float)isum;
}

template <int R, int MODE>
__device__ __forceinline__ void gemv_q8k_q6k_body(const signed char* __restrict__ xq, const float* __restrict__ xs,
                                                  const uchar* __restrict__ w, float* __restrict__ y,
                                                  const float* __restrict__ bs, uint K, uint N) {
    const uint lane = threadIdx.x & 63u;
    const uint row0 = (blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)) * R;
    if (row0 >= N) return;
    const uint nsb = K >> 8, g = lane >> 2, hf = (lane >> 1) & 1u, l0 = (lane & 1u) * 16u;
    float acc[R], add[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        acc[r] = 0.0f;
        add[r] = store_addend<MODE>(y, bs, min(row0 + r, N - 1u));
    }
    for (uint sb = g; sb < nsb; sb += 16u) {
        Q6kW raw[R];
#pragma unroll
        for (int r = 0; r < R; r++) {
            uint row = min(row0 + r, N - 1u);
            raw[r] = q6k_load_w(w + ((size_t)row * nsb + sb) * Q6K_BYTES, hf, l0);
        }
        Q6kX f = q6k_load_x(xq, xs, sb, hf, l0);
#pragma unroll
        for (int r = 0; r < R; r++) acc[r] += q6k_lane_dot(raw[r], f);
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
        float s = wave_sum(acc[r]);
        if (lane == 0 && row0 + r < N) store_row_with<MODE>(y, row0 + r, s, add[r]);
    }
}

GEMV_Q8K_ENTRIES(q6k, gemv_q8k_q6k_body)

// ---- the fused launches for the other K-quants ---------------------------------------------------
// A Q4_K_M file keeps some tensors of a stage in Q6_K or Q5_K (attention v, the feed-forward down) beside Q4_K ones;
// the reference fuses q/k/v and gate/up+activation for every format it decodes with
// (crates/ojas-cuda/src/kernels/gemv_q8.rs:105-143, :229-260).  These entries take a GGUF type per tensor (12 = Q4_K,
// 13 = Q5_K, 14 = Q6_K, one per byte of TYPES) and give every row the lane map and the order of operations of that
// type's single-tensor matvec — gemv_q8k_<fmt> — so each output has the bits of a launch of its own.  One row per wave.
//   gemv_q8k_kq_x4(xq, xs, w0, w1, w2, w3, y0, y1, y2, y3, K, E0, E1, E2, E3, TYPES)
//   ffn_gu_q8k_kq(xq, xs, wg, wu, out, K, N, ACT, TYPES)        TYPES: byte 0 gate, byte 1 up
__device__ __forceinline__ float kq_row_dot(uint type, const uchar* __restrict__ wrow, const signed char* __restrict__ xq,
                                            const float* __restrict__ xs, uint nsb, uint lane) {
    float acc = 0.0f;
    if (type == 14u) {            // gemv_q8k_q6k_body: four lanes per super-block
        const uint g = lane >> 2, hf = (lane >> 1) & 1u, l0 = (lane & 1u) * 16u;
        for (uint sb = g; sb < nsb; sb += 16u) {
            const Q6kW raw = q6k_load_w(wrow + (size_t)sb * Q6K_BYTES, hf, l0);
            const Q6kX f = q6k_load_x(xq, xs, sb, hf, l0);
            acc += q6k_lane_dot(raw, f);
        }
    } else {
        const uint g = lane >> 3, l = lane & 7u, c = l >> 1;
        if (type == 13u) {        // gemv_q8k_q5k_body
            for (uint sb = g; sb < nsb; sb += 8u) {
                const uchar* blk = wrow + (size_t)sb * Q5K_BYTES;
                const uint4 hdr = *(const uint4*)blk, qh = *(const uint4*)(blk + 16u + (l & 1u) * 16u);
                const uint4 qs = *(const uint4*)(blk + 48u + l * 16u);
                const Q4kFrag f = q4k_load_frag(xq, xs, sb, l);
                acc += q5k_lane_dot(hdr, qs, qh, c, f);
            }
        } else {                  // gemv_q8k_q4k_body
            for (uint sb = g; sb < nsb; sb += 8u) {
                const uchar* blk = wrow + (size_t)sb * Q4K_BYTES;
                const uint4 hdr = *(const uint4*)blk, qs = *(const uint4*)(blk + 16u + l * 16u);
                const Q4kFrag f = q4k_load_frag(xq, xs, sb, l);
                acc += q4k_lane_dot(hdr, qs, c, f);
            }
        }
    }
    return wave_sum(acc);
}
__device__ __forceinline__ uint kq_block_bytes(uint type) { return type == 14u ? Q6K_BYTES : type == 13u ? Q5K_BYTES : Q4K_BYTES; }

extern "C" __global__ void __launch_bounds__(256)
gemv_q8k_kq_x4(const signed char* xq, const float* xs, const uchar* w0, const uchar* w1, const uchar* w2, const uchar* w3,
               float* y0, float* y1, float* y2, float* y3, uint K, uint E0, uint E1, uint E2, uint E3, uint TYPES) {
    const uint lane = threadIdx.x & 63u;
    const uint gr = (uint)__builtin_amdgcn_readfirstlane((int)(blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)));
    if (gr >= E3) return;
    const uint nsb = K >> 8;
    const uchar* w;
    float* y;
    uint lr, type;
    if (gr < E0) { w = w0; y = y0; lr = gr; type = TYPES & 0xFFu; }
    else if (gr < E1) { w = w1; y = y1; lr = gr - E0; type = (TYPES >> 8) & 0xFFu; }
    else if (gr < E2) { w = w2; y = y2; lr = gr - E1; type = (TYPES >> 16) & 0xFFu; }
    else { w = w3; y = y3; lr = gr - E2; type = TYPES >> 24; }
    const float t = kq_row_dot(type, w + (size_t)lr * nsb * kq_block_bytes(type), xq, xs, nsb, lane);
    if (lane == 0) y[lr] = t;
}

extern "C" __global__ void __launch_bounds__(256)
ffn_gu_q8k_kq(const signed char* __restrict__ xq, const float* __restrict__ xs, const uchar* __restrict__ wg,
              const uchar* __restrict__ wu, float* __restrict__ out, uint K, uint N, uint ACT, uint TYPES) {
    const uint lane = threadIdx.x & 63u;
    const uint row = (uint)__builtin_amdgcn_readfirstlane((int)(blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)));
    if (row >= N) return;
    const uint nsb = K >> 8, tg = TYPES & 0xFFu, tu = (TYPES >> 8) & 0xFFu;
    const float sg = kq_row_dot(tg, wg + (size_t)row * nsb * kq_block_bytes(tg), xq, xs, nsb, lane);
    const float su = kq_row_dot(tu, wu + (size_t)row * nsb * kq_block_bytes(tu), xq, xs, nsb, lane);
    if (lane == 0) out[row] = ffn_act(sg, ACT) * su;
}

// Tall matrices (an output head): rows grid-stride, the wave's share of the quantized activations
// loaded once and kept in registers (21 per 4096 of K), so the per-row traffic through the vector
// memory path is the row's own bytes only (head 151936 x 4096: 104 -> 93 us; the same form of the
// Q4_K kernel, whose activation fragment is a third the size, measured 5 % slower than one wave
// per two rows and is not built).
//   gemv_q8k_q6k_px(xq, xs, w, y, K, N)     K <= 8192; any grid of 256-thread workgroups
template <int NS>
__device__ __forceinline__ void gemv_q8k_q6k_px_body(const signed char* __restrict__ xq, const float* __restrict__ xs,
                                                     const uchar* __restrict__ w, float* __restrict__ y, uint K, uint N) {
    constexpr int R = 2;
    const uint lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint nsb = K >> 8, g = lane >> 2, hf = (lane >> 1) & 1u, l0 = (lane & 1u) * 16u;
    Q6kX f[NS];
#pragma unroll
    for (int s = 0; s < NS; s++) {
        const uint sb = (uint)s * 16u + g;
        f[s] = q6k_load_x(xq, xs, min(sb, nsb - 1u), hf, l0);
        if (sb >= nsb) f[s].sx = 0.0f;            // lanes past the row's end contribute nothing
    }
    for (uint row0 = (blockIdx.x * 4u + wave) * R; row0 < N; row0 += gridDim.x * 4u * R) {
        float acc[R];
#pragma unroll
        for (int r = 0; r < R; r++) acc[r] = 0.0f;
#pragma unroll
        for (int s = 0; s < NS; s++) {
            const uint sb = min((uint)s * 16u + g, nsb - 1u);
            Q6kW raw[R];
#pragma unroll
            for (int r = 0; r < R; r++)
                raw[r] = q6k_load_w(w + ((size_t)min(row0 + r, N - 1u) * nsb + sb) * Q6K_BYTES, hf, l0);
#pragma unroll
            for (int r = 0; r < R; r++) acc[r] += q6k_lane_dot(raw[r], f[s]);
        }
#pragma unroll
        for (int r = 0; r < R; r++) {
            const float t = wave_sum(acc[r]);
            if (lane == 0 && row0 + r < N) y[row0 + r] = t;
        }
    }
}
extern "C" __global__ void __launch_bounds__(256)
gemv_q8k_q6k_px(const signed char* xq, const float* xs, const uchar* w, float* y, uint K, uint N) {
    if (K <= 4096u) gemv_q8k_q6k_px_body<1>(xq, xs, w, y, K, N);
    else gemv_q8k_q6k_px_body<2>(xq, xs, w, y, K, N);
}

template <int MT>
__device__ __forceinline__ void gemv_q8k_q6k_m_body(const signed char* __restrict__ xq, const float* __restrict__ xs,
                                                    const uchar* __restrict__ w, float* __restrict__ y,
                                                    uint K, uint N, uint M, uint ACC) {
    const uint lane = threadIdx.x & 63u;
    const uint row = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (row >= N) return;
    const uint nsb = K >> 8, g = lane >> 2, hf = (lane >> 1) & 1u, l0 = (lane & 1u) * 16u;
    for (uint m0 = 0; m0 < M; m0 += MT) {
        float acc[MT];
#pragma unroll
        for (int i = 0; i < MT; i++) acc[i] = 0.0f;
        for (uint sb = g; sb < nsb; sb += 16u) {
            Q6kW raw = q6k_load_w(w + ((size_t)row * nsb + sb) * Q6K_BYTES, hf, l0);
#pragma unroll
            for (int i = 0; i < MT; i++) {
                uint m = min(m0 + i, M - 1u);
                Q6kX f = q6k_load_x(xq + (size_t)m * nsb * 256u, xs + (size_t)m * nsb, sb, hf, l0);
                acc[i] += q6k_lane_dot(raw, f);
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

extern "C" __global__ void __launch_bounds__(256)
gemv_q8k_q6k_m(const signed char* xq, const float* xs, const uchar* w, float* y, uint K, uint N, uint M, uint ACC) {
    if (M <= 2) gemv_q8k_q6k_m_body<2>(xq, xs, w, y, K, N, M, ACC);
    else if (M <= 4) gemv_q8k_q6k_m_body<4>(xq, xs, w, y, K, N, M, ACC);
    else gemv_q8k_q6k_m_body<8>(xq, xs, w, y, K, N, M, ACC);
}

// Few tokens against a long tensor (speculative verify on the output head): the quantized
// activations of all M <= 16 tokens are staged once per workgroup in LDS, laid out so that the 64
// lanes of a wave read 64 consecutive 16-byte pieces per (token, step, quarter); a wave then
// walks rows grid-stride, turns a row's codes into signed bytes once (w - 32: flip bit 5, then
// copy the flipped bit into bits 6 and 7) and runs plain int8 dots against every token.
//   gemv_q8k_q6k_mx(xq, xs, w, y, K, N, M, ACC)    M <= 16, M * ceil(K/4096) <= 19 (80 KB of LDS,
//                                                  two workgroups per CU); any grid of 256-thread blocks
#define Q6K_MX_LDS 81920u
template <int MT>
__device__ __forceinline__ void gemv_q8k_q6k_mx_body(const signed char* __restrict__ xq, const float* __restrict__ xs,
                                                     const uchar* __restrict__ w, float* __restrict__ y,
                                                     uint K, uint N, uint M, uint ACC, uchar* lds) {
    const uint tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint nsb = K >> 8, nstep = (nsb + 15u) >> 4;
    // LDS: token t, step s, quarter q, lane -> 16 bytes at ((t * nstep + s) * 4 + q) * 1024 + lane * 16;
    // then the scales, token-major, one float per super-block (zero beyond nsb)
    const uint xbytes = M * nstep * 4096u;
    float* lsx = (float*)(lds + xbytes);
    for (uint i = tid; i < M * nstep * 256u; i += 256u) {   // one 16-byte piece per trip
        const uint ln = i & 63u, q = (i >> 6) & 3u, ts = i >> 8, s = ts % nstep, t = ts / nstep;
        const uint sb = s * 16u + (ln >> 2);
        uint4 v = make_uint4(0u, 0u, 0u, 0u);
        if (sb < nsb) v = *(const uint4*)(xq + (size_t)t * nsb * 256u + sb * 256u + ((ln >> 1) & 1u) * 128u + q * 32u + (ln & 1u) * 16u);
        *(uint4*)(lds + (size_t)i * 16u) = v;
    }
    for (uint i = tid; i < M * nstep * 16u; i += 256u) {
        const uint sb = i % (nstep * 16u), t = i / (nstep * 16u);
        lsx[i] = sb < nsb ? xs[(size_t)t * nsb + sb] : 0.0f;
    }
    __syncthreads();
    const uint g = lane >> 2, hf = (lane >> 1) & 1u, l0 = (lane & 1u) * 16u;
    constexpr int R = 2;   // rows per wave and trip: twice the loads in flight, half the LDS reads per row
    for (uint row0 = (blockIdx.x * 4u + wave) * R; row0 < N; row0 += gridDim.x * 4u * R) {
        float acc[R][MT];
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int t = 0; t < MT; t++) acc[r][t] = 0.0f;
        for (uint s = 0; s < nstep; s++) {
            const uint sb = min(s * 16u + g, nsb - 1u);   // lanes past the row's end re-read its last block against zero scales
            Q6kW raw[R];
#pragma unroll
            for (int r = 0; r < R; r++)
                raw[r] = q6k_load_w(w + ((size_t)min(row0 + r, N - 1u) * nsb + sb) * Q6K_BYTES, hf, l0);
            uint c[R][4][4];
            int sc[R][4];
            float d[R];
#pragma unroll
            for (int r = 0; r < R; r++) {
                q6k_codes<0>(raw[r], c[r][0]); q6k_codes<1>(raw[r], c[r][1]);
                q6k_codes<2>(raw[r], c[r][2]); q6k_codes<3>(raw[r], c[r][3]);
#pragma unroll
                for (int q = 0; q < 4; q++)
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        const uint x = c[r][q][j] ^ 0x20202020u, m = x & 0x20202020u;
                        c[r][q][j] = x | (m << 1) | (m << 2);
                    }
                sc[r][0] = (int)(signed char)(raw[r].sc4); sc[r][1] = (int)(signed char)(raw[r].sc4 >> 8);
                sc[r][2] = (int)(signed char)(raw[r].sc4 >> 16); sc[r][3] = (int)raw[r].sc4 >> 24;
                d[r] = f16_bits_to_f32(raw[r].d16);
            }
#pragma unroll
            for (int t = 0; t < MT; t++) {
                if (t < (int)M) {
                    const uchar* px = lds + ((size_t)(t * nstep + s) * 4u) * 1024u + lane * 16u;
                    const uint4 x0 = *(const uint4*)px, x1 = *(const uint4*)(px + 1024);
                    const uint4 x2 = *(const uint4*)(px + 2048), x3 = *(const uint4*)(px + 3072);
                    const float sx = lsx[(t * nstep + s) * 16u + g];
#pragma unroll
                    for (int r = 0; r < R; r++) {
                        const int isum = sc[r][0] * dot16(c[r][0], x0) + sc[r][1] * dot16(c[r][1], x1) +
                                         sc[r][2] * dot16(c[r][2], x2) + sc[r][3] * dot16(c[r][3], x3);
                        acc[r][t] += sx * d[r] * (float)isum;
                    }
                }
            }
        }
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int t = 0; t < MT; t++) {
                if (t < (int)M) {
                    const float sum = wave_sum(acc[r][t]);
                    if (lane == 0 && row0 + r < N) {
                        float* o = y + (size_t)t * N + row0 + r;
                        *o = ACC ? *o + sum : sum;
                    }
                }
            }
    }
}

extern "C" __global__ void __launch_bounds__(256)
gemv_q8k_q6k_mx(const signed char* xq, const float* xs, const uchar* w, float* y, uint K, uint N, uint M, uint ACC) {
    __shared__ __attribute__((aligned(16))) uchar lds_mx[Q6K_MX_LDS];
    if (M <= 4) gemv_q8k_q6k_mx_body<4>(xq, xs, w, y, K, N, M, ACC, lds_mx);
    else if (M <= 8) gemv_q8k_q6k_mx_body<8>(xq, xs, w, y, K, N, M, ACC, lds_mx);
    else gemv_q8k_q6k_mx_body<16>(xq, xs, w, y, K, N, M, ACC, lds_mx);
}

// ---- Q6_K against up to 16 tokens on the int8 matrix cores ------------------------------------
//   gemv_q8k_q6k_mf(xq, xs, w, y, K, N, M, ACC)    M <= 16, MT (K + 32) + K / 4 + 256 <= 69632 (MT = 8 or 16)
// The verify head reads 510 MB of weights whatever the token count; with integer dots the work
// per row grows with M and the launch turns compute-bound from M = 4.  Here a wave owns 16 rows
// and runs them against 8 tokens at a time with v_mfma_i32_16x16x32_i8:
//   * B (weights): lane (n, kg) = (lane % 16, lane / 16) builds, for each of the eight 32-weight
//     quarters of a super-block, the signed codes q - 32 of positions 8 kg .. 8 kg + 7 of row n;
//   * a quarter holds two 16-weight groups with their own int8 scale, and an MFMA sums over all
//     32 positions.  So the 16 token rows of A are 8 tokens twice: rows 0-7 carry only positions
//     0-15 (lanes kg < 2), rows 8-15 only positions 16-31 (lanes kg >= 2); the other lanes read
//     zeros (from one 256-byte LDS region, so no lane is switched off around the reads).  D then has a token's two group dots in different rows, each multiplied by
//     its own scale with one integer multiply-add; the two halves meet once per 16-row tile;
//   * activations wait in LDS, token rows 32 bytes longer than K so that the 32 live lanes of an
//     8-byte read fall in 64 distinct banks.
// Per super-block and lane the arithmetic is dot_q6k's: sx * d * sum_g scale_g * idot_g, integer
// sums exact (crates/ojas-cpu/src/cpu_math.rs:674-722).
typedef int q6k_i4 __attribute__((ext_vector_type(4)));

struct Q6kMfW {          // lane (n, kg): its bytes of one super-block of row n
    u32x2_a2 la[2], lb[2], qh[2];   // per half: ql[8 kg ..], ql[32 + 8 kg ..], qh[8 kg ..]
    u32x4_a2 sc;
    uint d16;
};
__device__ __forceinline__ Q6kMfW q6k_mf_load(const uchar* blk, uint kg) {
    Q6kMfW r;
    const uint sh = ((uint)(size_t)blk & 2u) << 3;
    const uchar* b4 = blk - ((size_t)blk & 2u);
#pragma unroll
    for (int hf = 0; hf < 2; hf++) {
        r.la[hf] = q6k_ld8(b4 + 64u * hf + 8u * kg, sh);
        r.lb[hf] = q6k_ld8(b4 + 64u * hf + 32u + 8u * kg, sh);
        r.qh[hf] = q6k_ld8(b4 + 128u + 32u * hf + 8u * kg, sh);
    }
    const uint* ps = (const uint*)(b4 + 192u);
    const uint s0 = ps[0], s1 = ps[1], s2 = ps[2], s3 = ps[3], s4 = ps[4];   // scales, d and up to two bytes more
    r.sc.x = __builtin_amdgcn_alignbit(s1, s0, sh);
    r.sc.y = __builtin_amdgcn_alignbit(s2, s1, sh);
    r.sc.z = __builtin_amdgcn_alignbit(s3, s2, sh);
    r.sc.w = __builtin_amdgcn_alignbit(s4, s3, sh);
    r.d16 = (s4 >> sh) & 0xFFFFu;
    return r;
}

// Token rows 0 .. rows - 1 (K int8 each, zeros from row M on) into LDS rows S bytes apart: 16 bytes per
// thread and step, eight loads in flight before the first store (one load, one store, one wait per
// step is a chain of cache latencies: fourteen of them for 8 tokens of K = 14336 and 512 threads).
__device__ __forceinline__ void q8k_stage_tokens(uchar* lds, const signed char* __restrict__ xq, uint K, uint S, uint M, uint rows) {
    const uint per_row = K >> 4, total = rows * per_row, nt = blockDim.x;
    for (uint i0 = threadIdx.x; i0 < total; i0 += 8u * nt) {
        uint4 v[8];
        uint dst[8];
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const uint i = i0 + (uint)u * nt, t = i / per_row, o = (i - t * per_row) << 4;
            v[u] = make_uint4(0u, 0u, 0u, 0u);
            dst[u] = t * S + o;
            if (i < total && t < M) v[u] = *(const uint4*)(xq + (size_t)t * K + o);
        }
#pragma unroll
        for (int u = 0; u < 8; u++)
            if (i0 + (uint)u * nt < total) *(uint4*)(lds + dst[u]) = v[u];
    }
}

// One super-block of a 16-row tile against P passes of 8 tokens: acc += sx * d * sum_g scale_g * idot_g.
// xp[p]: the lane's 8 bytes of pass p's token row at this super-block (row n % 8, byte 8 kg) if its A
// rows carry its positions, else 256 bytes of zeros; sx: the super-block's 16 token scales.
template <int P>
__device__ __forceinline__ void q6k_mf_superblock(const Q6kMfW& cur, const uchar* const (&xp)[P], uint kg, const float* sx16,
                                                  float (&acc)[P][4]) {
    const uint h = kg >> 1;                        // which 16-weight group of a quarter the lane's D rows hold
    int isum[P][4];
#pragma unroll
    for (int p = 0; p < P; p++)
#pragma unroll
        for (int v = 0; v < 4; v++) isum[p][v] = 0;
#pragma unroll
    for (int hf = 0; hf < 2; hf++) {
        // scales 8 hf + 2 q + h, q = 0..3: bytes h, 2 + h of the half's two dwords
        const uint s_lo = (hf ? cur.sc.z : cur.sc.x) >> (8u * h), s_hi = (hf ? cur.sc.w : cur.sc.y) >> (8u * h);
        const int scl[4] = {(int)(signed char)s_lo, (int)(signed char)(s_lo >> 16), (int)(signed char)s_hi,
                            (int)(signed char)(s_hi >> 16)};
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const u32x2_a2 ql = (q & 1) ? cur.lb[hf] : cur.la[hf];
            const long B = q6k_signed8(ql.x, ql.y, cur.qh[hf].x, cur.qh[hf].y, q);
#pragma unroll
            for (int p = 0; p < P; p++) {
                const long A = *(const long*)(xp[p] + 128u * hf + 32u * q);
                const q6k_i4 zero = {0, 0, 0, 0};
                const q6k_i4 D = __builtin_amdgcn_mfma_i32_16x16x32_i8(A, B, zero, 0, 0, 0);
#pragma unroll
                for (int v = 0; v < 4; v++) isum[p][v] += __mul24(scl[q], D[v]);
            }
        }
    }
    const float d = f16_bits_to_f32(cur.d16);
#pragma unroll
    for (int p = 0; p < P; p++) {
        const float4 sx = *(const float4*)(sx16 + 8u * p + 4u * (kg & 1u));
        acc[p][0] += sx.x * d * (float)isum[p][0];
        acc[p][1] += sx.y * d * (float)isum[p][1];
        acc[p][2] += sx.z * d * (float)isum[p][2];
        acc[p][3] += sx.w * d * (float)isum[p][3];
    }
}

template <int P>   // P passes of 8 tokens
__device__ __forceinline__ void gemv_q8k_q6k_mf_body(const signed char* __restrict__ xq, const float* __restrict__ xs,
                                                     const uchar* __restrict__ w, float* __restrict__ y,
                                                     uint K, uint N, uint M, uint ACC, uchar* lds) {
    const uint tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint nsb = K >> 8, S = K + 32u;
    float* lsx = (float*)(lds + (size_t)(8 * P) * S);       // [sb][16] token scales
    uchar* zeros = (uchar*)(lsx + nsb * 16u);               // 256 bytes the idle half of the A lanes reads
    if (tid < 64u) ((uint*)zeros)[tid] = 0u;
    // stage the tokens (rows past M are zero) and their scales
    q8k_stage_tokens(lds, xq, K, S, M, (uint)(8 * P));
    for (uint i = tid; i < nsb * 16u; i += blockDim.x) {
        const uint sb = i >> 4, t = i & 15u;
        lsx[i] = t < M ? xs[(size_t)t * nsb + sb] : 0.0f;
    }
    __syncthreads();
    const uint n = lane & 15u, kg = lane >> 4;
    const bool live = (n < 8u) == (kg < 2u);       // this lane's A rows carry its positions
    const uchar* xa = live ? lds + (size_t)(n & 7u) * S + 8u * kg : zeros + 8u * kg;
    const uint xstep = live ? 256u : 0u, xpass = live ? 8u * S : 0u;
    const uint tiles = (N + 15u) >> 4;
    const uint nwave = blockDim.x >> 6;
    for (uint tile = blockIdx.x * nwave + wave; tile < tiles; tile += gridDim.x * nwave) {
        const uint row = min(tile * 16u + n, N - 1u);
        const uchar* wr = w + (size_t)row * nsb * Q6K_BYTES;
        float acc[P][4];
#pragma unroll
        for (int p = 0; p < P; p++)
#pragma unroll
            for (int v = 0; v < 4; v++) acc[p][v] = 0.0f;
        // two super-blocks ahead: a wave has ~8 KB on its way, which is what eight waves per CU need
        Q6kMfW cur = q6k_mf_load(wr, kg), nx = q6k_mf_load(wr + (size_t)min(1u, nsb - 1u) * Q6K_BYTES, kg);
        for (uint sb = 0; sb < nsb; sb++) {
            const Q6kMfW nx2 = q6k_mf_load(wr + (size_t)min(sb + 2u, nsb - 1u) * Q6K_BYTES, kg);
            const uchar* xp[P];
#pragma unroll
            for (int p = 0; p < P; p++) xp[p] = xa + sb * xstep + p * xpass;
            q6k_mf_superblock<P>(cur, xp, kg, lsx + sb * 16u, acc);
            cur = nx;
            nx = nx2;
        }
        // D rows 4 kg + v: token 4 (kg & 1) + v, first group in lanes kg < 2, second in kg >= 2
#pragma unroll
        for (int p = 0; p < P; p++)
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const float tot = acc[p][v] + __shfl_xor(acc[p][v], 32, 64);
                const uint t = 8u * p + 4u * kg + v;
                if (kg < 2u && t < M && tile * 16u + n < N) {
                    float* o = y + (size_t)t * N + tile * 16u + n;
                    *o = ACC ? *o + tot : tot;
                }
            }
    }
}

#define Q6K_MF_LDS 69632u    // 16 tokens of K = 4096: two workgroups per CU
extern "C" __global__ void __launch_bounds__(256)
gemv_q8k_q6k_mf(const signed char* xq, const float* xs, const uchar* w, float* y, uint K, uint N, uint M, uint ACC) {
    __shared__ __attribute__((aligned(16))) uchar lds_mf[Q6K_MF_LDS];
    if (M <= 8) gemv_q8k_q6k_mf_body<1>(xq, xs, w, y, K, N, M, ACC, lds_mf);
    else gemv_q8k_q6k_mf_body<2>(xq, xs, w, y, K, N, M, ACC, lds_mf);
}

// ---- the same tile on few rows: its super-blocks split over the workgroup's waves --------------
//   gemv_q8k_q6k_mk(xq, xs, w, y, K, N, M, ACC)   M <= 16, block 512, 8 P (K + 32) + K / 4 + 256 + 4096 P <= 163840
// A projection of a few thousand rows has fewer 16-row tiles than the GPU has waves, and a wave
// that walks a whole row of K = 14336 alone is a chain of 56 dependent steps.  Here a workgroup
// owns a tile: wave w takes super-blocks w, w + 8, ...; the eight partial sums meet in LDS and are
// added in wave order.  All of LDS belongs to the one workgroup of a CU, so 8 tokens of K up to
// 18000 (16 of K up to 9000) wait there whole.
#define Q6K_MK_LDS 163840u
template <int P>
__device__ __forceinline__ void gemv_q8k_q6k_mk_body(const signed char* __restrict__ xq, const float* __restrict__ xs,
                                                     const uchar* __restrict__ w, float* __restrict__ y,
                                                     uint K, uint N, uint M, uint ACC, uchar* lds) {
    const uint tid = threadIdx.x, lane = tid & 63u;
    const uint wave = (uint)__builtin_amdgcn_readfirstlane((int)(tid >> 6)), nw = blockDim.x >> 6;
    const uint nsb = K >> 8, S = K + 32u;
    float* lsx = (float*)(lds + (size_t)(8 * P) * S);       // [sb][16] token scales
    uchar* zeros = (uchar*)(lsx + nsb * 16u);               // 256 bytes the idle half of the A lanes reads
    float* red = (float*)(zeros + 256u);                    // [wave][4 P][32]
    if (tid < 64u) ((uint*)zeros)[tid] = 0u;
    q8k_stage_tokens(lds, xq, K, S, M, (uint)(8 * P));
    for (uint i = tid; i < nsb * 16u; i += blockDim.x) {
        const uint sb = i >> 4, t = i & 15u;
        lsx[i] = t < M ? xs[(size_t)t * nsb + sb] : 0.0f;
    }
    __syncthreads();
    const uint n = lane & 15u, kg = lane >> 4;
    const bool live = (n < 8u) == (kg < 2u);
    const uchar* xa = live ? lds + (size_t)(n & 7u) * S + 8u * kg : zeros + 8u * kg;
    const uint xstep = live ? 256u : 0u, xpass = live ? 8u * S : 0u;
    const uint tiles = (N + 15u) >> 4;
    for (uint tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
        const uint row = min(tile * 16u + n, N - 1u);
        const uchar* wr = w + (size_t)row * nsb * Q6K_BYTES;
        float acc[P][4];
#pragma unroll
        for (int p = 0; p < P; p++)
#pragma unroll
            for (int v = 0; v < 4; v++) acc[p][v] = 0.0f;
        Q6kMfW cur = q6k_mf_load(wr + (size_t)min(wave, nsb - 1u) * Q6K_BYTES, kg);
        for (uint sb = wave; sb < nsb; sb += nw) {
            const Q6kMfW nx = q6k_mf_load(wr + (size_t)min(sb + nw, nsb - 1u) * Q6K_BYTES, kg);
            const uchar* xp[P];
#pragma unroll
            for (int p = 0; p < P; p++) xp[p] = xa + sb * xstep + p * xpass;
            q6k_mf_superblock<P>(cur, xp, kg, lsx + sb * 16u, acc);
            cur = nx;
        }
        // D rows 4 kg + v: token 4 (kg & 1) + v, first group in lanes kg < 2, second in kg >= 2
#pragma unroll
        for (int p = 0; p < P; p++)
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const float tot = acc[p][v] + __shfl_xor(acc[p][v], 32, 64);
                if (lane < 32u) red[(wave * (uint)(4 * P) + (uint)(4 * p + v)) * 32u + lane] = tot;
            }
        __syncthreads();
        if (tid < (uint)(128 * P)) {
            const uint l32 = tid & 31u, pv = tid >> 5;
            float sum = red[pv * 32u + l32];
            for (uint w8 = 1; w8 < nw; w8++) sum += red[(w8 * (uint)(4 * P) + pv) * 32u + l32];
            const uint nn = l32 & 15u, t = 8u * (pv >> 2) + 4u * (l32 >> 4) + (pv & 3u);
            if (t < M && tile * 16u + nn < N) {
                float* o = y + (size_t)t * N + tile * 16u + nn;
                *o = ACC ? *o + sum : sum;
            }
        }
        __syncthreads();                                    // before the next tile's partial sums
    }
}

extern "C" __global__ void __launch_bounds__(512)
gemv_q8k_q6k_mk(const signed char* xq, const float* xs, const uchar* w, float* y, uint K, uint N, uint M, uint ACC) {
    __shared__ __attribute__((aligned(16))) uchar lds_mk[Q6K_MK_LDS];
    if (M <= 8) gemv_q8k_q6k_mk_body<1>(xq, xs, w, y, K, N, M, ACC, lds_mk);
    else gemv_q8k_q6k_mk_body<2>(xq, xs, w, y, K, N, M, ACC, lds_mk);
}

// ---- the same tile with the weights copied through LDS ----------------------------------------
//   gemv_q8k_q6k_ml(xq, xs, w, y, K, N, M, ACC)    M <= 16, 512 threads, w 16-byte aligned and readable up to the next
//       multiple of 16 past its last row, rows within 4 GiB,
//       8 (K + 32) + K / 4 + 87040 <= 163840 (M <= 8)   16 (K + 32) + K / 4 + 58112 <= 163840 (M > 8)
// gemv_q8k_q6k_mf is bound by its loads: 8-byte pieces of sixteen rows a row apart, three aligned
// dwords fetched and shifted for each.  Here the memory system copies them: one
// global_load_lds_dwordx4 moves four super-blocks (rows 4 i .. 4 i + 3 of the tile at one k),
// fourteen lanes each, into 224-byte LDS slots.  A super-block is 210 bytes and starts at any even
// address; the copy starts at the 16-byte boundary below it (copies from 2-byte-aligned addresses
// run a tenth slower: 102 -> 92 us for the bare copy stream of a 151936 x 4096 head), and 224
// bytes from there always hold the block, m = 0, 2 .. 14 bytes into the slot.  The readers fetch
// the aligned dwords around each 8-byte piece and shift (m & 2), as gemv_q8k_q6k_mf does from
// memory.  Each wave owns a ring of D units (one unit = the wave's 16 rows at one super-block,
// four copies) and walks its tiles as one stream of units, D copies ahead across tile borders (a
// unit's slot is given to the copy D units on as soon as its bytes are in registers);
// waves never wait for each other after the tokens are staged.
// The sixteen slots of a unit are packed (row n at 224 n, 16 bytes further for n >= 8: 224 bytes are 56 banks, so rows
// 0 .. 7 start at banks 0, 56, .. 8 and rows 8 .. 15 between them).  The readers' dword fetches still meet two to a bank
// (the conflict counter reads 57 % of LDS-active cycles with this layout as with slots 1024 bytes apart); LDS time is
// not what bounds the kernel.  A unit is 3616 bytes (the last slot's readers may fetch a dword past it):
// rings are 4 units deep up to 8 tokens and 3 beyond where that fits beside the tokens (one less where not), so 4 (3)
// units of 3360 weight bytes are on their way per wave while it works.
#define Q6K_ML_SLOT 224u
#define Q6K_ML_UNIT 3616u
#define Q6K_ML_LDS 163840u

template <int P, int D>
__device__ __forceinline__ void gemv_q8k_q6k_ml_body(const signed char* __restrict__ xq, const float* __restrict__ xs,
                                                     const uchar* __restrict__ w, float* __restrict__ y,
                                                     uint K, uint N, uint M, uint ACC, uchar* lds, uint lds_addr) {
    const uint tid = threadIdx.x, lane = tid & 63u;
    const uint wave = (uint)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint nsb = K >> 8, S = K + 32u;
    const uint o_lsx = (uint)(8 * P) * S, o_zero = o_lsx + nsb * 64u, o_ring = o_zero + 256u + wave * ((uint)D * Q6K_ML_UNIT);
    float* lsx = (float*)(lds + o_lsx);            // [sb][16] token scales
    if (tid < 64u) ((uint*)(lds + o_zero))[tid] = 0u;   // what the idle half of the A lanes reads
    q8k_stage_tokens(lds, xq, K, S, M, (uint)(8 * P));
    for (uint i = tid; i < nsb * 16u; i += blockDim.x) {
        const uint sb = i >> 4, t = i & 15u;
        lsx[i] = t < M ? xs[(size_t)t * nsb + sb] : 0.0f;
    }
    __syncthreads();                               // the only barrier; these loads are older than every copy
    // wave ids interleave over the workgroups, so each CU gets its share of the waves with one tile more
    const uint tiles = (N + 15u) >> 4, stride = gridDim.x * (blockDim.x >> 6), first = wave * gridDim.x + blockIdx.x;
    const uint my_tiles = first < tiles ? (tiles - first + stride - 1u) / stride : 0u;
    const uint total = my_tiles * nsb;             // units this wave walks
    const uint row_bytes = nsb * Q6K_BYTES;
    // the copy stream: lane -> slot cq of a copy, piece cpc of the slot
    const uint cq = lane / 14u, cpc = lane - cq * 14u;
    const bool con = lane < 56u;
    uint i_off[4], iu = 0u, i_sb = 0u, i_tile = first, i_slot = 0u;
    auto issue_next = [&]() {
        if (i_sb == 0u) {
#pragma unroll
            for (uint i = 0; i < 4u; i++) i_off[i] = min(i_tile * 16u + 4u * i + cq, N - 1u) * row_bytes;
        }
        const uint dst = lds_addr + o_ring + i_slot * Q6K_ML_UNIT, sbo = i_sb * Q6K_BYTES;
        if (con) {
#pragma unroll
            for (uint i = 0; i < 4u; i++) lds_dma16(w, ((i_off[i] + sbo) & ~15u) + cpc * 16u, dst + i * 896u + (i >> 1) * 16u);
        }
        iu++;
        i_slot = i_slot + 1u == (uint)D ? 0u : i_slot + 1u;
        if (++i_sb == nsb) {
            i_sb = 0u;
            i_tile += stride;
        }
    };
    for (uint k = 0; k < (uint)D; k++)
        if (iu < total) issue_next();
    const uint n = lane & 15u, kg = lane >> 4;
    const bool live = (n < 8u) == (kg < 2u);
    const uchar* xa = live ? lds + (size_t)(n & 7u) * S + 8u * kg : lds + o_zero + 8u * kg;
    const uint xstep = live ? 256u : 0u, xpass = live ? 8u * S : 0u;
    const uchar* rd = lds + o_ring + n * Q6K_ML_SLOT + (n >> 3) * 16u;
    // the lane's row starts (row nsb) & 7 super-blocks past a 16-byte boundary, each 2 bytes further
    uint c_r8 = min(first * 16u + n, N - 1u) * nsb;
    float acc[P][4];
#pragma unroll
    for (int p = 0; p < P; p++)
#pragma unroll
        for (int v = 0; v < 4; v++) acc[p][v] = 0.0f;
    uint c_sb = 0u, c_tile = first, c_slot = 0u;
    for (uint u = 0; u < total; u++) {
        vm_wait(min(total - 1u - u, (uint)D - 1u) * 4u);
        const uchar* blk = rd + c_slot * Q6K_ML_UNIT + (((c_r8 + c_sb) & 7u) << 1);
        c_slot = c_slot + 1u == (uint)D ? 0u : c_slot + 1u;
        const Q6kMfW cur = q6k_mf_load(blk, kg);
        // the unit is in registers: its slot takes unit u + D while this one is worked on
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (iu < total) issue_next();
        const uchar* xp[P];
#pragma unroll
        for (int p = 0; p < P; p++) xp[p] = xa + c_sb * xstep + p * xpass;
        q6k_mf_superblock<P>(cur, xp, kg, lsx + c_sb * 16u, acc);
        if (++c_sb == nsb) {
            // D rows 4 kg + v: token 4 (kg & 1) + v, first group in lanes kg < 2, second in kg >= 2
#pragma unroll
            for (int p = 0; p < P; p++)
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    const float tot = acc[p][v] + __shfl_xor(acc[p][v], 32, 64);
                    const uint t = 8u * p + 4u * kg + v;
                    if (kg < 2u && t < M && c_tile * 16u + n < N) {
                        float* o = y + (size_t)t * N + c_tile * 16u + n;
                        *o = ACC ? *o + tot : tot;
                    }
                    acc[p][v] = 0.0f;
                }
            c_sb = 0u;
            c_tile += stride;
            c_r8 = min(c_tile * 16u + n, N - 1u) * nsb;
        }
    }
}

extern "C" __global__ void __launch_bounds__(512)
gemv_q8k_q6k_ml(const signed char* xq, const float* xs, const uchar* w, float* y, uint K, uint N, uint M, uint ACC) {
    __shared__ __attribute__((aligned(16))) uchar lds_ml[Q6K_ML_LDS];
    const uint lds_addr = (uint)(size_t)(__attribute__((address_space(3))) uchar*)lds_ml;
    // the deepest ring that fits beside the tokens
    const uint fixed = (M <= 8 ? 8u : 16u) * (K + 32u) + (K >> 2) + 256u;
    if (M <= 8) {
        if (fixed + 8u * 4u * Q6K_ML_UNIT <= Q6K_ML_LDS) gemv_q8k_q6k_ml_body<1, 4>(xq, xs, w, y, K, N, M, ACC, lds_ml, lds_addr);
        else gemv_q8k_q6k_ml_body<1, 3>(xq, xs, w, y, K, N, M, ACC, lds_ml, lds_addr);
    } else {
        if (fixed + 8u * 3u * Q6K_ML_UNIT <= Q6K_ML_LDS) gemv_q8k_q6k_ml_body<2, 3>(xq, xs, w, y, K, N, M, ACC, lds_ml, lds_addr);
        else gemv_q8k_q6k_ml_body<2, 2>(xq, xs, w, y, K, N, M, ACC, lds_ml, lds_addr);
    }
}
