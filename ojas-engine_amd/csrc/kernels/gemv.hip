// Family "gemv": fused-dequant matvecs on raw GGUF blocks with f32 activations — the contract
// of the reference's GPU kernels gemv_nat_<fmt>{,_accum,_bias,_m}
// (crates/ojas-cuda/src/kernels/nat.rs:69-89; bodies crates/ojas-core/src/quant_src.rs:779-824
// Q4_K, :833-867 Q6_K, :1028-1057 Q8_0, :1154-1180 batched).  IQ4_NL and IQ4_XS rows ride the same
// entries; their arithmetic is the CPU path's dot_iq4nl / dot_iq4xs, which also reads f32 activations
// (crates/ojas-cpu/src/cpu_math.rs:993-1010, :943-967).
//
//   gemv_nat_<fmt>{,_accum}(x, w, y, K, N)        y[n] (=,+=) sum_k W[n,k] x[k]
//   gemv_nat_<fmt>_bias(x, w, y, bs, K, N)        y[n] = ... + bs[n]
//   gemv_nat_<fmt>_m(x, w, y, K, N, M, ACC)       x[M][K], y[M][N]
//
// wave64 plan, common to the three formats: a group of lanes shares one block, a wave walks
// several blocks per step, the activation fragment of a step is loaded once and reused across
// the R rows of the wave.  Scales stay factored: the lane accumulates sum(code * x) per sub-block
// and applies d*sc (and -dmin*m*sum(x) for Q4_K) once per sub-block.
#include "ojk_common.h"
#include "ojk_rows.h"
#include "ojk_rowdot.h"

// ------------------------------------------------------------------ Q4_K
// Lane (g, l) = (lane/8, lane%8): 16 quant bytes l*16.. of super-block g -> 16 weights of
// sub-block 2c (low nibbles) and 16 of sub-block 2c+1 (high nibbles), c = l/2.
struct Q4kFragF {
    float4 xl[4], xh[4];
    float sl, sh;  // sums of the two 16-float halves (for the -dmin*m term)
};

__device__ __forceinline__ Q4kFragF q4k_load_frag_f(const float* x, uint sb, uint l) {
    Q4kFragF f;
    const float4* p = (const float4*)(x + (size_t)sb * 256u + (l >> 1) * 64u + (l & 1u) * 16u);
    float sl = 0.0f, sh = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        f.xl[i] = p[i];
        f.xh[i] = p[8 + i];
        sl += sum4(f.xl[i]);
        sh += sum4(f.xh[i]);
    }
    f.sl = sl;
    f.sh = sh;
    return f;
}

__device__ __forceinline__ float q4k_lane_dot_f(uint4 hdr, uint4 qs, uint c, const Q4kFragF& f) {
    const uint M4 = 0x0F0F0F0Fu;
    float al = dot4_ub(qs.x & M4, f.xl[0], 0.0f);
    al = dot4_ub(qs.y & M4, f.xl[1], al);
    al = dot4_ub(qs.z & M4, f.xl[2], al);
    al = dot4_ub(qs.w & M4, f.xl[3], al);
    float ah = dot4_ub((qs.x >> 4) & M4, f.xh[0], 0.0f);
    ah = dot4_ub((qs.y >> 4) & M4, f.xh[1], ah);
    ah = dot4_ub((qs.z >> 4) & M4, f.xh[2], ah);
    ah = dot4_ub((qs.w >> 4) & M4, f.xh[3], ah);
    uint sc, mn;
    q4k_scale_min_pair(hdr.y, hdr.z, hdr.w, c, sc, mn);
    float d = f16_bits_to_f32(hdr.x & 0xFFFFu), dmin = f16_bits_to_f32(hdr.x >> 16);
    float pos = (float)(sc & 0xFFu) * al + (float)(sc >> 8) * ah;
    float neg = (float)(mn & 0xFFu) * f.sl + (float)(mn >> 8) * f.sh;
    return d * pos - dmin * neg;
}

template <int R, int MODE>
__device__ __forceinline__ void gemv_nat_q4k_rows(const float* __restrict__ x, const uchar* __restrict__ w,
                                                  float* __restrict__ y, const float* __restrict__ bs,
                                                  uint K, uint N, uint row0) {
    const uint lane = threadIdx.x & 63u;
    const uint nsb = K >> 8, g = lane >> 3, l = lane & 7u, c = l >> 1;
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = 0.0f;
    for (uint sb = g; sb < nsb; sb += 8u) {
        uint4 hdr[R], qs[R];
#pragma unroll
        for (int r = 0; r < R; r++) {
            uint row = min(row0 + r, N - 1u);
            const uchar* blk = w + ((size_t)row * nsb + sb) * Q4K_BYTES;
            hdr[r] = *(const uint4*)blk;
            qs[r] = *(const uint4*)(blk + 16u + l * 16u);
        }
        Q4kFragF f = q4k_load_frag_f(x, sb, l);
#pragma unroll
        for (int r = 0; r < R; r++) acc[r] += q4k_lane_dot_f(hdr[r], qs[r], c, f);
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
        float t = wave_sum(acc[r]);
        if (lane == 0 && row0 + r < N) store_row<MODE>(y, bs, row0 + r, t);
    }
}

template <int R, int MODE>
__device__ __forceinline__ void gemv_nat_q4k_body(const float* __restrict__ x, const uchar* __restrict__ w,
                                                  float* __restrict__ y, const float* __restrict__ bs,
                                                  uint K, uint N) {
    const uint row0 = (blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)) * R;
    if (row0 < N) gemv_nat_q4k_rows<R, MODE>(x, w, y, bs, K, N, row0);
}

template <int MT>
__device__ __forceinline__ void gemv_nat_q4k_m_body(const float* __restrict__ x, const uchar* __restrict__ w,
                                                    float* __restrict__ y, uint K, uint N, uint M, uint ACC) {
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
                Q4kFragF f = q4k_load_frag_f(x + (size_t)m * K, sb, l);
                acc[t] += q4k_lane_dot_f(hdr, qs, c, f);
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

// Many rows (an output head, K <= 4096): rows grid-stride, two per wave and step, and the wave's share of
// the f32 activations — two fragments of 32 floats and their sums per lane — stays in registers for the
// whole launch.  With a fragment fetched per row group the launch is bound by those fetches (eight
// 16-byte loads per lane against two for the weights), not by HBM.  Same lane arithmetic and order
// as the entries above: the same bits.   gemv_nat_q4k_px(x, w, y, K, N)
__device__ __forceinline__ void gemv_nat_q4k_px_body(const float* __restrict__ x, const uchar* __restrict__ w,
                                                     float* __restrict__ y, uint K, uint N) {
    const uint lane = threadIdx.x & 63u;
    const uint nsb = K >> 8, g = lane >> 3, l = lane & 7u, c = l >> 1;
    Q4kFragF f[2];
    uint sbc[2];
#pragma unroll
    for (int s = 0; s < 2; s++) {
        const uint sb = g + 8u * (uint)s;
        sbc[s] = min(sb, nsb - 1u);
        f[s] = q4k_load_frag_f(x, sbc[s], l);
        if (sb >= nsb) {                              // a step past K: zeros, so that its repeated block adds nothing
#pragma unroll
            for (int i = 0; i < 4; i++) f[s].xl[i] = f[s].xh[i] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            f[s].sl = f[s].sh = 0.0f;
        }
    }
    const uint nwaves = gridDim.x * (blockDim.x >> 6);
    for (uint row0 = (blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)) * 2u; row0 < N; row0 += nwaves * 2u) {
        const uchar* r0 = w + (size_t)row0 * nsb * Q4K_BYTES;
        const uchar* r1 = w + (size_t)min(row0 + 1u, N - 1u) * nsb * Q4K_BYTES;
        float a0 = 0.0f, a1 = 0.0f;
#pragma unroll
        for (int s = 0; s < 2; s++) {
            const uchar* b0 = r0 + (size_t)sbc[s] * Q4K_BYTES;
            const uchar* b1 = r1 + (size_t)sbc[s] * Q4K_BYTES;
            const uint4 h0 = *(const uint4*)b0, q0 = *(const uint4*)(b0 + 16u + l * 16u);
            const uint4 h1 = *(const uint4*)b1, q1 = *(const uint4*)(b1 + 16u + l * 16u);
            a0 += q4k_lane_dot_f(h0, q0, c, f[s]);
            a1 += q4k_lane_dot_f(h1, q1, c, f[s]);
        }
        a0 = wave_sum(a0);
        a1 = wave_sum(a1);
        if (lane == 0) {
            y[row0] = a0;
            if (row0 + 1u < N) y[row0 + 1u] = a1;
        }
    }
}
extern "C" __global__ void __launch_bounds__(256)
gemv_nat_q4k_px(const float* x, const uchar* w, float* y, uint K, uint N) { gemv_nat_q4k_px_body(x, w, y, K, N); }

// ------------------------------------------------------------------ Q6_K
// Lane (g, t) = (lane/16, lane%16): half hf = t/8, weights l0..l0+3 (l0 = 4*(t%8)) of each of the
// four quarters of that half; one int8 sub-scale per quarter.
struct Q6kFragF {
    float4 x[4];
    float s[4];
};

__device__ __forceinline__ Q6kFragF q6k_load_frag_f(const float* x, uint sb, uint hf, uint l0) {
    Q6kFragF f;
    const float* p = x + (size_t)sb * 256u + hf * 128u + l0;
#pragma unroll
    for (int q = 0; q < 4; q++) {
        f.x[q] = *(const float4*)(p + 32 * q);
        f.s[q] = sum4(f.x[q]);
    }
    return f;
}

struct Q6kRaw {
    uint qa, qb, qh, sc4, d16;
};

__device__ __forceinline__ Q6kRaw q6k_load_raw(const uchar* blk, uint hf, uint l0) {
    Q6kRaw r;
    r.qa = *(const u32_a2*)(blk + hf * 64u + l0);
    r.qb = *(const u32_a2*)(blk + hf * 64u + 32u + l0);
    r.qh = *(const u32_a2*)(blk + 128u + hf * 32u + l0);
    u32x2_a2 s = *(const u32x2_a2*)(blk + 192u + hf * 8u);
    uint is = l0 >> 4;
    uint a = s.x >> (8u * is), b = s.y >> (8u * is);
    r.sc4 = (a & 0xFFu) | ((a >> 8) & 0xFF00u) | ((b & 0xFFu) << 16) | ((b << 8) & 0xFF000000u);
    r.d16 = *(const ushort*)(blk + 208u);
    return r;
}

__device__ __forceinline__ float q6k_lane_dot_f(const Q6kRaw& r, const Q6kFragF& f) {
    const uint M4 = 0x0F0F0F0Fu, H2 = 0x30303030u;
    uint w0 = (r.qa & M4) | ((r.qh << 4) & H2);
    uint w1 = (r.qb & M4) | ((r.qh << 2) & H2);
    uint w2 = ((r.qa >> 4) & M4) | (r.qh & H2);
    uint w3 = ((r.qb >> 4) & M4) | ((r.qh >> 2) & H2);
    // sum((code - 32) * x) = sum(code * x) - 32 * sum(x)
    float t0 = dot4_ub(w0, f.x[0], -32.0f * f.s[0]);
    float t1 = dot4_ub(w1, f.x[1], -32.0f * f.s[1]);
    float t2 = dot4_ub(w2, f.x[2], -32.0f * f.s[2]);
    float t3 = dot4_ub(w3, f.x[3], -32.0f * f.s[3]);
    float s0 = (float)(signed char)(r.sc4), s1 = (float)(signed char)(r.sc4 >> 8);
    float s2 = (float)(signed char)(r.sc4 >> 16), s3 = (float)((int)r.sc4 >> 24);
    return f16_bits_to_f32(r.d16) * ((s0 * t0 + s1 * t1) + (s2 * t2 + s3 * t3));
}

template <int R, int MODE>
__device__ __forceinline__ void gemv_nat_q6k_rows(const float* __restrict__ x, const uchar* __restrict__ w,
                                                  float* __restrict__ y, const float* __restrict__ bs,
                                                  uint K, uint N, uint row0) {
    const uint lane = threadIdx.x & 63u;
    const uint nsb = K >> 8, g = lane >> 4, t = lane & 15u, hf = t >> 3, l0 = (t & 7u) * 4u;
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = 0.0f;
    for (uint sb = g; sb < nsb; sb += 4u) {
        Q6kRaw raw[R];
#pragma unroll
        for (int r = 0; r < R; r++) {
            uint row = min(row0 + r, N - 1u);
            raw[r] = q6k_load_raw(w + ((size_t)row * nsb + sb) * Q6K_BYTES, hf, l0);
        }
        Q6kFragF f = q6k_load_frag_f(x, sb, hf, l0);
#pragma unroll
        for (int r = 0; r < R; r++) acc[r] += q6k_lane_dot_f(raw[r], f);
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
        float s = wave_sum(acc[r]);
        if (lane == 0 && row0 + r < N) store_row<MODE>(y, bs, row0 + r, s);
    }
}

template <int R, int MODE>
__device__ __forceinline__ void gemv_nat_q6k_body(const float* __restrict__ x, const uchar* __restrict__ w,
                                                  float* __restrict__ y, const float* __restrict__ bs,
                                                  uint K, uint N) {
    const uint row0 = (blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)) * R;
    if (row0 < N) gemv_nat_q6k_rows<R, MODE>(x, w, y, bs, K, N, row0);
}

template <int MT>
__device__ __forceinline__ void gemv_nat_q6k_m_body(const float* __restrict__ x, const uchar* __restrict__ w,
                                                    float* __restrict__ y, uint K, uint N, uint M, uint ACC) {
    const uint lane = threadIdx.x & 63u;
    const uint row = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (row >= N) return;
    const uint nsb = K >> 8, g = lane >> 4, t = lane & 15u, hf = t >> 3, l0 = (t & 7u) * 4u;
    for (uint m0 = 0; m0 < M; m0 += MT) {
        float acc[MT];
#pragma unroll
        for (int i = 0; i < MT; i++) acc[i] = 0.0f;
        for (uint sb = g; sb < nsb; sb += 4u) {
            Q6kRaw raw = q6k_load_raw(w + ((size_t)row * nsb + sb) * Q6K_BYTES, hf, l0);
#pragma unroll
            for (int i = 0; i < MT; i++) {
                uint m = min(m0 + i, M - 1u);
                Q6kFragF f = q6k_load_frag_f(x + (size_t)m * K, sb, hf, l0);
                acc[i] += q6k_lane_dot_f(raw, f);
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

// The same for Q6_K rows: four fragments of 16 floats and their sums per lane (K <= 4096).
//   gemv_nat_q6k_px(x, w, y, K, N)
__device__ __forceinline__ void gemv_nat_q6k_px_body(const float* __restrict__ x, const uchar* __restrict__ w,
                                                     float* __restrict__ y, uint K, uint N) {
    const uint lane = threadIdx.x & 63u;
    const uint nsb = K >> 8, g = lane >> 4, t = lane & 15u, hf = t >> 3, l0 = (t & 7u) * 4u;
    Q6kFragF f[4];
    uint sbc[4];
#pragma unroll
    for (int s = 0; s < 4; s++) {
        const uint sb = g + 4u * (uint)s;
        sbc[s] = min(sb, nsb - 1u);
        f[s] = q6k_load_frag_f(x, sbc[s], hf, l0);
        if (sb >= nsb) {
#pragma unroll
            for (int q = 0; q < 4; q++) {
                f[s].x[q] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                f[s].s[q] = 0.0f;
            }
        }
    }
    const uint nwaves = gridDim.x * (blockDim.x >> 6);
    for (uint row0 = (blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)) * 2u; row0 < N; row0 += nwaves * 2u) {
        const uchar* r0 = w + (size_t)row0 * nsb * Q6K_BYTES;
        const uchar* r1 = w + (size_t)min(row0 + 1u, N - 1u) * nsb * Q6K_BYTES;
        float a0 = 0.0f, a1 = 0.0f;
#pragma unroll
        for (int s = 0; s < 4; s++) {
            const Q6kRaw w0 = q6k_load_raw(r0 + (size_t)sbc[s] * Q6K_BYTES, hf, l0);
            const Q6kRaw w1 = q6k_load_raw(r1 + (size_t)sbc[s] * Q6K_BYTES, hf, l0);
            a0 += q6k_lane_dot_f(w0, f[s]);
            a1 += q6k_lane_dot_f(w1, f[s]);
        }
        a0 = wave_sum(a0);
        a1 = wave_sum(a1);
        if (lane == 0) {
            y[row0] = a0;
            if (row0 + 1u < N) y[row0 + 1u] = a1;
        }
    }
}
extern "C" __global__ void __launch_bounds__(256)
gemv_nat_q6k_px(const float* x, const uchar* w, float* y, uint K, uint N) { gemv_nat_q6k_px_body(x, w, y, K, N); }

// ------------------------------------------------------------------ Q8_0
// Four lanes share a 34-byte block (8 int8 each); a wave walks 16 blocks (512 weights) per step.
__device__ __forceinline__ float q80_lane_dot(uint d16, u32x2_a2 q, float4 x0, float4 x1) {
    float a = sb0(q.x) * x0.x;
    a = fmaf(sb1(q.x), x0.y, a);
    a = fmaf(sb2(q.x), x0.z, a);
    a = fmaf(sb3(q.x), x0.w, a);
    a = fmaf(sb0(q.y), x1.x, a);
    a = fmaf(sb1(q.y), x1.y, a);
    a = fmaf(sb2(q.y), x1.z, a);
    a = fmaf(sb3(q.y), x1.w, a);
    return f16_bits_to_f32(d16) * a;
}

template <int R, int MODE>
__device__ __forceinline__ void gemv_nat_q80_body(const float* __restrict__ x, const uchar* __restrict__ w,
                                                  float* __restrict__ y, const float* __restrict__ bs,
                                                  uint K, uint N) {
    const uint lane = threadIdx.x & 63u;
    const uint row0 = (blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)) * R;
    if (row0 >= N) return;
    const uint nb = K >> 5, g = lane >> 2, p = lane & 3u;
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = 0.0f;
    for (uint b = g; b < nb; b += 16u) {
        uint d16[R];
        u32x2_a2 q[R];
#pragma unroll
        for (int r = 0; r < R; r++) {
            uint row = min(row0 + r, N - 1u);
            const uchar* blk = w + ((size_t)row * nb + b) * Q80_BYTES;
            d16[r] = *(const ushort*)blk;
            q[r] = *(const u32x2_a2*)(blk + 2u + p * 8u);
        }
        const float4* xp = (const float4*)(x + (size_t)b * 32u + p * 8u);
        float4 x0 = xp[0], x1 = xp[1];
#pragma unroll
        for (int r = 0; r < R; r++) acc[r] += q80_lane_dot(d16[r], q[r], x0, x1);
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
        float s = wave_sum(acc[r]);
        if (lane == 0 && row0 + r < N) store_row<MODE>(y, bs, row0 + r, s);
    }
}

template <int MT>
__device__ __forceinline__ void gemv_nat_q80_m_body(const float* __restrict__ x, const uchar* __restrict__ w,
                                                    float* __restrict__ y, uint K, uint N, uint M, uint ACC) {
    const uint lane = threadIdx.x & 63u;
    const uint row = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (row >= N) return;
    const uint nb = K >> 5, g = lane >> 2, p = lane & 3u;
    for (uint m0 = 0; m0 < M; m0 += MT) {
        float acc[MT];
#pragma unroll
        for (int i = 0; i < MT; i++) acc[i] = 0.0f;
        for (uint b = g; b < nb; b += 16u) {
            const uchar* blk = w + ((size_t)row * nb + b) * Q80_BYTES;
            uint d16 = *(const ushort*)blk;
            u32x2_a2 q = *(const u32x2_a2*)(blk + 2u + p * 8u);
#pragma unroll
            for (int i = 0; i < MT; i++) {
                uint m = min(m0 + i, M - 1u);
                const float4* xp = (const float4*)(x + (size_t)m * K + (size_t)b * 32u + p * 8u);
                acc[i] += q80_lane_dot(d16, q, xp[0], xp[1]);
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

// ------------------------------------------------------------------ IQ4_NL, IQ4_XS and the legacy 32-weight blocks
// (row traits Iq4nlW, Iq4xsW, Q40W, Q41W, Q50W, Q51W, Mxfp4W: ojk_rows.h)
GEMV_NAT_SUB32_PX(iq4nl, Iq4nlS32)
GEMV_NAT_SUB32_PX(iq4xs, Iq4xsS32)
typedef LegacyS32<false, false> Q40S32;
typedef LegacyS32<false, true> Q41S32;
typedef LegacyS32<true, false> Q50S32;
typedef LegacyS32<true, true> Q51S32;
GEMV_NAT_SUB32_PX(q40, Q40S32)
GEMV_NAT_SUB32_PX(q41, Q41S32)
GEMV_NAT_SUB32_PX(q50, Q50S32)
GEMV_NAT_SUB32_PX(q51, Q51S32)
GEMV_NAT_IQ4_PX(mxfp4, Mxfp4W)
GEMV_NAT_IQ4_PX(q5k, Q5kW)

template <int R, int MODE>
__device__ __forceinline__ void gemv_nat_q5k_body(const float* x, const uchar* w, float* y, const float* bs, uint K, uint N) {
    gemv_nat_iq4_body<Q5kW, R, MODE>(x, w, y, bs, K, N);
}
template <int MT>
__device__ __forceinline__ void gemv_nat_q5k_m_body(const float* x, const uchar* w, float* y, uint K, uint N, uint M, uint ACC) {
    gemv_nat_iq4_m_body<Q5kW, MT>(x, w, y, K, N, M, ACC);
}
template <int R, int MODE>
__device__ __forceinline__ void gemv_nat_q40_body(const float* x, const uchar* w, float* y, const float* bs, uint K, uint N) {
    gemv_nat_iq4_body<Q40W, R, MODE>(x, w, y, bs, K, N);
}
template <int MT>
__device__ __forceinline__ void gemv_nat_q40_m_body(const float* x, const uchar* w, float* y, uint K, uint N, uint M, uint ACC) {
    gemv_nat_iq4_m_body<Q40W, MT>(x, w, y, K, N, M, ACC);
}
template <int R, int MODE>
__device__ __forceinline__ void gemv_nat_q41_body(const float* x, const uchar* w, float* y, const float* bs, uint K, uint N) {
    gemv_nat_iq4_body<Q41W, R, MODE>(x, w, y, bs, K, N);
}
template <int MT>
__device__ __forceinline__ void gemv_nat_q41_m_body(const float* x, const uchar* w, float* y, uint K, uint N, uint M, uint ACC) {
    gemv_nat_iq4_m_body<Q41W, MT>(x, w, y, K, N, M, ACC);
}
template <int R, int MODE>
__device__ __forceinline__ void gemv_nat_q50_body(const float* x, const uchar* w, float* y, const float* bs, uint K, uint N) {
    gemv_nat_iq4_body<Q50W, R, MODE>(x, w, y, bs, K, N);
}
template <int MT>
__device__ __forceinline__ void gemv_nat_q50_m_body(const float* x, const uchar* w, float* y, uint K, uint N, uint M, uint ACC) {
    gemv_nat_iq4_m_body<Q50W, MT>(x, w, y, K, N, M, ACC);
}
template <int R, int MODE>
__device__ __forceinline__ void gemv_nat_mxfp4_body(const float* x, const uchar* w, float* y, const float* bs, uint K, uint N) {
    gemv_nat_iq4_body<Mxfp4W, R, MODE>(x, w, y, bs, K, N);
}
template <int MT>
__device__ __forceinline__ void gemv_nat_mxfp4_m_body(const float* x, const uchar* w, float* y, uint K, uint N, uint M, uint ACC) {
    gemv_nat_iq4_m_body<Mxfp4W, MT>(x, w, y, K, N, M, ACC);
}
template <int R, int MODE>
__device__ __forceinline__ void gemv_nat_q51_body(const float* x, const uchar* w, float* y, const float* bs, uint K, uint N) {
    gemv_nat_iq4_body<Q51W, R, MODE>(x, w, y, bs, K, N);
}
template <int MT>
__device__ __forceinline__ void gemv_nat_q51_m_body(const float* x, const uchar* w, float* y, uint K, uint N, uint M, uint ACC) {
    gemv_nat_iq4_m_body<Q51W, MT>(x, w, y, K, N, M, ACC);
}
template <int R, int MODE>
__device__ __forceinline__ void gemv_nat_iq4nl_body(const float* x, const uchar* w, float* y, const float* bs, uint K, uint N) {
    gemv_nat_iq4_body<Iq4nlW, R, MODE>(x, w, y, bs, K, N);
}
template <int MT>
__device__ __forceinline__ void gemv_nat_iq4nl_m_body(const float* x, const uchar* w, float* y, uint K, uint N, uint M, uint ACC) {
    gemv_nat_iq4_m_body<Iq4nlW, MT>(x, w, y, K, N, M, ACC);
}
template <int R, int MODE>
__device__ __forceinline__ void gemv_nat_iq4xs_body(const float* x, const uchar* w, float* y, const float* bs, uint K, uint N) {
    gemv_nat_iq4_body<Iq4xsW, R, MODE>(x, w, y, bs, K, N);
}
template <int MT>
__device__ __forceinline__ void gemv_nat_iq4xs_m_body(const float* x, const uchar* w, float* y, uint K, uint N, uint M, uint ACC) {
    gemv_nat_iq4_m_body<Iq4xsW, MT>(x, w, y, K, N, M, ACC);
}

// ------------------------------------------------------------------ Q8_0, rows staged through LDS
//   gemv_nat_q80_lds{,_accum}(x, w, y, K, N, KC)   gemv_nat_q80_lds_bias(x, w, y, bs, K, N, KC)
// 34-byte blocks defeat wide per-lane loads, and f32 activations are four bytes per weight byte
// if they come through the cache every time.  Here a wave keeps its activations in registers
// for the whole launch and has its rows copied into LDS by the memory system itself:
//   * K is cut into KC (1, 2 or 4) chunks of CB = K / 32 / KC <= 128 blocks; wave w of the
//     workgroup owns chunk w % KC of row slot w / KC (4 / KC rows per workgroup step);
//   * lane l holds the 64 activations of blocks 2l and 2l + 1 of its chunk (lanes past CB / 2 idle);
//   * a row's chunk (CB * 34 bytes, a multiple of 16) goes global -> LDS with
//     global_load_lds_dwordx4, 1 KB per instruction and perfectly coalesced, the next row in
//     flight while one is consumed (deeper queues and more resident waves measured slower);
//   * the lane reads its 68 bytes back as 17 dwords (stride 17 banks: conflict-free) and runs
//     dot_q80's arithmetic: per block sum_j (float)q_j x_j, times d, added up
//     (crates/ojas-cpu/src/cpu_math.rs:971-981);
//   * chunks of a row meet in LDS and are added in chunk order.
// Rows are grid-stride; every wave of a workgroup runs the same number of steps (surplus rows are
// clamped and not stored), so the workgroup barriers line up.
#define Q80L_CHUNK 4352u   // 128 blocks
#define Q80L_DEPTH 2u

__device__ __forceinline__ float q80l_dot4(uint v, float a, float x0, float x1, float x2, float x3) {
    a = fmaf(sb0(v), x0, a);
    a = fmaf(sb1(v), x1, a);
    a = fmaf(sb2(v), x2, a);
    return fmaf(sb3(v), x3, a);
}

template <int MODE>
__device__ __forceinline__ void gemv_nat_q80_lds_body(const float* __restrict__ x, const uchar* __restrict__ w,
                                                      float* __restrict__ y, const float* __restrict__ bs,
                                                      uint K, uint N, uint KC) {
    __shared__ __attribute__((aligned(16))) uchar stage[4u * Q80L_DEPTH * Q80L_CHUNK];
    __shared__ float part[2][4];
    const uint lane = threadIdx.x & 63u;
    const uint wave = (uint)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const uint nb = K >> 5, CB = nb / KC, chunk = wave % KC, slot = wave / KC, RPB = 4u / KC;
    const uint chunk_bytes = CB * Q80_BYTES, n16 = chunk_bytes >> 4, NI = (n16 + 63u) >> 6;
    const size_t row_bytes = (size_t)nb * Q80_BYTES;
    const bool on = 2u * lane < CB;
    const uint lds0 = (uint)(size_t)(__attribute__((address_space(3))) uchar*)stage + wave * (Q80L_DEPTH * Q80L_CHUNK);
    const uchar* mine = stage + wave * (Q80L_DEPTH * Q80L_CHUNK) + lane * 68u;
    const uint steps = (N + RPB - 1u) / RPB;                        // workgroup steps in the launch
    const uint my_steps = blockIdx.x < steps ? (steps - blockIdx.x + gridDim.x - 1u) / gridDim.x : 0u;
    // row of step k: (blockIdx.x + k * gridDim.x) * RPB + slot, clamped
    auto issue = [&](uint k) {
        const uint row = min((blockIdx.x + k * gridDim.x) * RPB + slot, N - 1u);
        const uchar* base = w + (size_t)row * row_bytes + (size_t)chunk * chunk_bytes;
        const uint dst = lds0 + (k % Q80L_DEPTH) * Q80L_CHUNK;
        for (uint i = 0; i < NI; i++)
            if (i * 64u + lane < n16) lds_dma16(base, (i * 64u + lane) << 4, dst + i * 1024u);
    };
    // the wave's activations: blocks 2l, 2l+1 of its chunk
    float xr[64];
    {
        const float4* xp = (const float4*)(x + ((size_t)chunk * CB + (on ? 2u * lane : 0u)) * 32u);
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const float4 v = xp[i];
            xr[4 * i] = v.x; xr[4 * i + 1] = v.y; xr[4 * i + 2] = v.z; xr[4 * i + 3] = v.w;
        }
    }
    // the activation loads above are older than every row copy, so counting copies alone is safe
    for (uint k = 0; k + 1u < Q80L_DEPTH; k++)
        if (k < my_steps) issue(k);
    for (uint k = 0; k < my_steps; k++) {
        if (k + Q80L_DEPTH - 1u < my_steps) issue(k + Q80L_DEPTH - 1u);
        vm_wait(min(my_steps - 1u - k, Q80L_DEPTH - 1u) * NI);
        const uint* p = (const uint*)(mine + (k % Q80L_DEPTH) * Q80L_CHUNK);
        uint d[17];
#pragma unroll
        for (int i = 0; i < 17; i++) d[i] = p[i];
        // block 2l: scale in the low half of dword 0, quants at bytes 2 .. 33
        float s0 = fmaf(sb2(d[0]), xr[0], 0.0f);
        s0 = fmaf(sb3(d[0]), xr[1], s0);
#pragma unroll
        for (int j = 1; j < 8; j++) s0 = q80l_dot4(d[j], s0, xr[4 * j - 2], xr[4 * j - 1], xr[4 * j], xr[4 * j + 1]);
        s0 = fmaf(sb0(d[8]), xr[30], s0);
        s0 = fmaf(sb1(d[8]), xr[31], s0);
        // block 2l+1: scale in the high half of dword 8, quants in dwords 9 .. 16
        float s1 = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; j++) s1 = q80l_dot4(d[9 + j], s1, xr[32 + 4 * j], xr[33 + 4 * j], xr[34 + 4 * j], xr[35 + 4 * j]);
        float v = on ? f16_bits_to_f32(d[0] & 0xFFFFu) * s0 + f16_bits_to_f32(d[8] >> 16) * s1 : 0.0f;
        v = wave_sum(v);
        const uint row = (blockIdx.x + k * gridDim.x) * RPB + slot;
        if (KC == 1u) {
            if (lane == 0 && row < N) store_row<MODE>(y, bs, row, v);
        } else {
            if (lane == 0) part[k & 1u][wave] = v;
            __syncthreads();
            if (lane == 0 && chunk == 0u && row < N) {
                float t = part[k & 1u][wave];
                for (uint c = 1; c < KC; c++) t += part[k & 1u][wave + c];
                store_row<MODE>(y, bs, row, t);
            }
        }
    }
}

extern "C" __global__ void __launch_bounds__(256)
gemv_nat_q80_lds(const float* x, const uchar* w, float* y, uint K, uint N, uint KC) {
    gemv_nat_q80_lds_body<ST_SET>(x, w, y, nullptr, K, N, KC);
}
extern "C" __global__ void __launch_bounds__(256)
gemv_nat_q80_lds_accum(const float* x, const uchar* w, float* y, uint K, uint N, uint KC) {
    gemv_nat_q80_lds_body<ST_ACCUM>(x, w, y, nullptr, K, N, KC);
}
extern "C" __global__ void __launch_bounds__(256)
gemv_nat_q80_lds_bias(const float* x, const uchar* w, float* y, const float* bs, uint K, uint N, uint KC) {
    gemv_nat_q80_lds_body<ST_BIAS>(x, w, y, bs, K, N, KC);
}

// ------------------------------------------------------------------ entries
// ------------------------------------------------------------------ Q2_K and Q3_K rows, f32 activations
// Both keep four 2-bit planes per byte: within a half of 128 weights, byte l of the half's 32 code bytes
// holds weights l, l + 32, l + 64, l + 96 at bits 0, 2, 4, 6, and scale 8 half + 2 j + l / 16 covers
// (plane j, l / 16).  Sixteen lanes share a super-block: lane c takes dword c of the 64 code bytes — half
// c / 8, bytes 4 (c % 8) .. + 3 — so its 16 weights meet four float4 of x 32 floats apart, and a wave walks
// four super-blocks per step.  Codes stay unsigned bytes (v_cvt_f32_ubyteN); what is subtracted meets the
// sum of each plane's four activations:
//   Q2_K  d * sum_j sc_j (q_j . x_j)  -  dmin * sum_j m_j sum(x_j)
//   Q3_K  d * sum_j (sc_j - 32) ((q_j | bit << 2) . x_j  -  4 sum(x_j))      (mask bit set = no subtraction)
// The reference has these two on its GPU path and in dequant_to_f16 only
// (crates/ojas-core/src/quant_src.rs:97-98, :357-420; crates/ojas-formats/src/gguf.rs:730-795).
struct Q2kW {
    static constexpr uint BYTES = Q2K_BYTES;
    struct Frag { uint q, s0, s1, dd; };
    static __device__ __forceinline__ Frag load(const uchar* row, uint u, uint lane) {
        const uint* blk = (const uint*)(row + (size_t)u * Q2K_BYTES);
        const uint c = lane & 15u;
        Frag f;
        f.s0 = blk[(c >> 3) * 2u];
        f.s1 = blk[(c >> 3) * 2u + 1u];
        f.q = blk[4u + c];
        f.dd = blk[20];
        return f;
    }
    static __device__ __forceinline__ float dot(const Frag& f, uint lane, const float4 (&xv)[4], const float (&xs)[4]) {
        const uint sh = (lane & 4u) << 1;     // bytes 4 (c % 8) .. from 16 on: the second scale of each plane
        float ad = 0.0f, am = 0.0f;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint sc = ((j < 2 ? f.s0 : f.s1) >> (16u * (j & 1) + sh)) & 0xFFu;
            ad = fmaf((float)(sc & 0xFu), dot4_ub((f.q >> (2 * j)) & 0x03030303u, xv[j], 0.0f), ad);
            am = fmaf((float)(sc >> 4), xs[j], am);
        }
        return f16_bits_to_f32(f.dd & 0xFFFFu) * ad - f16_bits_to_f32(f.dd >> 16) * am;
    }
};

struct Q3kW {
    static constexpr uint BYTES = Q3K_BYTES;
    struct Frag { uint q, h, r0, r1, r2, d16; };
    static __device__ __forceinline__ Frag load(const uchar* row, uint u, uint lane) {
        const uchar* blk = row + (size_t)u * Q3K_BYTES;     // 110 bytes: two-byte alignment only
        const uint c = lane & 15u;
        Frag f;
        f.h = *(const u32_a2*)(blk + (c & 7u) * 4u);
        f.q = *(const u32_a2*)(blk + 32u + c * 4u);
        f.r0 = *(const u32_a2*)(blk + 96);
        f.r1 = *(const u32_a2*)(blk + 100);
        f.r2 = *(const u32_a2*)(blk + 104);
        f.d16 = *(const ushort*)(blk + 108);
        return f;
    }
    static __device__ __forceinline__ float dot(const Frag& f, uint lane, const float4 (&xv)[4], const float (&xs)[4]) {
        const uint c = lane & 15u, half = c >> 3, part = (c >> 2) & 1u;
        float a = 0.0f;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint code = ((f.q >> (2 * j)) & 0x03030303u) | (((f.h >> (half * 4u + j)) & 0x01010101u) << 2);
            const int sc = q3k_scale6(f.r0, f.r1, f.r2, half * 8u + 2u * j + part);
            a = fmaf((float)sc, dot4_ub(code, xv[j], 0.0f) - 4.0f * xs[j], a);
        }
        return f16_bits_to_f32(f.d16) * a;
    }
};

// the lane's four activation fragments of super-block u
__device__ __forceinline__ void kq2_x(const float* __restrict__ x, uint u, uint lane, float4 (&xv)[4], float (&xs)[4]) {
    const uint c = lane & 15u;
    const float* xp = x + (size_t)u * 256u + (c >> 3) * 128u + (c & 7u) * 4u;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        xv[j] = *(const float4*)(xp + 32 * j);
        xs[j] = sum4(xv[j]);
    }
}

template <class W, int R, int MODE>
__device__ __forceinline__ void gemv_nat_kq2_body(const float* __restrict__ x, const uchar* __restrict__ w,
                                                  float* __restrict__ y, const float* __restrict__ bs,
                                                  uint K, uint N) {
    const uint lane = threadIdx.x & 63u;
    const uint row0 = (blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)) * R;
    if (row0 >= N) return;
    const uint nu = K >> 8;
    const size_t rb = (size_t)nu * W::BYTES;
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = 0.0f;
    for (uint u = lane >> 4; u < nu; u += 4u) {
        typename W::Frag f[R];
#pragma unroll
        for (int r = 0; r < R; r++) f[r] = W::load(w + (size_t)min(row0 + r, N - 1u) * rb, u, lane);
        float4 xv[4];
        float xs[4];
        kq2_x(x, u, lane, xv, xs);
#pragma unroll
        for (int r = 0; r < R; r++) acc[r] += W::dot(f[r], lane, xv, xs);
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
        float s = wave_sum(acc[r]);
        if (lane == 0 && row0 + r < N) store_row<MODE>(y, bs, row0 + r, s);
    }
}

template <class W, int MT>
__device__ __forceinline__ void gemv_nat_kq2_m_body(const float* __restrict__ x, const uchar* __restrict__ w,
                                                    float* __restrict__ y, uint K, uint N, uint M, uint ACC) {
    const uint lane = threadIdx.x & 63u;
    const uint row = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (row >= N) return;
    const uint nu = K >> 8;
    const uchar* wr = w + (size_t)row * nu * W::BYTES;
    for (uint m0 = 0; m0 < M; m0 += MT) {
        float acc[MT];
#pragma unroll
        for (int i = 0; i < MT; i++) acc[i] = 0.0f;
        for (uint u = lane >> 4; u < nu; u += 4u) {
            const typename W::Frag f = W::load(wr, u, lane);
#pragma unroll
            for (int i = 0; i < MT; i++) {
                float4 xv[4];
                float xs[4];
                kq2_x(x + (size_t)min(m0 + i, M - 1u) * K, u, lane, xv, xs);
                acc[i] += W::dot(f, lane, xv, xs);
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

// Many rows, K <= 4096: rows grid-stride, the lane's share of x (four steps of 16 floats) in registers;
// steps past the row hold zeros and repeat its last super-block.
template <class W>
__device__ __forceinline__ void gemv_nat_kq2_px_body(const float* __restrict__ x, const uchar* __restrict__ w,
                                                     float* __restrict__ y, uint K, uint N) {
    const uint lane = threadIdx.x & 63u;
    const uint nu = K >> 8;
    const size_t rb = (size_t)nu * W::BYTES;
    float4 xr[4][4];
    float xs[4][4];
    uint uc[4];
#pragma unroll
    for (int s = 0; s < 4; s++) {
        const uint u = (lane >> 4) + 4u * (uint)s;
        uc[s] = min(u, nu - 1u);
        if (u < nu) {
            kq2_x(x, u, lane, xr[s], xs[s]);
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                xr[s][j] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                xs[s][j] = 0.0f;
            }
        }
    }
    const uint nwaves = gridDim.x * (blockDim.x >> 6);
    for (uint row0 = (blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)) * 2u; row0 < N; row0 += nwaves * 2u) {
        const uchar* r0 = w + (size_t)row0 * rb;
        const uchar* r1 = w + (size_t)min(row0 + 1u, N - 1u) * rb;
        float a0 = 0.0f, a1 = 0.0f;
#pragma unroll
        for (int s = 0; s < 4; s++) {
            const typename W::Frag f0 = W::load(r0, uc[s], lane), f1 = W::load(r1, uc[s], lane);
            a0 += W::dot(f0, lane, xr[s], xs[s]);
            a1 += W::dot(f1, lane, xr[s], xs[s]);
        }
        a0 = wave_sum(a0);
        a1 = wave_sum(a1);
        if (lane == 0) {
            y[row0] = a0;
            if (row0 + 1u < N) y[row0 + 1u] = a1;
        }
    }
}

#define GEMV_NAT_KQ2(FMT, W)                                                                                \
    template <int R, int MODE>                                                                              \
    __device__ __forceinline__ void gemv_nat_##FMT##_body(const float* x, const uchar* w, float* y,         \
                                                          const float* bs, uint K, uint N) {                \
        gemv_nat_kq2_body<W, R, MODE>(x, w, y, bs, K, N); }                                                 \
    template <int MT>                                                                                       \
    __device__ __forceinline__ void gemv_nat_##FMT##_m_body(const float* x, const uchar* w, float* y,       \
                                                            uint K, uint N, uint M, uint ACC) {             \
        gemv_nat_kq2_m_body<W, MT>(x, w, y, K, N, M, ACC); }                                                \
    extern "C" __global__ void __launch_bounds__(256) gemv_nat_##FMT##_px(                                  \
        const float* x, const uchar* w, float* y, uint K, uint N) {                                         \
        gemv_nat_kq2_px_body<W>(x, w, y, K, N); }
GEMV_NAT_KQ2(q2k, Q2kW)
GEMV_NAT_KQ2(q3k, Q3kW)

GEMV_NAT_ENTRIES(q80)
GEMV_NAT_ENTRIES(q4k)
GEMV_NAT_ENTRIES(q6k)
GEMV_NAT_ENTRIES(iq4nl)
GEMV_NAT_ENTRIES(iq4xs)
GEMV_NAT_ENTRIES(q40)
GEMV_NAT_ENTRIES(q41)
GEMV_NAT_ENTRIES(q50)
GEMV_NAT_ENTRIES(q51)
GEMV_NAT_ENTRIES(mxfp4)
GEMV_NAT_ENTRIES(q2k)
GEMV_NAT_ENTRIES(q3k)
GEMV_NAT_ENTRIES(q5k)
