// The lane-level Q4_K x int8 dot shared by the decode matvecs and the MoE expert kernels:
// the arithmetic of the CPU reference's dot_q4k (crates/ojas-cpu/src/cpu_math.rs:609-635) for the
// 32 weights one lane owns.
#pragma once
#include "ojk_common.h"

__device__ __forceinline__ int bytesum4(uint4 v) {
    int s = dot4_i8_first(v.x, 0x01010101u);
    s = dot4_i8(v.y, 0x01010101u, s);
    s = dot4_i8(v.z, 0x01010101u, s);
    return dot4_i8(v.w, 0x01010101u, s);
}

// Eight lanes share a super-block and a wave walks eight super-blocks (2048 weights) per step.
// Lane (g, l) = (lane/8, lane%8) owns the 16 quant bytes l*16..l*16+15 of super-block g: 16
// low-nibble weights of sub-block 2c and 16 high-nibble weights of sub-block 2c+1, c = l/2.  The
// activation fragment (2 x 16 int8, their sums, the segment scale) is loaded once per step and
// reused across the R rows of the wave.
struct Q4kFrag {
    uint4 xl, xh;  // int8 activations for the low / high nibble halves
    int bl, bh;    // their sums (the lane's part of bsums)
    float sx;      // activation scale of the super-block
};

__device__ __forceinline__ Q4kFrag q4k_load_frag(const signed char* xq, const float* xs, uint sb, uint l) {
    Q4kFrag f;
    const signed char* p = xq + (size_t)sb * 256u + (l >> 1) * 64u + (l & 1u) * 16u;
    f.xl = *(const uint4*)p;
    f.xh = *(const uint4*)(p + 32);
    f.bl = bytesum4(f.xl);
    f.bh = bytesum4(f.xh);
    f.sx = xs[sb];
    return f;
}

// The same fragment straight from f32 activations: the eight lanes of a group hold the 256 values
// of super-block `sb` between them, so the segment's quantizer (scale = amax/127, 1 if all zero;
// q = clamp(round_half_away(v * (1/scale))), crates/ojas-cpu/src/cpu_math.rs:539-563) needs one
// maximum over the group and nothing outside registers.  Same operations as the quantize_q8k
// kernel, hence the same bytes.
__device__ __forceinline__ uint q8k_pack4(float4 v, float inv) {
    float a = sat127(roundf(__fmul_rn(v.x, inv)));
    float b = sat127(roundf(__fmul_rn(v.y, inv)));
    float c = sat127(roundf(__fmul_rn(v.z, inv)));
    float d = sat127(roundf(__fmul_rn(v.w, inv)));
    return ((uint)(int)a & 0xFFu) | (((uint)(int)b & 0xFFu) << 8) | (((uint)(int)c & 0xFFu) << 16) | ((uint)(int)d << 24);
}

__device__ __forceinline__ float amax4(float4 v) { return fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))); }

__device__ __forceinline__ Q4kFrag q4k_quant_frag(const float* x, uint sb, uint l) {
    const float4* p = (const float4*)(x + (size_t)sb * 256u + (l >> 1) * 64u + (l & 1u) * 16u);
    float4 lo[4], hi[4];
#pragma unroll
    for (int i = 0; i < 4; i++) { lo[i] = p[i]; hi[i] = p[8 + i]; }
    float a = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; i++) a = fmaxf(a, fmaxf(amax4(lo[i]), amax4(hi[i])));
    a = fmaxf(a, dpp_f32<OJK_DPP_QUAD_XOR1>(a));
    a = fmaxf(a, dpp_f32<OJK_DPP_QUAD_XOR2>(a));
    a = fmaxf(a, dpp_f32<OJK_DPP_ROW_HALF_MIRROR>(a));
    Q4kFrag f;
    f.sx = a > 0.0f ? __fdiv_rn(a, 127.0f) : 1.0f;
    const float inv = __fdiv_rn(1.0f, f.sx);
    f.xl = make_uint4(q8k_pack4(lo[0], inv), q8k_pack4(lo[1], inv), q8k_pack4(lo[2], inv), q8k_pack4(lo[3], inv));
    f.xh = make_uint4(q8k_pack4(hi[0], inv), q8k_pack4(hi[1], inv), q8k_pack4(hi[2], inv), q8k_pack4(hi[3], inv));
    f.bl = bytesum4(f.xl);
    f.bh = bytesum4(f.xh);
    return f;
}

// One lane's 32 weights of one super-block against one activation fragment.
__device__ __forceinline__ float q4k_lane_dot(uint4 hdr, uint4 qs, uint c, const Q4kFrag& f) {
    const uint M4 = 0x0F0F0F0Fu;
    int il = dot4_i8_first(qs.x & M4, f.xl.x);
    il = dot4_i8(qs.y & M4, f.xl.y, il);
    il = dot4_i8(qs.z & M4, f.xl.z, il);
    il = dot4_i8(qs.w & M4, f.xl.w, il);
    int ih = dot4_i8_first((qs.x >> 4) & M4, f.xh.x);
    ih = dot4_i8((qs.y >> 4) & M4, f.xh.y, ih);
    ih = dot4_i8((qs.z >> 4) & M4, f.xh.z, ih);
    ih = dot4_i8((qs.w >> 4) & M4, f.xh.w, ih);
    uint sc, mn;
    q4k_scale_min_pair(hdr.y, hdr.z, hdr.w, c, sc, mn);
    // 24-bit multiplies (full rate; a 32-bit integer multiply is a quarter-rate instruction): the scales are 6 bits,
    // a sum of sixteen nibble x int8 products stays below 2^15, a sum of sixteen int8 below 2^11
    int isum = __mul24((int)(sc & 0xFFu), il) + __mul24((int)(sc >> 8), ih);
    int msum = __mul24((int)(mn & 0xFFu), f.bl) + __mul24((int)(mn >> 8), f.bh);
    float d = f16_bits_to_f32(hdr.x & 0xFFFFu), dmin = f16_bits_to_f32(hdr.x >> 16);
    return f.sx * (d * (float)isum - dmin * (float)msum);
}

// Q5_K: the same 32 weights with their fifth bits.  Bit j of qh[l] belongs to weight l of
// sub-block j (crates/ojas-cpu/src/cpu_math.rs:638-670); `qh` holds the 16 bytes at the positions
// of the lane's 16 quant bytes.
__device__ __forceinline__ float q5k_lane_dot(uint4 hdr, uint4 qs, uint4 qh, uint c, const Q4kFrag& f) {
    const uint M4 = 0x0F0F0F0Fu, B1 = 0x01010101u;
    const uint sl = 2u * c, sh = 2u * c + 1u;
    int il = dot4_i8_first(qs.x & M4, f.xl.x);
    il = dot4_i8(qs.y & M4, f.xl.y, il);
    il = dot4_i8(qs.z & M4, f.xl.z, il);
    il = dot4_i8(qs.w & M4, f.xl.w, il);
    int bl = dot4_i8_first((qh.x >> sl) & B1, f.xl.x);
    bl = dot4_i8((qh.y >> sl) & B1, f.xl.y, bl);
    bl = dot4_i8((qh.z >> sl) & B1, f.xl.z, bl);
    bl = dot4_i8((qh.w >> sl) & B1, f.xl.w, bl);
    int ih = dot4_i8_first((qs.x >> 4) & M4, f.xh.x);
    ih = dot4_i8((qs.y >> 4) & M4, f.xh.y, ih);
    ih = dot4_i8((qs.z >> 4) & M4, f.xh.z, ih);
    ih = dot4_i8((qs.w >> 4) & M4, f.xh.w, ih);
    int bh = dot4_i8_first((qh.x >> sh) & B1, f.xh.x);
    bh = dot4_i8((qh.y >> sh) & B1, f.xh.y, bh);
    bh = dot4_i8((qh.z >> sh) & B1, f.xh.z, bh);
    bh = dot4_i8((qh.w >> sh) & B1, f.xh.w, bh);
    uint sc, mn;
    q4k_scale_min_pair(hdr.y, hdr.z, hdr.w, c, sc, mn);
    const int isum = (int)(sc & 0xFFu) * (il + 16 * bl) + (int)(sc >> 8) * (ih + 16 * bh);
    const int msum = (int)(mn & 0xFFu) * f.bl + (int)(mn >> 8) * f.bh;
    const float d = f16_bits_to_f32(hdr.x & 0xFFFFu), dmin = f16_bits_to_f32(hdr.x >> 16);
    return f.sx * (d * (float)isum - dmin * (float)msum);
}

// A lane's bytes of one super-block of one row, by format: what the MoE kernels are written over.
struct W4k {
    static constexpr uint BYTES = Q4K_BYTES;
    uint4 h, q;
    __device__ __forceinline__ void load(const uchar* blk, uint l) {
        h = *(const uint4*)blk;
        q = *(const uint4*)(blk + 16u + l * 16u);
    }
    __device__ __forceinline__ float dot(uint c, const Q4kFrag& f) const { return q4k_lane_dot(h, q, c, f); }
};
struct W5k {
    static constexpr uint BYTES = Q5K_BYTES;
    uint4 h, q, qh;
    __device__ __forceinline__ void load(const uchar* blk, uint l) {
        h = *(const uint4*)blk;
        qh = *(const uint4*)(blk + 16u + (l & 1u) * 16u);
        q = *(const uint4*)(blk + 48u + l * 16u);
    }
    __device__ __forceinline__ float dot(uint c, const Q4kFrag& f) const { return q5k_lane_dot(h, q, qh, c, f); }
};

// Q6_K on the same lane map (eight lanes per super-block; lane l: 64-weight chunk c = l / 2, run h = l % 2).
// The lane's two runs of 16 activations — positions 64 c + 16 h + i and 32 further on — are quarters
// q = 2 (c % 2) and q + 1 of half c / 2 at in-quarter offset 16 h: ql bytes 64 hf + 16 h + i and 32 further
// on (low nibbles when c is even, high when odd), qh bytes 32 hf + 16 h + i (bit pairs 2 q and 2 q + 2), scales
// 8 hf + 2 q + h and two further on, d at byte 208 (crates/ojas-formats/src/gguf.rs:1086-1108).  The
// arithmetic is dot_q6k's per 16-weight group: sx * d * sum_g scale_g * (sum code x - 32 sum x)
// (crates/ojas-cpu/src/cpu_math.rs:674-722), integer sums exact.
struct W6k {
    static constexpr uint BYTES = Q6K_BYTES;
    u32x4_a2 qa, qb, qh;
    uint sc2, d16;      // the two scales in bytes 0 and 1
    __device__ __forceinline__ void load(const uchar* blk, uint l) {
        const uint c = l >> 1, h = l & 1u, hf = c >> 1, q = 2u * (c & 1u);
        qa = *(const u32x4_a2*)(blk + 64u * hf + 16u * h);
        qb = *(const u32x4_a2*)(blk + 64u * hf + 32u + 16u * h);
        qh = *(const u32x4_a2*)(blk + 128u + 32u * hf + 16u * h);
        const uchar* ps = blk + 192u + 8u * hf + 2u * q + h;
        sc2 = (uint)ps[0] | ((uint)ps[2] << 8);
        d16 = *(const ushort*)(blk + 208u);
    }
    __device__ __forceinline__ float dot(uint c, const Q4kFrag& f) const {
        const uint M4 = 0x0F0F0F0Fu, H2 = 0x30303030u;
        const uint nsh = 4u * (c & 1u);            // nibble of ql; also the bit pair of qh for the first run
        // codes 0..63 as bytes: ql nibble | two bits of qh moved to bits 4-5
        #define OJK_Q6_CODE(QL, QH, SH) ((((QL) >> nsh) & M4) | ((((QH) >> (SH)) << 4) & H2))
        int ia = dot4_i8_first(OJK_Q6_CODE(qa.x, qh.x, nsh), f.xl.x);
        ia = dot4_i8(OJK_Q6_CODE(qa.y, qh.y, nsh), f.xl.y, ia);
        ia = dot4_i8(OJK_Q6_CODE(qa.z, qh.z, nsh), f.xl.z, ia);
        ia = dot4_i8(OJK_Q6_CODE(qa.w, qh.w, nsh), f.xl.w, ia);
        int ib = dot4_i8_first(OJK_Q6_CODE(qb.x, qh.x, nsh + 2u), f.xh.x);
        ib = dot4_i8(OJK_Q6_CODE(qb.y, qh.y, nsh + 2u), f.xh.y, ib);
        ib = dot4_i8(OJK_Q6_CODE(qb.z, qh.z, nsh + 2u), f.xh.z, ib);
        ib = dot4_i8(OJK_Q6_CODE(qb.w, qh.w, nsh + 2u), f.xh.w, ib);
        #undef OJK_Q6_CODE
        const int sa = (int)(signed char)(sc2 & 0xFFu), sb = (int)(signed char)(sc2 >> 8);
        const int isum = sa * (ia - 32 * f.bl) + sb * (ib - 32 * f.bh);
        return f.sx * f16_bits_to_f32(d16) * (float)isum;
    }
};
