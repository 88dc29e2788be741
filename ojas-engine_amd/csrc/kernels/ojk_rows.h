// Row traits of the formats whose 32-weight groups keep weights 0..15 in the low nibbles of 16 bytes and
// weights 16..31 in the high nibbles (IQ4_NL, IQ4_XS, Q4_0, Q4_1, Q5_0, Q5_1), for kernels that multiply raw
// rows with f32 activations: the dense matvecs and the expert products share them.
// A trait W gives the lane map of one wave step — units(K) blocks in a row, STEP of them per step, lane ->
// unit_of(lane), the lane's two float4 of x at x_unit * u + x_off(lane) and XGAP floats further on — and
// load / dot for the lane's fragment of a block.
#pragma once
#include "ojk_common.h"

__device__ __forceinline__ float ub0(uint v) { return (float)(v & 0xFFu); }
__device__ __forceinline__ float ub1(uint v) { return (float)((v >> 8) & 0xFFu); }
__device__ __forceinline__ float ub2(uint v) { return (float)((v >> 16) & 0xFFu); }
__device__ __forceinline__ float ub3(uint v) { return (float)(v >> 24); }

// sum of 4 unsigned bytes of `w` times 4 floats
__device__ __forceinline__ float dot4_ub(uint w, float4 x, float acc) {
    acc = fmaf(ub0(w), x.x, acc);
    acc = fmaf(ub1(w), x.y, acc);
    acc = fmaf(ub2(w), x.z, acc);
    return fmaf(ub3(w), x.w, acc);
}
__device__ __forceinline__ float sum4(float4 v) { return (v.x + v.y) + (v.z + v.w); }

__device__ __forceinline__ float sb0(uint v) { return (float)(signed char)(v); }
__device__ __forceinline__ float sb1(uint v) { return (float)(signed char)(v >> 8); }
__device__ __forceinline__ float sb2(uint v) { return (float)(signed char)(v >> 16); }
__device__ __forceinline__ float sb3(uint v) { return (float)((int)v >> 24); }

// ------------------------------------------------------------------ IQ4_NL, IQ4_XS
// Both store 4-bit indices into the sixteen-level codebook; within a 32-weight group the low
// nibbles of its 16 bytes are weights 0..15 and the high nibbles weights 16..31.  A lane takes one
// dword of indices: four low-nibble weights and the four 16 further on, against two float4 of x.
// IQ4_NL: 18-byte blocks {f16 d; qs[16]}, four lanes per block, a wave walks 16 blocks per step.
// IQ4_XS: 136-byte super-blocks {f16 d; u16 scales_h; u8 scales_l[4]; qs[128]}, 32 lanes per
// super-block (lane / 4 = sub-block, its 6-bit scale minus 32 times d applied per lane).
__device__ __forceinline__ float iq4_lane_dot(uint q, float4 x0, float4 x1) {
    const uint lo = iq4_levels4(q & 0x0F0F0F0Fu), hi = iq4_levels4((q >> 4) & 0x0F0F0F0Fu);
    float a = sb0(lo) * x0.x;
    a = fmaf(sb0(hi), x1.x, a);
    a = fmaf(sb1(lo), x0.y, a);
    a = fmaf(sb1(hi), x1.y, a);
    a = fmaf(sb2(lo), x0.z, a);
    a = fmaf(sb2(hi), x1.z, a);
    a = fmaf(sb3(lo), x0.w, a);
    return fmaf(sb3(hi), x1.w, a);
}

struct Iq4nlW {
    static constexpr uint XGAP = 16u;            // floats between the lane's two x fragments
    static constexpr uint STEP = 16u;            // blocks a wave walks per step
    static constexpr uint BYTES = IQ4NL_BYTES;
    static __device__ __forceinline__ uint units(uint K) { return K >> 5; }
    // lane -> (block of the step, float offset of its first x fragment inside the block)
    static __device__ __forceinline__ uint unit_of(uint lane) { return lane >> 2; }
    static __device__ __forceinline__ uint x_off(uint lane) { return (lane & 3u) * 4u; }
    static __device__ __forceinline__ uint x_unit(uint) { return 32u; }
    struct Frag { uint d16, q; };
    static __device__ __forceinline__ Frag load(const uchar* row, uint u, uint lane) {
        const uchar* blk = row + (size_t)u * IQ4NL_BYTES;
        Frag f;
        f.d16 = *(const ushort*)blk;
        f.q = *(const u32_a2*)(blk + 2u + (lane & 3u) * 4u);
        return f;
    }
    static __device__ __forceinline__ float dot(const Frag& f, uint, float4 x0, float4 x1, float) {
        return f16_bits_to_f32(f.d16) * iq4_lane_dot(f.q, x0, x1);
    }
};

// ... and a lane per 32-weight group, for the head form (gemv_nat_sub32_px_body): the group's 16 code bytes in one load.
struct __attribute__((packed, aligned(4))) u32x4_a4 { uint x, y, z, w; };
__device__ __forceinline__ float iq4_dot32(uint q0, uint q1, uint q2, uint q3, const float4 (&x)[8]) {
    const uint q[4] = {q0, q1, q2, q3};
    float a = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint lo = iq4_levels4(q[i] & 0x0F0F0F0Fu), hi = iq4_levels4((q[i] >> 4) & 0x0F0F0F0Fu);
        a = fmaf(sb0(lo), x[i].x, a);
        a = fmaf(sb1(lo), x[i].y, a);
        a = fmaf(sb2(lo), x[i].z, a);
        a = fmaf(sb3(lo), x[i].w, a);
        a = fmaf(sb0(hi), x[4 + i].x, a);
        a = fmaf(sb1(hi), x[4 + i].y, a);
        a = fmaf(sb2(hi), x[4 + i].z, a);
        a = fmaf(sb3(hi), x[4 + i].w, a);
    }
    return a;
}
struct Iq4nlS32 {
    static __device__ __forceinline__ size_t row_bytes(uint K) { return (size_t)(K >> 5) * IQ4NL_BYTES; }
    static __device__ __forceinline__ float dot32(const uchar* row, uint sub, const float4 (&x)[8], float) {
        const uchar* blk = row + (size_t)sub * IQ4NL_BYTES;
        const u32x4_a2 q = *(const u32x4_a2*)(blk + 2u);
        return f16_bits_to_f32(*(const ushort*)blk) * iq4_dot32(q.x, q.y, q.z, q.w, x);
    }
};
struct Iq4xsS32 {
    static __device__ __forceinline__ size_t row_bytes(uint K) { return (size_t)(K >> 8) * IQ4XS_BYTES; }
    static __device__ __forceinline__ float dot32(const uchar* row, uint sub, const float4 (&x)[8], float) {
        const uchar* blk = row + (size_t)(sub >> 3) * IQ4XS_BYTES;
        const uint ib = sub & 7u;
        const uint2 h = *(const uint2*)blk;
        const u32x4_a4 q = *(const u32x4_a4*)(blk + 8u + 16u * ib);
        const uint ls = ((h.y >> (4u * ib)) & 0xFu) | ((((h.x >> 16) >> (2u * ib)) & 3u) << 4);
        return f16_bits_to_f32(h.x & 0xFFFFu) * (float)((int)ls - 32) * iq4_dot32(q.x, q.y, q.z, q.w, x);
    }
};

struct Iq4xsW {
    static constexpr uint XGAP = 16u;
    static constexpr uint STEP = 2u;             // super-blocks per step
    static constexpr uint BYTES = IQ4XS_BYTES;
    static __device__ __forceinline__ uint units(uint K) { return K >> 8; }
    static __device__ __forceinline__ uint unit_of(uint lane) { return lane >> 5; }
    static __device__ __forceinline__ uint x_off(uint lane) { return ((lane & 31u) >> 2) * 32u + (lane & 3u) * 4u; }
    static __device__ __forceinline__ uint x_unit(uint) { return 256u; }
    struct Frag { uint h0, sl, q; };
    static __device__ __forceinline__ Frag load(const uchar* row, uint u, uint lane) {
        const uint* blk = (const uint*)(row + (size_t)u * IQ4XS_BYTES);
        Frag f;
        f.h0 = blk[0];
        f.sl = blk[1];
        f.q = blk[2u + (lane & 31u)];
        return f;
    }
    static __device__ __forceinline__ float dot(const Frag& f, uint lane, float4 x0, float4 x1, float) {
        const uint ib = (lane & 31u) >> 2;
        const uint ls = ((f.sl >> (4u * ib)) & 0xFu) | ((((f.h0 >> 16) >> (2u * ib)) & 3u) << 4);
        return f16_bits_to_f32(f.h0 & 0xFFFFu) * (float)((int)ls - 32) * iq4_lane_dot(f.q, x0, x1);
    }
};

// The legacy 32-weight blocks Q4_0 / Q4_1 / Q5_0 / Q5_1 share IQ4_NL's layout — a header, then 16 bytes whose
// low nibbles are weights 0..15 and high nibbles 16..31 — with a linear code instead of the table:
// w = d (q - 8), d q + m, d (q5 - 16), d q5 + m, the fifth bit of weight j being bit j of a 4-byte field.
// Four lanes per block; codes stay unsigned (v_cvt_f32_ubyteN) and the offset or minimum meets the sum of the
// lane's eight activations once per block:  d * (sum q x - off * sum x)  or  d * sum q x + m * sum x.
template <bool FIVE, bool AFFINE>
struct LegacyW {
    static constexpr uint XGAP = 16u;
    static constexpr uint STEP = 16u;
    static constexpr uint BYTES = 18u + (AFFINE ? 2u : 0u) + (FIVE ? 4u : 0u);
    static constexpr uint HDR = AFFINE ? 4u : 2u;
    static __device__ __forceinline__ uint units(uint K) { return K >> 5; }
    static __device__ __forceinline__ uint unit_of(uint lane) { return lane >> 2; }
    static __device__ __forceinline__ uint x_off(uint lane) { return (lane & 3u) * 4u; }
    static __device__ __forceinline__ uint x_unit(uint) { return 32u; }
    struct Frag { uint hdr, q, qh; };
    static __device__ __forceinline__ Frag load(const uchar* row, uint u, uint lane) {
        const uchar* blk = row + (size_t)u * BYTES;
        Frag f;
        f.hdr = AFFINE ? *(const u32_a2*)blk : (uint)*(const ushort*)blk;
        f.qh = FIVE ? *(const u32_a2*)(blk + HDR) : 0u;
        f.q = *(const u32_a2*)(blk + HDR + (FIVE ? 4u : 0u) + (lane & 3u) * 4u);
        return f;
    }
    // bits b .. b + 3 of `v` -> bit 4 of bytes 0 .. 3
    static __device__ __forceinline__ uint spread4(uint v, uint b) {
        const uint n = (v >> b) & 0xFu;
        return ((n & 1u) << 4) | ((n & 2u) << 11) | ((n & 4u) << 18) | ((n & 8u) << 25);
    }
    static __device__ __forceinline__ float dot(const Frag& f, uint lane, float4 x0, float4 x1, float xsum) {
        uint lo = f.q & 0x0F0F0F0Fu, hi = (f.q >> 4) & 0x0F0F0F0Fu;
        if (FIVE) {
            const uint p4 = (lane & 3u) * 4u;
            lo |= spread4(f.qh, p4);
            hi |= spread4(f.qh, p4 + 16u);
        }
        const float a = dot4_ub(hi, x1, dot4_ub(lo, x0, 0.0f));
        const float d = f16_bits_to_f32(f.hdr & 0xFFFFu);
        if (AFFINE) return d * a + f16_bits_to_f32(f.hdr >> 16) * xsum;
        return d * (a - (FIVE ? 16.0f : 8.0f) * xsum);
    }
};
// ... a lane per block, for the head form
template <bool FIVE, bool AFFINE>
struct LegacyS32 {
    typedef LegacyW<FIVE, AFFINE> W;
    static __device__ __forceinline__ size_t row_bytes(uint K) { return (size_t)(K >> 5) * W::BYTES; }
    static __device__ __forceinline__ float dot32(const uchar* row, uint sub, const float4 (&x)[8], float xsum) {
        const uchar* blk = row + (size_t)sub * W::BYTES;
        const uint hdr = AFFINE ? *(const u32_a2*)blk : (uint)*(const ushort*)blk;
        const uint qh = FIVE ? *(const u32_a2*)(blk + W::HDR) : 0u;
        const u32x4_a2 qq = *(const u32x4_a2*)(blk + W::HDR + (FIVE ? 4u : 0u));
        const uint q[4] = {qq.x, qq.y, qq.z, qq.w};
        float a = 0.0f;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            uint lo = q[i] & 0x0F0F0F0Fu, hi = (q[i] >> 4) & 0x0F0F0F0Fu;
            if (FIVE) {
                lo |= W::spread4(qh, 4u * (uint)i);
                hi |= W::spread4(qh, 4u * (uint)i + 16u);
            }
            a = dot4_ub(hi, x[4 + i], dot4_ub(lo, x[i], a));
        }
        const float d = f16_bits_to_f32(hdr & 0xFFFFu);
        if (AFFINE) return d * a + f16_bits_to_f32(hdr >> 16) * xsum;
        return d * (a - (FIVE ? 16.0f : 8.0f) * xsum);
    }
};
typedef LegacyW<false, false> Q40W;
typedef LegacyW<false, true> Q41W;
typedef LegacyW<true, false> Q50W;
typedef LegacyW<true, true> Q51W;


// Q5_K on f32 activations (the reference's native matvec for the format, crates/ojas-core/src/quant_src.rs:100):
// a 176-byte super-block {f16 d, dmin; 12 scale bytes; qh[32]; qs[128]}.  Within chunk c of 64 weights the low
// nibbles of qs[32c .. 32c+31] are sub-block 2c and the high nibbles sub-block 2c+1, so a dword of qs meets two
// float4 of x 32 floats apart; the fifth bit of weight l of sub-block s is bit s of qh[l].  32 lanes per
// super-block, w = d sc q - dmin m (crates/ojas-formats/src/gguf.rs:1060-1085).
struct Q5kW {
    static constexpr uint XGAP = 32u;
    static constexpr uint STEP = 2u;
    static constexpr uint BYTES = Q5K_BYTES;
    static __device__ __forceinline__ uint units(uint K) { return K >> 8; }
    static __device__ __forceinline__ uint unit_of(uint lane) { return lane >> 5; }
    static __device__ __forceinline__ uint x_off(uint lane) { return ((lane & 31u) >> 3) * 64u + (lane & 7u) * 4u; }
    static __device__ __forceinline__ uint x_unit(uint) { return 256u; }
    struct Frag { uint hdr, s0, s1, s2, h, q; };
    static __device__ __forceinline__ Frag load(const uchar* row, uint u, uint lane) {
        const uint* blk = (const uint*)(row + (size_t)u * Q5K_BYTES);
        Frag f;
        f.hdr = blk[0];
        f.s0 = blk[1];
        f.s1 = blk[2];
        f.s2 = blk[3];
        f.h = blk[4u + (lane & 7u)];
        f.q = blk[12u + (lane & 31u)];
        return f;
    }
    static __device__ __forceinline__ float dot(const Frag& f, uint lane, float4 x0, float4 x1, float) {
        const uint c = (lane & 31u) >> 3;
        uint sc, mn;
        q4k_scale_min_pair(f.s0, f.s1, f.s2, c, sc, mn);
        const uint lo = (f.q & 0x0F0F0F0Fu) | (((f.h >> (2u * c)) & 0x01010101u) << 4);
        const uint hi = ((f.q >> 4) & 0x0F0F0F0Fu) | (((f.h >> (2u * c + 1u)) & 0x01010101u) << 4);
        const float a = (float)(sc & 0xFFu) * dot4_ub(lo, x0, 0.0f) + (float)(sc >> 8) * dot4_ub(hi, x1, 0.0f);
        const float b = (float)(mn & 0xFFu) * sum4(x0) + (float)(mn >> 8) * sum4(x1);
        return f16_bits_to_f32(f.hdr & 0xFFFFu) * a - f16_bits_to_f32(f.hdr >> 16) * b;
    }
};

// Q4_K on f32 activations with the same lane map (the reference's `moe_gu_q4k` multiplies the raw rows with f32
// activations, crates/ojas-metal/src/kernels/moe.rs:497-527): 144-byte super-blocks {f16 d, dmin; 12 scale bytes;
// qs[128]}, 32 lanes per super-block, a dword of qs against two float4 of x 32 floats apart.
struct Q4kW {
    static constexpr uint XGAP = 32u;
    static constexpr uint STEP = 2u;
    static constexpr uint BYTES = Q4K_BYTES;
    static __device__ __forceinline__ uint units(uint K) { return K >> 8; }
    static __device__ __forceinline__ uint unit_of(uint lane) { return lane >> 5; }
    static __device__ __forceinline__ uint x_off(uint lane) { return ((lane & 31u) >> 3) * 64u + (lane & 7u) * 4u; }
    static __device__ __forceinline__ uint x_unit(uint) { return 256u; }
    struct Frag { uint hdr, s0, s1, s2, q; };
    static __device__ __forceinline__ Frag load(const uchar* row, uint u, uint lane) {
        const uint* blk = (const uint*)(row + (size_t)u * Q4K_BYTES);
        Frag f;
        f.hdr = blk[0];
        f.s0 = blk[1];
        f.s1 = blk[2];
        f.s2 = blk[3];
        f.q = blk[4u + (lane & 31u)];
        return f;
    }
    static __device__ __forceinline__ float dot(const Frag& f, uint lane, float4 x0, float4 x1, float) {
        const uint c = (lane & 31u) >> 3;
        uint sc, mn;
        q4k_scale_min_pair(f.s0, f.s1, f.s2, c, sc, mn);
        const float a = (float)(sc & 0xFFu) * dot4_ub(f.q & 0x0F0F0F0Fu, x0, 0.0f) + (float)(sc >> 8) * dot4_ub((f.q >> 4) & 0x0F0F0F0Fu, x1, 0.0f);
        const float b = (float)(mn & 0xFFu) * sum4(x0) + (float)(mn >> 8) * sum4(x1);
        return f16_bits_to_f32(f.hdr & 0xFFFFu) * a - f16_bits_to_f32(f.hdr >> 16) * b;
    }
};

// Q6_K on f32 activations (the reference's `moe_down_q6k`, crates/ojas-metal/src/kernels/moe.rs:768-815): 210-byte
// super-blocks {ql[128]; qh[64]; i8 scales[16]; f16 d}, only 2-byte aligned.  Per half of 128 weights the low nibbles
// of its 64 ql bytes are weights 0..63 and the high nibbles weights 64..127, so a dword of ql meets two float4 of x
// 64 floats apart; qh byte l % 32 of the half carries the upper two bits of weights l, l+32, l+64, l+96 (bit pairs
// 0..3); one int8 scale per 16 weights; w = d * sc * (code - 32) (crates/ojas-formats/src/gguf.rs:1086-1108).
struct Q6kW {
    static constexpr uint XGAP = 64u;
    static constexpr uint STEP = 2u;
    static constexpr uint BYTES = Q6K_BYTES;
    static __device__ __forceinline__ uint units(uint K) { return K >> 8; }
    static __device__ __forceinline__ uint unit_of(uint lane) { return lane >> 5; }
    static __device__ __forceinline__ uint x_off(uint lane) { return ((lane & 31u) >> 4) * 128u + (lane & 15u) * 4u; }
    static __device__ __forceinline__ uint x_unit(uint) { return 256u; }
    struct Frag { uint ql, qh, sa, sb, d; };
    static __device__ __forceinline__ Frag load(const uchar* row, uint u, uint lane) {
        typedef uint __attribute__((aligned(2))) uint_u;
        const uchar* blk = row + (size_t)u * Q6K_BYTES;
        const uint hf = (lane & 31u) >> 4, i = lane & 15u;
        const uint quarter = i >> 3, grp = (i & 7u) >> 2;   // low-nibble weights: quarter 0 or 1; 16-weight group within it
        Frag f;
        f.ql = *(const uint_u*)(blk + hf * 64u + i * 4u);
        f.qh = *(const uint_u*)(blk + 128u + hf * 32u + (i & 7u) * 4u) >> (2u * quarter);
        f.sa = blk[192u + hf * 8u + 2u * quarter + grp];
        f.sb = blk[192u + hf * 8u + 2u * (quarter + 2u) + grp];
        f.d = *(const ushort*)(blk + 208u);
        return f;
    }
    static __device__ __forceinline__ float dot(const Frag& f, uint, float4 x0, float4 x1, float) {
        const uint lo = (f.ql & 0x0F0F0F0Fu) | ((f.qh << 4) & 0x30303030u);        // bit pair `quarter`
        const uint hi = ((f.ql >> 4) & 0x0F0F0F0Fu) | (f.qh & 0x30303030u);        // bit pair `quarter + 2`
        const float a = (float)(signed char)f.sa * (dot4_ub(lo, x0, 0.0f) - 32.0f * sum4(x0));
        const float b = (float)(signed char)f.sb * (dot4_ub(hi, x1, 0.0f) - 32.0f * sum4(x1));
        return f16_bits_to_f32(f.d) * (a + b);
    }
};

// ------------------------------------------------------------------ MXFP4
// The reference's native MXFP4 block (crates/ojas-core/src/quant_src.rs:333-353): { u8 e; u8 qs[16] }, 17 bytes per 32
// weights, w = 2^(e - 127) * E2M1[code], weight 2j the low and 2j + 1 the high nibble of qs[j].  Four lanes per
// block: a lane's dword of codes is eight consecutive weights.  The E2M1 magnitudes are halves of {0, 1, 2, 3, 4, 6,
// 8, 12} — one byte permute — and a code's bit 3 is the sign; the scale, a power of two, meets the lane's sum once.
// Blocks sit at odd addresses: every load is byte-aligned.
struct Mxfp4W {
    static constexpr uint XGAP = 4u;
    static constexpr uint STEP = 16u;
    static constexpr uint BYTES = MXFP4_BYTES;
    static __device__ __forceinline__ uint units(uint K) { return K >> 5; }
    static __device__ __forceinline__ uint unit_of(uint lane) { return lane >> 2; }
    static __device__ __forceinline__ uint x_off(uint lane) { return (lane & 3u) * 8u; }
    static __device__ __forceinline__ uint x_unit(uint) { return 32u; }
    struct Frag { uint e, q; };
    static __device__ __forceinline__ Frag load(const uchar* row, uint u, uint lane) {
        const uchar* blk = row + (size_t)u * MXFP4_BYTES;
        Frag f;
        f.e = blk[0];
        f.q = *(const u32_a1*)(blk + 1u + (lane & 3u) * 4u);
        return f;
    }
    // twice the magnitudes of four codes (one per byte, bits 0 .. 2), and the codes' sign bits moved to bit 31
    static __device__ __forceinline__ uint mags4(uint n) { return __builtin_amdgcn_perm(0x0C080604u, 0x03020100u, n & 0x07070707u); }
    static __device__ __forceinline__ float val(uint m, uint n, uint byte) {
        const float a = (float)((m >> (8u * byte)) & 0xFFu);
        return __uint_as_float(__float_as_uint(a) | (((n >> (8u * byte + 3u)) & 1u) << 31));
    }
    static __device__ __forceinline__ float dot(const Frag& f, uint, float4 x0, float4 x1, float) {
        const uint lo = f.q & 0x0F0F0F0Fu, hi = (f.q >> 4) & 0x0F0F0F0Fu;      // weights 0, 2, 4, 6 and 1, 3, 5, 7 of the eight
        const uint ml = mags4(lo), mh = mags4(hi);
        float a = val(ml, lo, 0) * x0.x;
        a = fmaf(val(mh, hi, 0), x0.y, a);
        a = fmaf(val(ml, lo, 1), x0.z, a);
        a = fmaf(val(mh, hi, 1), x0.w, a);
        a = fmaf(val(ml, lo, 2), x1.x, a);
        a = fmaf(val(mh, hi, 2), x1.y, a);
        a = fmaf(val(ml, lo, 3), x1.z, a);
        a = fmaf(val(mh, hi, 3), x1.w, a);
        return __uint_as_float(f.e << 23) * (0.5f * a);
    }
};
