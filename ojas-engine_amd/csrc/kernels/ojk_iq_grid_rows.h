// Row traits of the grid-codebook GGUF formats — IQ2_XXS, IQ2_XS, IQ2_S, IQ3_XXS, IQ3_S, IQ1_S, IQ1_M
// (crates/ojas-formats/src/gguf.rs:840-1041) — for the decoders, the matvecs and the expert products.
//
// A 256-weight block is 32 groups of 8 weights; a group is one codebook entry (IQ3: two entries of four) of
// magnitudes, a sign per weight and the scale of its 32- or 16-weight sub-block:
//     w = d * scale * (+-magnitude)            IQ2_*, IQ3_*
//     w = d * (2 s + 1) * (value + delta)      IQ1_*: values -1 / 0 / +1, delta = +-1/8 per group
// One lane owns one group (32 lanes per block, a wave walks two blocks per step).  decode() turns the lane's bytes
// into a fragment { dl, delta, w0, w1 }: the full scale, the offset, and the eight values as signed bytes, ready
// for integer dots against int8 activations or for a conversion each against f32 activations.  Every factor chain
// is exact in f32 (an f16 d, scales below 32 in halves, values below 64): products may be taken in any order and
// the decoders still round once, to f16, like the reference.
//
// Codebooks come packed at 16 bits per entry (ojk_iq_grids.h); an entry's digits become byte selectors of one
// v_perm_b32 over the alphabet.  The 128-entry sign table of IQ2_XXS / IQ2_XS / IQ3_XXS is its closed form: the
// seven stored bits plus the bit that makes their parity even.
#pragma once
#include "ojk_common.h"
#include "ojk_rows.h"
#define OJK_GRID_CONST static __device__ const
#include "ojk_iq_grids.h"

#define IQ2XXS_BYTES 66u
#define IQ2XS_BYTES 74u
#define IQ2S_BYTES 82u
#define IQ3XXS_BYTES 98u
#define IQ3S_BYTES 110u
#define IQ1S_BYTES 50u
#define IQ1M_BYTES 56u

struct IqgFrag { float dl, delta; uint w0, w1; };

__device__ __forceinline__ uint iqg_ksigns(uint i) {
    i &= 127u;
    return i | (((uint)__popc(i) & 1u) << 7);
}
// four 2-bit (3-bit) digits in the low bits of e -> one digit per byte
__device__ __forceinline__ uint iqg_spread2(uint e) { return (e & 3u) | ((e & 0xCu) << 6) | ((e & 0x30u) << 12) | ((e & 0xC0u) << 18); }
__device__ __forceinline__ uint iqg_spread3(uint e) { return (e & 7u) | ((e & 0x38u) << 5) | ((e & 0x1C0u) << 10) | ((e & 0xE00u) << 15); }
// four magnitudes (bytes, 1 .. 62) with the signs of bits 0 .. 3 of sg -> four signed bytes
__device__ __forceinline__ uint iqg_apply_signs(uint m, uint sg) {
    const uint s4 = (sg & 1u) | ((sg & 2u) << 7) | ((sg & 4u) << 14) | ((sg & 8u) << 21);
    return (m ^ (s4 * 0xFFu)) + s4;      // -m = ~m + 1 byte by byte; m > 0, so no byte carries into the next
}
// A workgroup may expand the codebook it needs into LDS once (G::init(), then a barrier) and decode with
// decode<true>: one ds_read per entry instead of a dependent global load and the digit unpacking.  decode<false>
// reads the packed table in global memory — for the decoders, whose workgroups each see eight blocks only.
template <uint N2>
__device__ __forceinline__ uint2* iqg_lds64() { __shared__ uint2 tab[N2]; return tab; }
template <uint N1>
__device__ __forceinline__ uint* iqg_lds32() { __shared__ uint tab[N1]; return tab; }
__device__ __forceinline__ uint2 iqg_iq2_mags(uint e) {
    return make_uint2(__builtin_amdgcn_perm(0u, 0x002B1908u, iqg_spread2(e & 0xFFu)), __builtin_amdgcn_perm(0u, 0x002B1908u, iqg_spread2(e >> 8)));
}
#define IQG_TABLE64(NAME, N, PK, EXPAND)                                                                    \
    static __device__ __forceinline__ uint2* table() { return iqg_lds64<N>(); }                             \
    static __device__ __forceinline__ void init() {                                                         \
        uint2* t = table();                                                                                 \
        for (uint i = threadIdx.x; i < N; i += blockDim.x) t[i] = EXPAND((uint)PK[i]);                      \
    }                                                                                                       \
    template <bool LDS> static __device__ __forceinline__ uint2 entry(uint i) { return LDS ? table()[i] : EXPAND((uint)PK[i]); }
#define IQG_TABLE32(NAME, N, PK, EXPAND)                                                                    \
    static __device__ __forceinline__ uint* table() { return iqg_lds32<N>(); }                              \
    static __device__ __forceinline__ void init() {                                                         \
        uint* t = table();                                                                                  \
        for (uint i = threadIdx.x; i < N; i += blockDim.x) t[i] = EXPAND((uint)PK[i]);                      \
    }                                                                                                       \
    template <bool LDS> static __device__ __forceinline__ uint entry(uint i) { return LDS ? table()[i] : EXPAND((uint)PK[i]); }
__device__ __forceinline__ uint2 iqg_iq1_vals(uint e) {
    return make_uint2(__builtin_amdgcn_perm(0u, 0x000100FFu, iqg_spread2(e & 0xFFu)), __builtin_amdgcn_perm(0u, 0x000100FFu, iqg_spread2(e >> 8)));
}
__device__ __forceinline__ uint iqg_iq3xxs_mags(uint e) { return __builtin_amdgcn_perm(0x3E342C24u, 0x1C140C04u, iqg_spread3(e)); }
__device__ __forceinline__ uint iqg_iq3s_mags(uint e) { return __builtin_amdgcn_perm(0x0F0D0B09u, 0x07050301u, iqg_spread3(e)); }
__device__ __forceinline__ void iqg_signed(uint2 m, uint sg, IqgFrag& f) {
    f.w0 = iqg_apply_signs(m.x, sg & 15u);
    f.w1 = iqg_apply_signs(m.y, sg >> 4);
}
// The 128-entry sign table expanded in LDS: entry i = eight byte masks, 0xFF where weight j of the group is negative
// (bit j of i, and for j = 7 the bit that makes the parity even).  iqg_signs_init(), then a barrier, then
// iqg_masked(m, iqg_sign_masks()[i]) = the magnitudes m with those signs: (m ^ s) - s byte by byte, and since m > 0 no
// byte borrows from the next.
__device__ __forceinline__ uint2* iqg_sign_masks() { __shared__ uint2 tab[128]; return tab; }
__device__ __forceinline__ void iqg_signs_init() {
    uint2* t = iqg_sign_masks();
    for (uint i = threadIdx.x; i < 128u; i += blockDim.x) {
        const uint sg = iqg_ksigns(i), lo = sg & 15u, hi = sg >> 4;
        const uint l4 = (lo & 1u) | ((lo & 2u) << 7) | ((lo & 4u) << 14) | ((lo & 8u) << 21);
        const uint h4 = (hi & 1u) | ((hi & 2u) << 7) | ((hi & 4u) << 14) | ((hi & 8u) << 21);
        t[i] = make_uint2(l4 * 0xFFu, h4 * 0xFFu);
    }
}
__device__ __forceinline__ uint iqg_masked(uint m, uint s) { return (m ^ s) + (s & 0x01010101u); }
// ... and the same for the formats that store a raw sign byte per group (IQ2_S, IQ3_S): 256 entries
__device__ __forceinline__ uint2* iqg_sign_masks256() { __shared__ uint2 tab[256]; return tab; }
__device__ __forceinline__ void iqg_signs256_init() {
    uint2* t = iqg_sign_masks256();
    for (uint i = threadIdx.x; i < 256u; i += blockDim.x) {
        const uint lo = i & 15u, hi = i >> 4;
        const uint l4 = (lo & 1u) | ((lo & 2u) << 7) | ((lo & 4u) << 14) | ((lo & 8u) << 21);
        const uint h4 = (hi & 1u) | ((hi & 2u) << 7) | ((hi & 4u) << 14) | ((hi & 8u) << 21);
        t[i] = make_uint2(l4 * 0xFFu, h4 * 0xFFu);
    }
}

struct Iq2xxsG {   // { f16 d; u16 qs[32] }: per sub-block 4 index bytes, then 4 x 7 sign-table bits + a 4-bit scale
    static constexpr uint BYTES = IQ2XXS_BYTES;
    IQG_TABLE64(iq2xxs, 256u, ojk_iq2xxs_grid_pk, iqg_iq2_mags)
    template <bool LDS = false> static __device__ __forceinline__ IqgFrag decode(const uchar* blk, uint t) {
        const uint ib = t >> 2, l = t & 3u;
        const uint a0 = *(const u32_a2*)(blk + 2u + 8u * ib), a1 = *(const u32_a2*)(blk + 6u + 8u * ib);
        IqgFrag f;
        f.dl = f16_bits_to_f32(*(const ushort*)blk) * (0.5f + (float)(a1 >> 28)) * 0.25f;
        f.delta = 0.0f;
        iqg_signed(entry<LDS>((a0 >> (8u * l)) & 255u), iqg_ksigns(a1 >> (7u * l)), f);
        return f;
    }
    // One lane, one 32-weight sub-block against its 32 int8 activations: d * scale * idot32, the integer dot exact
    // (after init(), iqg_signs_init() and a barrier).
    // One lane, one 32-weight sub-block (after init(), signs_init() and a barrier): its weights as signed bytes, four to
    // a word, and the scale of its first and second sixteen.
    static __device__ __forceinline__ void signs_init() { iqg_signs_init(); }
    static __device__ __forceinline__ void vals32(const uchar* blk, uint ib, uint (&w)[8], float& dl0, float& dl1) {
        const u32x2_a2 a = *(const u32x2_a2*)(blk + 2u + 8u * ib);
        const uint2* sm = iqg_sign_masks();
#pragma unroll
        for (uint l = 0; l < 4u; l++) {
            const uint2 m = table()[(a.x >> (8u * l)) & 255u], s = sm[(a.y >> (7u * l)) & 127u];
            w[2 * l] = iqg_masked(m.x, s.x);
            w[2 * l + 1] = iqg_masked(m.y, s.y);
        }
        dl0 = dl1 = f16_bits_to_f32(*(const ushort*)blk) * ((0.5f + (float)(a.y >> 28)) * 0.25f);
    }
};
struct Iq2xsG {    // { f16 d; u16 qs[32]; u8 scales[8] }: 9 index bits + 7 sign-table bits per group, a scale nibble per 16
    static constexpr uint BYTES = IQ2XS_BYTES;
    IQG_TABLE64(iq2xs, 512u, ojk_iq2xs_grid_pk, iqg_iq2_mags)
    template <bool LDS = false> static __device__ __forceinline__ IqgFrag decode(const uchar* blk, uint t) {
        const uint ib = t >> 2, l = t & 3u;
        const uint q = *(const ushort*)(blk + 2u + 2u * t), sc = blk[66u + ib];
        IqgFrag f;
        f.dl = f16_bits_to_f32(*(const ushort*)blk) * (0.5f + (float)(l < 2u ? sc & 15u : sc >> 4)) * 0.25f;
        f.delta = 0.0f;
        iqg_signed(entry<LDS>(q & 511u), iqg_ksigns(q >> 9), f);
        return f;
    }
};
struct Iq2sG {     // { f16 d; u8 qs[32]; u8 signs[32]; u8 qh[8]; u8 scales[8] }: 10 index bits, a raw sign byte
    static constexpr uint BYTES = IQ2S_BYTES;
    IQG_TABLE64(iq2s, 1024u, ojk_iq2s_grid_pk, iqg_iq2_mags)
    template <bool LDS = false> static __device__ __forceinline__ IqgFrag decode(const uchar* blk, uint t) {
        const uint ib = t >> 2, l = t & 3u;
        const uint idx = (uint)blk[2u + t] | ((((uint)blk[66u + ib]) << (8u - 2u * l)) & 0x300u), sc = blk[74u + ib];
        IqgFrag f;
        f.dl = f16_bits_to_f32(*(const ushort*)blk) * (0.5f + (float)(l < 2u ? sc & 15u : sc >> 4)) * 0.25f;
        f.delta = 0.0f;
        iqg_signed(entry<LDS>(idx), blk[34u + t], f);
        return f;
    }
    static __device__ __forceinline__ void signs_init() { iqg_signs256_init(); }
    static __device__ __forceinline__ void vals32(const uchar* blk, uint ib, uint (&w)[8], float& dl0, float& dl1) {
        const uint lo = *(const u32_a2*)(blk + 2u + 4u * ib), sg = *(const u32_a2*)(blk + 34u + 4u * ib);
        const uint h = blk[66u + ib], sc = blk[74u + ib];
        const uint2* sm = iqg_sign_masks256();
#pragma unroll
        for (uint l = 0; l < 4u; l++) {
            const uint2 m = table()[((lo >> (8u * l)) & 255u) | ((h << (8u - 2u * l)) & 0x300u)], s = sm[(sg >> (8u * l)) & 255u];
            w[2 * l] = iqg_masked(m.x, s.x);
            w[2 * l + 1] = iqg_masked(m.y, s.y);
        }
        const float d = f16_bits_to_f32(*(const ushort*)blk);
        dl0 = d * ((0.5f + (float)(sc & 15u)) * 0.25f);
        dl1 = d * ((0.5f + (float)(sc >> 4)) * 0.25f);
    }
};
struct Iq3xxsG {   // { f16 d; u8 qs[64]; u32 ss[8] }: two 4-weight entries per group; ss as IQ2_XXS's second word
    static constexpr uint BYTES = IQ3XXS_BYTES;
    IQG_TABLE32(iq3xxs, 256u, ojk_iq3xxs_grid_pk, iqg_iq3xxs_mags)
    template <bool LDS = false> static __device__ __forceinline__ IqgFrag decode(const uchar* blk, uint t) {
        const uint ib = t >> 2, l = t & 3u;
        const uint q = *(const ushort*)(blk + 2u + 2u * t), a = *(const u32_a2*)(blk + 66u + 4u * ib);
        const uint sg = iqg_ksigns(a >> (7u * l));
        IqgFrag f;
        f.dl = f16_bits_to_f32(*(const ushort*)blk) * (0.5f + (float)(a >> 28)) * 0.5f;
        f.delta = 0.0f;
        iqg_signed(make_uint2(entry<LDS>(q & 255u), entry<LDS>(q >> 8)), sg, f);
        return f;
    }
    static __device__ __forceinline__ void signs_init() { iqg_signs_init(); }
    static __device__ __forceinline__ void vals32(const uchar* blk, uint ib, uint (&w)[8], float& dl0, float& dl1) {
        const u32x2_a2 ix = *(const u32x2_a2*)(blk + 2u + 8u * ib);
        const uint a = *(const u32_a2*)(blk + 66u + 4u * ib);
        const uint2* sm = iqg_sign_masks();
        const uint* tb = table();
#pragma unroll
        for (uint l = 0; l < 4u; l++) {
            const uint q = l < 2u ? ix.x >> (16u * l) : ix.y >> (16u * (l - 2u));
            const uint2 s = sm[(a >> (7u * l)) & 127u];
            w[2 * l] = iqg_masked(tb[q & 255u], s.x);
            w[2 * l + 1] = iqg_masked(tb[(q >> 8) & 255u], s.y);
        }
        dl0 = dl1 = f16_bits_to_f32(*(const ushort*)blk) * ((0.5f + (float)(a >> 28)) * 0.5f);
    }
};
struct Iq3sG {     // { f16 d; u8 qs[64]; u8 qh[8]; u8 signs[32]; u8 scales[4] }: 9 index bits, raw signs, scale 1 + 2 s
    static constexpr uint BYTES = IQ3S_BYTES;
    IQG_TABLE32(iq3s, 512u, ojk_iq3s_grid_pk, iqg_iq3s_mags)
    template <bool LDS = false> static __device__ __forceinline__ IqgFrag decode(const uchar* blk, uint t) {
        const uint g = t >> 2, l = t & 3u;
        const uint q = *(const ushort*)(blk + 2u + 2u * t), h = blk[66u + g], sg = blk[74u + t];
        const uint s = ((uint)blk[106u + (g >> 1)] >> (4u * (g & 1u))) & 15u;
        const uint i1 = (q & 255u) | ((h << (8u - 2u * l)) & 256u), i2 = (q >> 8) | ((h << (7u - 2u * l)) & 256u);
        IqgFrag f;
        f.dl = f16_bits_to_f32(*(const ushort*)blk) * (1.0f + 2.0f * (float)s);
        f.delta = 0.0f;
        iqg_signed(make_uint2(entry<LDS>(i1), entry<LDS>(i2)), sg, f);
        return f;
    }
    static __device__ __forceinline__ void signs_init() { iqg_signs256_init(); }
    static __device__ __forceinline__ void vals32(const uchar* blk, uint ib, uint (&w)[8], float& dl0, float& dl1) {
        const u32x2_a2 ix = *(const u32x2_a2*)(blk + 2u + 8u * ib);
        const uint sg = *(const u32_a2*)(blk + 74u + 4u * ib), h = blk[66u + ib];
        const uint sc = ((uint)blk[106u + (ib >> 1)] >> (4u * (ib & 1u))) & 15u;
        const uint2* sm = iqg_sign_masks256();
        const uint* tb = table();
#pragma unroll
        for (uint l = 0; l < 4u; l++) {
            const uint q = l < 2u ? ix.x >> (16u * l) : ix.y >> (16u * (l - 2u));
            const uint2 s = sm[(sg >> (8u * l)) & 255u];
            w[2 * l] = iqg_masked(tb[(q & 255u) | ((h << (8u - 2u * l)) & 256u)], s.x);
            w[2 * l + 1] = iqg_masked(tb[((q >> 8) & 255u) | ((h << (7u - 2u * l)) & 256u)], s.y);
        }
        dl0 = dl1 = f16_bits_to_f32(*(const ushort*)blk) * (1.0f + 2.0f * (float)sc);
    }
};
struct Iq1sG {     // { f16 d; u8 qs[32]; u16 qh[8] }: qh = 4 x 3 high index bits, a 3-bit scale, the sign of delta
    static constexpr uint BYTES = IQ1S_BYTES;
    IQG_TABLE64(iq1s, 2048u, ojk_iq1s_grid_pk, iqg_iq1_vals)
    template <bool LDS = false> static __device__ __forceinline__ IqgFrag decode(const uchar* blk, uint t) {
        const uint ib = t >> 2, l = t & 3u;
        const uint qh = *(const ushort*)(blk + 34u + 2u * ib);
        IqgFrag f;
        f.dl = f16_bits_to_f32(*(const ushort*)blk) * (float)(2u * ((qh >> 12) & 7u) + 1u);
        f.delta = qh & 0x8000u ? -0.125f : 0.125f;
        const uint2 v = entry<LDS>((uint)blk[2u + t] | (((qh >> (3u * l)) & 7u) << 8));
        f.w0 = v.x;
        f.w1 = v.y;
        return f;
    }
};
struct Iq1mG {     // { u8 qs[32]; u8 qh[16]; u16 scales[4] }: d in the top nibbles of the scale words, two 3-bit scales per 32
    static constexpr uint BYTES = IQ1M_BYTES;
    IQG_TABLE64(iq1m, 2048u, ojk_iq1s_grid_pk, iqg_iq1_vals)
    template <bool LDS = false> static __device__ __forceinline__ IqgFrag decode(const uchar* blk, uint t) {
        const uint ib = t >> 2, l = t & 3u;
        const u32x2_a2 sc = *(const u32x2_a2*)(blk + 48u);      // scale words 0, 1 | 2, 3
        const uint dbits = ((sc.x >> 12) & 0xFu) | ((sc.x >> 24) & 0xF0u) | ((sc.y >> 4) & 0xF00u) | ((sc.y >> 16) & 0xF000u);
        const uint w = ((ib & 4u ? sc.y : sc.x) >> (8u * (ib & 2u))) & 0xFFFFu;          // scales[ib / 2]
        const uint s = (w >> (6u * (ib & 1u) + 3u * (l >> 1))) & 7u;
        const uint h = blk[32u + 2u * ib + (l >> 1)];
        const uint hi = l & 1u ? (h << 4) & 0x700u : (h << 8) & 0x700u;
        IqgFrag f;
        f.dl = f16_bits_to_f32(dbits) * (float)(2u * s + 1u);
        f.delta = h & (l & 1u ? 0x80u : 0x08u) ? -0.125f : 0.125f;
        const uint2 v = entry<LDS>((uint)blk[t] | hi);
        f.w0 = v.x;
        f.w1 = v.y;
        return f;
    }
};

// The trait the matvec and expert bodies take (their kernels call W::init() and a barrier first): lane -> (block of the step, group of the block); the lane's eight
// activations are two consecutive float4.
template <class G>
struct IqGridW {
    static constexpr uint XGAP = 4u;
    static constexpr uint STEP = 2u;
    static constexpr uint BYTES = G::BYTES;
    static __device__ __forceinline__ uint units(uint K) { return K >> 8; }
    static __device__ __forceinline__ uint unit_of(uint lane) { return lane >> 5; }
    static __device__ __forceinline__ uint x_off(uint lane) { return (lane & 31u) * 8u; }
    static __device__ __forceinline__ uint x_unit(uint) { return 256u; }
    typedef IqgFrag Frag;
    static __device__ __forceinline__ void init() { G::init(); }
    static __device__ __forceinline__ Frag load(const uchar* row, uint u, uint lane) {
        return G::template decode<true>(row + (size_t)u * G::BYTES, lane & 31u);     // after G::init() and a barrier
    }
    static __device__ __forceinline__ float dot(const Frag& f, uint, float4 x0, float4 x1, float xsum) {
        float a = sb0(f.w0) * x0.x;
        a = fmaf(sb1(f.w0), x0.y, a);
        a = fmaf(sb2(f.w0), x0.z, a);
        a = fmaf(sb3(f.w0), x0.w, a);
        a = fmaf(sb0(f.w1), x1.x, a);
        a = fmaf(sb1(f.w1), x1.y, a);
        a = fmaf(sb2(f.w1), x1.z, a);
        a = fmaf(sb3(f.w1), x1.w, a);
        return f.dl * fmaf(f.delta, xsum, a);
    }
};
typedef IqGridW<Iq2xxsG> Iq2xxsW;
typedef IqGridW<Iq2xsG> Iq2xsW;
typedef IqGridW<Iq2sG> Iq2sW;
typedef IqGridW<Iq3xxsG> Iq3xxsW;
typedef IqGridW<Iq3sG> Iq3sW;
typedef IqGridW<Iq1sG> Iq1sW;
typedef IqGridW<Iq1mG> Iq1mW;
