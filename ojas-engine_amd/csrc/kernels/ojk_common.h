// Device-side helpers shared by every gfx950 kernel family: block-format constants,
// f16 / bf16 bit conversions, wave64 reductions on DPP, 2-byte-aligned vector loads.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

typedef unsigned int uint;
typedef unsigned char uchar;
typedef unsigned short ushort;

#define OJK_WAVE 64

// GGUF block sizes (reference: crates/ojas-formats/src/gguf.rs:563-591).
#define Q80_BYTES 34u
#define Q4K_BYTES 144u
#define Q5K_BYTES 176u
#define Q6K_BYTES 210u
#define IQ4NL_BYTES 18u
#define IQ4XS_BYTES 136u
#define Q2K_BYTES 84u
#define Q3K_BYTES 110u

// Vector types that may sit on a 2-byte boundary: Q8_0 (34 B) and Q6_K (210 B) blocks are only
// 2-byte aligned inside a row.  gfx950 runs in unaligned-access mode, so these compile to one
// global_load_dwordxN each.
struct __attribute__((packed, aligned(2))) u32x4_a2 { uint x, y, z, w; };
struct __attribute__((packed, aligned(2))) u32x2_a2 { uint x, y; };
typedef uint __attribute__((aligned(2))) u32_a2;
typedef uint __attribute__((aligned(1))) u32_a1;
#define MXFP4_BYTES 17u

// Scale i (0 .. 15) of a Q3_K block from its three packed words (crates/ojas-formats/src/gguf.rs:764-774):
// the low nibble sits in byte i (i < 8) or in the high nibble of byte i - 8, the two high bits in byte
// 8 + i % 4 at bit 2 (i / 4); stored biased by 32.
__device__ __forceinline__ int q3k_scale6(uint r0, uint r1, uint r2, uint i) {
    const uint src = (i & 4u) ? r1 : r0;
    const uint lo = (src >> (8u * (i & 3u) + ((i & 8u) >> 1))) & 0xFu;
    const uint hi = (r2 >> (8u * (i & 3u) + 2u * (i >> 2))) & 3u;
    return (int)(lo | (hi << 4)) - 32;
}

__device__ __forceinline__ float f16_bits_to_f32(uint bits16) {
    return __half2float(__ushort_as_half((ushort)bits16));
}
__device__ __forceinline__ float bf16_bits_to_f32(uint bits16) {
    return __uint_as_float(bits16 << 16);
}
// f32 -> bf16, round to nearest even (NaN kept quiet).
__device__ __forceinline__ ushort f32_to_bf16_bits(float f) {
    uint x = __float_as_uint(f);
    if ((x & 0x7F800000u) == 0x7F800000u && (x & 0x7FFFFFu)) return (ushort)((x >> 16) | 0x40u);
    x += 0x7FFFu + ((x >> 16) & 1u);
    return (ushort)(x >> 16);
}

// ---- DPP cross-lane moves (wave64) --------------------------------------------------------
#define OJK_DPP_QUAD_XOR1 0xB1   // quad_perm:[1,0,3,2]
#define OJK_DPP_QUAD_XOR2 0x4E   // quad_perm:[2,3,0,1]
#define OJK_DPP_ROW_HALF_MIRROR 0x141
#define OJK_DPP_ROW_MIRROR 0x140
#define OJK_DPP_ROW_SHL4 0x104          // lane i reads lane i + 4 of its row of 16 (zero past the row)
#define OJK_DPP_ROW_SHL8 0x108

template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}
template <int CTRL>
__device__ __forceinline__ int dpp_i32(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, true);
}

// The sums below start from a rounded value: without the empty asm the compiler contracts a
// product feeding the first step into fma(a, b, neighbour's product), which rounds differently
// from lane to lane and from one call site to the next.
__device__ __forceinline__ float rounded(float v) {
    asm("" : "+v"(v));
    return v;
}

// Sum over the 16 lanes of a DPP row; every lane of the row ends with the row total.
__device__ __forceinline__ float row16_sum(float v) {
    v = rounded(v);
    v += dpp_f32<OJK_DPP_QUAD_XOR1>(v);
    v += dpp_f32<OJK_DPP_QUAD_XOR2>(v);
    v += dpp_f32<OJK_DPP_ROW_HALF_MIRROR>(v);
    v += dpp_f32<OJK_DPP_ROW_MIRROR>(v);
    return v;
}
// Sum over groups of 8 adjacent lanes; every lane of the group ends with the group total.
__device__ __forceinline__ float oct_sum(float v) {
    v = rounded(v);
    v += dpp_f32<OJK_DPP_QUAD_XOR1>(v);
    v += dpp_f32<OJK_DPP_QUAD_XOR2>(v);
    v += dpp_f32<OJK_DPP_ROW_HALF_MIRROR>(v);
    return v;
}
// Sum over all 64 lanes; the total is returned in every lane (as a wave-uniform value).
__device__ __forceinline__ float wave_sum(float v) {
    v = row16_sum(v);
    float a = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
    float b = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
    float c = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
    float d = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
    return (a + b) + (c + d);
}
// Four sums at once, with the additions of row16_sum / wave_sum in their order (so: their bits) but a third of the
// instructions: after each of the first two steps a lane keeps only the value its position names — value (lane & 3) —
// and hands the other to the neighbour that keeps it; the steps across quads read the same position of the next quad.
// row16_sum4: lane j (j < 4) of every row of 16 ends with that row's total of value j; the other lanes hold partial sums.
// wave_sum4: lanes 0 .. 3 end with the wave's totals of values 0 .. 3.
__device__ __forceinline__ float row16_sum4(float v0, float v1, float v2, float v3, uint lane) {
    v0 = rounded(v0); v1 = rounded(v1); v2 = rounded(v2); v3 = rounded(v3);
    const bool odd = (lane & 1u) != 0u, up = (lane & 2u) != 0u;
    const float a = (odd ? v1 : v0) + dpp_f32<OJK_DPP_QUAD_XOR1>(odd ? v0 : v1);
    const float b = (odd ? v3 : v2) + dpp_f32<OJK_DPP_QUAD_XOR1>(odd ? v2 : v3);
    float c = (up ? b : a) + dpp_f32<OJK_DPP_QUAD_XOR2>(up ? a : b);
    c += dpp_f32<OJK_DPP_ROW_SHL4>(c);
    c += dpp_f32<OJK_DPP_ROW_SHL8>(c);
    return c;
}
// ... and two: lanes 0 / 1 end with the wave's totals of v0 / v1
__device__ __forceinline__ float wave_sum2(float v0, float v1, uint lane) {
    v0 = rounded(v0); v1 = rounded(v1);
    const bool odd = (lane & 1u) != 0u;
    float c = (odd ? v1 : v0) + dpp_f32<OJK_DPP_QUAD_XOR1>(odd ? v0 : v1);
    c += dpp_f32<OJK_DPP_QUAD_XOR2>(c);
    c += dpp_f32<OJK_DPP_ROW_SHL4>(c);
    c += dpp_f32<OJK_DPP_ROW_SHL8>(c);
    c += __shfl_xor(c, 16);
    c += __shfl_xor(c, 32);
    return c;
}
__device__ __forceinline__ float wave_sum4(float v0, float v1, float v2, float v3, uint lane) {
    float c = row16_sum4(v0, v1, v2, v3, lane);
    c += __shfl_xor(c, 16);
    c += __shfl_xor(c, 32);
    return c;
}
// The same in f64 (the two halves of a double travel as two 32-bit DPP moves): lanes 1, 2 apart, mirrored in eights and
// sixteens, then the four rows as (r0 + r1) + (r2 + r3).  One fixed order: whoever sums a segment's 64 lane values with
// this gets the same bits.
template <int CTRL>
__device__ __forceinline__ double dpp_f64(double v) {
    const long b = __double_as_longlong(v);
    const int lo = __builtin_amdgcn_update_dpp(0, (int)b, CTRL, 0xF, 0xF, true);
    const int hi = __builtin_amdgcn_update_dpp(0, (int)(b >> 32), CTRL, 0xF, 0xF, true);
    return __longlong_as_double(((long)hi << 32) | (unsigned int)lo);
}
__device__ __forceinline__ double readlane_f64(double v, int lane) {
    const long b = __double_as_longlong(v);
    const int lo = __builtin_amdgcn_readlane((int)b, lane), hi = __builtin_amdgcn_readlane((int)(b >> 32), lane);
    return __longlong_as_double(((long)hi << 32) | (unsigned int)lo);
}
__device__ __forceinline__ double wave_sum_f64(double v) {
    v += dpp_f64<OJK_DPP_QUAD_XOR1>(v);
    v += dpp_f64<OJK_DPP_QUAD_XOR2>(v);
    v += dpp_f64<OJK_DPP_ROW_HALF_MIRROR>(v);
    v += dpp_f64<OJK_DPP_ROW_MIRROR>(v);
    return (readlane_f64(v, 0) + readlane_f64(v, 16)) + (readlane_f64(v, 32) + readlane_f64(v, 48));
}
// The sum of part[0 .. n - 1] (n <= 64, in LDS) in one fixed order: term i in lane i, zeros above (adding 0.0 changes
// nothing), then wave_sum_f64's tree — one LDS trip and a dozen steps instead of n dependent ones.
__device__ __forceinline__ double tree_sum_f64(const double* part, uint n, uint lane) {
    return wave_sum_f64(lane < n ? part[lane] : 0.0);
}
// Saturation of a rounded activation to the int8 range as the reference's quantizers do it,
// `.round().clamp(-127.0, 127.0) as i8` (crates/ojas-cpu/src/cpu_math.rs:174-179, :545-563): a NaN passes through
// clamp and becomes 0 in the cast (fmaxf alone would turn it into -127).
__device__ __forceinline__ float sat127(float r) {
    const float c = fminf(fmaxf(r, -127.0f), 127.0f);
    return r == r ? c : 0.0f;
}
__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, dpp_f32<OJK_DPP_QUAD_XOR1>(v));
    v = fmaxf(v, dpp_f32<OJK_DPP_QUAD_XOR2>(v));
    v = fmaxf(v, dpp_f32<OJK_DPP_ROW_HALF_MIRROR>(v));
    v = fmaxf(v, dpp_f32<OJK_DPP_ROW_MIRROR>(v));
    float a = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
    float b = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
    float c = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
    float d = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
    return fmaxf(fmaxf(a, b), fmaxf(c, d));
}
__device__ __forceinline__ int wave_sum_i32(int v) {
    v += dpp_i32<OJK_DPP_QUAD_XOR1>(v);
    v += dpp_i32<OJK_DPP_QUAD_XOR2>(v);
    v += dpp_i32<OJK_DPP_ROW_HALF_MIRROR>(v);
    v += dpp_i32<OJK_DPP_ROW_MIRROR>(v);
    return __builtin_amdgcn_readlane(v, 0) + __builtin_amdgcn_readlane(v, 16) +
           __builtin_amdgcn_readlane(v, 32) + __builtin_amdgcn_readlane(v, 48);
}

// 4 x (i8 * i8) + acc on v_dot4_i32_i8.
__device__ __forceinline__ int dot4_i8(uint a, uint b, int acc) {
    return __builtin_amdgcn_sdot4((int)a, (int)b, acc, false);
}

// The first product of a chain.  Built with OJK_ASM_FIRST_DOT it is the three-operand encoding with a literal zero as
// the addend: left to itself the compiler picks the two-operand form, which accumulates in place and so needs a register
// cleared first — one more vector instruction per chain.  A family asks for it where that was measured to pay (the
// matvecs and the grouped expert dots, which issue instructions most of their time); in the single-launch chain the
// same change made the row workgroups a fifth slower, so the default is the builtin.
__device__ __forceinline__ int dot4_i8_first(uint a, uint b) {
#ifdef OJK_ASM_FIRST_DOT
    int r;
    asm("v_dot4_i32_i8 %0, %1, %2, 0" : "=v"(r) : "v"(a), "v"(b));
    return r;
#else
    return __builtin_amdgcn_sdot4((int)a, (int)b, 0, false);
#endif
}

// ---- Q4_K scale / min unpack ---------------------------------------------------------------
// The 12 scale bytes of a Q4_K / Q5_K super-block as three dwords (s0 = bytes 0..3, s1 = 4..7,
// s2 = 8..11).  Returns, for the sub-block pair (2c, 2c+1), the two 6-bit scales in bytes 0/1 of
// `sc` and the two 6-bit mins in bytes 0/1 of `mn`
// (reference: get_scale_min_k4, crates/ojas-formats/src/gguf.rs:1132-1140).
__device__ __forceinline__ void q4k_scale_min_pair(uint s0, uint s1, uint s2, uint c, uint& sc, uint& mn) {
    uint sh = (c & 1u) * 16u;
    uint y = s0 >> sh, z = s1 >> sh, w = s2 >> sh;
    uint sc_lo = y & 0x3F3Fu, mn_lo = z & 0x3F3Fu;
    uint sc_hi = (w & 0x0F0Fu) | ((y >> 2) & 0x3030u);
    uint mn_hi = ((w >> 4) & 0x0F0Fu) | ((z >> 2) & 0x3030u);
    sc = c < 2u ? sc_lo : sc_hi;
    mn = c < 2u ? mn_lo : mn_hi;
}

// ---- the IQ4 codebook ---------------------------------------------------------------------------
// IQ4_NL and IQ4_XS store 4-bit indices into sixteen fixed int8 levels
// (-127 -104 -83 -65 -49 -35 -22 -10 1 13 25 38 53 69 89 113; crates/ojas-core/src/iq_tables.rs:881-884).
// Four indices (one per byte, 0..15) -> their four levels as bytes: two byte-permutes over the halves
// of the table, merged by bit 3 of each index.
__device__ __forceinline__ uint iq4_levels4(uint idx4) {
    const uint sel = idx4 & 0x07070707u;
    const uint lo = __builtin_amdgcn_perm(0xF6EADDCFu, 0xBFAD9881u, sel);   // levels 0..7
    const uint hi = __builtin_amdgcn_perm(0x71594535u, 0x26190D01u, sel);   // levels 8..15
    const uint m1 = (idx4 >> 3) & 0x01010101u;
    const uint mask = (m1 << 8) - m1;                                       // 0xFF in every byte whose index is >= 8
    return (hi & mask) | (lo & ~mask);
}

// ---- global -> LDS copies by the memory system ------------------------------------------------
// One instruction moves 16 bytes per lane from base + voff to LDS bytes lds_addr + 16 lane .. (1 KB
// per wave, contiguous in LDS whatever the global addresses; lds_addr is the same in every lane).
// Completion is counted by vmcnt.
__device__ __forceinline__ void lds_dma16(const void* base, uint voff, uint lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(voff), "s"(base), "s"(__builtin_amdgcn_readfirstlane((int)lds_addr))
                 : "memory");
}
// wait until at most `n` vector memory operations are outstanding (a count not listed waits for all)
__device__ __forceinline__ void vm_wait(uint n) {
    switch (n) {
    case 0: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
    case 1: asm volatile("s_waitcnt vmcnt(1)" ::: "memory"); break;
    case 2: asm volatile("s_waitcnt vmcnt(2)" ::: "memory"); break;
    case 3: asm volatile("s_waitcnt vmcnt(3)" ::: "memory"); break;
    case 4: asm volatile("s_waitcnt vmcnt(4)" ::: "memory"); break;
    case 5: asm volatile("s_waitcnt vmcnt(5)" ::: "memory"); break;
    case 6: asm volatile("s_waitcnt vmcnt(6)" ::: "memory"); break;
    case 7: asm volatile("s_waitcnt vmcnt(7)" ::: "memory"); break;
    case 8: asm volatile("s_waitcnt vmcnt(8)" ::: "memory"); break;
    case 9: asm volatile("s_waitcnt vmcnt(9)" ::: "memory"); break;
    case 10: asm volatile("s_waitcnt vmcnt(10)" ::: "memory"); break;
    case 12: asm volatile("s_waitcnt vmcnt(12)" ::: "memory"); break;
    case 15: asm volatile("s_waitcnt vmcnt(15)" ::: "memory"); break;
    default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
    }
}

