// Q4_K super-blocks against 16 tokens on the int8 matrix cores: the pieces shared by the dense
// entries (family "gemm_q8k") and the grouped MoE entries (family "moe").
#pragma once
#include "ojk_common.h"

typedef int gq_i4 __attribute__((ext_vector_type(4)));
typedef float gq_f4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ long gq_pack(uint lo, uint hi) { return (long)(((unsigned long)hi << 32) | lo); }

// Four codes (a byte each, <= 15) times a factor <= 7 given as a pair of equal 16-bit halves: no byte's product
// (<= 105) carries into its neighbour, so one packed 16-bit multiply scales all four.
typedef ushort gq_u16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint gq_mul4(uint codes, gq_u16x2 f) {
    return __builtin_bit_cast(uint, __builtin_bit_cast(gq_u16x2, codes) * f);
}

struct GqW {            // lane (n, kg): its bytes of one super-block of row n
    uint4 hdr;          // d, dmin, the 12 scale bytes
    uint2 q[4];         // codes of positions 8 kg .. 8 kg + 7 of each 64-weight chunk (low | high nibbles)
};
__device__ __forceinline__ GqW gq_load(const uchar* blk, uint kg) {
    GqW r;
    r.hdr = *(const uint4*)blk;
#pragma unroll
    for (int c = 0; c < 4; c++) r.q[c] = *(const uint2*)(blk + 16u + 32u * c + 8u * kg);
    return r;
}

// One super-block of a 16-row tile against one pass of 16 tokens:
//   acc[v] += sx * (d * sum_j sc_j idot_j - dmin * sum_j m_j bsum_j)   for token 4 kg + v, row n.
// xp: the lane's 8 bytes of token n at this super-block (byte 8 kg); pq: token n's split sums
// (eight lo parts, eight hi parts); sx16: the super-block's 16 token scales.
__device__ __forceinline__ void gq_superblock(const GqW& cur, const uchar* xp, const uchar* pq, const float* sx16, uint kg,
                                              float (&acc)[4]) {
    const gq_i4 zero = {0, 0, 0, 0};
    const float d = f16_bits_to_f32(cur.hdr.x & 0xFFFFu), dmin = f16_bits_to_f32(cur.hdr.x >> 16);
    // all eight 6-bit scales and mins at once, a byte each (get_scale_min_k4, crates/ojas-formats/src/gguf.rs:1132-1140):
    // sub-blocks 0-3 are the low six bits of bytes 0-3 / 4-7, sub-blocks 4-7 a nibble of bytes 8-11 under
    // the top two bits of bytes 0-3 / 4-7
    const uint sc_lo = cur.hdr.y & 0x3F3F3F3Fu, mn_lo = cur.hdr.z & 0x3F3F3F3Fu;
    const uint sc_hi = (cur.hdr.w & 0x0F0F0F0Fu) | ((cur.hdr.y >> 2) & 0x30303030u);
    const uint mn_hi = ((cur.hdr.w >> 4) & 0x0F0F0F0Fu) | ((cur.hdr.z >> 2) & 0x30303030u);
    int sc[8];
    long B[8];
#pragma unroll
    for (int c = 0; c < 4; c++) {
        sc[c] = (int)((sc_lo >> (8 * c)) & 0xFFu);
        sc[4 + c] = (int)((sc_hi >> (8 * c)) & 0xFFu);
        B[2 * c] = gq_pack(cur.q[c].x & 0x0F0F0F0Fu, cur.q[c].y & 0x0F0F0F0Fu);
        B[2 * c + 1] = gq_pack((cur.q[c].x >> 4) & 0x0F0F0F0Fu, (cur.q[c].y >> 4) & 0x0F0F0F0Fu);
    }
    const long Bm = kg == 0u ? gq_pack(mn_lo, mn_hi) : 0;       // mins 0..7 in bytes 0..7; only positions 0..7 carry them
    int isum[4] = {0, 0, 0, 0};
#pragma unroll
    for (int jj = 0; jj < 8; jj++) {
        const long A = *(const long*)(xp + 32 * jj);
        const gq_i4 D = __builtin_amdgcn_mfma_i32_16x16x32_i8(A, B[jj], zero, 0, 0, 0);
#pragma unroll
        for (int v = 0; v < 4; v++) isum[v] += __mul24(sc[jj], D[v]);
    }
    // (masked, not branched over: a branch here splits the unrolled code into basic blocks and costs registers)
    const long km_ = kg == 0u ? -1l : 0l;
    const long Alo = *(const long*)pq & km_, Ahi = *(const long*)(pq + 8) & km_;
    const gq_i4 Dlo = __builtin_amdgcn_mfma_i32_16x16x32_i8(Alo, Bm, zero, 0, 0, 0);
    const gq_i4 Dhi = __builtin_amdgcn_mfma_i32_16x16x32_i8(Ahi, Bm, zero, 0, 0, 0);
    const float4 sx = *(const float4*)(sx16 + 4u * kg);
    acc[0] += sx.x * (d * (float)isum[0] - dmin * (float)(64 * Dhi[0] + Dlo[0]));
    acc[1] += sx.y * (d * (float)isum[1] - dmin * (float)(64 * Dhi[1] + Dlo[1]));
    acc[2] += sx.z * (d * (float)isum[2] - dmin * (float)(64 * Dhi[2] + Dlo[2]));
    acc[3] += sx.w * (d * (float)isum[3] - dmin * (float)(64 * Dhi[3] + Dlo[3]));
}

