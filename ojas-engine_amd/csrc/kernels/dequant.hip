// Family "dequant": GGUF blocks -> IEEE binary16, bit-exact with the reference decoder
// (crates/ojas-formats/src/gguf.rs:612-1116; arms :704-709 Q8_0, :1042-1059 Q4_K,
// :1060-1085 Q5_K, :1086-1108 Q6_K, :796-813 IQ4_NL, :814-840 IQ4_XS, :653-703 Q4_0 / Q5_0 / Q4_1 / Q5_1; MXFP4: crates/ojas-formats/src/mxfp4.rs).
//
// Bit-exactness rules: every product and difference is a separately rounded f32 operation
// (__fmul_rn / __fsub_rn, never an FMA), in the reference's association order, followed by one
// round-to-nearest-even conversion to binary16.  The file is also compiled with
// -ffp-contract=off.
//
// Signature convention: pointers first, then u32 scalars.
//   dequant_<fmt>_f16(const uchar* w, ushort* out, uint nblocks)
#include "ojk_common.h"

// The f32 value is pinned in a register before the conversion: left to itself the compiler folds
// "multiply, then convert" into one mixed-precision FMA, which rounds once instead of twice and
// loses the sign of a zero product.
__device__ __forceinline__ ushort f32_to_f16_bits(float v) {
    asm volatile("" : "+v"(v));
    return __half_as_ushort(__float2half_rn(v));
}

// Eight consecutive values leave as one 16-byte store where the output is 16-byte aligned (a thread's eight start at a
// multiple of eight, so that is a property of the output pointer), as eight 2-byte stores otherwise.  (A thread per
// weight, or eight 2-byte stores per thread, kept these kernels at 1.9 - 2.7 TB/s; the 16-byte form reaches what the
// grid-codebook decoders do.)
// (The 16-byte store is spelled as an instruction: written as a plain store the compiler merged it with the
// fallback's stores of the same values and kept the 2-byte ones.)
typedef uint dq_u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void store8_f16(ushort* o, const ushort (&h)[8]) {
    if (((size_t)o & 15u) == 0) {
        const dq_u32x4 v = {(uint)h[0] | ((uint)h[1] << 16), (uint)h[2] | ((uint)h[3] << 16),
                            (uint)h[4] | ((uint)h[5] << 16), (uint)h[6] | ((uint)h[7] << 16)};
        asm volatile("global_store_dwordx4 %0, %1, off" : : "v"(o), "v"(v) : "memory");
    } else {
#pragma unroll
        for (int i = 0; i < 8; i++) o[i] = h[i];
    }
}
__device__ __forceinline__ uint byte_of(uint lo, uint hi, int i) { return ((i < 4 ? lo : hi) >> (8 * (i & 3))) & 0xFFu; }

extern "C" __global__ void __launch_bounds__(256)
dequant_q80_f16(const uchar* __restrict__ w, ushort* __restrict__ out, uint nblocks) {
    // four threads per block, eight consecutive weights each
    size_t tid = (size_t)blockIdx.x * 256u + threadIdx.x;
    size_t b = tid >> 2;
    if (b >= nblocks) return;
    const uint j = (uint)tid & 3u;
    const uchar* blk = w + b * Q80_BYTES;
    const float d = f16_bits_to_f32(*(const ushort*)blk);
    const u32x2_a2 q = *(const u32x2_a2*)(blk + 2u + 8u * j);
    ushort h[8];
#pragma unroll
    for (int i = 0; i < 8; i++) h[i] = f32_to_f16_bits(__fmul_rn(d, (float)(signed char)byte_of(q.x, q.y, i)));
    store8_f16(out + b * 32u + 8u * j, h);
}

// Embedding gather straight out of Q8_0 storage (crates/ojas-cuda/src/kernels/gemv_q8.rs:262-293): row `token`
// of the table as f32, each value the exact f32 product d * q (the decoder above rounds it once more to
// f16).  embed_q80(table, out, token, d) takes the id as a launch constant, embed_q80_g(table, out, ctl, d)
// reads it from ctl[0] on the device, so a recorded decode step replays without re-recording per token.
// Any grid of up to 256-thread blocks (a thread per weight, grid-stride).  ROWS, appended by the dispatcher
// from the table's extent, is not in the reference's argument list: an id past the table yields zeros.
__device__ __forceinline__ void embed_q80_row(const uchar* __restrict__ table, float* __restrict__ out,
                                              uint token, uint d, uint ROWS) {
    const uchar* row = table + (size_t)token * (d >> 5) * Q80_BYTES;
    for (uint i = blockIdx.x * blockDim.x + threadIdx.x; i < d; i += gridDim.x * blockDim.x) {
        float v = 0.0f;
        if (token < ROWS) {
            const uchar* blk = row + (size_t)(i >> 5) * Q80_BYTES;
            v = __fmul_rn(f16_bits_to_f32(*(const ushort*)blk), (float)(signed char)blk[2u + (i & 31u)]);
        }
        out[i] = v;
    }
}
extern "C" __global__ void __launch_bounds__(256)
embed_q80(const uchar* __restrict__ table, float* __restrict__ out, uint token, uint d, uint ROWS) {
    embed_q80_row(table, out, token, d, ROWS);
}
extern "C" __global__ void __launch_bounds__(256)
embed_q80_g(const uchar* __restrict__ table, float* __restrict__ out, const uint* __restrict__ ctl, uint d, uint ROWS) {
    embed_q80_row(table, out, ctl[0], d, ROWS);
}

extern "C" __global__ void __launch_bounds__(256)
dequant_q4k_f16(const uchar* __restrict__ w, ushort* __restrict__ out, uint nblocks) {
    // 32 threads per super-block; thread t owns eight consecutive weights: chunk c = t / 8 (64 weights, the low
    // nibbles of its 32 bytes then the high ones), half hi = (t / 4) % 2, bytes 8 (t % 4) .. + 7 of the chunk.
    size_t tid = (size_t)blockIdx.x * 256u + threadIdx.x;
    size_t b = tid >> 5;
    if (b >= nblocks) return;
    const uint t = (uint)tid & 31u, c = t >> 3, hi = (t >> 2) & 1u, part = t & 3u;
    const uchar* blk = w + b * Q4K_BYTES;
    const uint* hdr = (const uint*)blk;
    const uint dd = hdr[0];
    const float d = f16_bits_to_f32(dd & 0xFFFFu), dmin = f16_bits_to_f32(dd >> 16);
    uint sc, mn;
    q4k_scale_min_pair(hdr[1], hdr[2], hdr[3], c, sc, mn);
    const float dl = __fmul_rn(d, (float)(hi ? sc >> 8 : sc & 0xFFu)), ml = __fmul_rn(dmin, (float)(hi ? mn >> 8 : mn & 0xFFu));
    const uint q0 = (hdr[4u + c * 8u + 2u * part] >> (4u * hi)) & 0x0F0F0F0Fu;
    const uint q1 = (hdr[5u + c * 8u + 2u * part] >> (4u * hi)) & 0x0F0F0F0Fu;
    ushort h[8];
#pragma unroll
    for (int i = 0; i < 8; i++) h[i] = f32_to_f16_bits(__fsub_rn(__fmul_rn(dl, (float)byte_of(q0, q1, i)), ml));
    store8_f16(out + b * 256u + c * 64u + hi * 32u + part * 8u, h);
}

extern "C" __global__ void __launch_bounds__(256)
dequant_q5k_f16(const uchar* __restrict__ w, ushort* __restrict__ out, uint nblocks) {
    // As Q4_K, plus the fifth bit: bit 2 c + hi of qh[l], l the byte's place among the chunk's 32.
    size_t tid = (size_t)blockIdx.x * 256u + threadIdx.x;
    size_t b = tid >> 5;
    if (b >= nblocks) return;
    const uint t = (uint)tid & 31u, c = t >> 3, hi = (t >> 2) & 1u, part = t & 3u;
    const uchar* blk = w + b * Q5K_BYTES;
    const uint* hdr = (const uint*)blk;
    const uint dd = hdr[0];
    const float d = f16_bits_to_f32(dd & 0xFFFFu), dmin = f16_bits_to_f32(dd >> 16);
    uint sc, mn;
    q4k_scale_min_pair(hdr[1], hdr[2], hdr[3], c, sc, mn);
    const float dl = __fmul_rn(d, (float)(hi ? sc >> 8 : sc & 0xFFu)), ml = __fmul_rn(dmin, (float)(hi ? mn >> 8 : mn & 0xFFu));
    const uint h0 = (hdr[4u + 2u * part] >> (2u * c + hi)) & 0x01010101u, h1 = (hdr[5u + 2u * part] >> (2u * c + hi)) & 0x01010101u;
    const uint q0 = (hdr[12u + c * 8u + 2u * part] >> (4u * hi)) & 0x0F0F0F0Fu;
    const uint q1 = (hdr[13u + c * 8u + 2u * part] >> (4u * hi)) & 0x0F0F0F0Fu;
    ushort h[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const float fifth = byte_of(h0, h1, i) ? 16.0f : 0.0f;
        h[i] = f32_to_f16_bits(__fsub_rn(__fmul_rn(dl, __fadd_rn((float)byte_of(q0, q1, i), fifth)), ml));
    }
    store8_f16(out + b * 256u + c * 64u + hi * 32u + part * 8u, h);
}

extern "C" __global__ void __launch_bounds__(256)
dequant_q6k_f16(const uchar* __restrict__ w, ushort* __restrict__ out, uint nblocks) {
    // 32 threads per super-block; thread t owns eight consecutive weights: half hf = t / 16, quarter j = (t / 4) % 4 of
    // its 128 (weights 32 j ..: the low nibbles of ql[0..31], of ql[32..63], then the high nibbles of each), places
    // l = 8 (t % 4) .. + 7; bits 2 j, 2 j + 1 of qh[l] on top, scale l / 16 + 2 j.
    // The value is (d * sc) * q, left to right, as the reference writes it.
    size_t tid = (size_t)blockIdx.x * 256u + threadIdx.x;
    size_t b = tid >> 5;
    if (b >= nblocks) return;
    const uint t = (uint)tid & 31u, hf = t >> 4, j = (t >> 2) & 3u, l0 = (t & 3u) * 8u;
    const uchar* blk = w + b * Q6K_BYTES;
    const u32x2_a2 ql = *(const u32x2_a2*)(blk + hf * 64u + (j & 1u) * 32u + l0);
    const u32x2_a2 qh = *(const u32x2_a2*)(blk + 128u + hf * 32u + l0);
    const float d = f16_bits_to_f32(*(const ushort*)(blk + 208u));
    const float dl = __fmul_rn(d, (float)((const signed char*)(blk + 192u + hf * 8u))[(l0 >> 4) + 2u * j]);
    const uint n0 = (ql.x >> (4u * (j >> 1))) & 0x0F0F0F0Fu, n1 = (ql.y >> (4u * (j >> 1))) & 0x0F0F0F0Fu;
    const uint h0 = (qh.x >> (2u * j)) & 0x03030303u, h1 = (qh.y >> (2u * j)) & 0x03030303u;
    ushort h[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const int q = (int)(byte_of(n0, n1, i) | (byte_of(h0, h1, i) << 4)) - 32;
        h[i] = f32_to_f16_bits(__fmul_rn(dl, (float)q));
    }
    store8_f16(out + b * 256u + hf * 128u + j * 32u + l0, h);
}

// relayout_q4k_q4l(w, nib, qa, qb, nblocks): Q4_K super-blocks -> the Q4L side arrays of the
// reference's prefill GEMM (crates/ojas-formats/src/quant.rs:192-222): per 32-weight block j of
// a super-block, qa = f16(d*sc_j), qb = f16(-dmin*m_j), and 16 bytes holding weights (2i, 2i+1)
// of the block as (low, high) nibble.  Rows are whole super-blocks, so the arrays are indexed
// by the running super-block number.  One thread per 32-weight block.
extern "C" __global__ void __launch_bounds__(256)
relayout_q4k_q4l(const uchar* __restrict__ w, uchar* __restrict__ nib, ushort* __restrict__ qa,
                 ushort* __restrict__ qb, uint nblocks) {
    size_t tid = (size_t)blockIdx.x * 256u + threadIdx.x;
    size_t b = tid >> 3;
    if (b >= nblocks) return;
    const uint j = (uint)tid & 7u, c = j >> 1, hi = j & 1u;
    const uchar* blk = w + b * Q4K_BYTES;
    const uint* hdr = (const uint*)blk;
    const uint dd = hdr[0];
    const float d = f16_bits_to_f32(dd & 0xFFFFu), ndm = -f16_bits_to_f32(dd >> 16);
    uint sc, mn;
    q4k_scale_min_pair(hdr[1], hdr[2], hdr[3], c, sc, mn);
    const uint s_ = hi ? sc >> 8 : sc & 0xFFu, m_ = hi ? mn >> 8 : mn & 0xFFu;
    qa[tid] = f32_to_f16_bits(__fmul_rn(d, (float)s_));
    qb[tid] = f32_to_f16_bits(__fmul_rn(ndm, (float)m_));
    const uint* qq = hdr + 4 + c * 8u;   // the chunk's 32 bytes
    uint out[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {        // 8 source bytes -> 4 packed bytes
        uint a = qq[2 * i] >> (4u * hi), e = qq[2 * i + 1] >> (4u * hi);
        uint p0 = (a & 0xFu) | (((a >> 8) & 0xFu) << 4), p1 = ((a >> 16) & 0xFu) | (((a >> 24) & 0xFu) << 4);
        uint p2 = (e & 0xFu) | (((e >> 8) & 0xFu) << 4), p3 = ((e >> 16) & 0xFu) | (((e >> 24) & 0xFu) << 4);
        out[i] = p0 | (p1 << 8) | (p2 << 16) | (p3 << 24);
    }
    *(uint4*)(nib + tid * 16u) = make_uint4(out[0], out[1], out[2], out[3]);
}

extern "C" __global__ void __launch_bounds__(256)
dequant_iq4nl_f16(const uchar* __restrict__ w, ushort* __restrict__ out, uint nblocks) {
    // four threads per block, eight consecutive weights each: weights 0..15 are the low nibbles of qs[0..15], 16..31
    // the high nibbles
    size_t tid = (size_t)blockIdx.x * 256u + threadIdx.x;
    size_t b = tid >> 2;
    if (b >= nblocks) return;
    const uint j = (uint)tid & 3u, hi = j >> 1, part = j & 1u;
    const uchar* blk = w + b * IQ4NL_BYTES;
    const float d = f16_bits_to_f32(*(const ushort*)blk);
    const u32x2_a2 q = *(const u32x2_a2*)(blk + 2u + 8u * part);
    const uint l0 = iq4_levels4((q.x >> (4u * hi)) & 0x0F0F0F0Fu), l1 = iq4_levels4((q.y >> (4u * hi)) & 0x0F0F0F0Fu);
    ushort h[8];
#pragma unroll
    for (int i = 0; i < 8; i++) h[i] = f32_to_f16_bits(__fmul_rn(d, (float)(signed char)byte_of(l0, l1, i)));
    store8_f16(out + b * 32u + 16u * hi + 8u * part, h);
}

extern "C" __global__ void __launch_bounds__(256)
dequant_iq4xs_f16(const uchar* __restrict__ w, ushort* __restrict__ out, uint nblocks) {
    // 32 threads per super-block; thread t owns eight consecutive weights of sub-block ib = t / 4: the low (hi = 0) or
    // high nibbles of its bytes 8 (t % 2) .. + 7, which are weights 16 hi + 8 (t % 2) .. of the sub-block.
    size_t tid = (size_t)blockIdx.x * 256u + threadIdx.x;
    size_t b = tid >> 5;
    if (b >= nblocks) return;
    const uint t = (uint)tid & 31u, ib = t >> 2, hi = (t >> 1) & 1u, part = t & 1u;
    const uchar* blk = w + b * IQ4XS_BYTES;
    const uint* hdr = (const uint*)blk;
    const uint h0 = hdr[0], sl = hdr[1];
    const float d = f16_bits_to_f32(h0 & 0xFFFFu);
    const uint sh = h0 >> 16;
    const uint ls = ((sl >> (4u * ib)) & 0xFu) | (((sh >> (2u * ib)) & 3u) << 4);
    const float dl = __fmul_rn(d, (float)((int)ls - 32));
    const uint l0 = iq4_levels4((hdr[2u + ib * 4u + 2u * part] >> (4u * hi)) & 0x0F0F0F0Fu);
    const uint l1 = iq4_levels4((hdr[3u + ib * 4u + 2u * part] >> (4u * hi)) & 0x0F0F0F0Fu);
    ushort h[8];
#pragma unroll
    for (int i = 0; i < 8; i++) h[i] = f32_to_f16_bits(__fmul_rn(dl, (float)(signed char)byte_of(l0, l1, i)));
    store8_f16(out + b * 256u + ib * 32u + 16u * hi + 8u * part, h);
}

// Q2_K and Q3_K keep four 2-bit planes per byte: within a half of 128 weights, byte l of the half's 32 code
// bytes holds weights l, l + 32, l + 64, l + 96 at bits 0, 2, 4, 6, and scale 8 half + 2 j + l / 16 covers the
// 16 weights (plane j, l / 16).  32 threads per super-block; thread t decodes the eight consecutive weights
// 128 half + 32 j + 8 (t % 4) .. + 7 with half = t / 16, j = (t / 4) % 4.
extern "C" __global__ void __launch_bounds__(256)
dequant_q2k_f16(const uchar* __restrict__ w, ushort* __restrict__ out, uint nblocks) {
    // block { u8 scales[16]; u8 qs[64]; half d; half dmin; }: w = (d * sc) * q - dmin * m, every step rounded
    // (crates/ojas-formats/src/gguf.rs:730-754)
    size_t tid = (size_t)blockIdx.x * 256u + threadIdx.x;
    size_t b = tid >> 5;
    if (b >= nblocks) return;
    const uint t = (uint)tid & 31u, half = t >> 4, j = (t >> 2) & 3u, l0 = (t & 3u) * 8u;
    const uchar* blk = w + b * Q2K_BYTES;
    const uint sc = blk[half * 8u + j * 2u + (l0 >> 4)];
    const uint dd = *(const uint*)(blk + 80);
    const float dl = __fmul_rn(f16_bits_to_f32(dd & 0xFFFFu), (float)(sc & 0xFu));
    const float ml = __fmul_rn(f16_bits_to_f32(dd >> 16), (float)(sc >> 4));
    const uint* qp = (const uint*)(blk + 16u + half * 32u + l0);
    const uint q0 = (qp[0] >> (2u * j)) & 0x03030303u, q1 = (qp[1] >> (2u * j)) & 0x03030303u;
    ushort h[8];
#pragma unroll
    for (int i = 0; i < 8; i++) h[i] = f32_to_f16_bits(__fsub_rn(__fmul_rn(dl, (float)byte_of(q0, q1, i)), ml));
    store8_f16(out + b * 256u + half * 128u + j * 32u + l0, h);
}

extern "C" __global__ void __launch_bounds__(256)
dequant_q3k_f16(const uchar* __restrict__ w, ushort* __restrict__ out, uint nblocks) {
    // block { u8 hmask[32]; u8 qs[64]; u8 scales[12]; half d; }: w = (d * (sc - 32)) * (q - (mask bit ? 0 : 4)),
    // bit 4 half + j of hmask[l] belonging to weight (half, j, l) (crates/ojas-formats/src/gguf.rs:755-795).
    // Blocks are 110 bytes: two-byte alignment is all a block has.
    size_t tid = (size_t)blockIdx.x * 256u + threadIdx.x;
    size_t b = tid >> 5;
    if (b >= nblocks) return;
    const uint t = (uint)tid & 31u, half = t >> 4, j = (t >> 2) & 3u, l0 = (t & 3u) * 8u;
    const uchar* blk = w + b * Q3K_BYTES;
    const u32_a2* raw = (const u32_a2*)(blk + 96);
    const int sc = q3k_scale6(raw[0], raw[1], raw[2], half * 8u + j * 2u + (l0 >> 4));
    const float dl = __fmul_rn(f16_bits_to_f32(*(const ushort*)(blk + 108)), (float)sc);
    const u32_a2* qp = (const u32_a2*)(blk + 32u + half * 32u + l0);
    const u32_a2* hp = (const u32_a2*)(blk + l0);
    const uint sh = half * 4u + j;
    ushort ho[8];
#pragma unroll
    for (int v = 0; v < 2; v++) {
        const uint q = (qp[v] >> (2u * j)) & 0x03030303u, h = (hp[v] >> sh) & 0x01010101u;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int code = (int)((q >> (8 * i)) & 0xFFu) - (((h >> (8 * i)) & 1u) ? 0 : 4);
            ho[4 * v + i] = f32_to_f16_bits(__fmul_rn(dl, (float)code));
        }
    }
    store8_f16(out + b * 256u + half * 128u + j * 32u + l0, ho);
}

// The legacy 32-weight blocks: four threads per block, eight consecutive weights each (weight j < 16 is the low nibble
// of qs[j], else the high nibble of qs[j - 16]).  AFFINE: {d, m} header and w = d * q + m (a product and a sum, each
// rounded), else w = d * (q - 8 | 16); FIVE: a 4-byte field of fifth bits ahead of the nibbles.
template <bool FIVE, bool AFFINE>
__device__ __forceinline__ void dequant_legacy(const uchar* __restrict__ w, ushort* __restrict__ out, uint nblocks) {
    const uint BYTES = 18u + (AFFINE ? 2u : 0u) + (FIVE ? 4u : 0u), HDR = AFFINE ? 4u : 2u;
    size_t tid = (size_t)blockIdx.x * 256u + threadIdx.x;
    size_t b = tid >> 2;
    if (b >= nblocks) return;
    const uint j4 = (uint)tid & 3u, hi = j4 >> 1, part = j4 & 1u;
    const uchar* blk = w + b * BYTES;
    const u32x2_a2 qs = *(const u32x2_a2*)(blk + HDR + (FIVE ? 4u : 0u) + 8u * part);
    const uint q0 = (qs.x >> (4u * hi)) & 0x0F0F0F0Fu, q1 = (qs.y >> (4u * hi)) & 0x0F0F0F0Fu;
    uint qh = 0u;
    if (FIVE) qh = ((uint)*(const ushort*)(blk + HDR) | ((uint)*(const ushort*)(blk + HDR + 2u) << 16)) >> (16u * hi + 8u * part);
    const float d = f16_bits_to_f32(*(const ushort*)blk);
    const float m = AFFINE ? f16_bits_to_f32(*(const ushort*)(blk + 2)) : 0.0f;
    ushort h[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        uint q = byte_of(q0, q1, i);
        if (FIVE) q |= ((qh >> i) & 1u) << 4;
        float v;
        if (AFFINE) v = __fadd_rn(__fmul_rn(d, (float)q), m);
        else v = __fmul_rn(d, __fsub_rn((float)q, FIVE ? 16.0f : 8.0f));
        h[i] = f32_to_f16_bits(v);
    }
    store8_f16(out + b * 32u + 16u * hi + 8u * part, h);
}
extern "C" __global__ void __launch_bounds__(256)
dequant_q40_f16(const uchar* w, ushort* out, uint nblocks) { dequant_legacy<false, false>(w, out, nblocks); }
extern "C" __global__ void __launch_bounds__(256)
dequant_q41_f16(const uchar* w, ushort* out, uint nblocks) { dequant_legacy<false, true>(w, out, nblocks); }
extern "C" __global__ void __launch_bounds__(256)
dequant_q50_f16(const uchar* w, ushort* out, uint nblocks) { dequant_legacy<true, false>(w, out, nblocks); }
extern "C" __global__ void __launch_bounds__(256)
dequant_q51_f16(const uchar* w, ushort* out, uint nblocks) { dequant_legacy<true, true>(w, out, nblocks); }

// MXFP4 (crates/ojas-formats/src/mxfp4.rs:40-58): { u8 e; u8 qs[16] }, w = 2^(e - 127) * E2M1[code], weight 2j the low
// and 2j + 1 the high nibble of qs[j].  The product of a power of two and a 2-bit significand is exact; one rounding to f16.
extern "C" __global__ void __launch_bounds__(256)
dequant_mxfp4_f16(const uchar* __restrict__ w, ushort* __restrict__ out, uint nblocks) {
    // four threads per block, eight consecutive weights each: the nibbles of four consecutive bytes of codes
    const size_t tid = (size_t)blockIdx.x * 256u + threadIdx.x;
    const size_t b = tid >> 2;
    if (b >= nblocks) return;
    const uint p = (uint)tid & 3u;
    const uchar* blk = w + b * 17u;
    const float d = __uint_as_float((uint)blk[0] << 23);
    ushort h[8];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const uint q = blk[1u + 4u * p + (uint)j];
#pragma unroll
        for (int hh = 0; hh < 2; hh++) {
            const uint c = hh ? q >> 4 : q & 15u, m = c & 7u;
            const float a = 0.5f * (float)(m < 5u ? m : m == 5u ? 6u : m == 6u ? 8u : 12u);
            h[2 * j + hh] = f32_to_f16_bits(__fmul_rn(d, __uint_as_float(__float_as_uint(a) | ((c >> 3) << 31))));
        }
    }
    store8_f16(out + b * 32u + 8u * p, h);
}
