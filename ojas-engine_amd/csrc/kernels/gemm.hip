// Family "gemm": prefill / verify matmul  y[M,N] (+)= x[M,K] . W^T  with W in GGUF blocks.
//
// Contract (reference: crates/ojas-cuda/src/kernels/gemm_q.rs:1-56; raw K-quant twin
// crates/ojas-metal/src/kernels/gemm_fat.rs:243-368): activations rounded to f16 on their way into
// the tile, weights dequantized to f16 into the tile, f32 accumulation, f32 y; any M and N (loads
// clamped, stores masked, nothing written past row M).  Here the dequantized tile holds exactly
// the bits `dequant_to_f16` produces (crates/ojas-formats/src/gguf.rs:612-1116): every product and
// difference is rounded on its own (the file is compiled with -ffp-contract=off), then one
// round-to-nearest-even to binary16.
//
//   gemm_mm_<fmt>(xh, w, y, K, N, accum, M)        xh: f16 [M][K]; grid [ceil(N/128), ceil(M/256), 1]
//   gemm_mm_<fmt>_sk(xh, w, y, K, N, M, nsplit)    grid.z = nsplit; adds its K slice into y with
//                                                  f32 atomics (zero y first for a plain product)
//
// CDNA4 plan: one workgroup of 4 waves (one per SIMD) owns a 256 (tokens) x 128 (outputs) tile
// and walks K in steps of 64.  Per step the 256 threads stage the activation slab (256 x 64 f16)
// and dequantize the weight slab (128 rows x 64 weights, 32 per thread) into LDS, rows padded to
// 144 bytes so 16-byte fragment reads of 16 consecutive rows fall in distinct banks.  Each wave
// owns 128 x 64 of the tile as 4 x 2 blocks of v_mfma_f32_32x32x16_f16 (A = activations, B =
// weights, so a D register holds 32 consecutive outputs of one token: coalesced stores).
// With one wave per SIMD nothing else hides latency, so the step is a hand-built pipeline:
//   * global loads run three steps ahead in registers: ordinary loads the compiler tracks itself, held in
//     place by a scheduling fence so that they are not sunk to their use;
//   * the dequantization of step t+1 (vector ALU) is interleaved with the MFMAs of step t
//     (sched_group_barrier), its LDS writes go to the other stage, one barrier per step.
#include "ojk_common.h"

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float2v __attribute__((ext_vector_type(2)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef uint u32x4 __attribute__((ext_vector_type(4)));

#define GM_BM 256
#define GM_BN 128
#define GM_BK 64
#define GM_STRIDE 144  // bytes per LDS row: 64 f16 + 16 bytes of padding
#define GM_STAGE ((GM_BM + GM_BN) * GM_STRIDE)

// Two f32 -> packed f16, round to nearest even.  The values are pinned in registers first so that
// "multiply/subtract, then convert" cannot be folded into a mixed-precision FMA (which would
// round once instead of twice and lose the sign of a zero product).
__device__ __forceinline__ uint pack2(float a, float b) {
    asm volatile("" : "+v"(a), "+v"(b));
    float2v f = {a, b};
    return __builtin_bit_cast(uint, __builtin_convertvector(f, half2v));
}

// ---- global loads --------------------------------------------------------------------------------
// Ordinary loads: the compiler sees every one of them, counts them in its own s_waitcnt and never reads a
// destination register before its load has landed.  What keeps a prefetch three steps ahead of its use is the
// scheduling fence behind each group of loads (gm_fence): the scheduler may not sink them past it.
__device__ __forceinline__ u32x4 gm_load16(const void* p) {
    // (blocks of 34 and 210 bytes are only 2-byte aligned; the target runs in unaligned-access mode)
    typedef u32x4 __attribute__((aligned(2))) u32x4_u;
    return *(const u32x4_u*)p;
}
__device__ __forceinline__ uint gm_load_u16(const void* p) { return *(const ushort*)p; }
__device__ __forceinline__ uint gm_load_u8(const void* p) { return *(const uchar*)p; }
__device__ __forceinline__ void gm_fence() { __builtin_amdgcn_sched_barrier(0); }
// 8 activations at element offset `at` as f16: loaded as such, or converted from f32 (round to nearest even)
template <bool XF32>
__device__ __forceinline__ u32x4 gm_load_x(const ushort* xh, const float* xf, size_t at) {
    if (!XF32) return *(const u32x4*)(xh + at);
    const float4 a = *(const float4*)(xf + at), b = *(const float4*)(xf + at + 4);
    return (u32x4){pack2(a.x, a.y), pack2(a.z, a.w), pack2(b.x, b.y), pack2(b.z, b.w)};
}

// ------------------------------------------------------------------ per-format slab loaders
// A loader owns, for one thread, 32 weights of one row of the 128 x 64 slab: thread t -> row
// t/2, half h = t%2.  `load` issues the global loads (NL of them); after the wait, `prep` unpacks
// the scales, `part<I>` dequantizes a quarter of the weights (so the work can be spread between
// MFMAs), `flush` writes the 32 f16 to the LDS row.
// What a kernel passes for its weights: the block bytes, plus the side arrays of the formats that have them.
struct GmSrc {
    const uchar* w;
    const ushort* qa;
    const ushort* qb;
};

struct LoaderQ4K {
    static constexpr int NL = 2;
    typedef const uchar* Row;
    static __device__ __forceinline__ Row row(const GmSrc& s, uint n, uint K) { return s.w + (size_t)n * row_bytes(K); }
    u32x4 hdr, qs;
    uint c;
    float dl1, ml1, dl2, ml2;
    uint lo[8], hi[8];
    static __device__ __forceinline__ size_t row_bytes(uint K) { return (size_t)(K >> 8) * Q4K_BYTES; }
    __device__ __forceinline__ void load(const uchar* row, uint k0, uint h) {
        const uchar* blk = row + (size_t)(k0 >> 8) * Q4K_BYTES;
        c = (k0 >> 6) & 3u;  // 32-byte chunk of the super-block = sub-blocks 2c, 2c+1
        hdr = gm_load16(blk);
        qs = gm_load16(blk + 16u + c * 32u + h * 16u);
    }
    __device__ __forceinline__ void prep() {
        uint sc, mn;
        q4k_scale_min_pair(hdr.y, hdr.z, hdr.w, c, sc, mn);
        float d = f16_bits_to_f32(hdr.x & 0xFFFFu), dmin = f16_bits_to_f32(hdr.x >> 16);
        dl1 = __fmul_rn(d, (float)(sc & 0xFFu));
        ml1 = __fmul_rn(dmin, (float)(mn & 0xFFu));
        dl2 = __fmul_rn(d, (float)(sc >> 8));
        ml2 = __fmul_rn(dmin, (float)(mn >> 8));
    }
    template <int I>
    __device__ __forceinline__ void part() {
        const uint v = qs[I], l = v & 0x0F0F0F0Fu, u = (v >> 4) & 0x0F0F0F0Fu;
        float a0 = (float)(l & 0xFFu), a1 = (float)((l >> 8) & 0xFFu), a2 = (float)((l >> 16) & 0xFFu), a3 = (float)(l >> 24);
        float b0 = (float)(u & 0xFFu), b1 = (float)((u >> 8) & 0xFFu), b2 = (float)((u >> 16) & 0xFFu), b3 = (float)(u >> 24);
        lo[2 * I] = pack2(__fsub_rn(__fmul_rn(dl1, a0), ml1), __fsub_rn(__fmul_rn(dl1, a1), ml1));
        lo[2 * I + 1] = pack2(__fsub_rn(__fmul_rn(dl1, a2), ml1), __fsub_rn(__fmul_rn(dl1, a3), ml1));
        hi[2 * I] = pack2(__fsub_rn(__fmul_rn(dl2, b0), ml2), __fsub_rn(__fmul_rn(dl2, b1), ml2));
        hi[2 * I + 1] = pack2(__fsub_rn(__fmul_rn(dl2, b2), ml2), __fsub_rn(__fmul_rn(dl2, b3), ml2));
    }
    // 16 low-nibble weights -> slab columns 16h.., 16 high-nibble weights -> columns 32+16h..
    __device__ __forceinline__ void flush(uchar* lds_row, uint h) const {
        u32x4* p = (u32x4*)(lds_row + h * 32u);
        p[0] = (u32x4){lo[0], lo[1], lo[2], lo[3]};
        p[1] = (u32x4){lo[4], lo[5], lo[6], lo[7]};
        u32x4* ph = (u32x4*)(lds_row + 64u + h * 32u);
        ph[0] = (u32x4){hi[0], hi[1], hi[2], hi[3]};
        ph[1] = (u32x4){hi[4], hi[5], hi[6], hi[7]};
    }
};

// Q5_K: the Q4_K slab with a fifth bit per weight out of qh[32] (bit 2c for the low-nibble sub-block of chunk c,
// bit 2c + 1 for the high-nibble one): w = f16(d*sc * (nibble + 16 bit) - dmin*m), every operation rounded on its own
// (crates/ojas-formats/src/gguf.rs:1060-1085).  176-byte blocks: d, dmin, scales[12], qh[32], qs[128].
struct LoaderQ5K {
    static constexpr int NL = 3;
    typedef const uchar* Row;
    static __device__ __forceinline__ Row row(const GmSrc& s, uint n, uint K) { return s.w + (size_t)n * row_bytes(K); }
    u32x4 hdr, qs, qh;
    uint c;
    float dl1, ml1, dl2, ml2;
    uint lo[8], hi[8];
    static __device__ __forceinline__ size_t row_bytes(uint K) { return (size_t)(K >> 8) * Q5K_BYTES; }
    __device__ __forceinline__ void load(const uchar* row, uint k0, uint h) {
        const uchar* blk = row + (size_t)(k0 >> 8) * Q5K_BYTES;
        c = (k0 >> 6) & 3u;
        hdr = gm_load16(blk);
        qh = gm_load16(blk + 16u + h * 16u);
        qs = gm_load16(blk + 48u + c * 32u + h * 16u);
    }
    __device__ __forceinline__ void prep() {
        uint sc, mn;
        q4k_scale_min_pair(hdr.y, hdr.z, hdr.w, c, sc, mn);
        float d = f16_bits_to_f32(hdr.x & 0xFFFFu), dmin = f16_bits_to_f32(hdr.x >> 16);
        dl1 = __fmul_rn(d, (float)(sc & 0xFFu));
        ml1 = __fmul_rn(dmin, (float)(mn & 0xFFu));
        dl2 = __fmul_rn(d, (float)(sc >> 8));
        ml2 = __fmul_rn(dmin, (float)(mn >> 8));
    }
    template <int I>
    __device__ __forceinline__ void part() {
        const uint v = qs[I], b = qh[I] >> (2u * c);
        const uint l = (v & 0x0F0F0F0Fu) | ((b << 4) & 0x10101010u), u = ((v >> 4) & 0x0F0F0F0Fu) | ((b << 3) & 0x10101010u);
        float a0 = (float)(l & 0xFFu), a1 = (float)((l >> 8) & 0xFFu), a2 = (float)((l >> 16) & 0xFFu), a3 = (float)(l >> 24);
        float b0 = (float)(u & 0xFFu), b1 = (float)((u >> 8) & 0xFFu), b2 = (float)((u >> 16) & 0xFFu), b3 = (float)(u >> 24);
        lo[2 * I] = pack2(__fsub_rn(__fmul_rn(dl1, a0), ml1), __fsub_rn(__fmul_rn(dl1, a1), ml1));
        lo[2 * I + 1] = pack2(__fsub_rn(__fmul_rn(dl1, a2), ml1), __fsub_rn(__fmul_rn(dl1, a3), ml1));
        hi[2 * I] = pack2(__fsub_rn(__fmul_rn(dl2, b0), ml2), __fsub_rn(__fmul_rn(dl2, b1), ml2));
        hi[2 * I + 1] = pack2(__fsub_rn(__fmul_rn(dl2, b2), ml2), __fsub_rn(__fmul_rn(dl2, b3), ml2));
    }
    __device__ __forceinline__ void flush(uchar* lds_row, uint h) const {
        u32x4* p = (u32x4*)(lds_row + h * 32u);
        p[0] = (u32x4){lo[0], lo[1], lo[2], lo[3]};
        p[1] = (u32x4){lo[4], lo[5], lo[6], lo[7]};
        u32x4* ph = (u32x4*)(lds_row + 64u + h * 32u);
        ph[0] = (u32x4){hi[0], hi[1], hi[2], hi[3]};
        ph[1] = (u32x4){hi[4], hi[5], hi[6], hi[7]};
    }
};

// 64-column slab j of a Q6_K super-block = half hf = j/2, quarters 2(j%2) and 2(j%2)+1: thread half
// h owns columns 16h..16h+15 of each quarter (ql[16h..], ql[32+16h..], qh[16h..]), one sub-scale
// per quarter: sc[2q + h].
struct LoaderQ6K {
    static constexpr int NL = 6;
    typedef const uchar* Row;
    static __device__ __forceinline__ Row row(const GmSrc& s, uint n, uint K) { return s.w + (size_t)n * row_bytes(K); }
    u32x4 qa, qb, qh;
    uint sca, scb, d16, p;  // p = j%2: which nibble of ql and which bit pairs of qh
    float s0, s1;
    uint o0[8], o1[8];
    static __device__ __forceinline__ size_t row_bytes(uint K) { return (size_t)(K >> 8) * Q6K_BYTES; }
    __device__ __forceinline__ void load(const uchar* row, uint k0, uint h) {
        const uchar* blk = row + (size_t)(k0 >> 8) * Q6K_BYTES;
        uint j = (k0 >> 6) & 3u, hf = j >> 1;
        p = j & 1u;
        qa = gm_load16(blk + hf * 64u + h * 16u);
        qb = gm_load16(blk + hf * 64u + 32u + h * 16u);
        qh = gm_load16(blk + 128u + hf * 32u + h * 16u);
        const uchar* sc = blk + 192u + hf * 8u + p * 4u + h;
        sca = gm_load_u8(sc);
        scb = gm_load_u8(sc + 2);
        d16 = gm_load_u16(blk + 208u);
    }
    __device__ __forceinline__ void prep() {
        float d = f16_bits_to_f32(d16);
        s0 = __fmul_rn(d, (float)(signed char)sca);
        s1 = __fmul_rn(d, (float)(signed char)scb);
    }
    template <int I>
    __device__ __forceinline__ void part() {
        // low 4 bits: nibble p of ql; high 2 bits: bits 4p..4p+1 (first quarter) / 4p+2..4p+3 of qh
        const uint a = (qa[I] >> (4u * p)) & 0x0F0F0F0Fu, b = (qb[I] >> (4u * p)) & 0x0F0F0F0Fu;
        const uint h = qh[I] >> (4u * p);
        const uint w0 = a | ((h << 4) & 0x30303030u), w1 = b | ((h << 2) & 0x30303030u);
        float e0[4], e1[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            e0[e] = __fmul_rn(s0, (float)((int)((w0 >> (8 * e)) & 0xFFu) - 32));
            e1[e] = __fmul_rn(s1, (float)((int)((w1 >> (8 * e)) & 0xFFu) - 32));
        }
        o0[2 * I] = pack2(e0[0], e0[1]);
        o0[2 * I + 1] = pack2(e0[2], e0[3]);
        o1[2 * I] = pack2(e1[0], e1[1]);
        o1[2 * I + 1] = pack2(e1[2], e1[3]);
    }
    __device__ __forceinline__ void flush(uchar* lds_row, uint h) const {
        u32x4* q = (u32x4*)(lds_row + h * 32u);
        q[0] = (u32x4){o0[0], o0[1], o0[2], o0[3]};
        q[1] = (u32x4){o0[4], o0[5], o0[6], o0[7]};
        u32x4* qh_ = (u32x4*)(lds_row + 64u + h * 32u);
        qh_[0] = (u32x4){o1[0], o1[1], o1[2], o1[3]};
        qh_[1] = (u32x4){o1[4], o1[5], o1[6], o1[7]};
    }
};

// The slab's two Q8_0 blocks: thread half h owns block h = slab columns 32h..32h+31.
struct LoaderQ80 {
    static constexpr int NL = 3;
    typedef const uchar* Row;
    static __device__ __forceinline__ Row row(const GmSrc& s, uint n, uint K) { return s.w + (size_t)n * row_bytes(K); }
    u32x4 qa, qb;
    uint d16;
    float d;
    uint o[16];
    static __device__ __forceinline__ size_t row_bytes(uint K) { return (size_t)(K >> 5) * Q80_BYTES; }
    __device__ __forceinline__ void load(const uchar* row, uint k0, uint h) {
        const uchar* blk = row + (size_t)((k0 >> 5) + h) * Q80_BYTES;
        d16 = gm_load_u16(blk);
        qa = gm_load16(blk + 2u);
        qb = gm_load16(blk + 18u);
    }
    __device__ __forceinline__ void prep() { d = f16_bits_to_f32(d16); }
    template <int I>
    __device__ __forceinline__ void part() {
#pragma unroll
        for (int s = 0; s < 2; s++) {
            const uint q = s ? qb[I] : qa[I];
            float v0 = __fmul_rn(d, (float)(signed char)(q)), v1 = __fmul_rn(d, (float)(signed char)(q >> 8));
            float v2 = __fmul_rn(d, (float)(signed char)(q >> 16)), v3 = __fmul_rn(d, (float)((int)q >> 24));
            o[8 * s + 2 * I] = pack2(v0, v1);
            o[8 * s + 2 * I + 1] = pack2(v2, v3);
        }
    }
    __device__ __forceinline__ void flush(uchar* lds_row, uint h) const {
        u32x4* q = (u32x4*)(lds_row + h * 64u);
#pragma unroll
        for (int i = 0; i < 4; i++) q[i] = (u32x4){o[4 * i], o[4 * i + 1], o[4 * i + 2], o[4 * i + 3]};
    }
};

// IQ4_NL: an 18-byte block = f16 d + 16 bytes of 4-bit indices into the sixteen non-linear levels; weight j < 16 is
// the low nibble of byte j, weight 16 + j its high nibble; value f16(d * level), the bits of `dequant_iq4nl_f16`
// (crates/ojas-formats/src/gguf.rs:796-812).  Thread half h owns block h of the slab = columns 32h..32h+31.
struct LoaderIQ4NL {
    static constexpr int NL = 2;
    typedef const uchar* Row;
    static __device__ __forceinline__ Row row(const GmSrc& s, uint n, uint K) { return s.w + (size_t)n * row_bytes(K); }
    u32x4 q;
    uint d16;
    float d;
    uint o[16];
    static __device__ __forceinline__ size_t row_bytes(uint K) { return (size_t)(K >> 5) * IQ4NL_BYTES; }
    __device__ __forceinline__ void load(const uchar* row, uint k0, uint h) {
        const uchar* blk = row + (size_t)((k0 >> 5) + h) * IQ4NL_BYTES;
        d16 = gm_load_u16(blk);
        q = gm_load16(blk + 2u);
    }
    __device__ __forceinline__ void prep() { d = f16_bits_to_f32(d16); }
    template <int I>
    __device__ __forceinline__ void part() {
#pragma unroll
        for (int s = 0; s < 2; s++) {
            const uint lv = iq4_levels4((q[I] >> (4 * s)) & 0x0F0F0F0Fu);
            float v0 = __fmul_rn(d, (float)(signed char)(lv)), v1 = __fmul_rn(d, (float)(signed char)(lv >> 8));
            float v2 = __fmul_rn(d, (float)(signed char)(lv >> 16)), v3 = __fmul_rn(d, (float)((int)lv >> 24));
            o[8 * s + 2 * I] = pack2(v0, v1);
            o[8 * s + 2 * I + 1] = pack2(v2, v3);
        }
    }
    __device__ __forceinline__ void flush(uchar* lds_row, uint h) const {
        u32x4* p = (u32x4*)(lds_row + h * 64u);
#pragma unroll
        for (int i = 0; i < 4; i++) p[i] = (u32x4){o[4 * i], o[4 * i + 1], o[4 * i + 2], o[4 * i + 3]};
    }
};

// IQ4_XS: a 136-byte super-block of 256 = f16 d, 16 bits of scale high pairs, 4 bytes of scale low nibbles, 128 bytes
// of indices (sub-block ib of 32: bytes 16 ib .., nibbles laid out as in IQ4_NL); value f16((d * (ls - 32)) * level),
// the bits of `dequant_iq4xs_f16` (crates/ojas-formats/src/gguf.rs:814-838).  Thread half h owns sub-block
// (k0 / 32 + h) % 8 of super-block k0 / 256; rows are whole super-blocks (K a multiple of 256).
struct LoaderIQ4XS {
    static constexpr int NL = 3;
    typedef const uchar* Row;
    static __device__ __forceinline__ Row row(const GmSrc& s, uint n, uint K) { return s.w + (size_t)n * row_bytes(K); }
    u32x4 q;
    uint h0, sl, ib;
    float d;
    uint o[16];
    static __device__ __forceinline__ size_t row_bytes(uint K) { return (size_t)(K >> 8) * IQ4XS_BYTES; }
    __device__ __forceinline__ void load(const uchar* row, uint k0, uint h) {
        const uchar* blk = row + (size_t)(k0 >> 8) * IQ4XS_BYTES;      // 136-byte blocks: 8-byte aligned with the tensor
        ib = ((k0 >> 5) & 7u) + h;
        h0 = *(const uint*)blk;
        sl = *(const uint*)(blk + 4u);
        q = gm_load16(blk + 8u + 16u * ib);
    }
    __device__ __forceinline__ void prep() {
        const uint ls = ((sl >> (4u * ib)) & 0xFu) | ((((h0 >> 16) >> (2u * ib)) & 3u) << 4);
        d = __fmul_rn(f16_bits_to_f32(h0 & 0xFFFFu), (float)((int)ls - 32));
    }
    template <int I>
    __device__ __forceinline__ void part() {
#pragma unroll
        for (int s = 0; s < 2; s++) {
            const uint lv = iq4_levels4((q[I] >> (4 * s)) & 0x0F0F0F0Fu);
            float v0 = __fmul_rn(d, (float)(signed char)(lv)), v1 = __fmul_rn(d, (float)(signed char)(lv >> 8));
            float v2 = __fmul_rn(d, (float)(signed char)(lv >> 16)), v3 = __fmul_rn(d, (float)((int)lv >> 24));
            o[8 * s + 2 * I] = pack2(v0, v1);
            o[8 * s + 2 * I + 1] = pack2(v2, v3);
        }
    }
    __device__ __forceinline__ void flush(uchar* lds_row, uint h) const {
        u32x4* p = (u32x4*)(lds_row + h * 64u);
#pragma unroll
        for (int i = 0; i < 4; i++) p[i] = (u32x4){o[4 * i], o[4 * i + 1], o[4 * i + 2], o[4 * i + 3]};
    }
};

// The legacy 32-weight blocks Q4_0 / Q4_1 / Q5_0 / Q5_1: {f16 d [, f16 m]} [4 bytes of fifth bits] 16 bytes of nibbles;
// weight j < 16 is the low nibble of byte j, weight 16 + j its high nibble, fifth bit = bit (weight index) of the
// 4-byte field.  AFFINE: w = d * q + m (a product and a sum, each rounded), else w = d * (q - 8 | 16) — the bits of
// `dequant_q{40,41,50,51}_f16` (crates/ojas-formats/src/gguf.rs:653-700).  Thread half h owns block h of the slab.
template <bool FIVE, bool AFFINE>
struct LoaderLegacy {
    static constexpr int NL = 2 + (FIVE ? 1 : 0);
    static constexpr uint BYTES = 18u + (AFFINE ? 2u : 0u) + (FIVE ? 4u : 0u), HDR = AFFINE ? 4u : 2u;
    typedef const uchar* Row;
    static __device__ __forceinline__ Row row(const GmSrc& s, uint n, uint K) { return s.w + (size_t)n * row_bytes(K); }
    u32x4 q;
    uint hdr, qh;
    float d, m;
    uint o[16];
    static __device__ __forceinline__ size_t row_bytes(uint K) { return (size_t)(K >> 5) * BYTES; }
    __device__ __forceinline__ void load(const uchar* row, uint k0, uint h) {
        const uchar* blk = row + (size_t)((k0 >> 5) + h) * BYTES;
        typedef uint __attribute__((aligned(2))) u32_u;
        if (AFFINE) hdr = *(const u32_u*)blk;
        else hdr = gm_load_u16(blk);
        qh = 0u;
        if (FIVE) qh = *(const u32_u*)(blk + HDR);
        q = gm_load16(blk + HDR + (FIVE ? 4u : 0u));
    }
    __device__ __forceinline__ void prep() {
        d = f16_bits_to_f32(hdr & 0xFFFFu);
        m = AFFINE ? f16_bits_to_f32(hdr >> 16) : 0.0f;
    }
    __device__ __forceinline__ float value(uint code) const {
        if (AFFINE) return __fadd_rn(__fmul_rn(d, (float)code), m);
        return __fmul_rn(d, __fsub_rn((float)code, FIVE ? 16.0f : 8.0f));
    }
    template <int I>
    __device__ __forceinline__ void part() {
#pragma unroll
        for (int s = 0; s < 2; s++) {
            uint nib = (q[I] >> (4 * s)) & 0x0F0F0F0Fu;
            if (FIVE) {
                const uint f = qh >> (16 * s + 4 * I);      // bits 0..3: the four weights of this dword and nibble half
                nib |= ((f & 1u) << 4) | ((f & 2u) << 11) | ((f & 4u) << 18) | ((f & 8u) << 25);
            }
            o[8 * s + 2 * I] = pack2(value(nib & 0xFFu), value((nib >> 8) & 0xFFu));
            o[8 * s + 2 * I + 1] = pack2(value((nib >> 16) & 0xFFu), value(nib >> 24));
        }
    }
    __device__ __forceinline__ void flush(uchar* lds_row, uint h) const {
        u32x4* p = (u32x4*)(lds_row + h * 64u);
#pragma unroll
        for (int i = 0; i < 4; i++) p[i] = (u32x4){o[4 * i], o[4 * i + 1], o[4 * i + 2], o[4 * i + 3]};
    }
};

// MXFP4 (crates/ojas-formats/src/mxfp4.rs:40-58): a 17-byte block { u8 e; u8 qs[16] }, w = 2^(e - 127) * E2M1[code],
// weight 2j the low and 2j + 1 the high nibble of qs[j]: consecutive weights sit in consecutive nibbles.  The bits of
// `dequant_mxfp4_f16`.  Blocks start at any byte.
struct LoaderMXFP4 {
    static constexpr int NL = 3;
    typedef const uchar* Row;
    static __device__ __forceinline__ Row row(const GmSrc& s, uint n, uint K) { return s.w + (size_t)n * row_bytes(K); }
    u32x4 q;
    uint e8, q4, sh;
    float d;
    uint o[16];
    static __device__ __forceinline__ size_t row_bytes(uint K) { return (size_t)(K >> 5) * 17u; }
    __device__ __forceinline__ void load(const uchar* row, uint k0, uint h) {
        const uchar* blk = row + (size_t)((k0 >> 5) + h) * 17u;
        // the 16 code bytes start at any byte: the aligned dwords around them, shifted into place after the wait (a
        // byte-aligned 16-byte load is split into narrow ones).  The fifth dword holds code bytes whenever it is used.
        typedef u32x4 __attribute__((aligned(4))) u32x4_a4;
        const uchar* cb = blk + 1u;
        sh = (uint)((size_t)cb & 3u);
        const uchar* al = cb - sh;
        e8 = gm_load_u8(blk);
        q = *(const u32x4_a4*)al;
        q4 = *(const uint*)(al + (sh ? 16u : 12u));
    }
    __device__ __forceinline__ void prep() {
        d = __uint_as_float(e8 << 23);
        const uint a0 = q[0], a1 = q[1], a2 = q[2], a3 = q[3];
        q[0] = __builtin_amdgcn_alignbyte(a1, a0, sh);
        q[1] = __builtin_amdgcn_alignbyte(a2, a1, sh);
        q[2] = __builtin_amdgcn_alignbyte(a3, a2, sh);
        q[3] = __builtin_amdgcn_alignbyte(q4, a3, sh);
    }
    // four codes (one per byte) -> twice their E2M1 values as signed bytes (0 1 2 3 4 6 8 12 and their negatives): two
    // byte permutes over the halves of the table, merged by the sign bit.  (Code 8, -0, comes out as +0: the same
    // product in every sum.)  d/2 * level is exact, so the one rounding to f16 is the decoder's.
    static __device__ __forceinline__ uint levels4(uint idx4) {
        const uint sel = idx4 & 0x07070707u;
        const uint pos = __builtin_amdgcn_perm(0x0C080604u, 0x03020100u, sel);
        const uint neg = __builtin_amdgcn_perm(0xF4F8FAFCu, 0xFDFEFF00u, sel);
        const uint m1 = (idx4 >> 3) & 0x01010101u;
        const uint mask = (m1 << 8) - m1;
        return (neg & mask) | (pos & ~mask);
    }
    template <int I>
    __device__ __forceinline__ void part() {      // dword I: weights 8 I .. 8 I + 7, nibble by nibble
        const float dh = __fmul_rn(d, 0.5f);
        const uint lo = levels4(q[I] & 0x0F0F0F0Fu), hi = levels4((q[I] >> 4) & 0x0F0F0F0Fu);
        o[4 * I] = pack2(__fmul_rn(dh, (float)(signed char)lo), __fmul_rn(dh, (float)(signed char)hi));
        o[4 * I + 1] = pack2(__fmul_rn(dh, (float)(signed char)(lo >> 8)), __fmul_rn(dh, (float)(signed char)(hi >> 8)));
        o[4 * I + 2] = pack2(__fmul_rn(dh, (float)(signed char)(lo >> 16)), __fmul_rn(dh, (float)(signed char)(hi >> 16)));
        o[4 * I + 3] = pack2(__fmul_rn(dh, (float)((int)lo >> 24)), __fmul_rn(dh, (float)((int)hi >> 24)));
    }
    __device__ __forceinline__ void flush(uchar* lds_row, uint h) const {
        u32x4* p = (u32x4*)(lds_row + h * 64u);
#pragma unroll
        for (int i = 0; i < 4; i++) p[i] = (u32x4){o[4 * i], o[4 * i + 1], o[4 * i + 2], o[4 * i + 3]};
    }
};

// Q2_K and Q3_K keep four 2-bit planes per byte: within a half of 128 weights, byte l of the half's 32 code bytes holds
// weights l, l + 32, l + 64, l + 96 at bits 0, 2, 4, 6, and scale 8 half + 2 j + l / 16 covers (plane j, l / 16).  The
// thread's 32 consecutive weights are one plane of one half: s = (k0 / 32 + h) % 8, half = s / 4, j = s % 4 — all 32 code
// bytes of the half at bits 2 j.  Rows are whole super-blocks (K a multiple of 256).
// Q2_K: w = (d * sc) * q - dmin * m, every step rounded — the bits of `dequant_q2k_f16`
// (crates/ojas-formats/src/gguf.rs:730-754).
struct LoaderQ2K {
    static constexpr int NL = 4;
    typedef const uchar* Row;
    static __device__ __forceinline__ Row row(const GmSrc& s, uint n, uint K) { return s.w + (size_t)n * row_bytes(K); }
    u32x4 qa, qb;
    uint sc2, dd, j;
    float dl[2], ml[2];
    uint o[16];
    static __device__ __forceinline__ size_t row_bytes(uint K) { return (size_t)(K >> 8) * Q2K_BYTES; }
    __device__ __forceinline__ void load(const uchar* row, uint k0, uint h) {
        const uchar* blk = row + (size_t)(k0 >> 8) * Q2K_BYTES;       // 84-byte blocks: 4-byte aligned with the tensor
        const uint s = ((k0 >> 5) & 7u) + h, half = s >> 2;
        j = s & 3u;
        sc2 = gm_load_u16(blk + half * 8u + j * 2u);
        dd = *(const uint*)(blk + 80u);
        typedef u32x4 __attribute__((aligned(4))) u32x4_a4;
        qa = *(const u32x4_a4*)(blk + 16u + half * 32u);
        qb = *(const u32x4_a4*)(blk + 32u + half * 32u);
    }
    __device__ __forceinline__ void prep() {
        const float d = f16_bits_to_f32(dd & 0xFFFFu), dmin = f16_bits_to_f32(dd >> 16);
#pragma unroll
        for (int g = 0; g < 2; g++) {
            const uint sc = (sc2 >> (8 * g)) & 0xFFu;
            dl[g] = __fmul_rn(d, (float)(sc & 0xFu));
            ml[g] = __fmul_rn(dmin, (float)(sc >> 4));
        }
    }
    template <int I>
    __device__ __forceinline__ void part() {      // weights 8 I .. 8 I + 7 of the 32: code bytes 8 I .. of the half
        const float a = dl[I >> 1], b = ml[I >> 1];
#pragma unroll
        for (int v = 0; v < 2; v++) {
            const uint q = ((I < 2 ? qa : qb)[2 * (I & 1) + v] >> (2u * j)) & 0x03030303u;
            o[4 * I + 2 * v] = pack2(__fsub_rn(__fmul_rn(a, (float)(q & 0xFFu)), b), __fsub_rn(__fmul_rn(a, (float)((q >> 8) & 0xFFu)), b));
            o[4 * I + 2 * v + 1] = pack2(__fsub_rn(__fmul_rn(a, (float)((q >> 16) & 0xFFu)), b), __fsub_rn(__fmul_rn(a, (float)(q >> 24)), b));
        }
    }
    __device__ __forceinline__ void flush(uchar* lds_row, uint h) const {
        u32x4* p = (u32x4*)(lds_row + h * 64u);
#pragma unroll
        for (int i = 0; i < 4; i++) p[i] = (u32x4){o[4 * i], o[4 * i + 1], o[4 * i + 2], o[4 * i + 3]};
    }
};

// Q3_K: block { u8 hmask[32]; u8 qs[64]; u8 scales[12]; half d; } of 110 bytes (two-byte alignment only);
// w = (d * (sc - 32)) * (q - (mask bit ? 0 : 4)), bit 4 half + j of hmask[l] belonging to weight (half, j, l) — the bits
// of `dequant_q3k_f16` (crates/ojas-formats/src/gguf.rs:755-795).
struct LoaderQ3K {
    static constexpr int NL = 8;
    typedef const uchar* Row;
    static __device__ __forceinline__ Row row(const GmSrc& s, uint n, uint K) { return s.w + (size_t)n * row_bytes(K); }
    u32x4 qa, qb, ha, hb;
    uint r0, r1, r2, d16, s;
    float dl[2];
    uint o[16];
    static __device__ __forceinline__ size_t row_bytes(uint K) { return (size_t)(K >> 8) * Q3K_BYTES; }
    __device__ __forceinline__ void load(const uchar* row, uint k0, uint h) {
        const uchar* blk = row + (size_t)(k0 >> 8) * Q3K_BYTES;
        s = ((k0 >> 5) & 7u) + h;
        const uint half = s >> 2;
        ha = gm_load16(blk);
        hb = gm_load16(blk + 16u);
        qa = gm_load16(blk + 32u + half * 32u);
        qb = gm_load16(blk + 48u + half * 32u);
        r0 = *(const u32_a2*)(blk + 96u);
        r1 = *(const u32_a2*)(blk + 100u);
        r2 = *(const u32_a2*)(blk + 104u);
        d16 = gm_load_u16(blk + 108u);
    }
    __device__ __forceinline__ void prep() {
        const float d = f16_bits_to_f32(d16);
        const uint half = s >> 2, j = s & 3u;
#pragma unroll
        for (int g = 0; g < 2; g++) dl[g] = __fmul_rn(d, (float)q3k_scale6(r0, r1, r2, half * 8u + j * 2u + (uint)g));
    }
    __device__ __forceinline__ float value(float a, uint c) const { return __fmul_rn(a, __fsub_rn((float)c, 4.0f)); }
    template <int I>
    __device__ __forceinline__ void part() {
        const float a = dl[I >> 1];
        const uint j = s & 3u, sh = (s >> 2) * 4u + j;
#pragma unroll
        for (int v = 0; v < 2; v++) {
            const uint q = ((I < 2 ? qa : qb)[2 * (I & 1) + v] >> (2u * j)) & 0x03030303u;
            const uint hm = ((I < 2 ? ha : hb)[2 * (I & 1) + v] >> sh) & 0x01010101u;
            const uint c = q | (hm << 2);       // 0..7 per byte: the weight is c - 4 (an exact difference, then the decoder's one product)
            o[4 * I + 2 * v] = pack2(value(a, c & 0xFFu), value(a, (c >> 8) & 0xFFu));
            o[4 * I + 2 * v + 1] = pack2(value(a, (c >> 16) & 0xFFu), value(a, c >> 24));
        }
    }
    __device__ __forceinline__ void flush(uchar* lds_row, uint h) const {
        u32x4* p = (u32x4*)(lds_row + h * 64u);
#pragma unroll
        for (int i = 0; i < 4; i++) p[i] = (u32x4){o[4 * i], o[4 * i + 1], o[4 * i + 2], o[4 * i + 3]};
    }
};

// Plain f16 rows [N][K] (a tensor the caller keeps in f16, or any block format decoded into scratch by its
// `dequant_<fmt>_f16` kernel ahead of the product): thread half h owns columns 32h..32h+31 of the slab, 64 bytes.
struct LoaderF16 {
    static constexpr int NL = 4;
    typedef const uchar* Row;
    static __device__ __forceinline__ Row row(const GmSrc& s, uint n, uint K) { return s.w + (size_t)n * row_bytes(K); }
    u32x4 q[4];
    static __device__ __forceinline__ size_t row_bytes(uint K) { return (size_t)K * 2u; }
    __device__ __forceinline__ void load(const uchar* row, uint k0, uint h) {
        const uchar* p = row + (size_t)(k0 + 32u * h) * 2u;
#pragma unroll
        for (int i = 0; i < 4; i++) q[i] = *(const u32x4*)(p + 16 * i);
    }
    __device__ __forceinline__ void prep() {}
    template <int I>
    __device__ __forceinline__ void part() {}
    __device__ __forceinline__ void flush(uchar* lds_row, uint h) const {
        u32x4* o = (u32x4*)(lds_row + h * 64u);
#pragma unroll
        for (int i = 0; i < 4; i++) o[i] = q[i];
    }
};

// Q4L: Q4_K relaid by `relayout_q4k_q4l` (crates/ojas-formats/src/quant.rs:192-222) — nibbles w4[N][K/2], byte i of a
// 32-weight block = weights 2i (low nibble) and 2i+1 (high), and per block the f16 pair qa = d*sc, qb = -dmin*m.  Every
// weight enters the tile as the binary16 fma qa*q + qb, the arithmetic of the reference's `gemm_mm_q4l`
// (crates/ojas-cuda/src/kernels/gemm_q.rs:104-142).  Thread half h owns block h of the slab = columns 32h..32h+31.
struct LoaderQ4L {
    static constexpr int NL = 3;
    struct Row { const uchar* w; const ushort* qa; const ushort* qb; };
    static __device__ __forceinline__ Row row(const GmSrc& s, uint n, uint K) {
        return {s.w + (size_t)n * (K >> 1), s.qa + (size_t)n * (K >> 5), s.qb + (size_t)n * (K >> 5)};
    }
    u32x4 nib;
    uint a16, c16;
    half2v a2, c2;
    uint o[16];
    __device__ __forceinline__ void load(const Row& r, uint k0, uint h) {
        nib = gm_load16(r.w + (k0 >> 1) + h * 16u);
        a16 = gm_load_u16(r.qa + (k0 >> 5) + h);
        c16 = gm_load_u16(r.qb + (k0 >> 5) + h);
    }
    __device__ __forceinline__ void prep() {
        const _Float16 a = __builtin_bit_cast(_Float16, (ushort)a16), c = __builtin_bit_cast(_Float16, (ushort)c16);
        a2 = (half2v){a, a};
        c2 = (half2v){c, c};
    }
    template <int I>
    __device__ __forceinline__ void part() {
        const half2v k1024 = {(_Float16)1024.0f, (_Float16)1024.0f};
        const uint u = nib[I];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint by = (u >> (8 * j)) & 0xFFu;
            // the nibbles as the halves 1024 + q, then q exactly, then one rounding in the fma
            const uint hbits = 0x64006400u | (by & 0x0Fu) | ((by & 0xF0u) << 12);
            const half2v q = __builtin_bit_cast(half2v, hbits) - k1024;
            o[4 * I + j] = __builtin_bit_cast(uint, __builtin_elementwise_fma(q, a2, c2));
        }
    }
    __device__ __forceinline__ void flush(uchar* lds_row, uint h) const {
        u32x4* q = (u32x4*)(lds_row + h * 64u);
#pragma unroll
        for (int i = 0; i < 4; i++) q[i] = (u32x4){o[4 * i], o[4 * i + 1], o[4 * i + 2], o[4 * i + 3]};
    }
};

// ------------------------------------------------------------------ the tile
// XF32: the activations arrive as f32 [M][K] and are rounded to f16 on their way into the tile (the reference's plain
// entries); each slab's loads are then consumed where they are issued, which is correct but not pipelined — callers
// that care convert once (copy_f32_half) and take the f16 entries, as the reference's own `mm` does for split-K.
// MI: 32-token blocks per wave along M — the tile is 64 MI tokens x 128 rows: 4 (256 tokens), or 2 for batches of up to 128
// tokens, which would leave half of the taller tile's matrix instructions multiplying padding.
// which row of x and of y token m of the launch is: itself, or (grouped expert products) an entry of a list — the
// activation row that entry divided by DIV (an assignment's token), the output row the entry itself
struct GmDense {
    __device__ __forceinline__ uint in_row(uint m) const { return m; }
    __device__ __forceinline__ uint out_row(uint m) const { return m; }
};
struct GmList {
    const uint* lst;
    uint last, div;
    __device__ __forceinline__ uint out_row(uint m) const { return min(lst[m], last); }
    __device__ __forceinline__ uint in_row(uint m) const { return out_row(m) / div; }
};
template <class Loader, bool SPLITK, bool XF32 = false, int MI = 4, class TM = GmDense>
__device__ __forceinline__ void gemm_mm_body(const void* __restrict__ xv, const GmSrc src,
                                             float* __restrict__ y, uint K, uint N, uint accum, uint M, uint nsplit,
                                             const TM tm = TM(), uint ty = blockIdx.y) {
    const ushort* xh = (const ushort*)xv;
    const float* xf = (const float*)xv;
    constexpr uint BM = 64u * MI, STAGE = (BM + GM_BN) * GM_STRIDE, NX = 2u * MI;   // NX: activation rows per thread and slab
    __shared__ __attribute__((aligned(16))) uchar lds[2 * STAGE];
    const uint tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint n0 = blockIdx.x * GM_BN, m0 = ty * BM;
    // this block's K range (whole multiples of 64)
    uint k_begin = 0, k_end = K;
    if (SPLITK) {
        uint steps = K / GM_BK, per = (steps + nsplit - 1) / nsplit;
        k_begin = min(blockIdx.z * per, steps) * GM_BK;
        k_end = min((blockIdx.z + 1) * per, steps) * GM_BK;
        if (k_begin >= k_end) return;
    }
    // staging roles
    const uint xr = tid >> 3, xc = (tid & 7u) * 8u;  // activation slab: rows xr + 32 i, 8 f16 at column xc
    const uint wr = tid >> 1, wh = tid & 1u;         // weight slab: row wr, half wh
    const typename Loader::Row wrow = Loader::row(src, min(n0 + wr, N - 1u), K);
    size_t xrow[NX];   // element offset of the thread's 8 activations in each of its rows
#pragma unroll
    for (int i = 0; i < (int)NX; i++) xrow[i] = (size_t)tm.in_row(min(m0 + xr + 32u * i, M - 1u)) * K + xc;
    const uint x_lds = xr * GM_STRIDE + xc * 2u;                   // + i * 32 rows
    const uint w_lds = BM * GM_STRIDE + wr * GM_STRIDE;

    // wave tile: 32 MI (m) x 64 (n)
    const uint wm = (wave >> 1) * (32u * MI), wn = (wave & 1u) * 64u;
    const uint fr = lane & 31u, kg = lane >> 5;
    const uint a_lds = (wm + fr) * GM_STRIDE + kg * 16u;           // + i * 32 rows, + ks * 32 bytes
    const uint b_lds = BM * GM_STRIDE + (wn + fr) * GM_STRIDE + kg * 16u;
    float16v acc[MI][2];
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;

    u32x4 xs0[NX], xs1[NX], xs2[NX];
    Loader ld0, ld1, ld2;
    const uint nt = (k_end - k_begin) / GM_BK;

#define GM_LOAD(XS, LD, T)                                                                       \
    do {                                                                                         \
        const uint kk_ = k_begin + (T) * GM_BK;                                                  \
        _Pragma("unroll") for (int i_ = 0; i_ < (int)NX; i_++) XS[i_] = gm_load_x<XF32>(xh, xf, xrow[i_] + kk_); \
        LD.load(wrow, kk_, wh);                                                                  \
        gm_fence();                                                                              \
    } while (0)
#define GM_STORE_X(XS, STG)                                                                      \
    do {                                                                                         \
        uchar* a_ = lds + (STG) * STAGE + x_lds;                                                 \
        _Pragma("unroll") for (int i_ = 0; i_ < (int)NX; i_++) *(u32x4*)(a_ + i_ * 32u * GM_STRIDE) = XS[i_]; \
    } while (0)
// fragments of K sub-step KS of stage STG into registers AF/BF; the MFMAs that consume them
#define GM_READ(STG, KS, AF, BF)                                                                 \
    do {                                                                                         \
        const uchar* s_ = lds + (STG) * STAGE;                                                   \
        _Pragma("unroll") for (int i = 0; i < MI; i++)                                            \
            AF[i] = *(const half8*)(s_ + a_lds + i * 32u * GM_STRIDE + (KS) * 32u);              \
        _Pragma("unroll") for (int j = 0; j < 2; j++)                                            \
            BF[j] = *(const half8*)(s_ + b_lds + j * 32u * GM_STRIDE + (KS) * 32u);              \
    } while (0)
#define GM_MMA(AF, BF)                                                                           \
    do {                                                                                         \
        _Pragma("unroll") for (int i = 0; i < MI; i++)                                           \
            _Pragma("unroll") for (int j = 0; j < 2; j++)                                        \
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(AF[i], BF[j], acc[i][j], 0, 0, 0); \
    } while (0)
#define GM_MFMA(STG, KS)                                                                         \
    do {                                                                                         \
        half8 af_[MI], bf_[2];                                                                    \
        GM_READ(STG, KS, af_, bf_);                                                              \
        GM_MMA(af_, bf_);                                                                        \
    } while (0)
// interleave: one MFMA, one LDS read (the next sub-step's fragments), a few vector-ALU
// instructions (the next step's dequantization) — once per matrix instruction of the sub-step
#define GM_MIX()                                                                                 \
    do {                                                                                         \
        _Pragma("unroll") for (int g_ = 0; g_ < 2 * MI; g_++) {                                  \
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                   \
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);                                   \
            __builtin_amdgcn_sched_group_barrier(0x002, MI == 4 ? 5 : 10, 0);                                   \
        }                                                                                        \
    } while (0)
// Interior step T (steps T+1 .. T+3 exist): no branches, so MFMAs and dequantization share one
// scheduling region.  Fragments are read one sub-step ahead of the MFMAs that use them.
#define GM_STEP_FULL(T, XS_FREE, LD_FREE, XS_NEXT, LD_NEXT)                                      \
    do {                                                                                         \
        const uint cur_ = (T) & 1u, nxt_ = cur_ ^ 1u;                                            \
        half8 afA[MI], bfA[2], afB[MI], bfB[2];                                                    \
        GM_READ(cur_, 0, afA, bfA);                                                              \
        GM_LOAD(XS_FREE, LD_FREE, (T) + 3u);                                                     \
        LD_NEXT.prep();                                                                          \
        GM_READ(cur_, 1, afB, bfB); GM_MMA(afA, bfA); LD_NEXT.template part<0>(); GM_MIX();      \
        GM_READ(cur_, 2, afA, bfA); GM_MMA(afB, bfB); LD_NEXT.template part<1>(); GM_MIX();      \
        GM_READ(cur_, 3, afB, bfB); GM_MMA(afA, bfA); LD_NEXT.template part<2>(); GM_MIX();      \
        GM_MMA(afB, bfB); LD_NEXT.template part<3>(); GM_MIX();                                  \
        GM_STORE_X(XS_NEXT, nxt_);                                                               \
        LD_NEXT.flush(lds + nxt_ * STAGE + w_lds, wh);                                           \
        __syncthreads();                                                                         \
    } while (0)
// Guarded step for the head and tail of the K range.
#define GM_STEP_ANY(T, XS_FREE, LD_FREE, XS_NEXT, LD_NEXT)                                       \
    do {                                                                                         \
        if ((T) + 3u < nt) GM_LOAD(XS_FREE, LD_FREE, (T) + 3u);                                  \
        const uint cur_ = (T) & 1u, nxt_ = cur_ ^ 1u;                                            \
        GM_MFMA(cur_, 0); GM_MFMA(cur_, 1); GM_MFMA(cur_, 2); GM_MFMA(cur_, 3);                  \
        if ((T) + 1u < nt) {                                                                     \
            LD_NEXT.prep();                                                                      \
            LD_NEXT.template part<0>(); LD_NEXT.template part<1>();                              \
            LD_NEXT.template part<2>(); LD_NEXT.template part<3>();                              \
            GM_STORE_X(XS_NEXT, nxt_);                                                           \
            LD_NEXT.flush(lds + nxt_ * STAGE + w_lds, wh);                                       \
        }                                                                                        \
        __syncthreads();                                                                         \
    } while (0)

    GM_LOAD(xs0, ld0, 0u);
    if (nt > 1u) GM_LOAD(xs1, ld1, 1u);
    if (nt > 2u) GM_LOAD(xs2, ld2, 2u);
    ld0.prep();
    ld0.template part<0>(); ld0.template part<1>(); ld0.template part<2>(); ld0.template part<3>();
    GM_STORE_X(xs0, 0u);
    ld0.flush(lds + w_lds, wh);
    __syncthreads();

    uint t = 0;
    for (; t + 6u <= nt; t += 3u) {  // steps t, t+1, t+2 all have three successors
        GM_STEP_FULL(t, xs0, ld0, xs1, ld1);
        GM_STEP_FULL(t + 1u, xs1, ld1, xs2, ld2);
        GM_STEP_FULL(t + 2u, xs2, ld2, xs0, ld0);
    }
    for (; t < nt; t += 3u) {
        GM_STEP_ANY(t, xs0, ld0, xs1, ld1);
        if (t + 1u < nt) GM_STEP_ANY(t + 1u, xs1, ld1, xs2, ld2);
        if (t + 2u < nt) GM_STEP_ANY(t + 2u, xs2, ld2, xs0, ld0);
    }
#undef GM_LOAD
#undef GM_STORE_X
#undef GM_MFMA
#undef GM_READ
#undef GM_MMA
#undef GM_MIX
#undef GM_STEP_FULL
#undef GM_STEP_ANY

    // epilogue: D register v of block (i, j) holds row 8*(v/4) + 4*kg + v%4, column fr
#pragma unroll
    for (int i = 0; i < MI; i++) {
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const uint n = n0 + wn + 32u * j + fr;
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const uint m = m0 + wm + 32u * i + 8u * (v >> 2) + 4u * kg + (v & 3u);
                if (m < M && n < N) {
                    float* o = y + (size_t)tm.out_row(m) * N + n;
                    if (SPLITK) atomicAdd(o, acc[i][j][v]);
                    else *o = accum ? *o + acc[i][j][v] : acc[i][j][v];
                }
            }
        }
    }
}

// `_m128`: the 128-token tile, grid [ceil(N/128), ceil(M/128), nsplit]
#define GEMM_ENTRIES(FMT, LOADER)                                                                                 \
    extern "C" __global__ void __launch_bounds__(256) gemm_mm_##FMT(                                              \
        const ushort* xh, const uchar* w, float* y, uint K, uint N, uint accum, uint M) {                         \
        gemm_mm_body<LOADER, false>(xh, GmSrc{w, nullptr, nullptr}, y, K, N, accum, M, 1u); }                     \
    extern "C" __global__ void __launch_bounds__(256) gemm_mm_##FMT##_sk(                                         \
        const ushort* xh, const uchar* w, float* y, uint K, uint N, uint M, uint nsplit) {                        \
        gemm_mm_body<LOADER, true>(xh, GmSrc{w, nullptr, nullptr}, y, K, N, 1u, M, nsplit); }                     \
    extern "C" __global__ void __launch_bounds__(256) gemm_mm_##FMT##_m128(                                       \
        const ushort* xh, const uchar* w, float* y, uint K, uint N, uint accum, uint M) {                         \
        gemm_mm_body<LOADER, false, false, 2>(xh, GmSrc{w, nullptr, nullptr}, y, K, N, accum, M, 1u); }           \
    extern "C" __global__ void __launch_bounds__(256) gemm_mm_##FMT##_m128_sk(                                    \
        const ushort* xh, const uchar* w, float* y, uint K, uint N, uint M, uint nsplit) {                        \
        gemm_mm_body<LOADER, true, false, 2>(xh, GmSrc{w, nullptr, nullptr}, y, K, N, 1u, M, nsplit); }

GEMM_ENTRIES(q4k, LoaderQ4K)
GEMM_ENTRIES(q5k, LoaderQ5K)
GEMM_ENTRIES(q6k, LoaderQ6K)
GEMM_ENTRIES(q8_0, LoaderQ80)
GEMM_ENTRIES(f16, LoaderF16)
GEMM_ENTRIES(iq4nl, LoaderIQ4NL)
GEMM_ENTRIES(iq4xs, LoaderIQ4XS)
typedef LoaderLegacy<false, false> LoaderQ40;
typedef LoaderLegacy<false, true> LoaderQ41;
typedef LoaderLegacy<true, false> LoaderQ50;
typedef LoaderLegacy<true, true> LoaderQ51;
GEMM_ENTRIES(q40, LoaderQ40)
GEMM_ENTRIES(q41, LoaderQ41)
GEMM_ENTRIES(q50, LoaderQ50)
GEMM_ENTRIES(q51, LoaderQ51)
GEMM_ENTRIES(mxfp4, LoaderMXFP4)
GEMM_ENTRIES(q2k, LoaderQ2K)
GEMM_ENTRIES(q3k, LoaderQ3K)

// ------------------------------------------------------------------ few tokens: weights straight into the matrix operand
// The tile above stages 128 rows x 64 weights through LDS for 128 token columns; with a handful of tokens seven eighths of
// its matrix work multiply padding and every K step still pays the staging and a barrier (14336 x 4096 at 8 .. 64 tokens:
// 32 - 36 us whatever the format).  Here a workgroup owns 16 rows, its waves take the 128-weight chunks of K in turn, and
// nothing goes through LDS but the final sums: v_mfma_f32_16x16x32_f16 with A = 16 tokens, B = 16 rows; lane (i, g) of
// either operand holds 8 consecutive positions of K group g.  The order of K inside an instruction is free as long as both
// operands agree, so lane (n, g) decodes the whole 32-weight block g of the chunk for row n (the per-thread loaders of the
// tile: one or two wide loads) and feeds it to four instructions, 8 weights each; lane (m, g) reads the matching 64 bytes
// of token m.  Up to 16 TG tokens per launch (TG accumulators); partial sums of the waves meet in LDS in wave order.
//   gemm_few_<fmt>{,_r4}_t{1,2,4}(xh, w, y, K, N, accum, M)     grid [ceil(N / 16 RG),1,1] x 256 (or 512 where RG TG <= 4),
//   K a multiple of 128, M <= 16 TG; `_r4`: RG = 4 groups of 16 rows per workgroup
typedef float float4v __attribute__((ext_vector_type(4)));
template <int J, class L>
__device__ __forceinline__ half8 gm_frag(const L& ld) {
    return __builtin_bit_cast(half8, (u32x4){ld.o[4 * J], ld.o[4 * J + 1], ld.o[4 * J + 2], ld.o[4 * J + 3]});
}
template <int J>
__device__ __forceinline__ half8 gm_frag(const LoaderF16& ld) { return __builtin_bit_cast(half8, ld.q[J]); }

template <class Loader, int TG, int RG, class TM>
__device__ __forceinline__ void gemm_few_body(const ushort* __restrict__ xh, const uchar* __restrict__ w, float* __restrict__ y,
                                              uint K, uint N, uint accum, uint M, const TM tm) {
    // RG groups of 16 rows per workgroup share every token fragment a lane reads (the tokens' bytes, re-read by every
    // workgroup, are most of the traffic of the 16-row form: 14336 rows x 16 tokens of K = 4096 read them 896 times)
    __shared__ float red[RG * TG > 4 ? 4 : 8][RG * TG][256];     // (eight waves only where that stays within 32 KB)
    const uint tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, nw = blockDim.x >> 6;
    const uint i16 = lane & 15u, g = lane >> 4;
    const uint n0 = blockIdx.x * (16u * RG);
    const size_t rb = Loader::row_bytes(K);
    const uchar* wrow[RG];
#pragma unroll
    for (int r = 0; r < RG; r++) wrow[r] = w + (size_t)min(n0 + 16u * r + i16, N - 1u) * rb;
    const ushort* xrow[TG];
#pragma unroll
    for (int tg = 0; tg < TG; tg++) xrow[tg] = xh + (size_t)tm.in_row(min(16u * tg + i16, M - 1u)) * K + g * 32u;
    float4v acc[RG][TG];
#pragma unroll
    for (int r = 0; r < RG; r++)
#pragma unroll
        for (int tg = 0; tg < TG; tg++) acc[r][tg] = (float4v){0.0f, 0.0f, 0.0f, 0.0f};
    const uint nchunk = K >> 7;
    Loader ld0, ld1;
    // one row group of one chunk: the next group's (or the next chunk's first group's) block is asked for first
#define GF_GROUP(CUR, NXT, R, NEXT_ROW, NEXT_C)                                                                   \
    do {                                                                                                          \
        if ((NEXT_C) < nchunk) NXT.load(NEXT_ROW, (NEXT_C) * 128u + g * 32u, 0u);                                 \
        gm_fence();                                                                                               \
        CUR.prep();                                                                                               \
        CUR.template part<0>(); CUR.template part<1>(); CUR.template part<2>(); CUR.template part<3>();           \
        _Pragma("unroll") for (int tg = 0; tg < TG; tg++) {                                                      \
            acc[R][tg] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xv[tg][0], gm_frag<0>(CUR), acc[R][tg], 0, 0, 0);  \
            acc[R][tg] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xv[tg][1], gm_frag<1>(CUR), acc[R][tg], 0, 0, 0);  \
            acc[R][tg] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xv[tg][2], gm_frag<2>(CUR), acc[R][tg], 0, 0, 0);  \
            acc[R][tg] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xv[tg][3], gm_frag<3>(CUR), acc[R][tg], 0, 0, 0);  \
        }                                                                                                         \
    } while (0)
    uint c = wave;
    if (c < nchunk) ld0.load(wrow[0], c * 128u + g * 32u, 0u);
    for (; c < nchunk; c += nw) {
        half8 xv[TG][4];
#pragma unroll
        for (int tg = 0; tg < TG; tg++)
#pragma unroll
            for (int j = 0; j < 4; j++) xv[tg][j] = *(const half8*)(xrow[tg] + c * 128u + 8u * j);
        if (RG == 1) {
            // (two chunks per trip so that the loaders alternate by name)
            GF_GROUP(ld0, ld1, 0, wrow[0], c + nw);
            c += nw;
            if (c < nchunk) {
#pragma unroll
                for (int tg = 0; tg < TG; tg++)
#pragma unroll
                    for (int j = 0; j < 4; j++) xv[tg][j] = *(const half8*)(xrow[tg] + c * 128u + 8u * j);
                GF_GROUP(ld1, ld0, 0, wrow[0], c + nw);
            }
        } else {
#pragma unroll
            for (int r = 0; r < RG; r += 2) {
                GF_GROUP(ld0, ld1, r, wrow[r + 1 < RG ? r + 1 : 0], c);
                GF_GROUP(ld1, ld0, r + 1 < RG ? r + 1 : 0, wrow[r + 2 < RG ? r + 2 : 0], r + 2 < RG ? c : c + nw);
            }
        }
    }
#undef GF_GROUP
    // D: lane (n = lane % 16, g) holds tokens 4 g + v of its group against row n
#pragma unroll
    for (int r = 0; r < RG; r++)
#pragma unroll
        for (int tg = 0; tg < TG; tg++)
#pragma unroll
            for (int v = 0; v < 4; v++) red[wave][r * TG + tg][(g * 4u + v) * 16u + i16] = acc[r][tg][v];
    __syncthreads();
    for (uint e = tid; e < (uint)(RG * TG) * 256u; e += blockDim.x) {
        const uint rt = e >> 8, r = rt / TG, tg = rt % TG, idx = e & 255u, tok = 16u * tg + (idx >> 4), row = n0 + 16u * r + (idx & 15u);
        float sum = red[0][rt][idx];
        for (uint k = 1; k < nw; k++) sum += red[k][rt][idx];
        if (tok < M && row < N) {
            float* o = y + (size_t)tm.out_row(tok) * N + row;
            *o = accum ? *o + sum : sum;
        }
    }
}

#define GEMM_FEW_ENTRY(FMT, LOADER, SUF, TG, RG)                                                                  \
    extern "C" __global__ void __launch_bounds__(512) gemm_few_##FMT##SUF(                                        \
        const ushort* xh, const uchar* w, float* y, uint K, uint N, uint accum, uint M) {                         \
        gemm_few_body<LOADER, TG, RG, GmDense>(xh, w, y, K, N, accum, M, GmDense()); }
#define GEMM_FEW_ENTRIES(FMT, LOADER)                                                                             \
    GEMM_FEW_ENTRY(FMT, LOADER, _t1, 1, 1)                                                                        \
    GEMM_FEW_ENTRY(FMT, LOADER, _t2, 2, 1)                                                                        \
    GEMM_FEW_ENTRY(FMT, LOADER, _t4, 4, 1)                                                                        \
    GEMM_FEW_ENTRY(FMT, LOADER, _r4_t1, 1, 4)                                                                     \
    GEMM_FEW_ENTRY(FMT, LOADER, _r4_t2, 2, 4)                                                                     \
    GEMM_FEW_ENTRY(FMT, LOADER, _r4_t4, 4, 4)
GEMM_FEW_ENTRIES(q8_0, LoaderQ80)
GEMM_FEW_ENTRIES(f16, LoaderF16)
GEMM_FEW_ENTRIES(iq4nl, LoaderIQ4NL)
GEMM_FEW_ENTRIES(iq4xs, LoaderIQ4XS)
GEMM_FEW_ENTRIES(q40, LoaderQ40)
GEMM_FEW_ENTRIES(q41, LoaderQ41)
GEMM_FEW_ENTRIES(q50, LoaderQ50)
GEMM_FEW_ENTRIES(q51, LoaderQ51)
GEMM_FEW_ENTRIES(mxfp4, LoaderMXFP4)
GEMM_FEW_ENTRIES(q2k, LoaderQ2K)
GEMM_FEW_ENTRIES(q3k, LoaderQ3K)

// Grouped expert products on the same tile (128 tokens x 128 rows): expert e = blockIdx.z % E owns rows e N .. of its
// tensor and the assignments list[offsets[e] .. offsets[e + 1]); blockIdx.z / E picks the tensor and output of a pair
// (gate and up of a mixture-of-experts layer in one launch; w1 / y1 unused with a grid of E).  Assignment a reads
// activation row a / DIV (its token: DIV = slots per token; 1 where the activations are per assignment, as for the
// down projection) and writes row a.  Token tiles blockIdx.y, + gridDim.y, .. of the expert; workgroups past its count
// leave at once.
//   moe_mm_<fmt>(xh, w0, w1, y0, y1, offsets, list, K, N, NA, E, DIV)    grid [ceil(N / 128), 1 .., E or 2 E] x 256
#define MOE_MM_ENTRY(FMT, LOADER, ROWBYTES)                                                                       \
    extern "C" __global__ void __launch_bounds__(256) moe_mm_##FMT(                                               \
        const ushort* xh, const uchar* w0, const uchar* w1, float* y0, float* y1, const uint* offsets,            \
        const uint* list, uint K, uint N, uint NA, uint E, uint DIV) {                                            \
        const uint e = blockIdx.z % E, second = blockIdx.z / E;                                                   \
        const uint a0 = min(offsets[e], NA), a1 = min(offsets[e + 1], NA);                                        \
        if (a0 >= a1) return;                                                                                     \
        GmList tm;                                                                                                \
        tm.lst = list + a0;                                                                                       \
        tm.last = NA - 1u;                                                                                        \
        tm.div = DIV;                                                                                             \
        const uchar* w = (second ? w1 : w0) + (size_t)e * N * (ROWBYTES);                                         \
        for (uint ty = blockIdx.y; ty * 128u < a1 - a0; ty += gridDim.y) {                                        \
            gemm_mm_body<LOADER, false, false, 2, GmList>(xh, GmSrc{w, nullptr, nullptr}, second ? y1 : y0, K, N, \
                                                          0u, a1 - a0, 1u, tm, ty);                               \
            __syncthreads();                                                                                      \
        }                                                                                                         \
    }
MOE_MM_ENTRY(q8_0, LoaderQ80, (size_t)(K / 32u) * 34u)
MOE_MM_ENTRY(iq4nl, LoaderIQ4NL, (size_t)(K / 32u) * IQ4NL_BYTES)
MOE_MM_ENTRY(iq4xs, LoaderIQ4XS, (size_t)(K / 256u) * IQ4XS_BYTES)
MOE_MM_ENTRY(f16, LoaderF16, (size_t)K * 2u)          // (experts decoded into f16 beforehand: formats without a loader here)

// The same grouped products for experts that received a few dozen tokens, on the few-token kernel (64 rows per workgroup,
// 32 assignments per pass, weights decoded straight into the matrix operand): passes blockIdx.y, + gridDim.y, .. of the expert.
//   moe_few_<fmt>(xh, w0, w1, y0, y1, offsets, list, K, N, NA, E, DIV)    grid [ceil(N / 64), 1 .., E or 2 E] x 256, K % 128 == 0
#define MOE_FEW_ENTRY(FMT, LOADER, ROWBYTES)                                                                      \
    extern "C" __global__ void __launch_bounds__(256) moe_few_##FMT(                                              \
        const ushort* xh, const uchar* w0, const uchar* w1, float* y0, float* y1, const uint* offsets,            \
        const uint* list, uint K, uint N, uint NA, uint E, uint DIV) {                                            \
        const uint e = blockIdx.z % E, second = blockIdx.z / E;                                                   \
        const uint a0 = min(offsets[e], NA), a1 = min(offsets[e + 1], NA);                                        \
        if (a0 >= a1) return;                                                                                     \
        const uchar* w = (second ? w1 : w0) + (size_t)e * N * (ROWBYTES);                                         \
        for (uint ty = blockIdx.y; ty * 32u < a1 - a0; ty += gridDim.y) {                                         \
            GmList tm;                                                                                            \
            tm.lst = list + a0 + ty * 32u;                                                                        \
            tm.last = NA - 1u;                                                                                    \
            tm.div = DIV;                                                                                         \
            gemm_few_body<LOADER, 2, 4, GmList>(xh, w, second ? y1 : y0, K, N, 0u, min(32u, a1 - a0 - ty * 32u), tm); \
            __syncthreads();                                                                                      \
        }                                                                                                         \
    }
MOE_FEW_ENTRY(q8_0, LoaderQ80, (size_t)(K / 32u) * 34u)
MOE_FEW_ENTRY(iq4nl, LoaderIQ4NL, (size_t)(K / 32u) * IQ4NL_BYTES)
MOE_FEW_ENTRY(iq4xs, LoaderIQ4XS, (size_t)(K / 256u) * IQ4XS_BYTES)

// act16[i] = f16(silu(g[i]) * u[i]): what the grouped gate / up launch hands to the grouped down launch
// (crates/ojas-cuda/src/kernels/moe.rs:75-102 forms the same product in f32)
extern "C" __global__ void __launch_bounds__(256)
moe_act_half(const float* __restrict__ g, const float* __restrict__ u, ushort* __restrict__ act16, uint n) {
    // eight values a thread (two 16-byte loads of each input, one 16-byte store) where the three arrays allow it
    const uint n8 = ((((size_t)g | (size_t)u | (size_t)act16) & 15u) == 0) ? n >> 3 : 0u;
    for (uint i = blockIdx.x * 256u + threadIdx.x; i < n8; i += gridDim.x * 256u) {
        const float4 g0 = ((const float4*)g)[2u * i], g1 = ((const float4*)g)[2u * i + 1u];
        const float4 u0 = ((const float4*)u)[2u * i], u1 = ((const float4*)u)[2u * i + 1u];
        const float gs[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
        const float us[8] = {u0.x, u0.y, u0.z, u0.w, u1.x, u1.y, u1.z, u1.w};
        uint h[8];
#pragma unroll
        for (int j = 0; j < 8; j++) h[j] = __half_as_ushort(__float2half_rn((gs[j] / (1.0f + expf(-gs[j]))) * us[j]));
        ((uint4*)act16)[i] = make_uint4(h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16), h[6] | (h[7] << 16));
    }
    for (uint i = (n8 << 3) + blockIdx.x * 256u + threadIdx.x; i < n; i += gridDim.x * 256u) {
        const float gs = g[i];
        act16[i] = __half_as_ushort(__float2half_rn((gs / (1.0f + expf(-gs))) * u[i]));
    }
}

// The reference's entries for Q4L weights, under their names and argument lists
// (crates/ojas-cuda/src/kernels/gemm_q.rs:26-38, :505-542; dispatched by `CudaSsm::mm`, crates/ojas-cuda/src/qwen35.rs:683,690):
//   gemm_mm_q4l(x f32, w4, y, qa, qb, K, N, accum, M)      gemm_mm_q4l_hb(xh f16, ...)      gemm_mm_q4l_sk(xh f16, w4, y, qa, qb, K, N, M, nsplit)
// on this library's tile: grid [ceil(N/128), ceil(M/256), nsplit].
extern "C" __global__ void __launch_bounds__(256) gemm_mm_q4l(
    const float* x, const uchar* w4, float* y, const ushort* qa, const ushort* qb, uint K, uint N, uint accum, uint M) {
    gemm_mm_body<LoaderQ4L, false, true>(x, GmSrc{w4, qa, qb}, y, K, N, accum, M, 1u);
}
extern "C" __global__ void __launch_bounds__(256) gemm_mm_q4l_hb(
    const ushort* xh, const uchar* w4, float* y, const ushort* qa, const ushort* qb, uint K, uint N, uint accum, uint M) {
    gemm_mm_body<LoaderQ4L, false>(xh, GmSrc{w4, qa, qb}, y, K, N, accum, M, 1u);
}
extern "C" __global__ void __launch_bounds__(256) gemm_mm_q4l_sk(
    const ushort* xh, const uchar* w4, float* y, const ushort* qa, const ushort* qb, uint K, uint N, uint M, uint nsplit) {
    gemm_mm_body<LoaderQ4L, true>(xh, GmSrc{w4, qa, qb}, y, K, N, 1u, M, nsplit);
}
