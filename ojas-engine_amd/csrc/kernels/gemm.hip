// Family "gemm": prefill / verify matmul  y[M,N] (+)= x[M,K] . W^T  with W in GGUF blocks.
//
// Contract (reference: crates/ojas-cuda/src/kernels/gemm_q.rs:1-56; raw K-quant twin
// crates/ojas-metal/src/kernels/gemm_fat.rs:243-368): activations rounded to f16 on their way into
// the tile, weights dequantized to f16 into the tile, f32 accumulation, f32 y; any M and N (loads
// clamped, stores masked, nothing written past row M).  Here the dequantized tile holds exactly
// the bits `dequant_to_f16` produces (crates/ojas-formats/src/gguf.rs:612-1116): every product and
// difference is rounded on its own, then one round-to-nearest-even to binary16.
//
//   gemm_mm_<fmt>(xh, w, y, K, N, accum, M)        xh: f16 [M][K]; grid [ceil(N/128), ceil(M/256), 1]
//   gemm_mm_<fmt>_sk(xh, w, y, K, N, M, nsplit)    grid.z = nsplit; adds its K slice into y with
//                                                  f32 atomics (zero y first for a plain product)
//
// CDNA4 plan: one workgroup of 4 waves owns a 256 (tokens) x 128 (outputs) tile and walks K in
// steps of 64.  Per step the 256 threads stage the activation slab (256 x 64 f16) and dequantize
// the weight slab (128 rows x one 32-byte chunk of quants = 64 weights each) into LDS, rows padded
// to 144 bytes so 16-byte fragment reads of 16 consecutive rows fall in distinct banks.  Each wave
// owns 128 x 64 of the tile as 4 x 2 blocks of v_mfma_f32_32x32x16_f16 (A = activations, B =
// weights, so a D register holds 32 consecutive outputs of one token: coalesced stores).  Global
// loads run three steps ahead in registers and are written to the other LDS stage after the
// MFMAs of the current step: one barrier per step.
#include "ojk_common.h"

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));

#define GM_BM 256
#define GM_BN 128
#define GM_BK 64
#define GM_STRIDE 144  // bytes per LDS row: 64 f16 + 16 bytes of padding
#define GM_STAGE ((GM_BM + GM_BN) * GM_STRIDE)

// f32 -> f16 bits, the value pinned first so that "multiply/subtract, then convert" cannot be
// folded into one mixed-precision FMA (which would round once and lose the sign of zero).
__device__ __forceinline__ uint f16_bits_rn(float v) {
    asm volatile("" : "+v"(v));
    return (uint)__half_as_ushort(__float2half_rn(v));
}
__device__ __forceinline__ uint pack2(float a, float b) { return f16_bits_rn(a) | (f16_bits_rn(b) << 16); }

// ---- global loads whose issue point the compiler may not move -----------------------------------
// The compiler sinks ordinary loads down to their first use to save registers, which turns a
// three-steps-ahead prefetch into load-then-wait.  These loads are opaque to it: they are issued
// where they are written, and the consumer waits with an explicit s_waitcnt (gm_wait) that also
// re-defines the destination registers, so nothing that reads them can be scheduled above it.
// Vector memory operations retire in order, so "at most n outstanding" means every load issued
// before the last n has landed.
typedef uint u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ u32x4 gm_load16(const void* p) {
    u32x4 v;
    asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(v) : "v"(p) : "memory");
    return v;
}
__device__ __forceinline__ uint gm_load_u16(const void* p) {
    uint v;
    asm volatile("global_load_ushort %0, %1, off" : "=v"(v) : "v"(p) : "memory");
    return v;
}
__device__ __forceinline__ uint gm_load_u8(const void* p) {
    uint v;
    asm volatile("global_load_ubyte %0, %1, off" : "=v"(v) : "v"(p) : "memory");
    return v;
}
template <int N>
__device__ __forceinline__ void gm_wait(u32x4 (&x)[8]) {
    asm volatile("s_waitcnt vmcnt(%8)"
                 : "+v"(x[0]), "+v"(x[1]), "+v"(x[2]), "+v"(x[3]), "+v"(x[4]), "+v"(x[5]), "+v"(x[6]), "+v"(x[7])
                 : "n"(N)
                 : "memory");
}

// ------------------------------------------------------------------ per-format slab loaders
// A loader owns, for one thread, 32 weights of one row of the 128 x 64 slab: thread t -> row
// t/2, half h = t%2.  `load` issues the global loads; `store` dequantizes into the LDS row.
struct LoaderQ4K {
    static constexpr int NL = 2;  // global loads per slab
    u32x4 hdr, qs;
    uint c;
    __device__ __forceinline__ void pin() { asm volatile("" : "+v"(hdr), "+v"(qs)::"memory"); }
    static __device__ __forceinline__ size_t row_bytes(uint K) { return (size_t)(K >> 8) * Q4K_BYTES; }
    __device__ __forceinline__ void load(const uchar* row, uint k0, uint h) {
        const uchar* blk = row + (size_t)(k0 >> 8) * Q4K_BYTES;
        c = (k0 >> 6) & 3u;  // 32-byte chunk of the super-block = sub-blocks 2c, 2c+1
        hdr = gm_load16(blk);
        qs = gm_load16(blk + 16u + c * 32u + h * 16u);
    }
    // 16 low-nibble weights -> slab columns 16h.., 16 high-nibble weights -> columns 32+16h..
    __device__ __forceinline__ void store(uchar* lds_row, uint h) const {
        uint sc, mn;
        q4k_scale_min_pair(hdr.y, hdr.z, hdr.w, c, sc, mn);
        float d = f16_bits_to_f32(hdr.x & 0xFFFFu), dmin = f16_bits_to_f32(hdr.x >> 16);
        float dl1 = __fmul_rn(d, (float)(sc & 0xFFu)), ml1 = __fmul_rn(dmin, (float)(mn & 0xFFu));
        float dl2 = __fmul_rn(d, (float)(sc >> 8)), ml2 = __fmul_rn(dmin, (float)(mn >> 8));
        uint q[4] = {qs.x, qs.y, qs.z, qs.w};
        uint lo[8], hi[8];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            uint v = q[i];
            float a0 = (float)(v & 0xFu), a1 = (float)((v >> 8) & 0xFu), a2 = (float)((v >> 16) & 0xFu),
                  a3 = (float)((v >> 24) & 0xFu);
            float b0 = (float)((v >> 4) & 0xFu), b1 = (float)((v >> 12) & 0xFu), b2 = (float)((v >> 20) & 0xFu),
                  b3 = (float)(v >> 28);
            lo[2 * i] = pack2(__fsub_rn(__fmul_rn(dl1, a0), ml1), __fsub_rn(__fmul_rn(dl1, a1), ml1));
            lo[2 * i + 1] = pack2(__fsub_rn(__fmul_rn(dl1, a2), ml1), __fsub_rn(__fmul_rn(dl1, a3), ml1));
            hi[2 * i] = pack2(__fsub_rn(__fmul_rn(dl2, b0), ml2), __fsub_rn(__fmul_rn(dl2, b1), ml2));
            hi[2 * i + 1] = pack2(__fsub_rn(__fmul_rn(dl2, b2), ml2), __fsub_rn(__fmul_rn(dl2, b3), ml2));
        }
        uint4* p = (uint4*)(lds_row + h * 32u);
        p[0] = make_uint4(lo[0], lo[1], lo[2], lo[3]);
        p[1] = make_uint4(lo[4], lo[5], lo[6], lo[7]);
        uint4* ph = (uint4*)(lds_row + 64u + h * 32u);
        ph[0] = make_uint4(hi[0], hi[1], hi[2], hi[3]);
        ph[1] = make_uint4(hi[4], hi[5], hi[6], hi[7]);
    }
};

struct LoaderQ6K {
    static constexpr int NL = 6;
    u32x4 qa, qb, qh;
    uint sca, scb, d16, hi_half;  // sca, scb: the sub-scales of the slab's two quarters for this thread's 16 columns
    __device__ __forceinline__ void pin() {
        asm volatile("" : "+v"(qa), "+v"(qb), "+v"(qh), "+v"(sca), "+v"(scb), "+v"(d16)::"memory");
    }
    static __device__ __forceinline__ size_t row_bytes(uint K) { return (size_t)(K >> 8) * Q6K_BYTES; }
    __device__ __forceinline__ void load(const uchar* row, uint k0, uint h) {
        const uchar* blk = row + (size_t)(k0 >> 8) * Q6K_BYTES;
        uint j = (k0 >> 6) & 3u, hf = j >> 1;  // 64-column slab j of the super-block: half hf, quarters 2(j%2), +1
        hi_half = j & 1u;
        qa = gm_load16(blk + hf * 64u + h * 16u);
        qb = gm_load16(blk + hf * 64u + 32u + h * 16u);
        qh = gm_load16(blk + 128u + hf * 32u + h * 16u);
        const uchar* sc = blk + 192u + hf * 8u + (j & 1u) * 4u + h;  // sc[2q + h], q = 2(j%2), 2(j%2)+1
        sca = gm_load_u8(sc);
        scb = gm_load_u8(sc + 2);
        d16 = gm_load_u16(blk + 208u);
    }
    __device__ __forceinline__ void store(uchar* lds_row, uint h) const {
        float d = f16_bits_to_f32(d16);
        float s0 = __fmul_rn(d, (float)(signed char)sca), s1 = __fmul_rn(d, (float)(signed char)scb);
        uint a[4] = {qa.x, qa.y, qa.z, qa.w}, b[4] = {qb.x, qb.y, qb.z, qb.w}, hq[4] = {qh.x, qh.y, qh.z, qh.w};
        uint o0[8], o1[8];
        const uint sh_h0 = hi_half ? 4u : 0u, sh_h1 = hi_half ? 6u : 2u, sh_l = hi_half ? 4u : 0u;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            float w0[4], w1[4];
#pragma unroll
            for (int e = 0; e < 4; e++) {
                uint av = (a[i] >> (8 * e)) & 0xFFu, bv = (b[i] >> (8 * e)) & 0xFFu, hv = (hq[i] >> (8 * e)) & 0xFFu;
                int q0 = (int)(((av >> sh_l) & 0xFu) | (((hv >> sh_h0) & 3u) << 4)) - 32;
                int q1 = (int)(((bv >> sh_l) & 0xFu) | (((hv >> sh_h1) & 3u) << 4)) - 32;
                w0[e] = __fmul_rn(s0, (float)q0);
                w1[e] = __fmul_rn(s1, (float)q1);
            }
            o0[2 * i] = pack2(w0[0], w0[1]);
            o0[2 * i + 1] = pack2(w0[2], w0[3]);
            o1[2 * i] = pack2(w1[0], w1[1]);
            o1[2 * i + 1] = pack2(w1[2], w1[3]);
        }
        uint4* p = (uint4*)(lds_row + h * 32u);
        p[0] = make_uint4(o0[0], o0[1], o0[2], o0[3]);
        p[1] = make_uint4(o0[4], o0[5], o0[6], o0[7]);
        uint4* ph = (uint4*)(lds_row + 64u + h * 32u);
        ph[0] = make_uint4(o1[0], o1[1], o1[2], o1[3]);
        ph[1] = make_uint4(o1[4], o1[5], o1[6], o1[7]);
    }
};

struct LoaderQ80 {
    static constexpr int NL = 3;
    u32x4 qa, qb;
    uint d16;
    __device__ __forceinline__ void pin() { asm volatile("" : "+v"(qa), "+v"(qb), "+v"(d16)::"memory"); }
    static __device__ __forceinline__ size_t row_bytes(uint K) { return (size_t)(K >> 5) * Q80_BYTES; }
    __device__ __forceinline__ void load(const uchar* row, uint k0, uint h) {
        const uchar* blk = row + (size_t)((k0 >> 5) + h) * Q80_BYTES;  // block h of the slab's two
        d16 = gm_load_u16(blk);
        qa = gm_load16(blk + 2u);
        qb = gm_load16(blk + 18u);
    }
    // block h fills slab columns 32h..32h+31
    __device__ __forceinline__ void store(uchar* lds_row, uint h) const {
        float d = f16_bits_to_f32(d16);
        uint q[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
        uint o[16];
#pragma unroll
        for (int i = 0; i < 8; i++) {
            float v0 = __fmul_rn(d, (float)(signed char)(q[i]));
            float v1 = __fmul_rn(d, (float)(signed char)(q[i] >> 8));
            float v2 = __fmul_rn(d, (float)(signed char)(q[i] >> 16));
            float v3 = __fmul_rn(d, (float)((int)q[i] >> 24));
            o[2 * i] = pack2(v0, v1);
            o[2 * i + 1] = pack2(v2, v3);
        }
        uint4* p = (uint4*)(lds_row + h * 64u);
#pragma unroll
        for (int i = 0; i < 4; i++) p[i] = make_uint4(o[4 * i], o[4 * i + 1], o[4 * i + 2], o[4 * i + 3]);
    }
};

// ------------------------------------------------------------------ the tile
template <class Loader, bool SPLITK>
__device__ __forceinline__ void gemm_mm_body(const ushort* __restrict__ xh, const uchar* __restrict__ w,
                                             float* __restrict__ y, uint K, uint N, uint accum, uint M, uint nsplit) {
    __shared__ __attribute__((aligned(16))) uchar lds[2 * GM_STAGE];
    const uint tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint n0 = blockIdx.x * GM_BN, m0 = blockIdx.y * GM_BM;
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
    const uchar* wrow = w + (size_t)min(n0 + wr, N - 1u) * Loader::row_bytes(K);
    const ushort* xrow[8];
#pragma unroll
    for (int i = 0; i < 8; i++) xrow[i] = xh + (size_t)min(m0 + xr + 32u * i, M - 1u) * K + xc;

    // wave tile: 128 (m) x 64 (n)
    const uint wm = (wave >> 1) * 128u, wn = (wave & 1u) * 64u;
    const uint fr = lane & 31u, kg = lane >> 5;
    float16v acc[4][2];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;

    // Three register sets hold the slabs of steps t+1 .. t+3 while step t runs from LDS: loads are
    // in flight for two whole steps before anyone waits for them (one wave per SIMD cannot lean
    // on other waves to cover HBM latency).
    u32x4 xs0[8], xs1[8], xs2[8];
    Loader ld0, ld1, ld2;
    const uint nt = (k_end - k_begin) / GM_BK;

#define GM_LOAD(XS, LD, T)                                                                       \
    do {                                                                                         \
        const uint kk_ = k_begin + (T) * GM_BK;                                                  \
        _Pragma("unroll") for (int i_ = 0; i_ < 8; i_++) XS[i_] = gm_load16(xrow[i_] + kk_);      \
        LD.load(wrow, kk_, wh);                                                                  \
    } while (0)
#define GM_STORE(XS, LD, STG)                                                                    \
    do {                                                                                         \
        uchar* a_ = lds + (STG) * GM_STAGE;                                                      \
        _Pragma("unroll") for (int i_ = 0; i_ < 8; i_++)                                         \
            *(u32x4*)(a_ + (xr + 32u * i_) * GM_STRIDE + xc * 2u) = XS[i_];                      \
        LD.store(a_ + GM_BM * GM_STRIDE + wr * GM_STRIDE, wh);                                   \
    } while (0)
#define GM_COMPUTE(STG)                                                                          \
    do {                                                                                         \
        const uchar* a_ = lds + (STG) * GM_STAGE;                                                \
        const uchar* b_ = a_ + GM_BM * GM_STRIDE;                                                \
        _Pragma("unroll") for (int ks = 0; ks < GM_BK / 16; ks++) {                              \
            half8 af[4], bf[2];                                                                  \
            _Pragma("unroll") for (int i = 0; i < 4; i++)                                        \
                af[i] = *(const half8*)(a_ + (wm + 32u * i + fr) * GM_STRIDE + (ks * 16u + kg * 8u) * 2u); \
            _Pragma("unroll") for (int j = 0; j < 2; j++)                                        \
                bf[j] = *(const half8*)(b_ + (wn + 32u * j + fr) * GM_STRIDE + (ks * 16u + kg * 8u) * 2u); \
            _Pragma("unroll") for (int i = 0; i < 4; i++)                                        \
                _Pragma("unroll") for (int j = 0; j < 2; j++)                                    \
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], bf[j], acc[i][j], 0, 0, 0); \
        }                                                                                        \
    } while (0)
// step T: refill the set that step T's slab came from, run step T, stage step T+1
#define GM_STEP(T, XS_FREE, LD_FREE, XS_NEXT, LD_NEXT)                                           \
    do {                                                                                         \
        if ((T) + 3u < nt) GM_LOAD(XS_FREE, LD_FREE, (T) + 3u);                                  \
        GM_COMPUTE((T) & 1u);                                                                    \
        if ((T) + 1u < nt) {                                                                     \
            GM_WAIT_FOR(XS_NEXT, LD_NEXT, (T) + 1u);                                             \
            GM_STORE(XS_NEXT, LD_NEXT, ((T) + 1u) & 1u);                                         \
        }                                                                                        \
        __syncthreads();                                                                         \
    } while (0)
// wait for the slab of step T: the slabs of steps T+1 and T+2, where they exist, were issued later
#define GM_WAIT_FOR(XS, LD, T)                                                                   \
    do {                                                                                         \
        if ((T) + 2u < nt) gm_wait<2 * LPS>(XS);                                                 \
        else if ((T) + 1u < nt) gm_wait<LPS>(XS);                                                \
        else gm_wait<0>(XS);                                                                     \
        LD.pin();                                                                                \
    } while (0)
    constexpr int LPS = 8 + Loader::NL;  // loads per slab

    GM_LOAD(xs0, ld0, 0u);
    if (nt > 1u) GM_LOAD(xs1, ld1, 1u);
    if (nt > 2u) GM_LOAD(xs2, ld2, 2u);
    GM_WAIT_FOR(xs0, ld0, 0u);
    GM_STORE(xs0, ld0, 0u);
    __syncthreads();
    for (uint t = 0; t < nt; t += 3u) {
        GM_STEP(t, xs0, ld0, xs1, ld1);
        if (t + 1u < nt) GM_STEP(t + 1u, xs1, ld1, xs2, ld2);
        if (t + 2u < nt) GM_STEP(t + 2u, xs2, ld2, xs0, ld0);
    }
#undef GM_LOAD
#undef GM_STORE
#undef GM_COMPUTE
#undef GM_STEP
#undef GM_WAIT_FOR

    // epilogue: D register v of block (i, j) holds row 8*(v/4) + 4*kg + v%4, column fr
#pragma unroll
    for (int i = 0; i < 4; i++) {
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const uint n = n0 + wn + 32u * j + fr;
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const uint m = m0 + wm + 32u * i + 8u * (v >> 2) + 4u * kg + (v & 3u);
                if (m < M && n < N) {
                    float* o = y + (size_t)m * N + n;
                    if (SPLITK) atomicAdd(o, acc[i][j][v]);
                    else *o = accum ? *o + acc[i][j][v] : acc[i][j][v];
                }
            }
        }
    }
}

#define GEMM_ENTRIES(FMT, LOADER)                                                                                 \
    extern "C" __global__ void __launch_bounds__(256) gemm_mm_##FMT(                                              \
        const ushort* xh, const uchar* w, float* y, uint K, uint N, uint accum, uint M) {                         \
        gemm_mm_body<LOADER, false>(xh, w, y, K, N, accum, M, 1u); }                                              \
    extern "C" __global__ void __launch_bounds__(256) gemm_mm_##FMT##_sk(                                         \
        const ushort* xh, const uchar* w, float* y, uint K, uint N, uint M, uint nsplit) {                        \
        gemm_mm_body<LOADER, true>(xh, w, y, K, N, 1u, M, nsplit); }

GEMM_ENTRIES(q4k, LoaderQ4K)
GEMM_ENTRIES(q6k, LoaderQ6K)
GEMM_ENTRIES(q8_0, LoaderQ80)
