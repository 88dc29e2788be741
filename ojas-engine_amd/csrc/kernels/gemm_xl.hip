// Family "gemm_xl": the prefill matmul  y[M,N] (+)= x[M,K] . W^T  on raw Q4_K blocks with the
// arithmetic of the reference's GPU prefill kernel `gemm_mm_q4l`
// (crates/ojas-cuda/src/kernels/gemm_q.rs:104-140 over crates/ojas-formats/src/quant.rs:187-222):
// per 32-weight sub-block  qa = f16(d*sc),  qb = f16(-dmin*m),  and every weight enters the tile as
// the f16 fused multiply-add  qa*q + qb  (one rounding).  The reference computes qa / qb in a
// load-time relayout pass; here they are formed in the kernel from the raw super-block header, so
// the weights stay in the file's layout.  Activations are f16 [M][K], accumulation is f32.
//
//   gemm_mm_q4kl(xh, w, y, K, N, accum, M)        grid [ceil(N/256), ceil(M/256), 1]
//   gemm_mm_q4kl_sk(xh, w, y, K, N, M, nsplit)    grid.z = nsplit; f32 atomic adds into y
//
// CDNA4 plan.  One workgroup of 4 waves (one per SIMD) owns BM x 256 outputs and walks K in steps
// of 64; a wave owns (BM/2) x 128 as (BM/64) x 4 blocks of v_mfma_f32_32x32x16_f16, 256
// accumulator registers at BM = 256.  What bounds such a tile on this chip is LDS bandwidth
// (128 bytes per clock per CU, shared by the four SIMDs) and vector-ALU issue, not the matrix
// pipe, so the design spends as little of either as it can:
//   * a wave tile of 128 x 128 reads 512 LDS bytes per MFMA (a 128 x 64 wave tile reads 768);
//   * activations go from global memory straight into LDS (global_load_lds_dwordx4), never
//     through registers; rows are 128 bytes, and the 16-byte chunk c of row r sits in slot
//     c ^ ((r >> 1) & 7), applied on the global side of the copy: LDS has 64 four-byte banks, two
//     rows span them once, so 16 consecutive rows reading the same chunk touch every bank
//     exactly once and a 128-bit fragment read runs at the full 256 bytes per clock, unpadded;
//   * a nibble becomes the f16 1024 + q by or-ing it into 0x6400; subtracting 1024 and one packed
//     fma per pair of weights finish the job: about 2 vector instructions per weight;
//   * the raw weight bytes take the same road (a thread's 48 bytes per step: super-block header
//     and one 32-byte chunk), two steps ahead, and are read back from LDS by the thread that
//     dequantizes them: no asynchronous load ever targets a register, so there is nothing the
//     compiler could copy or sink before it has landed; the copies are awaited with s_waitcnt.
#include "ojk_common.h"

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float2v __attribute__((ext_vector_type(2)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef uint u32x4 __attribute__((ext_vector_type(4)));

#define GX_BN 256u
#define GX_BK 64u
#define GX_ROW 128u                   // bytes per LDS row: 64 f16
#define GX_WSTAGE (GX_BN * GX_ROW)    // 32 KB
#define GX_RAW (GX_BN * 48u)           // raw bytes of a weight slab: 16 (header) + 32 (chunk) per row

// 16 bytes per lane from `base + voff` to LDS at `lds_addr + 16 * lane` (base and lds_addr uniform).
__device__ __forceinline__ void gx_load_lds16(const void* base, uint voff, uint lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(voff), "s"(base), "s"(lds_addr)
                 : "memory");
}
template <int N>
__device__ __forceinline__ void gx_wait() {
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

// One thread's share of a weight slab: 64 weights of one row = one 32-byte chunk c of a Q4_K
// super-block (low nibbles: sub-block 2c, high nibbles: sub-block 2c+1) plus the header.
struct GxQ4K {
    u32x4 hdr, q0, q1;
    uint c;
    half2v a_lo, c_lo, a_hi, c_hi;
    // from the raw staging slot: header, then the two halves of the chunk (4 KB apart per part)
    __device__ __forceinline__ void read(const uchar* raw, uint chunk) {
        c = chunk;
        hdr = *(const u32x4*)raw;
        q0 = *(const u32x4*)(raw + 4096u);
        q1 = *(const u32x4*)(raw + 8192u);
    }
    __device__ __forceinline__ void prep() {
        uint sc, mn;
        q4k_scale_min_pair(hdr.y, hdr.z, hdr.w, c, sc, mn);
        const float d = f16_bits_to_f32(hdr.x & 0xFFFFu), ndm = -f16_bits_to_f32(hdr.x >> 16);
        // products of an f16 and a 6-bit integer are exact in f32: one rounding, to f16
        // (pinned, so that a product of zero keeps its sign through the conversion)
        float p1 = d * (float)(sc & 0xFFu), r1 = ndm * (float)(mn & 0xFFu);
        float p2 = d * (float)(sc >> 8), r2 = ndm * (float)(mn >> 8);
        asm volatile("" : "+v"(p1), "+v"(r1), "+v"(p2), "+v"(r2));
        const _Float16 a1 = (_Float16)p1, b1 = (_Float16)r1, a2 = (_Float16)p2, b2 = (_Float16)r2;
        a_lo = (half2v){a1, a1};
        c_lo = (half2v){b1, b1};
        a_hi = (half2v){a2, a2};
        c_hi = (half2v){b2, b2};
    }
    static __device__ __forceinline__ uint fma2(uint bits, half2v a, half2v c) {
        const half2v k1024 = {(_Float16)1024.0f, (_Float16)1024.0f};
        half2v q = __builtin_bit_cast(half2v, bits) - k1024;
        return __builtin_bit_cast(uint, __builtin_elementwise_fma(q, a, c));
    }
    // (x & 0x000F000F) | 0x64006400 in one instruction: two nibbles as the halves 1024 + q.
    // (The mask travels in a scalar register, the magic in a vector register: a VOP3 instruction
    // of this target reads one scalar operand.)
    static __device__ __forceinline__ uint nib2h(uint x, uint magic) {
        uint r;
        asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(x), "s"(0x000F000Fu), "v"(magic));
        return r;
    }
    // dword I (0..7) of the chunk: bytes 4I..4I+3 -> columns 4I..4I+3 (low) and 32+4I.. (high)
    template <int I>
    __device__ __forceinline__ void part(uint (&lo)[2], uint (&hi)[2], uint magic) const {
        const uint v = I < 4 ? q0[I & 3] : q1[I & 3];
        const uint p0 = __builtin_amdgcn_perm(0u, v, 0x0C010C00u);  // bytes (b0, 0, b1, 0)
        const uint p1 = __builtin_amdgcn_perm(0u, v, 0x0C030C02u);  // bytes (b2, 0, b3, 0)
        lo[0] = fma2(nib2h(p0, magic), a_lo, c_lo);
        lo[1] = fma2(nib2h(p1, magic), a_lo, c_lo);
        hi[0] = fma2(nib2h(p0 >> 4, magic), a_hi, c_hi);
        hi[1] = fma2(nib2h(p1 >> 4, magic), a_hi, c_hi);
    }
};

// MI = 32-row blocks per wave along M: the tile is (64 MI) x 256.
// ACCUM is a template parameter, not the kernel's run-time flag: with the choice made per stored element the
// 256 x 256 instance, which has no register to spare, spills in its epilogue.
template <int MI, bool SPLITK, bool ACCUM>
__device__ __forceinline__ void gemm_xl_body(const ushort* __restrict__ xh, const uchar* __restrict__ w,
                                             float* __restrict__ y, uint K, uint N, uint M, uint nsplit, uchar* lds) {
    constexpr uint BM = 64u * MI;
    constexpr uint XSTAGE = BM * GX_ROW;
    constexpr int XL = MI * 2;  // LDS-direct loads per wave and slab
    const uint tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint n0 = blockIdx.x * GX_BN, m0 = blockIdx.y * BM;
    uint k_begin = 0, k_end = K;
    if (SPLITK) {
        uint steps = K / GX_BK, per = (steps + nsplit - 1) / nsplit;
        k_begin = min(blockIdx.z * per, steps) * GX_BK;
        k_end = min((blockIdx.z + 1) * per, steps) * GX_BK;
        if (k_begin >= k_end) return;
    }
    const uint nt = (k_end - k_begin) / GX_BK;
    const uint lds0 = (uint)(size_t)(__attribute__((address_space(3))) uchar*)lds;

    // activation slab: wave `wave`, copy i moves rows (wave*XL + i)*8 .. +7; lane -> row lane/8,
    // slot lane%8, which holds source chunk (lane%8) ^ ((row/2)%8)
    uint xoff[XL];
#pragma unroll
    for (int i = 0; i < XL; i++) {
        const uint r = (wave * XL + i) * 8u + (lane >> 3);
        const uint m = min(m0 + r, M - 1u);
        xoff[i] = m * K * 2u + (((lane & 7u) ^ ((r >> 1) & 7u)) << 4);
    }
    // (wave-uniform by construction; readfirstlane tells the compiler so)
    const uint x_lds = lds0 + (uint)__builtin_amdgcn_readfirstlane((int)wave) * XL * 1024u;  // + stage * XSTAGE + i * 1024
    // weight slab: thread -> row tid, all 64 columns.  Raw bytes: three 4 KB parts per staging
    // slot (headers, first and second half of the chunk), a thread's 16 bytes at 16 * tid.
    const uint wrow_off = min(n0 + tid, N - 1u) * ((K >> 8) * Q4K_BYTES);
    const uint raw_off = 2u * XSTAGE + 2u * GX_WSTAGE;
    const uint raw_lds = lds0 + raw_off + (uint)__builtin_amdgcn_readfirstlane((int)wave) * 1024u;  // + slot * GX_RAW + part * 4096
    const uchar* const raw_rd = lds + raw_off + tid * 16u;                                          // + slot * GX_RAW + part * 4096
    uchar* const w_lds = lds + 2u * XSTAGE + tid * GX_ROW;  // + stage * GX_WSTAGE + slot * 16
    const uint wsw = (tid >> 1) & 7u;

    // wave tile: rows wy*32*MI.., columns wx*128..
    const uint wy = wave >> 1, wx = wave & 1u;
    const uint fr = lane & 31u, kg = lane >> 5, sw = (fr >> 1) & 7u;
    const uint a_lds = (wy * 32u * MI + fr) * GX_ROW;
    const uint b_lds = 2u * XSTAGE + (wx * 128u + fr) * GX_ROW;
    float16v acc[MI][4];
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;

    GxQ4K ld;
    uint magic = 0x64006400u;
    asm volatile("" : "+v"(magic));  // kept in a register: see nib2h
    const uchar* xbase = (const uchar*)xh;
    const uint last = nt - 1u;

// Requests past the last slab are clamped onto it: every step is then the same straight-line
// code (the surplus slab is fetched and dequantized into a stage nobody reads again).
// copy I of the XL + 3 that bring in slab TX's activations (I < XL) and slab TW's raw weights
#define GX_COPY(I, TX, TW)                                                                       \
    do {                                                                                         \
        if ((I) < XL) {                                                                          \
            const uchar* b_ = xbase + (size_t)(k_begin + min((TX), last) * GX_BK) * 2u;          \
            gx_load_lds16(b_, xoff[(I) < XL ? (I) : 0], x_lds + ((TX) & 1u) * XSTAGE + (I) * 1024u); \
        } else {                                                                                 \
            const uint k0_ = k_begin + min((TW), last) * GX_BK;                                  \
            const uchar* b_ = w + (size_t)(k0_ >> 8) * Q4K_BYTES;                                \
            if ((I) > XL) b_ += ((k0_ >> 6) & 3u) * 32u + 16u * ((I) - XL);                      \
            gx_load_lds16(b_, wrow_off, raw_lds + ((TW) & 1u) * GX_RAW + ((I) - XL) * 4096u);    \
        }                                                                                        \
    } while (0)
#define GX_READ_W(T) ld.read(raw_rd + ((T) & 1u) * GX_RAW, ((k_begin >> 6) + min((T), last)) & 3u)
// dequantize dword I of the chunk into OUT (two low-nibble, two high-nibble pairs)
#define GX_PART(I, LO, HI) ld.template part<I>(LO, HI, magic)
// write slots P (low nibbles) and 4+P (high) of the thread's row from the pairs of dwords 2P, 2P+1
#define GX_PUT(STG, P, L0, H0, L1, H1)                                                           \
    do {                                                                                         \
        uchar* r_ = w_lds + (STG) * GX_WSTAGE;                                                   \
        *(u32x4*)(r_ + ((((uint)(P)) ^ wsw) << 4)) = (u32x4){L0[0], L0[1], L1[0], L1[1]};        \
        *(u32x4*)(r_ + (((4u + (P)) ^ wsw) << 4)) = (u32x4){H0[0], H0[1], H1[0], H1[1]};         \
    } while (0)
#define GX_READ(STG, KS, AF, BF)                                                                 \
    do {                                                                                         \
        const uint o_ = (((2u * (KS) + kg) ^ sw) << 4);                                          \
        const uchar* xa_ = lds + (STG) * XSTAGE + a_lds + o_;                                    \
        const uchar* wb_ = lds + (STG) * GX_WSTAGE + b_lds + o_;                                 \
        _Pragma("unroll") for (int i = 0; i < MI; i++) AF[i] = *(const half8*)(xa_ + i * 32u * GX_ROW); \
        _Pragma("unroll") for (int j = 0; j < 4; j++) BF[j] = *(const half8*)(wb_ + j * 32u * GX_ROW);  \
    } while (0)
#define GX_MMA1(Q, AF, BF)                                                                       \
    acc[(Q) >> 2][(Q) & 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(AF[(Q) >> 2], BF[(Q) & 3], acc[(Q) >> 2][(Q) & 3], 0, 0, 0)
#define GX_MMA(AF, BF)                                                                           \
    do {                                                                                         \
        _Pragma("unroll") for (int q_ = 0; q_ < 4 * MI; q_++) GX_MMA1(q_, AF, BF);               \
    } while (0)
// One K sub-step's worth of interleaving: 4 MI MFMAs.  The LDS reads (the next sub-step's
// fragments) go out in pairs behind the first MFMAs so that their data is back long before the
// sub-step ends; NV vector-ALU instructions of the dequantization follow every MFMA; the LDS
// writes of the finished chunks come last.
#define GX_MIX(NV, NW)                                                                           \
    do {                                                                                         \
        _Pragma("unroll") for (int g_ = 0; g_ < 4 * MI; g_++) {                                  \
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                   \
            if (g_ < (MI + 4 + 1) / 2) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);        \
            __builtin_amdgcn_sched_group_barrier(0x002, NV, 0);                                  \
        }                                                                                        \
        __builtin_amdgcn_sched_group_barrier(0x200, NW, 0);                                      \
    } while (0)
// Step T, entered with the fragments of its first K sub-step in afA / bfA and the raw weights of
// slab T+1 unpacked in `ld`.  Sub-steps 0..2 carry the dequantization of slab T+1; then every
// wave waits for its copies and meets the others (slab T+1 complete in LDS, slab T's stages
// free); sub-step 3 — its fragments already in registers — covers what must follow the
// barrier: the first fragments of slab T+1, the raw weights of slab T+2 out of their slot, and
// the requests for slab T+2's activations and slab T+3's raw weights, one between two MFMAs.
#define GX_STEP(T)                                                                               \
    do {                                                                                         \
        const uint cur_ = (T) & 1u, nxt_ = cur_ ^ 1u;                                            \
        uint l0_[2], h0_[2], l1_[2], h1_[2], l2_[2], h2_[2];                                     \
        __builtin_amdgcn_sched_barrier(0);                                                       \
        GX_READ(cur_, 1, afB, bfB); GX_MMA(afA, bfA);                                            \
        GX_PART(0, l0_, h0_); GX_PART(1, l1_, h1_); GX_PUT(nxt_, 0, l0_, h0_, l1_, h1_); GX_PART(2, l2_, h2_); \
        GX_MIX(5, 2);                                                                            \
        GX_READ(cur_, 2, afA, bfA); GX_MMA(afB, bfB);                                            \
        GX_PART(3, l0_, h0_); GX_PUT(nxt_, 1, l2_, h2_, l0_, h0_);                               \
        GX_PART(4, l1_, h1_); GX_PART(5, l2_, h2_); GX_PUT(nxt_, 2, l1_, h1_, l2_, h2_);         \
        GX_MIX(5, 4);                                                                            \
        GX_READ(cur_, 3, afB, bfB); GX_MMA(afA, bfA);                                            \
        GX_PART(6, l0_, h0_); GX_PART(7, l1_, h1_); GX_PUT(nxt_, 3, l0_, h0_, l1_, h1_);         \
        GX_MIX(4, 2);                                                                            \
        __builtin_amdgcn_sched_barrier(0);                                                       \
        gx_wait<0>();                                                                            \
        __syncthreads();                                                                         \
        GX_READ(nxt_, 0, afA, bfA);                                                              \
        GX_READ_W((T) + 2u);                                                                     \
        GX_MMA1(0, afB, bfB);                                                                    \
        __builtin_amdgcn_sched_barrier(0);                                                       \
        _Pragma("unroll") for (int q_ = 1; q_ < 4 * MI; q_++) {                                  \
            if (q_ - 1 < XL + 3) {                                                               \
                GX_COPY(q_ - 1, (T) + 2u, (T) + 3u);                                             \
                GX_MMA1(q_, afB, bfB);                                                           \
                __builtin_amdgcn_sched_barrier(0);                                               \
            } else {                                                                             \
                GX_MMA1(q_, afB, bfB);                                                           \
            }                                                                                    \
        }                                                                                        \
        if (XL + 3 > 4 * MI - 1) {                                                               \
            _Pragma("unroll") for (int c_ = 4 * MI - 1; c_ < XL + 3; c_++) GX_COPY(c_, (T) + 2u, (T) + 3u); \
        }                                                                                        \
        ld.prep();                                                                               \
        _Pragma("unroll") for (int g_ = 0; g_ < 4 * MI; g_++) {                                  \
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                   \
            __builtin_amdgcn_sched_group_barrier(0x002, 10, 0);                                  \
        }                                                                                        \
    } while (0)

    // prologue: slab 0 in place; then the state a step expects on entry
    half8 afA[MI], bfA[4], afB[MI], bfB[4];
    _Pragma("unroll") for (int c_ = 0; c_ < XL + 3; c_++) GX_COPY(c_, 0u, 0u);
    gx_wait<0>();
    GX_READ_W(0u);
    ld.prep();
    {
        uint l0_[2], h0_[2], l1_[2], h1_[2];
        GX_PART(0, l0_, h0_); GX_PART(1, l1_, h1_); GX_PUT(0u, 0, l0_, h0_, l1_, h1_);
        GX_PART(2, l0_, h0_); GX_PART(3, l1_, h1_); GX_PUT(0u, 1, l0_, h0_, l1_, h1_);
        GX_PART(4, l0_, h0_); GX_PART(5, l1_, h1_); GX_PUT(0u, 2, l0_, h0_, l1_, h1_);
        GX_PART(6, l0_, h0_); GX_PART(7, l1_, h1_); GX_PUT(0u, 3, l0_, h0_, l1_, h1_);
    }
    _Pragma("unroll") for (int c_ = XL; c_ < XL + 3; c_++) GX_COPY(c_, 0u, 1u);
    gx_wait<0>();
    __syncthreads();
    GX_READ(0u, 0, afA, bfA);
    GX_READ_W(1u);
    _Pragma("unroll") for (int c_ = 0; c_ < XL + 3; c_++) GX_COPY(c_, 1u, 2u);
    ld.prep();

    for (uint t = 0; t < nt; t++) GX_STEP(t);
    gx_wait<0>();
#undef GX_READ_W
#undef GX_COPY
#undef GX_PART
#undef GX_PUT
#undef GX_READ
#undef GX_MMA1
#undef GX_MMA
#undef GX_MIX
#undef GX_STEP

    // epilogue: D register v of block (i, j) holds token row 8*(v/4) + 4*kg + v%4, output fr
    // (lane and wave ids are asked of the hardware again here, so that nothing derived from them has to stay in a
    // register through the loop — the 256 x 256 instance has none to spare)
    const uint le = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
    const uint we = (uint)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const uint efr = le & 31u, ekg = le >> 5, ewy = we >> 1, ewx = we & 1u;
#pragma unroll
    for (int i = 0; i < MI; i++) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint n = blockIdx.x * GX_BN + ewx * 128u + 32u * j + efr;
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const uint m = blockIdx.y * BM + ewy * 32u * MI + 32u * i + 8u * (v >> 2) + 4u * ekg + (v & 3u);
                if (m < M && n < N) {
                    float* o = y + (size_t)m * N + n;
                    if (SPLITK) atomicAdd(o, acc[i][j][v]);
                    else if (ACCUM) *o += acc[i][j][v];
                    else *o = acc[i][j][v];
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// The same product with the weights dequantized straight into the matrix cores' B registers:
//   gemm_mm_q4kl_bd(xh, w, y, K, N, accum, M)         grid [ceil(N/256), ceil(M/128), 1]
//   gemm_mm_q4kl_bd_sk(xh, w, y, K, N, M, nsplit)     grid.z = nsplit (slices of whole super-blocks); f32 atomic adds
// In the tiles above a thread dequantizes one weight row into LDS and every wave reads the f16 tile back as B
// fragments: per K step 32 KB of LDS writes, a barrier's worth of waiting for them, and 64 KB of fragment reads that
// carry nothing the wave could not have made itself.  Here a wave owns 64 weight rows against all 128 tokens of the
// tile (4 x 2 blocks of v_mfma_f32_32x32x16_f16, 128 accumulators): lane (n, g) of the B operand holds 8 consecutive
// k of row n, and 8 consecutive weights of a Q4_K chunk are the low (or high) nibbles of 8 consecutive bytes, so the
// lane fetches 16 bytes of its two rows per K step and turns them into the four sub-steps' B registers itself — the
// same two vector instructions per weight, no LDS round trip, and only the activations are shared through LDS
// (one 16 KB stage per K step, all four waves read all of it).  The K order inside a step is the lane's:
// sub-steps cover weights {0, 8, 32, 40} + 16 g + 0..7 (low nibbles of its bytes 0-7 and 8-15, then the high ones),
// and the activation fragments are read from the same positions.  Raw bytes travel global -> LDS -> the same lane
// (three K steps ahead for the nibbles, a header slot per super-block), so nothing asynchronous targets a register
// and no barrier guards them; the one barrier per step is for the activation stage.  80 KB of LDS and at most 128
// vector registers beside the accumulators: two workgroups per CU, one's dequantization under the other's MFMAs.
// MI = 32-token blocks per tile: 4 (128 tokens) or 8 (256 tokens: all 256 accumulators, one workgroup per CU).
#define GB_XSTAGE(MI) (32u * (MI) * GX_ROW)        // 16 / 32 KB
#define GB_NIB(MI) (2u * GB_XSTAGE(MI))            // 4 slots x 4 waves x 2 rows x 1 KB
#define GB_HDR(MI) (GB_NIB(MI) + 32768u)           // 2 slots x 4 waves x 2 rows x 1 KB
#define GB_LDS(MI) (GB_HDR(MI) + 16384u)

struct GbRow {
    u32x4 hdr, q;
    half2v a_lo, c_lo, a_hi, c_hi;
    __device__ __forceinline__ void prep(uint c) {
        uint sc, mn;
        q4k_scale_min_pair(hdr.y, hdr.z, hdr.w, c, sc, mn);
        const float d = f16_bits_to_f32(hdr.x & 0xFFFFu), ndm = -f16_bits_to_f32(hdr.x >> 16);
        float p1 = d * (float)(sc & 0xFFu), r1 = ndm * (float)(mn & 0xFFu);
        float p2 = d * (float)(sc >> 8), r2 = ndm * (float)(mn >> 8);
        asm volatile("" : "+v"(p1), "+v"(r1), "+v"(p2), "+v"(r2));
        const _Float16 a1 = (_Float16)p1, b1 = (_Float16)r1, a2 = (_Float16)p2, b2 = (_Float16)r2;
        a_lo = (half2v){a1, a1};
        c_lo = (half2v){b1, b1};
        a_hi = (half2v){a2, a2};
        c_hi = (half2v){b2, b2};
    }
    // sub-step S (0, 1: low nibbles of bytes 0-7, 8-15; 2, 3: the high ones) as a B fragment of 8 weights
    template <int S>
    __device__ __forceinline__ half8 frag(uint magic) const {
        const uint v0 = q[2 * (S & 1)], v1 = q[2 * (S & 1) + 1];
        constexpr uint sh = S >= 2 ? 4u : 0u;
        const half2v a = S >= 2 ? a_hi : a_lo, c = S >= 2 ? c_hi : c_lo;
        const uint p0 = __builtin_amdgcn_perm(0u, v0, 0x0C010C00u) >> sh, p1 = __builtin_amdgcn_perm(0u, v0, 0x0C030C02u) >> sh;
        const uint p2 = __builtin_amdgcn_perm(0u, v1, 0x0C010C00u) >> sh, p3 = __builtin_amdgcn_perm(0u, v1, 0x0C030C02u) >> sh;
        const u32x4 r = {GxQ4K::fma2(GxQ4K::nib2h(p0, magic), a, c), GxQ4K::fma2(GxQ4K::nib2h(p1, magic), a, c),
                         GxQ4K::fma2(GxQ4K::nib2h(p2, magic), a, c), GxQ4K::fma2(GxQ4K::nib2h(p3, magic), a, c)};
        return __builtin_bit_cast(half8, r);
    }
};

// SPLITK: 0 the whole K; 1 K slices that add into y with f32 atomics (y zeroed or holding the sum to extend: the
// reference's `_sk` contract, crates/ojas-cuda/src/kernels/gemm_q.rs:26-38); 2 K slices that leave their partial tiles
// in `part` and count themselves in `cnt`, the last one to arrive adding the slices in order and storing y (`_sr`).
// KW: the workgroup's four waves share 64 weight rows and split K between them instead (a quarter of the slice's
// super-blocks each, met in LDS at the end, in wave order): 64-row tiles for shapes whose 256-row tiles are too few to
// fill the chip.  Every wave then runs a pipeline of its own — its own activation stages, no barrier inside the loop.
template <int SPLITK, bool ACCUM, int MI, bool KW = false>
__device__ __forceinline__ void gemm_bd_body(const ushort* __restrict__ xh, const uchar* __restrict__ w,
                                             float* __restrict__ y, uint K, uint N, uint M, uint nsplit, uchar* lds,
                                             float* __restrict__ part = nullptr, uint* __restrict__ cnt = nullptr,
                                             uint acc_y = 0u) {
    static_assert(!KW || (MI == 4 && SPLITK != 2), "the K-over-waves form: 128 tokens, plain or atomic stores");
    constexpr uint XS = GB_XSTAGE(MI);
    constexpr uint NX = KW ? 4u * MI : (uint)MI;                 // activation copies a wave issues per step
    constexpr uint NSLOT = KW ? 3u : 4u, HSLOT = KW ? 1u : 2u;   // nibble / header slots (KW: 160 KB of LDS in all)
    constexpr uint NIB0 = KW ? 8u * XS : GB_NIB(MI), HDR0 = NIB0 + NSLOT * 8192u;
    const uint tid = threadIdx.x, lane = tid & 63u;
    const uint wave = (uint)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    // (An XCD-aware order — XCD c taking row tiles c, c + 8, ... and all token tiles of one before the next, so that a
    // row tile's weights are fetched into one L2 instead of four — was measured: 2-4 % slower at every size.  The tile
    // does not wait for memory.)
    const uint bx = blockIdx.x, by = blockIdx.y;
    const uint n0 = bx * (KW ? 64u : GX_BN), m0 = by * (32u * MI);
    const uint nsb = K >> 8;
    uint sb_begin = 0, sb_end = nsb;
    if (SPLITK != 0) {
        const uint per = (nsb + nsplit - 1) / nsplit;
        sb_begin = min(blockIdx.z * per, nsb);
        sb_end = min((blockIdx.z + 1) * per, nsb);
        if (sb_begin >= sb_end) return;
    }
    if (KW) {
        const uint per4 = (sb_end - sb_begin + 3u) / 4u;
        sb_begin = min(sb_begin + wave * per4, sb_end);
        sb_end = min(sb_begin + per4, sb_end);
    }
    const uint nt = (sb_end - sb_begin) * 4u, last = nt - 1u;       // (KW: a wave may be left without a share, nt = 0)
    const uint k_begin = sb_begin << 8;
    const uint lds0 = (uint)(size_t)(__attribute__((address_space(3))) uchar*)lds;

    // activation stage: wave `wave`, copy i moves rows (wave*MI + i)*8 .. +7; lane -> row lane/8, slot lane%8, which
    // holds source chunk (lane%8) ^ ((row/2)%8)
    // (KW: every wave copies all 32 MI rows into stages of its own)
    uint xoff[NX];
#pragma unroll
    for (uint i = 0; i < NX; i++) {
        const uint r = ((KW ? 0u : wave * (uint)MI) + i) * 8u + (lane >> 3);
        const uint m = min(m0 + r, M - 1u);
        xoff[i] = m * K * 2u + (((lane & 7u) ^ ((r >> 1) & 7u)) << 4);
    }
    const uint x_lds = KW ? lds0 + wave * 2u * XS : lds0 + wave * ((uint)MI * 1024u);   // + stage * XS + i * 1024
    // the lane's two weight rows: B column fr of blocks j = 0, 1; its 16 nibble bytes are bytes 16 g .. of a chunk
    const uint fr = lane & 31u, kg = lane >> 5, sw = (fr >> 1) & 7u;
    const uint row_bytes = nsb * Q4K_BYTES;
    const uint nw = n0 + (KW ? 0u : wave * 64u);
    const uint ro0 = min(nw + fr, N - 1u) * row_bytes, ro1 = min(nw + 32u + fr, N - 1u) * row_bytes;
    const uint nib_lds = lds0 + NIB0 + wave * 2048u;           // + slot * 8192 + j * 1024
    const uint hdr_lds = lds0 + HDR0 + wave * 2048u;           // + slot * 8192 + j * 1024
    const uchar* const nib_rd = lds + NIB0 + wave * 2048u + lane * 16u;
    const uchar* const hdr_rd = lds + HDR0 + wave * 2048u + lane * 16u;
    const uchar* const a_rd = lds + (KW ? wave * 2u * XS : 0u) + fr * GX_ROW;   // + stage * XS + i * 32 rows + chunk slot
    // nibble slot of step t: t mod 4, or t mod 3 (t < 2^16: K < 2^22)
    auto nslot = [](uint t) -> uint { return NSLOT == 4u ? t & 3u : t - 3u * ((t * 0xAAABu) >> 17); };

    float16v acc[MI][2];
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;
    uint magic = 0x64006400u;
    asm volatile("" : "+v"(magic));
    const uchar* xbase = (const uchar*)xh;

    // requests past the last step are clamped onto it, so that every step issues the same eight copies
    auto copy_x = [&](uint t) {
        const uchar* b = xbase + (size_t)(k_begin + min(t, last) * GX_BK) * 2u;
#pragma unroll
        for (uint i = 0; i < NX; i++) gx_load_lds16(b, xoff[i], x_lds + (t & 1u) * XS + i * 1024u);
    };
    auto copy_nib = [&](uint t) {
        const uint tc = min(t, last);
        const uchar* bn = w + (size_t)(sb_begin + (tc >> 2)) * Q4K_BYTES + 16u + (tc & 3u) * 32u;
        gx_load_lds16(bn, ro0 + 16u * kg, nib_lds + nslot(t) * 8192u);
        gx_load_lds16(bn, ro1 + 16u * kg, nib_lds + nslot(t) * 8192u + 1024u);
    };
    auto copy_hdr = [&](uint t) {               // the header of step t's super-block (a slot per super-block parity)
        const uint tc = min(t, last);
        const uchar* bh = w + (size_t)(sb_begin + (tc >> 2)) * Q4K_BYTES;
        gx_load_lds16(bh, ro0, hdr_lds + (HSLOT == 2u ? (tc >> 2) & 1u : 0u) * 8192u);
        gx_load_lds16(bh, ro1, hdr_lds + (HSLOT == 2u ? (tc >> 2) & 1u : 0u) * 8192u + 1024u);
    };
    GbRow r0, r1;
    half8 afA[MI], afB[MI], b0, b1, c0, c1;
#define GB_READ_A(T, CH, AF)                                                                           \
    do {                                                                                               \
        const uchar* xa_ = a_rd + ((T) & 1u) * XS + ((((CH) + 2u * kg) ^ sw) << 4);                    \
        _Pragma("unroll") for (int i = 0; i < MI; i++) AF[i] = *(const half8*)(xa_ + i * 32u * GX_ROW); \
    } while (0)
// the raw rows of step T out of their slots (the header only where T starts a super-block), scales of chunk C1
#define GB_READ_W(T, C1, HDR)                                                                          \
    do {                                                                                               \
        const uint slot_ = nslot(T) * 8192u;                                                           \
        r0.q = *(const u32x4*)(nib_rd + slot_);                                                        \
        r1.q = *(const u32x4*)(nib_rd + slot_ + 1024u);                                                \
        if (HDR) {                                                                                     \
            const uint hs_ = (HSLOT == 2u ? (min((T), last) >> 2) & 1u : 0u) * 8192u;                  \
            r0.hdr = *(const u32x4*)(hdr_rd + hs_);                                                    \
            r1.hdr = *(const u32x4*)(hdr_rd + hs_ + 1024u);                                            \
        }                                                                                              \
        r0.prep(C1);                                                                                   \
        r1.prep(C1);                                                                                   \
    } while (0)
#define GB_MMA(AF, B0, B1)                                                                             \
    do {                                                                                               \
        _Pragma("unroll") for (int i = 0; i < MI; i++) {                                               \
            acc[i][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(AF[i], B0, acc[i][0], 0, 0, 0);         \
            acc[i][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(AF[i], B1, acc[i][1], 0, 0, 0);         \
        }                                                                                              \
    } while (0)
// a sub-step's 2 MI MFMAs with the next fragments' LDS reads behind the first ones and NV vector instructions
// (NV / 2 when the sub-step has sixteen MFMAs to spread them over) behind each
#define GB_MIX(NV)                                                                                     \
    do {                                                                                               \
        _Pragma("unroll") for (int g_ = 0; g_ < 2 * MI; g_++) {                                        \
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                         \
            if (g_ < MI / 2) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);                        \
            __builtin_amdgcn_sched_group_barrier(0x002, MI == 4 ? (NV) : ((NV) + 1) / 2, 0);           \
        }                                                                                              \
    } while (0)
// Step T = 4 s + C of super-block s, entered with the fragments of its first sub-step in afA / b0 / b1 and its raw rows
// unpacked in r0 / r1.  Sub-steps 0..2 build the next sub-step's B fragments under their MFMAs.  Then the copies are
// awaited (stage (T + 1) & 1 must be whole, and everyone done with stage T & 1 before it is overwritten) and the next
// requests go out: activations two steps ahead, nibbles three, the next super-block's header from its second step
// (one header copy per super-block, not per step: a copy instruction walks 32 rows' cache lines whatever it moves).
// Copies complete in order, so the wait names how many younger ones may still be on their way.  Sub-step 3, its
// fragments already in registers, covers the next step's first activation fragments and raw rows.  The chunk index
// C is a compile-time constant of each of the four unrolled steps, which is what makes the scale unpacking cheap.
#define GB_STEP(C, T)                                                                                  \
    do {                                                                                               \
        __builtin_amdgcn_sched_barrier(0);                                                             \
        GB_READ_A(T, 1u, afB); GB_MMA(afA, b0, b1);                                                    \
        c0 = r0.frag<1>(magic); c1 = r1.frag<1>(magic);                                                \
        GB_MIX(4);                                                                                     \
        GB_READ_A(T, 4u, afA); GB_MMA(afB, c0, c1);                                                    \
        b0 = r0.frag<2>(magic); b1 = r1.frag<2>(magic);                                                \
        GB_MIX(5);                                                                                     \
        GB_READ_A(T, 5u, afB); GB_MMA(afA, b0, b1);                                                    \
        c0 = r0.frag<3>(magic); c1 = r1.frag<3>(magic);                                                \
        GB_MIX(5);                                                                                     \
        __builtin_amdgcn_sched_barrier(0);                                                             \
        gx_wait<(C) == 2 ? 4 : 2>();                                                                   \
        if (!KW) __syncthreads();                                                                      \
        copy_x((T) + 2u);                                                                              \
        copy_nib((T) + 3u);                                                                            \
        if ((C) == 1) copy_hdr((T) + 3u);                                                              \
        __builtin_amdgcn_sched_barrier(0);                                                             \
        GB_READ_A((T) + 1u, 0u, afA);                                                                  \
        GB_READ_W((T) + 1u, ((C) + 1) & 3, (C) == 3);                                                  \
        GB_MMA(afB, c0, c1);                                                                           \
        b0 = r0.frag<0>(magic); b1 = r1.frag<0>(magic);                                                \
        _Pragma("unroll") for (int g_ = 0; g_ < 2 * MI; g_++) {                                        \
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                         \
            if (g_ < MI / 2 + 2) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);                    \
            __builtin_amdgcn_sched_group_barrier(0x002, MI == 4 ? 11 : 6, 0);                          \
        }                                                                                              \
    } while (0)
    // prologue: the state a step expects on entry
    if (!KW || nt != 0u) {
        copy_nib(0u);
        copy_hdr(0u);
        copy_nib(1u);
        copy_x(0u);
        gx_wait<0>();
        if (!KW) __syncthreads();
        GB_READ_A(0u, 0u, afA);
        GB_READ_W(0u, 0, true);
        b0 = r0.frag<0>(magic);
        b1 = r1.frag<0>(magic);
        copy_x(1u);
        copy_nib(2u);
        for (uint t = 0; t < nt; t += 4u) {
            GB_STEP(0, t);
            GB_STEP(1, t + 1u);
            GB_STEP(2, t + 2u);
            GB_STEP(3, t + 3u);
        }
        gx_wait<0>();
    }
#undef GB_READ_A
#undef GB_READ_W
#undef GB_MMA
#undef GB_MIX
#undef GB_STEP

    if (SPLITK == 2) {
        // The slice's tile goes to `part` as the registers hold it (the halves of thread t's q-th float4 at [q][half][t]:
        // 512 contiguous bytes per wave and store), then the slice counts itself; the workgroup that finds every other slice counted reads them all back —
        // its own too, so that the sum ((s0 + s1) + s2) + ... does not depend on who came last — and owns y.  Nobody
        // waits: a slice that is not last is done.
        const uint per = (nsb + nsplit - 1) / nsplit, ns_eff = (nsb + per - 1) / per;
        const uint tile = by * gridDim.x + bx;
        constexpr uint TILE_F4 = (uint)MI * 8u * 256u;
        // The partial tiles bypass the L2 both ways (system-scope accesses: written through, read from behind the
        // cache): the slices of a tile run on different XCDs, whose L2s do not see each other's lines, and a fence
        // of device scope would write back and invalidate a whole L2 per workgroup (measured: twice the kernel time).
        // Reading the slices back is what this form costs: one workgroup per tile, every load a trip to memory.
        typedef unsigned long long u64;
        u64* const mine = (u64*)part + ((size_t)tile * ns_eff + blockIdx.z) * TILE_F4 * 2u + tid;      // [q][half][thread]
#pragma unroll
        for (int i = 0; i < MI; i++)
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    u64* const o = mine + (size_t)((i * 2 + j) * 4 + q) * 512u;
                    const u64 lo = (u64)__float_as_uint(acc[i][j][4 * q]) | ((u64)__float_as_uint(acc[i][j][4 * q + 1]) << 32);
                    const u64 hi = (u64)__float_as_uint(acc[i][j][4 * q + 2]) | ((u64)__float_as_uint(acc[i][j][4 * q + 3]) << 32);
                    __hip_atomic_store(o, lo, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                    __hip_atomic_store(o + 256, hi, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                }
        // Every wave's partial-tile stores (written through, system scope) must have been acknowledged before the
        // slice is counted: said with the instruction itself — a workgroup-scope release fence need not wait for
        // vector memory on this target, and nothing wider is affordable here (see above).
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __syncthreads();
        if (tid == 0u) *(volatile uint*)lds = atomicAdd(cnt + tile, 1u);
        __syncthreads();
        if ((uint)__builtin_amdgcn_readfirstlane((int)*(volatile uint*)lds) != ns_eff - 1u) return;
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        const u64* const all = (const u64*)part + (size_t)tile * ns_eff * TILE_F4 * 2u + tid;
#pragma unroll
        for (int i = 0; i < MI; i++)
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const u64* const at = all + (size_t)((i * 2 + j) * 4 + q) * 512u;
                    float4 sum = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                    for (uint sl = 0; sl < ns_eff; sl++) {
                        const u64 lo = __hip_atomic_load(at + (size_t)sl * TILE_F4 * 2u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                        const u64 hi = __hip_atomic_load(at + (size_t)sl * TILE_F4 * 2u + 256, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                        const float4 v = make_float4(__uint_as_float((uint)lo), __uint_as_float((uint)(lo >> 32)),
                                                     __uint_as_float((uint)hi), __uint_as_float((uint)(hi >> 32)));
                        if (sl == 0u) sum = v;
                        else { sum.x += v.x; sum.y += v.y; sum.z += v.z; sum.w += v.w; }
                    }
                    acc[i][j][4 * q] = sum.x; acc[i][j][4 * q + 1] = sum.y; acc[i][j][4 * q + 2] = sum.z; acc[i][j][4 * q + 3] = sum.w;
                }
        if (tid == 0u) cnt[tile] = 0u;        // ready for the next launch
    }
    if (KW) {
        // The waves' partial tiles meet in LDS: each wave leaves its 128 accumulators in its own activation stages (32 KB,
        // a float4 of every lane per row: 1 KB), then wave w adds token block w of all four, in wave order, and stores it.
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        float4* const dump = (float4*)(lds + wave * 2u * XS) + lane;
#pragma unroll
        for (int i = 0; i < MI; i++)
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int q = 0; q < 4; q++)
                    dump[((i * 2 + j) * 4 + q) * 64] = make_float4(acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]);
        __syncthreads();
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const float4* const src = (const float4*)lds + ((wave * 2u + j) * 4u + q) * 64u + lane;
                float4 sum = src[0];
#pragma unroll
                for (uint o = 1; o < 4u; o++) {
                    const float4 v = src[o * (2u * XS / 16u)];
                    sum.x += v.x; sum.y += v.y; sum.z += v.z; sum.w += v.w;
                }
                acc[0][j][4 * q] = sum.x; acc[0][j][4 * q + 1] = sum.y; acc[0][j][4 * q + 2] = sum.z; acc[0][j][4 * q + 3] = sum.w;
            }
    }
    // epilogue: D register v of block (i, j) holds token row 32 i + 8 (v / 4) + 4 kg + v % 4, output 64 wave + 32 j + fr
    // (KW: the wave stores token block `wave` alone, summed into acc[0])
#pragma unroll
    for (int i = 0; i < (KW ? 1 : MI); i++) {
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const uint n = nw + 32u * j + fr;
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const uint m = m0 + 32u * (KW ? wave : (uint)i) + 8u * (v >> 2) + 4u * kg + (v & 3u);
                if (m < M && n < N) {
                    float* o = y + (size_t)m * N + n;
                    if (SPLITK == 1) atomicAdd(o, acc[i][j][v]);
                    else if (SPLITK == 2) *o = acc_y ? *o + acc[i][j][v] : acc[i][j][v];
                    else if (ACCUM) *o += acc[i][j][v];
                    else *o = acc[i][j][v];
                }
            }
        }
    }
}

// (Variants with three activation stages, or four and a barrier every other step, were built and measured: 96 / 112 KB,
// one workgroup per CU, slower at 224 workgroups — the activation copies are not what a step waits for.)
extern "C" __global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2)))
gemm_mm_q4kl_bd(const ushort* xh, const uchar* w, float* y, uint K, uint N, uint accum, uint M) {
    __shared__ __attribute__((aligned(1024))) uchar lds[GB_LDS(4)];
    if (accum) gemm_bd_body<0, true, 4>(xh, w, y, K, N, M, 1u, lds);
    else gemm_bd_body<0, false, 4>(xh, w, y, K, N, M, 1u, lds);
}
extern "C" __global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2)))
gemm_mm_q4kl_bd_sk(const ushort* xh, const uchar* w, float* y, uint K, uint N, uint M, uint nsplit) {
    __shared__ __attribute__((aligned(1024))) uchar lds[GB_LDS(4)];
    gemm_bd_body<1, true, 4>(xh, w, y, K, N, M, nsplit, lds);
}
// 256 tokens per tile: the wave's 64 rows are dequantized once for twice the MFMAs
extern "C" __global__ void __launch_bounds__(256)
gemm_mm_q4kl_bd256(const ushort* xh, const uchar* w, float* y, uint K, uint N, uint accum, uint M) {
    __shared__ __attribute__((aligned(1024))) uchar lds[GB_LDS(8)];
    if (accum) gemm_bd_body<0, true, 8>(xh, w, y, K, N, M, 1u, lds);
    else gemm_bd_body<0, false, 8>(xh, w, y, K, N, M, 1u, lds);
}
extern "C" __global__ void __launch_bounds__(256)
gemm_mm_q4kl_bd256_sk(const ushort* xh, const uchar* w, float* y, uint K, uint N, uint M, uint nsplit) {
    __shared__ __attribute__((aligned(1024))) uchar lds[GB_LDS(8)];
    gemm_bd_body<1, true, 8>(xh, w, y, K, N, M, nsplit, lds);
}
// 64-row tiles, K over the workgroup's waves: grid [ceil(N/64), ceil(M/128), 1 | nsplit]
extern "C" __global__ void __launch_bounds__(256)
gemm_mm_q4kl_bdk(const ushort* xh, const uchar* w, float* y, uint K, uint N, uint accum, uint M) {
    __shared__ __attribute__((aligned(1024))) uchar lds[8u * GB_XSTAGE(4) + 4u * 8192u];
    if (accum) gemm_bd_body<0, true, 4, true>(xh, w, y, K, N, M, 1u, lds);
    else gemm_bd_body<0, false, 4, true>(xh, w, y, K, N, M, 1u, lds);
}
extern "C" __global__ void __launch_bounds__(256)
gemm_mm_q4kl_bdk_sk(const ushort* xh, const uchar* w, float* y, uint K, uint N, uint M, uint nsplit) {
    __shared__ __attribute__((aligned(1024))) uchar lds[8u * GB_XSTAGE(4) + 4u * 8192u];
    gemm_bd_body<1, true, 4, true>(xh, w, y, K, N, M, nsplit, lds);
}
// K slices without atomics and without a zero fill: partial tiles through `part` (tiles x slices x 128 KB, 256 KB for
// the 256-token tile), one counter per tile in `cnt` (zero before the first launch; every launch leaves zeros), the
// slices added in their order: results do not depend on arrival.
//   gemm_mm_q4kl_bd{,256}_sr(xh, w, y, part, cnt, K, N, M, nsplit, ACC)     grid [ceil(N/256), ceil(M/128 | 256), nsplit]
extern "C" __global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2)))
gemm_mm_q4kl_bd_sr(const ushort* xh, const uchar* w, float* y, float* part, uint* cnt, uint K, uint N, uint M, uint nsplit,
                   uint ACC) {
    __shared__ __attribute__((aligned(1024))) uchar lds[GB_LDS(4)];
    gemm_bd_body<2, true, 4>(xh, w, y, K, N, M, nsplit, lds, part, cnt, ACC);
}
extern "C" __global__ void __launch_bounds__(256)
gemm_mm_q4kl_bd256_sr(const ushort* xh, const uchar* w, float* y, float* part, uint* cnt, uint K, uint N, uint M,
                      uint nsplit, uint ACC) {
    __shared__ __attribute__((aligned(1024))) uchar lds[GB_LDS(8)];
    gemm_bd_body<2, true, 8>(xh, w, y, K, N, M, nsplit, lds, part, cnt, ACC);
}

// LDS of a tile: two activation stages, two dequantized-weight stages, two raw-weight slots
#define GX_LDS(MI) __shared__ __attribute__((aligned(1024))) uchar lds[2 * 64 * (MI) * GX_ROW + 2 * GX_WSTAGE + 2 * GX_RAW]

extern "C" __global__ void __launch_bounds__(256)
gemm_mm_q4kl(const ushort* xh, const uchar* w, float* y, uint K, uint N, uint accum, uint M) {
    GX_LDS(4);
    if (accum) gemm_xl_body<4, false, true>(xh, w, y, K, N, M, 1u, lds);
    else gemm_xl_body<4, false, false>(xh, w, y, K, N, M, 1u, lds);
}
extern "C" __global__ void __launch_bounds__(256)
gemm_mm_q4kl_sk(const ushort* xh, const uchar* w, float* y, uint K, uint N, uint M, uint nsplit) {
    GX_LDS(4);
    gemm_xl_body<4, true, true>(xh, w, y, K, N, M, nsplit, lds);
}
