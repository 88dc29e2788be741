// Family "rowq8": the row-int8 matmul of the reference's CPU models — weights requantized at load
// time to int8 with one f32 scale per row, activations quantized per whole vector, integer dots,
//   y[t][n] = bias[n] + ((float)(sum_k qw[n][k] * qx[t][k]) * sw[n]) * sx[t]
// (crates/ojas-cpu/src/cpu_math.rs:14-23 `W::Q8`, :174-179 `quant_row_i8`, :187-289 `matmul`,
// :404-415 `dot_i8`; the load-time requantization crates/ojas-formats/src/quant.rs:16-39).
//
//   rows_q8_from_f16(w16, q, scale, K, N)        grid N, block 256: q = clamp(round(w / sv)), sv = amax/127
//   quant_rows_i8(x, q, scale, K, M)             grid M, block 64 .. 1024: q = clamp(round(x * (1/s))), s = amax/127
//   matmul_q8row(xq, sx, wq, sw, y, K, N, M)             grid ceil(N/4), block 256: one wave per row,
//   matmul_q8row_bias(xq, sx, wq, sw, y, bs, K, N, M)    the row read once per 8 tokens
//
// The integer sum is exact, and the three f32 operations of the epilogue are rounded one by one in
// the reference's order (the file is compiled with contraction off), so results are bit-identical
// to the CPU path's.  K must be a multiple of 16.
#include "ojk_common.h"

// amax over a row by all waves of the workgroup (up to 16)
__device__ __forceinline__ float block_amax(float a, float* sh) {
    const uint lane = threadIdx.x & 63u, nw = blockDim.x >> 6;
    a = wave_max(a);
    if (lane == 0) sh[threadIdx.x >> 6] = a;
    __syncthreads();
    return wave_max(lane < nw ? sh[lane] : 0.0f);
}

extern "C" __global__ void __launch_bounds__(256)
rows_q8_from_f16(const ushort* __restrict__ w16, signed char* __restrict__ q, float* __restrict__ scale, uint K, uint N) {
    __shared__ float sh[16];
    const uint r = blockIdx.x, tid = threadIdx.x;
    const ushort* row = w16 + (size_t)r * K;
    float a = 0.0f;
    for (uint c = tid; c < K; c += 256u) a = fmaxf(a, fabsf(f16_bits_to_f32(row[c])));
    const float amax = block_amax(a, sh);
    const float sv = amax > 0.0f ? __fdiv_rn(amax, 127.0f) : 1.0f;
    if (tid == 0) scale[r] = sv;
    for (uint c = tid; c < K; c += 256u) {
        float v = roundf(__fdiv_rn(f16_bits_to_f32(row[c]), sv));
        q[(size_t)r * K + c] = (signed char)(int)sat127(v);
    }
}

__device__ __forceinline__ uint quant_i8_byte(float x, float inv) {
    return (uint)(int)sat127(roundf(__fmul_rn(x, inv))) & 0xffu;
}
// Any whole number of waves up to 16.  A row of up to 16 values per thread (and 16-byte aligned) is read once, as
// float4, and waits in registers while the workgroup finds its amax; longer or unaligned rows are read twice.
extern "C" __global__ void __launch_bounds__(1024)
quant_rows_i8(const float* __restrict__ x, signed char* __restrict__ q, float* __restrict__ scale, uint K, uint M) {
    __shared__ float sh[16];
    const uint r = blockIdx.x, tid = threadIdx.x, nt = blockDim.x;
    const float* row = x + (size_t)r * K;
    signed char* qr = q + (size_t)r * K;
    const uint K4 = K >> 2;
    if ((K & 3u) == 0u && K4 <= 4u * nt && ((uintptr_t)row & 15u) == 0u && ((uintptr_t)qr & 3u) == 0u) {
        float4 v[4];
        float a = 0.0f;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint c = tid + (uint)i * nt;
            v[i] = c < K4 ? ((const float4*)row)[c] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            a = fmaxf(fmaxf(a, fmaxf(fabsf(v[i].x), fabsf(v[i].y))), fmaxf(fabsf(v[i].z), fabsf(v[i].w)));
        }
        const float amax = block_amax(a, sh);
        const float s = amax > 0.0f ? __fdiv_rn(amax, 127.0f) : 1.0f;
        const float inv = __fdiv_rn(1.0f, s);
        if (tid == 0) scale[r] = s;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint c = tid + (uint)i * nt;
            if (c < K4)
                ((uint*)qr)[c] = quant_i8_byte(v[i].x, inv) | quant_i8_byte(v[i].y, inv) << 8 |
                                 quant_i8_byte(v[i].z, inv) << 16 | quant_i8_byte(v[i].w, inv) << 24;
        }
        return;
    }
    float a = 0.0f;
    for (uint c = tid; c < K; c += nt) a = fmaxf(a, fabsf(row[c]));
    const float amax = block_amax(a, sh);
    const float s = amax > 0.0f ? __fdiv_rn(amax, 127.0f) : 1.0f;
    const float inv = __fdiv_rn(1.0f, s);
    if (tid == 0) scale[r] = s;
    for (uint c = tid; c < K; c += nt) {
        float v = roundf(__fmul_rn(row[c], inv));
        qr[c] = (signed char)(int)sat127(v);
    }
}

template <bool BIAS>
__device__ __forceinline__ void matmul_q8row_body(const signed char* __restrict__ xq, const float* __restrict__ sx,
                                                  const signed char* __restrict__ wq, const float* __restrict__ sw,
                                                  float* __restrict__ y, const float* __restrict__ bs, uint K, uint N,
                                                  uint M) {
    constexpr int MT = 8;
    const uint lane = threadIdx.x & 63u;
    const uint row = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (row >= N) return;
    const signed char* wrow = wq + (size_t)row * K;
    const float s_w = sw[row], b = BIAS ? bs[row] : 0.0f;
    for (uint m0 = 0; m0 < M; m0 += MT) {
        int acc[MT];
#pragma unroll
        for (int t = 0; t < MT; t++) acc[t] = 0;
        for (uint k = lane * 16u; k < K; k += 1024u) {
            const uint4 wv = *(const uint4*)(wrow + k);
#pragma unroll
            for (int t = 0; t < MT; t++) {
                const uint m = min(m0 + t, M - 1u);
                const uint4 xv = *(const uint4*)(xq + (size_t)m * K + k);
                acc[t] = dot4_i8(wv.x, xv.x, acc[t]);
                acc[t] = dot4_i8(wv.y, xv.y, acc[t]);
                acc[t] = dot4_i8(wv.z, xv.z, acc[t]);
                acc[t] = dot4_i8(wv.w, xv.w, acc[t]);
            }
        }
#pragma unroll
        for (int t = 0; t < MT; t++) {
            const int s = wave_sum_i32(acc[t]);
            if (lane == 0 && m0 + t < M)
                y[(size_t)(m0 + t) * N + row] = __fadd_rn(b, __fmul_rn(__fmul_rn((float)s, s_w), sx[m0 + t]));
        }
    }
}

extern "C" __global__ void __launch_bounds__(256)
matmul_q8row(const signed char* xq, const float* sx, const signed char* wq, const float* sw, float* y, uint K, uint N,
             uint M) {
    matmul_q8row_body<false>(xq, sx, wq, sw, y, nullptr, K, N, M);
}
extern "C" __global__ void __launch_bounds__(256)
matmul_q8row_bias(const signed char* xq, const float* sx, const signed char* wq, const float* sw, float* y,
                  const float* bs, uint K, uint N, uint M) {
    matmul_q8row_body<true>(xq, sx, wq, sw, y, bs, K, N, M);
}

// ---- batches: the same product on the int8 matrix instruction -------------------------------------
//   matmul_q8row_mt(xq, sx, wq, sw, y, bs, K, N, M)                        grid [ceil(N/128), ceil(M/64), 1]
//   matmul_q8row_mt128(xq, sx, wq, sw, y, bs, K, N, M)                     grid [ceil(N/128), ceil(M/128), 1]
//   matmul_q8row_mt_sr(xq, sx, wq, sw, y, bs, part, cnt, K, N, M, NSPLIT)   grid [ceil(N/128), ceil(M/64), slices]
// (`bs` may be null: no bias).  v_mfma_i32_32x32x32_i8 sums 32 positions of 32 tokens x 32 rows in int32; both operands
// are plain int8 rows, so a lane's 16 bytes are 16 consecutive positions of its token (A) or its weight row (B) — the
// instruction pairs byte i of A with byte i of B, and an integer sum does not depend on the order of its terms.
// A workgroup owns 128 rows x 64 or 128 tokens in steps of 128 positions.  A step's rows and tokens are copied into LDS
// by all threads, eight threads to a 128-byte line (rows read from lanes' own 32-byte pieces instead made every line
// arrive in four instructions, and the lines did not stay in the L1 in between); LDS rows are 144 bytes apart (16
// lanes' 16-byte reads then cover all banks); two stages, one barrier per step.  64 tokens: wave w takes rows 32 w ..
// against both blocks of 32 tokens; 128 tokens: the waves form 2 x 2, each 64 rows x 64 tokens (two row operands and two
// token operands feed four instructions).  Blocks of 32 tokens past M are skipped.  Positions past K (a multiple of 16)
// are zeros on both sides.  The epilogue is that of `matmul_q8row`, so the results are the same bits.
// `_sr`: K slices whose int32 partial tiles meet in `part` (tiles x slices x 32 KB) and are summed — exactly, in any
// order — by the last slice to arrive; `cnt` (a zeroed uint per tile) is left at zero.
struct ojk_true { static constexpr bool value = true; };
struct ojk_false { static constexpr bool value = false; };
typedef int q8r_i4 __attribute__((ext_vector_type(4)));
typedef int q8r_i16 __attribute__((ext_vector_type(16)));
#define Q8R_STRIDE 144u

// RB x TB blocks of 32 rows x 32 tokens per wave, the four waves WR x WT
template <int RB, int TB, int WR, int WT, bool SPLIT>
__device__ __forceinline__ void matmul_q8row_mt_body(const signed char* xq, const float* __restrict__ sx,
                                                     const signed char* wq, const float* __restrict__ sw,
                                                     float* __restrict__ y, const float* __restrict__ bs, uint K, uint N,
                                                     uint M, uchar* lds, int* part = nullptr, uint* cnt = nullptr,
                                                     uint nsplit = 1u) {
    static_assert(WR * WT == 4 && RB * WR == 4, "four waves, 128 rows");
    constexpr uint RPG = 128u, TPG = 32u * (uint)(TB * WT);
    constexpr uint STAGE = (RPG + TPG) * Q8R_STRIDE;      // rows first, then tokens
    constexpr int NPR = 4, NPT = (int)(TPG / 32u);        // 16-byte pieces a thread copies per step: rows, tokens
    const uint tid = threadIdx.x, lane = tid & 63u;
    const uint wave = (uint)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint wr = wave % (uint)WR, wt = wave / (uint)WR;
    const uint nks = (K + 127u) >> 7;
    const uint per = SPLIT ? (nks + nsplit - 1u) / nsplit : nks;
    const uint s0 = SPLIT ? blockIdx.z * per : 0u, s1 = SPLIT ? min(nks, s0 + per) : nks;
    if (SPLIT && s0 >= s1) return;                        // (the host launches only slices that hold a step)
    // tiles in an order that keeps a row tile's token tiles on one XCD, next to each other in time (workgroups go to the
    // XCDs in turn): the rows then come from memory once and from that XCD's L2 for the other token tiles
    uint bx = blockIdx.x, by = blockIdx.y;
    {
        const uint total = gridDim.x * gridDim.y, pid = by * gridDim.x + bx;
        const uint xcd = pid & 7u, local = pid >> 3, base = total >> 3, rem = total & 7u;
        const uint q = xcd < rem ? xcd * (base + 1u) + local : rem * (base + 1u) + (xcd - rem) * base + local;
        bx = q / gridDim.y;
        by = q - bx * gridDim.y;
    }
    const uint m0 = by * TPG, n0 = bx * RPG, fr = lane & 31u, kg = lane >> 5;
    // blocks of 32 tokens of this wave that hold tokens
    const uint mw = m0 + 32u * (uint)TB * wt;
    const uint nblk = mw < M ? min((M - mw + 31u) >> 5, (uint)TB) : 0u;

    // copies: thread -> piece tid % 8 of line tid / 8 + 32 p
    const uint c_line = tid >> 3, c_ch = tid & 7u;
    // (no branches: lines past N or M repeat the last one, whose results nobody stores; a piece past K is read from the
    // last piece instead and set to zero on the token side, which makes its products zero.  Named registers, not
    // arrays: the compiler kept arrays of pieces in scratch memory.)
    static_assert(NPR == 4 && (NPT == 2 || NPT == 4), "pieces are spelled out");
    const signed char* const rp0 = wq + (size_t)min(n0 + c_line, N - 1u) * K;
    const signed char* const rp1 = wq + (size_t)min(n0 + c_line + 32u, N - 1u) * K;
    const signed char* const rp2 = wq + (size_t)min(n0 + c_line + 64u, N - 1u) * K;
    const signed char* const rp3 = wq + (size_t)min(n0 + c_line + 96u, N - 1u) * K;
    const signed char* const tp0 = xq + (size_t)min(m0 + c_line, M - 1u) * K;
    const signed char* const tp1 = xq + (size_t)min(m0 + c_line + 32u, M - 1u) * K;
    const signed char* const tp2 = xq + (size_t)min(m0 + c_line + 64u, M - 1u) * K;
    const signed char* const tp3 = xq + (size_t)min(m0 + c_line + 96u, M - 1u) * K;
    // two sets of pieces in flight: a step's loads leave two steps of arithmetic before LDS needs them (one step was
    // less than the latency of a load from memory, and the waves waited for it every step)
    const uint4 z4 = make_uint4(0u, 0u, 0u, 0u);
    uint4 r0a, r1a, r2a, r3a, t0a, t1a, t2a = z4, t3a = z4, r0b, r1b, r2b, r3b, t0b, t1b, t2b = z4, t3b = z4;
    auto zero_past = [](uint4 v, uint keep) { return make_uint4(v.x & keep, v.y & keep, v.z & keep, v.w & keep); };
#define Q8R_FETCH(S, X)                                                       \
    {                                                                         \
        const uint k_ = min((S), s1 - 1u) * 128u + 16u * c_ch, kc_ = min(k_, K - 16u); \
        const uint keep_ = k_ < K ? 0xffffffffu : 0u;                         \
        r0##X = *(const uint4*)(rp0 + kc_);                                   \
        r1##X = *(const uint4*)(rp1 + kc_);                                   \
        r2##X = *(const uint4*)(rp2 + kc_);                                   \
        r3##X = *(const uint4*)(rp3 + kc_);                                   \
        t0##X = zero_past(*(const uint4*)(tp0 + kc_), keep_);                 \
        t1##X = zero_past(*(const uint4*)(tp1 + kc_), keep_);                 \
        if (NPT == 4) {                                                       \
            t2##X = zero_past(*(const uint4*)(tp2 + kc_), keep_);             \
            t3##X = zero_past(*(const uint4*)(tp3 + kc_), keep_);             \
        }                                                                     \
    }
#define Q8R_PUT(ST, X)                                                        \
    {                                                                         \
        uchar* o_ = (ST) + c_line * Q8R_STRIDE + 16u * c_ch;                  \
        *(uint4*)o_ = r0##X;                                                  \
        *(uint4*)(o_ + 32u * Q8R_STRIDE) = r1##X;                             \
        *(uint4*)(o_ + 64u * Q8R_STRIDE) = r2##X;                             \
        *(uint4*)(o_ + 96u * Q8R_STRIDE) = r3##X;                             \
        *(uint4*)(o_ + RPG * Q8R_STRIDE) = t0##X;                             \
        *(uint4*)(o_ + (RPG + 32u) * Q8R_STRIDE) = t1##X;                     \
        if (NPT == 4) {                                                       \
            *(uint4*)(o_ + (RPG + 64u) * Q8R_STRIDE) = t2##X;                 \
            *(uint4*)(o_ + (RPG + 96u) * Q8R_STRIDE) = t3##X;                 \
        }                                                                     \
    }

    q8r_i16 acc[RB][TB];
#pragma unroll
    for (int b = 0; b < RB; b++)
#pragma unroll
        for (int i = 0; i < TB; i++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[b][i][v] = 0;

    // a step's matrix instructions; FULL: every block of the wave holds tokens (no test per block)
    auto mma = [&](const uchar* stage, auto full) {
        const uchar* st = stage + fr * Q8R_STRIDE + 16u * kg;
        const uchar* sr = st + 32u * (uint)RB * wr * Q8R_STRIDE;
        const uchar* stt = st + (RPG + 32u * (uint)TB * wt) * Q8R_STRIDE;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            q8r_i4 bv[RB];
#pragma unroll
            for (int b = 0; b < RB; b++) bv[b] = *(const q8r_i4*)(sr + (uint)b * 32u * Q8R_STRIDE + 32 * j);
#pragma unroll
            for (int i = 0; i < TB; i++) {
                if (decltype(full)::value || (uint)i < nblk) {
                    const q8r_i4 a = *(const q8r_i4*)(stt + (uint)i * 32u * Q8R_STRIDE + 32 * j);
#pragma unroll
                    for (int b = 0; b < RB; b++)
                        acc[b][i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, bv[b], acc[b][i], 0, 0, 0);
                }
            }
        }
    };
    // One loop per case: a test inside the loop made the compiler keep two sets of accumulators and copy between them.
    // At the top of the loop LDS stage 0 holds step s and set a is step s + 1 on its way.
#define Q8R_STEPS(FULL)                                                  \
    for (uint s = s0; s < s1; s += 2u) {                                 \
        Q8R_FETCH(s + 2u, b)                                             \
        __builtin_amdgcn_sched_barrier(0);                               \
        mma(lds, FULL{});                                                \
        __builtin_amdgcn_sched_barrier(0);                               \
        Q8R_PUT(lds + STAGE, a)                                          \
        __syncthreads();                                                 \
        if (s + 1u >= s1) break;                                         \
        Q8R_FETCH(s + 3u, a)                                             \
        __builtin_amdgcn_sched_barrier(0);                               \
        mma(lds + STAGE, FULL{});                                        \
        __builtin_amdgcn_sched_barrier(0);                               \
        Q8R_PUT(lds, b)                                                  \
        __syncthreads();                                                 \
    }
    Q8R_FETCH(s0, a)
    Q8R_PUT(lds, a)
    __syncthreads();
    Q8R_FETCH(s0 + 1u, a)
    if (nblk == (uint)TB) Q8R_STEPS(ojk_true)
    else Q8R_STEPS(ojk_false)
#undef Q8R_STEPS
#undef Q8R_FETCH
#undef Q8R_PUT

    if (SPLIT) {
        // partial tiles out as the registers hold them ([pair][thread]), written through and read from behind the L2
        // (a tile's slices run on different XCDs); the stores are awaited by instruction before the slice is counted
        static_assert(!SPLIT || (RB == 1 && TB == 2), "partial tiles are laid out for 32 rows x 64 tokens a wave");
        typedef unsigned long long u64;
        const uint ns_eff = (nks + per - 1u) / per;
        const uint tile = by * gridDim.x + bx;
        u64* const mine = (u64*)part + ((size_t)tile * ns_eff + blockIdx.z) * 16u * 256u + tid;
        // register pair h of block i holds tokens 32 i + 8 (h / 2) ..: only the pairs that hold tokens travel
        const uint live = M - m0;
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int h = 0; h < 8; h++)
                if (32u * (uint)i + 8u * (uint)(h >> 1) < live)
                    __hip_atomic_store(mine + (size_t)(i * 8 + h) * 256u,
                                       (u64)(uint)acc[0][i % TB][2 * h] | ((u64)(uint)acc[0][i % TB][2 * h + 1] << 32),
                                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __syncthreads();
        if (tid == 0u) *(volatile uint*)lds = atomicAdd(cnt + tile, 1u);
        __syncthreads();
        if ((uint)__builtin_amdgcn_readfirstlane((int)*(volatile uint*)lds) != ns_eff - 1u) return;
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        const u64* const all = (const u64*)part + (size_t)tile * ns_eff * 16u * 256u + tid;
#pragma unroll
        for (int i = 0; i < TB; i++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[0][i][v] = 0;
        for (uint sl = 0; sl < ns_eff; sl++) {
            u64 v[16];
#pragma unroll
            for (int i = 0; i < 16; i++) {
                v[i] = 0ull;
                if (32u * (uint)(i >> 3) + 8u * (uint)((i & 7) >> 1) < live)
                    v[i] = __hip_atomic_load(all + ((size_t)sl * 16u + (uint)i) * 256u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            }
#pragma unroll
            for (int i = 0; i < 16; i++) {
                acc[0][(i / 8) % TB][2 * (i % 8)] += (int)(uint)v[i];
                acc[0][(i / 8) % TB][2 * (i % 8) + 1] += (int)(uint)(v[i] >> 32);
            }
        }
        if (tid == 0u) cnt[tile] = 0u;                               // ready for the next launch
    }
    // D register v of a block: token 8 (v / 4) + 4 kg + v % 4 of its 32, row fr of its 32
#pragma unroll
    for (int b = 0; b < RB; b++) {
        const uint n = n0 + 32u * ((uint)RB * wr + (uint)b) + fr;
        if (n >= N) continue;
        const float s_w = sw[n], bv = bs ? bs[n] : 0.0f;
#pragma unroll
        for (int i = 0; i < TB; i++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const uint t = mw + 32u * (uint)i + 8u * (uint)(v >> 2) + 4u * kg + (uint)(v & 3);
                if (t < M) y[(size_t)t * N + n] = __fadd_rn(bv, __fmul_rn(__fmul_rn((float)acc[b][i][v], s_w), sx[t]));
            }
    }
}

extern "C" __global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2)))
matmul_q8row_mt(const signed char* xq, const float* sx, const signed char* wq, const float* sw, float* y, const float* bs,
                uint K, uint N, uint M) {
    __shared__ __attribute__((aligned(16))) uchar lds_q8r[2 * 192 * Q8R_STRIDE];
    matmul_q8row_mt_body<1, 2, 4, 1, false>(xq, sx, wq, sw, y, bs, K, N, M, lds_q8r);
}
extern "C" __global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2)))
matmul_q8row_mt128(const signed char* xq, const float* sx, const signed char* wq, const float* sw, float* y,
                   const float* bs, uint K, uint N, uint M) {
    __shared__ __attribute__((aligned(16))) uchar lds_q8r[2 * 256 * Q8R_STRIDE];
    matmul_q8row_mt_body<2, 2, 2, 2, false>(xq, sx, wq, sw, y, bs, K, N, M, lds_q8r);
}
extern "C" __global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2)))
matmul_q8row_mt_sr(const signed char* xq, const float* sx, const signed char* wq, const float* sw, float* y,
                   const float* bs, int* part, uint* cnt, uint K, uint N, uint M, uint NSPLIT) {
    __shared__ __attribute__((aligned(16))) uchar lds_q8r[2 * 192 * Q8R_STRIDE];
    matmul_q8row_mt_body<1, 2, 4, 1, true>(xq, sx, wq, sw, y, bs, K, N, M, lds_q8r, part, cnt, NSPLIT);
}

// ---- 1 to 8 tokens: rows streamed once, the tokens' int8 waiting in LDS ------------------------------
//   matmul_q8row_dec(xq, sx, wq, sw, y, bs, K, N, M)     M K <= 64 KB     grid: rows grid-stride, block 256 .. 1024
//   matmul_q8row_dec_l(..)                               M K <= 128 KB    (one workgroup per CU)
// (`bs` may be null.)  A wave takes two rows per pass and its lanes the 16-byte pieces lane, lane + 64, ..: two row
// loads feed 8 M integer dots against the tokens' pieces from LDS; the sums meet across the wave.  Same integer sums,
// same epilogue, same bits as `matmul_q8row`.
// lane ^ (1 << B)'s value
template <int B>
__device__ __forceinline__ int q8r_xor_lane(int v, uint lane) {
    if (B == 0) return dpp_i32<OJK_DPP_QUAD_XOR1>(v);
    if (B == 1) return dpp_i32<OJK_DPP_QUAD_XOR2>(v);
    if (B == 2) return __builtin_amdgcn_ds_swizzle(v, (4 << 10) | 0x1f);
    if (B == 3) return __builtin_amdgcn_ds_swizzle(v, (8 << 10) | 0x1f);
    if (B == 4) return __builtin_amdgcn_ds_swizzle(v, (16 << 10) | 0x1f);
    return __builtin_amdgcn_ds_bpermute((int)((lane ^ 32u) << 2), v);
}
template <int V, int B>
__device__ __forceinline__ void q8r_fold(int (&a)[V], uint lane) {
    if constexpr ((1 << B) < V) {
        const bool hi = (lane >> B) & 1u;
#pragma unroll
        for (int i = 0; i < (V >> (B + 1)); i++) {
            const int keep = hi ? a[2 * i + 1] : a[2 * i], send = hi ? a[2 * i] : a[2 * i + 1];
            a[i] = keep + q8r_xor_lane<B>(send, lane);
        }
        q8r_fold<V, B + 1>(a, lane);
    } else if constexpr (B < 6) {
        a[0] += q8r_xor_lane<B>(a[0], lane);
        q8r_fold<V, B + 1>(a, lane);
    }
}
// The wave's sums of V values at once: every lane returns the sum of a[lane % V] (V a power of two up to 16).  Each
// step over a lane bit halves the values a lane still carries, so 16 values cost 17 exchanges instead of 16 x 6.
template <int V>
__device__ __forceinline__ int q8r_wave_sums(int (&a)[V], uint lane) {
    q8r_fold<V, 0>(a, lane);
    return a[0];
}

template <int MT>
__device__ __forceinline__ void matmul_q8row_dec_rows(const uchar* xl, const float* __restrict__ sx,
                                                      const signed char* __restrict__ wq, const float* __restrict__ sw,
                                                      float* __restrict__ y, const float* __restrict__ bs, uint K, uint N,
                                                      uint M) {
    const uint lane = threadIdx.x & 63u, nw = blockDim.x >> 6, wave = threadIdx.x >> 6, K16 = K >> 4;
    for (uint n0 = (blockIdx.x * nw + wave) * 2u; n0 < N; n0 += gridDim.x * nw * 2u) {
        const uint n1 = min(n0 + 1u, N - 1u);
        const uint4* r0 = (const uint4*)(wq + (size_t)n0 * K);
        const uint4* r1 = (const uint4*)(wq + (size_t)n1 * K);
        int acc[2 * MT];                                              // [2 t + r]: token t, row n0 + r
#pragma unroll
        for (int i = 0; i < 2 * MT; i++) acc[i] = 0;
        for (uint p = lane; p < K16; p += 64u) {
            const uint4 w0 = r0[p], w1 = r1[p];
#pragma unroll
            for (int t = 0; t < MT; t++) {
                const uint4 xv = ((const uint4*)xl)[min((uint)t, M - 1u) * K16 + p];
                acc[2 * t + 0] = dot4_i8(w0.x, xv.x, acc[2 * t + 0]);
                acc[2 * t + 0] = dot4_i8(w0.y, xv.y, acc[2 * t + 0]);
                acc[2 * t + 0] = dot4_i8(w0.z, xv.z, acc[2 * t + 0]);
                acc[2 * t + 0] = dot4_i8(w0.w, xv.w, acc[2 * t + 0]);
                acc[2 * t + 1] = dot4_i8(w1.x, xv.x, acc[2 * t + 1]);
                acc[2 * t + 1] = dot4_i8(w1.y, xv.y, acc[2 * t + 1]);
                acc[2 * t + 1] = dot4_i8(w1.z, xv.z, acc[2 * t + 1]);
                acc[2 * t + 1] = dot4_i8(w1.w, xv.w, acc[2 * t + 1]);
            }
        }
        const int mine = q8r_wave_sums<2 * MT>(acc, lane);            // lane 2 t + r: token t, row n0 + r
        const uint t = lane >> 1, n = n0 + (lane & 1u);
        if (lane < 2u * MT && t < M && n < N)
            y[(size_t)t * N + n] = __fadd_rn(bs ? bs[n] : 0.0f, __fmul_rn(__fmul_rn((float)mine, sw[n]), sx[t]));
    }
}

template <uint LDS_BYTES>
__device__ __forceinline__ void matmul_q8row_dec_body(const signed char* __restrict__ xq, const float* __restrict__ sx,
                                                      const signed char* __restrict__ wq, const float* __restrict__ sw,
                                                      float* __restrict__ y, const float* __restrict__ bs, uint K, uint N,
                                                      uint M, uchar* xl) {
    const uint chunks = (M * K) >> 4;                                    // (the host checks M K <= LDS_BYTES)
    for (uint c = threadIdx.x; c < chunks; c += blockDim.x) ((uint4*)xl)[c] = ((const uint4*)xq)[c];
    __syncthreads();
    if (M == 1u) matmul_q8row_dec_rows<1>(xl, sx, wq, sw, y, bs, K, N, M);
    else if (M == 2u) matmul_q8row_dec_rows<2>(xl, sx, wq, sw, y, bs, K, N, M);
    else if (M <= 4u) matmul_q8row_dec_rows<4>(xl, sx, wq, sw, y, bs, K, N, M);
    else matmul_q8row_dec_rows<8>(xl, sx, wq, sw, y, bs, K, N, M);
}

extern "C" __global__ void __launch_bounds__(1024)
matmul_q8row_dec(const signed char* xq, const float* sx, const signed char* wq, const float* sw, float* y, const float* bs,
                 uint K, uint N, uint M) {
    __shared__ __attribute__((aligned(16))) uchar lds_x[65536];
    matmul_q8row_dec_body<65536u>(xq, sx, wq, sw, y, bs, K, N, M, lds_x);
}
extern "C" __global__ void __launch_bounds__(1024)
matmul_q8row_dec_l(const signed char* xq, const float* sx, const signed char* wq, const float* sw, float* y,
                   const float* bs, uint K, uint N, uint M) {
    __shared__ __attribute__((aligned(16))) uchar lds_x[131072];
    matmul_q8row_dec_body<131072u>(xq, sx, wq, sw, y, bs, K, N, M, lds_x);
}
